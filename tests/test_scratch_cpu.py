"""The activation pool: a step arena and two arenas the layers take in turn."""
import torch

import hector_engine_amd  # noqa: F401
from hector_engine_amd.engine.scratch import ScratchPool


def test_a_layers_tensors_outlive_the_next_layer_but_not_the_one_after():
    pool = ScratchPool("cpu", initial_bytes=1 << 12)
    pool.reset()
    resid = pool.alloc((4, 8), torch.float32)            # lives as long as the step
    resid.fill_(1.0)
    seen = []
    for layer in range(5):
        pool.begin_layer()
        t = pool.alloc((16,), torch.float32)
        t.fill_(float(layer))
        seen.append(t)
        if layer >= 1:
            assert seen[layer - 1].eq(float(layer - 1)).all()      # the predecessor's output is intact
        if layer >= 2:
            assert seen[layer - 2].data_ptr() == t.data_ptr()       # the one before that gave its place
    pool.end_layers()
    logits = pool.alloc((3,), torch.float32)
    logits.fill_(7.0)
    assert resid.eq(1.0).all() and seen[-1].eq(4.0).all()
    assert logits.data_ptr() != resid.data_ptr()


def test_release_gives_back_a_turns_temporaries():
    pool = ScratchPool("cpu", initial_bytes=1 << 16)
    pool.reset()
    pool.begin_layer()
    keep = pool.alloc((8,), torch.float32)
    mark = pool.mark()
    a = pool.alloc((100,), torch.float32)
    pool.release(mark)
    b = pool.alloc((100,), torch.float32)
    assert a.data_ptr() == b.data_ptr() and keep.data_ptr() != b.data_ptr()


def test_an_arena_that_was_too_small_is_made_whole_at_the_next_step_and_a_frozen_pool_refuses():
    pool = ScratchPool("cpu", initial_bytes=256)
    pool.reset()
    pool.begin_layer()
    first = pool.alloc((64,), torch.float32)
    first.fill_(3.0)
    big = pool.alloc((10000,), torch.float32)             # replaces the layer arena
    big.fill_(5.0)
    assert first.eq(3.0).all()                            # the old view keeps its memory
    mark = pool.mark()
    pool.release(mark)
    peak = pool.peak
    assert peak >= 10000 * 4 + 256
    pool.reset()
    pool.begin_layer()
    x = pool.alloc((64,), torch.float32)
    y = pool.alloc((10000,), torch.float32)
    assert y.data_ptr() - x.data_ptr() == 256             # one piece now
    pool.reset()
    pool.frozen = True
    pool.begin_layer()
    pool.alloc((10000,), torch.float32)
    try:
        pool.alloc((1 << 22,), torch.float32)
    except RuntimeError as e:
        assert "cannot grow" in str(e)
    else:
        raise AssertionError("a frozen pool grew")


def test_which_library_products_are_cut_along_k():
    """The rule that sends a long-K product of up to 512 rows to the library in K slices: the down projections of
    the Qwen2 shapes in 2 to 8 slices, nothing for short K, wide outputs, more than 512 rows, or a K that does not divide."""
    from hector_engine_amd.parts.linear import Linear

    def slices(N, K, rows):
        return Linear(torch.empty(N, K, dtype=torch.bfloat16, device="meta"))._library_slices(rows)
    assert [slices(3584, 18944, r) for r in (65, 200, 256, 512, 513, 2048)] == [8, 8, 8, 4, 1, 1]
    assert slices(5120, 27648, 128) == 8 and slices(5120, 27648, 300) == 4
    assert slices(8192, 29568, 128) == 4 and slices(8192, 29568, 300) == 2
    assert slices(4608, 3584, 200) == 1 and slices(37888, 3584, 200) == 1 and slices(3584, 3584, 128) == 1
    assert slices(152064, 3584, 100) == 1
    assert slices(64, 8200, 100) == 1 and slices(64, 8208, 100) == 2 and slices(64, 8224, 100) == 4


def test_which_one_token_steps_count_as_uneven():
    """The engine's flag for a step in which one sequence has several times the keys of the others: the longest
    has 4096 or more and at least four times the mean; a single sequence, equal lengths or short ones do not count."""
    import types
    from hector_engine_amd.engine.engine import Engine, StepEntry

    def uneven(lengths):
        fake = types.SimpleNamespace(cache=types.SimpleNamespace(length=lambda slot: lengths[slot]))
        return Engine._uneven_keys(fake, [StepEntry(i, [1], [0]) for i in range(len(lengths))])
    assert uneven([30000] + [200] * 7) and uneven([30000, 30000] + [500] * 62) and uneven([4096, 10, 10, 10, 10])
    assert not uneven([30000]) and not uneven([8000] * 8) and not uneven([16000, 16000] + [1000] * 6)
    assert not uneven([4000, 10, 10, 10, 10]) and not uneven([5000, 4000, 3000])
