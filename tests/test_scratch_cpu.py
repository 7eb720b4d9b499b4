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

