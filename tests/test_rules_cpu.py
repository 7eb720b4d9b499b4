"""Host-side rules that choose how a step runs: which library products are cut along K, which
one-token steps count as uneven."""
import torch

import hector_engine_amd  # noqa: F401


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
