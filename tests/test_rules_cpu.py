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
    """The attention part's hint for a one-token step in which one sequence has several times the keys of the
    others: the longest has 4096 or more and at least four times the mean; a single sequence, equal lengths or
    short ones do not count."""
    from hector_engine_amd.parts.attention import Attention, keys_uneven
    assert Attention.step_hint is keys_uneven

    def uneven(lengths, was=False):
        return keys_uneven(lengths, was)
    assert uneven([30000] + [200] * 7) and uneven([30000, 30000] + [500] * 62) and uneven([4096, 10, 10, 10, 10])
    assert not uneven([30000]) and not uneven([8000] * 8) and not uneven([16000, 16000] + [1000] * 6)
    assert not uneven([4000, 10, 10, 10, 10]) and not uneven([5000, 4000, 3000])
    # once up, the flag stays up until the longest has fewer than three times the mean
    assert not uneven([9000, 1000, 1000, 1000]) and uneven([9000, 1000, 1000, 1000], was=True)
    assert not uneven([5000, 1000, 1000, 1000], was=True) and not uneven([4000, 10, 10], was=True)


def test_sync_each_launch_names_the_op(monkeypatch):
    """The debugging mode waits for the GPU after every launch and, when that wait reports an
    error, raises one that names the op; outside the mode a launcher is called as it is."""
    from hector_engine_amd.kernels import profiler
    calls = []

    @profiler.op("toy_op")
    def launch(x):
        calls.append(x)
        return x + 1

    waits = []
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a: waits.append(1))
    assert launch(1) == 2 and waits == []                  # no mode, no wait
    with profiler.sync_each_launch():
        assert launch(2) == 3 and waits == [1]

        def broken(*a):
            raise RuntimeError("HIP error: an illegal memory access was encountered")
        monkeypatch.setattr(torch.cuda, "synchronize", broken)
        try:
            launch(3)
        except profiler.LaunchFault as exc:
            assert "toy_op" in str(exc) and "illegal memory access" in str(exc)
        else:
            raise AssertionError("the fault was not reported")
        try:
            with profiler.span("library_gemm"):
                pass
        except profiler.LaunchFault as exc:
            assert "library_gemm" in str(exc)
        else:
            raise AssertionError("the fault was not reported")
    assert launch(4) == 5 and calls == [1, 2, 3, 4]         # the mode ends with its context


def test_profiler_reads_its_oldest_events_on_the_way(monkeypatch):
    """A long profiled run does not pile up events: once MAX_PENDING launches wait to be read,
    the older half is read into the totals."""
    from hector_engine_amd.kernels import profiler

    class FakeEvent:
        def __init__(self, enable_timing=False):
            pass

        def record(self):
            pass

        def synchronize(self):
            pass

        def elapsed_time(self, other):
            return 0.5
    monkeypatch.setattr(torch.cuda, "Event", FakeEvent)
    monkeypatch.setattr(profiler, "MAX_PENDING", 8)
    prof = profiler.OpProfiler()
    for i in range(30):
        with prof.span("a" if i % 2 else "b"):
            pass
        assert len(prof._pending) < 8
    rows = {name: (calls, ms) for name, calls, ms, _, _ in prof.rows()}
    assert rows == {"a": (15, 7.5), "b": (15, 7.5)} and prof._pending == []
