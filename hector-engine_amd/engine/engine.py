"""The engine: a model, its cache and the one step function.

A step takes, for each sequence of a batch, its slot, its next tokens (a whole
prompt, one token, or any run of tokens) and the places whose logits are wanted.
It runs exactly those tokens, packed without padding, against the cache that
earlier steps left, and returns fp32 logits at the wanted places. The reference
runs one sequence with one position scalar (src/graph_builder.hpp:222-231,
src/engine.cpp:138-145); packing, slots and per-row positions are this
engine's own. One-token steps are captured once per batch-size bucket into a
HIP graph and replayed (the reference's build-once, replay-many decode:
src/engine.cpp:151-269); so are short prompt steps and steps that mix prompts
with one-token entries, per bucket of their sizes (rows, sequences, longest run
of new tokens, keys, wanted places).
"""
from __future__ import annotations

import collections
import dataclasses
import warnings

import numpy as np
import torch

from ..cache.paged import PagedCache
from ..cache.pages import CacheError, CacheFull  # noqa: F401
from ..config.base import ModelConfig, stop_token_ids
from ..kernels import lib as kernel_lib
from ..kernels import library_tuning, profiler
from ..parts.base import BuildEnv, StepContext
from ..registry import build_model, load_config
from ..weights.loader import load_tensors
from ..weights.random_init import random_tensors
from .scratch import ScratchPool

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
           "fp32": torch.float32}

GRAPH_MAX_BUCKET = 256
# Steps other than all-one-token ones are captured too when they have at most so many rows: a
# longer prompt keeps the GPU busy for longer than the host needs to issue it, and its sizes
# rarely come again. So many such graphs are kept, the least recently used one goes first.
GRAPH_MAX_STEP_ROWS = 512
GRAPH_MAX_STEP_PLANS = 24
# A longer step is captured as it is, without padding rows (which the library's products would
# compute), when its row count is a multiple of GRAPH_CHUNK_MULTIPLE up to GRAPH_MAX_CHUNK_ROWS: the
# fixed chunks a long prompt is fed in come again and again (2,048 tokens at the Qwen2.5-7B shape:
# 24.7 ms of kernels, 25.2 ms issued launch by launch).
GRAPH_CHUNK_MULTIPLE = 256
GRAPH_MAX_CHUNK_ROWS = 4096
GRAPH_CHUNK_MAX_WANTS = 64      # (a bucket keeps its logits: thousands of wanted rows of a long vocabulary are gigabytes)
ROW_TABLES_MAX_BYTES = 256 * 1024     # page table rows that a one-token step takes along with its metadata


class StepError(ValueError):
    """A step that cannot run as asked; nothing has been changed."""


@dataclasses.dataclass
class StepEntry:
    slot: int
    tokens: list
    want: list = dataclasses.field(default_factory=list)   # places among `tokens`


class _Meta:
    """Packed int32 metadata of a step: one host buffer, one copy, views on the device."""

    FIELDS = ("tokens", "positions", "row_seq", "seq_slot", "cu_seqlens", "seq_start", "want_rows")

    def __init__(self, rows: int, seqs: int, wants: int, row_tables: int = 0):
        """row_tables: ints of room behind the fields for the page table rows of the step's rows."""
        sizes = (rows, rows, rows, seqs, seqs + 1, seqs, max(wants, 1))
        self.offsets = {}
        off = 0
        for name, n in zip(self.FIELDS, sizes):
            self.offsets[name] = (off, n)
            off += n
        if row_tables:
            off = (off + 31) // 32 * 32          # from a cache line's start
            self.offsets["row_tables"] = (off, row_tables)
            off += row_tables
        self.total = off

    def views(self, buf):
        return {name: buf[o:o + n] for name, (o, n) in self.offsets.items()}


def _pow2(n: int, least: int = 1) -> int:
    return max(least, 1 << (max(n, 1) - 1).bit_length())


class _GraphBucket:
    def __init__(self, size: int, device, seqs: int | None = None, wants: int | None = None,
                 row_tables: int = 0):
        self.size = size
        self.meta = _Meta(size, size if seqs is None else seqs, size if wants is None else wants, row_tables)
        self.dev = torch.zeros(self.meta.total, dtype=torch.int32, device=device)
        self.views = self.meta.views(self.dev)
        self.pool = ScratchPool(device)
        self.graph: torch.cuda.CUDAGraph | None = None
        self.logits: torch.Tensor | None = None
        self.uses = 0
        self.capture_failed: str | None = None    # why this bucket runs without a graph


class Engine:
    def __init__(self, model_dir: str | None = None, *, config: ModelConfig | None = None,
                 seed: int | None = None, dtype: str = "bfloat16", max_tokens: int = 8192,
                 max_slots: int | None = None, max_seq_len: int | None = None,
                 device: str = "cuda:0", fast_kernels: bool = True, use_graphs: bool = True,
                 tune_library: bool = False, beyond_max_positions: bool = False, profile: bool = False,
                 sync_each_launch: bool = False, graph_step_rows: int = GRAPH_MAX_STEP_ROWS,
                 graph_chunk_rows: int = GRAPH_MAX_CHUNK_ROWS):
        """max_seq_len: the longest sequence (default: the positions the model's configuration
        allows; more than that is refused unless beyond_max_positions says it is meant).
        tune_library: let the library's autotuner choose the kernel of each tall bfloat16
        matrix product the first time its shape is seen (kernels/library_tuning.py).
        profile: time every kernel with a pair of events (kernels/profiler.py; steps then run
        without HIP graphs); profile_summary() gives the table.
        graph_step_rows: prompt steps and mixed steps of up to so many rows are captured as HIP
        graphs too, one per bucket of their sizes (0: only one-token steps are).
        graph_chunk_rows: longer steps are captured as well, unpadded, when their row count is a
        multiple of 256 and at most this and they want at most 64 places (fixed prompt chunks; 0,
        or graph_step_rows 0: none).
        sync_each_launch: a debugging mode (the reference's sync_after_each_op, src/engine.cpp:318-334):
        steps run without HIP graphs and the host waits for the GPU after every launch, so that
        a fault is reported with the name of the op that raised it."""
        if dtype not in _DTYPES:
            raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, got {dtype!r}")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU: this engine runs its HIP kernels on an MI355X only")
        kernel_lib.load()   # fails loudly when the kernel library is missing
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.dtype = _DTYPES[dtype]
        if self.dtype == torch.float32:
            # the library matrix product is not on the float32 path; make sure no
            # reduced-precision mode could slip in through torch either
            torch.backends.cuda.matmul.allow_tf32 = False
        self.env = BuildEnv(self.device, self.dtype, fast_kernels)
        if tune_library and self.dtype == torch.bfloat16:
            library_tuning.enable()
        if model_dir is not None:
            self.config = load_config(model_dir)
        elif config is not None:
            self.config = config
        else:
            raise ValueError("give a model folder, or a configuration and a seed")
        # what ends a sequence when a caller of generate() names no stop ids
        self.stop_ids = stop_token_ids(model_dir, self.config)
        self.model = build_model(self.config, self.env)
        specs = self.model.tensor_specs()
        if model_dir is not None:
            tensors = load_tensors(model_dir, specs, self.dtype, self.device, self.model.spec.unused_tensors)
        else:
            if seed is None:
                raise ValueError("random weights need a seed")
            tensors = random_tensors(specs, seed, self.dtype, self.device)
        self.model.bind(tensors)
        del tensors
        self.vocab_size = self.model.spec.vocab_size
        allowed = self.model.spec.max_positions
        if max_seq_len is not None and max_seq_len > allowed and not beyond_max_positions:
            raise ValueError(f"max_seq_len {max_seq_len} exceeds the {allowed} positions the model's "
                             "configuration allows (pass beyond_max_positions=True if that is meant)")
        max_seq_len = max_seq_len or allowed
        self.cache = PagedCache(self.model.run_plans(), max_tokens=max_tokens,
                                max_slots=max_slots or 256, max_seq_len=min(max_seq_len, max_tokens),
                                dtype=self.dtype, device=self.device)
        # the cache counts in whole pages; the engine holds sequences to the length asked for
        self._max_seq_len = min(max_seq_len, self.cache.max_seq_len)
        self.caches = [self.cache.layer_cache(r) for r in range(len(self.model.schedule))]
        self.scratch = ScratchPool(self.device)
        self.profiler = profiler.OpProfiler() if profile else None
        self.sync_each_launch = sync_each_launch
        self.use_graphs = use_graphs and self.model.graph_safe() and not profile and not sync_each_launch
        self._buckets: dict[tuple[int, tuple], _GraphBucket] = {}
        self._hint_fns = self.model.step_hints()      # what parts want to know of a one-token step (parts/base.py)
        self._hints_before: dict[int, tuple] = {}     # per bucket size: the hints of the step before
        self.graph_step_rows = graph_step_rows
        self.graph_chunk_rows = graph_chunk_rows
        self._plans: collections.OrderedDict[tuple, _GraphBucket] = collections.OrderedDict()
        self._pinned = [torch.empty(1 << 16, dtype=torch.int32).pin_memory() for _ in range(4)]
        self._pinned_events: list[torch.cuda.Event | None] = [None] * 4
        self._pinned_next = 0
        self._iota_cache = np.arange(64, dtype=np.int32)
        self.stats = {"steps": 0, "graph_replays": 0, "graph_captures": 0, "eager_steps": 0,
                      "graph_capture_failures": 0, "step_graph_captures": 0, "step_graph_replays": 0}
        self.capture_failures: list[str] = []         # one line per bucket whose capture failed

    # -- slots ----------------------------------------------------------------
    def acquire(self) -> int:
        return self.cache.acquire()

    def release(self, slot: int) -> None:
        self.cache.release(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    def truncate(self, slot: int, length: int) -> None:
        """Drops the tokens of the slot beyond its first `length` (a turn that is taken back:
        the reference rewinds its cache so, src/kv_cache.hpp:93-96, src/inference_session.cpp:682-693)
        and gives back the pages that held only them. The next step of the slot continues at
        position `length`, with the logits a fresh run of the kept tokens would give."""
        self.cache.truncate(slot, length)

    @property
    def max_seq_len(self) -> int:
        return self._max_seq_len

    # -- the step function -------------------------------------------------------
    def step(self, entries: list[StepEntry], device_tokens: torch.Tensor | None = None) -> torch.Tensor | None:
        """Runs the entries' tokens as one batch. Returns fp32 logits
        [number of wanted places, vocab] in the order of the entries and of their
        `want`, or None if nothing is wanted. The tensor is valid until the next step.

        device_tokens: int32 [len(entries)] on the device, for a step of one token a sequence:
        the tokens to run, in place of the entries' own (which only have to be valid ids). A
        sampler's ids go from one step into the next this way without a trip to the host, so
        several steps can be queued before the host reads any of them."""
        if not entries:
            raise StepError("a step needs at least one entry")
        if device_tokens is not None:
            if device_tokens.dtype != torch.int32 or device_tokens.device != self.device \
                    or device_tokens.numel() != len(entries) or any(len(e.tokens) != 1 for e in entries):
                raise StepError("device_tokens: int32 on the engine's device, one for each entry of one token")
        seen = set()
        growth = []
        for e in entries:
            if e.slot in seen:
                raise StepError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"slot {e.slot}: an entry needs at least one token")
            start = self.cache.length(e.slot)
            if start + n > self._max_seq_len:
                raise StepError(f"slot {e.slot}: {start} cached + {n} new tokens exceed the "
                                f"longest sequence {self._max_seq_len}")
            if n == 1 and type(e.tokens[0]) is int:     # the common one-token step, without numpy
                in_range = 0 <= e.tokens[0] < self.vocab_size
            else:
                toks = np.asarray(e.tokens, dtype=np.int64)
                in_range = toks.ndim == 1 and toks.min() >= 0 and toks.max() < self.vocab_size
            if not in_range:
                raise StepError(f"slot {e.slot}: token ids must lie in [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"slot {e.slot}: wanted place {w} outside its {n} tokens")
            growth.append((e.slot, start + n))
        self.cache.reserve(growth)          # all pages or an error, before anything runs
        all_single = all(len(e.tokens) == 1 for e in entries)
        every_wanted = all(list(e.want) == [0] for e in entries)
        self.stats["steps"] += 1
        with profiler.active(self.profiler), profiler.sync_each_launch(self.sync_each_launch):
            plan = None
            if self.use_graphs and all_single and every_wanted and len(entries) <= GRAPH_MAX_BUCKET:
                logits = self._graph_step(entries, device_tokens)
            elif self.use_graphs and device_tokens is None and (plan := self._step_plan(entries, all_single)):
                logits = self._planned_step(entries, plan)
            else:
                logits = self._eager_step(entries, all_single, device_tokens)
        self.cache.commit(growth)
        return logits

    def profile_summary(self) -> str:
        """The table of the kernels' times since the engine was made (or since the profiler
        was cleared): calls, total, average, share, as the reference prints its own
        (src/engine.cpp:372-435)."""
        if self.profiler is None:
            return "No profiling data"
        return self.profiler.format()

    # -- packing ---------------------------------------------------------------
    def _pack(self, entries, meta: _Meta, rows_padded: int, seqs_padded: int):
        """Fills a pinned host buffer with the step's metadata; returns it and the
        number of wanted rows."""
        if meta.total > self._pinned[0].numel():
            need = 1 << (meta.total - 1).bit_length()
            self._pinned = [torch.empty(need, dtype=torch.int32).pin_memory() for _ in range(4)]
            self._pinned_events = [None] * 4
        i = self._pinned_next
        self._pinned_next = (i + 1) % len(self._pinned)
        if self._pinned_events[i] is not None:
            self._pinned_events[i].synchronize()
        host = self._pinned[i][:meta.total]
        a = host.numpy()
        v = meta.views(a)
        v["row_seq"][:] = -1
        v["tokens"][:] = 0
        v["positions"][:] = 0
        v["seq_slot"][:] = -1
        v["seq_start"][:] = 0
        v["want_rows"][:] = 0               # places beyond the wanted ones name row 0: never an index out of range
        if all(len(e.tokens) == 1 for e in entries):
            # one token a sequence: whole columns at once
            k = len(entries)
            starts = [self.cache.length(e.slot) for e in entries]
            v["tokens"][:k] = [e.tokens[0] for e in entries]
            v["positions"][:k] = starts
            v["seq_start"][:k] = starts
            v["seq_slot"][:k] = [e.slot for e in entries]
            v["row_seq"][:k] = self._iota(k)
            v["cu_seqlens"][:k] = self._iota(k)
            v["cu_seqlens"][k:] = k
            nw = 0
            for row, e in enumerate(entries):
                for w in e.want:
                    v["want_rows"][nw] = row + int(w)
                    nw += 1
            return host, i, nw
        row = 0
        nw = 0
        for s, e in enumerate(entries):
            n = len(e.tokens)
            start = self.cache.length(e.slot)
            v["tokens"][row:row + n] = e.tokens
            v["positions"][row:row + n] = np.arange(start, start + n, dtype=np.int32)
            v["row_seq"][row:row + n] = s
            v["seq_slot"][s] = e.slot
            v["cu_seqlens"][s] = row
            v["seq_start"][s] = start
            for w in e.want:
                v["want_rows"][nw] = row + int(w)
                nw += 1
            row += n
        v["cu_seqlens"][len(entries):] = row
        return host, i, nw

    def _iota(self, n: int) -> np.ndarray:
        if n > self._iota_cache.size:
            self._iota_cache = np.arange(1 << (n - 1).bit_length(), dtype=np.int32)
        return self._iota_cache[:n]

    def _upload(self, host, index: int, dev: torch.Tensor) -> None:
        dev.copy_(host, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._pinned_events[index] = ev

    def _context(self, views, rows, seqs, max_q_len, all_single, pool) -> StepContext:
        return StepContext(rows=rows, num_seqs=seqs, positions=views["positions"],
                           row_seq=views["row_seq"], seq_slot=views["seq_slot"],
                           cu_seqlens=views["cu_seqlens"], seq_start=views["seq_start"],
                           max_q_len=max_q_len, max_keys=self.cache.max_seq_len,
                           all_single=all_single, env=self.env, scratch=pool)

    def _step_hints(self, entries, before: tuple | None = None) -> tuple:
        """What the parts' step_hint functions say of a one-token step of these entries, one value
        per function (before: the values of the bucket's step before)."""
        if not self._hint_fns:
            return ()
        lengths = [self.cache.length(e.slot) for e in entries]
        return tuple(fn(lengths, None if before is None else before[i]) for i, fn in enumerate(self._hint_fns))

    def _eager_step(self, entries, all_single: bool, device_tokens=None):
        rows = sum(len(e.tokens) for e in entries)
        wants = sum(len(e.want) for e in entries)
        meta = _Meta(rows, len(entries), wants)
        host, idx, nw = self._pack(entries, meta, rows, len(entries))
        self.scratch.reset()
        dev = self.scratch.alloc((meta.total,), torch.int32)
        self._upload(host, idx, dev)
        views = meta.views(dev)
        if device_tokens is not None:
            views["tokens"][:len(entries)].copy_(device_tokens)
        ctx = self._context(views, rows, len(entries), max(len(e.tokens) for e in entries),
                            all_single, self.scratch)
        if all_single:
            ctx.hints = dict(zip(self._hint_fns, self._step_hints(entries)))
        ctx.host = {"q_lens": [len(e.tokens) for e in entries],
                    "starts": [self.cache.length(e.slot) for e in entries],
                    "slots": [e.slot for e in entries]}
        ctx.most_keys = max(s + n for s, n in zip(ctx.host["starts"], ctx.host["q_lens"]))
        want = meta.views(host.numpy())["want_rows"][:nw]
        ctx.want_all = nw == rows and bool((want == np.arange(rows, dtype=np.int32)).all())
        self.stats["eager_steps"] += 1
        return self.model.forward(views["tokens"], ctx, self.caches, views["want_rows"], nw)

    def _graph_step(self, entries, device_tokens=None):
        n = len(entries)
        size = 1 << (n - 1).bit_length()
        hints = self._hints_before[size] = self._step_hints(entries, self._hints_before.get(size))
        bucket = self._buckets.get((size, hints))
        groups, blocks = len(self.cache.groups), self.cache.max_blocks
        # The page table rows of the step's rows travel with its metadata (where they are few KiB):
        # a mixer then has its pages' numbers without the chain row -> sequence -> slot -> table,
        # each link of which is a trip to memory in every layer (7B shape, batch 8: the page numbers
        # are there 1.8 us after the kernel's start instead of 3.0).
        by_row = groups * size * blocks if groups * size * blocks * 4 <= ROW_TABLES_MAX_BYTES else 0
        if bucket is None:
            bucket = self._buckets[(size, hints)] = _GraphBucket(size, self.device, row_tables=by_row)
        # every row of the bucket gets logits; padding rows are inert (row_seq -1)
        padded = [StepEntry(e.slot, e.tokens, [0]) for e in entries]
        host, idx, _ = self._pack(padded, bucket.meta, size, size)
        host.numpy()[bucket.meta.offsets["want_rows"][0]:][:size] = np.arange(size, dtype=np.int32)
        if by_row:
            o, count = bucket.meta.offsets["row_tables"]
            tables = host.numpy()[o:o + count].reshape(groups, size, blocks)
            tables[:, n:] = -1
            self.cache.rows_of_tables([e.slot for e in entries], tables)
        self._upload(host, idx, bucket.dev)
        if device_tokens is not None:
            bucket.views["tokens"][:n].copy_(device_tokens)
        bucket.uses += 1
        if bucket.graph is None:
            ctx = self._context(bucket.views, size, size, 1, True, bucket.pool)
            ctx.want_all = True
            ctx.hints = dict(zip(self._hint_fns, hints))
            ctx.padded = True
            if by_row:
                dev_tables = bucket.views["row_tables"].view(groups, size, blocks)
                ctx.row_tables = {g.page_table.data_ptr(): dev_tables[gi] for gi, g in enumerate(self.cache.groups)}
            if bucket.uses == 1:
                # first use: run eagerly; it also sizes the bucket's scratch pool
                return self._bucket_eager(bucket, ctx, n)
            if bucket.capture_failed is not None:
                return self._bucket_eager(bucket, ctx, n)
            bucket.pool.reset()          # sized by the eager run; from here on it must not move
            bucket.pool.frozen = True
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            try:
                with library_tuning.no_new_tuning(), torch.cuda.graph(graph):
                    bucket.pool.reset()
                    bucket.logits = self.model.forward(bucket.views["tokens"], ctx, self.caches,
                                                       bucket.views["want_rows"], size)
            except Exception as exc:     # the reference falls back the same way: src/engine.cpp:233-261
                # This bucket alone runs without a graph from here on. The same step is run again
                # eagerly below: an error that is the step's own (a kernel's refusal, a part's
                # bug) is raised again there and reaches the caller; only a failure of the
                # capture itself ends in the fallback.
                bucket.capture_failed = f"{size} rows{f', hints {hints}' if any(hints) else ''}: {exc!r}"
                self.capture_failures.append(bucket.capture_failed)
                self.stats["graph_capture_failures"] += 1
                bucket.pool.frozen = False
                del graph
                torch.cuda.synchronize()
                logits = self._bucket_eager(bucket, ctx, n)
                warnings.warn(f"capturing the one-token step of {bucket.capture_failed} as a HIP graph "
                              "failed; steps of this size run without a graph from here on", stacklevel=3)
                return logits
            bucket.graph = graph
            self.stats["graph_captures"] += 1
        bucket.graph.replay()
        self.stats["graph_replays"] += 1
        return bucket.logits[:n]

    # -- prompt steps and mixed steps as graphs ------------------------------------
    def _step_plan(self, entries, all_single: bool):
        """The bucket of sizes a step that is not all one-token (or does not want every row)
        runs in as a graph, or None when it runs eagerly: (rows, sequences, longest run of new
        tokens, most keys of a sequence after the step, wanted places, every row wanted in
        order, all one-token), each rounded up to a power of two (the rows of a longer step that
        is a whole chunk stay as they are). The sizes decide every
        grid, so steps of one bucket replay one graph; rows and sequences beyond the step's
        own are padding (row_seq -1, slot -1) that every kernel passes over."""
        rows = sum(len(e.tokens) for e in entries)
        wants = sum(len(e.want) for e in entries)
        if rows <= self.graph_step_rows:
            R = _pow2(rows, 16)
        elif self.graph_step_rows and rows <= self.graph_chunk_rows and rows % GRAPH_CHUNK_MULTIPLE == 0 \
                and wants <= GRAPH_CHUNK_MAX_WANTS:
            R = rows                 # a whole chunk: its own bucket, no padding rows
        else:
            return None
        want_all = wants == rows and all(list(e.want) == list(range(len(e.tokens))) for e in entries)
        most = max(self.cache.length(e.slot) + len(e.tokens) for e in entries)
        keys = min(_pow2(most, 256), max(self.cache.max_seq_len, 256))
        return (R, _pow2(len(entries)), min(_pow2(max(len(e.tokens) for e in entries)), R), keys,
                R if want_all else (_pow2(wants) if wants else 0), want_all, all_single)

    def _planned_step(self, entries, plan):
        R, S, Q, keys, W, want_all, all_single = plan
        bucket = self._plans.get(plan)
        if bucket is None:
            if len(self._plans) >= GRAPH_MAX_STEP_PLANS:
                self._plans.popitem(last=False)          # the least recently used graph and its buffers
            bucket = self._plans[plan] = _GraphBucket(R, self.device, S, max(W, 1))
        self._plans.move_to_end(plan)
        host, idx, nw = self._pack(entries, bucket.meta, R, S)
        self._upload(host, idx, bucket.dev)
        rows = sum(len(e.tokens) for e in entries)
        bucket.uses += 1
        n_out = rows if want_all else nw

        def forward(ctx):
            return self.model.forward(bucket.views["tokens"], ctx, self.caches, bucket.views["want_rows"], W)

        if bucket.graph is None:
            ctx = self._context(bucket.views, R, S, Q, all_single, bucket.pool)
            ctx.want_all = want_all
            ctx.most_keys = keys
            ctx.padded = True
            if bucket.uses == 1 or bucket.capture_failed is not None:
                bucket.pool.reset()          # first use: eagerly; it also sizes the bucket's scratch pool
                self.stats["eager_steps"] += 1
                logits = forward(ctx)
                return None if logits is None or n_out == 0 else logits[:n_out]
            bucket.pool.reset()
            bucket.pool.frozen = True
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            try:
                with library_tuning.no_new_tuning(), torch.cuda.graph(graph):
                    bucket.pool.reset()
                    bucket.logits = forward(ctx)
            except Exception as exc:
                bucket.capture_failed = f"step of {plan}: {exc!r}"
                self.capture_failures.append(bucket.capture_failed)
                self.stats["graph_capture_failures"] += 1
                bucket.pool.frozen = False
                del graph
                torch.cuda.synchronize()
                bucket.pool.reset()
                self.stats["eager_steps"] += 1
                logits = forward(ctx)       # the step's own errors are raised again here
                warnings.warn(f"capturing the {bucket.capture_failed} as a HIP graph failed; steps of these "
                              "sizes run without a graph from here on", stacklevel=3)
                return None if logits is None or n_out == 0 else logits[:n_out]
            bucket.graph = graph
            self.stats["step_graph_captures"] += 1
        bucket.graph.replay()
        self.stats["step_graph_replays"] += 1
        return None if bucket.logits is None or n_out == 0 else bucket.logits[:n_out]

    def _bucket_eager(self, bucket, ctx, n: int):
        """The bucket's step without a graph, on its own buffers."""
        bucket.pool.reset()
        self.stats["eager_steps"] += 1
        logits = self.model.forward(bucket.views["tokens"], ctx, self.caches,
                                    bucket.views["want_rows"], bucket.size)
        return logits[:n]

    # -- convenience -----------------------------------------------------------
    def synchronize(self) -> None:
        torch.cuda.synchronize(self.device)

    def memory_report(self) -> dict:
        return {"cache_bytes_per_token": self.cache.bytes_per_token(),
                "pages": self.cache.num_pages, "free_pages": self.cache.free_pages,
                "slots": self.cache.max_slots, "scratch_peak": self.scratch.peak,
                "allocated": torch.cuda.memory_allocated(self.device)}
