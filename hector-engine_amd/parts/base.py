"""What a layer is made of: the interfaces of the parts, their registries and
the data that selects them.

A model is described by data (:class:`ModelSpec`): one :class:`PartSpec` per
part with its sizes and constants, one block per layer, and a schedule that
says in which order layers run and whose cache each run reads. Parts are built
from that data through the registries below and never learn which model they
are in. Another mixer, feed-forward, norm, position encoding or block is a
class registered under a new kind; nothing else changes.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable

import torch

# ----------------------------------------------------------------------------
# data
# ----------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class PartSpec:
    """Selects a part (`kind` is the registry key) and gives its parameters."""

    kind: str
    params: dict = dataclasses.field(default_factory=dict)


@dataclasses.dataclass(frozen=True)
class TensorSpec:
    """A weight tensor a part expects: shape, and how the random mode fills it.

    init: ("normal", std) | ("gain", mean, std) | ("zeros",) | ("constant", value), or any kind
    registered with weights.random_init.register_init
    integer: integer tables are kept as int32, everything else follows the run dtype rule.
    """

    shape: tuple
    init: tuple = ("normal", 0.02)
    integer: bool = False


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    prefix: str       # tensor name prefix of the layer, e.g. "model.layers.3."
    block: PartSpec   # arrangement of mixer, feed-forward and norms


@dataclasses.dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer. cache_from names an earlier entry of the schedule
    whose cache this run reads instead of writing one of its own."""

    layer: int
    cache_from: int | None = None


@dataclasses.dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    embedding_prefix: str
    layers: list[LayerSpec]
    schedule: list[ScheduleEntry]
    final_norm: PartSpec
    final_norm_prefix: str
    head: PartSpec
    head_prefix: str
    max_positions: int
    # full names of tensors a model folder may hold although the model does not use them
    # (an output matrix stored beside the embedding it is tied to)
    unused_tensors: frozenset = frozenset()


PAGE_TOKENS = 64     # tokens of a cache page


@dataclasses.dataclass(frozen=True)
class KVNeed:
    """What a mixer keeps per token in the cache: per kv head a key of `head_dim` and a value
    of `value_dim` elements (0: as wide as the key), all of them (window 0) or only the last
    `window`. Mixers with equal needs share a group of the cache.

    k_page_elems, v_page_elems: the elements of one page (64 tokens of one kv head) in the
    group's two pools. The order inside a page is the mixer's own business: the cache hands out
    pages of these sizes and never looks inside. 0: 64 x head_dim and 64 x value_dim, token by
    token. A mixer with kernels that want their operands padded or tiled (the attention part:
    kernels/kv_layout.py), or that keeps something else per token (a latent, a code), says so
    here."""

    kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: int = 0
    k_page_elems: int = 0
    v_page_elems: int = 0

    @property
    def v_dim(self) -> int:
        return self.value_dim or self.head_dim

    @property
    def k_elems(self) -> int:
        return self.k_page_elems or PAGE_TOKENS * self.head_dim

    @property
    def v_elems(self) -> int:
        return self.v_page_elems or PAGE_TOKENS * self.v_dim


@dataclasses.dataclass
class BuildEnv:
    """Where and in which precision parts live."""

    device: torch.device
    dtype: torch.dtype            # activation dtype: torch.float32 or torch.bfloat16
    fast_kernels: bool = True     # False: the plain kernels also under bfloat16


# ----------------------------------------------------------------------------
# per-step context handed to every part
# ----------------------------------------------------------------------------


class StepContext:
    """The packed batch of one step, on the device. Rows are tokens; a padding
    row has row_seq -1. Every part receives this and nothing model-specific."""

    def __init__(self, *, rows: int, num_seqs: int, positions, row_seq, seq_slot, cu_seqlens,
                 seq_start, max_q_len: int, max_keys: int, all_single: bool, env: BuildEnv,
                 scratch, host=None):
        self.rows = rows                  # token rows in this step (with padding rows)
        self.num_seqs = num_seqs          # sequences (with padding sequences)
        self.positions = positions        # int32 [rows] absolute position of each row
        self.row_seq = row_seq            # int32 [rows] index into seq_slot, -1 = padding
        self.seq_slot = seq_slot          # int32 [num_seqs] cache slot of each sequence
        self.cu_seqlens = cu_seqlens      # int32 [num_seqs + 1] first row of each sequence
        self.seq_start = seq_start        # int32 [num_seqs] cached length before this step
        self.max_q_len = max_q_len        # longest run of new tokens of one sequence
        self.max_keys = max_keys          # upper bound of any sequence's length (the cache's)
        self.most_keys = max_keys         # the most keys a sequence of this step has after it, or a bound on that
        self.all_single = all_single      # every sequence brings exactly one token
        self.env = env
        self.scratch = scratch            # ScratchPool: alloc(shape, dtype)
        self.host = host                  # {"q_lens", "starts", "slots"}: lists per sequence, eager steps only
        self.hints: dict = {}             # what the parts' step_hint functions said of this step (function -> value)
        self.want_all = False             # the wanted rows are all rows, in order
        self.padded = False               # the step may hold padding rows and sequences (row_seq -1, slot -1: a step that
                                          # runs as a graph of its bucket of sizes); a part leaves such rows finite
        self.row_tables: dict = {}        # a cache group's page table (its data_ptr) -> int32 [rows, blocks]: the table
                                          # rows of the step's rows, gathered by the host into the step's metadata
                                          # (one-token steps that replay a graph; a mixer may read it in place of
                                          # LayerCache.page_table[seq_slot[row_seq[row]]] and skip that chain)
        self.next_norm = None             # the norm that reads the stream after the running block (set by the model)
        self.sink = None                  # ResidualSink offered to the running mixer / feed-forward

    def alloc(self, shape, dtype=None) -> torch.Tensor:
        return self.scratch.alloc(shape, dtype or self.env.dtype)

    def take_sink(self):
        """The residual sink offered to the running part, at most once (see ResidualSink)."""
        sink, self.sink = self.sink, None
        return sink


@dataclasses.dataclass
class LayerCache:
    """The cache as one run of a layer sees it."""

    kpool: torch.Tensor | None        # [pages, kv_heads, elements of a page (KVNeed.k_elems)], the order inside a page the mixer's own
    vpool: torch.Tensor | None
    page_table: torch.Tensor | None   # int32 [slots, blocks] of the layer's group
    writes: bool                      # False: the keys/values are another run's
    state: torch.Tensor | None        # uint8 [slots, state_bytes] of this run, or None


# ----------------------------------------------------------------------------
# interfaces
# ----------------------------------------------------------------------------


class Part:
    """Base of all parts: declares its tensors by full name and receives them."""

    # False for a part that plans on the host from ctx.host (sequence lengths as Python
    # lists); one-token steps of a model holding such a part are not captured into graphs.
    graph_safe = True
    # A part whose launches for a one-token step should depend on what the host knows of the
    # step names a function here: step_hint(lengths, before) -> a hashable value, where `lengths`
    # are the cached lengths of the step's sequences and `before` is the value it gave for the
    # bucket's step before (None at first). The engine calls each distinct function once a step
    # (parts that name the same function share the call), runs steps with different values as
    # different graphs, and hands the values over as ctx.hints[function]. None: no such wish.
    step_hint = None

    def __init__(self, prefix: str, env: BuildEnv):
        self.prefix = prefix
        self.env = env

    def tensor_specs(self) -> dict[str, TensorSpec]:
        """Full tensor name -> spec, children included."""
        return {}

    def bind(self, tensors: dict[str, torch.Tensor]) -> None:
        """Takes its tensors (on the device, in their run dtype); may fuse them."""

    def children(self) -> list["Part"]:
        return []


class Norm(Part):
    def carried(self) -> tuple[torch.Tensor, float] | None:
        """(gain [D], eps) when the norm is y = x * gain / sqrt(mean(x^2) + eps), so that a
        pair of products can carry it (ResidualSink, NormedRows); None otherwise."""
        return None

    def add_norm(self, resid: torch.Tensor, delta, rows: int, ctx: StepContext,
                 want_out: bool = True) -> torch.Tensor | None:
        """resid (fp32 [rows, D], in place) += delta (a tensor in the activation dtype, or
        None); returns norm(resid) in the activation dtype (or None when want_out is False)."""
        raise NotImplementedError


class PositionEncoding(Part):
    # True for an encoding that must run through apply() on q and k; False for a
    # rotation the fused q/k kernel applies (rotary() gives its table) or for none.
    custom = False

    def rotary(self) -> tuple[torch.Tensor, int] | None:
        """(inv_freq fp32 [r/2], r) when the encoding is a rotation the fused
        q/k kernel can apply; None otherwise."""
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, ctx: StepContext) -> None:
        """In-place encoding of q [rows, H, hd] and k [rows, KVH, hd] for
        encodings that are not a plain rotation. Default: none."""


class Mixer(Part):
    # True for a part whose forward takes x as NormedRows as well as a tensor
    # (its first product applies the row scale); others get a tensor.
    accepts_normed_rows = False

    def kv_need(self) -> KVNeed | None:
        """Keys/values per token this mixer keeps, or None."""
        return None

    def state_bytes(self) -> int:
        """Bytes of fixed-size state per sequence."""
        return 0

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache):
        """x: [rows, D] normed activations. Returns [rows, D], or None when its last product
        has added the result to the residual stream through the sink it was offered."""
        raise NotImplementedError


class FeedForward(Part):
    accepts_normed_rows = False

    def forward(self, x: torch.Tensor, ctx: StepContext):
        """Returns [rows, D], or None when its last product has added the result to the residual
        stream through the sink it was offered."""
        raise NotImplementedError


class Block(Part):
    """Arrangement of a layer's parts around the residual stream."""

    mixer: Mixer

    def first_norm(self) -> "Norm | None":
        """The norm through which this block first reads the residual stream, when that is all
        it reads the stream through before adding to it; None otherwise. The block that runs
        before may then leave the stream as rows prepared for that norm (ResidualSink)."""
        return None

    def forward(self, stream: "ResidualStream", ctx: StepContext, cache: LayerCache) -> None:
        raise NotImplementedError


@dataclasses.dataclass
class NormedRows:
    """Rows of an RMS norm whose per-row scale is still owed: `scaled` = r * gain in the
    activation dtype, and the sum of r^2 of a row as `partials[row, :]` (fp32, added in
    index order by lanes of 64, then across the lanes). norm(r) = scaled / sqrt(sum / dim +
    eps). A product applies the scale to its sums (parts.linear.Linear); tensor() gives the
    normalised rows to anything else. pieces: `scaled` lies piece-major
    (kernels.ops.pieces_shape(rows, dim))."""

    scaled: torch.Tensor
    partials: torch.Tensor
    eps: float
    rows: int
    pieces: bool = False

    @property
    def dim(self) -> int:
        return self.scaled.shape[0] * 8 if self.pieces else self.scaled.shape[-1]

    def tensor(self, ctx: StepContext) -> torch.Tensor:
        from ..kernels import ops
        out = ctx.alloc((self.rows, self.dim), self.scaled.dtype)
        ops.scale_rows(out, self.scaled, self.partials, self.eps, self.rows, self.pieces)
        return out


@dataclasses.dataclass
class PieceRows:
    """bf16 rows handed from one kernel to a product in the piece-major layout
    (kernels.ops.pieces_shape): only to a Linear that says reads_pieces(rows, ctx)."""

    pieces: torch.Tensor


class ResidualSink:
    """Offered (ctx.sink) to a mixer or feed-forward whose output goes straight into the
    residual stream and then into `norm`: its last product may add its result to
    stream.resid itself and leave the rows for that norm (Linear(..., sink=ctx.take_sink())),
    returning None instead of a tensor. A part that ignores the offer loses nothing."""

    def __init__(self, stream: "ResidualStream", norm: Norm):
        self.stream = stream
        self.norm = norm


class ResidualStream:
    """The fp32 residual rows of a step plus one branch output not yet added:
    the add is fused into the next norm."""

    def __init__(self, resid: torch.Tensor, rows: int):
        self.resid = resid
        self.rows = rows
        self.pending: torch.Tensor | None = None
        self.prepared: tuple[Norm, NormedRows] | None = None   # rows already made for that norm

    def add(self, delta, ctx: StepContext) -> None:
        """delta: a tensor [rows, D], or None when the producer has added its result through a
        ResidualSink."""
        if delta is None:
            return
        self.prepared = None
        if self.pending is not None:
            self.materialize(ctx)
        self.pending = delta

    def sink_for(self, norm: Norm | None, ctx: StepContext) -> "ResidualSink | None":
        """A sink for the part that runs next, when `norm` (the norm that will read the stream
        after it) can be carried and the kernels for that are in use."""
        if norm is None or self.pending is not None or norm.carried() is None:
            return None
        if not ctx.env.fast_kernels or ctx.env.dtype != torch.bfloat16:
            return None
        return ResidualSink(self, norm)

    def normed(self, norm: Norm, ctx: StepContext, rows_ok: bool = False):
        """norm(resid + pending) in the activation dtype. With rows_ok the caller takes
        NormedRows too (rows a product has left for this norm)."""
        prepared, self.prepared = self.prepared, None
        if prepared is not None and prepared[0] is norm and self.pending is None:
            return prepared[1] if rows_ok else prepared[1].tensor(ctx)
        out = norm.add_norm(self.resid, self.pending, self.rows, ctx)
        self.pending = None
        return out

    def materialize(self, ctx: StepContext) -> torch.Tensor:
        if self.pending is not None:
            from ..kernels import ops
            ops.residual_add(self.resid, self.pending, self.rows)
            self.pending = None
        return self.resid


# ----------------------------------------------------------------------------
# registries
# ----------------------------------------------------------------------------

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
_registries: dict[str, dict[str, Callable[..., Part]]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, factory: Callable[..., Part] | None = None):
    """Registers `factory(params: dict, prefix: str, env: BuildEnv) -> Part` under
    (category, kind); usable as a decorator on a class with that constructor."""
    if category not in _registries:
        raise KeyError(f"unknown part category '{category}', have {CATEGORIES}")

    def deco(f):
        _registries[category][kind] = f
        return f

    return deco(factory) if factory is not None else deco


def build_part(category: str, spec: PartSpec, prefix: str, env: BuildEnv) -> Part:
    try:
        factory = _registries[category][spec.kind]
    except KeyError:
        raise KeyError(f"no {category} of kind '{spec.kind}' is registered; "
                       f"registered: {sorted(_registries.get(category, {}))}") from None
    return factory(dict(spec.params), prefix, env)


def registered(category: str) -> list[str]:
    return sorted(_registries[category])


def param(params: dict, key: str, kind: type, default: Any = dataclasses.MISSING) -> Any:
    """A part's own typed parameter access with a clear error."""
    if key not in params or params[key] is None:
        if default is dataclasses.MISSING:
            raise KeyError(f"part parameter '{key}' is required")
        return default
    value = params[key]
    if kind in (int, float) and isinstance(value, bool):
        raise TypeError(f"part parameter '{key}': expected {kind.__name__}, got {value!r}")
    if kind is float and isinstance(value, int):
        value = float(value)
    if not isinstance(value, kind):
        raise TypeError(f"part parameter '{key}': expected {kind.__name__}, got {value!r}")
    return value
