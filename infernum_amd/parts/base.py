"""What a model is put together from: part specifications, the registry of part
kinds, and the interfaces that a mixer, a feed-forward, a norm, a position
encoding and a block arrangement have to keep.

A part is made from a :class:`PartSpec` (its kind and its own sizes and
constants) and knows nothing about the model it sits in: not its name, not its
other layers, not the names of its weights in a file (those are given to it as a
prefix).  The reference gets the same separation from its ``define_block!``
macro (infernum-macros/src/lib.rs:32-106) and builds a layer from such blocks in
infernum-llama/src/graph_builder.rs:446-507.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Mapping, Optional, Sequence, Tuple

import torch

# ----------------------------------------------------------------------- specs


@dataclass(frozen=True)
class PartSpec:
    """Kind of a part, its parameters, and the prefix of its weights' names."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    prefix: str = ""

    def with_prefix(self, prefix: str) -> "PartSpec":
        return PartSpec(self.kind, self.params, prefix)


@dataclass(frozen=True)
class WeightSpec:
    """One tensor a part wants: its shape, how random weights are drawn for it,
    whether it is a matrix that follows the compute dtype, and the full name of
    another tensor that stands in when the file does not hold this one."""

    shape: Tuple[int, ...]
    init: Tuple = ("normal", 0.02)          # ("normal", std) | ("ones",) | ("uniform", lo, hi) | ("zeros",)
    follows_compute_dtype: bool = True      # False: kept as stored (fp32 stays fp32, integers become int32)
    fallback: Optional[str] = None          # full tensor name used when this one is absent
    write_when_random: bool = True          # False: random-weights mode leaves it out (e.g. a tied head)


@dataclass(frozen=True)
class PageTensor:
    """One tensor of a page's payload.  ``shape`` is what one token stores; the page holds ``page_size`` tokens
    along a new axis put in at ``token_axis``: the pool is [num_pages, *shape[:token_axis], page_size,
    *shape[token_axis:]].  ``dtype`` None: the compute type."""

    name: str
    shape: Tuple[int, ...]
    token_axis: int = 0
    dtype: Optional[torch.dtype] = None

    def pool_shape(self, num_pages: int, page_size: int) -> Tuple[int, ...]:
        if not 0 <= self.token_axis <= len(self.shape):
            raise ValueError(f"page tensor {self.name!r}: token_axis {self.token_axis} is outside its shape {self.shape}")
        return (num_pages,) + tuple(self.shape[:self.token_axis]) + (page_size,) + tuple(self.shape[self.token_axis:])


@dataclass(frozen=True)
class CacheSpec:
    """What a mixer needs of the paged cache: which positions are kept (all of them, 'full', or the last
    ``window``, 'window'), and what a page holds for them (``payload``: named tensors with a per-token shape).
    With ``num_kv_heads`` and ``head_dim`` and no payload it is keys and values as the attention kernels read
    them: "k" [nkv, page_size, d] and "v", transposed within the page, [nkv, d, page_size]."""

    kind: str                      # "full" | "window"
    num_kv_heads: int = 0
    head_dim: int = 0
    window: int = 0
    payload: Tuple[PageTensor, ...] = ()

    def __post_init__(self) -> None:
        if not self.payload:
            if self.num_kv_heads <= 0 or self.head_dim <= 0:
                raise ValueError("a CacheSpec needs a payload, or num_kv_heads and head_dim for keys and values")
            object.__setattr__(self, "payload", (
                PageTensor("k", (self.num_kv_heads, self.head_dim), token_axis=1),
                # values are kept transposed within a page: what the PV product of the matrix cores reads
                PageTensor("v", (self.num_kv_heads, self.head_dim), token_axis=2)))
        names = [t.name for t in self.payload]
        if len(set(names)) != len(names):
            raise ValueError(f"page tensors of one CacheSpec need different names, got {names}")

    def group_key(self) -> Tuple:
        """Layers with equal keys share page tables (one group of the cache manager)."""
        return (self.kind, self.window)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state per request that a mixer keeps between steps (fp32 unless said)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class LayerSpec:
    """One layer: how its parts are arranged (``block``) and the parts themselves.  An arrangement that has no
    use for one of the four leaves it None; what it needs beyond them goes into ``extra`` under names of its
    own: a PartSpec (a norm), or (category, PartSpec) for a part of any category."""

    block: str
    mixer: PartSpec
    feed_forward: Optional[PartSpec] = None
    mixer_norm: Optional[PartSpec] = None
    feed_forward_norm: Optional[PartSpec] = None
    extra: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``cache_of`` names an earlier entry of the schedule
    whose keys and values (or state) this run reads instead of writing its own."""

    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    """A whole decoder as data: embedding, layers, the order they run in, head."""

    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: Sequence[LayerSpec]
    schedule: Sequence[ScheduleEntry]
    final_norm: Optional[PartSpec]
    head: PartSpec
    max_position: int = 0
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None


# -------------------------------------------------------------------- run time


@dataclass
class Runtime:
    """Where and in what precision a model runs."""

    device: torch.device
    dtype: torch.dtype                       # torch.bfloat16 or torch.float32: activations, matrices, cache
    max_tokens_per_step: int = 8192
    # "auto": the fast kernel for each operation where it takes the size; "generic": the plain twins only
    # (one fp32 multiply-add chain per output element, one wave per token and head in attention), in either type
    kernels: str = "auto"

    def __post_init__(self) -> None:
        if self.kernels not in ("auto", "generic"):
            raise ValueError(f"kernels must be 'auto' or 'generic', got {self.kernels!r}")

    @property
    def is_fp32(self) -> bool:
        return self.dtype == torch.float32


@dataclass
class CacheView:
    """What one run of a layer sees of the cache.

    ``pages``: the pools of its schedule entry (or of the entry it reads) by the names of the mixer's
    CacheSpec payload, each [num_pages, ...] with the page's tokens along the declared axis; ``k_pages`` and
    ``v_pages`` are the "k" and "v" of them.  ``group`` indexes the step's block tables and slots;
    ``writable`` is False when the pages belong to another entry.  ``state`` is the entry's
    [num_slots, *shape] tensor when the mixer declared a StateSpec.  ``others``: the views of the layer's
    further cached parts, under the names of ``Block.cached_parts`` (a layer with an attention and a mixer
    with state side by side has two).
    """

    group: int = -1
    pages: Mapping[str, torch.Tensor] = field(default_factory=dict)
    writable: bool = True
    state: Optional[torch.Tensor] = None
    others: Mapping[str, "CacheView"] = field(default_factory=dict)

    @property
    def k_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("k")

    @property
    def v_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("v")


@dataclass
class StepContext:
    """One step's batch, as the parts see it (all tensors on the device).

    Tokens of one request are consecutive rows.  Requests that bring a single
    token come first (``num_decode`` of them, rows 0 .. num_decode-1), requests
    that bring a portion of a prompt after them.
    """

    num_tokens: int
    num_seqs: int
    num_decode: int
    token_ids: torch.Tensor                 # [N] int32
    positions: torch.Tensor                 # [N] int32 position of each token in its request
    token_seq: torch.Tensor                 # [N] int32 index of each token's request in this batch
    seq_starts: torch.Tensor                # [B+1] int32 first row of each request
    seq_ctx: torch.Tensor                   # [B] int32 tokens each request had in the cache before this step
    state_slots: torch.Tensor               # [B] int32 slot of each request's fixed-size state
    block_tables: List[torch.Tensor]        # per cache group: [B, MB] int32, -1 where no page is held
    slots: List[torch.Tensor]               # per cache group: [N] int32 page*page_size+offset of each token
    logit_rows: torch.Tensor                # [R] int32 rows whose logits are wanted
    # host copies, for choosing kernels and grids without reading the device
    q_lens: Sequence[int] = ()
    ctx_lens: Sequence[int] = ()
    max_q_len: int = 0
    max_total_len: int = 0                  # largest ctx + q over the batch
    # lists of row tiles by tile height, as far as the step's packing made them (see ``row_tiles``)
    packed_row_tiles: Dict[int, Tuple[torch.Tensor, int]] = field(default_factory=dict)
    extras: Dict[str, Any] = field(default_factory=dict)

    def row_tiles(self, rows: int) -> Tuple[torch.Tensor, int]:
        """The portions of prompts of this step cut into tiles of ``rows`` rows: an int32 tensor [n, 2] of
        (request, first row of the tile among the request's rows) on the device, and n.  A part that wants
        them says so in ``step_needs`` ({"row_tiles": rows}); then they came with the step's one copy.
        Otherwise they are made here, once per step and height, and copied over."""
        hit = self.packed_row_tiles.get(rows)
        if hit is None:
            pairs = [(s, first) for s in range(self.num_decode, self.num_seqs)
                     for first in range(0, self.q_lens[s], rows)]
            t = torch.tensor(pairs or [(0, 0)], dtype=torch.int32).to(self.token_ids.device)
            hit = self.packed_row_tiles[rows] = (t, len(pairs))
        return hit


# ------------------------------------------------------------------ interfaces


class Part:
    """Base of all parts.  ``weights`` lists what it wants; ``load`` receives them."""

    category = "part"
    # True when ``forward`` only launches kernels on the current stream with shapes that follow from the
    # step's sizes, and reads nothing from the device on the host: such a step can be recorded and replayed.
    graph_safe = False

    def __init__(self, rt: Runtime, **params: Any):
        self.rt = rt

    def weights(self) -> Dict[str, WeightSpec]:
        """Local tensor name (appended to the spec's prefix) -> WeightSpec."""
        return {}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Take the tensors of ``weights`` (by local name), already on the device."""

    def native(self, program: Any, view: Optional["CacheView"], **kw: Any) -> None:
        """Write this part into the program of a step (``engine.program.StepProgram``): the operations that
        make the launches of ``forward``, reading and leaving the program's registers as ``forward`` reads its
        arguments and returns its result.  Every category has a default that calls back into ``forward``; a
        part with launchers of its own writes them instead (``program.op``)."""
        raise NotImplementedError(f"{type(self).__name__} has no category that a program knows")

    def step_needs(self) -> Dict[str, Any]:
        """Arrays that the part wants packed with every step beyond those every step has.  Known:
        ``{"row_tiles": rows}``: the list of :meth:`StepContext.row_tiles` for that height."""
        return {}


class Norm(Part):
    category = "norm"

    def forward(self, h: torch.Tensor, delta: Any, out: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """h [N, H] fp32 += delta (in place, when given); returns norm(h) in the compute dtype.
        ``delta`` is what a mixer or a feed-forward returned: a tensor [N, H] in the compute dtype, or
        a ``kernels.api.SplitSum`` (fp32 partial sums [S, N, H] that are added here)."""
        raise NotImplementedError

    def native(self, program: Any, view: Optional["CacheView"] = None, rows: bool = False) -> None:
        """Reads ``program.h`` and ``program.pending``, leaves the normalised rows in ``program.x`` (of the wanted
        rows only with ``rows``).  This default calls ``forward``."""
        pending, H, dt = program.pending, program.hidden_size, self.rt.dtype

        def call(ctx: "StepContext") -> None:
            n = ctx.num_tokens
            h = program.h.view(torch.float32, n, H)
            picked = ctx.logit_rows if rows else None
            n_out = int(picked.numel()) if rows else n
            if n_out == 0:
                return
            out = program.x.view(dt, n_out, H)
            y = self.forward(h, program.read(pending, n), out=out, rows=picked)
            if y.data_ptr() != out.data_ptr():
                out.copy_(y)
        program.python(call, type(self).__name__)
        program.pending = None


class PositionEncoding(Part):
    """Owns what the rotation kernel needs: ``inv_freq`` (float64 or fp32 [rotary_dim / 2] on the device, or None
    for no rotation) and ``rotary_dim``.  The kernels pair the first half of a head's rotated values with the
    second, (x[i], x[i + rotary_dim / 2]); an encoding that pairs other values gives the order in which it wants
    a head's values through ``head_permutation``."""

    category = "position"

    def head_permutation(self) -> Optional[torch.Tensor]:
        """None, or a permutation p of range(head_dim) (int64, on any device): the attention mixer then keeps its
        query and key projections with the rows of every head in the order p, so that value p[j] of the
        encoding's own order stands at place j.  Scores are sums over a head's values and do not care about their
        order, as long as queries and keys share it; an encoding that rotates neighbouring pairs
        (x[2i], x[2i + 1]) asks for [0, 2, 4, ..., 1, 3, 5, ...] and is then served by the kernels' half-split
        pairs.  (A ``qk_transform`` sees the heads in the permuted order.)"""
        return None


class QKTransform(Part):
    """What an attention mixer may do to its projected queries and keys before they are rotated and the keys
    are written to the cache (a norm per head, a bias, a scale): the seam between projection and rotation."""

    category = "qk_transform"

    def forward(self, qkv: torch.Tensor, num_q_heads: int, num_kv_heads: int, head_dim: int,
                ctx: "StepContext") -> torch.Tensor:
        """qkv [N, (num_q_heads + 2 num_kv_heads) head_dim] in the compute dtype: the query heads, then the key
        heads, then the value heads of every token (num_kv_heads is 0 for a run that reads another run's keys
        and values: then the rows hold queries only).  Returns the tensor to go on with (it may be qkv itself,
        changed in place)."""
        raise NotImplementedError


class Mixer(Part):
    category = "mixer"

    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView) -> Any:
        """x [N, H] in the compute dtype -> [N, H] (a tensor in the compute dtype, or a SplitSum that the
        next norm joins); reads and writes its cache view."""
        raise NotImplementedError

    def native(self, program: Any, view: Optional["CacheView"]) -> None:
        """Reads ``program.x``, leaves its result as ``program.pending``.  This default calls ``forward``."""
        _call_forward(self, program, "mixer.out", lambda x, ctx: self.forward(x, ctx, view))


class FeedForward(Part):
    category = "feed_forward"

    def forward(self, x: torch.Tensor, ctx: StepContext) -> Any:
        """x [N, H] in the compute dtype -> [N, H] (a tensor, or a SplitSum that the next norm joins)."""
        raise NotImplementedError

    def native(self, program: Any, view: Optional["CacheView"] = None) -> None:
        """Reads ``program.x``, leaves its result as ``program.pending``.  This default calls ``forward``."""
        _call_forward(self, program, "feed_forward.out", lambda x, ctx: self.forward(x, ctx))


class Embedding(Part):
    category = "embedding"

    def forward(self, ctx: StepContext) -> torch.Tensor:
        """-> the residual stream h [N, H] in fp32."""
        raise NotImplementedError

    def native(self, program: Any, view: Optional["CacheView"] = None) -> None:
        """Fills ``program.h``.  This default calls ``forward``."""
        H = program.hidden_size
        program.python(lambda ctx: program.h.view(torch.float32, ctx.num_tokens, H).copy_(self.forward(ctx)),
                       type(self).__name__)
        program.pending = None


class Head(Part):
    category = "head"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x [R, H] -> logits [R, V] fp32."""
        raise NotImplementedError

    def native(self, program: Any, view: Optional["CacheView"] = None) -> None:
        """Reads the wanted rows from ``program.x``, fills the step's logits.  This default calls ``forward``."""
        H, dt = program.hidden_size, self.rt.dtype

        def call(ctx: "StepContext") -> None:
            R = int(ctx.logit_rows.numel())
            if R:
                program.step_logits().copy_(self.forward(program.x.view(dt, R, H)))
        program.python(call, type(self).__name__)


class Block:
    """Arrangement of a layer's parts around the residual stream.

    ``forward`` takes the fp32 residual stream ``h`` and a ``pending`` delta that
    has not been added to it yet (so that the add can be fused into the next
    norm), and returns the next pending delta.
    """

    category = "block"
    graph_safe = False

    def __init__(self, rt: Runtime, mixer: Mixer, feed_forward: Optional[FeedForward], mixer_norm: Optional[Norm],
                 feed_forward_norm: Optional[Norm], extra: Mapping[str, Part]):
        self.rt = rt
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm
        self.extra = dict(extra)

    def forward(self, h: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext,
                cache: CacheView) -> torch.Tensor:
        raise NotImplementedError

    def cached_parts(self) -> Dict[str, Part]:
        """The parts of this layer that keep something between steps (those with a ``cache_spec`` or a
        ``state_spec``), by name.  "mixer" gets the view that ``forward`` is handed; every other name is found in
        that view's ``others``.  Each gets pages and state slots of its own from the cache manager."""
        return {"mixer": self.mixer}

    def native(self, program: Any, view: CacheView) -> None:
        """Write the arrangement into a step's program: its parts' operations in the order ``forward`` runs them
        (each part's ``native``).  This default calls ``forward`` for the whole layer."""
        pending, H, dt = program.pending, program.hidden_size, self.rt.dtype
        buf, value = program.store("block.out", H)

        def call(ctx: StepContext) -> None:
            n = ctx.num_tokens
            out = self.forward(program.h.view(torch.float32, n, H), program.read(pending, n), ctx, view)
            _put(buf.view(dt, n, H), out, dt)
        program.python(call, type(self).__name__)
        program.pending = value


def _put(dst: torch.Tensor, y: Any, dtype: torch.dtype) -> None:
    """What a part's ``forward`` returned (a tensor or partial sums), into a buffer of the program."""
    if hasattr(y, "joined"):
        y = y.joined(dtype)
    dst.copy_(y)


def _call_forward(part: Part, program: Any, key: str, forward: Callable[[torch.Tensor, StepContext], Any]) -> None:
    H, dt = program.hidden_size, part.rt.dtype
    buf, value = program.store(key, H)

    def call(ctx: StepContext) -> None:
        n = ctx.num_tokens
        _put(buf.view(dt, n, H), forward(program.x.view(dt, n, H), ctx), dt)
    program.python(call, type(part).__name__)
    program.pending = value


# -------------------------------------------------------------------- registry

_REGISTRY: Dict[Tuple[str, str], Callable[..., Any]] = {}


def register_part(category: str, kind: str, factory: Callable[..., Any], replace: bool = False) -> None:
    """Make ``kind`` available for specs of ``category`` ('mixer', 'feed_forward',
    'norm', 'position', 'embedding', 'head', 'block')."""
    key = (category, kind)
    if key in _REGISTRY and not replace and _REGISTRY[key] is not factory:
        raise ValueError(f"{category} kind {kind!r} is registered already")
    _REGISTRY[key] = factory


def part_kinds(category: str) -> List[str]:
    return sorted(k for (c, k) in _REGISTRY if c == category)


def make_part(category: str, spec: PartSpec, rt: Runtime) -> Any:
    factory = _REGISTRY.get((category, spec.kind))
    if factory is None:
        raise KeyError(f"no {category} of kind {spec.kind!r}; registered: {part_kinds(category)}")
    return factory(rt, **dict(spec.params))


def block_factory(kind: str) -> Callable[..., Block]:
    factory = _REGISTRY.get(("block", kind))
    if factory is None:
        raise KeyError(f"no block arrangement {kind!r}; registered: {part_kinds('block')}")
    return factory
