"""Interfaces of the parts a model is put together from, their specs and their registry.

A model is data: a ``ModelSpec`` lists its layers, each layer names a block arrangement, a
mixer, a feed-forward and its norms as ``PartSpec`` (a kind and its parameters), and a
schedule says in which order the layers run and whose cache each run reads. The classes
behind the kinds know nothing about the model they are in: all sizes and constants are
constructor parameters.

The reference hard-wires Llama's block (core/src/model_executor/models/llama/llama.rs:276-385)
and repeats it per architecture (gemma.rs, chatglm.rs); its only plug point is the weight format
of the linear layers (core/src/model_executor/layers/linear.rs:28-42).
"""
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Mapping, Optional, Sequence, Tuple

import torch


# --------------------------------------------------------------------------- runtime


@dataclass
class Runtime:
    """What every part needs to run: the kernels, the device and the compute dtype."""

    ops: Any                       # kernel object (lmsf_amd.ops.HipOps)
    device: torch.device
    dtype: torch.dtype             # activations, cache and weights loaded as "float": float32 or bfloat16
    max_positions: int             # longest sequence the engine will be asked to hold
    shared: Dict[Any, Any] = field(default_factory=dict)   # tables that equal parts share (rotary tables)


# --------------------------------------------------------------------------- specs (data)


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by the configuration: which implementation and with which parameters."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def with_params(self, **more) -> "PartSpec":
        p = dict(self.params)
        p.update(more)
        return PartSpec(self.kind, p)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: its weight prefix, its arrangement and its parts."""

    prefix: str                    # e.g. "model.layers.3"
    block: PartSpec                # arrangement of the parts, e.g. PartSpec("prenorm_residual")
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]  # the norms the arrangement asks for, by role


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer. ``cache_from`` is None for a run that owns a cache, or the index of an
    earlier entry of the schedule whose cache this run reads instead of writing its own."""

    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    vocab_size: int
    hidden_size: int


# --------------------------------------------------------------------------- what parts declare


@dataclass(frozen=True)
class TensorDecl:
    """A checkpoint tensor a part expects. kind "float": loaded in the runtime dtype; "int": loaded as int32.
    ``keeps_float32``: a tensor stored in 32 bits stays so in a bfloat16 run (the norms' weights: their kernels
    compute in float32 anyway and take the weight as it is); the matrices of the products are cast as the
    reference casts everything (core/src/model_executor/models/model_factory.rs:124-139). ``init`` says how
    the random-weights mode fills it: "normal" (mean 0, the mode's standard deviation), "ones" or "zeros"."""

    shape: Tuple[int, ...]
    kind: str = "float"
    init: str = "normal"
    keeps_float32: bool = False


@dataclass(frozen=True)
class CacheSpec:
    """Paged key/value needs of a mixer. Runs with equal specs share a page pool and block tables.
    window None: all keys are kept; window W: only the last W positions are ever read, pages that
    the window has passed are given back. ``head_dim`` is the width of a key; a value has ``v_head_dim``
    (None: the same). The attention kernels of this package take equal widths; a mixer with unequal ones
    reads and writes its pages itself."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state of a mixer: one tensor of ``shape`` and ``dtype`` per live request. A slot
    is all zeros when a request's first tokens run: the engine clears it when the request takes it."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class CacheBinding:
    """What a run of a layer is given at build time to reach its cache and state."""

    group: Optional[int] = None            # index of the cache group (page pool + block tables)
    k_pages: Optional[torch.Tensor] = None  # [pages, kv_heads, page_size, head_dim]
    v_pages: Optional[torch.Tensor] = None  # [pages, kv_heads, v_head_dim, page_size]
    writes_cache: bool = True              # False: reads another run's pages
    state: Optional[torch.Tensor] = None   # [slots, *StateSpec.shape]


class Part:
    """Base of every part. ``prefix`` is where its tensors live in the checkpoint.

    ``graph_safe`` says that the part's forward only launches work whose shapes and addresses follow
    from the step's shapes (token count, table widths, ``max_context``), never from the values that
    change from step to step on the host, so that a step can be captured as a HIP graph and replayed
    with new contents in the same buffers. The engine captures decode steps only if every part of the
    model says so; a part that loops over the step's requests in Python leaves it False."""

    graph_safe = False

    # A mixer or feed-forward whose ``forward`` takes ``pending_ok=True`` and may then return its last
    # product unfinished (ops.handles.PendingProduct) sets this; a norm that takes such a branch in
    # ``forward_add`` sets ``accepts_pending``. A block hands a pending product only to a norm that accepts
    # it; ``rt.ops.materialize`` finishes one anywhere else. Parts that know nothing of this never see one.
    may_return_pending = False
    accepts_pending = False

    # A norm whose ``forward_add`` takes ``defer_ok=True`` and may then return the norm not yet computed
    # (ops.handles.ScaledRows) sets ``may_defer``; a mixer or feed-forward whose ``forward`` takes such an
    # ``h`` (it hands it to ``rt.ops.qkv_rope_cache`` or ``rt.ops.linear_gated``, or calls ``rt.ops.materialize``
    # first) sets ``accepts_normed``. A block asks for a deferred norm only where both say so.
    may_defer = False
    accepts_normed = False

    def __init__(self, prefix: str, rt: Runtime):
        self.prefix = prefix
        self.rt = rt

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        """Full checkpoint names of the tensors this part (not its children) reads."""
        return {}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        """Take the declared tensors (``fetch(name)`` gives a device tensor) and keep what is needed."""

    def children(self) -> Sequence["Part"]:
        return ()

    def tensors(self) -> Sequence[torch.Tensor]:
        """The device tensors this part (not its children) holds after loading: what memory sizing and the
        count of a step's bytes look at. The default finds ``weight`` and ``bias``; a part that keeps its
        tensors elsewhere (a list of experts) returns them here."""
        return [t for t in (getattr(self, "weight", None), getattr(self, "bias", None)) if isinstance(t, torch.Tensor)]

    def walk(self):
        yield self
        for c in self.children():
            yield from c.walk()


class Norm(Part):
    """forward(x): norm of x [N, H] in the runtime dtype.
    forward_add(branch, residual): residual (float32, in place) += branch; returns norm(residual).
    branch None: returns norm(residual). rows: compute only these rows (residual untouched).
    A norm with ``may_defer`` also takes ``defer_ok``."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward_add(self, branch: Optional[torch.Tensor], residual: torch.Tensor,
                    rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """Encodes positions into queries and keys. A mixer that owns one asks it for what its fused
    kernel needs (``rotary_table``) or lets it act on the tensors (``apply``)."""

    def rotary_table(self):
        """(float32 table [max_positions, rot] = [cos | sin], rot, neox pairing) if the encoding is a rotation
        that the fused rotate-and-store kernel can apply; None (the default) if it acts through ``apply``."""
        return None

    def apply(self, qkv: torch.Tensor, nh: int, nkv: int, d: int, positions: torch.Tensor) -> None:
        raise NotImplementedError


class Mixer(Part):
    """Mixes information across the tokens of a request.

    forward(h, ctx, binding): h [N, H] in the runtime dtype for the step's N tokens; ``ctx`` is the
    step's batch description (engine.batch.StepContext); ``binding`` reaches this run's cache pages
    and state. Returns [N, H]."""

    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """forward(h): [N, H] -> [N, H], token by token."""

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of norms, a mixer and a feed-forward around the residual stream.

    forward(branch, residual, ctx, binding) -> branch: ``residual`` is the float32 stream [N, H],
    updated in place; ``branch`` is the output of the previous block that has not been added to
    the stream yet (None before the first block). The returned branch is likewise not added yet,
    so that the addition fuses with the next norm."""

    ROLES: Tuple[str, ...] = ()   # names of the norms this arrangement needs

    # Set by the model where whatever receives this block's returned branch (the next block's first norm,
    # the final norm) accepts a pending product; a block that does not look at it always returns a tensor.
    pending_output_ok = False

    @property
    def accepts_pending_branch(self) -> bool:
        """Whether the ``branch`` argument of ``forward`` may be a pending product."""
        return False

    def __init__(self, prefix: str, rt: Runtime, mixer: Mixer, feed_forward: FeedForward, norms: Dict[str, Norm]):
        super().__init__(prefix, rt)
        missing = [r for r in self.ROLES if r not in norms]
        if missing:
            raise ValueError("block %s needs norms %s" % (type(self).__name__, ", ".join(missing)))
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms

    def children(self):
        return [self.mixer, self.feed_forward] + list(self.norms.values())

    def forward(self, branch: Optional[torch.Tensor], residual: torch.Tensor, ctx,
                binding: CacheBinding) -> torch.Tensor:
        raise NotImplementedError


# --------------------------------------------------------------------------- registry of kinds

CATEGORIES = ("embedding", "norm", "position", "mixer", "feed_forward", "block", "head")
_PARTS: Dict[Tuple[str, str], type] = {}


def register_part(category: str, kind: str, replace: bool = False):
    """Class decorator: makes ``kind`` available to specs of ``category``."""
    if category not in CATEGORIES:
        raise ValueError("unknown part category %r (known: %s)" % (category, ", ".join(CATEGORIES)))

    def deco(cls):
        if (category, kind) in _PARTS and not replace:
            raise ValueError("%s kind %r is already registered" % (category, kind))
        _PARTS[(category, kind)] = cls
        return cls

    return deco


def unregister_part(category: str, kind: str) -> None:
    _PARTS.pop((category, kind), None)


def part_class(category: str, kind: str) -> type:
    try:
        return _PARTS[(category, kind)]
    except KeyError:
        known = sorted(k for c, k in _PARTS if c == category)
        raise ValueError("no %s of kind %r is registered (known: %s)" % (category, kind, ", ".join(known) or "none"))


def build_part(category: str, spec: PartSpec, prefix: str, rt: Runtime, **extra) -> Part:
    """Instantiate the class registered for (category, spec.kind) with the spec's parameters."""
    cls = part_class(category, spec.kind)
    params = {k: v for k, v in spec.params.items() if k != "prefix"}   # "prefix" places the part, see callers
    try:
        return cls(prefix, rt, **params, **extra)
    except TypeError as e:
        raise TypeError("building %s %r at %r: %s" % (category, spec.kind, prefix, e)) from e
