"""Interfaces of the parts that a layer is put together from, and their registries.

A model is described by data: a ``ModelSpec`` holds one ``BlockSpec`` per layer (which norm,
which mixer, which feed-forward, each with its own sizes and constants and the names of its
tensors in the checkpoint) and an ``order``: the list of layer calls of one step.  A call
names the block to run and the cache it works on, so a block may run twice and a layer may
read the cache that another layer wrote.  No part knows which model it is in.

Every kind of part is a class registered under a name; a ``PartSpec`` names the kind and
carries the constructor's keyword arguments.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One tensor of a part, in the layout of the checkpoint."""
    shape: Tuple[int, ...]
    kind: str = "matrix"    # "matrix": computed in the run's dtype; "vector": always fp32; "int": int32
    init: str = "normal"    # random-weights mode: "normal" N(0,std), "ones" 1+N(0,std), "zeros"


@dataclass(frozen=True)
class KVNeed:
    """Keys and values in pages: heads, the width of a key and of a value, and which keys a
    query may read."""
    n_kv_heads: int
    head_dim: int                     # width of a key (and of a value, unless v_head_dim says otherwise)
    visibility: str = "full"          # "full" | "chunk" | "window"
    span: int = 0                     # chunk size or window
    v_head_dim: Optional[int] = None  # width of a value where it differs from a key's (the pool's two halves are sized apart)

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else int(self.v_head_dim)


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: a tensor of this shape for every request slot."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class CacheNeed:
    kv: Optional[KVNeed] = None
    state: Optional[StateNeed] = None


@dataclass
class PartSpec:
    kind: str
    args: Dict[str, Any] = field(default_factory=dict)
    names: Dict[str, str] = field(default_factory=dict)   # local tensor name -> checkpoint name


@dataclass
class BlockSpec:
    kind: str                    # arrangement, e.g. "prenorm"
    norm1: PartSpec
    mixer: Any                   # a PartSpec; an arrangement with several mixers takes what it likes here (a dict of them)
    norm2: PartSpec
    ffn: PartSpec


@dataclass(frozen=True)
class LayerCall:
    block: int                   # index into ModelSpec.blocks
    cache: Any                   # cache id; the call with write=True fills it.  A block with several caches
    write: bool = True           # (``Block.cache_needs``) names them all: {the block's name of a cache: cache id}

    def cache_ids(self) -> Dict[str, int]:
        """{the block's name of a cache: cache id}; a call with one id serves a block with one cache."""
        return dict(self.cache) if isinstance(self.cache, dict) else {"": int(self.cache)}


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    blocks: List[BlockSpec]
    order: List[LayerCall]
    final_norm: PartSpec
    embed_name: Optional[str] = None     # shorthand for embedding = token_table under this tensor name
    head_name: Optional[str] = None      # shorthand for head = linear_head; None: tied to the embedding's table
    eos_token_ids: Tuple[int, ...] = ()
    max_position: int = 1 << 20  # the default context limit of generation (the step function itself has none)
    strip_prefixes: Tuple[str, ...] = ("language_model.",)   # taken off the checkpoint's tensor names
    ignore_prefixes: Tuple[str, ...] = ()   # tensors of the checkpoint that belong to no part of this model
    embedding: Optional[PartSpec] = None    # other kinds of the two ends than the shorthands above name
    head: Optional[PartSpec] = None


class Part:
    """Base of all parts: declares its tensors and takes them when they are loaded."""

    #: True when ``forward`` only launches work on the GPU whose arguments are the step's
    #: device buffers: such a step can be captured in a graph and replayed.  A part that
    #: reads the step's metadata on the host (``ctx.host``) must leave this False.
    graph_safe = False

    #: names of derived arrays of the step's metadata that ``forward`` reads from
    #: ``ctx.derived`` (see ``register_step_array``)
    step_arrays: Tuple[str, ...] = ()

    def params(self) -> Dict[str, ParamSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """``tensors``: local name -> tensor on the GPU, already in its resident dtype."""

    def slow_paths(self, page_size: int) -> List[str]:
        """After loading: one line for every way in which this part, at its sizes and the cache's
        page size, will run a kernel far slower than the one meant for it (a product or an
        attention on plain FMAs in a bfloat16 run).  The engine prints them once when it is built."""
        return []


class Norm(Part):
    def can_project(self, proj) -> bool:
        """Whether forward() takes this ``proj`` with a ``proj_out``: a small fp32 matrix [P, d]
        whose products with the normed fp32 rows are formed in the same pass (router logits).
        The norm knows what its kernel can hold."""
        return False

    def forward(self, h, out, *, d1=None, d2=None, out32=None, rows=None, write_h=True) -> None:
        """h (fp32 [T,d]) += d1 + d2 (kept if write_h); out[i] (and out32[i]) = norm(h[r]), r =
        rows[i] or i."""
        raise NotImplementedError


class PositionEncoding(Part):
    #: True when the fused rotation kernel applies this encoding (see kernel_args).
    fused = True

    def kernel_args(self) -> Dict[str, Any]:
        return {"use_rope": False, "inv_freq": None, "adjacent": False}

    def score_slopes(self, n_heads: int):
        """For encodings that work on the scores instead of on q and k: an fp32 tensor [n_heads]
        on the GPU, head h's score of (query at p, key at j) gets slopes[h] * (j - p) added (before
        a cap, if there is one), or None.  The attention kernels take it as an option."""
        return None

    def transform(self, qkv, positions, n_heads, n_kv_heads, head_dim) -> None:
        """For encodings the fused kernel does not know: change q and k of the fused
        projection's rows in place before they are normed and cached."""


class Mixer(Part):
    def cache_need(self) -> CacheNeed:
        return CacheNeed()

    def forward(self, x, ctx, cache):
        """x [T,d] in the run's dtype -> fp32 [T,d], the residual's increment, taken from
        ``ctx.ws`` (it must stay valid until the next layer call has consumed it)."""
        raise NotImplementedError


class FeedForward(Part):
    #: ask the block for the normed input in fp32 as well (routers want it)
    wants_f32_input = False

    def input_projection(self):
        """An fp32 matrix [P, d] whose products with the fp32 normed input this part wants
        (router logits), or None.  A block whose norm ``projects`` then calls
        ``forward(x, None, ctx, projected=logits)`` instead of handing over x32."""
        return None

    def forward(self, x, x32, ctx, projected=None):
        """x [T,d] (x32: the same in fp32, if asked for) -> a tuple of one or two fp32 [T,d]
        increments of the residual, taken from ``ctx.ws``."""
        raise NotImplementedError


class Embedding(Part):
    #: the table [V, d] after loading, for a head that is tied to it (None if there is none)
    table = None

    def forward(self, token_ids, h, ctx) -> None:
        """h (fp32 [T,d]) = the residual stream's first value for the step's token ids (int32 [T])."""
        raise NotImplementedError


class Head(Part):
    def tie(self, embedding: Embedding) -> None:
        """Called once after loading, with the model's embedding (a tied head takes its table)."""

    def forward(self, x, logits, ctx) -> None:
        """logits (fp32 [n,V]) from the final norm's rows x ([n,d] in the run's dtype)."""
        raise NotImplementedError


def two_increments(h, pending):
    """A norm adds up to two increments to the residual stream itself; what ``pending`` holds beyond
    two (a feed-forward with three or more results a token, each written by a grouped product
    to rows of its own) is added to ``h`` here first, in order.  Returns the two for the norm."""
    if len(pending) > 2:
        from ..csrc import hipops
        for d in pending[2:]:
            hipops.add_into(h, d[:h.shape[0]])
    return (pending[0] if len(pending) > 0 else None, pending[1] if len(pending) > 1 else None)


class Block(Part):
    def cache_needs(self) -> Dict[str, CacheNeed]:
        """What the block's parts ask of the cache manager, by names of the block's own choosing.
        A block with one mixer has one entry (any name); a block with several mixers, or a mixer
        with caches of two shapes, names each, and its layer calls give every name a cache id
        (``LayerCall(block, {"attn": 0, "state": 1})``); ``forward`` then gets a dict of
        ``LayerCache`` by those names instead of one.  Default: the ``mixer`` attribute's need."""
        return {"": self.mixer.cache_need()}

    def forward(self, h, pending, ctx, cache):
        """Runs the layer on the residual stream h (fp32 [T,d]); ``pending`` are the increments
        not yet added to h (see ``two_increments``).  Returns the new pending increments."""
        raise NotImplementedError

    def stages(self):
        """The block's forward as a row of ``(graph_safe, fn(state, ctx, cache))``, cut where a part
        that cannot be captured in a graph begins or ends; run in order they are ``forward``.
        ``state["h"]`` and ``state["pending"]`` are forward's arguments and result; a stage may
        leave what the next one needs under keys of its own.  The engine's graphs hold the safe
        stages; the others run eagerly between them.  Default: the whole block as one stage."""
        def whole(state, ctx, cache):
            state["pending"] = self.forward(state["h"], state["pending"], ctx, cache)
        return [(self.graph_safe, whole)]


# ----------------------------------------------------------------------------- derived step metadata
_STEP_ARRAYS: Dict[str, Callable] = {}


def register_step_array(name: str, fn: Callable) -> None:
    """``fn(host) -> (int32 numpy array, info)``: an array derived from the step's metadata on
    the host (``host``: slots, starts, counts, cu_seqlens of the entries) that a part's kernels
    want on the GPU.  It is computed only for models in which a part lists ``name`` in its
    ``step_arrays``, travels in the step's one metadata copy, and is found under
    ``ctx.derived[name]`` as ``(device array, info)``; ``info`` is any host-side fact that goes
    with it.  The function must depend on its argument alone.  A captured decode step is
    replayed only for steps whose metadata lies at the same places in the step's buffer, so an
    array whose size changes between two decode steps of one shape costs a new capture each time
    it does: keep its size a function of the step's shape (entries and their token counts)."""
    _STEP_ARRAYS[name] = fn


def step_array_builder(name: str) -> Callable:
    if name not in _STEP_ARRAYS:
        raise KeyError(f"no step array {name!r} is registered (known: {sorted(_STEP_ARRAYS)})")
    return _STEP_ARRAYS[name]


# ----------------------------------------------------------------------------- registries
_REGISTRIES: Dict[str, Dict[str, Callable]] = {
    "norm": {}, "position": {}, "mixer": {}, "ffn": {}, "block": {}, "embedding": {}, "head": {},
}


class UnknownPart(KeyError):
    pass


def register(category: str, kind: str, cls=None):
    """``register("mixer", "attention", Attention)`` or as a decorator."""
    if category not in _REGISTRIES:
        raise KeyError(f"no part category {category!r} (known: {sorted(_REGISTRIES)})")

    def deco(c):
        _REGISTRIES[category][kind] = c
        return c
    return deco(cls) if cls is not None else deco


def build(category: str, spec: PartSpec, env) -> Part:
    reg = _REGISTRIES[category]
    if spec.kind not in reg:
        raise UnknownPart(f"no {category} of kind {spec.kind!r} is registered (known: {sorted(reg)})")
    return reg[spec.kind](env=env, **spec.args)


def registered(category: str):
    return sorted(_REGISTRIES[category])
