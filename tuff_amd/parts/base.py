"""What a part is: the interfaces of mixers, feed-forwards, norms, position encodings and
blocks, the declaration of their weights and caches, and the registries that name them.

A part is built in two phases.  Its constructor takes sizes and constants only and allocates
nothing, so a whole model can be described, its weights listed and its caches sized without a
GPU.  `bind(weights, runtime)` then attaches device tensors and the compute dtype.  No part
knows which model it is in: names of checkpoint tensors come in through `names`.
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Optional

import torch


# ---------------------------------------------------------------------- declarations
@dataclasses.dataclass(frozen=True)
class WeightDecl:
    """One tensor a part needs from the checkpoint."""
    name: str                       # name in the checkpoint
    shape: tuple
    init: str = "normal"            # random-weights mode: "normal" N(0, 0.02) | "norm" 1 + N(0, 0.01)
    alt_shapes: tuple = ()          # shapes that are accepted and reshaped to `shape`
    aliases: tuple = ()             # other names the same tensor may have
    role: str = ""                  # "projection": the matrix of a Linear (every token is multiplied by it)


@dataclasses.dataclass(frozen=True)
class PagedKV:
    """Keys and values that grow by one entry a token, kept in pages.  `window`: only the
    last `window` positions are ever read (None: all).  `value_dim`: the width of a value where
    it is not the keys' (None: head_dim).  `value_rows`: values lie as keys do, a row a position
    ([page, kv_head, offset, value_dim]), instead of transposed within the page ([page, kv_head,
    value_dim, offset], which is what the matrix cores of the framework's own attention kernels
    read).  Those kernels take equal widths and transposed values only and refuse another cache by
    its shape; a mixer with kernels of its own declares what suits them."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None
    value_rows: bool = False

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclasses.dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size, zero for a new request.  dtype: "float32", "bfloat16" or
    "int32"."""
    shape: tuple
    dtype: str = "float32"

    def nbytes(self) -> int:
        n = {"float32": 4, "bfloat16": 2, "int32": 4}[self.dtype]
        for d in self.shape:
            n *= d
        return n


@dataclasses.dataclass(frozen=True)
class TokenInput:
    """Integers that come with every token of a step beside its id: `cols` of them a token (the row and the
    column of an image patch, a segment number).  A part that reads them declares them (Part.token_inputs); the
    caller brings them in StepEntry.inputs[name], and a step's context holds them as ctx.inputs[name], int32
    [T, cols].  `default`: what a token gets whose entry brings none ("position": its position in the request,
    in every column; an int: that value; None: the entry must bring them)."""
    name: str
    cols: int = 1
    default: object = None


def cache_specs_of(mixer) -> tuple:
    """A mixer's cache declarations as a tuple (empty: it keeps nothing), and whether forward()
    is handed a tuple of views (True) or one view / None (False)."""
    spec = mixer.cache_spec()
    if spec is None:
        return (), False
    if isinstance(spec, (tuple, list)):
        return tuple(spec), True
    return (spec,), False


@dataclasses.dataclass
class Runtime:
    """What parts need at bind time: where tensors live and in which type they compute."""
    device: torch.device
    dtype: torch.dtype              # torch.bfloat16 (serving) or torch.float32 (true 32-bit)

    def empty(self, *shape, dtype=None) -> torch.Tensor:
        return torch.empty(*shape, dtype=dtype or self.dtype, device=self.device)


# -------------------------------------------------------------------------- interfaces
class Part:
    """Base of all parts.  `names` maps the part's own weight names to checkpoint names."""

    def weight_decls(self) -> list[WeightDecl]:
        return []

    def bind(self, weights: dict[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt

    def kernel_modules(self) -> list[str]:
        """Kernel libraries (names of tuff_amd.csrc.build.MODULES) this part launches."""
        return []

    def token_inputs(self) -> list:
        """TokenInput declarations: what this part reads of a step's tokens beside ids and positions."""
        return []

    #: True if forward() only launches kernels on the current stream and reads nothing back to
    #: the host, so that a step through this part can be recorded into a graph and replayed.
    graph_safe = False

    #: True if a step with prompt portions through this part can be recorded in sections: outside
    #: of ctx.run_eagerly(fn) the part is graph_safe and reads of ctx only T, tokens, req_of_token,
    #: q_start, q_len and state_slot (they stay in place between replays, with q_len 0 for requests
    #: beyond the step's own); everything else of the step (positions, tables, wanted rows, host
    #: facts) it reads inside fn(ctx), which runs again at every replay with that step's ctx, on
    #: tensors it was given from outside (they keep their place too).
    records_portions = False

    #: True if forward() may be handed a parts.norm.PendingNorm in place of the normed tensor h
    #: (the part passes it straight to a Linear, which can run the norm inside its kernel).
    accepts_pending_norm = False

    #: True if forward() touches the residual stream exactly once, as its last operation, through
    #: Linear.forward(accumulate_into=residual, next_norm=next_norm), and takes a keyword next_norm
    #: for it.  The block then tells it which norm reads the stream next, and that product may
    #: leave the norm its operand (see Linear.forward).
    adds_once_through_linear = False


class Norm(Part):
    """forward(x float32 [T, d], rows=None) -> [T or len(rows), d] in the compute dtype."""

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """Encodes positions into q and k of an attention mixer, after their norm and before the
    cache write (the cache holds encoded keys).

    Either `rotary_tables()` returns (inv_freq float32 [rotary_dim/2], rotary_dim, interleaved)
    and the mixer applies it inside its fused kernel, or it returns None and the mixer calls
    `apply_step(q [T, H*hd], k [T, Hkv*hd], ctx)`, which rewrites both in place; that is
    `apply(q, k, ctx.positions)` unless the encoding reads more of the step than positions (what it
    declares in token_inputs(), from ctx.inputs).
    """

    def rotary_tables(self):
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        raise NotImplementedError

    def apply_step(self, q: torch.Tensor, k: torch.Tensor, ctx) -> None:
        self.apply(q, k, ctx.positions)


class Mixer(Part):
    """Token mixer.  forward adds its output to `residual` (float32 [T, d]).

    h: [T, d] in the compute dtype, already normed.  ctx: the step's StepContext.
    cache: the view of this run's cache entry (PagedKVView, StateView or None).
    write_cache=False: read the cache of another run without writing to it.
    """

    def cache_spec(self):
        """None, one declaration (PagedKV or FixedState), or a tuple of declarations for a mixer
        that keeps several things per request (keys and values beside a state, a convolution's
        tail beside a recurrent matrix).  forward() gets None, one view, or a tuple of views in
        the order of the declarations."""
        return None

    def forward(self, h, ctx, cache, residual, write_cache: bool = True) -> None:
        """A mixer with adds_once_through_linear is also passed next_norm=<Norm or None>: the
        norm that reads the residual stream right after this mixer, to be handed on to the
        Linear that adds into it (Linear.forward(..., next_norm=...))."""
        raise NotImplementedError


class FeedForward(Part):
    """forward(h [T, d] compute dtype, ctx, residual float32 [T, d]) adds its output."""

    def forward(self, h, ctx, residual) -> None:
        """As for mixers: with adds_once_through_linear the call carries next_norm=<Norm or None>."""
        raise NotImplementedError


class Block(Part):
    """Arrangement of norms, a mixer and a feed-forward around the residual stream.
    forward(x float32 [T, d], ctx, cache, write_cache) updates x in place."""

    mixer: Mixer

    def forward(self, x, ctx, cache, write_cache: bool = True) -> None:
        raise NotImplementedError


# --------------------------------------------------------------------------- registries
class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: dict[str, Callable] = {}

    def register(self, name: str, item=None):
        def put(obj):
            if name in self._items and self._items[name] is not obj:
                raise ValueError(f"{self.what} '{name}' is already registered")
            self._items[name] = obj
            return obj
        return put if item is None else put(item)

    def get(self, name: str):
        if name not in self._items:
            raise KeyError(f"unknown {self.what} '{name}'; registered: {sorted(self._items)}")
        return self._items[name]

    def names(self) -> list[str]:
        return sorted(self._items)

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
