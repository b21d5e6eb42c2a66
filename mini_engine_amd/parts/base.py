"""What every model part is: a small tree of named parameters plus a forward.

A model is assembled from parts (mixer, feed-forward, norm, position encoding,
embedding/head, block arrangement). A part takes its sizes and constants as
constructor arguments, declares the parameters it needs (`ParamSpec`), and never
learns which model it sits in. The weight loader fills declared parameters by
name; the step function hands each part the per-step metadata it may need.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterator

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One parameter tensor of a part.

    ``init`` names the distribution used by the random-weights mode:
    ``"matrix"`` ~ N(0, 0.02) (linears, embeddings), ``"norm"`` ~ 1 + U(-0.1, 0.1); or it is a
    function ``(shape, generator, device) -> float32 tensor`` for a parameter that wants another start
    (a decay rate in (0, 1), a table of integers, ...): it draws from `generator` only, so that the
    values depend on the seed alone.
    ``dtype`` is ``"compute"`` (the engine's dtype: bfloat16 or float32),
    ``"float32"`` (always 32-bit: norm weights, exact for both stored forms),
    ``"int32"`` (integer tables) or ``"stored"`` (what the checkpoint holds: bfloat16
    stays bfloat16, 32-bit stays 32-bit).
    """

    shape: tuple
    init: object = "matrix"       # "matrix", "norm" or a function (shape, generator, device) -> tensor
    dtype: str = "compute"


PAGE = "page"      # stands in a PageTensor's shape for the axis that counts a page's tokens


@dataclass(frozen=True)
class PageTensor:
    """One tensor a mixer keeps per cached token. `shape` is what one page of one layer call looks
    like, with PAGE where the page's tokens are counted: keys stored token by token under their head
    are (heads, PAGE, head size); values transposed inside a page are (heads, head size, PAGE); one
    latent vector per token is (PAGE, width). The pool allocates [pages, *shape] with PAGE replaced by
    the engine's page size. `dtype`: "compute" (the engine's), "float32", "bfloat16" or "int32"."""

    name: str
    shape: tuple
    dtype: str = "compute"

    def __post_init__(self):
        if sum(1 for d in self.shape if d == PAGE) != 1:
            raise ValueError(f"page tensor {self.name!r}: exactly one axis of {self.shape} must be PAGE")

    def sized(self, page_size: int) -> tuple:
        return tuple(page_size if d == PAGE else int(d) for d in self.shape)


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer wants from the paged cache: which tensors per token, and for how long.

    ``window``: None keeps every token; n keeps the last n positions (pages that
    the window has passed are given back). Layers with equal needs share one
    group of pages and one block table per request.
    """

    tensors: tuple                     # of PageTensor
    window: int | None = None

    @classmethod
    def keys_and_values(cls, num_kv_heads: int, head_dim: int, window: int | None = None) -> "CacheNeed":
        """The layout of the attention kernels: K [pages, heads, page, head size], V [pages, heads, head
        size, page] (V transposed inside a page: the P.V operand of the matrix cores is then one load)."""
        return cls((PageTensor("k", (num_kv_heads, PAGE, head_dim)), PageTensor("v", (num_kv_heads, head_dim, PAGE))),
                   window)

    def group_key(self) -> tuple:
        return (self.tensors, self.window)


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size per-request state of a mixer: one tensor ``[num_slots + 1, *shape]``; the last row is
    a spare that belongs to no request (padding rows of a step with a fixed layout name it).
    ``initial``: what the state of a request holds before its first token: None for zeros, a number, or
    nested tuples of numbers of `shape` (a running maximum starts at -inf, a product at 1, ...). The step
    function writes it into a request's row when the request's tokens start at position 0."""

    shape: tuple
    dtype: str = "float32"
    initial: object = None


class Part:
    """Base of all parts: named parameters and named child parts."""

    # Whether a step that contains this part may be captured as a graph: its forward must then use device
    # operations only (no value may travel to the host: no .tolist(), .item(), nonzero(), ...). A part that
    # needs the host sets this to False; the model's steps then always run eagerly.
    capturable = True

    def __init__(self):
        self._specs: dict[str, ParamSpec] = {}
        self._children: dict[str, "Part"] = {}

    # -- declaration -------------------------------------------------------
    def add_param(self, name: str, spec: ParamSpec) -> None:
        self._specs[name] = spec
        setattr(self, name, None)

    def add_child(self, name: str, part: "Part") -> "Part":
        self._children[name] = part
        setattr(self, name, part)
        return part

    # -- traversal ---------------------------------------------------------
    def named_specs(self, prefix: str = "") -> Iterator[tuple]:
        """Yield (full name, owning part, local name, spec) over the whole tree."""
        seen: set[int] = set()
        yield from self._named_specs(prefix, seen)

    def _named_specs(self, prefix, seen):
        if id(self) in seen:        # a part shared by several parents declares its parameters once
            return
        seen.add(id(self))
        for local, spec in self._specs.items():
            yield prefix + local, self, local, spec
        for cname, child in self._children.items():
            yield from child._named_specs(prefix + cname + ".", seen)

    def parts(self) -> Iterator["Part"]:
        seen: set[int] = set()
        stack = [self]
        while stack:
            p = stack.pop()
            if id(p) in seen:
                continue
            seen.add(id(p))
            yield p
            stack.extend(p._children.values())

    # -- binding -----------------------------------------------------------
    def set_param(self, local: str, tensor: torch.Tensor) -> None:
        spec = self._specs[local]
        if tuple(tensor.shape) != tuple(spec.shape):
            raise ValueError(f"{type(self).__name__}.{local}: shape {tuple(tensor.shape)} != {tuple(spec.shape)}")
        setattr(self, local, tensor)

    def finalize(self, device: torch.device, dtype: torch.dtype, max_positions: int) -> None:
        """Called once after all parameters are bound (build tables, derived layouts)."""


class Norm(Part):
    def forward(self, x: torch.Tensor, residual: torch.Tensor | None):
        """-> (normalised x in the compute dtype, new residual in float32).

        ``residual`` None starts the residual stream from ``x``; otherwise the new
        residual is ``x + residual`` (summed in 32-bit) and that sum is normalised.
        """
        raise NotImplementedError

    # Optional: linear_behind(x, residual, weight, out_dtype, gated=False) -> (forward(x, residual)[0] . weight^T,
    # new residual), norm and product as one kernel, or None where there is no such kernel for these shapes
    # (gated: weight is a packed gate/up weight and the product is silu(gate) * up).


class PendingNorm:
    """A norm that has not run yet, in place of its output. A block hands one to a mixer or feed-forward
    that declares `takes_pending_norm = True`; such a part passes it to its first `Linear`, which may run
    norm and product as one kernel (`Norm.linear_behind`), or asks `value()` for the normed rows as a
    tensor. Whichever happens first also yields the new residual, which the block reads afterwards."""

    def __init__(self, norm: "Norm", x: torch.Tensor, residual: torch.Tensor | None):
        self.norm, self.x, self.residual = norm, x, residual
        self._y = None
        self._new_residual = None

    def value(self) -> torch.Tensor:
        if self._y is None:
            x = self.x
            if x.dim() == 3 and not getattr(self.norm, "accepts_partials", False):
                x = x.sum(0)
            self._y, self._new_residual = self.norm.forward(x, self.residual)
        return self._y

    def into_linear(self, weight: torch.Tensor, out_dtype=None, gated: bool = False):
        """The product of the normed rows with `weight` ([out, in]) if the norm can run inside it, else None.
        gated: `weight` is a packed gate/up weight and the product is silu(gate) * up."""
        behind = getattr(self.norm, "linear_behind", None)
        if self._y is not None or behind is None:
            return None
        got = behind(self.x, self.residual, weight, out_dtype, gated) if gated else behind(self.x, self.residual, weight, out_dtype)
        if got is None:
            return None
        y, self._new_residual = got
        return y

    def new_residual(self) -> torch.Tensor:
        if self._new_residual is None:
            self.value()
        return self._new_residual


class PositionEncoding(Part):
    """Something applied to queries and keys as a function of token positions."""

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        """Rotate/shift ``q`` [T, Hq, D] and ``k`` [T, Hkv, D] in place."""
        raise NotImplementedError

    def rotary_table(self) -> torch.Tensor | None:
        """[P, D/2, 2] float32 (cos, sin) if this is a half-split rotary encoding that the
        fused query/key kernel can apply; None means ``apply`` must be called."""
        return None


class Mixer(Part):
    """Token mixing: the only part that looks at other positions of a request."""

    def cache_need(self) -> CacheNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    def forward(self, x: torch.Tensor, step, cache, state) -> torch.Tensor:
        """x: [T, hidden] -> [T, hidden].

        ``step``: the `StepContext` of this step. ``cache``: a `CacheView` (pages of this
        call's layer, or of the layer it reads) or None. ``state``: this call's state
        tensor ``[num_slots + 1, *shape]`` or None; rows are ``step.state_slots``.
        """
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Hidden rows to float32 logits. `project` is what a head implements; `forward` is what the model calls."""

    def project(self, x: torch.Tensor) -> torch.Tensor:
        """x [rows, hidden] -> float32 [rows, vocabulary]."""
        raise NotImplementedError

    def forward(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """`out`: a float32 [rows, vocabulary] tensor the logits must end up in (a step with a fixed layout
        keeps one). A head whose product can write there overrides this; by default the result is copied."""
        y = self.project(x)
        if out is None:
            return y
        out.copy_(y)
        return out


@dataclass
class LayerCall:
    """One entry of a model's run order.

    ``layer``: index into the model's layers (a layer may be named by several
    entries: its weights are then shared, each entry has a cache of its own).
    ``cache_of``: index of an *earlier entry* whose cache this entry reads
    instead of owning one; it then writes nothing.
    """

    layer: int
    cache_of: int | None = None


@dataclass
class CacheView:
    """The pages one layer call reads and writes: per tensor of its CacheNeed, [num_pages + 1, *shape
    of a page]. The last page is a spare that belongs to no request: padding rows of a step with a fixed
    layout write there."""

    group: int                 # index of the page group (selects block table and slot mapping)
    tensors: dict              # PageTensor name -> tensor
    page_size: int
    write: bool = True

    @property
    def k(self) -> torch.Tensor:           # [pages, Hkv, page, D] of a keys-and-values layout
        return self.tensors["k"]

    @property
    def v(self) -> torch.Tensor:           # [pages, Hkv, D, page]
        return self.tensors["v"]


# ---------------------------------------------------------------- registries

_REGISTRIES: dict[str, dict[str, type]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position_encoding": {}, "block": {},
}


def register_part(kind: str, name: str):
    """Class decorator: make a part constructible by ``make_part(kind, name, ...)``."""
    if kind not in _REGISTRIES:
        raise KeyError(f"unknown part kind {kind!r}; kinds: {sorted(_REGISTRIES)}")

    def deco(cls):
        _REGISTRIES[kind][name] = cls
        return cls

    return deco


def make_part(kind: str, name: str, **kwargs) -> Part:
    try:
        cls = _REGISTRIES[kind][name]
    except KeyError:
        raise KeyError(f"no {kind} named {name!r}; registered: {sorted(_REGISTRIES.get(kind, {}))}") from None
    return cls(**kwargs)


def registered(kind: str) -> list:
    return sorted(_REGISTRIES[kind])
