"""What every part of a layer looks like to the rest of the engine.

A model is put together from parts that know their own sizes and constants and
nothing about the model they are in: an embedding, blocks (each a norm, a
mixer, a norm and a feed-forward in some arrangement), a final norm and a head.
Parts are chosen by name from the registries below, layer by layer, so one
model may use different mixers and feed-forwards in different layers, and a new
part is added by registering a class: no file of the engine changes.

Interfaces
----------
every part:
    kernel_libraries        names of the HIP libraries it launches (built on demand)
    param_sources()         checkpoint tensors it wants: ParamSource(name, shape, kind),
                            names relative to the prefix the model gives the part
    load(tensors, dtype, device)   take them (keyed by the same names); may fuse
norm:            forward(x, residual) -> (y, new_residual)    residual may be None
mixer:           cache_spec() -> PagedKVSpec | StateSpec | None
                 forward(x, ctx, cache) -> y      x, y: [T, hidden]
feed-forward:    forward(x) -> y
position:        rotary_inv_freq() -> float32 [D/2] or None;  apply(q, k, positions) in place
embedding:       forward(token_ids int32 [T]) -> [T, hidden]
head:            forward(x [R, hidden]) -> float32 logits [R, vocab]
block:           forward(h, residual, ctx, cache) -> (h, residual); may set the flags
                 can_defer_output (forward then takes defer_output=True and may return a
                 pending h) and takes_pending_product (its h may arrive pending)

Work handed on instead of done (optional; a part that knows nothing of it is given tensors)
------------------------------------------------------------------------------------------
For the few rows of a decode step a kernel costs more in starting than in running, so two
parts may pass each other a value that is not finished yet when the receiver can finish it
inside a kernel it launches anyway:
    PendingProduct(x, w)      x @ w.T not computed yet. A mixer or feed-forward whose class
                              says ``can_defer_output`` returns it for its last projection when
                              called with defer_output=True; a norm whose class says
                              ``takes_pending_product`` computes the product, the residual sum
                              and its own share in one kernel.
    PendingScale(values, scale)   rows that still lack a factor (the rsqrt of an RMSNorm). A
                              norm returns it when called with scale_ok=True; a mixer or
                              feed-forward whose class says ``takes_pending_scale`` applies the
                              factor to the results of its first product.
Both have .tensor(), which finishes the work with separate kernels. The block (and the model,
between blocks) asks the classes for these flags and passes plain tensors to everyone else.

``ctx`` is the StepContext of engine/batch.py: the flat batch (positions,
q_start, ctx_len, per cache group its block table and slot mapping, the state
slot of every sequence). ``cache`` is the view of the one cache layer the call
was given: for a paged spec .k/.v pools of that layer, .group, .writable; for a
state spec .state [max_num_seqs, *shape].
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSource:
    name: str                 # relative to the part's prefix, e.g. "q_proj.weight"
    shape: Tuple[int, ...]
    kind: str = "matrix"      # "matrix": held in the engine dtype; "vector": held in float32;
                              # "table": integers, held as int32
    init: Optional[Tuple] = None   # how the random-weights mode draws it. None: by kind (matrix
                              # N(0, std), vector 1 + N(0, norm_std): a norm weight, table
                              # uniform integers). Else ("normal", mean, std), ("uniform", low,
                              # high) or ("constant", value): biases, decay rates, gates


@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values of every token, in pages; ``window``: only the last
    ``window`` positions are ever read again, older pages can be given back."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    """A tensor of fixed size per request (in the slot of the request)."""
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None     # None: the engine dtype


class PendingProduct:
    """x @ w.T that has not been computed (see the module text). ``blocked``: the decode copy
    of w (parts/linear.py), if the part keeps one."""
    __slots__ = ("x", "w", "blocked")

    def __init__(self, x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor] = None):
        self.x, self.w, self.blocked = x, w, blocked

    @property
    def shape(self):
        return (self.x.shape[0], self.w.shape[0])

    def tensor(self) -> torch.Tensor:
        from .linear import linear
        return linear(self.x, self.w, blocked=self.blocked)


class PendingScale:
    """Rows that still lack a factor (see the module text); ``scale`` is an ops.RowScale."""
    __slots__ = ("values", "scale")

    def __init__(self, values: torch.Tensor, scale):
        self.values, self.scale = values, scale

    @property
    def shape(self):
        return self.values.shape

    def tensor(self) -> torch.Tensor:
        from .. import ops
        return ops.row_scale(self.values, self.scale)


def as_tensor(v):
    """``v`` finished, if it is one of the pending values."""
    return v.tensor() if isinstance(v, (PendingProduct, PendingScale)) else v


def run_norm(norm, x, residual, consumer=None):
    """norm.forward for an x that may be pending, on behalf of ``consumer`` (the part that gets
    the result; None: someone who wants a tensor)."""
    if getattr(norm, "takes_pending_product", False):
        return norm.forward(x, residual, scale_ok=getattr(consumer, "takes_pending_scale", False))
    return norm.forward(as_tensor(x), residual)


class Part:
    kernel_libraries: Tuple[str, ...] = ()
    takes_pending_product = False     # norms, blocks
    takes_pending_scale = False       # mixers, feed-forwards
    can_defer_output = False          # mixers, feed-forwards, blocks
    graph_capturable = True           # False: forward waits for the device or reads device data
                                      # on the host; steps of a model with such a part are
                                      # launched kernel by kernel, never replayed as graphs

    def param_sources(self) -> List[ParamSource]:
        return []

    def load(self, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device) -> None:
        pass

    def make_decode_copies(self) -> int:
        """Optional: build what the part keeps beside its weights to run decode steps faster
        (second copies in another layout, say) and return the bytes it took. Called once after
        the weights are loaded, when the engine is told to spend memory on speed."""
        return 0


PART_KINDS = ("embedding", "norm", "mixer", "feed_forward", "position", "head", "block")
PART_REGISTRY: Dict[str, Dict[str, Any]] = {k: {} for k in PART_KINDS}


def register_part(kind: str, name: str):
    """Class decorator: make ``name`` available for ``kind`` in layer specs."""
    if kind not in PART_REGISTRY:
        raise KeyError(f"unknown part kind {kind!r}; kinds: {PART_KINDS}")

    def deco(cls):
        PART_REGISTRY[kind][name] = cls
        return cls
    return deco


def build_part(kind: str, name: str, **kwargs):
    try:
        cls = PART_REGISTRY[kind][name]
    except KeyError:
        raise KeyError(f"no {kind} part named {name!r}; registered: "
                       f"{sorted(PART_REGISTRY.get(kind, {}))}") from None
    return cls(**kwargs)


def place(t: torch.Tensor, kind: str, dtype: torch.dtype, device) -> torch.Tensor:
    """A checkpoint tensor as the engine holds it: matrices in the engine dtype,
    vectors in float32, integer tables as int32."""
    if kind == "vector":
        return t.to(device=device, dtype=torch.float32).contiguous()
    if kind == "table":
        return t.to(device=device, dtype=torch.int32).contiguous()
    return t.to(device=device, dtype=dtype).contiguous()
