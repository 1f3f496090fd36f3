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
mixer:           cache_spec() -> PagedSpec | StateSpec | None
                 forward(x, ctx, cache) -> y      x, y: [T, hidden]
                 work_lists() -> WorkList, ...   (optional) how its kernels cut the query rows
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
was given: for a paged spec the pools of that layer by the names of the spec's
tensors (.k, .v for keys and values; .tensors[name]), .group, .page_size, .writable;
for a state spec .state [max_num_seqs + 1, *shape]. The last row of a state tensor is
the padding slot: rows that pad a recorded step to its size class name it (several rows
of a step may), so it holds arbitrary values that no request ever reads.
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
class PagedTensor:
    """One tensor that a paged cache layer keeps for every token. ``shape`` is that of one
    token; a page of the tensor has the shape shape[:token_axis] + (page_size,) +
    shape[token_axis:], so that a kernel can have the tokens of a page where it reads them
    best (keys and values: (kv heads, head size) with token_axis 1 gives pages of
    [kv heads, page_size, head size])."""
    name: str
    shape: Tuple[int, ...]
    token_axis: int = 0
    dtype: Optional[torch.dtype] = None     # None: the engine dtype

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        if not 0 <= self.token_axis <= len(self.shape):
            raise ValueError(f"paged tensor {self.name!r}: token_axis {self.token_axis} outside "
                             f"its {len(self.shape)} dimensions")
        return tuple(self.shape[:self.token_axis]) + (int(page_size),) + tuple(self.shape[self.token_axis:])


@dataclass(frozen=True)
class PagedSpec:
    """What a mixer keeps for every token, in pages: any number of named tensors. ``window``:
    only the last ``window`` positions are ever read again, older pages can be given back.
    Cache layers with equal specs share a page pool and a block table per request."""
    tensors: Tuple[PagedTensor, ...]
    window: Optional[int] = None

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a paged cache spec needs tensors with names of their own, got {names}")


def paged_kv_spec(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> PagedSpec:
    """Keys and values of every token: tensors "k" and "v", pages of [kv heads, page_size, head size]."""
    shape = (int(num_kv_heads), int(head_dim))
    return PagedSpec((PagedTensor("k", shape, 1), PagedTensor("v", shape, 1)), window)


@dataclass(frozen=True)
class WorkList:
    """A list of (sequence, first query row) pairs that cuts the query rows of a step into
    blocks of ``block_rows`` rows, one block a work item of a kernel, the blocks with the most
    keys first. A part names the lists its kernels walk (``work_lists()``); the engine builds
    them for every step, also for the padded steps it records as graphs, and hands them over
    as ``ctx.work[WorkList(...)]`` = (sequence int32 [W], first row int32 [W]). In a recorded
    step W is the most the step's size class can need, and items beyond the real ones are
    empty: their first row is not below the rows their sequence brings.
    ``after_decode``: only the sequences after the leading ones that bring a single token
    (which a kernel specialised for decoding takes)."""
    block_rows: int
    after_decode: bool = False


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
