"""Python faces of the HIP kernels: each checks on the host that the operands
match what the kernel and its grid assume (device, dtype, shape, strides) and
then launches on torch's current stream. There is no CPU path and no library
fallback: an operand that is not on the GPU, or a size a kernel does not take,
raises.
"""
from __future__ import annotations

import contextlib
import ctypes
import functools
from typing import Optional

import torch

from . import library

_F32, _BF16 = 0, 1


class KernelError(RuntimeError):
    pass


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _F32
    if t.dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("HIP kernels need tensors on the GPU (there is no CPU path); "
                              f"got a tensor on {t.device}")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    # torch's current stream as a raw handle (the two calls below take a fraction of a
    # microsecond; torch.cuda.current_stream() builds a Stream object and takes ten)
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def to_device(values, dtype: torch.dtype, device) -> torch.Tensor:
    """A short list of numbers as a device tensor, through pinned memory and without a wait
    (torch.tensor(..., device=...) copies from pageable memory and blocks the host until the
    stream has come that far, which undoes any step launched ahead)."""
    t = torch.tensor(values, dtype=dtype)
    if torch.device(device).type == "cpu":
        return t
    return t.pin_memory().to(device, non_blocking=True)


def _check(code: int, what: str) -> None:
    if code == 0:
        return
    if code == -1:
        raise KernelError(f"{what}: the kernel refused these sizes or arguments")
    raise KernelError(f"{what}: kernel launch failed (code {code})")


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor")


# ---------------------------------------------------------------------------
def embedding(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids int32 [T]."""
    _need_gpu(table, ids)
    _i32(ids, "ids")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous [V, H] matrix")
    V, H = table.shape
    T = ids.numel()
    out = torch.empty((T, H), dtype=table.dtype, device=table.device)
    lib = library.load("embedding")
    _check(lib.ptl_embedding(_ptr(out), _ptr(table), _ptr(ids), T, H, V, _dtype_code(table),
                             _stream()), "embedding")
    return out


def stage_step(dst: torch.Tensor, src: torch.Tensor, tokens: Optional[torch.Tensor] = None,
               tok_at: int = 0, n_tok: int = 0) -> None:
    """dst (int32, device) <- src (int32, pinned host memory of the same length), read by a
    kernel over the bus; dst[tok_at : tok_at + n_tok] <- tokens (int32, device) when given."""
    _need_gpu(dst)
    if src.is_cuda or not src.is_pinned():
        raise KernelError("stage_step: the source must be pinned host memory")
    if (dst.dtype != torch.int32 or src.dtype != torch.int32 or dst.numel() != src.numel()
            or not dst.is_contiguous() or not src.is_contiguous()):
        raise KernelError("stage_step: two contiguous int32 buffers of one length")
    if tokens is not None:
        _need_gpu(tokens)
        _i32(tokens, "tokens")
        if not (0 <= tok_at and 0 <= n_tok <= tokens.numel() and tok_at + n_tok <= dst.numel()):
            raise KernelError("stage_step: the tokens do not fit where they are to go")
    lib = library.load("embedding")
    _check(lib.ptl_stage_step(_ptr(dst), ctypes.c_void_p(src.data_ptr()), dst.numel(),
                              _ptr(tokens) if tokens is not None else None, int(tok_at),
                              int(n_tok) if tokens is not None else 0, _stream()), "stage_step")


def add_rmsnorm(x: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor,
                eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = rmsnorm(x + residual) * weight; ``residual`` (if given) is replaced
    by the sum in place. weight is float32 [H]. Returns y."""
    _need_gpu(x, residual, weight)
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("add_rmsnorm: x must be a contiguous [T, H] matrix")
    T, H = x.shape
    if weight.dtype != torch.float32 or weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"add_rmsnorm: weight must be float32 [{H}]")
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype
                                 or not residual.is_contiguous()):
        raise KernelError("add_rmsnorm: residual must match x in shape and dtype")
    y = out if out is not None else torch.empty_like(x)
    lib = library.load("norm")
    _check(lib.ptl_add_rmsnorm(_ptr(y), _ptr(x), _ptr(residual), _ptr(weight), T, H,
                               ctypes.c_float(eps), _dtype_code(x), _stream()), "add_rmsnorm")
    return y


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """out[:, i] = silu(gate_up[:, i]) * gate_up[:, I + i] for a [T, 2I] input."""
    _need_gpu(gate_up)
    if gate_up.dim() != 2 or not gate_up.is_contiguous() or gate_up.shape[1] % 2:
        raise KernelError("silu_mul: input must be a contiguous [T, 2I] matrix")
    T, I2 = gate_up.shape
    out = torch.empty((T, I2 // 2), dtype=gate_up.dtype, device=gate_up.device)
    lib = library.load("activation")
    _check(lib.ptl_silu_mul(_ptr(out), _ptr(gate_up), T, I2 // 2, _dtype_code(gate_up), _stream()),
           "silu_mul")
    return out


def rope_store(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor,
               inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
               k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
               page_size: int = 1, k_in_place: bool = False) -> None:
    """Rotate q in place (and k, when ``k_in_place``) by the angles
    positions * inv_freq and write the rotated k and v into the caches
    [num_pages, Hkv, page_size, D] at ``slots`` (int32, page*page_size+offset).
    q, k, v are [T, heads, D] views that share one row stride (slices of one
    projection output). inv_freq None: no rotation. slots None: no store."""
    _need_gpu(q, k, v, positions, inv_freq, slots, k_cache, v_cache)
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    if k.shape != (T, Hkv, D) or v.shape != (T, Hkv, D):
        raise KernelError("rope_store: k and v must be [T, Hkv, D]")
    rs = q.stride(0)
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.stride(2) != 1 or (t.shape[1] > 1 and t.stride(1) != D) or (T > 1 and t.stride(0) != rs) \
                or t.dtype != q.dtype:
            raise KernelError(f"rope_store: {name} must be a [T, heads, D] view with dense heads "
                              "and the common row stride")
    _i32(positions, "positions")
    if positions.numel() != T:
        raise KernelError("rope_store: one position per token")
    if D % 2:
        raise KernelError(f"rope_store: head size {D} must be even")
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != D // 2
                                 or not inv_freq.is_contiguous()):
        raise KernelError(f"rope_store: inv_freq must be float32 [{D // 2}]")
    if slots is not None:
        if slots.dtype != torch.int32 or slots.numel() != T or not slots.is_contiguous():
            raise KernelError("rope_store: slots must be contiguous int32 [T]")
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c is None or c.dim() != 4 or c.shape[1:] != (Hkv, page_size, D) \
                    or c.dtype != q.dtype or not c.is_contiguous():
                raise KernelError(f"rope_store: {name} must be contiguous "
                                  f"[pages, {Hkv}, {page_size}, {D}] of {q.dtype}")
    lib = library.load("rope")
    _check(lib.ptl_rope_store(_ptr(q), _ptr(k), _ptr(v), ctypes.c_long(rs), _ptr(positions),
                              _ptr(inv_freq), _ptr(slots), _ptr(k_cache), _ptr(v_cache),
                              T, Hq, Hkv, D, page_size, int(k_in_place), _dtype_code(q),
                              _stream()), "rope_store")


def gemm_nt(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w.T with float32 accumulation through the vector-FMA kernel.
    x [M, K] (rows may be strided), w [N, K] contiguous, same dtype."""
    _need_gpu(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"gemm_nt: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    if x.dtype != w.dtype:
        raise KernelError(f"gemm_nt: x is {x.dtype} but w is {w.dtype}")
    if x.stride(1) != 1 or not w.is_contiguous():
        raise KernelError("gemm_nt: x rows and w must be dense")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32 and out_dtype != torch.float32:
        raise KernelError("gemm_nt: float32 inputs give float32 outputs")
    y = out if out is not None else torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0:
        return y
    lib = library.load("gemm")
    _check(lib.ptl_gemm_nt(_ptr(y), _ptr(x), _ptr(w), M, N, K, ctypes.c_long(x.stride(0)),
                           ctypes.c_long(y.stride(0)), _dtype_code(x),
                           _F32 if out_dtype == torch.float32 else _BF16, _stream()), "gemm_nt")
    return y


SKINNY_MAX_ROWS = 64
BLOCKED_MAX_ROWS = 64      # rows of x up to which the kernels take the blocked copy of a weight


def blocked_weight(w: torch.Tensor) -> Optional[torch.Tensor]:
    """A second copy of the bfloat16 matrix w [N, K] for the decode kernels: tiles of 16 rows x
    32 columns, each tile row-major in 1 KB, the tiles of a row block one after the other along
    K (shape [ceil(N / 16), K / 32, 16, 32]; rows beyond N are zero). A wave's load instruction
    then reads 1 KB in one piece instead of 16 pieces of 64 bytes that lie a row apart (see
    gs_row_ptr in csrc/gemm.hip). None when w cannot be cut so (K no multiple of 32)."""
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] % 32 or not w.is_contiguous():
        return None
    N, K = w.shape
    rows = -(-N // 16) * 16
    if rows != N:
        w = torch.cat([w, w.new_zeros((rows - N, K))], dim=0)
    return w.view(rows // 16, 16, K // 32, 32).permute(0, 2, 1, 3).contiguous()


def _weight_arg(w: torch.Tensor, blocked: Optional[torch.Tensor], M: int, what: str):
    """(pointer, flag) of the weight a decode kernel is to read: the blocked copy when one is
    given and the rows of x are few enough, else w."""
    if blocked is None or M > BLOCKED_MAX_ROWS:
        return _ptr(w), 0
    N, K = w.shape
    if (blocked.dtype != torch.bfloat16 or not blocked.is_cuda or not blocked.is_contiguous()
            or tuple(blocked.shape) != (-(-N // 16), K // 32, 16, 32) or K % 32
            or blocked.data_ptr() % 16):
        raise KernelError(f"{what}: the blocked copy does not belong to a [{N}, {K}] bfloat16 matrix")
    return _ptr(blocked), 1


def gemm_skinny_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming matrix-core kernel takes this product."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and 0 < x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(1) == 1
            and (x.shape[0] == 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0)


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                blocked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w.T for at most 64 rows of bfloat16 x, streaming w once
    (see csrc/gemm.hip). Output bfloat16 or float32. ``blocked``: ``blocked_weight(w)``, read
    instead of w when x has at most 16 rows."""
    _need_gpu(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"gemm_skinny: shapes {tuple(x.shape)} x {tuple(w.shape)}^T do not match")
    if not gemm_skinny_fits(x, w):
        raise KernelError("gemm_skinny: needs bfloat16, at most 64 rows, K a multiple of 8 and "
                          "16-byte aligned rows")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("gemm_skinny: output is bfloat16 or float32")
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    ldx = x.stride(0) if M > 1 else max(K, 8)
    lib = library.load("gemm")
    wp, wb = _weight_arg(w, blocked, M, "gemm_skinny")
    _check(lib.ptl_gemm_skinny_bf16(_ptr(y), _ptr(x), wp, wb, M, N, K, ctypes.c_long(ldx),
                                    ctypes.c_long(N), _F32 if out_dtype == torch.float32 else _BF16,
                                    _stream()), "gemm_skinny")
    return y


def gemm_library_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_library`` takes x [M, K] and w [N, K]: bfloat16, dense rows of w,
    16-byte aligned rows of both."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2
            and x.shape[1] == w.shape[1] and x.stride(1) == 1 and w.is_contiguous()
            and x.shape[1] % 8 == 0 and (x.shape[0] == 1 or x.stride(0) % 8 == 0)
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


_timed_products = False        # inside ``timed_library_products``


def gemm_library(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                 checked: bool = False) -> torch.Tensor:
    """y = x @ w.T by hipBLASLt, called directly with the descriptors and the algorithm of
    the shape kept from its first call (see csrc/blaslt.hip). Output bfloat16 or float32.
    ``checked``: the caller has just asked ``gemm_library_fits``. The library's first proposal
    runs, except inside ``timed_library_products``."""
    _need_gpu(x, w)
    if not checked and not gemm_library_fits(x, w):
        raise KernelError("gemm_library: needs bfloat16 x [M, K] and w [N, K] with K a multiple of 8 "
                          "and 16-byte aligned rows")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("gemm_library: output is bfloat16 or float32")
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    ldx = x.stride(0) if M > 1 else max(K, 8)
    lib = library.load("blaslt")
    _check(lib.ptl_blaslt_gemm_bf16(_ptr(y), _ptr(x), _ptr(w), M, N, K, ctypes.c_long(ldx),
                                    ctypes.c_long(N), _F32 if out_dtype == torch.float32 else _BF16,
                                    1 if _timed_products else 0, _stream()), "gemm_library")
    return y


@contextlib.contextmanager
def timed_library_products(on: bool = True):
    """Inside, ``gemm_library`` runs the proposal of the library that a timing of the shape
    kept: the first such call of a shape times the library's proposals on its own operands
    (it waits for the stream; not while the stream is captured) and keeps the fastest whose
    result agrees with the first proposal's (csrc/blaslt.hip). For the warm-up pass and the
    recording of a step that is replayed as a graph: such shapes come back with every replay.
    Outside, every call runs the library's first proposal, whatever was timed. ``on=False``:
    no effect (for callers that pass a switch on)."""
    global _timed_products
    before = _timed_products
    _timed_products = bool(on) or before
    try:
        yield
    finally:
        _timed_products = before


def library_product_choice(M: int, N: int, K: int, ldx: int, out_dtype: torch.dtype = torch.bfloat16) -> int:
    """The proposal kept for a shape by its timing (0 = the library's first), -1 if the shape
    has not been timed."""
    lib = library.load("blaslt")
    return int(lib.ptl_blaslt_timed_choice(int(M), int(N), int(K), ctypes.c_long(int(ldx)), ctypes.c_long(int(N)),
                                           _F32 if out_dtype == torch.float32 else _BF16))


FUSED_MAX_ROWS = 16


class RowScale:
    """The normalisation factor that rows of a tensor still lack: row m is to be multiplied by
    rsqrt(sum(partials[m]) / size + eps). ``partials`` [M, count] float32 are the sums of squares
    of the un-normalised row over column blocks (written by ``gemm_skinny_add_norm``)."""
    __slots__ = ("partials", "size", "eps")

    def __init__(self, partials: torch.Tensor, size: int, eps: float):
        self.partials, self.size, self.eps = partials, int(size), float(eps)

    def args(self, M: int, K: int, what: str):
        p = self.partials
        if (p.dtype != torch.float32 or p.dim() != 2 or p.shape[0] != M or not p.is_contiguous()
                or not p.is_cuda):
            raise KernelError(f"{what}: partial sums must be contiguous float32 [{M}, count] on the GPU")
        if self.size != K:
            raise KernelError(f"{what}: rows of {K} elements, but the partial sums are of rows of "
                              f"{self.size}")
        return _ptr(p), int(p.shape[1]), ctypes.c_float(self.eps)


_NO_SCALE = (ctypes.c_void_p(0), 0, ctypes.c_float(0.0))


def gemm_skinny_add_norm_fits(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor,
                              norm_weight: torch.Tensor) -> bool:
    return (_fused_x_ok(x, w) and residual.dtype == torch.bfloat16 and residual.is_cuda
            and residual.dim() == 2 and residual.shape == (x.shape[0], w.shape[0])
            and residual.stride(1) == 1 and norm_weight.dtype == torch.float32
            and norm_weight.is_cuda and norm_weight.is_contiguous()
            and norm_weight.numel() == w.shape[0])


def gemm_skinny_add_norm(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor,
                         norm_weight: torch.Tensor, eps: float, blocked: Optional[torch.Tensor] = None):
    """The product x @ w.T, the residual sum and the part of an RMSNorm that does not need the
    whole row, in one kernel for at most 16 rows of bfloat16 x (see AddNormArgs in
    csrc/gemm.hip): ``residual`` becomes x @ w.T + residual in place; returned are
    y = bfloat16(residual * norm_weight) and the RowScale that y still lacks."""
    if not gemm_skinny_add_norm_fits(x, w, residual, norm_weight):
        raise KernelError("gemm_skinny_add_norm: needs bfloat16 x, w, residual [M, N] with M <= 16, "
                          "K a multiple of 8, aligned rows, a float32 norm weight [N]")
    M, K = x.shape
    N = w.shape[0]
    lib = library.load("gemm")
    count = int(lib.ptl_gemm_skinny_partials(N))
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    partials = torch.empty((M, count), dtype=torch.float32, device=x.device)
    wp, wb = _weight_arg(w, blocked, M, "gemm_skinny_add_norm")
    _check(lib.ptl_gemm_skinny_add_norm_bf16(
        _ptr(y), _ptr(x), wp, wb, _ptr(residual), _ptr(norm_weight), _ptr(partials), M, N, K,
        ctypes.c_long(x.stride(0) if M > 1 else max(K, 8)), ctypes.c_long(N),
        ctypes.c_long(residual.stride(0) if M > 1 else N), _stream()), "gemm_skinny_add_norm")
    return y, RowScale(partials, N, eps)


def row_scale(v: torch.Tensor, scale: RowScale) -> torch.Tensor:
    """v with the factor of ``scale`` applied to its rows (bfloat16 [M, H])."""
    _need_gpu(v)
    if v.dtype != torch.bfloat16 or v.dim() != 2 or not v.is_contiguous():
        raise KernelError("row_scale: needs a contiguous bfloat16 [M, H] tensor")
    M, H = v.shape
    pp, count, eps = scale.args(M, H, "row_scale")
    y = torch.empty_like(v)
    lib = library.load("norm")
    _check(lib.ptl_row_scale_bf16(_ptr(y), _ptr(v), pp, count, M, H, eps, _stream()), "row_scale")
    return y


def _fused_x_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and 0 < x.shape[0] <= FUSED_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(1) == 1
            and (x.shape[0] == 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0 and w.shape[1] == x.shape[1])


# Rows from which, and up to which, the products of csrc/gemm_rows.hip take a decode step (they
# work up to 128). Measured on MI355X at the 1B widths against the library's product followed by
# the separate kernel (cold weights, microseconds at 32 / 64 / 128 rows): output projection + norm
# 9.8 / 11.2 / 14.8 against 11.9 / 12.5 / 12.2; down projection + norm 15.8 / 17.2 / 21.7 against
# 19.5 / 25.9 / 25.1; gate-up + SiLU-multiply 19.5 / 22.7 / 31.2 against 21.5 / 22.3 / 25.5; q|k|v +
# rotation + cache write 10.0 / 13.7 / 18.5 against 13.7 / 14.1 / 17.1; the head of 128,256 columns
# 101 / 112 / 206 against 131 / 137 / 150. Against the fused kernels for at most 16 rows, whole
# decode steps of 16 rows: 1.287 -> 1.243 ms at the 1B widths, 4.73 -> 4.58 ms at the 8B widths,
# 3.04 -> 3.07 ms at the 3B widths (product by product the faster one depends on the shape): from
# 9 rows on a step takes these kernels, where they fit.
ROWS_MIN = 9
ROWS_MAX = {"plain": 64, "add_norm": 64, "gate_up": 64, "qkv": 64}


def _rows_x_ok(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor], use: str = "") -> bool:
    """Whether the kernels for some tens of rows take x with this weight (they read the blocked
    copy) and, with ``use``, whether they are the faster way for that many rows."""
    return (blocked is not None and x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and x.dim() == 2 and ROWS_MIN <= x.shape[0] <= ROWS_MAX.get(use, 128) and x.shape[1] % 32 == 0
            and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.dim() == 2 and w.shape[1] == x.shape[1])


def _rows_weight(w: torch.Tensor, blocked: torch.Tensor, what: str):
    N, K = w.shape
    if (blocked.dtype != torch.bfloat16 or not blocked.is_cuda or not blocked.is_contiguous()
            or tuple(blocked.shape) != (-(-N // 16), K // 32, 16, 32) or blocked.data_ptr() % 16):
        raise KernelError(f"{what}: the blocked copy does not belong to a [{N}, {K}] bfloat16 matrix")
    return _ptr(blocked)


def gemm_rows_fits(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor]) -> bool:
    """Whether ``gemm_rows`` takes the product and is the faster way for it: without slices of K
    it gives every compute unit a workgroup only if the matrix has 64 rows for each (a head)."""
    return _rows_x_ok(x, w, blocked, "plain") and w.shape[0] >= 64 * compute_units(x.device)


def gemm_rows(x: torch.Tensor, w: torch.Tensor, blocked: torch.Tensor,
              out_dtype: Optional[torch.dtype] = None, splits: int = 1) -> torch.Tensor:
    """y = x @ w.T for 9 to 128 rows of bfloat16 x, streaming the blocked copy of w once (see
    csrc/gemm_rows.hip). Output bfloat16 or float32 [M, N]; with ``splits`` > 1 the float32
    partial sums [splits, M, N] over that many slices of K (for ``sum_add_rmsnorm``)."""
    if not _rows_x_ok(x, w, blocked):
        raise KernelError("gemm_rows: needs 9 to 128 rows of bfloat16 x with aligned rows, K a multiple "
                          "of 32 and the blocked copy of w")
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype not in (torch.bfloat16, torch.float32) or (splits > 1 and out_dtype != torch.float32):
        raise KernelError("gemm_rows: output is bfloat16 or float32, partial sums are float32")
    y = torch.empty((splits, M, N) if splits > 1 else (M, N), dtype=out_dtype, device=x.device)
    lib = library.load("gemm_rows")
    _check(lib.ptl_rows_gemm_bf16(_ptr(y), _ptr(x), _rows_weight(w, blocked, "gemm_rows"), M, N, K,
                                  ctypes.c_long(x.stride(0)), ctypes.c_long(N),
                                  _F32 if out_dtype == torch.float32 else _BF16, int(splits),
                                  _stream()), "gemm_rows")
    return y


def gemm_rows_splits(M: int, N: int, K: int) -> int:
    """The slices of K that ``gemm_rows`` should leave partial sums of when a norm follows."""
    return int(library.load("gemm_rows").ptl_rows_gemm_splits(int(M), int(N), int(K)))


def sum_add_rmsnorm(partials: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                    eps: float) -> torch.Tensor:
    """y = rmsnorm(bfloat16(sum of partials) + residual) * weight for float32 partial sums
    [splits, M, N] (or a float32 product [M, N]); ``residual`` (bfloat16 [M, N]) becomes the sum
    in place. One kernel (csrc/gemm_rows.hip)."""
    _need_gpu(partials, residual, weight)
    if partials.dim() == 2:
        partials = partials.unsqueeze(0)
    S, M, N = partials.shape
    if (partials.dtype != torch.float32 or not partials.is_contiguous() or residual.dtype != torch.bfloat16
            or residual.shape != (M, N) or not residual.is_contiguous() or weight.dtype != torch.float32
            or weight.shape != (N,) or not weight.is_contiguous() or N % 8 or N > 8192):
        raise KernelError("sum_add_rmsnorm: needs contiguous float32 partial sums [S, M, N], a bfloat16 "
                          "residual [M, N], a float32 weight [N], N a multiple of 8 up to 8192")
    y = torch.empty((M, N), dtype=torch.bfloat16, device=partials.device)
    lib = library.load("gemm_rows")
    _check(lib.ptl_rows_sum_add_rmsnorm(_ptr(y), _ptr(partials), S, _ptr(residual), _ptr(weight), M, N,
                                        ctypes.c_float(eps), _stream()), "sum_add_rmsnorm")
    return y


def gemm_rows_add_rmsnorm_fits(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor],
                               residual: torch.Tensor, norm_weight: torch.Tensor) -> bool:
    N = w.shape[0]
    return (_rows_x_ok(x, w, blocked, "add_norm") and residual.dtype == torch.bfloat16 and residual.is_cuda
            and residual.shape == (x.shape[0], N) and residual.is_contiguous()
            and norm_weight.dtype == torch.float32 and norm_weight.is_cuda and norm_weight.is_contiguous()
            and norm_weight.numel() == N and N % 8 == 0 and N <= 8192)


def gemm_rows_add_rmsnorm(x: torch.Tensor, w: torch.Tensor, blocked: torch.Tensor, residual: torch.Tensor,
                          norm_weight: torch.Tensor, eps: float) -> torch.Tensor:
    """rmsnorm(x @ w.T + residual) * norm_weight for 9 to 128 rows, ``residual`` replaced by the
    sum: the product as float32 partial sums over slices of K (so that a matrix with few rows
    still gives every compute unit a workgroup), then one kernel that adds them up and
    normalises whole rows."""
    M, K = x.shape
    partials = gemm_rows(x, w, blocked, torch.float32, splits=gemm_rows_splits(M, w.shape[0], K))
    return sum_add_rmsnorm(partials, residual, norm_weight, eps)


def gate_up_silu_fits(x: torch.Tensor, w: torch.Tensor, blocked: Optional[torch.Tensor] = None) -> bool:
    """Whether ``gate_up_silu`` is the way to go for x. ``blocked``: the blocked copy of w, which
    the kernel for some tens of rows reads."""
    if _rows_x_ok(x, w, blocked, "gate_up") and w.shape[0] % 64 == 0:
        return True
    return _fused_x_ok(x, w) and w.shape[0] % 32 == 0


def gate_up_silu(x: torch.Tensor, w: torch.Tensor, scale: Optional[RowScale] = None,
                 blocked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) for w = [Wg; Wu] ([2I, K]) in one kernel: for at most 16 rows
    of bfloat16 x the one of csrc/gemm.hip, from ROWS_MIN rows on, with the blocked copy of w,
    the one of csrc/gemm_rows.hip. ``scale``: the factor that the rows of x still lack (at most
    16 rows); it is applied to both products."""
    rows = scale is None and _rows_x_ok(x, w, blocked) and w.shape[0] % 64 == 0
    if not (rows or (_fused_x_ok(x, w) and w.shape[0] % 32 == 0)):
        raise KernelError("gate_up_silu: needs bfloat16, K a multiple of 8, I a multiple of 16, aligned "
                          "rows, at most 16 of them (up to 128 with the blocked copy of w, K and I "
                          "multiples of 32)")
    M, K = x.shape
    I = w.shape[0] // 2
    out = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
    if rows:
        _check(library.load("gemm_rows").ptl_rows_gate_up_silu(
            _ptr(out), _ptr(x), _rows_weight(w, blocked, "gate_up_silu"), M, I, K,
            ctypes.c_long(x.stride(0)), _stream()), "gate_up_silu")
        return out
    lib = library.load("gemm")
    pp, count, eps = scale.args(M, K, "gate_up_silu") if scale is not None else _NO_SCALE
    wp, wb = _weight_arg(w, blocked, M, "gate_up_silu")
    _check(lib.ptl_gate_up_silu_bf16(_ptr(out), _ptr(x), wp, wb, M, I, K,
                                     ctypes.c_long(x.stride(0) if M > 1 else max(K, 8)),
                                     pp, count, eps, _stream()),
           "gate_up_silu")
    return out


def qkv_rope_store_fits(x: torch.Tensor, w: torch.Tensor, head_dim: int,
                        blocked: Optional[torch.Tensor] = None) -> bool:
    """Whether ``qkv_rope_store`` is the way to go for x. ``blocked``: the blocked copy of w, which
    the kernel for some tens of rows reads."""
    return (_fused_x_ok(x, w) or _rows_x_ok(x, w, blocked, "qkv")) and head_dim % 32 == 0


def qkv_rope_store(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor,
                   inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                   scale: Optional[RowScale] = None, blocked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q, k, v = x @ w.T (rows of w: q | k | v), q and k rotated, k and v written
    into the cache pages at ``slots``; returns the rotated q [M, Hq, D]. At most 16
    rows of bfloat16 x (see csrc/gemm.hip), or, with the blocked copy of w, ROWS_MIN to 128
    (csrc/gemm_rows.hip); head sizes in steps of 32. ``scale``: the factor that the rows of x
    still lack (at most 16 rows); it is applied to the products."""
    rows = scale is None and _rows_x_ok(x, w, blocked)
    if not ((rows or _fused_x_ok(x, w)) and head_dim % 32 == 0):
        raise KernelError("qkv_rope_store: needs bfloat16, K a multiple of 8, a head size in steps of "
                          "32, aligned rows, at most 16 of them (up to 128 with the blocked copy of w "
                          "and K a multiple of 32)")
    M, K = x.shape
    Hq, Hkv, D = num_heads, num_kv_heads, head_dim
    if w.shape[0] != (Hq + 2 * Hkv) * D:
        raise KernelError(f"qkv_rope_store: weight has {w.shape[0]} rows, "
                          f"({Hq} + 2*{Hkv}) * {D} expected")
    _need_gpu(positions, inv_freq, slots, k_cache, v_cache)
    _i32(positions, "positions")
    if positions.numel() != M:
        raise KernelError("qkv_rope_store: one position per row of x")
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != D // 2
                                 or not inv_freq.is_contiguous()):
        raise KernelError(f"qkv_rope_store: inv_freq must be float32 [{D // 2}]")
    if slots is not None:
        if slots.dtype != torch.int32 or slots.numel() != M or not slots.is_contiguous():
            raise KernelError("qkv_rope_store: slots must be contiguous int32 [M]")
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c is None or c.dim() != 4 or c.shape[1:] != (Hkv, page_size, D) \
                    or c.dtype != torch.bfloat16 or not c.is_contiguous():
                raise KernelError(f"qkv_rope_store: {name} must be contiguous bfloat16 "
                                  f"[pages, {Hkv}, {page_size}, {D}]")
    q = torch.empty((M, Hq, D), dtype=torch.bfloat16, device=x.device)
    if rows:
        # the projection as float32 partial sums over slices of K (few rows of W: so that every
        # compute unit gets a workgroup), then one kernel that adds them up, rotates and stores
        partials = gemm_rows(x, w, blocked, torch.float32, splits=gemm_rows_splits(M, w.shape[0], K))
        _check(library.load("gemm_rows").ptl_rows_sum_rope_store(
            _ptr(q), ctypes.c_long(Hq * D), _ptr(partials), partials.shape[0] if partials.dim() == 3 else 1, M,
            _ptr(positions), _ptr(inv_freq), _ptr(slots), _ptr(k_cache), _ptr(v_cache), Hq, Hkv, D,
            int(page_size), _stream()), "qkv_rope_store")
        return q
    lib = library.load("gemm")
    pp, count, eps = scale.args(M, K, "qkv_rope_store") if scale is not None else _NO_SCALE
    wp, wb = _weight_arg(w, blocked, M, "qkv_rope_store")
    _check(lib.ptl_qkv_rope_store_bf16(
        _ptr(q), ctypes.c_long(Hq * D), _ptr(x), wp, wb, M, K,
        ctypes.c_long(x.stride(0) if M > 1 else max(K, 8)), _ptr(positions), _ptr(inv_freq),
        _ptr(slots), _ptr(k_cache), _ptr(v_cache), Hq, Hkv, D, int(page_size), pp, count, eps,
        _stream()),
        "qkv_rope_store")
    return q


def attention_generic(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                      block_table: torch.Tensor, work_seq: torch.Tensor, work_qoff: torch.Tensor,
                      scale: float, window: int = 0) -> None:
    """Attention of a mixed batch over the paged cache (see csrc/attention.hip).
    q [T, Hq, D] (rows may be strided), out [T, Hq, D], caches
    [pages, Hkv, page_size, D], q_start [n+1], ctx_len [n], block_table [n, max_pages],
    work_seq / work_qoff: the list of 16-row query blocks."""
    _need_gpu(out, q, k_cache, v_cache, q_start, ctx_len, block_table, work_seq, work_qoff)
    T, Hq, D = q.shape
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.shape[3] != D:
        raise KernelError("attention: caches must be [pages, Hkv, page_size, D]")
    Hkv, page_size = k_cache.shape[1], k_cache.shape[2]
    if D > 256:
        raise KernelError(f"attention: head size {D} exceeds the kernel's limit of 256")
    if Hq % Hkv:
        raise KernelError(f"attention: {Hq} query heads are not a multiple of {Hkv} kv heads")
    if q.stride(2) != 1 or out.stride(2) != 1 or (Hq > 1 and (q.stride(1) != D or out.stride(1) != D)):
        raise KernelError("attention: q and out need dense heads")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attention: q, out and the caches must share one dtype")
    if not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous")
    for name, t in (("q_start", q_start), ("ctx_len", ctx_len), ("work_seq", work_seq),
                    ("work_qoff", work_qoff)):
        _i32(t, name)
    n = ctx_len.numel()
    if q_start.numel() != n + 1 or work_seq.numel() != work_qoff.numel():
        raise KernelError("attention: inconsistent sequence tables")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.shape[0] < n \
            or block_table.stride(1) != 1:
        raise KernelError("attention: block_table must be int32 [n, max_pages]")
    lib = library.load("attention")
    _check(lib.ptl_attention_generic(
        _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
        _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
        int(block_table.stride(0)), _ptr(work_seq), _ptr(work_qoff), int(work_seq.numel()),
        Hq, Hkv, D, page_size, int(window), ctypes.c_float(scale), _dtype_code(q), _stream()),
        "attention")


def _attention_common(out, q, k_cache, v_cache, q_start, ctx_len, block_table, what):
    _need_gpu(out, q, k_cache, v_cache, q_start, ctx_len, block_table)
    T, Hq, D = q.shape
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.shape[3] != D:
        raise KernelError(f"{what}: caches must be [pages, Hkv, page_size, D]")
    Hkv, page_size = k_cache.shape[1], k_cache.shape[2]
    if Hq % Hkv:
        raise KernelError(f"{what}: {Hq} query heads are not a multiple of {Hkv} kv heads")
    if q.stride(2) != 1 or out.stride(2) != 1 or (Hq > 1 and (q.stride(1) != D or out.stride(1) != D)):
        raise KernelError(f"{what}: q and out need dense heads")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError(f"{what}: q, out and the caches must share one dtype")
    if not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError(f"{what}: caches must be contiguous")
    _i32(q_start, "q_start")
    _i32(ctx_len, "ctx_len")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError(f"{what}: block_table must be int32 [n, max_pages]")
    return T, Hq, Hkv, D, page_size


def attention_decode_mfma_fits(dtype, Hq: int, Hkv: int, D: int, page_size: int = 16) -> bool:
    """Whether the matrix-core decode kernel takes this case: bfloat16, head size 32, 64, 96
    or 128, at most 16 heads a kv head, a page size that is a power of two, pages (of all kv
    heads) below 4 GiB."""
    return (dtype == torch.bfloat16 and D % 32 == 0 and 0 < D <= 128 and Hq // Hkv <= 16
            and page_size > 0 and page_size & (page_size - 1) == 0
            and Hkv * page_size * D * 2 < 2 ** 32)


def attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                     block_table: torch.Tensor, n_seq: int, scale: float, window: int = 0,
                     num_splits: int = 1, matrix_cores: bool = False, unroll: int = 0) -> None:
    """Split-KV attention of the first ``n_seq`` sequences of the tables, each of
    which brings exactly one query token (see csrc/attention.hip). Head sizes in
    steps of 16 up to 256, float32 or bfloat16. ``matrix_cores``: the MFMA
    variant (bfloat16, head sizes 32/64/96/128, at most 16 heads a kv head, a page
    size that is a power of two); ``unroll``: its 16-key tiles per wave and turn
    (1 or 2; 0 leaves the choice to the kernel)."""
    T, Hq, Hkv, D, page_size = _attention_common(out, q, k_cache, v_cache, q_start, ctx_len,
                                                 block_table, "attention_decode")
    if D % 16 or D > 256:
        raise KernelError(f"attention_decode: head size {D} is not a multiple of 16 up to 256")
    if n_seq > ctx_len.numel() or q_start.numel() < n_seq + 1 or block_table.shape[0] < n_seq:
        raise KernelError("attention_decode: tables are shorter than n_seq")
    if num_splits < 1:
        raise KernelError("attention_decode: num_splits must be >= 1")
    part_acc = part_ml = None
    if num_splits > 1:
        part_acc = torch.empty((n_seq, Hq, num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_seq, Hq, num_splits, 2), dtype=torch.float32, device=q.device)
    lib = library.load("attention")
    if matrix_cores:
        if (not attention_decode_mfma_fits(q.dtype, Hq, Hkv, D, page_size) or q.stride(0) % 8
                or q.data_ptr() % 16):
            raise KernelError("attention_decode: the matrix-core variant needs bfloat16, a head "
                              "size of 32/64/96/128, at most 16 heads a kv head, a page size that "
                              "is a power of two, aligned q rows")
        _check(lib.ptl_attention_decode_mfma(
            _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
            _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
            int(block_table.stride(0)), _ptr(part_acc), _ptr(part_ml), int(n_seq), Hq, Hkv, D,
            page_size, int(window), ctypes.c_float(scale), int(num_splits), int(unroll), _stream()),
            "attention_decode_mfma")
        return
    _check(lib.ptl_attention_decode(
        _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
        _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
        int(block_table.stride(0)), _ptr(part_acc), _ptr(part_ml), int(n_seq), Hq, Hkv, D, page_size,
        int(window), ctypes.c_float(scale), int(num_splits), _dtype_code(q), _stream()),
        "attention_decode")


def attention_prefill_mfma_fits(dtype: torch.dtype, num_kv_heads: int, head_dim: int,
                                page_size: int) -> bool:
    """Whether ``attention_prefill_mfma`` takes this case: bfloat16, head size 32, 64, 96 or
    128, a page size that is a power of two, pages (of all kv heads) below 4 GiB."""
    return (dtype == torch.bfloat16 and head_dim % 32 == 0 and 0 < head_dim <= 128
            and page_size > 0 and page_size & (page_size - 1) == 0
            and num_kv_heads * page_size * head_dim * 2 < 2 ** 32)


@functools.lru_cache(maxsize=None)
def _compute_units(device_index: int) -> int:
    return int(torch.cuda.get_device_properties(device_index).multi_processor_count)


def compute_units(device) -> int:
    """Compute units of the GPU ``device`` (256 on MI355X)."""
    device = torch.device(device)
    return _compute_units(device.index if device.index is not None else torch.cuda.current_device())


def attention_prefill_mfma_plan(device: torch.device, num_heads: int, head_dim: int,
                                blocks_of_64: int, blocks_of_128: int, max_keys: int = 0):
    """(block_rows, groups) for ``attention_prefill_mfma``, from sweeps on MI355X (one sequence
    of 512 to 16,384 tokens, and 2,048-token portions behind prefixes up to 14,336, head sizes
    64 and 128). With t = the workgroups a head can have resident at once (three a compute unit
    up to head size 64, two above): 128-row blocks (keys and values are staged half as often)
    once there are 1.25 t of them, 64-row blocks before; at head sizes above 64 also from 0.5 t
    on when some sequence has 4,096 keys or more (``max_keys``: the longest context of the
    step, or a bound of it): a portion behind a long prefix has few blocks, all of them long
    (at 32 heads of 128, 2,048 rows on 14,336 keys: 578 against 811 us; with no prefix the two
    are level, at head size 64 they are level throughout). A workgroup for every block while
    there are at most 2 t blocks (the longest start first and the short ones fill in behind
    them), beyond that t workgroups that share the sorted list as a snake, which evens out the
    causal triangle."""
    resident = compute_units(device) * (3 if head_dim <= 64 else 2)
    t = max(1, resident // num_heads)
    wide = 4 * blocks_of_128 >= 5 * t or (head_dim > 64 and max_keys >= 4096 and 2 * blocks_of_128 >= t)
    rows, blocks = (128, blocks_of_128) if wide else (64, blocks_of_64)
    return rows, max(1, blocks if blocks <= 2 * t else t)


def attention_prefill_mfma(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                           block_table: torch.Tensor, work_seq: torch.Tensor,
                           work_qoff: torch.Tensor, scale: float, window: int = 0,
                           block_rows: int = 64, groups: int = 0) -> None:
    """bfloat16 attention of prompt portions on the matrix cores; the work list
    names query blocks of ``block_rows`` (64 or 128) rows, those with the most
    keys first. ``groups`` workgroups a head share the list (0: one for every
    block). Head sizes 32, 64, 96, 128."""
    T, Hq, Hkv, D, page_size = _attention_common(out, q, k_cache, v_cache, q_start, ctx_len,
                                                 block_table, "attention_prefill_mfma")
    if q.dtype != torch.bfloat16:
        raise KernelError("attention_prefill_mfma: bfloat16 only")
    if D % 32 or D > 128:
        raise KernelError(f"attention_prefill_mfma: head size {D} is not 32, 64, 96 or 128")
    if not attention_prefill_mfma_fits(q.dtype, Hkv, D, page_size):
        raise KernelError(f"attention_prefill_mfma: page size {page_size} is not a power of two "
                          "(or a page of all kv heads reaches 4 GiB)")
    _need_gpu(work_seq, work_qoff)
    _i32(work_seq, "work_seq")
    _i32(work_qoff, "work_qoff")
    if work_seq.numel() != work_qoff.numel():
        raise KernelError("attention_prefill_mfma: inconsistent work list")
    if block_rows not in (64, 128):
        raise KernelError("attention_prefill_mfma: query blocks are 64 or 128 rows")
    if q.stride(0) % 8 or out.stride(0) % 4 or q.data_ptr() % 16 or out.data_ptr() % 8:
        raise KernelError("attention_prefill_mfma: q rows must be 16-byte aligned, out rows 8-byte")
    lib = library.load("attention_prefill")
    n_work = int(work_seq.numel())
    _check(lib.ptl_attention_prefill_mfma(
        _ptr(out), ctypes.c_long(out.stride(0)), _ptr(q), ctypes.c_long(q.stride(0)),
        _ptr(k_cache), _ptr(v_cache), _ptr(q_start), _ptr(ctx_len), _ptr(block_table),
        int(block_table.stride(0)), _ptr(work_seq), _ptr(work_qoff), n_work,
        min(n_work, int(groups)) if groups > 0 else n_work, int(block_rows), Hq, Hkv, D, page_size,
        int(window), ctypes.c_float(scale), _stream()), "attention_prefill_mfma")


def argmax(logits: torch.Tensor, host_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy token per row of float32 logits [R, V]; ties go to the lowest id. ``host_out``:
    pinned int32 host memory (at least R long) that the kernel fills as well, over the bus;
    it holds the choices once the kernel has ended (an event after it, say)."""
    _need_gpu(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax: logits must be float32 [R, V] with dense rows")
    R, V = logits.shape
    if host_out is not None and (host_out.is_cuda or not host_out.is_pinned() or host_out.dtype != torch.int32
                                 or not host_out.is_contiguous() or host_out.numel() < R):
        raise KernelError("argmax: host_out must be pinned int32 host memory with a place for every row")
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    chunks = -(-V // 4096)
    ws_val = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
    ws_idx = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
    lib = library.load("sampling")
    _check(lib.ptl_argmax(_ptr(out), _ptr(logits), R, V, ctypes.c_long(logits.stride(0)),
                          _ptr(ws_val), _ptr(ws_idx), _ptr(host_out), _stream()), "argmax")
    return out


SAMPLE_WIDE_FROM = 16384      # rows at least this long are sampled by many workgroups a row
SAMPLE_WIDE_UP_TO = 64 * 4096


def sample_top_p(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
                 uniform: torch.Tensor, return_probs: bool = False, wide: Optional[bool] = None):
    """One token per row from the nucleus of softmax(logits / temperature).
    temperature, top_p, uniform: float32 [R] on the GPU. ``wide``: spread a row over
    many workgroups (several kernels; None: for rows of vocabulary size) or keep it
    in one (one kernel); both follow the same rule."""
    _need_gpu(logits, temperature, top_p, uniform)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample_top_p: logits must be float32 [R, V] with dense rows")
    R, V = logits.shape
    for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
        if t.dtype != torch.float32 or t.numel() != R or not t.is_contiguous():
            raise KernelError(f"sample_top_p: {name} must be float32 [{R}]")
    if wide is None:
        wide = SAMPLE_WIDE_FROM <= V <= SAMPLE_WIDE_UP_TO
    elif wide and V > SAMPLE_WIDE_UP_TO:
        raise KernelError(f"sample_top_p: the many-workgroup form takes rows up to {SAMPLE_WIDE_UP_TO}")
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    probs = torch.empty((R, V), dtype=torch.float32, device=logits.device)   # scratch, then result
    lib = library.load("sampling")
    if wide:
        lib.ptl_sample_top_p_wide_workspace.restype = ctypes.c_size_t
        nbytes = int(lib.ptl_sample_top_p_wide_workspace(R, V))
        ws = torch.empty((nbytes // 4,), dtype=torch.float32, device=logits.device)
        _check(lib.ptl_sample_top_p_wide(_ptr(out), _ptr(probs), int(return_probs), _ptr(logits), R, V,
                                         ctypes.c_long(logits.stride(0)), _ptr(temperature),
                                         _ptr(top_p), _ptr(uniform), _ptr(ws), _stream()),
               "sample_top_p")
    else:
        _check(lib.ptl_sample_top_p(_ptr(out), _ptr(probs), int(return_probs), _ptr(logits), R, V,
                                    ctypes.c_long(logits.stride(0)), _ptr(temperature), _ptr(top_p),
                                    _ptr(uniform), _stream()), "sample_top_p")
    return (out, probs) if return_probs else out


def token_logprob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """log_softmax(logits[r])[tokens[r]] for float32 logits [R, V] and int32 tokens [R]."""
    _need_gpu(logits, tokens)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("token_logprob: logits must be float32 [R, V] with dense rows")
    _i32(tokens, "tokens")
    R, V = logits.shape
    if tokens.numel() != R:
        raise KernelError("token_logprob: one token per row")
    out = torch.empty((R,), dtype=torch.float32, device=logits.device)
    lib = library.load("sampling")
    _check(lib.ptl_token_logprob(_ptr(out), _ptr(logits), _ptr(tokens), R, V,
                                 ctypes.c_long(logits.stride(0)), _stream()), "token_logprob")
    return out


def probe_stream_read(buf: torch.Tensor, blocks: int = 512) -> None:
    """Launch the kernel that only reads ``buf`` (see csrc/probe.hip); time it from outside."""
    _need_gpu(buf)
    if not buf.is_contiguous() or buf.data_ptr() % 16:
        raise KernelError("probe_stream_read: a contiguous, 16-byte aligned tensor")
    sink = torch.empty(blocks * 256, dtype=torch.int32, device=buf.device)
    lib = library.load("probe")
    _check(lib.ptl_probe_stream_read(_ptr(buf), ctypes.c_size_t(buf.numel() * buf.element_size()),
                                     int(blocks), _ptr(sink), _stream()), "probe_stream_read")


PROBE_MFMA_FLOPS_PER_ITER = 4 * 8 * 16 * 16 * 32 * 2      # per workgroup of four waves


def probe_mfma(iters: int, blocks: int, device="cuda") -> None:
    """Launch ``blocks`` workgroups of four waves that each issue ``iters`` * 8 independent
    bfloat16 MFMAs (see csrc/probe.hip): blocks * iters * PROBE_MFMA_FLOPS_PER_ITER operations."""
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    lib = library.load("probe")
    _check(lib.ptl_probe_mfma(_ptr(out), int(iters), int(blocks), _stream()), "probe_mfma")
