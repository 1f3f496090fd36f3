"""y = x W^T for the projections of every part.

The reference runs all of them through cuBLAS (nn.Linear / F.linear,
lite_llama/models/llama.py:37-40,61,120,221). Here: float32 always goes through
the package's own vector-FMA kernel (a true 32-bit product, no reduced-precision
matrix mode can be switched on underneath it); bfloat16 uses the package's
skinny weight-streaming kernel for the few rows of a decode step and the
library product (hipBLASLt, called directly: ops.gemm_library) for the many rows
of a prompt.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops

LINEAR_LIBRARIES = ("gemm", "gemm_rows", "blaslt")
SKINNY_ROWS = 8          # rows up to which the skinny kernel takes a bfloat16 product
SKINNY_ROWS_F32 = 16     # ... when float32 output is wanted (the head)


def decode_copy(w: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """The second, blocked copy of a weight matrix that the kernels for the few rows of a decode
    step read faster (ops.blocked_weight); None where there is none to be had (float32, a K that
    does not divide)."""
    if w is None or not w.is_cuda or w.dtype != torch.bfloat16:
        return None
    return ops.blocked_weight(w)


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           blocked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``blocked``: decode_copy(w), for the kernels that take it."""
    if not x.is_cuda:
        raise ops.KernelError("linear: tensors must be on the GPU (there is no CPU path)")
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        return ops.gemm_nt(x, w, torch.float32)
    M = x.shape[0]
    to_f32 = out_dtype == torch.float32
    # measured on MI355X at the 1B shapes: the weight-streaming kernel is level with the
    # library up to 8 rows (and ahead for the vocabulary-sized head); beyond that the library
    if M <= SKINNY_ROWS and ops.gemm_skinny_fits(x, w):
        return ops.gemm_skinny(x, w, out_dtype, blocked=blocked)
    # some tens of rows (a large decoding batch, from ops.ROWS_MIN rows on): the kernel that
    # streams the blocked copy with x staged through LDS, where measured faster than the library
    # (and, for a vocabulary-sized head of 9 to 16 rows, than the skinny kernel)
    if ops.gemm_rows_fits(x, w, blocked):
        return ops.gemm_rows(x, w, blocked, out_dtype)
    if to_f32 and M <= SKINNY_ROWS_F32 and ops.gemm_skinny_fits(x, w):
        return ops.gemm_skinny(x, w, out_dtype, blocked=blocked)
    if ops.gemm_library_fits(x, w):
        return ops.gemm_library(x, w, out_dtype, checked=True)
    if to_f32:
        return ops.gemm_nt(x, w, torch.float32)
    return torch.nn.functional.linear(x, w)         # (rows that are not 16-byte aligned)
