"""y = x W^T for the projections of every part.

The reference runs all of them through cuBLAS (nn.Linear / F.linear,
lite_llama/models/llama.py:37-40,61,120,221). Here: float32 always goes through
the package's own vector-FMA kernel (a true 32-bit product, no reduced-precision
matrix mode can be switched on underneath it); bfloat16 uses the package's
skinny weight-streaming kernel for the few rows of a decode step and the
library product (hipBLASLt through torch) for the many rows of a prompt.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops

LINEAR_LIBRARIES = ("gemm",)


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    if not x.is_cuda:
        raise ops.KernelError("linear: tensors must be on the GPU (there is no CPU path)")
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        return ops.gemm_nt(x, w, torch.float32)
    if ops.gemm_skinny_fits(x, w):
        return ops.gemm_skinny(x, w, out_dtype)
    if out_dtype == torch.float32:
        return ops.gemm_nt(x, w, torch.float32)
    return torch.nn.functional.linear(x, w)
