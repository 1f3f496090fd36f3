"""RMSNorm with the residual sum fused in front of it."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, PendingProduct, PendingScale, as_tensor, place, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """y = (x + residual) * rsqrt(mean((x + residual)^2) + eps) * weight, with the
    sum returned as the new residual (lite_llama/kernels/skip_rmsnorm.py:94-181;
    call sites lite_llama/models/llama.py:149,160,219). Without a residual the
    input itself is the residual (:181)."""
    kernel_libraries = ("norm", "gemm", "gemm_rows")
    takes_pending_product = True

    def __init__(self, size: int, eps: float, weight_name: str = "weight"):
        self.size = int(size)
        self.eps = float(eps)
        self.weight_name = weight_name
        self.weight: Optional[torch.Tensor] = None

    def param_sources(self) -> List[ParamSource]:
        return [ParamSource(self.weight_name, (self.size,), "vector")]

    def load(self, tensors, dtype, device) -> None:
        self.weight = place(tensors[self.weight_name], "vector", dtype, device)

    def forward(self, x, residual: Optional[torch.Tensor], scale_ok: bool = False):
        if isinstance(x, PendingProduct):
            # some tens of rows (from ops.ROWS_MIN on): the product as partial sums over slices of
            # K, then one kernel that adds them up, adds the residual and normalises
            if (residual is not None and x.blocked is not None
                    and ops.gemm_rows_add_rmsnorm_fits(x.x, x.w, x.blocked, residual, self.weight)):
                y = ops.gemm_rows_add_rmsnorm(x.x, x.w, x.blocked, residual, self.weight, self.eps)
                return y, residual
            # the few rows of a decode step: the product, the residual sum and the weight in one
            # kernel; the rsqrt factor is left to the part that takes the result
            if (scale_ok and residual is not None
                    and ops.gemm_skinny_add_norm_fits(x.x, x.w, residual, self.weight)):
                y, scale = ops.gemm_skinny_add_norm(x.x, x.w, residual, self.weight, self.eps,
                                                    blocked=x.blocked)
                return PendingScale(y, scale), residual
        x = as_tensor(x)
        y = ops.add_rmsnorm(x, residual, self.weight, self.eps)
        return y, (x if residual is None else residual)
