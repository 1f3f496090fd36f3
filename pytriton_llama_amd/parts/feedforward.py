"""The dense gated feed-forward."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, PendingProduct, PendingScale, as_tensor, place, register_part
from .linear import LINEAR_LIBRARIES, decode_copy, linear


@register_part("feed_forward", "swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)), three matrices without bias
    (lite_llama/models/llama.py:107-120, lite_llama/kernels/swiglu.py:44-67).
    gate and up are concatenated at load into one [2I, hidden] matrix (rows
    gate | up) so that one product feeds the SiLU-multiply kernel."""
    kernel_libraries = ("activation", "norm") + LINEAR_LIBRARIES
    takes_pending_scale = True
    can_defer_output = True

    def __init__(self, hidden_size: int, intermediate_size: int,
                 gate_name: str = "gate_proj.weight", up_name: str = "up_proj.weight",
                 down_name: str = "down_proj.weight"):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.names = (gate_name, up_name, down_name)
        self.gate_up: Optional[torch.Tensor] = None
        self.down: Optional[torch.Tensor] = None
        self.gate_up_blocked: Optional[torch.Tensor] = None      # decode copies (make_decode_copies)
        self.down_blocked: Optional[torch.Tensor] = None

    def param_sources(self) -> List[ParamSource]:
        g, u, d = self.names
        return [ParamSource(g, (self.intermediate_size, self.hidden_size)),
                ParamSource(u, (self.intermediate_size, self.hidden_size)),
                ParamSource(d, (self.hidden_size, self.intermediate_size))]

    def load(self, tensors, dtype, device) -> None:
        g, u, d = self.names
        self.gate_up = place(torch.cat([tensors[g], tensors[u]], dim=0), "matrix", dtype, device)
        self.down = place(tensors[d], "matrix", dtype, device)

    def make_decode_copies(self) -> int:
        self.gate_up_blocked, self.down_blocked = decode_copy(self.gate_up), decode_copy(self.down)
        return sum(t.numel() * t.element_size() for t in (self.gate_up_blocked, self.down_blocked)
                   if t is not None)

    def forward(self, x, defer_output: bool = False):
        scale = None
        if isinstance(x, PendingScale) and ops.gate_up_silu_fits(x.values, self.gate_up):
            x, scale = x.values, x.scale
        x = as_tensor(x)
        if ops.gate_up_silu_fits(x, self.gate_up, self.gate_up_blocked):
            # the few rows of a decode step: product and SiLU-multiply in one kernel
            a = ops.gate_up_silu(x, self.gate_up, scale, blocked=self.gate_up_blocked)
            if defer_output:
                return PendingProduct(a, self.down, self.down_blocked)
            return linear(a, self.down, blocked=self.down_blocked)
        a = ops.silu_mul(linear(x, self.gate_up, blocked=self.gate_up_blocked))
        if defer_output:                    # (the norm that follows picks the kernels by the rows)
            return PendingProduct(a, self.down, self.down_blocked)
        return linear(a, self.down, blocked=self.down_blocked)
