"""Token embedding and the output head."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, place, register_part
from .linear import LINEAR_LIBRARIES, decode_copy, linear


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    """h[t] = E[ids[t]], no scaling (lite_llama/models/llama.py:179,201)."""
    kernel_libraries = ("embedding",)

    def __init__(self, vocab_size: int, hidden_size: int, weight_name: str = "weight"):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight_name = weight_name
        self.weight: Optional[torch.Tensor] = None

    def param_sources(self) -> List[ParamSource]:
        return [ParamSource(self.weight_name, (self.vocab_size, self.hidden_size))]

    def load(self, tensors, dtype, device) -> None:
        self.weight = place(tensors[self.weight_name], "matrix", dtype, device)

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return ops.embedding(self.weight, token_ids)


@register_part("head", "linear_head")
class LinearHead(Part):
    """logits = x W^T in float32 for the wanted rows only
    (lite_llama/models/llama.py:183,221 computes every row in half precision).
    ``tied_to``: an embedding part whose table is the matrix; then the head has
    no tensor of its own."""
    kernel_libraries = LINEAR_LIBRARIES

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: Optional[TokenEmbedding] = None,
                 weight_name: str = "weight"):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to
        self.weight_name = weight_name
        self._weight: Optional[torch.Tensor] = None
        self.blocked: Optional[torch.Tensor] = None              # decode copy (make_decode_copies)

    @property
    def weight(self) -> torch.Tensor:
        return self.tied_to.weight if self.tied_to is not None else self._weight

    def param_sources(self) -> List[ParamSource]:
        if self.tied_to is not None:
            return []
        return [ParamSource(self.weight_name, (self.vocab_size, self.hidden_size))]

    def load(self, tensors, dtype, device) -> None:
        if self.tied_to is None:
            self._weight = place(tensors[self.weight_name], "matrix", dtype, device)

    def make_decode_copies(self) -> int:
        self.blocked = decode_copy(self.weight)
        return 0 if self.blocked is None else self.blocked.numel() * self.blocked.element_size()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear(x, self.weight, out_dtype=torch.float32, blocked=self.blocked)
