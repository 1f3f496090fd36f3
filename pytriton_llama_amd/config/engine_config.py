"""Options of the engine itself, apart from the model's config.json.

The reference mixes max_batch_size / max_seq_len / device into the model
configuration (lite_llama/models/model_config.py:37-39) and sizes the cache
from free memory at 0.9 utilisation (lite_llama/executor/model_executor.py:
197-201); here they are their own record.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "float": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"engine dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"engine dtype must be one of {sorted(_DTYPES)}, got {name!r}") from None


@dataclass
class EngineConfig:
    dtype: torch.dtype = torch.bfloat16
    device: str = "cuda:0"
    page_size: int = 16
    num_pages: Optional[int] = None          # None: from gpu_memory_fraction
    gpu_memory_fraction: float = 0.9         # reference: gpu_memory_utilization=0.9
    max_num_seqs: int = 64                   # reference: max_batch_size=64
    max_num_batched_tokens: int = 2048       # token budget of one step
    prefill_chunk: Optional[int] = None      # largest portion of one prompt in a step
    max_model_len: int = 2048                # reference: max_seq_len
    seed: int = 0
    use_graphs: bool = True                  # replay decode-only steps, and steps that bring one
                                             # portion of one prompt (up to 2,048 tokens), as HIP graphs
    decode_weight_copies: bool = True        # keep a second copy of the weights in the layout the
                                             # decode kernels read fastest (doubles the memory the
                                             # weights take; False on a small card)
    timed_library_products: bool = True      # recorded steps run, for each shape of a library matrix
                                             # product, the fastest of the library's algorithms by a
                                             # timing at recording (checked against the first one's
                                             # result). Which one wins can differ between processes,
                                             # and with it the last bit of bfloat16 results; False:
                                             # always the library's first, the same bits every time
    async_decode: bool = True                # launch a decode step before the tokens of the one
                                             # before it have reached the host

    def __post_init__(self):
        self.dtype = parse_dtype(self.dtype)
        if self.page_size <= 0:
            raise ValueError("page_size must be positive")
        if self.max_num_seqs <= 0 or self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
        if self.prefill_chunk is not None and self.prefill_chunk <= 0:
            raise ValueError("prefill_chunk must be positive")
