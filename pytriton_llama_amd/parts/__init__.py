from .base import (PART_KINDS, PART_REGISTRY, PagedSpec, PagedTensor, ParamSource, Part, StateSpec, WorkList,
                   build_part, paged_kv_spec,
                   place, register_part)
from .linear import linear
from .norm import RMSNorm
from .rotary import RotaryEncoding, default_inv_freq, llama3_inv_freq
from .attention import PagedAttention
from .feedforward import SwiGLU
from .embedding import LinearHead, TokenEmbedding
from .block import PreNormBlock
