from . import library
from .library import KernelLibraryError
from .kernels import (KernelError, add_rmsnorm, argmax, attention_generic, embedding, gemm_nt,
                      rope_store, sample_top_p, silu_mul)
