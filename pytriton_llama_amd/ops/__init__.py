from . import library
from .library import KernelLibraryError
from .kernels import (PROBE_MFMA_FLOPS_PER_ITER, ROWS_MIN, KernelError, RowScale, add_rmsnorm, argmax, attention_decode,
                      attention_decode_mfma_fits, attention_generic, attention_prefill_mfma,
                      attention_prefill_mfma_fits, attention_prefill_mfma_plan, blocked_weight, compute_units, embedding, gate_up_silu, gate_up_silu_fits,
                      gemm_library, gemm_library_fits, timed_library_products, library_product_choice, gemm_nt, gemm_rows, gemm_rows_add_rmsnorm, gemm_rows_add_rmsnorm_fits, gemm_rows_fits, gemm_rows_splits, sum_add_rmsnorm, gemm_skinny, gemm_skinny_add_norm, gemm_skinny_add_norm_fits,
                      gemm_skinny_fits, probe_mfma, probe_stream_read, qkv_rope_store, qkv_rope_store_fits,
                      rope_store, row_scale,
                      sample_top_p, silu_mul, stage_step, to_device, token_logprob)
