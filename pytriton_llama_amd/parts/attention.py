"""The attention mixer over the paged cache."""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from .. import ops
from .base import (ParamSource, Part, PendingProduct, PendingScale, WorkList, as_tensor,
                   paged_kv_spec, place, register_part)
from .linear import LINEAR_LIBRARIES, decode_copy, linear


# How the attention kernels cut the query rows of a step: 16 rows a work item for the vector-FMA
# kernel (over all sequences, or over those the split-KV decode kernel does not take), 64 or 128
# for the matrix-core kernel for prompt portions.
ALL_16 = WorkList(16)
PORTIONS_16 = WorkList(16, after_decode=True)
PORTIONS_64 = WorkList(64, after_decode=True)
PORTIONS_128 = WorkList(128, after_decode=True)


@register_part("mixer", "paged_attention")
class PagedAttention(Part):
    """Grouped-query attention: q/k/v projections without bias, a position
    encoding on q and k, the new keys and values written into cache pages, then
    every token attends its sequence's keys in the pages up to its own
    position, and the output projection (lite_llama/models/llama.py:26-62 for a
    prompt, :64-105 for one decoded token; here both are one path because the
    kernels read only the cache). scale defaults to head_dim^-0.5 (llama.py:173).

    The three projection matrices are concatenated at load into one
    [(Hq + 2 Hkv) D, hidden] matrix, rows q | k | v (the reference fuses k and
    v, lite_llama/executor/weight_convert.py:229-246)."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[Part] = None, scale: Optional[float] = None,
                 window: Optional[int] = None,
                 q_name: str = "q_proj.weight", k_name: str = "k_proj.weight",
                 v_name: str = "v_proj.weight", o_name: str = "o_proj.weight"):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim % 2 or head_dim > 256:
            raise ValueError(f"the attention kernels take even head sizes up to 256, got {head_dim}")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.num_kv_heads, self.head_dim = int(num_kv_heads), int(head_dim)
        self.position = position
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.window = int(window) if window else None
        self.names = (q_name, k_name, v_name, o_name)
        self.force_decode_splits = 0        # tests set it to try other splits
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.qkv: Optional[torch.Tensor] = None
        self.o: Optional[torch.Tensor] = None
        self.qkv_blocked: Optional[torch.Tensor] = None          # decode copies (make_decode_copies)
        self.o_blocked: Optional[torch.Tensor] = None
        libs = ("attention", "rope") + LINEAR_LIBRARIES
        if self.head_dim % 32 == 0 and self.head_dim <= 128:
            libs += ("attention_prefill",)          # the matrix-core kernel for prompt portions
        if position is not None:
            libs += tuple(position.kernel_libraries)
        self.kernel_libraries = tuple(dict.fromkeys(libs))

    def work_lists(self):
        return (ALL_16, PORTIONS_16, PORTIONS_64, PORTIONS_128)

    def cache_spec(self):
        return paged_kv_spec(self.num_kv_heads, self.head_dim, self.window)

    @property
    def graph_capturable(self) -> bool:
        return self.position is None or getattr(self.position, "graph_capturable", True)

    def param_sources(self) -> List[ParamSource]:
        qn, kn, vn, on = self.names
        return [ParamSource(qn, (self.q_size, self.hidden_size)),
                ParamSource(kn, (self.kv_size, self.hidden_size)),
                ParamSource(vn, (self.kv_size, self.hidden_size)),
                ParamSource(on, (self.hidden_size, self.q_size))]

    def load(self, tensors, dtype, device) -> None:
        qn, kn, vn, on = self.names
        self.qkv = place(torch.cat([tensors[qn], tensors[kn], tensors[vn]], dim=0),
                         "matrix", dtype, device)
        self.o = place(tensors[on], "matrix", dtype, device)
        if self.position is not None:
            self.position.load({}, dtype, device)

    def make_decode_copies(self) -> int:
        self.qkv_blocked, self.o_blocked = decode_copy(self.qkv), decode_copy(self.o)
        return sum(t.numel() * t.element_size() for t in (self.qkv_blocked, self.o_blocked)
                   if t is not None)

    takes_pending_scale = True
    can_defer_output = True

    def forward(self, x, ctx, cache, defer_output: bool = False):
        T = x.shape[0]
        Hq, Hkv, D = self.num_heads, self.num_kv_heads, self.head_dim
        group = ctx.groups[cache.group]
        rotary = self.position.rotary_inv_freq() if self.position is not None else None
        fused = self.position is None or rotary is not None
        scale = None
        if isinstance(x, PendingScale) and fused and ops.qkv_rope_store_fits(x.values, self.qkv, D):
            x, scale = x.values, x.scale
        x = as_tensor(x)
        if fused and ops.qkv_rope_store_fits(x, self.qkv, D, self.qkv_blocked):
            # the few rows of a decode step: projection, rotation and cache write in one kernel
            q = ops.qkv_rope_store(x, self.qkv, ctx.positions, rotary,
                                   group.slots if cache.writable else None, cache.k, cache.v,
                                   Hq, Hkv, D, cache.page_size, scale, blocked=self.qkv_blocked)
            out = torch.empty((T, Hq, D), dtype=x.dtype, device=x.device)
            self.attend(out, q, cache, ctx, group)
            if defer_output:
                return PendingProduct(out.view(T, Hq * D), self.o, self.o_blocked)
            return linear(out.view(T, Hq * D), self.o, blocked=self.o_blocked)
        qkv = linear(x, self.qkv, blocked=self.qkv_blocked)
        q = qkv[:, :self.q_size].view(T, Hq, D)
        k = qkv[:, self.q_size:self.q_size + self.kv_size].view(T, Hkv, D)
        v = qkv[:, self.q_size + self.kv_size:].view(T, Hkv, D)
        inv_freq = None
        if self.position is not None:
            inv_freq = self.position.rotary_inv_freq()
            if inv_freq is None:
                self.position.apply(q, k, ctx.positions)
        ops.rope_store(q, k, v, ctx.positions, inv_freq,
                       group.slots if cache.writable else None, cache.k, cache.v,
                       cache.page_size)
        out = torch.empty((T, Hq, D), dtype=x.dtype, device=x.device)
        self.attend(out, q, cache, ctx, group)
        if defer_output:                    # (the norm that follows picks the kernels by the rows)
            return PendingProduct(out.view(T, Hq * D), self.o, self.o_blocked)
        return linear(out.view(T, Hq * D), self.o, blocked=self.o_blocked)

    # ---- which kernel takes which sequences --------------------------------------
    def decode_splits(self, ctx, n_dec: int, matrix_cores: bool, device) -> int:
        """How many workgroups share one sequence's keys: enough to fill the compute
        units a few times over, never finer than one turn of a workgroup."""
        if self.force_decode_splits:
            return self.force_decode_splits
        D = self.head_dim
        G = self.num_heads // self.num_kv_heads
        if matrix_cores:
            turn = 128                              # keys a workgroup takes per turn
            groups = self.num_kv_heads
        else:
            lpk = 1
            while lpk * 16 < D:
                lpk <<= 1
            turn = 2 * (256 // lpk)
            groups = self.num_kv_heads * (-(-G // 4))
        span = max(ctx.ctx_lens[:n_dec])
        if self.window:
            span = min(span, self.window)
        # measured on MI355X (256 compute units): the matrix-core kernel is best with about two
        # workgroups a compute unit, and without splits once the batch brings 1.75 for each
        # (batch 56 with 8 kv heads; at batch 24 to 48 two splits are 2 to 3 % of a step faster
        # than one); the other one with about four
        base = max(1, n_dec * groups)
        cus = ops.compute_units(device)
        if matrix_cores:
            want = 1 if 4 * base >= 7 * cus else -(-2 * cus // base)
        else:
            want = -(-4 * cus // base)
        return max(1, min(want, -(-span // turn), 64))

    def attend(self, out, q, cache, ctx, group) -> None:
        D, window = self.head_dim, self.window or 0
        n_dec = ctx.num_decode_seqs if D % 16 == 0 else 0
        if n_dec:
            mfma = (ops.attention_decode_mfma_fits(q.dtype, self.num_heads, self.num_kv_heads, D,
                                                   cache.page_size)
                    and q.stride(0) % 8 == 0)
            ops.attention_decode(out, q, cache.k, cache.v, ctx.q_start, ctx.ctx_len,
                                 group.block_table, n_dec, self.scale, window,
                                 self.decode_splits(ctx, n_dec, mfma, q.device), matrix_cores=mfma)
        if n_dec == ctx.num_seqs:
            return
        if (ops.attention_prefill_mfma_fits(q.dtype, self.num_kv_heads, D, cache.page_size)
                and q.stride(0) % 8 == 0):
            keys = max(ctx.ctx_lens[n_dec:])
            rows, groups = ops.attention_prefill_mfma_plan(
                q.device, self.num_heads, D, ctx.work[PORTIONS_64][0].numel(),
                ctx.work[PORTIONS_128][0].numel(), min(keys, window) if window else keys)
            ws, wo = ctx.work[PORTIONS_128 if rows == 128 else PORTIONS_64]
            ops.attention_prefill_mfma(out, q, cache.k, cache.v, ctx.q_start, ctx.ctx_len,
                                       group.block_table, ws, wo, self.scale, window, rows, groups)
        else:
            ws, wo = ctx.work[PORTIONS_16 if n_dec else ALL_16]
            ops.attention_generic(out, q, cache.k, cache.v, ctx.q_start, ctx.ctx_len,
                                  group.block_table, ws, wo, self.scale, window)

