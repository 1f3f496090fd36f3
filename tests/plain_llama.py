"""Plain, slow implementation of the Llama decoder: the oracle of the test suite.

Whole sequences, no cache, one function for each part, float32 (or float64)
torch on the CPU. It shares no code with ``pytriton_llama_amd``: it reads
config.json and model.safetensors by itself and spells every formula out from
the reference's text. Each function cites the reference file:line it was read
from (paths relative to the reference tree, ``lite_llama/...``).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --------------------------------------------------------------------------
# reading a model folder (independent of the product's loader)
# --------------------------------------------------------------------------
def read_model_folder(folder: str, dtype=torch.float32):
    """Return (config dict, {HF tensor name: tensor in ``dtype``})."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return cfg, tensors


def head_dim_of(cfg: dict) -> int:
    # lite_llama/models/llama.py:17 takes config.head_dim when it is given and
    # hidden_size // num_heads otherwise.
    hd = cfg.get("head_dim")
    return int(hd) if hd else cfg["hidden_size"] // cfg["num_attention_heads"]


# --------------------------------------------------------------------------
# RMSNorm (with the residual sum in front of it)
# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """lite_llama/kernels/skip_rmsnorm.py:113-119: var = sum(x*x/N),
    rrms = 1/sqrt(var+eps), y = x*rrms*w. eps sits inside the square root."""
    var = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(var + eps)) * w


def add_rms_norm(x, residual, w, eps):
    """lite_llama/kernels/skip_rmsnorm.py:142-155 and :159-181: the residual is
    added first (x += r), the sum is what is returned as the new residual, and
    the norm is taken of the sum. Without a residual the input itself is
    returned as the residual (:181)."""
    if residual is not None:
        x = x + residual
    return rms_norm(x, w, eps), x


# --------------------------------------------------------------------------
# rotary position encoding
# --------------------------------------------------------------------------
def rope_inv_freq_default(theta: float, dim: int) -> torch.Tensor:
    """lite_llama/models/RotaryEmbedding.py:51: 1/(base**(arange(0,dim,2)/dim))."""
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))


def rope_inv_freq_llama3(theta: float, dim: int, scaling: dict) -> torch.Tensor:
    """lite_llama/models/RotaryEmbedding.py:77-100. Wavelengths longer than
    original/low_freq_factor are divided by ``factor``; shorter than
    original/high_freq_factor are kept; between them a linear blend."""
    inv_freq = rope_inv_freq_default(theta, dim)
    factor = scaling["factor"]
    low = scaling["low_freq_factor"]
    high = scaling["high_freq_factor"]
    old_len = scaling["original_max_position_embeddings"]
    low_wavelen = old_len / low
    high_wavelen = old_len / high
    wavelen = 2 * math.pi / inv_freq
    out = torch.where(wavelen > low_wavelen, inv_freq / factor, inv_freq)
    smooth = (old_len / wavelen - low) / (high - low)
    smoothed = (1 - smooth) * out / factor + smooth * out
    medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
    return torch.where(medium, smoothed, out)


def rope_inv_freq(cfg: dict) -> torch.Tensor:
    """lite_llama/models/RotaryEmbedding.py:133-136: the kind is
    rope_scaling["rope_type"] (older files: "type"), "default" without scaling."""
    dim = head_dim_of(cfg)
    theta = float(cfg.get("rope_theta", 10000.0))
    scaling = cfg.get("rope_scaling")
    if scaling is None:
        return rope_inv_freq_default(theta, dim)
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind == "llama3":
        return rope_inv_freq_llama3(theta, dim, scaling)
    if kind == "default":
        return rope_inv_freq_default(theta, dim)
    raise KeyError(kind)


def rope_cos_sin(inv_freq: torch.Tensor, positions: torch.Tensor):
    """lite_llama/models/RotaryEmbedding.py:200-220: angle = position*inv_freq
    in float32, the two halves of the head get the same angles, and
    attention_scaling (1.0, :48) multiplies both tables."""
    freqs = positions.float()[:, None] * inv_freq.float()[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos() * 1.0, emb.sin() * 1.0


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """lite_llama/kernels/rope_emb.py:75-103 (and torch_rotary_emb, :265-283):
    pairs are (j, j + D/2); o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin.
    x: [S, heads, D]; cos, sin: [S, D]."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c, s = cos[:, None, :half], sin[:, None, :half]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------
def causal_attention(q, k, v, scale: float, window: Optional[int] = None, query_positions=None):
    """q: [S, Hq, D]; k, v: [S, Hkv, D]. Query head a reads key/value head
    a // (Hq//Hkv) (lite_llama/kernels/flashattentionv2.py:108); scores are
    q.k*scale with scale = 1/sqrt(D) (lite_llama/models/llama.py:173), keys
    after the query are masked out (flashattentionv2.py:24,37-38), softmax over
    the keys, then the weighted sum of the values (:40-61,160). ``window`` is
    not in the reference (Llama has none); it is here for the engine's general
    attention part: a query at p then sees keys p-window+1 .. p.
    ``query_positions``: q holds only the queries at these positions of the
    sequence ([R, Hq, D]; the result has the same rows), so that a few rows of
    a long sequence cost R x S scores instead of S x S."""
    S = k.shape[0]
    Hq = q.shape[1]
    Hkv = k.shape[1]
    G = Hq // Hkv
    kk = k.repeat_interleave(G, dim=1)
    vv = v.repeat_interleave(G, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, kk) * scale
    qi = (torch.arange(S) if query_positions is None
          else torch.as_tensor(query_positions, dtype=torch.long))[:, None]
    ki = torch.arange(S)[None, :]
    mask = ki <= qi
    if window is not None:
        mask = mask & (ki > qi - window)
    scores = scores.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    return torch.einsum("hqk,khd->qhd", p, vv)


def attention_block(x, w, prefix, cfg, cos, sin):
    """lite_llama/models/llama.py:37-61: q/k/v projections without bias, RoPE on
    q and k, causal attention, output projection."""
    S = x.shape[0]
    Hq = cfg["num_attention_heads"]
    Hkv = cfg.get("num_key_value_heads") or Hq
    D = head_dim_of(cfg)
    q = (x @ w[prefix + "q_proj.weight"].T).view(S, Hq, D)
    k = (x @ w[prefix + "k_proj.weight"].T).view(S, Hkv, D)
    v = (x @ w[prefix + "v_proj.weight"].T).view(S, Hkv, D)
    q = apply_rope(q, cos, sin)
    k = apply_rope(k, cos, sin)
    o = causal_attention(q, k, v, 1.0 / math.sqrt(D))
    return o.reshape(S, Hq * D) @ w[prefix + "o_proj.weight"].T


# --------------------------------------------------------------------------
# feed-forward
# --------------------------------------------------------------------------
def silu(x):
    """lite_llama/kernels/swiglu.py:44-46: x * sigmoid(x)."""
    return x * torch.sigmoid(x)


def swiglu_mlp(x, w, prefix):
    """lite_llama/models/llama.py:120 with lite_llama/kernels/swiglu.py:64-66:
    down(silu(gate(x)) * up(x))."""
    g = x @ w[prefix + "gate_proj.weight"].T
    u = x @ w[prefix + "up_proj.weight"].T
    return (silu(g) * u) @ w[prefix + "down_proj.weight"].T


# --------------------------------------------------------------------------
# whole model
# --------------------------------------------------------------------------
def forward(cfg: dict, w: Dict[str, torch.Tensor], token_ids: Sequence[int],
            return_hidden: bool = False, first_position: int = 0) -> torch.Tensor:
    """Logits [S, V] of one whole sequence. lite_llama/models/llama.py:189-223:
    embedding, then per layer (llama.py:149-162) add+norm, attention, add+norm,
    MLP with the residual carried beside the hidden state, a last add+norm
    (:219) and the head (:221). With tied embeddings the head is the embedding
    matrix (lite_llama/executor/weight_convert.py:196)."""
    ids = torch.as_tensor(list(token_ids), dtype=torch.long)
    dtype = w["model.embed_tokens.weight"].dtype
    eps = float(cfg.get("rms_norm_eps", 1e-5))
    h = w["model.embed_tokens.weight"][ids]
    cos, sin = rope_cos_sin(rope_inv_freq(cfg), first_position + torch.arange(len(ids)))
    cos, sin = cos.to(dtype), sin.to(dtype)
    residual = None
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h, residual = add_rms_norm(h, residual, w[p + "input_layernorm.weight"], eps)
        h = attention_block(h, w, p + "self_attn.", cfg, cos, sin)
        h, residual = add_rms_norm(h, residual, w[p + "post_attention_layernorm.weight"], eps)
        h = swiglu_mlp(h, w, p + "mlp.")
    h, _ = add_rms_norm(h, residual, w["model.norm.weight"], eps)
    if return_hidden:
        return h
    head = w.get("lm_head.weight")
    if head is None or cfg.get("tie_word_embeddings", True):
        head = w["model.embed_tokens.weight"]
    return h @ head.T


def greedy_generate(cfg, w, prompt: Sequence[int], n_new: int) -> List[int]:
    """lite_llama/generate_stream.py:150: argmax of the last position's logits,
    appended, and the whole sequence run again (no cache here)."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(cfg, w, ids)[-1]
        t = int(torch.argmax(logits))
        ids.append(t)
        out.append(t)
    return out


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------
def top_p_probs(logits: torch.Tensor, temperature: float, top_p: float) -> torch.Tensor:
    """The distribution lite_llama/generate.py:30-38 draws from: softmax of
    logits/temperature (generate_stream.py:146), sorted descending, a token is
    dropped when the mass before it exceeds top_p, the rest renormalised.
    Returned in vocabulary order."""
    probs = torch.softmax(logits.double() / temperature, dim=-1)
    sp, idx = torch.sort(probs, dim=-1, descending=True)
    cum = torch.cumsum(sp, dim=-1)
    sp = torch.where(cum - sp > top_p, torch.zeros_like(sp), sp)
    sp = sp / sp.sum(dim=-1, keepdim=True)
    out = torch.zeros_like(probs)
    out.scatter_(-1, idx, sp)
    return out
