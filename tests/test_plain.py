"""What fixes the plain implementation beside the reference's text: special
cases that reduce to a library routine, invariants, and the few vectors the
reference's own tests hold. Each is chosen so that a plausible mistake (a wrong
sign or pairing, a norm in the wrong place, eps outside the root) fails it."""
import copy
import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as pl
from tiny_configs import TINY_A, TINY_B


def random_weights(cfg, seed=0, std=0.1):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    D = pl.head_dim_of(cfg)
    Hq, Hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    r = lambda *s: std * torch.randn(*s, generator=g)
    w = {"model.embed_tokens.weight": r(V, H), "model.norm.weight": 1 + r(H)}
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = r(V, H)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w.update({p + "input_layernorm.weight": 1 + r(H), p + "post_attention_layernorm.weight": 1 + r(H),
                  p + "self_attn.q_proj.weight": r(Hq * D, H), p + "self_attn.k_proj.weight": r(Hkv * D, H),
                  p + "self_attn.v_proj.weight": r(Hkv * D, H), p + "self_attn.o_proj.weight": r(H, Hq * D),
                  p + "mlp.gate_proj.weight": r(I, H), p + "mlp.up_proj.weight": r(I, H),
                  p + "mlp.down_proj.weight": r(H, I)})
    return w


# ---- RMSNorm ---------------------------------------------------------------------
def test_rmsnorm_is_the_library_routine():
    x, w = torch.randn(5, 72, dtype=torch.double), torch.randn(72, dtype=torch.double)
    torch.testing.assert_close(pl.rms_norm(x, w, 1e-3), F.rms_norm(x, (72,), w, 1e-3))


def test_rmsnorm_invariants():
    x = torch.randn(4, 64, dtype=torch.double)
    y = pl.rms_norm(x, torch.ones(64, dtype=torch.double), 0.0)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(4, dtype=torch.double))
    torch.testing.assert_close(pl.rms_norm(7.5 * x, torch.ones(64, dtype=torch.double), 0.0), y)
    # eps sits inside the root: for x -> 0 the output is x / sqrt(eps)
    tiny = 1e-9 * x
    torch.testing.assert_close(pl.rms_norm(tiny, torch.ones(64, dtype=torch.double), 1e-4), tiny / 1e-2)


def test_add_rmsnorm_returns_the_sum_and_norms_it():
    x, r, w = torch.randn(3, 16), torch.randn(3, 16), torch.randn(16)
    y, res = pl.add_rms_norm(x, r, w, 1e-5)
    assert torch.equal(res, x + r)
    torch.testing.assert_close(y, pl.rms_norm(x + r, w, 1e-5))
    y0, res0 = pl.add_rms_norm(x, None, w, 1e-5)
    assert res0 is x                                    # skip_rmsnorm.py:181


def test_rmsnorm_reference_oracle_shapes():
    # python_rmsnorm of the reference (skip_rmsnorm.py:186-190): x / sqrt(mean(x^2)+eps) * w
    x, w = torch.randn(4, 128), torch.randn(128)
    var = x.pow(2).mean(dim=-1, keepdim=True)
    torch.testing.assert_close(pl.rms_norm(x, w, 1e-5), x / torch.sqrt(var + 1e-5) * w)


# ---- RoPE -------------------------------------------------------------------------
def test_inv_freq_default():
    f = pl.rope_inv_freq_default(10000.0, 8)
    assert f.shape == (4,) and f[0] == 1.0
    torch.testing.assert_close(f, torch.tensor([1.0, 0.1, 0.01, 0.001]))


def test_rope_is_complex_multiplication_on_half_split_pairs():
    """(x_j + i x_{j+D/2}) * exp(i pos w_j), the complex form of the reference's
    tests/test_torch_rope.py:40-68 on the half-split pairing of :242-272."""
    D, S = 16, 9
    x = torch.randn(S, 3, D, dtype=torch.double)
    inv = pl.rope_inv_freq_default(100.0, D).double()
    pos = torch.arange(S) * 3
    cos, sin = pl.rope_cos_sin(inv, pos)
    got = pl.apply_rope(x, cos.double(), sin.double())
    z = torch.complex(x[..., : D // 2], x[..., D // 2:])
    rot = torch.polar(torch.ones(S, D // 2, dtype=torch.double), pos[:, None].double() * inv[None])
    zz = z * rot[:, None]
    torch.testing.assert_close(got, torch.cat([zz.real, zz.imag], -1), atol=1e-6, rtol=1e-6)


def test_rope_invariants():
    D = 32
    inv = pl.rope_inv_freq_default(10000.0, D)
    q, k = torch.randn(1, 1, D, dtype=torch.double), torch.randn(1, 1, D, dtype=torch.double)

    def rot(x, p):
        c, s = pl.rope_cos_sin(inv, torch.tensor([p]))
        return pl.apply_rope(x, c.double(), s.double())

    assert torch.equal(rot(q, 0), q)                                     # position 0 is the identity
    c, s = pl.rope_cos_sin(inv, torch.tensor([5]))
    assert torch.equal(c[:, : D // 2], c[:, D // 2:])                     # halves share the angles
    r = rot(q, 11)
    torch.testing.assert_close(r[..., : D // 2] ** 2 + r[..., D // 2:] ** 2,
                               q[..., : D // 2] ** 2 + q[..., D // 2:] ** 2)  # each pair keeps its length
    a = (rot(q, 7) * rot(k, 3)).sum()
    b = (rot(q, 104) * rot(k, 100)).sum()
    torch.testing.assert_close(a, b, atol=1e-4, rtol=1e-4)               # only the distance counts
    assert abs(float(a - (rot(q, 3) * rot(k, 7)).sum())) > 1e-3           # and its sign does


def test_llama3_reduces_to_default():
    sc = {"rope_type": "llama3", "factor": 1.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 64}
    torch.testing.assert_close(pl.rope_inv_freq_llama3(5e5, 32, sc), pl.rope_inv_freq_default(5e5, 32))
    sc = dict(sc, factor=8.0, original_max_position_embeddings=10 ** 12)
    torch.testing.assert_close(pl.rope_inv_freq_llama3(5e5, 32, sc), pl.rope_inv_freq_default(5e5, 32))


def test_llama3_bands_of_tiny_b():
    sc = TINY_B["rope_scaling"]
    base = pl.rope_inv_freq_default(5e5, 32)
    got = pl.rope_inv_freq_llama3(5e5, 32, sc)
    wavelen = 2 * math.pi / base
    kept = wavelen < 64 / 4
    divided = wavelen > 64 / 1
    mid = ~kept & ~divided
    assert (int(kept.sum()), int(mid.sum()), int(divided.sum())) == (2, 1, 13)
    torch.testing.assert_close(got[kept], base[kept])
    torch.testing.assert_close(got[divided], base[divided] / 8)
    assert torch.all(got[mid] > base[mid] / 8) and torch.all(got[mid] < base[mid])


def _both_llama3(theta, dim, sc):
    """The plain function and the product's, on the same numbers."""
    from pytriton_llama_amd.parts.rotary import llama3_inv_freq
    return (pl.rope_inv_freq_llama3(theta, dim, sc),
            llama3_inv_freq(theta, dim, sc["factor"], sc["low_freq_factor"], sc["high_freq_factor"],
                            sc["original_max_position_embeddings"]))


@pytest.mark.parametrize("at, weight_of_kept", [(0.0, 0.0), (0.25, 0.25), (0.5, 0.5), (0.9, 0.9), (1.0, 1.0)])
def test_llama3_blend_weight_at_constructed_wavelengths(at, weight_of_kept):
    # RotaryEmbedding.py:90-98. dim 4 has the frequencies 1 and theta^-1/2; the original length
    # is chosen so that original / wavelength of the second lies at low + at * (high - low):
    # at = 0 is the edge of the divided band (result inv / factor), at = 1 the edge of the kept
    # band (result inv), and between them the kept share grows linearly with ``at``. A blend
    # weight the wrong way round (smooth <-> 1 - smooth) gives 0.75 where 0.25 is due.
    theta, factor, low, high = 400.0, 8.0, 1.0, 4.0
    inv = 1.0 / math.sqrt(theta)
    wavelen = 2 * math.pi / inv
    original = (low + at * (high - low)) * wavelen
    sc = {"factor": factor, "low_freq_factor": low, "high_freq_factor": high,
          "original_max_position_embeddings": original}
    want = inv * (weight_of_kept + (1.0 - weight_of_kept) / factor)
    for got in _both_llama3(theta, 4, sc):
        assert got.dtype == torch.float32 and got.shape == (2,)
        assert float(got[0]) == 1.0                                   # wavelength 2 pi: kept
        assert abs(float(got[1]) - want) <= 2e-6 * want, (float(got[1]), want)


def test_llama3_values_of_the_1b_parameters():
    # theta 5e5, head size 64, factor 32, low 1, high 4, original 8192 (Llama-3.2-1B's
    # config.json). Worked out in float64 outside both implementations: wavelengths below 2,048
    # are kept (j <= 14), above 8,192 divided by 32 (j >= 18), and j = 15, 16, 17 lie between
    # (2,948.30, 4,442.88 and 6,695.11): 8192 / wavelength = 2.7785, 1.8438, 1.2236, so the kept
    # share is 0.5928, 0.2813 and 0.0745.
    sc = {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
    want = {0: 1.0, 13: 0.004839421345719893, 14: 0.003211445994752591,
            15: 0.0012905479282092638, 16: 0.0004295567965593682, 17: 9.70828780262767e-05,
            18: 1.9461638184831125e-05, 19: 1.291476718704739e-05, 31: 9.41830672543491e-08}
    for got in _both_llama3(5e5, 64, sc):
        assert got.shape == (32,)
        for j, w in want.items():
            assert abs(float(got[j]) - w) <= 3e-6 * w, (j, float(got[j]), w)


def test_rope_parameters_of_the_reference_unit_test():
    # RotaryEmbedding.py:316-357: head_dim 4, llama3 (8, 1, 4, original 100): inv_freq has
    # head_dim // 2 entries and the cos/sin scale is 1.0
    cfg = {"hidden_size": 32, "num_attention_heads": 8, "head_dim": 4, "rope_theta": 10000,
           "rope_scaling": {"factor": 8, "low_freq_factor": 1, "high_freq_factor": 4,
                            "original_max_position_embeddings": 100, "rope_type": "llama3"}}
    inv = pl.rope_inv_freq(cfg)
    assert inv.shape[0] == 2
    cos, sin = pl.rope_cos_sin(inv, torch.arange(10))
    assert cos.shape == (10, 4) and sin.shape == (10, 4) and cos[0].eq(1).all() and sin[0].eq(0).all()
    with pytest.raises(KeyError):
        pl.rope_inv_freq(dict(cfg, rope_scaling={"rope_type": "yarn"}))


# ---- attention ------------------------------------------------------------------------
def test_attention_is_sdpa_with_repeated_kv():
    S, Hq, Hkv, D = 32, 4, 2, 64          # the reference's own test uses B2 H4 S32 D64
    q, k, v = torch.randn(S, Hq, D), torch.randn(S, Hkv, D), torch.randn(S, Hkv, D)
    got = pl.causal_attention(q, k, v, D ** -0.5)
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None],
                                          vv.transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)


def test_attention_group_mapping_is_blockwise():
    """Query head a reads kv head a // G (not a % Hkv)."""
    S, D = 5, 8
    q = torch.randn(S, 4, D)
    k, v = torch.randn(S, 2, D), torch.zeros(S, 2, D)
    v[:, 0] = 1.0
    v[:, 1] = -1.0
    out = pl.causal_attention(q, k, v, D ** -0.5)
    assert torch.allclose(out[:, 0], torch.ones(S, D)) and torch.allclose(out[:, 1], torch.ones(S, D))
    assert torch.allclose(out[:, 2], -torch.ones(S, D)) and torch.allclose(out[:, 3], -torch.ones(S, D))


def test_attention_invariants():
    S, D = 12, 16
    q, k, v = torch.randn(S, 2, D), torch.randn(S, 2, D), torch.randn(S, 2, D)
    out = pl.causal_attention(q, k, v, D ** -0.5)
    torch.testing.assert_close(out[0], v[0])                      # the first token sees itself only
    k2, v2 = k.clone(), v.clone()
    k2[7:], v2[7:] = torch.randn(5, 2, D), torch.randn(5, 2, D)
    out2 = pl.causal_attention(q, k2, v2, D ** -0.5)
    assert torch.equal(out[:7], out2[:7]) and not torch.allclose(out[7:], out2[7:])
    # additive -inf mask and index mask agree (tests/test_mask.py of the reference)
    scores = torch.einsum("qhd,khd->hqk", q, k) * D ** -0.5
    add = torch.triu(torch.full((S, S), float("-inf")), diagonal=1)
    want = torch.einsum("hqk,khd->qhd", torch.softmax(scores + add, -1), v)
    torch.testing.assert_close(out, want)
    # a window of S is no window; a window of 1 returns v
    torch.testing.assert_close(pl.causal_attention(q, k, v, D ** -0.5, window=S), out)
    torch.testing.assert_close(pl.causal_attention(q, k, v, D ** -0.5, window=1), v)
    # a few query rows alone are the same rows of the whole (with and without a window)
    rows = [0, 3, 4, 11]
    for window in (None, 5):
        whole = pl.causal_attention(q, k, v, D ** -0.5, window=window)
        some = pl.causal_attention(q[rows], k, v, D ** -0.5, window=window, query_positions=rows)
        torch.testing.assert_close(some, whole[rows])


def test_mha_without_rotation_is_nn_multihead_attention():
    H, heads, S = 32, 4, 10
    mha = torch.nn.MultiheadAttention(H, heads, bias=False, batch_first=True).double()
    x = torch.randn(S, H, dtype=torch.double)
    wq, wk, wv = mha.in_proj_weight.detach().chunk(3)
    w = {"q_proj.weight": wq, "k_proj.weight": wk, "v_proj.weight": wv,
         "o_proj.weight": mha.out_proj.weight.detach()}
    cfg = {"num_attention_heads": heads, "num_key_value_heads": heads, "hidden_size": H}
    cos, sin = torch.ones(S, H // heads, dtype=torch.double), torch.zeros(S, H // heads, dtype=torch.double)
    got = pl.attention_block(x, w, "", cfg, cos, sin)
    mask = torch.triu(torch.ones(S, S, dtype=torch.bool), diagonal=1)
    want, _ = mha(x[None], x[None], x[None], attn_mask=mask, need_weights=False)
    torch.testing.assert_close(got, want[0].detach(), atol=1e-9, rtol=1e-9)


# ---- feed-forward --------------------------------------------------------------------------
def test_swiglu():
    g, u = 3 * torch.randn(4, 20), torch.randn(4, 20)
    torch.testing.assert_close(pl.silu(g) * u, F.silu(g) * u)
    assert torch.all(pl.silu(torch.zeros(3)) == 0)
    big = torch.tensor([30.0])
    torch.testing.assert_close(pl.silu(big), big)
    x = torch.randn(3, 8)
    w = {"gate_proj.weight": torch.randn(12, 8), "up_proj.weight": torch.randn(12, 8),
         "down_proj.weight": torch.randn(8, 12)}
    want = (F.silu(x @ w["gate_proj.weight"].T) * (x @ w["up_proj.weight"].T)) @ w["down_proj.weight"].T
    torch.testing.assert_close(pl.swiglu_mlp(x, w, ""), want)


# ---- whole model ------------------------------------------------------------------------------
def test_zero_output_projections_leave_the_embedding():
    cfg = copy.deepcopy(TINY_B)
    w = random_weights(cfg, 1)
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    ids = [3, 50, 7, 300]
    x = w["model.embed_tokens.weight"][ids]
    want = pl.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["lm_head.weight"].T
    torch.testing.assert_close(pl.forward(cfg, w, ids), want)


def test_tied_head_is_the_embedding():
    cfg = copy.deepcopy(TINY_A)
    w = random_weights(cfg, 2)
    ids = [1, 2, 3, 4, 5]
    h = pl.forward(cfg, w, ids, return_hidden=True)
    torch.testing.assert_close(pl.forward(cfg, w, ids), h @ w["model.embed_tokens.weight"].T)


def test_model_is_causal_and_shift_invariant():
    cfg = copy.deepcopy(TINY_A)
    w = {k: v.double() for k, v in random_weights(cfg, 3, std=0.3).items()}
    ids = [9, 8, 7, 6, 5, 4, 3, 2]
    a = pl.forward(cfg, w, ids)
    b = pl.forward(cfg, w, ids[:5] + [100, 101, 102])
    torch.testing.assert_close(a[:5], b[:5])
    assert not torch.allclose(a[5:], b[5:])
    # without frequency scaling only distances between positions count
    c = pl.forward(cfg, w, ids, first_position=37)
    torch.testing.assert_close(a, c, atol=1e-5, rtol=1e-5)
    # order matters (positions are really used)
    d = pl.forward(cfg, w, [ids[1], ids[0]] + ids[2:])
    assert not torch.allclose(a[-1], d[-1])


def test_greedy_generation_appends_the_argmax():
    cfg = copy.deepcopy(TINY_A)
    w = random_weights(cfg, 4, std=0.3)
    out = pl.greedy_generate(cfg, w, [1, 2, 3], 3)
    assert out[0] == int(pl.forward(cfg, w, [1, 2, 3])[-1].argmax())
    assert out[1] == int(pl.forward(cfg, w, [1, 2, 3, out[0]])[-1].argmax())


# ---- sampling -------------------------------------------------------------------------------------
def test_top_p_rule():
    logits = torch.log(torch.tensor([0.15, 0.5, 0.05, 0.3]))
    # mass before 0.3 is 0.5 <= 0.7: kept; before 0.15 it is 0.8 > 0.7: dropped
    p = pl.top_p_probs(logits, 1.0, 0.7)
    torch.testing.assert_close(p, torch.tensor([0.0, 0.625, 0.0, 0.375], dtype=torch.double))
    torch.testing.assert_close(pl.top_p_probs(logits, 1.0, 1.0), torch.softmax(logits.double(), -1))
    assert pl.top_p_probs(logits, 1.0, 1e-9).tolist() == [0, 1, 0, 0]
    t = pl.top_p_probs(logits, 0.5, 1.0)
    torch.testing.assert_close(t, torch.softmax(logits.double() / 0.5, -1))
    assert abs(float(pl.top_p_probs(torch.randn(50), 0.8, 0.9).sum()) - 1) < 1e-12
