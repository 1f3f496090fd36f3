"""Each part alone on the GPU, and a model put together from the package's parts
and the tests' toy parts: a mixer with state of its own beside windowed paged
attention, another norm, another feed-forward, a layer that runs twice."""
import copy
import math

import pytest
import torch

import cuttings
import plain_llama
import toy_parts  # noqa: F401
from engine_helpers import replay

pytestmark = pytest.mark.gpu


def test_rmsnorm_part(gpu_device):
    from pytriton_llama_amd.parts import build_part
    n = build_part("norm", "rmsnorm", size=72, eps=1e-3)
    w = 1 + 0.1 * torch.randn(72)
    n.load({"weight": w}, torch.float32, gpu_device)
    x, r = torch.randn(5, 72), torch.randn(5, 72)
    y, res = n.forward(x.cuda(), r.clone().cuda())
    wy, wr = plain_llama.add_rms_norm(x, r, w, 1e-3)
    torch.testing.assert_close(y.cpu(), wy, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(res.cpu(), wr)
    xc = x.cuda()
    y0, res0 = n.forward(xc, None)
    assert res0 is xc


def test_pending_values_between_parts(gpu_device):
    """A product left undone goes into the norm's kernel, the norm's rsqrt factor into the next
    product: a feed-forward -> norm -> feed-forward chain built that way gives what the parts give
    with finished tensors in between; a receiver that knows nothing of it gets tensors."""
    from pytriton_llama_amd.parts import build_part
    from pytriton_llama_amd.parts.base import PendingProduct, PendingScale, as_tensor, run_norm
    torch.manual_seed(3)
    H, I, M = 136, 208, 5
    ff1 = build_part("feed_forward", "swiglu", hidden_size=H, intermediate_size=I)
    ff2 = build_part("feed_forward", "swiglu", hidden_size=H, intermediate_size=I)
    for ff in (ff1, ff2):
        ff.load({"gate_proj.weight": 0.1 * torch.randn(I, H), "up_proj.weight": 0.1 * torch.randn(I, H),
                 "down_proj.weight": 0.1 * torch.randn(H, I)}, torch.bfloat16, gpu_device)
    norm = build_part("norm", "rmsnorm", size=H, eps=1e-5)
    norm.load({"weight": 1 + 0.2 * torch.randn(H)}, torch.bfloat16, gpu_device)
    x = torch.randn(M, H, device="cuda").to(torch.bfloat16)
    res = torch.randn(M, H, device="cuda").to(torch.bfloat16)
    # finished tensors everywhere
    r_plain = res.clone()
    y1 = ff1.forward(x)
    n1, r_plain = norm.forward(y1, r_plain)
    want = ff2.forward(n1)
    # work handed on
    r_lazy = res.clone()
    p = ff1.forward(x, defer_output=True)
    assert isinstance(p, PendingProduct) and p.shape == (M, H)
    torch.testing.assert_close(p.tensor().float(), y1.float(), atol=1e-2, rtol=1e-2)
    s, r_lazy = run_norm(norm, p, r_lazy, consumer=ff2)
    assert isinstance(s, PendingScale)
    assert torch.equal(r_lazy, r_plain)
    torch.testing.assert_close(s.tensor().float(), n1.float(), atol=3e-2, rtol=2e-2)
    got = ff2.forward(s)
    torch.testing.assert_close(got.float(), want.float(), atol=3e-2, rtol=3e-2)
    # a consumer without the flag, and no consumer: the norm finishes its work itself
    toy = build_part("feed_forward", "toy_relu", hidden_size=H, inner=64)
    r3 = res.clone()
    t, r3 = run_norm(norm, ff1.forward(x, defer_output=True), r3, consumer=toy)
    assert isinstance(t, torch.Tensor) and torch.equal(r3, r_plain)
    torch.testing.assert_close(t.float(), n1.float(), atol=3e-2, rtol=2e-2)
    assert as_tensor(t) is t
    # any number of rows is left to the norm, which picks the kernels by the rows: for 40 rows
    # (no blocked copy of the weights here) the product and the norm as separate kernels
    many = torch.randn(40, H, device="cuda").to(torch.bfloat16)
    res40 = torch.randn(40, H, device="cuda").to(torch.bfloat16)
    p40 = ff1.forward(many, defer_output=True)
    assert isinstance(p40, PendingProduct) and p40.shape == (40, H)
    r_a, r_b = res40.clone(), res40.clone()
    got40, r_a = run_norm(norm, p40, r_a, consumer=ff2)
    want40, r_b = norm.forward(ff1.forward(many), r_b)
    assert isinstance(got40, torch.Tensor) and torch.equal(got40, want40) and torch.equal(r_a, r_b)
    # ... and with the blocked copies, for 17 to 64 rows, the product as partial sums and one
    # kernel that adds them up and normalises
    # (widths that are multiples of 32, which the blocked copies need)
    H2, I2 = 128, 256
    ff3 = build_part("feed_forward", "swiglu", hidden_size=H2, intermediate_size=I2)
    ff3.load({"gate_proj.weight": 0.1 * torch.randn(I2, H2), "up_proj.weight": 0.1 * torch.randn(I2, H2),
              "down_proj.weight": 0.1 * torch.randn(H2, I2)}, torch.bfloat16, gpu_device)
    norm2 = build_part("norm", "rmsnorm", size=H2, eps=1e-5)
    norm2.load({"weight": 1 + 0.2 * torch.randn(H2)}, torch.bfloat16, gpu_device)
    many = torch.randn(40, H2, device="cuda").to(torch.bfloat16)
    res40 = torch.randn(40, H2, device="cuda").to(torch.bfloat16)
    r_b = res40.clone()
    want40, r_b = norm2.forward(ff3.forward(many), r_b)
    ff3.make_decode_copies()
    p40 = ff3.forward(many, defer_output=True)
    assert isinstance(p40, PendingProduct) and p40.blocked is not None
    r_c = res40.clone()
    got40b, r_c = run_norm(norm2, p40, r_c, consumer=ff3)
    assert isinstance(got40b, torch.Tensor)
    torch.testing.assert_close(got40b.float(), want40.float(), atol=3e-2, rtol=2e-2)
    torch.testing.assert_close(r_c.float(), r_b.float(), atol=2e-2, rtol=2e-2)


def test_rotary_part_alone(gpu_device):
    from pytriton_llama_amd.parts import build_part
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    rot = build_part("position", "rotary", head_dim=32, theta=5e5, **sc)
    torch.testing.assert_close(rot.inv_freq_host, plain_llama.rope_inv_freq_llama3(5e5, 32, sc))
    rot.load({}, torch.float32, gpu_device)
    buf = torch.randn(6, (3 + 1) * 32, device="cuda")
    orig = buf.cpu().clone()
    q, k = buf[:, :96].view(6, 3, 32), buf[:, 96:].view(6, 1, 32)
    pos = torch.tensor([0, 1, 63, 64, 500, 9], dtype=torch.int32, device="cuda")
    rot.apply(q, k, pos)
    cos, sin = plain_llama.rope_cos_sin(rot.inv_freq_host, pos.cpu())
    torch.testing.assert_close(q.cpu(), plain_llama.apply_rope(orig[:, :96].view(6, 3, 32), cos, sin),
                               atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(k.cpu(), plain_llama.apply_rope(orig[:, 96:].view(6, 1, 32), cos, sin),
                               atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_swiglu_part(gpu_device, dtype):
    from pytriton_llama_amd.parts import build_part
    ff = build_part("feed_forward", "swiglu", hidden_size=72, intermediate_size=200)
    w = {"gate_proj.weight": 0.1 * torch.randn(200, 72), "up_proj.weight": 0.1 * torch.randn(200, 72),
         "down_proj.weight": 0.1 * torch.randn(72, 200)}
    ff.load(w, dtype, gpu_device)
    x = torch.randn(9, 72)
    wr = {k: v.to(dtype).float() for k, v in w.items()}
    want = plain_llama.swiglu_mlp(x.to(dtype).float(), wr, "")
    got = ff.forward(x.to(dtype).cuda()).float().cpu()
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    torch.testing.assert_close(got, want, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_embedding_and_head_parts(gpu_device, dtype):
    from pytriton_llama_amd.parts import build_part
    emb = build_part("embedding", "token_embedding", vocab_size=300, hidden_size=72)
    table = torch.randn(300, 72)
    emb.load({"weight": table}, dtype, gpu_device)
    ids = torch.tensor([0, 299, 7], dtype=torch.int32, device="cuda")
    x = emb.forward(ids)
    assert torch.equal(x.cpu(), table.to(dtype)[[0, 299, 7]])
    head = build_part("head", "linear_head", vocab_size=300, hidden_size=72, tied_to=emb)
    assert head.param_sources() == []
    logits = head.forward(x)
    assert logits.dtype == torch.float32
    want = table.to(dtype).float()[[0, 299, 7]] @ table.to(dtype).float().T
    torch.testing.assert_close(logits.cpu(), want, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_attention_part_alone(gpu_device, dtype):
    """The mixer with a cache of its own, fed in two portions, against plain
    attention over the whole sequence; scale and window are parameters."""
    from pytriton_llama_amd.cache import CacheManager, CacheStorage
    from pytriton_llama_amd.engine.batch import StepEntry, build_context
    from pytriton_llama_amd.parts import build_part
    H, Hq, Hkv, D, S = 40, 4, 2, 16, 37
    for window, scale in ((None, None), (9, 0.5)):
        pos = build_part("position", "rotary", head_dim=D, theta=100.0)
        att = build_part("mixer", "paged_attention", hidden_size=H, num_heads=Hq, num_kv_heads=Hkv,
                         head_dim=D, position=pos, scale=scale, window=window)
        g = torch.Generator().manual_seed(3)
        w = {n: 0.15 * torch.randn(s, generator=g) for n, s in
             (("q_proj.weight", (Hq * D, H)), ("k_proj.weight", (Hkv * D, H)),
              ("v_proj.weight", (Hkv * D, H)), ("o_proj.weight", (H, Hq * D)))}
        att.load(w, dtype, gpu_device)
        x = torch.randn(S, H, generator=g).to(dtype)
        mgr = CacheManager([att.cache_spec()], 4, 12, 2)
        store = CacheStorage(mgr, dtype, gpu_device)
        mgr.admit("r")
        ys = []
        for lo, hi in ((0, 20), (20, 37)):
            ctx, _ = build_context([StepEntry("r", [0] * (hi - lo), [])], mgr, gpu_device,
                                   work_lists=att.work_lists())
            ys.append(att.forward(x[lo:hi].cuda(), ctx, store.view(0)))
            mgr.release_behind_window("r")
        got = torch.cat(ys).float().cpu()
        wr = {k: v.to(dtype).float() for k, v in w.items()}
        xf = x.float()
        q = (xf @ wr["q_proj.weight"].T).view(S, Hq, D)
        k = (xf @ wr["k_proj.weight"].T).view(S, Hkv, D)
        v = (xf @ wr["v_proj.weight"].T).view(S, Hkv, D)
        cos, sin = plain_llama.rope_cos_sin(plain_llama.rope_inv_freq_default(100.0, D), torch.arange(S))
        o = plain_llama.causal_attention(plain_llama.apply_rope(q, cos, sin),
                                         plain_llama.apply_rope(k, cos, sin), v,
                                         scale or 1 / math.sqrt(D), window)
        want = o.reshape(S, Hq * D) @ wr["o_proj.weight"].T
        # error relative to the largest output, as for logits: 2e-4 in float32; in bfloat16
        # q, k, v, the attention output and the result are each rounded to 8 bits
        err = float((got - want).abs().max() / want.abs().max())
        assert err < (2e-4 if dtype == torch.float32 else 3e-2), err
        if window:
            assert mgr.block_table("r", 0)[0] == -1          # pages behind the window went back


HYBRID = {"architectures": ["ToyStateLM"], "vocab_size": 90, "hidden_size": 48, "inner": 100,
          "layers": ["state", "attention", "attention"], "order": [0, 1, 2, 1], "decay": 0.7,
          "toy_norm": False, "toy_ffn": False, "heads": 3, "kv_heads": 1, "head_dim": 16,
          "window": 24, "initializer_range": 0.25}


def hybrid_plain(model, ids):
    """Whole-sequence forward of the hybrid toy model with plain formulas."""
    dev = "cpu"
    x = model.embedding.weight.float().cpu()[torch.as_tensor(ids)]
    h, residual = x, None
    for call in model.schedule:
        b = model.blocks[call.block]
        h, residual = plain_llama.add_rms_norm(h, residual, b.input_norm.weight.cpu(), b.input_norm.eps)
        m = b.mixer
        if hasattr(m, "decay"):
            u = h @ m.w.float().cpu().T
            s = torch.zeros(u.shape[1])
            ys = []
            for t in range(u.shape[0]):
                s = m.decay * s + u[t]
                ys.append(s)
            h = torch.stack(ys)
        else:
            S = h.shape[0]
            qkv = h @ m.qkv.float().cpu().T
            q = qkv[:, :m.q_size].view(S, m.num_heads, m.head_dim)
            k = qkv[:, m.q_size:m.q_size + m.kv_size].view(S, m.num_kv_heads, m.head_dim)
            v = qkv[:, m.q_size + m.kv_size:].view(S, m.num_kv_heads, m.head_dim)
            cos, sin = plain_llama.rope_cos_sin(m.position.inv_freq_host, torch.arange(S))
            o = plain_llama.causal_attention(plain_llama.apply_rope(q, cos, sin),
                                             plain_llama.apply_rope(k, cos, sin), v, m.scale, m.window)
            h = o.reshape(S, -1) @ m.o.float().cpu().T
        h, residual = plain_llama.add_rms_norm(h, residual, b.post_norm.weight.cpu(), b.post_norm.eps)
        ff = b.feed_forward
        gu = h @ ff.gate_up.float().cpu().T
        I = ff.intermediate_size
        h = (plain_llama.silu(gu[:, :I]) * gu[:, I:]) @ ff.down.float().cpu().T
    h, _ = plain_llama.add_rms_norm(h, residual, model.final_norm.weight.cpu(), model.final_norm.eps)
    return h @ model.head.weight.float().cpu().T


def test_toy_state_mixer_beside_windowed_attention(gpu_device):
    """Registered, built and stepped without a change to the package: layer 0
    keeps a state vector per request, layers 1 and 2 keep windowed keys in pages
    (given back as the window moves on), and layer 1 runs twice with a memory for
    each run. All cuttings agree with the plain whole-sequence result."""
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_random_weights
    model = build_model(copy.deepcopy(HYBRID))
    load_random_weights(model, 9, torch.float32, gpu_device, norm_std=0.1)
    g = torch.Generator().manual_seed(6)
    seqs = {f"r{i}": torch.randint(0, 90, (n,), generator=g).tolist()
            for i, n in enumerate([70, 35, 101, 64, 50])}
    want = {rid: hybrid_plain(model, t) for rid, t in seqs.items()}
    for steps in (cuttings.whole(seqs), cuttings.tail_decode(seqs, 32), cuttings.portions(seqs),
                  cuttings.mixed(seqs, seed=2)):
        runner = ModelRunner(model, page_size=8, num_pages=40, max_num_seqs=4)
        assert len(runner.manager.paged) == 1 and len(runner.manager.states) == 1
        got = replay(runner, steps, seqs)
        for rid in seqs:
            scale = float(want[rid].abs().max())
            err = (got[rid] - want[rid]).abs().max() / scale
            assert err < 2e-4, (rid, float(err))
        assert runner.manager.paged[0].pool.num_free == 40
    # with a window, a long request holds only the pages the window covers
    runner = ModelRunner(model, page_size=8, num_pages=40, max_num_seqs=4)
    replay(runner, [{"step": 0, "entries": [{"id": "r2", "tokens": seqs["r2"], "want": []}], "end": []}],
           {"r2": seqs["r2"]})
    held = sum(p >= 0 for p in runner.manager.block_table("r2", 0))
    assert held <= 24 // 8 + 2 < len(runner.manager.block_table("r2", 0))


ROUTED = {"architectures": ["ToyStateLM"], "vocab_size": 80, "hidden_size": 40, "inner": 24, "experts": 5,
          "layers": ["attention", "state", "attention"], "order": [0, 1, 2], "decay": 0.8, "heads": 5,
          "kv_heads": 1, "head_dim": 16, "toy_norm": True, "toy_ffn": True, "toy_position": True,
          "initializer_range": 0.25}


def routed_plain(model, ids):
    """Whole-sequence logits of the ROUTED toy model, no cache, formulas spelt out here."""
    ids = torch.as_tensor(ids)
    S = len(ids)
    h, residual = model.embedding.weight.float().cpu()[ids], None
    for call in model.schedule:
        b = model.blocks[call.block]
        s = h if residual is None else h + residual
        h, residual = s - s.mean(-1, keepdim=True), s
        m = b.mixer
        if hasattr(m, "decay"):
            u = h @ m.w.float().cpu().T
            st = torch.zeros(u.shape[1])
            ys = []
            for t in range(S):
                st = m.decay * st + u[t]
                ys.append(st)
            h = torch.stack(ys)
        else:
            qkv = h @ m.qkv.float().cpu().T
            q = qkv[:, :m.q_size].view(S, m.num_heads, m.head_dim)
            k = qkv[:, m.q_size:m.q_size + m.kv_size].view(S, m.num_kv_heads, m.head_dim)
            v = qkv[:, m.q_size + m.kv_size:].view(S, m.num_kv_heads, m.head_dim)
            f = torch.exp(torch.arange(S).float()[:, None, None] * m.position.log_g[None, None, :])
            o = plain_llama.causal_attention(q * f, k / f, v, m.scale)
            h = o.reshape(S, -1) @ m.o.float().cpu().T
        s = h + residual
        h, residual = s - s.mean(-1, keepdim=True), s
        ff = b.feed_forward
        logits = h @ ff.router.cpu().T
        out = torch.zeros_like(h)
        for t in range(S):
            top, idx = logits[t].topk(2)
            mix = torch.softmax(top, dim=-1)
            for slot in range(2):
                e = int(idx[slot])
                out[t] += mix[slot] * (torch.relu(h[t] @ ff.w1[e].float().cpu().T) @ ff.w2[e].float().cpu().T)
        h = out
    s = h + residual
    h = s - s.mean(-1, keepdim=True)
    return h @ model.head.weight.float().cpu().T


def test_toy_routed_feed_forward_and_toy_position_encoding(gpu_device):
    """A feed-forward with routing (five experts, two per token) and a position encoding that is
    no rotation, both defined in the tests, in a model with paged attention and a state mixer:
    all cuttings agree with the plain whole-sequence result."""
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_random_weights
    model = build_model(copy.deepcopy(ROUTED))
    load_random_weights(model, 4, torch.float32, gpu_device)
    g = torch.Generator().manual_seed(8)
    seqs = {f"r{i}": torch.randint(0, 80, (n,), generator=g).tolist() for i, n in enumerate([66, 40, 97, 51])}
    want = {rid: routed_plain(model, t) for rid, t in seqs.items()}
    # every expert is used by some token, or the routing is not tested
    ff = model.blocks[0].feed_forward
    x = model.embedding.weight[torch.tensor(seqs["r2"], device="cuda")]
    assert len(set((x.float() @ ff.router.T).topk(2, dim=-1).indices.flatten().tolist())) == 5
    for steps in (cuttings.whole(seqs), cuttings.tail_decode(seqs, 32), cuttings.portions(seqs),
                  cuttings.mixed(seqs, seed=3)):
        runner = ModelRunner(model, page_size=8, num_pages=48, max_num_seqs=4)
        got = replay(runner, steps, seqs)
        for rid in seqs:
            err = (got[rid] - want[rid]).abs().max() / float(want[rid].abs().max())
            assert err < 2e-4, (rid, float(err))
        assert runner.manager.paged[0].pool.num_free == 48


STATE_ON_DEVICE = {"architectures": ["ToyStateLM"], "vocab_size": 70, "hidden_size": 48, "inner": 96,
                   "layers": ["state_on_device", "attention", "state_on_device"], "order": [0, 1, 2],
                   "toy_norm": False, "toy_ffn": False, "heads": 3, "kv_heads": 1, "head_dim": 16,
                   "initializer_range": 0.25}


def state_on_device_plain(model, ids):
    """Whole-sequence logits of the model above, formulas spelt out, on the CPU."""
    h, residual = model.embedding.weight.float().cpu()[torch.as_tensor(ids)], None
    for call in model.schedule:
        b = model.blocks[call.block]
        h, residual = plain_llama.add_rms_norm(h, residual, b.input_norm.weight.cpu(), b.input_norm.eps)
        m = b.mixer
        if hasattr(m, "decay"):
            u = h @ m.w.float().cpu().T + m.bias.cpu()
            s, ys = torch.zeros(u.shape[1]), []
            for t in range(u.shape[0]):
                s = m.decay.cpu() * s + u[t]
                ys.append(s)
            h = torch.stack(ys)
        else:
            S = h.shape[0]
            qkv = h @ m.qkv.float().cpu().T
            q = qkv[:, :m.q_size].view(S, m.num_heads, m.head_dim)
            k = qkv[:, m.q_size:m.q_size + m.kv_size].view(S, m.num_kv_heads, m.head_dim)
            v = qkv[:, m.q_size + m.kv_size:].view(S, m.num_kv_heads, m.head_dim)
            cos, sin = plain_llama.rope_cos_sin(m.position.inv_freq_host, torch.arange(S))
            o = plain_llama.causal_attention(plain_llama.apply_rope(q, cos, sin),
                                             plain_llama.apply_rope(k, cos, sin), v, m.scale)
            h = o.reshape(S, -1) @ m.o.float().cpu().T
        h, residual = plain_llama.add_rms_norm(h, residual, b.post_norm.weight.cpu(), b.post_norm.eps)
        ff = b.feed_forward
        gu = h @ ff.gate_up.float().cpu().T
        I = ff.intermediate_size
        h = (plain_llama.silu(gu[:, :I]) * gu[:, I:]) @ ff.down.float().cpu().T
    h, _ = plain_llama.add_rms_norm(h, residual, model.final_norm.weight.cpu(), model.final_norm.eps)
    return h @ model.head.weight.float().cpu().T


def test_toy_state_mixer_keeps_graphs_and_steps_launched_ahead(gpu_device):
    """A model with fixed-size state per request is replayed as HIP graphs like any other (the
    rows that pad a step name the padding slot, and the run that records a graph touches no
    request's state), and its decode steps are launched ahead of their tokens."""
    from pytriton_llama_amd.config import EngineConfig, build_model
    from pytriton_llama_amd.engine import Engine, SamplingParams
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_random_weights
    model = build_model(copy.deepcopy(STATE_ON_DEVICE))
    assert model.graph_capturable()
    load_random_weights(model, 4, torch.float32, gpu_device, norm_std=0.1)
    decay = model.blocks[0].mixer.decay
    assert float(decay.min()) >= 0.5 and float(decay.max()) <= 0.9       # the part's own init hint
    g = torch.Generator().manual_seed(8)
    seqs = {f"r{i}": torch.randint(0, 70, (n,), generator=g).tolist() for i, n in enumerate([40, 21, 57, 33])}
    want = {rid: state_on_device_plain(model, t) for rid, t in seqs.items()}
    for steps in (cuttings.tail_decode(seqs, 12), cuttings.portions(seqs), cuttings.mixed(seqs, seed=4)):
        for st in steps:                         # one wanted place a portion: such steps are replayed
            for e in st["entries"]:
                e["want"] = e["want"][-1:]
        runner = ModelRunner(model, page_size=8, num_pages=40, max_num_seqs=4, max_model_len=64,
                             use_graphs=True)
        assert runner.graphs is not None and len(runner.manager.states) == 1
        # the padding slot belongs to nobody and may hold anything: what the rows that pad a
        # step read there and write back reaches no request
        runner.storage.state_pools[0][:, runner.manager.padding_slot] = float("nan")
        from engine_helpers import replay_wanted
        got = replay_wanted(runner, steps)
        assert all(bool(torch.isfinite(v).all()) for v in got.values())
        places = cuttings.wanted_places(steps)
        for rid in seqs:
            ref = want[rid][places[rid]]
            err = (got[rid] - ref).abs().max() / ref.abs().max()
            assert err < 2e-4, (rid, float(err))
        assert runner.graphs.buckets and runner.portion_graphs.buckets, "nothing was replayed"
    # through the engine: steps launched ahead give the tokens of the engine that waits
    prompts = [t[:9] for t in seqs.values()]
    sp = SamplingParams(temperature=0.0, max_new_tokens=10)
    outs = {}
    for name, kw in (("eager", dict(use_graphs=False)), ("ahead", dict(use_graphs=True, async_decode=True))):
        eng = Engine(copy.deepcopy(STATE_ON_DEVICE), EngineConfig(
            dtype="float32", page_size=8, num_pages=40, max_num_seqs=4, max_model_len=64, **kw),
            random_seed=4, norm_std=0.1)
        outs[name] = eng.generate(prompts, sp)
        assert (eng.runner.graphs is not None) == (name == "ahead")
    assert outs["eager"] == outs["ahead"]
    for p, o in zip(prompts, outs["eager"]):
        ref = state_on_device_plain(model, p + o)
        assert o == [int(ref[len(p) - 1 + i].argmax()) for i in range(len(o))]


CHUNKED = {"architectures": ["ToyStateLM"], "vocab_size": 75, "hidden_size": 48, "inner": 96,
           "layers": ["chunked", "attention", "chunked"], "order": [0, 1, 2], "decay": 0.85,
           "toy_norm": False, "toy_ffn": False, "heads": 3, "kv_heads": 1, "head_dim": 16,
           "initializer_range": 0.25}


def test_toy_mixer_gets_the_work_list_it_asks_for(gpu_device):
    """A mixer defined here that walks blocks of 32 query rows (no kernel of the package cuts
    rows so) names that list and finds it in every step: launched kernel by kernel (the list
    has exactly the step's blocks), in recorded decode steps and in recorded steps with a
    portion (the list has the size class's length and ends in empty items). All cuttings agree
    with the plain whole-sequence result; a row left out of the list would stay zero."""
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.parts import WorkList
    from pytriton_llama_amd.weights import load_random_weights
    from engine_helpers import replay_wanted
    model = build_model(copy.deepcopy(CHUNKED))
    assert model.graph_capturable()
    assert WorkList(32) in model.work_lists() and WorkList(64, after_decode=True) in model.work_lists()
    load_random_weights(model, 5, torch.float32, gpu_device, norm_std=0.1)
    g = torch.Generator().manual_seed(3)
    seqs = {f"r{i}": torch.randint(0, 75, (n,), generator=g).tolist() for i, n in enumerate([70, 33, 101, 45])}
    want = {rid: hybrid_plain(model, t) for rid, t in seqs.items()}
    for steps in (cuttings.whole(seqs), cuttings.tail_decode(seqs, 32), cuttings.portions(seqs),
                  cuttings.mixed(seqs, seed=5)):
        runner = ModelRunner(model, page_size=8, num_pages=40, max_num_seqs=4)
        got = replay(runner, steps, seqs)
        for rid in seqs:
            err = (got[rid] - want[rid]).abs().max() / float(want[rid].abs().max())
            assert err < 2e-4, (rid, float(err))
    only_portions = cuttings.portions(seqs, sizes=(40, 2, 33, 5, 64))      # (no step of single tokens)
    only_portions[0]["step"] = "portions"
    for steps in (cuttings.tail_decode(seqs, 12), only_portions, cuttings.mixed(seqs, seed=6)):
        for st in steps:                         # one wanted place a portion: such steps are replayed
            for e in st["entries"]:
                e["want"] = e["want"][-1:]
        runner = ModelRunner(model, page_size=8, num_pages=48, max_num_seqs=4, max_model_len=128,
                             use_graphs=True)
        got = replay_wanted(runner, steps)
        places = cuttings.wanted_places(steps)
        for rid in seqs:
            ref = want[rid][places[rid]]
            err = (got[rid] - ref).abs().max() / ref.abs().max()
            assert err < 2e-4, (rid, float(err))
        assert runner.portion_graphs.buckets and (runner.graphs.buckets or steps[0]["step"] == "portions"), \
            "nothing was replayed"
        # the recorded lists are longer than any step's own
        some = next(iter(runner.portion_graphs.buckets.values()))
        assert some.ctx.work[WorkList(32)][0].numel() == some.sizes.decode_rows + -(-some.sizes.multi_tokens // 32) + 1


LATENT = {"architectures": ["ToyStateLM"], "vocab_size": 60, "hidden_size": 40, "inner": 64, "latent": 12,
          "layers": ["latent", "attention", "latent"], "order": [0, 1, 2], "decay": 0.5,
          "toy_norm": True, "toy_ffn": True, "heads": 2, "kv_heads": 2, "head_dim": 16,
          "initializer_range": 0.3}


def latent_plain(model, ids):
    """Whole-sequence logits of the LATENT toy model, no cache, formulas spelt out here."""
    ids = torch.as_tensor(ids)
    S = len(ids)
    h, residual = model.embedding.weight.float().cpu()[ids], None
    for call in model.schedule:
        b = model.blocks[call.block]
        s = h if residual is None else h + residual
        h, residual = s - s.mean(-1, keepdim=True), s
        m = b.mixer
        if hasattr(m, "latent"):
            c = h @ m.wc.float().cpu().T
            q = h @ m.wq.float().cpu().T
            scores = (q @ c.T) / m.latent ** 0.5
            scores = scores.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), diagonal=1), float("-inf"))
            h = (torch.softmax(scores, dim=-1) @ c) @ m.wo.float().cpu().T
        else:
            qkv = h @ m.qkv.float().cpu().T
            q = qkv[:, :m.q_size].view(S, m.num_heads, m.head_dim)
            k = qkv[:, m.q_size:m.q_size + m.kv_size].view(S, m.num_kv_heads, m.head_dim)
            v = qkv[:, m.q_size + m.kv_size:].view(S, m.num_kv_heads, m.head_dim)
            cos, sin = plain_llama.rope_cos_sin(m.position.inv_freq_host, torch.arange(S))
            o = plain_llama.causal_attention(plain_llama.apply_rope(q, cos, sin),
                                             plain_llama.apply_rope(k, cos, sin), v, m.scale)
            h = o.reshape(S, -1) @ m.o.float().cpu().T
        s = h + residual
        h, residual = s - s.mean(-1, keepdim=True), s
        ff = b.feed_forward
        h = torch.relu(h @ ff.w1.float().cpu().T) @ ff.w2.float().cpu().T
    s = h + residual
    return (s - s.mean(-1, keepdim=True)) @ model.head.weight.float().cpu().T


def test_toy_mixer_with_one_paged_tensor_a_token(gpu_device):
    """A mixer defined here whose paged memory is a single tensor a token (no keys and values)
    is given pages, a block table and slots like attention: its cache spec names the tensor,
    the manager forms a group of its own for its two layers beside the attention layer's, and
    all cuttings (with so few pages that they are used again) agree with the plain result."""
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_random_weights
    model = build_model(copy.deepcopy(LATENT))
    load_random_weights(model, 11, torch.float32, gpu_device)
    g = torch.Generator().manual_seed(2)
    seqs = {f"r{i}": torch.randint(0, 60, (n,), generator=g).tolist() for i, n in enumerate([61, 38, 90, 47, 70])}
    want = {rid: latent_plain(model, t) for rid, t in seqs.items()}
    for steps in (cuttings.whole(seqs), cuttings.tail_decode(seqs, 32), cuttings.portions(seqs),
                  cuttings.mixed(seqs, seed=7)):
        pages = cuttings.max_live_tokens(steps, round_to=8) // 8
        assert pages < sum(-(-len(t) // 8) for t in seqs.values()) or len(steps) == len(seqs)
        runner = ModelRunner(model, page_size=8, num_pages=pages, max_num_seqs=4)
        specs = [grp.spec for grp in runner.manager.paged]
        assert [tuple(t.name for t in sp.tensors) for sp in specs] == [("latent",), ("k", "v")]
        assert [len(grp.layers) for grp in runner.manager.paged] == [2, 1]
        assert runner.storage.paged_pools[0]["latent"].shape == (2, pages, 8, 12)
        got = replay(runner, steps, seqs)
        for rid in seqs:
            err = (got[rid] - want[rid]).abs().max() / float(want[rid].abs().max())
            assert err < 2e-4, (rid, float(err))
        assert all(grp.pool.num_free == pages for grp in runner.manager.paged)


def test_parts_that_wait_for_the_device_are_never_recorded(gpu_device):
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_random_weights
    model = build_model(copy.deepcopy(HYBRID))
    assert not model.graph_capturable()
    load_random_weights(model, 9, torch.float32, gpu_device)
    runner = ModelRunner(model, page_size=8, num_pages=8, max_num_seqs=2, max_model_len=32, use_graphs=True)
    assert runner.graphs is None and runner.portion_graphs is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_rmsnorm_part_takes_any_width(gpu_device, dtype):
    """Rows wider than the kernel's LDS copy (15,000 elements) go through its two-pass form;
    a width is never refused after the weights have been loaded."""
    from pytriton_llama_amd.parts import build_part
    for H in (16384, 20004, 15001):
        n = build_part("norm", "rmsnorm", size=H, eps=1e-5)
        g = torch.Generator().manual_seed(H)
        w = 1 + 0.1 * torch.randn(H, generator=g)
        n.load({"weight": w}, dtype, gpu_device)
        x = torch.randn(3, H, generator=g).to(dtype)
        r = torch.randn(3, H, generator=g).to(dtype)
        rc = r.clone().cuda()
        y, res = n.forward(x.cuda(), rc)
        wy, wr = plain_llama.add_rms_norm(x.float(), r.float(), w, 1e-5)
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        torch.testing.assert_close(y.float().cpu(), wy, atol=tol, rtol=tol)
        torch.testing.assert_close(res.float().cpu(), wr.to(dtype).float(), atol=0, rtol=0)
        y0, _ = n.forward(x.cuda(), None)
        torch.testing.assert_close(y0.float().cpu(), plain_llama.rms_norm(x.float(), w, 1e-5), atol=tol, rtol=tol)
