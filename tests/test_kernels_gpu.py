"""Each HIP kernel alone against a plain float32 torch formula of the same
operation, at sizes other than the engine tests use."""
import math

import pytest
import torch

import plain_llama

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.bfloat16]
IDS = ["fp32", "bf16"]


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


@pytest.fixture(scope="module")
def ops(gpu_device):
    from pytriton_llama_amd import ops
    return ops


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_embedding(ops, dtype):
    table = torch.randn(301, 72, device="cuda").to(dtype)
    ids = torch.tensor([0, 300, 5, 5, 17], dtype=torch.int32, device="cuda")
    assert torch.equal(ops.embedding(table, ids), table[ids.long()])


def test_stage_step(ops):
    """The tables of a replayed step go from pinned host memory to the device buffer by a
    kernel; tokens that are still on the device take their places among them."""
    host = torch.arange(1000, 1000 + 777, dtype=torch.int32).pin_memory()
    dev = torch.zeros(777, dtype=torch.int32, device="cuda")
    ops.stage_step(dev, host)
    assert torch.equal(dev.cpu(), host)
    tokens = torch.tensor([7, 8, 9, 10], dtype=torch.int32, device="cuda")
    host[:] = torch.arange(777, dtype=torch.int32)
    ops.stage_step(dev, host, tokens, 300, 3)
    want = host.clone()
    want[300:303] = torch.tensor([7, 8, 9], dtype=torch.int32)
    assert torch.equal(dev.cpu(), want)
    with pytest.raises(ops.KernelError):
        ops.stage_step(dev, torch.zeros(777, dtype=torch.int32))          # not pinned
    with pytest.raises(ops.KernelError):
        ops.stage_step(dev, host, tokens, 775, 4)                         # past the end


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("shape", [(5, 72), (3, 2048), (2, 5000), (1, 16),
                                   (513, 328), (515, 2048), (600, 3072), (517, 4096)])
def test_add_rmsnorm(ops, dtype, shape):
    torch.manual_seed(0)
    x = torch.randn(shape, device="cuda").to(dtype)
    r = torch.randn(shape, device="cuda").to(dtype)
    w = (1 + 0.1 * torch.randn(shape[1], device="cuda")).float()
    eps = 1e-3
    want_y, want_r = plain_llama.add_rms_norm(x.float().cpu(), r.float().cpu(), w.cpu(), eps)
    res = r.clone()
    y = ops.add_rmsnorm(x, res, w, eps)
    torch.testing.assert_close(y.float().cpu(), want_y, **tol(dtype))
    torch.testing.assert_close(res.float().cpu(), want_r.to(dtype).float(), atol=0, rtol=0)
    # without a residual: the input stays what it is
    x2 = x.clone()
    y2 = ops.add_rmsnorm(x2, None, w, eps)
    torch.testing.assert_close(y2.float().cpu(), plain_llama.rms_norm(x.float().cpu(), w.cpu(), eps),
                               **tol(dtype))
    assert torch.equal(x2, x)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_silu_mul(ops, dtype):
    torch.manual_seed(1)
    gu = (3 * torch.randn(7, 2 * 200, device="cuda")).to(dtype)
    want = plain_llama.silu(gu[:, :200].float()) * gu[:, 200:].float()
    torch.testing.assert_close(ops.silu_mul(gu).float(), want, **tol(dtype))
    z = torch.zeros(1, 8, device="cuda", dtype=dtype)
    assert torch.all(ops.silu_mul(z) == 0)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("mnk", [(1, 300, 72), (7, 65, 130), (130, 257, 96), (64, 64, 16), (3, 1000, 2050)])
def test_gemm_nt(ops, dtype, mnk):
    M, N, K = mnk
    torch.manual_seed(2)
    x = torch.randn(M, K, device="cuda").to(dtype)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(dtype)
    want = (x.double() @ w.double().T).float()
    y = ops.gemm_nt(x, w)
    torch.testing.assert_close(y.float(), want, **tol(dtype))
    if dtype == torch.bfloat16:
        y32 = ops.gemm_nt(x, w, torch.float32)
        torch.testing.assert_close(y32, want, atol=1e-4, rtol=1e-4)
    # strided rows of x (a slice of a wider buffer)
    wide = torch.randn(M, K + 24, device="cuda").to(dtype)
    ys = ops.gemm_nt(wide[:, 8:8 + K], w)
    torch.testing.assert_close(ys.float(), (wide[:, 8:8 + K].double() @ w.double().T).float(),
                               **tol(dtype))


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["to_bf16", "to_fp32"])
@pytest.mark.parametrize("mnk", [(1, 300, 72), (7, 65, 136), (16, 3072, 2048), (17, 100, 200),
                                 (33, 16, 8192), (64, 1000, 64), (8, 2048, 8192), (5, 130, 2056),
                                 # a W wide enough for the streaming form: tiles past the end, K with a
                                 # partial last batch, one row and sixteen
                                 (1, 16384, 256), (8, 20003, 328), (16, 17000, 2048), (3, 40001, 72),
                                 # every way of packing the loads of x: 1, 2, 4, 8 rows a block, and none
                                 (2, 520, 264), (4, 136, 1032), (6, 264, 520), (9, 72, 296), (2, 4112, 2048)])
def test_gemm_skinny(ops, out_dtype, mnk):
    M, N, K = mnk
    torch.manual_seed(7)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    want = (x.double() @ w.double().T).float()
    y = ops.gemm_skinny(x, w, out_dtype)
    assert y.dtype == out_dtype
    t = dict(atol=1e-4, rtol=1e-4) if out_dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(y.float(), want, **t)
    # rows of x as a slice of a wider buffer
    wide = torch.randn(M, K + 24, device="cuda").to(torch.bfloat16)
    xs = wide[:, 8:8 + K]
    torch.testing.assert_close(ops.gemm_skinny(xs, w, out_dtype).float(),
                               (xs.double() @ w.double().T).float(), **t)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(torch.zeros(65, K, device="cuda", dtype=torch.bfloat16), w)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(x[:, :K - 4], w[:, :K - 4].contiguous())


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["to_bf16", "to_fp32"])
@pytest.mark.parametrize("mnk", [(1, 300, 72), (17, 100, 200), (64, 3072, 2048), (300, 130, 136),
                                 (512, 2048, 2048), (777, 1000, 328), (2048, 352, 176)])
def test_gemm_library(ops, out_dtype, mnk):
    """The library product called directly: against a float64 product, also for rows of x that
    are a slice of a wider buffer; the second call takes the kept plan, the third times the
    library's proposals for the shape and the fourth runs the fastest of them."""
    M, N, K = mnk
    torch.manual_seed(9)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    want = (x.double() @ w.double().T).float()
    t = dict(atol=1e-4, rtol=1e-4) if out_dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    for call in range(4):
        if call == 2:
            with ops.timed_library_products():
                y = ops.gemm_library(x, w, out_dtype)
        else:
            y = ops.gemm_library(x, w, out_dtype)
        assert y.dtype == out_dtype and y.shape == (M, N)
        torch.testing.assert_close(y.float(), want, **t)
    wide = torch.randn(M, K + 24, device="cuda").to(torch.bfloat16)
    xs = wide[:, 8:8 + K]
    torch.testing.assert_close(ops.gemm_library(xs, w, out_dtype).float(),
                               (xs.double() @ w.double().T).float(), **t)
    assert not ops.gemm_library_fits(wide[:, 1:1 + K], w)            # rows not 16-byte aligned
    assert not ops.gemm_library_fits(x.float(), w)
    with pytest.raises(ops.KernelError):
        ops.gemm_library(x.float(), w)


def test_gemm_library_runs_the_first_proposal_unless_asked_for_the_timed_one(ops):
    """A shape for which the timing keeps another proposal than the library's first on this
    GPU (64 rows, depth 8,192): calls outside ``timed_library_products`` give the same bits
    before and after the timing, the timed choice agrees with them within the rounding of
    bfloat16 (proposals add in different orders), and the choice can be asked for."""
    M, N, K = 64, 2048, 8192
    torch.manual_seed(11)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    before = ops.gemm_library(x, w)
    with ops.timed_library_products():
        timed = ops.gemm_library(x, w)
        again = ops.gemm_library(x, w)
    after = ops.gemm_library(x, w)
    assert torch.equal(before, after)
    assert torch.equal(timed, again)
    choice = ops.library_product_choice(M, N, K, K)
    assert choice >= 0
    assert ops.library_product_choice(M + 1, N, K, K) == -1               # never timed
    want = (x.double() @ w.double().T).float()
    ulp = 2.0 ** -7 * want.abs() + 1e-3 * float(want.abs().max())
    assert bool(((timed.float() - before.float()).abs() <= ulp).all())
    torch.testing.assert_close(timed.float(), want, atol=2e-2, rtol=2e-2)
    with ops.timed_library_products(False):                               # a switch passed on as off
        assert torch.equal(ops.gemm_library(x, w), before)


def test_gemm_library_times_nothing_while_a_graph_is_recorded(ops):
    """Timing switched on while a HIP graph is recorded: nothing waits for the stream there (the
    recording would fail), every replay gives the product, and the call after the recording,
    which does time the proposals, gives it too."""
    M, N, K = 48, 264, 520
    torch.manual_seed(10)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    want = (x.double() @ w.double().T).float()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.gemm_library(x, w)                                   # plan, handle and workspace
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), ops.timed_library_products():
        ys = [ops.gemm_library(x, w) for _ in range(3)]
    for _ in range(3):
        for y in ys:
            y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for y in ys:
            torch.testing.assert_close(y.float(), want, atol=2e-2, rtol=2e-2)
    with ops.timed_library_products():
        torch.testing.assert_close(ops.gemm_library(x, w).float(), want, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(ops.gemm_library(x, w).float(), want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("mik", [(1, 176, 64), (8, 8192, 2048), (16, 320, 136), (5, 48, 2056)])
def test_gate_up_silu(ops, mik):
    M, I, K = mik
    torch.manual_seed(8)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(2 * I, K, device="cuda") / math.sqrt(K) * 2).to(torch.bfloat16)
    got = ops.gate_up_silu(x, w)
    want = ops.silu_mul(ops.gemm_nt(x, w))              # the unfused kernels
    torch.testing.assert_close(got.float(), want.float(), atol=2e-2, rtol=2e-2)
    gu = (x.double() @ w.double().T).float()
    plain = plain_llama.silu(gu[:, :I]) * gu[:, I:]
    torch.testing.assert_close(got.float(), plain, atol=3e-2, rtol=3e-2)
    with pytest.raises(ops.KernelError):
        ops.gate_up_silu(torch.zeros(17, K, device="cuda", dtype=torch.bfloat16), w)


@pytest.mark.parametrize("dims", [(4, 2, 64, 16, 72), (3, 1, 32, 4, 128), (8, 8, 128, 16, 2048), (6, 3, 96, 5, 200)])
def test_qkv_rope_store(ops, dims):
    Hq, Hkv, D, P, K = dims
    M = 7
    torch.manual_seed(9)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    positions = torch.tensor([0, 1, 5, 77, 1000, 4095, 100000], dtype=torch.int32, device="cuda")
    inv_freq = plain_llama.rope_inv_freq_default(500000.0, D).cuda()
    pages = 5
    slots = torch.randperm(pages * P)[:M].to(torch.int32).cuda()
    slots[3] = -1                                           # this row's keys are not stored
    kc = torch.zeros(pages, Hkv, P, D, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    q = ops.qkv_rope_store(x, w, positions, inv_freq, slots, kc, vc, Hq, Hkv, D, P)
    # the unfused kernels on the same inputs
    qkv = ops.gemm_nt(x, w)
    q2 = qkv[:, :Hq * D].view(M, Hq, D)
    k2 = qkv[:, Hq * D:(Hq + Hkv) * D].view(M, Hkv, D)
    v2 = qkv[:, (Hq + Hkv) * D:].view(M, Hkv, D)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ops.rope_store(q2, k2, v2, positions, inv_freq, slots, kc2, vc2, P)
    torch.testing.assert_close(q.float(), q2.float(), atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(kc.float(), kc2.float(), atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(vc.float(), vc2.float(), atol=2e-2, rtol=2e-2)
    assert torch.all(kc.view(pages, Hkv, P, D)[:, :, :, :].sum() != 0)
    # and the plain formulas
    full = (x.double() @ w.double().T).float().cpu()
    cos, sin = plain_llama.rope_cos_sin(inv_freq.cpu(), positions.cpu())
    want_q = plain_llama.apply_rope(full[:, :Hq * D].view(M, Hq, D), cos, sin)
    torch.testing.assert_close(q.float().cpu(), want_q, atol=3e-2, rtol=3e-2)
    # without rotation and without a store
    q3 = ops.qkv_rope_store(x, w, positions, None, None, None, None, Hq, Hkv, D, P)
    torch.testing.assert_close(q3.float().cpu(), full[:, :Hq * D].view(M, Hq, D), atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("mnk", [(1, 64, 176), (8, 2048, 2048), (16, 136, 320), (5, 4096, 72), (3, 2056, 48)])
def test_gemm_skinny_add_norm_and_row_scale(ops, mnk):
    """Product + residual sum + norm weight in one kernel, the rsqrt factor left as partial sums:
    the residual it leaves, and its output once the factor is applied, are those of the product
    followed by add_rmsnorm, and of the plain formulas."""
    M, N, K = mnk
    torch.manual_seed(12)
    eps = 1e-5
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    res = torch.randn(M, N, device="cuda").to(torch.bfloat16)
    nw = (1.0 + 0.2 * torch.randn(N, device="cuda")).float()
    res_fused = res.clone()
    y, scale = ops.gemm_skinny_add_norm(x, w, res_fused, nw, eps)
    assert scale.partials.shape[0] == M and scale.size == N
    got = ops.row_scale(y, scale)
    # the separate kernels
    res_sep = res.clone()
    want = ops.add_rmsnorm(ops.gemm_skinny(x, w), res_sep, nw, eps)
    assert torch.equal(res_fused, res_sep)                       # same roundings, same sums
    torch.testing.assert_close(got.float(), want.float(), atol=3e-2, rtol=2e-2)
    # the sums of squares against the residual itself
    ss = scale.partials.sum(dim=1)
    torch.testing.assert_close(ss, (res_fused.float() ** 2).sum(dim=1), rtol=2e-2, atol=1e-3)
    # the plain formulas
    h = (x.double() @ w.double().T).float().cpu() + res.float().cpu()
    plain, _ = plain_llama.add_rms_norm(h, None, nw.cpu(), eps)
    torch.testing.assert_close(got.float().cpu(), plain, atol=5e-2, rtol=3e-2)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny_add_norm(torch.zeros(17, K, device="cuda", dtype=torch.bfloat16), w,
                                 torch.zeros(17, N, device="cuda", dtype=torch.bfloat16), nw, eps)
    with pytest.raises(ops.KernelError):
        ops.row_scale(y, ops.RowScale(scale.partials, N + 8, eps))


def test_fused_products_apply_a_row_scale(ops):
    """gate_up_silu and qkv_rope_store with rows that still lack their factor give what they
    give for the rows with the factor applied."""
    torch.manual_seed(13)
    M, H, I, Hq, Hkv, D, P = 6, 328, 176, 4, 2, 32, 8
    eps = 1e-6
    v = torch.randn(M, H, device="cuda").to(torch.bfloat16)
    partials = torch.rand(M, 41, device="cuda") * 30                 # any positive sums do
    scale = ops.RowScale(partials, H, eps)
    f = torch.rsqrt(partials.sum(dim=1) / H + eps)
    xs = (v.float() * f[:, None])                                     # the finished rows, float32
    wg = (torch.randn(2 * I, H, device="cuda") / math.sqrt(H)).to(torch.bfloat16)
    got = ops.gate_up_silu(v, wg, scale)
    gu = xs.double() @ wg.double().T
    want = (plain_llama.silu(gu[:, :I]) * gu[:, I:]).float()
    torch.testing.assert_close(got.float(), want, atol=3e-2, rtol=3e-2)
    wq = (torch.randn((Hq + 2 * Hkv) * D, H, device="cuda") / math.sqrt(H)).to(torch.bfloat16)
    positions = torch.tensor([0, 3, 9, 100, 2000, 7], dtype=torch.int32, device="cuda")
    inv_freq = plain_llama.rope_inv_freq_default(10000.0, D).cuda()
    slots = torch.arange(M, dtype=torch.int32, device="cuda")
    kc = torch.zeros(2, Hkv, P, D, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    q = ops.qkv_rope_store(v, wq, positions, inv_freq, slots, kc, vc, Hq, Hkv, D, P, scale)
    full = (xs.double() @ wq.double().T).float().cpu()
    cos, sin = plain_llama.rope_cos_sin(inv_freq.cpu(), positions.cpu())
    want_q = plain_llama.apply_rope(full[:, :Hq * D].view(M, Hq, D), cos, sin)
    torch.testing.assert_close(q.float().cpu(), want_q, atol=3e-2, rtol=3e-2)
    want_k = plain_llama.apply_rope(full[:, Hq * D:(Hq + Hkv) * D].view(M, Hkv, D), cos, sin)
    got_k = kc.view(2 * 1, Hkv, P, D).permute(0, 2, 1, 3).reshape(2 * P, Hkv, D)[:M]
    torch.testing.assert_close(got_k.float().cpu(), want_k, atol=3e-2, rtol=3e-2)
    want_v = full[:, (Hq + Hkv) * D:].view(M, Hkv, D)
    got_v = vc.permute(0, 2, 1, 3).reshape(2 * P, Hkv, D)[:M]
    torch.testing.assert_close(got_v.float().cpu(), want_v, atol=3e-2, rtol=3e-2)
    # the factor really is used: without it the result differs
    q_plain = ops.qkv_rope_store(v, wq, positions, inv_freq, None, None, None, Hq, Hkv, D, P)
    assert (q_plain.float() - q.float()).abs().max() > 0.1


def test_qkv_rope_store_with_a_large_row_scale(ops):
    """Rows whose pending factor is large (a residual stream that is nearly zero: one partial
    sum of 1e-3 .. 30 over 6,184 columns gives factors of 14 to 930) make q and k values of
    some hundreds. The kernel rounds the scaled projection to bfloat16 before it rotates, as
    the separate kernels store it between product and rotation, so an element of the result
    carries the rounding of both elements of its pair: the bound is half a bfloat16 ulp (at most
    2^-8 of the value) of x1 and of x2 from before the rotation plus half an ulp of the result,
    not a share of the element itself, which the rotation can make small. Every element must
    lie within that bound."""
    torch.manual_seed(249)
    M, K, D, Hq, Hkv, P = 13, 6184, 128, 7, 1, 5
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    partials = torch.logspace(-3, math.log10(30.0), M, device="cuda").view(M, 1).contiguous()
    scale = ops.RowScale(partials, K, 1e-6)
    f = torch.rsqrt(partials.sum(dim=1).double() / K + 1e-6)
    assert float(f.max()) > 900 and float(f.min()) < 20
    positions = torch.tensor([5000, 0, 0, 5000, 77, 77, 0, 77, 5000, 1, 77, 1, 100000],
                             dtype=torch.int32, device="cuda")
    inv_freq = plain_llama.rope_inv_freq_default(500000.0, D).cuda()
    npage = -(-M // P) + 1
    slots = torch.randperm(npage * P)[:M].to(torch.int32).cuda()
    kc = torch.zeros(npage, Hkv, P, D, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    q = ops.qkv_rope_store(x, w, positions, inv_freq, slots, kc, vc, Hq, Hkv, D, P, scale)
    full = ((x.double() * f[:, None]) @ w.double().T).cpu()
    cos, sin = plain_llama.rope_cos_sin(inv_freq.cpu(), positions.cpu())

    def check(got, projected, what, rotated=True):
        want = plain_llama.apply_rope(projected, cos.double(), sin.double()) if rotated else projected
        a = projected.abs()
        pair = a + torch.cat((a[..., D // 2:], a[..., :D // 2]), dim=-1) if rotated else a
        bound = 2.0 ** -8 * (pair + want.abs() if rotated else pair) + 1e-5 * a.amax(dim=(-2, -1), keepdim=True)
        over = (got.double() - want).abs() - bound
        assert float(over.max()) <= 0, f"{what}: {float(over.max()):.3g} beyond the rounding bound"
        assert float(want.abs().max()) > 300          # the case is about large values

    check(q.cpu(), full[:, :Hq * D].view(M, Hq, D), "q")
    rows = slots.long().cpu()
    got_k = kc.permute(0, 2, 1, 3).reshape(npage * P, Hkv, D).cpu()[rows]
    got_v = vc.permute(0, 2, 1, 3).reshape(npage * P, Hkv, D).cpu()[rows]
    check(got_k, full[:, Hq * D:(Hq + Hkv) * D].view(M, Hkv, D), "k")
    check(got_v, full[:, (Hq + Hkv) * D:].view(M, Hkv, D), "v", rotated=False)


@pytest.mark.parametrize("dims", [(8, 2048, 2048, 8192, 32, 8, 64, 16), (1, 2048, 2048, 8192, 32, 8, 64, 16),
                                  (16, 160, 224, 224, 3, 1, 32, 8), (5, 3072, 3072, 1024, 24, 8, 128, 16),
                                  (3, 64, 64, 160, 8, 2, 32, 4), (13, 4128, 96, 64, 2, 2, 96, 16),
                                  (7, 1000, 96, 48, 5, 5, 32, 2)])
def test_decode_kernels_read_the_blocked_copy_of_a_weight(ops, dims):
    """The decode kernels with the second, blocked copy of their weights (tiles of 16 rows x 32
    columns, each in one piece) give bit for bit what they give with the row-major matrix: the
    same sums in the same order, only fetched from other addresses. Widths that are no multiple
    of 16 rows (padding), 8- and 16-row tiles, one to sixteen rows of x."""
    M, H, Kin, I, Hq, Hkv, D, P = dims
    g = torch.Generator().manual_seed(M * 7 + H)
    rnd = lambda *s: torch.randn(*s, generator=g)
    dev = "cuda"
    x = rnd(M, Kin).to(torch.bfloat16).to(dev)
    wo = (rnd(H, Kin) / math.sqrt(Kin)).to(torch.bfloat16).to(dev)
    wgu = (rnd(2 * I, H) / math.sqrt(H)).to(torch.bfloat16).to(dev)
    wq = (rnd((Hq + 2 * Hkv) * D, H) / math.sqrt(H)).to(torch.bfloat16).to(dev)
    nw = (1 + 0.1 * rnd(H)).to(dev)
    res = rnd(M, H).to(torch.bfloat16).to(dev)
    bo, bgu, bq = ops.blocked_weight(wo), ops.blocked_weight(wgu), ops.blocked_weight(wq)
    assert bo.shape == (-(-H // 16), Kin // 32, 16, 32)
    # the layout itself: tile t, column block b holds rows 16 t .. 16 t + 15, columns 32 b .. 32 b + 31
    t, b = bo.shape[0] - 1, bo.shape[1] - 1
    rows = wo[16 * t:16 * t + 16, 32 * b:32 * b + 32]
    assert torch.equal(bo[t, b, :rows.shape[0]], rows) and bool((bo[t, b, rows.shape[0]:] == 0).all())
    for out_dtype in (torch.bfloat16, torch.float32):
        assert torch.equal(ops.gemm_skinny(x, wo, out_dtype), ops.gemm_skinny(x, wo, out_dtype, blocked=bo))
    r1, r2 = res.clone(), res.clone()
    y1, s1 = ops.gemm_skinny_add_norm(x, wo, r1, nw, 1e-5)
    y2, s2 = ops.gemm_skinny_add_norm(x, wo, r2, nw, 1e-5, blocked=bo)
    assert torch.equal(y1, y2) and torch.equal(r1, r2) and torch.equal(s1.partials, s2.partials)
    assert torch.equal(ops.gate_up_silu(y1, wgu, s1), ops.gate_up_silu(y1, wgu, s1, blocked=bgu))
    assert torch.equal(ops.gate_up_silu(y1, wgu), ops.gate_up_silu(y1, wgu, blocked=bgu))
    positions = torch.randint(0, 3000, (M,), generator=g).to(torch.int32).to(dev)
    inv_freq = plain_llama.rope_inv_freq_default(10000.0, D).to(dev)
    slots = (torch.randperm(2 * P, generator=g)[:M]).to(torch.int32).to(dev) if M <= 2 * P else None
    outs = []
    for blocked in (None, bq):
        kc = torch.zeros(2, Hkv, P, D, device=dev, dtype=torch.bfloat16)
        vc = torch.zeros_like(kc)
        q = ops.qkv_rope_store(y1, wq, positions, inv_freq, slots, kc if slots is not None else None,
                               vc if slots is not None else None, Hq, Hkv, D, P, s1, blocked=blocked)
        outs.append((q, kc, vc))
    for a, b2 in zip(*outs):
        assert torch.equal(a, b2)
    # a copy that belongs to another matrix is refused, more rows than the kernels take fall back
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(x, wo, blocked=torch.zeros((bo.shape[0] + 1, *bo.shape[1:]), dtype=torch.bfloat16, device=dev))
    x20 = rnd(20, Kin).to(torch.bfloat16).to(dev)
    assert torch.equal(ops.gemm_skinny(x20, wo), ops.gemm_skinny(x20, wo, blocked=bo))
    assert ops.blocked_weight(rnd(8, 40).to(torch.bfloat16).to(dev)) is None       # K no multiple of 32


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["to_bf16", "to_fp32"])
@pytest.mark.parametrize("mnk", [(17, 64, 32), (24, 1000, 96), (33, 2048, 2080), (64, 130, 4096), (100, 3000, 160),
                                 (128, 16400, 512), (5, 70, 64), (9, 200, 96), (16, 2048, 2048), (12, 70000, 64),
                                 (40, 66000, 96), (48, 3072, 2048), (37, 100, 4128)])
def test_gemm_rows(ops, out_dtype, mnk):
    """The product for some tens of rows (x through LDS, the blocked copy of W streamed): widths
    that are no multiple of a workgroup's 64 rows or of a tile's 16, depths that are no multiple
    of a chunk, one to eight tiles of x, one and two tiles of W a wave (two from 1,024 workgroups
    on), against a float64 product; and as partial sums over slices of K, whose sum is the
    product."""
    M, N, K = mnk
    torch.manual_seed(21)
    wide = torch.randn(M, K + 8, device="cuda").to(torch.bfloat16)
    x = wide[:, :K]                                               # rows of a wider buffer
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    b = ops.blocked_weight(w)
    want = (x.double() @ w.double().T).float()
    t = dict(atol=1e-4, rtol=1e-4) if out_dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    y = ops.gemm_rows(x, w, b, out_dtype) if M >= ops.ROWS_MIN else None
    if M >= ops.ROWS_MIN:
        assert y.dtype == out_dtype and y.shape == (M, N)
        torch.testing.assert_close(y.float(), want, **t)
        for splits in (2, 3, 8):
            parts = ops.gemm_rows(x, w, b, torch.float32, splits=splits)
            assert parts.shape == (splits, M, N)
            torch.testing.assert_close(parts.sum(dim=0), want, atol=1e-4, rtol=1e-4)
        with pytest.raises(ops.KernelError):
            ops.gemm_rows(x, w, b, torch.bfloat16, splits=2)      # partial sums are float32
        with pytest.raises(ops.KernelError):
            ops.gemm_rows(x, w, torch.zeros_like(b)[1:], out_dtype)   # a copy of another matrix
    else:
        with pytest.raises(ops.KernelError):
            ops.gemm_rows(x, w, b, out_dtype)                      # fewer rows than ROWS_MIN: the other kernels


@pytest.mark.parametrize("mnk", [(17, 64, 96), (40, 2048, 2048), (64, 2056, 320), (128, 4096, 8192), (9, 2048, 2048),
                                 (16, 264, 96), (48, 2048, 8192), (35, 72, 64)])
def test_gemm_rows_add_rmsnorm(ops, mnk):
    """Partial sums over slices of K, then one kernel that adds them up, adds the residual and
    normalises whole rows: the residual it leaves and its output are those of the product
    followed by add_rmsnorm, and of the plain formulas."""
    M, N, K = mnk
    torch.manual_seed(22)
    eps = 1e-5
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    b = ops.blocked_weight(w)
    res = torch.randn(M, N, device="cuda").to(torch.bfloat16)
    nw = (1.0 + 0.2 * torch.randn(N, device="cuda")).float()
    r1, r2 = res.clone(), res.clone()
    partials = ops.gemm_rows(x, w, b, torch.float32, splits=ops.gemm_rows_splits(M, N, K))
    got = ops.sum_add_rmsnorm(partials, r1, nw, eps)
    want = ops.add_rmsnorm(ops.gemm_nt(x, w), r2, nw, eps)               # the separate kernels
    torch.testing.assert_close(r1.float(), r2.float(), atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(got.float(), want.float(), atol=3e-2, rtol=2e-2)
    h = (x.double() @ w.double().T).float().cpu() + res.float().cpu()
    plain, plain_res = plain_llama.add_rms_norm(h, None, nw.cpu(), eps)
    torch.testing.assert_close(got.float().cpu(), plain, atol=5e-2, rtol=3e-2)
    torch.testing.assert_close(r1.float().cpu(), plain_res, atol=3e-2, rtol=2e-2)
    # a float32 product of one piece is a partial sum of one slice
    r3 = res.clone()
    one = ops.sum_add_rmsnorm(ops.gemm_rows(x, w, b, torch.float32), r3, nw, eps)
    torch.testing.assert_close(one.float(), got.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("mik", [(17, 64, 64), (33, 8192, 2048), (64, 352, 160), (128, 1024, 4096), (9, 64, 64),
                                 (16, 8192, 2048), (13, 352, 160), (44, 2048, 512), (48, 96, 64)])
def test_gate_up_silu_for_tens_of_rows(ops, mik):
    M, I, K = mik
    torch.manual_seed(23)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(2 * I, K, device="cuda") / math.sqrt(K) * 2).to(torch.bfloat16)
    got = ops.gate_up_silu(x, w, None, ops.blocked_weight(w))
    gu = (x.double() @ w.double().T).float()
    plain = plain_llama.silu(gu[:, :I]) * gu[:, I:]
    torch.testing.assert_close(got.float(), plain, atol=3e-2, rtol=3e-2)
    if M > 16:
        with pytest.raises(ops.KernelError):
            ops.gate_up_silu(x, w)                                       # no blocked copy: not this many rows
    else:                                                                # the kernel for at most 16 rows
        torch.testing.assert_close(ops.gate_up_silu(x, w).float(), plain, atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("dims", [(4, 2, 64, 16, 96, 20), (3, 1, 32, 4, 128, 33), (32, 8, 128, 16, 4096, 64),
                                  (6, 3, 96, 8, 224, 128), (32, 8, 64, 16, 2048, 9), (5, 5, 32, 2, 160, 16),
                                  (8, 2, 64, 16, 512, 48), (3, 3, 96, 4, 96, 37)])
def test_qkv_rope_store_for_tens_of_rows(ops, dims):
    """Partial sums of the projection, then one kernel that adds them up, rotates q and k and
    writes k and v into their pages, against the plain formulas; rows whose slot is -1 store
    nothing."""
    Hq, Hkv, D, P, K, M = dims
    torch.manual_seed(24)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    positions = torch.randint(0, 100000, (M,), device="cuda").to(torch.int32)
    positions[0] = 0
    inv_freq = plain_llama.rope_inv_freq_default(500000.0, D).cuda()
    pages = -(-M // P) + 2
    slots = torch.randperm(pages * P, device="cuda")[:M].to(torch.int32)
    slots[3] = -1
    kc = torch.zeros(pages, Hkv, P, D, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    q = ops.qkv_rope_store(x, w, positions, inv_freq, slots, kc, vc, Hq, Hkv, D, P, None, ops.blocked_weight(w))
    full = (x.double() @ w.double().T).float().cpu()
    cos, sin = plain_llama.rope_cos_sin(inv_freq.cpu(), positions.cpu())
    want_q = plain_llama.apply_rope(full[:, :Hq * D].view(M, Hq, D), cos, sin)
    torch.testing.assert_close(q.float().cpu(), want_q, atol=3e-2, rtol=3e-2)
    want_k = plain_llama.apply_rope(full[:, Hq * D:(Hq + Hkv) * D].view(M, Hkv, D), cos, sin)
    want_v = full[:, (Hq + Hkv) * D:].view(M, Hkv, D)
    flat_k = kc.permute(0, 2, 1, 3).reshape(pages * P, Hkv, D).float().cpu()
    flat_v = vc.permute(0, 2, 1, 3).reshape(pages * P, Hkv, D).float().cpu()
    stored = torch.zeros(pages * P, dtype=torch.bool)
    for m in range(M):
        sl = int(slots[m])
        if sl < 0:
            continue
        stored[sl] = True
        torch.testing.assert_close(flat_k[sl], want_k[m], atol=3e-2, rtol=3e-2)
        torch.testing.assert_close(flat_v[sl], want_v[m], atol=3e-2, rtol=3e-2)
    assert bool((flat_k[~stored] == 0).all()) and bool((flat_v[~stored] == 0).all())
    assert int(stored.sum()) == M - 1


def _rope_reference(x, positions, inv_freq):
    cos, sin = plain_llama.rope_cos_sin(inv_freq, positions)
    return plain_llama.apply_rope(x, cos, sin)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("dims", [(5, 2, 48, 4), (3, 1, 128, 16), (4, 4, 8, 2)])
def test_rope_store(ops, dtype, dims):
    Hq, Hkv, D, P = dims
    T = 9
    torch.manual_seed(3)
    width = (Hq + 2 * Hkv) * D
    qkv = torch.randn(T, width, device="cuda").to(dtype)
    orig = qkv.clone()
    q = qkv[:, :Hq * D].view(T, Hq, D)
    k = qkv[:, Hq * D:(Hq + Hkv) * D].view(T, Hkv, D)
    v = qkv[:, (Hq + Hkv) * D:].view(T, Hkv, D)
    positions = torch.tensor([0, 1, 2, 77, 1000, 4095, 8191, 100000, 5], dtype=torch.int32, device="cuda")
    inv_freq = plain_llama.rope_inv_freq_default(500000.0, D)
    pages = 7
    kc = torch.zeros(pages, Hkv, P, D, device="cuda", dtype=dtype)
    vc = torch.zeros_like(kc)
    slots = torch.randperm(pages * P)[:T].to(torch.int32).cuda()
    ops.rope_store(q, k, v, positions, inv_freq.cuda(), slots, kc, vc, P)
    o = orig.float().cpu()
    want_q = _rope_reference(o[:, :Hq * D].view(T, Hq, D), positions.cpu(), inv_freq)
    want_k = _rope_reference(o[:, Hq * D:(Hq + Hkv) * D].view(T, Hkv, D), positions.cpu(), inv_freq)
    torch.testing.assert_close(q.float().cpu(), want_q, **tol(dtype))
    # k in the projection buffer is untouched, the cache holds the rotated k and v
    assert torch.equal(k, orig[:, Hq * D:(Hq + Hkv) * D].view(T, Hkv, D))
    for t in range(T):
        page, off = int(slots[t]) // P, int(slots[t]) % P
        torch.testing.assert_close(kc[page, :, off].float().cpu(), want_k[t], **tol(dtype))
        assert torch.equal(vc[page, :, off], v[t])
    # untouched slots stay zero
    mask = torch.ones(pages * P, dtype=torch.bool)
    mask[slots.long().cpu()] = False
    assert torch.all(kc.permute(0, 2, 1, 3).reshape(pages * P, -1)[mask.cuda()] == 0)


def _paged_setup(seq_lens, q_lens, Hkv, D, P, dtype, seed, shuffle=True):
    """Random keys/values laid into shuffled pages; returns tensors and the dense copies."""
    g = torch.Generator().manual_seed(seed)
    n = len(seq_lens)
    pages_per = [-(-s // P) for s in seq_lens]
    total = sum(pages_per) + 3
    perm = torch.randperm(total, generator=g).tolist() if shuffle else list(range(total))
    kc = torch.randn(total, Hkv, P, D, generator=g).to(dtype)    # garbage everywhere first
    vc = torch.randn(total, Hkv, P, D, generator=g).to(dtype)
    maxp = max(pages_per)
    bt = torch.full((n, maxp), -1, dtype=torch.int32)
    dense_k, dense_v = [], []
    it = iter(perm)
    for i, s in enumerate(seq_lens):
        k = torch.randn(s, Hkv, D, generator=g).to(dtype)
        v = torch.randn(s, Hkv, D, generator=g).to(dtype)
        dense_k.append(k.float())
        dense_v.append(v.float())
        for j in range(pages_per[i]):
            pg = next(it)
            bt[i, j] = pg
            lo, hi = j * P, min(s, (j + 1) * P)
            kc[pg, :, :hi - lo] = k[lo:hi].transpose(0, 1)
            vc[pg, :, :hi - lo] = v[lo:hi].transpose(0, 1)
    return kc, vc, bt, dense_k, dense_v


def _attention_case(ops, dtype, seq_lens, q_lens, Hq, Hkv, D, P, window=0, seed=0, boost=None,
                    kernel="generic", splits=1, unroll=0, groups=0):
    kc, vc, bt, dk, dv = _paged_setup(seq_lens, q_lens, Hkv, D, P, dtype, seed)
    g = torch.Generator().manual_seed(seed + 100)
    T = sum(q_lens)
    q = torch.randn(T, Hq, D, generator=g).to(dtype)
    if boost is not None:
        boost(q, dk, kc, bt)
    q_start = [0]
    for ql in q_lens:
        q_start.append(q_start[-1] + ql)
    rows = {"mfma": 64, "mfma128": 128}.get(kernel, 16)
    work_seq, work_qoff = [], []
    for s, ql in enumerate(q_lens):
        for off in range(0, ql, rows):
            work_seq.append(s)
            work_qoff.append(off)
    dev = "cuda"
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    out = torch.zeros(T, Hq, D, dtype=dtype, device=dev)
    scale = 1.0 / math.sqrt(D)
    # q as the engine has it: a slice of a wider projection buffer
    wide = torch.zeros(T, Hq * D + 64, dtype=dtype, device=dev)
    wide[:, :Hq * D] = q.to(dev).view(T, Hq * D)
    qd = wide[:, :Hq * D].view(T, Hq, D)
    if kernel == "generic":
        ops.attention_generic(out, qd, kc.to(dev), vc.to(dev), i32(q_start), i32(seq_lens),
                              bt.to(dev), i32(work_seq), i32(work_qoff), scale, window)
    elif kernel in ("mfma", "mfma128"):
        ops.attention_prefill_mfma(out, qd, kc.to(dev), vc.to(dev), i32(q_start), i32(seq_lens),
                                   bt.to(dev), i32(work_seq), i32(work_qoff), scale, window, rows,
                                   groups)
    else:
        assert all(ql == 1 for ql in q_lens)
        ops.attention_decode(out, qd, kc.to(dev), vc.to(dev), i32(q_start), i32(seq_lens),
                             bt.to(dev), len(q_lens), scale, window, splits,
                             matrix_cores=(kernel == "decode_mfma"), unroll=unroll)
    # plain: full causal attention over the sequence, rows of the portion kept
    for i, (s, ql) in enumerate(zip(seq_lens, q_lens)):
        full_q = torch.zeros(s, Hq, D)
        full_q[s - ql:] = q[q_start[i]:q_start[i + 1]].float()
        want = plain_llama.causal_attention(full_q, dk[i], dv[i], scale,
                                            window if window else None)[s - ql:]
        got = out[q_start[i]:q_start[i + 1]].float().cpu()
        torch.testing.assert_close(got, want, **tol(dtype), msg=lambda m: f"sequence {i}: {m}")


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("case", [
    dict(seq_lens=[40], q_lens=[40], Hq=4, Hkv=4, D=64, P=16),            # whole prompt, MHA
    dict(seq_lens=[37, 5, 130], q_lens=[1, 1, 1], Hq=8, Hkv=2, D=48, P=4),  # decode, GQA
    dict(seq_lens=[100, 64, 33], q_lens=[30, 1, 33], Hq=6, Hkv=1, D=128, P=8),  # mixed, MQA
    dict(seq_lens=[70], q_lens=[19], Hq=2, Hkv=1, D=256, P=5),            # big heads, odd page size
    dict(seq_lens=[50, 21], q_lens=[17, 2], Hq=4, Hkv=2, D=8, P=3),       # tiny heads
])
def test_attention_generic(ops, dtype, case):
    _attention_case(ops, dtype, **case)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("splits", [1, 3, 8])
@pytest.mark.parametrize("case", [
    dict(seq_lens=[37, 5, 130, 1], Hq=8, Hkv=2, D=48, P=4),         # 3 lanes of 4 per key
    dict(seq_lens=[300, 64, 65], Hq=4, Hkv=4, D=64, P=16),          # MHA
    dict(seq_lens=[100, 257], Hq=16, Hkv=2, D=16, P=8),             # 8 heads a kv head: two groups
    dict(seq_lens=[90, 33], Hq=3, Hkv=1, D=128, P=16),              # 3 heads of a tile of 4
    dict(seq_lens=[70], Hq=2, Hkv=1, D=256, P=5),                   # widest head, odd page size
    dict(seq_lens=[50, 200], Hq=6, Hkv=3, D=80, P=16),              # 5 lanes of 8 per key
])
def test_attention_decode(ops, dtype, splits, case):
    _attention_case(ops, dtype, q_lens=[1] * len(case["seq_lens"]), kernel="decode", splits=splits,
                    **case)


@pytest.mark.parametrize("splits", [1, 2, 5])
@pytest.mark.parametrize("case", [
    dict(seq_lens=[300, 64, 65, 1], Hq=4, Hkv=4, D=64, P=16),
    dict(seq_lens=[100, 257], Hq=32, Hkv=2, D=32, P=8),             # 16 heads a kv head
    dict(seq_lens=[90, 33, 700], Hq=3, Hkv=1, D=128, P=16),
    dict(seq_lens=[70, 130], Hq=8, Hkv=2, D=96, P=4),
    dict(seq_lens=[500, 3, 129], Hq=4, Hkv=1, D=64, P=64),          # a page longer than a turn
])
@pytest.mark.parametrize("unroll", [1, 2])
def test_attention_decode_mfma(ops, splits, case, unroll):
    _attention_case(ops, torch.bfloat16, q_lens=[1] * len(case["seq_lens"]), kernel="decode_mfma",
                    splits=splits, unroll=unroll, **case)


def test_attention_decode_mfma_refuses_odd_page_size(ops):
    """A page size that is no power of two is for the general kernel; the fast one says so."""
    assert not ops.attention_decode_mfma_fits(torch.bfloat16, 8, 2, 96, 5)
    assert ops.attention_decode_mfma_fits(torch.bfloat16, 8, 2, 96, 4)
    with pytest.raises(ops.KernelError, match="power of two"):
        _attention_case(ops, torch.bfloat16, seq_lens=[70, 130], q_lens=[1, 1], Hq=8, Hkv=2, D=96,
                        P=5, kernel="decode_mfma")


def test_attention_decode_mfma_window(ops):
    _attention_case(ops, torch.bfloat16, seq_lens=[90, 40, 7], q_lens=[1, 1, 1], Hq=4, Hkv=2, D=32,
                    P=8, window=20, kernel="decode_mfma", splits=2)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_attention_decode_window(ops, dtype):
    _attention_case(ops, dtype, seq_lens=[90, 40, 7], q_lens=[1, 1, 1], Hq=4, Hkv=2, D=32, P=8,
                    window=20, kernel="decode", splits=2)


@pytest.mark.parametrize("case", [
    dict(seq_lens=[40], q_lens=[40], Hq=4, Hkv=4, D=64, P=16),
    dict(seq_lens=[200, 64, 33], q_lens=[130, 2, 33], Hq=6, Hkv=1, D=128, P=8),
    dict(seq_lens=[150], q_lens=[70], Hq=2, Hkv=1, D=32, P=32),
    dict(seq_lens=[129, 300], q_lens=[129, 65], Hq=4, Hkv=2, D=96, P=16),
    dict(seq_lens=[450], q_lens=[333], Hq=2, Hkv=1, D=64, P=128),      # a page longer than a tile
    dict(seq_lens=[1, 2, 64, 65], q_lens=[1, 2, 64, 65], Hq=2, Hkv=2, D=64, P=4),
])
@pytest.mark.parametrize("kernel", ["mfma", "mfma128"])
def test_attention_prefill_mfma(ops, case, kernel):
    _attention_case(ops, torch.bfloat16, kernel=kernel, **case)


@pytest.mark.parametrize("kernel", ["mfma", "mfma128"])
def test_attention_prefill_mfma_window(ops, kernel):
    _attention_case(ops, torch.bfloat16, seq_lens=[300, 90], q_lens=[150, 25], Hq=4, Hkv=2, D=64,
                    P=8, window=70, kernel=kernel)


def test_attention_prefill_mfma_refuses_odd_page_size(ops):
    """A page size that is no power of two is for the general kernel; the fast one says so."""
    assert not ops.attention_prefill_mfma_fits(torch.bfloat16, 1, 32, 5)
    assert ops.attention_prefill_mfma_fits(torch.bfloat16, 1, 32, 8)
    with pytest.raises(ops.KernelError, match="power of two"):
        _attention_case(ops, torch.bfloat16, seq_lens=[150], q_lens=[70], Hq=2, Hkv=1, D=32, P=5,
                        kernel="mfma")


@pytest.mark.parametrize("groups", [1, 2, 3, 5])
@pytest.mark.parametrize("kernel", ["mfma", "mfma128"])
def test_attention_prefill_mfma_workgroups_share_the_blocks(ops, kernel, groups):
    """Fewer workgroups a head than query blocks: each walks several blocks (of different
    sequences, with and without a prefix in the cache), forwards and backwards over the
    list, and reuses its LDS buffers from one block to the next."""
    _attention_case(ops, torch.bfloat16, seq_lens=[520, 90, 300], q_lens=[390, 90, 129], Hq=4, Hkv=2,
                    D=64, P=16, kernel=kernel, groups=groups)
    _attention_case(ops, torch.bfloat16, seq_lens=[333], q_lens=[333], Hq=2, Hkv=1, D=128, P=8,
                    window=100, kernel=kernel, groups=groups)


def test_attention_prefill_mfma_plan(ops):
    """128-row blocks once there are 1.25 t of them (t: workgroups a head can have resident);
    a workgroup a block up to 2 t blocks, t workgroups beyond; never more workgroups than blocks."""
    dev = torch.device("cuda", 0)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    t = max(1, 3 * cus // 32)
    plan = lambda n64, n128: ops.attention_prefill_mfma_plan(dev, 32, 64, n64, n128)
    assert plan(3, 2) == (64, 3)
    assert plan(2 * t, t) == (64, 2 * t)
    assert plan(2 * t + 2, t + 1) == (64, t)
    n128 = -(-5 * t // 4)
    assert plan(2 * n128, n128) == (128, n128)
    assert plan(2 * n128 - 2, n128 - 1)[0] == 64
    assert plan(8 * t, 4 * t) == (128, t)
    assert ops.attention_prefill_mfma_plan(dev, 4 * cus, 128, 1, 1) == (64, 1)
    # head sizes above 64: 128-row blocks from 0.5 t blocks on when a context has 4,096 keys
    t128 = max(1, 2 * cus // 32)
    wide = lambda n128, keys: ops.attention_prefill_mfma_plan(dev, 32, 128, 2 * n128, n128, keys)
    half = -(-t128 // 2)
    assert wide(half, 4096) == (128, half) and wide(half, 4095)[0] == 64 and wide(half, 0)[0] == 64
    if half > 1:
        assert wide(half - 1, 16384)[0] == 64
    assert plan(2 * half, half) == ops.attention_prefill_mfma_plan(dev, 32, 64, 2 * half, half, 16384)


def test_attention_prefill_mfma_long(ops):
    """Many key tiles, a prefix in the cache, rows that end inside a block."""
    _attention_case(ops, torch.bfloat16, seq_lens=[1100, 700], q_lens=[777, 300], Hq=4, Hkv=1, D=64,
                    P=16, kernel="mfma128")


def _hot_keys(dk, kc, bt, P, seq, places, value=2.0):
    """Key ``places[h]`` of kv head h of sequence ``seq`` becomes ``value`` in every element, in
    the pages and in the dense copy: a query of the same direction then reads that key alone."""
    D = kc.shape[-1]
    for h, pos in enumerate(places):
        kc[int(bt[seq, pos // P]), h, pos % P] = value
        dk[seq][pos, h] = torch.full((D,), value)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("keys", [8200, 16400])
def test_attention_decode_long_contexts(ops, D, keys):
    """Eight decoded rows over up to 8,200 and 16,400 keys with 32 heads on 8 kv heads, cut into
    the splits the attention part plans for such a step. In every group of four heads, two
    queries point at one key each (the first key, the last, both sides of a page's and of a
    split's edge, ...), so that a tile that is dropped or read twice changes the whole row, and
    two are random with scores spread over about three, so that the sums over all tiles count."""
    from types import SimpleNamespace

    from pytriton_llama_amd.parts.attention import PagedAttention
    Hq, Hkv, P = 32, 8, 16
    G = Hq // Hkv
    seq_lens = [keys, keys - 7, keys - 16, keys // 2 + 1, keys - 1, 4100, keys, keys - 33]
    n = len(seq_lens)
    part = PagedAttention(hidden_size=Hq * D, num_heads=Hq, num_kv_heads=Hkv, head_dim=D)
    splits = part.decode_splits(SimpleNamespace(ctx_lens=seq_lens), n, True, torch.device("cuda", 0))
    assert splits >= 4, "the case is meant to run with several splits"
    kc, vc, bt, dk, dv = _paged_setup(seq_lens, [1] * n, Hkv, D, P, torch.bfloat16, seed=keys + D)
    g = torch.Generator().manual_seed(5)
    q = (3.0 * torch.randn(n, Hq, D, generator=g)).to(torch.bfloat16)
    per_split = -(-seq_lens[0] // splits)
    special = [0, 1, P - 1, P, 127, 128, per_split - 1, per_split, 2 * per_split + 1, 4095, 4096]
    for i, s in enumerate(seq_lens):
        places = [(special[(i * Hkv + h) % len(special)] if (i + h) % 3 else s - 1 - h) % s
                  for h in range(Hkv)]
        _hot_keys(dk, kc, bt, P, i, places)
        q[i, 0::G] = 2.0
        q[i, 1::G] = 2.0
    dev = "cuda"
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    out = torch.zeros(n, Hq, D, dtype=torch.bfloat16, device=dev)
    scale = 1.0 / math.sqrt(D)
    ops.attention_decode(out, q.to(dev), kc.to(dev), vc.to(dev), i32(list(range(n + 1))),
                         i32(seq_lens), bt.to(dev), n, scale, 0, splits, matrix_cores=True)
    for i, s in enumerate(seq_lens):
        want = plain_llama.causal_attention(q[i:i + 1].float(), dk[i], dv[i], scale,
                                            query_positions=[s - 1])[0]
        got = out[i].float().cpu()
        # the rows that point at one key return its value
        assert float(want[0::G].abs().max()) > 0.5
        err = float((got - want).abs().max()) / float(want.abs().max())
        assert err < 2e-2, f"sequence {i} ({s} keys, {splits} splits): error {err:.3g} of the largest value"


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("prefix,rows", [(14336, 2048), (8192, 8192)])
def test_attention_prefill_mfma_long_prefix(ops, D, prefix, rows):
    """A portion of 2,048 rows behind 14,336 keys in the cache (one workgroup a block by the
    plan for 32 heads: 64-row blocks at head size 64, 128-row blocks at head size 128, where
    the long prefix decides) and one of 8,192 rows behind 8,192 (128-row blocks, the list shared
    by fewer workgroups than blocks), with the block size and workgroups that the plan gives
    and the work list the engine builds. Compared for the first, a middle and the last 128 rows;
    one query head a group points at one far key, the others are random with wide scores."""
    from pytriton_llama_amd.engine.batch import work_items
    Hq, Hkv, P = 32, 8, 16
    G = Hq // Hkv
    total = prefix + rows
    kc, vc, bt, dk, dv = _paged_setup([total], [rows], Hkv, D, P, torch.bfloat16, seed=prefix + D)
    g = torch.Generator().manual_seed(6)
    q = (3.0 * torch.randn(rows, Hq, D, generator=g)).to(torch.bfloat16)
    q[:, 0::G] = 2.0
    _hot_keys(dk, kc, bt, P, 0, [0, 15, 16, 4095, 8192, prefix - 1, prefix, prefix + 5])
    n64, n128 = -(-rows // 64), -(-rows // 128)
    block_rows, groups = ops.attention_prefill_mfma_plan(torch.device("cuda", 0), Hq, D, n64, n128, total)
    if rows == 8192:
        assert block_rows == 128 and groups < n128, "the case is meant to share the list"
    elif torch.cuda.get_device_properties(0).multi_processor_count <= 256:
        # few blocks, all of them long: 128 rows a block at head size 128, 64 at head size 64
        assert block_rows == (128 if D > 64 else 64) and groups == (n128 if D > 64 else n64)
    ws, wo = work_items([rows], [total], 0, block_rows)
    dev = "cuda"
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    out = torch.zeros(rows, Hq, D, dtype=torch.bfloat16, device=dev)
    scale = 1.0 / math.sqrt(D)
    ops.attention_prefill_mfma(out, q.to(dev), kc.to(dev), vc.to(dev), i32([0, rows]), i32([total]),
                               bt.to(dev), torch.from_numpy(ws).to(dev), torch.from_numpy(wo).to(dev),
                               scale, 0, block_rows, groups)
    out = out.float().cpu()
    for lo in (0, (rows // 2 // 128) * 128 - 64, rows - 128):
        sel = list(range(lo, lo + 128))
        want = plain_llama.causal_attention(q[sel].float(), dk[0], dv[0], scale,
                                            query_positions=[prefix + r for r in sel])
        err = float((out[sel] - want).abs().max()) / float(want.abs().max())
        assert err < 2e-2, f"rows {lo}..{lo + 127} behind {prefix} keys: error {err:.3g} of the largest value"


@pytest.mark.parametrize("kernel", ["decode", "decode_mfma", "mfma", "mfma128"])
def test_attention_far_key_stands_out_fast_kernels(ops, kernel):
    def boost(q, dk, kc, bt):
        direction = torch.ones(64) * 2.0
        q[-1, :, :] = direction.to(q.dtype)
        page = int(bt[0, 0])
        kc[page, :, 3] = direction.to(kc.dtype)
        dk[0][3] = direction
    ql = 2 if kernel.startswith("mfma") else 1
    _attention_case(ops, torch.bfloat16, seq_lens=[700], q_lens=[ql], Hq=2, Hkv=1, D=64, P=16,
                    boost=boost, kernel=kernel, splits=4)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_attention_window(ops, dtype):
    _attention_case(ops, dtype, seq_lens=[90, 40], q_lens=[25, 1], Hq=4, Hkv=2, D=32, P=8, window=20)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_attention_far_key_stands_out(ops, dtype):
    """One early key is made to dominate the last query's scores, so a kernel
    that drops or misplaces a far page fails."""
    def boost(q, dk, kc, bt):
        # key 3 of sequence 0 (first page) aligned with the last query, head 0
        direction = torch.ones(32) * 3.0
        q[-1, :, :] = direction.to(q.dtype)
        page = int(bt[0, 0])
        kc[page, :, 3] = direction.to(kc.dtype)
        dk[0][3] = direction
    _attention_case(ops, dtype, seq_lens=[300], q_lens=[1], Hq=2, Hkv=1, D=32, P=16, boost=boost)


def test_attention_page_placement_does_not_matter(ops):
    """The same keys in differently permuted pages give the same output bit for bit."""
    outs = []
    for shuffle_seed in (0, 1):
        kc, vc, bt, dk, dv = _paged_setup([75], [75], 2, 32, 8, torch.float32, seed=4, shuffle=True)
        if shuffle_seed:
            perm = torch.randperm(kc.shape[0], generator=torch.Generator().manual_seed(99))
            inv = torch.empty_like(perm)
            inv[perm] = torch.arange(len(perm))
            kc, vc = kc[perm], vc[perm]
            bt = torch.where(bt >= 0, inv[bt.clamp(min=0).long()].to(torch.int32), bt)
        q = torch.randn(75, 4, 32, generator=torch.Generator().manual_seed(8))
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
        out = torch.zeros(75, 4, 32, device="cuda")
        ops.attention_generic(out, q.cuda(), kc.cuda(), vc.cuda(), i32([0, 75]), i32([75]),
                              bt.cuda(), i32([0, 0, 0, 0, 0]), i32([0, 16, 32, 48, 64]),
                              1 / math.sqrt(32), 0)
        outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("V", [1003, 4096, 8193, 128256])
def test_argmax(ops, V):
    torch.manual_seed(5)
    logits = torch.randn(6, V, device="cuda")
    logits[2, 7] = logits[2, V - 100] = 50.0       # a tie goes to the lowest id, across chunks too
    logits[3, 401] = logits[3, 402] = 70.0         # ... and inside one 16-byte load
    logits[4, V - 1] = 60.0
    logits[1, 0] = logits[5, 9] = float("nan")     # a NaN is never the choice
    got = ops.argmax(logits).cpu()
    want = torch.argmax(torch.nan_to_num(logits.cpu(), nan=-float("inf")), dim=-1)
    want[2], want[3] = 7, 401
    assert got.tolist() == want.tolist()
    # the kernel can leave the choices in pinned host memory as well
    host = torch.full((8,), -1, dtype=torch.int32).pin_memory()
    again = ops.argmax(logits, host_out=host)
    torch.cuda.synchronize()
    assert again.cpu().tolist() == want.tolist() and host.tolist() == want.tolist() + [-1, -1]


def test_sample_top_p_distribution(ops):
    """The kernel's nucleus equals the plain rule's, and the draw follows it."""
    torch.manual_seed(6)
    R, V = 5, 777
    logits = (3 * torch.randn(R, V)).cuda()
    temperature = torch.tensor([0.8, 1.0, 0.5, 2.0, 0.7]).cuda()
    top_p = torch.tensor([0.9, 1.0, 0.3, 0.95, 1e-6]).cuda()
    u = torch.tensor([0.0, 0.5, 0.999, 0.25, 0.7]).cuda()
    tok, probs = ops.sample_top_p(logits, temperature, top_p, u, return_probs=True)
    for r in range(R):
        want = plain_llama.top_p_probs(logits[r].cpu(), float(temperature[r]), float(top_p[r]))
        torch.testing.assert_close(probs[r].cpu().double(), want, atol=1e-5, rtol=1e-4)
        # inverse CDF in vocabulary order
        cdf = torch.cumsum(want, 0)
        expect = int(torch.searchsorted(cdf, torch.tensor(float(u[r]), dtype=torch.double), right=True))
        got = int(tok[r])
        assert want[got] > 0
        assert abs(float(cdf[got]) - float(cdf[min(expect, V - 1)])) < 1e-4 or got == expect
    # top_p -> 0 is greedy
    assert int(tok[4]) == int(torch.argmax(logits[4]))


def test_sample_top_p_frequencies(ops):
    """Many draws with different uniforms reproduce the probabilities."""
    logits = torch.tensor([[2.0, 1.0, 0.0, -1.0, 0.5, -30.0]]).cuda().repeat(4000, 1)
    t = torch.full((4000,), 1.0).cuda()
    p = torch.full((4000,), 0.9).cuda()
    u = torch.rand(4000, generator=torch.Generator().manual_seed(1)).cuda()
    tok = ops.sample_top_p(logits, t, p, u).cpu()
    want = plain_llama.top_p_probs(logits[0].cpu(), 1.0, 0.9)
    freq = torch.bincount(tok.long(), minlength=6).double() / 4000
    assert torch.all((freq - want).abs() < 0.03), (freq, want)
    assert freq[want == 0].sum() == 0


@pytest.mark.parametrize("V", [16384, 20000, 128256])
def test_sample_top_p_one_and_many_workgroups_a_row_agree(ops, V):
    """The one-kernel and the many-workgroup samplers follow the same rule: the same nucleus
    (up to a token at its edge, where float32 sums taken in another order meet top_p) and the
    same draw, for peaked, ordinary and flat rows, top_p from almost 0 to 1, -inf and NaN
    logits, and u at both ends."""
    g = torch.Generator().manual_seed(V)
    R = 12
    logits = torch.randn(R, V, generator=g)
    scale = torch.tensor([8.0, 4.0, 2.0, 1.0, 0.3, 0.02, 3.0, 3.0, 3.0, 3.0, 3.0, 1e-3]).view(R, 1)
    logits = logits * scale
    logits[6, ::3] = float("-inf")
    logits[7, 5] = float("nan")
    logits[8, V - 1] = 30.0                                  # the last token holds the mass
    t = torch.tensor([0.6, 1.0, 0.8, 1.5, 1.0, 1.0, 0.7, 0.7, 0.7, 0.7, 0.7, 1.0])
    p = torch.tensor([0.9, 0.9, 0.5, 0.95, 0.9, 0.9, 0.9, 0.9, 0.9, 1.0, 1e-6, 0.37])
    u = torch.tensor([0.0, 0.3, 0.999999, 0.5, 0.77, 0.123, 0.9, 0.2, 0.5, 0.6, 0.4, 0.999])
    args = [a.cuda() for a in (logits, t, p, u)]
    tok1, pr1 = ops.sample_top_p(*args, return_probs=True, wide=False)
    tokw, prw = ops.sample_top_p(*args, return_probs=True, wide=True)
    tokw2 = ops.sample_top_p(*args, wide=True)
    assert tokw.tolist() == tokw2.tolist()                    # the same call, the same tokens
    for r in range(R):
        a, b = pr1[r].double().cpu(), prw[r].double().cpu()
        assert abs(float(b.sum()) - 1) < 1e-4
        assert float((a - b).abs().sum()) < 2e-3, r
        # the draw: same token, or a neighbour in the cumulative distribution
        ca = torch.cumsum(b, 0)
        assert int(tokw[r]) == int(tok1[r]) or abs(float(ca[int(tokw[r])] - ca[int(tok1[r])])) < 1e-3, r
        assert b[int(tokw[r])] > 0
    assert int(tokw[8]) == V - 1 and int(tokw[10]) == int(torch.argmax(logits[10]))
    for r in (0, 2, 4):                                       # against the plain rule
        want = plain_llama.top_p_probs(torch.nan_to_num(logits[r], nan=float("-inf")), float(t[r]), float(p[r]))
        assert float((prw[r].double().cpu() - want).abs().sum()) < 1e-3


@pytest.mark.parametrize("wide", [False, True], ids=["one_workgroup", "many_workgroups"])
def test_sample_top_p_nearly_flat_row_and_signed_zeros(ops, wide):
    """A nearly flat row with a top_p that admits two tokens keeps exactly those two (the most
    likely token is always kept, its neighbours only by the rule); +0 and -0 are one logit."""
    V = 20000
    g = torch.Generator().manual_seed(4)
    flat = torch.randn(V, generator=g) * 1e-3
    top = torch.topk(flat, 3).indices.tolist()
    zeros = torch.zeros(V)
    zeros[::2] = -0.0
    zeros[[11, 500]] = torch.tensor([1.0, 0.5])
    logits = torch.stack([flat, zeros]).cuda()
    t = torch.ones(2).cuda()
    # row 0: every token has about 1/V of the mass; the mass before the third token is ~2/V
    # row 1: tokens 11 and 500 hold e + sqrt(e) of e + sqrt(e) + V - 2; 0.01 lets in the zeros' first
    p = torch.tensor([1.5 / V, 0.01]).cuda()
    u = torch.tensor([0.99, 0.5]).cuda()
    tok, probs = ops.sample_top_p(logits, t, p, u, return_probs=True, wide=wide)
    kept0 = torch.nonzero(probs[0]).flatten().tolist()
    assert sorted(kept0) == sorted(top[:2]) and int(tok[0]) in kept0
    want = plain_llama.top_p_probs(zeros, 1.0, 0.01)
    got = probs[1].double().cpu()
    # all zeros, whatever their sign, are kept together (the plain sort would split them)
    rest = got[torch.arange(V)[(torch.arange(V) != 11) & (torch.arange(V) != 500)]]
    assert float(rest.min()) == float(rest.max()) and got[11] > got[500] > rest[0] >= 0
    assert bool((got > 0).all()) == bool(rest[0] > 0) and want[11] > 0


def test_kernels_refuse_cpu_tensors(ops):
    with pytest.raises(ops.KernelError):
        ops.silu_mul(torch.zeros(2, 4))
    with pytest.raises(ops.KernelError):
        ops.add_rmsnorm(torch.zeros(2, 64), None, torch.ones(64), 1e-5)
    with pytest.raises(ops.KernelError):        # a weight of the wrong length
        ops.add_rmsnorm(torch.zeros(2, 64, device="cuda"), None, torch.ones(63, device="cuda"), 1e-5)


def test_sample_top_p_large_vocabulary_and_ties(ops):
    """At vocabulary size, with a peaked and a flat row, and a row of many equal
    logits (more tokens in one histogram bin than the kernel gathers)."""
    torch.manual_seed(11)
    V = 128256
    logits = torch.randn(4, V)
    logits[0] *= 4.0                                   # peaked
    logits[1] *= 0.05                                  # nearly flat
    logits[2] = 0.0                                    # all equal but a few
    logits[2, [5, 77, 99999]] = torch.tensor([3.0, 2.0, 1.0])
    logits[3, 1234] = 40.0                             # one token holds all the mass
    t = torch.tensor([0.8, 1.0, 1.0, 0.6])
    p = torch.tensor([0.9, 0.5, 0.5, 0.9])
    u = torch.tensor([0.3, 0.9, 0.999999, 0.5])
    tok, probs = ops.sample_top_p(logits.cuda(), t.cuda(), p.cuda(), u.cuda(), return_probs=True)
    for r in (0, 1, 3):
        want = plain_llama.top_p_probs(logits[r], float(t[r]), float(p[r]))
        got = probs[r].cpu().double()
        # the nucleus may differ by a token or two at its edge where the float32 running
        # mass meets top_p; the mass that changes hands is tiny
        assert float((got - want).abs().sum()) < 1e-3
        assert want[int(tok[r])] > 0
    assert int(tok[3]) == 1234
    # equal logits are kept or dropped together: the three larger ones first, then all or none
    got2 = probs[2].cpu()
    assert got2[5] > got2[77] > got2[99999] > 0
    rest = got2[torch.arange(V)[(torch.arange(V) != 5) & (torch.arange(V) != 77) & (torch.arange(V) != 99999)]]
    assert float(rest.min()) == float(rest.max())
    assert abs(float(got2.sum()) - 1) < 1e-4
