"""Bit-exact checks of the bf16 matrix kernels at the shapes of the training step (B*T = 65536 rows).

With small integer operands every product and every fp32 partial sum of a contraction is exact whatever the order of
summation (|x| <= 4, |w| <= 4: sums stay below 2^24 up to a contraction length of 2^20), so the only rounding left is the
single conversion of the result to bf16, and the kernel's output must equal the integer matrix product rounded once -
bit for bit. A stale or misplaced operand tile, a wait that lets a stage be read before it has landed, a tile stored
twice or not at all, an epilogue applied to the wrong columns: each of them changes integers, not last bits.
The reference product is an fp32 matmul on the device (exact for the same reason), row chunk by row chunk.

Attention has no exact integer form (softmax weights 1/(t+1)); it is held at the benchmark shape to an fp32
formulation of the same mathematics, to a relative Frobenius bound, and to the exact zeros that Q = 0 (dK = 0) and
K = 0 (dQ = 0) force.
"""
import ctypes as CT

import numpy as np
import pytest

import gpu_lib as G

pytestmark = pytest.mark.gpu

N_ROWS = 65536


@pytest.fixture(scope="module", autouse=True)
def _cuda():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    yield
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def ints(shape, seed, lo=-4, hi=4, scale=1.0):
    """integer-valued bf16 tensor on the device, optionally scaled by a power of two"""
    import torch
    g = torch.Generator(device="cuda"); g.manual_seed(seed)
    t = torch.randint(lo, hi + 1, shape, generator=g, device="cuda", dtype=torch.int32).to(torch.float32) * scale
    return t.to(torch.bfloat16).contiguous()


def exact_nt(x, w, rows=None, chunk=8192):
    """fp32 x . w^T of integer-valued bf16 operands (exact), for all rows or the given ones"""
    import torch
    if rows is not None:
        return x[rows].float() @ w.float().t()
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32, device="cuda")
    wf = w.float().t().contiguous()
    for r in range(0, x.shape[0], chunk):
        out[r:r + chunk] = x[r:r + chunk].float() @ wf
    return out


def exact_tn(g, x, chunk=8192):
    """fp32 g^T . x (contraction over the rows), exact"""
    import torch
    out = torch.zeros((g.shape[1], x.shape[1]), dtype=torch.float32, device="cuda")
    for r in range(0, g.shape[0], chunk):
        out += g[r:r + chunk].float().t() @ x[r:r + chunk].float()
    return out


def assert_same_bits(got, want_f32, what):
    import torch
    want = want_f32.to(torch.bfloat16)
    if not torch.equal(got, want):
        bad = (got != want).nonzero()
        first = bad[0].tolist()
        raise AssertionError(f"{what}: {bad.shape[0]} of {got.numel()} elements differ, first at {first}: "
                             f"got {got[tuple(first)].item()}, want {want[tuple(first)].item()}")


# C -> OC of the per-layer projections of GPT-2 124M (qkv, attproj, fc, fcproj), and the widths of 350M / 1558M
LAYER_SHAPES = [(768, 2304), (768, 768), (768, 3072), (3072, 768), (1024, 4096), (1600, 4800), (6400, 1600)]


@pytest.mark.parametrize("C,OC", LAYER_SHAPES)
def test_forward_projection_is_the_integer_product(C, OC):
    import torch
    L = G.lib("bf16")
    M = N_ROWS if C * OC <= 3072 * 768 else N_ROWS // 4
    x, w, b = ints((M, C), 1), ints((OC, C), 2), ints((OC,), 3, -8, 8)
    out = torch.full((M, OC), 7.0, dtype=torch.bfloat16, device="cuda")
    L.llmk_matmul_forward(G.ptr(out), G.ptr(x), G.ptr(w), G.ptr(b), 1, M, C, OC, None, None, 1)
    G.sync()
    assert_same_bits(out, exact_nt(x, w) + b.float(), "out = x.w^T + b")
    # without a bias (the plain-store epilogue)
    L.llmk_matmul_forward(G.ptr(out), G.ptr(x), G.ptr(w), None, 1, M, C, OC, None, None, 1)
    G.sync()
    assert_same_bits(out, exact_nt(x, w), "out = x.w^T")
    G.check_no_error(L)


@pytest.mark.parametrize("M,C,OC", [(N_ROWS, 768, 768), (N_ROWS, 3072, 768), (N_ROWS // 2, 4096, 1024), (N_ROWS // 4, 6400, 1600),
                                    (N_ROWS // 4 + 72, 768, 832), (640, 768, 768)])
def test_forward_projection_with_residual_epilogue(M, C, OC):
    """out = bf16(bf16(x.w^T + b) + residual): the integer product rounded once, then the sum with a residual of
    non-integers rounded once more - and the same bits as the two kernels it stands for. The projections into the
    residual stream at the three model widths, a shape with ragged last tiles in both directions, and one too small for
    the fused epilogue (which then runs the two kernels itself)."""
    import torch
    L = G.lib("bf16")
    x, w, b = ints((M, C), 11), ints((OC, C), 12), ints((OC,), 13, -8, 8)
    g = torch.Generator(device="cuda"); g.manual_seed(14)
    res = (torch.randn((M, OC), generator=g, device="cuda") * 3.0).to(torch.bfloat16)
    out = torch.full((M, OC), 7.0, dtype=torch.bfloat16, device="cuda")
    for bias in (b, None):
        L.llmk_matmul_forward_residual(G.ptr(out), G.ptr(x), G.ptr(w), G.ptr(bias) if bias is not None else None, G.ptr(res),
                                       1, M, C, OC, None)
        G.sync()
        proj = exact_nt(x, w) + (bias.float() if bias is not None else 0.0)
        want = proj.to(torch.bfloat16).float() + res.float()
        assert_same_bits(out, want, "out = round(round(x.w^T + b) + residual)")
        two = torch.empty_like(out)
        L.llmk_matmul_forward(G.ptr(two), G.ptr(x), G.ptr(w), G.ptr(bias) if bias is not None else None, 1, M, C, OC, None, None, 1)
        L.llmk_residual_forward(G.ptr(two), G.ptr(res), G.ptr(two), M * OC, None)
        G.sync()
        assert torch.equal(out, two), "the fused epilogue and the two kernels differ"
    G.check_no_error(L)


@pytest.mark.parametrize("C,OC", [(768, 3072), (1024, 4096), (1600, 6400)])
def test_forward_projection_with_gelu_epilogue(C, OC):
    """The fc layer with GELU in the GEMM's epilogue: the pre-activation output is the exact product (operands scaled by
    powers of two so that it spans GELU's curved range), and the activated output is what the library's own GELU
    kernel makes of that tensor, bit for bit (both apply the same function to the bf16-rounded pre-activation)."""
    import torch
    L = G.lib("bf16")
    M = N_ROWS if OC <= 3072 else N_ROWS // 4
    x, w, b = ints((M, C), 4), ints((OC, C), 5, scale=1.0 / 64), ints((OC,), 6, -8, 8, scale=1.0 / 8)
    out = torch.zeros((M, OC), dtype=torch.bfloat16, device="cuda")
    pre = torch.zeros((M, OC), dtype=torch.bfloat16, device="cuda")
    L.llmk_matmul_forward(G.ptr(out), G.ptr(x), G.ptr(w), G.ptr(b), 1, M, C, OC, None, G.ptr(pre), 2)
    G.sync()
    assert_same_bits(pre, exact_nt(x, w) + b.float(), "pre_gelu")
    assert 0.5 < pre.float().abs().mean().item() < 8.0          # inside the range where GELU is not the identity or zero
    want = torch.zeros_like(out)
    L.llmk_gelu_forward(G.ptr(want), G.ptr(pre), M * OC, None)
    G.sync()
    assert torch.equal(out, want)
    G.check_no_error(L)


@pytest.mark.parametrize("C,OC", [(768, 3072), (1024, 4096), (1600, 6400)])
def test_gelu_fusion_3_epilogues_at_the_training_shapes(C, OC):
    """The fc layer forward with gelu_fusion 3 and the fcproj layer's dinp that consumes it: the activated output is the
    same bits as with fusion 2, the second output is the library's own GELU derivative of the exact pre-activation
    (what llmk_gelu_backward_inplace makes of a tensor of ones), and dinp is the exact product, rounded, times that
    stored value, rounded once (a product of two bf16 values is exact in fp32)."""
    import torch
    L = G.lib("bf16")
    M = N_ROWS if OC <= 3072 else N_ROWS // 4
    x, w, b = ints((M, C), 4), ints((OC, C), 5, scale=1.0 / 64), ints((OC,), 6, -8, 8, scale=1.0 / 8)
    out = torch.zeros((M, OC), dtype=torch.bfloat16, device="cuda")
    grad = torch.zeros((M, OC), dtype=torch.bfloat16, device="cuda")
    L.llmk_matmul_forward(G.ptr(out), G.ptr(x), G.ptr(w), G.ptr(b), 1, M, C, OC, None, G.ptr(grad), 3)
    G.sync()
    pre = (exact_nt(x, w) + b.float()).to(torch.bfloat16)
    want = torch.zeros_like(out)
    L.llmk_gelu_forward(G.ptr(want), G.ptr(pre), M * OC, None)
    want_grad = torch.ones_like(out)
    L.llmk_gelu_backward_inplace(G.ptr(want_grad), G.ptr(pre), M * OC, None)
    G.sync()
    assert torch.equal(out, want)
    assert torch.equal(grad, want_grad)
    del pre, want, want_grad, out
    # backward: dinp (M, OC) = (dout (M, C) . w2 (C, OC)) * stored derivative
    g, w2 = ints((M, C), 14, -2, 2), ints((C, OC), 13)
    dx = torch.zeros((M, OC), dtype=torch.bfloat16, device="cuda")
    dw = torch.zeros((C, OC), dtype=torch.bfloat16, device="cuda")
    inp = ints((M, OC), 12, -2, 2)
    L.llmk_matmul_backward(G.ptr(dx), G.ptr(dw), None, G.ptr(g), G.ptr(inp), G.ptr(w2), None, 1, M, OC, C, None, G.ptr(grad), 3)
    G.sync()
    lin = exact_nt(g, w2.t().contiguous()).to(torch.bfloat16)
    assert torch.equal(dx, (lin.float() * grad.float()).to(torch.bfloat16))
    assert_same_bits(dw, exact_tn(g, inp), "dweight")
    G.check_no_error(L)


@pytest.mark.parametrize("split_mode", [0, 1])
@pytest.mark.parametrize("C,OC", LAYER_SHAPES + [(1600, 1600), (1600, 6400)])
def test_backward_projection_is_the_integer_product(C, OC, split_mode):
    """dinp = dout . W (overwrites), dweight += dout^T . inp over 65536 rows (split K, partial sums in fp32), dbias +=
    column sums of dout (taken inside the weight-gradient GEMM). Both ways of cutting the contraction into work items:
    equal splits of every tile (0), one long and a few short pieces per tile where the shape allows them (1)."""
    import torch
    L = G.lib("bf16")
    L.llmk_matmul_backward_split_mode(split_mode)
    try:
        _backward_projection_case(L, C, OC)
    finally:
        L.llmk_matmul_backward_split_mode(-1)
    # the way asked for is the way that ran: with 256 workgroups the uneven pieces need 32 to 255 output tiles
    kind, pieces = CT.c_int(-1), CT.c_int(-1)
    L.llmk_matmul_backward_last_split(CT.byref(kind), CT.byref(pieces))
    ncu = CT.c_int(0)
    L.llmk_device_props(CT.byref(ncu), None, None)
    tiles = -(-OC // 256) * -(-C // 256)
    G_ = ncu.value & ~7
    if split_mode == 1 and tiles * 8 >= G_ and tiles < G_:
        assert kind.value == 2 and 2 <= pieces.value <= 6, (kind.value, pieces.value)
        assert (C, OC) in [(768, 3072), (3072, 768), (1024, 4096), (1600, 4800), (6400, 1600), (1600, 6400), (1600, 1600)]
    else:
        assert kind.value == 1 and pieces.value >= 1, (kind.value, pieces.value)


def _backward_projection_case(L, C, OC):
    import torch
    M = N_ROWS if C * OC <= 3072 * 768 else N_ROWS // 4
    x, w, g = ints((M, C), 7, -2, 2), ints((OC, C), 8), ints((M, OC), 9, -2, 2)
    dw0, db0 = ints((OC, C), 10, -50, 50), ints((OC,), 11, -50, 50)
    dx = torch.full((M, C), 7.0, dtype=torch.bfloat16, device="cuda")
    dw, db = dw0.clone(), db0.clone()
    scratch = torch.empty(max(1, L.llmk_matmul_backward_bias_scratch_floats(OC)), dtype=torch.float32, device="cuda")
    L.llmk_matmul_backward(G.ptr(dx), G.ptr(dw), G.ptr(db), G.ptr(g), G.ptr(x), G.ptr(w), G.ptr(scratch), 1, M, C, OC, None,
                           None, 1)
    G.sync()
    assert_same_bits(dx, exact_nt(g, w.t().contiguous()), "dinp = dout.W")
    assert_same_bits(dw, dw0.float() + exact_tn(g, x), "dweight += dout^T.inp")
    assert_same_bits(db, db0.float() + g.float().sum(0), "dbias += sum(dout)")
    G.check_no_error(L)


@pytest.mark.parametrize("C,OC", [(3072, 768), (4096, 1024), (6400, 1600)])
def test_backward_projection_with_gelu_epilogue(C, OC):
    """The fcproj layer's dinp with GELU backward in the GEMM's epilogue (gelu_fusion 2): the product of the once-rounded
    exact gradient with gelu'(pre), i.e. what the library's in-place GELU backward makes of the exact product."""
    import torch
    L = G.lib("bf16")
    M = N_ROWS if C <= 3072 else N_ROWS // 4
    x, w, g = ints((M, C), 12, -2, 2), ints((OC, C), 13), ints((M, OC), 14, -2, 2)
    pre = ints((M, C), 15, -24, 24, scale=1.0 / 8)
    dx = torch.zeros((M, C), dtype=torch.bfloat16, device="cuda")
    dw = torch.zeros((OC, C), dtype=torch.bfloat16, device="cuda")
    L.llmk_matmul_backward(G.ptr(dx), G.ptr(dw), None, G.ptr(g), G.ptr(x), G.ptr(w), None, 1, M, C, OC, None, G.ptr(pre), 2)
    G.sync()
    want = exact_nt(g, w.t().contiguous()).to(torch.bfloat16)
    L.llmk_gelu_backward_inplace(G.ptr(want), G.ptr(pre), M * C, None)
    G.sync()
    assert torch.equal(dx, want)
    assert_same_bits(dw, exact_tn(g, x), "dweight")
    G.check_no_error(L)


def test_lm_head_forward_and_backward_are_the_integer_products():
    """The (65536 x 768) . (768 x 50304) classifier GEMM: 64 sampled rows x all columns of the 6.6 GB of logits plus a
    checksum over all of them, and both gradients in full."""
    import torch
    L = G.lib("bf16")
    M, C, V = N_ROWS, 768, 50304
    x, w = ints((M, C), 16, -2, 2), ints((V, C), 17, -2, 2)
    out = torch.empty((M, V), dtype=torch.bfloat16, device="cuda")
    L.llmk_matmul_forward(G.ptr(out), G.ptr(x), G.ptr(w), None, 1, M, C, V, None, None, 1)
    G.sync()
    rows = torch.from_numpy(np.random.RandomState(0).choice(M, 64, replace=False).astype(np.int64)).cuda()
    rows[0], rows[1], rows[2] = 0, M - 1, 255
    assert_same_bits(out[rows], exact_nt(x, w, rows=rows), "logits (sampled rows)")
    # all rows: row sums of the logits = x . (sum of the rows of w), up to the bf16 rounding of each logit. A logit has a
    # standard deviation of 55 here (all but a few in a million are below 256), so its rounding error is at most half a unit and spread like a uniform variable: over a row's
    # 50304 columns that sums to a standard deviation of at most sqrt(50304 / 12) = 65. A missing, doubled or misplaced
    # tile moves the sums of its 256 rows by a signed sum of 256 logits, about sqrt(256) * 55 = 900 for a typical row.
    got = torch.zeros(M, dtype=torch.float64, device="cuda")
    for r in range(0, M, 4096):
        got[r:r + 4096] = out[r:r + 4096].double().sum(1)
    want = x.double() @ w.double().sum(0)
    assert (got - want).abs().max().item() < 400.0, (got - want).abs().max().item()
    # backward: dlogits in place of the logits (integers again), dinp and dwte in full
    g = ints((M, V), 18, -1, 1)
    dw0 = ints((V, C), 19, -50, 50)
    dw = dw0.clone()
    dx = torch.empty((M, C), dtype=torch.bfloat16, device="cuda")
    del out
    L.llmk_matmul_backward(G.ptr(dx), G.ptr(dw), None, G.ptr(g), G.ptr(x), G.ptr(w), None, 1, M, C, V, None, None, 1)
    G.sync()
    wt = w.float()
    for r in range(0, M, 4096):
        assert_same_bits(dx[r:r + 4096], g[r:r + 4096].float() @ wt, f"dinp rows {r}..")
    acc = torch.zeros((V, C), dtype=torch.float32, device="cuda")
    for r in range(0, M, 2048):
        acc += g[r:r + 2048].float().t() @ x[r:r + 2048].float()
    assert_same_bits(dw, dw0.float() + acc, "dwte += dlogits^T . x")
    G.check_no_error(L)


# ---------------------------------------------------------------------------------------------------------------------
def torch_attention(qkv, dout, NH):
    """causal softmax(Q K^T / sqrt(hs)) V and its gradient in fp32 on the device, per batch row"""
    import torch
    B, T, C3 = qkv.shape
    Cc = C3 // 3
    hs = Cc // NH
    out = torch.empty((B, T, Cc), dtype=torch.float32, device="cuda")
    lse = torch.empty((B, NH, T), dtype=torch.float32, device="cuda")
    dqkv = torch.empty((B, T, C3), dtype=torch.float32, device="cuda")
    mask = torch.ones((T, T), dtype=torch.bool, device="cuda").tril()
    for b in range(B):
        x = qkv[b].float().view(T, 3, NH, hs).permute(1, 2, 0, 3).contiguous().requires_grad_(True)      # (3, NH, T, hs)
        s = (x[0] @ x[1].transpose(1, 2)) * (1.0 / np.sqrt(hs))
        s = s.masked_fill(~mask, float("-inf"))
        lse[b] = torch.logsumexp(s, dim=-1).detach()
        o = torch.softmax(s, dim=-1) @ x[2]                                                             # (NH, T, hs)
        o.backward(dout[b].float().view(T, NH, hs).permute(1, 0, 2))
        out[b] = o.detach().permute(1, 0, 2).reshape(T, Cc)
        dqkv[b] = x.grad.permute(2, 0, 1, 3).reshape(T, C3)
    return out, lse, dqkv


def rel_fro(got, want):
    return ((got.float() - want).norm() / want.norm().clamp_min(1e-30)).item()


@pytest.mark.parametrize("B,T,NH", [(64, 1024, 12), (32, 1024, 16), (16, 1024, 25)])
def test_attention_at_the_benchmark_shapes(B, T, NH):
    """Every (batch, head) of the shapes the throughput is quoted on, forward and backward, against the fp32 formulation:
    relative Frobenius error of each of out, dQ, dK, dV below 1e-2 (bf16 operands and probabilities: 2^-9 relative
    rounding of a value, averaged over sums; measured values are around 3e-3), statistics to 2e-2 absolute."""
    import torch
    L = G.lib("bf16")
    Cc = NH * 64
    gen = torch.Generator(device="cuda"); gen.manual_seed(B + NH)
    qkv = torch.randn((B, T, 3 * Cc), generator=gen, device="cuda").to(torch.bfloat16)
    dout = torch.randn((B, T, Cc), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.zeros((B, T, Cc), dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
    dqkv = torch.full((B, T, 3 * Cc), 3.0, dtype=torch.bfloat16, device="cuda")
    L.llmk_attention_forward(G.ptr(out), G.ptr(stats), G.ptr(qkv), B, T, NH, Cc, None)
    L.llmk_attention_backward(G.ptr(dqkv), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
    G.sync()
    r_out, r_lse, r_d = torch_attention(qkv, dout, NH)
    assert rel_fro(out, r_out) < 1e-2
    assert (stats - r_lse).abs().max().item() < 2e-2
    d = dqkv.float().view(B, T, 3, Cc)
    rd = r_d.view(B, T, 3, Cc)
    for i, name in enumerate(("dQ", "dK", "dV")):
        e = rel_fro(d[:, :, i], rd[:, :, i])
        assert e < 1e-2, (name, e)
        # and per (batch, head): no single head is off (a wrong tile shows up here long before it moves the total)
        dh = (d[:, :, i] - rd[:, :, i]).view(B, T, NH, 64).pow(2).sum((1, 3)).sqrt()
        nh = rd[:, :, i].reshape(B, T, NH, 64).pow(2).sum((1, 3)).sqrt()
        assert (dh / nh).max().item() < 2e-2, (name, (dh / nh).max().item())
    G.check_no_error(L)


@pytest.mark.parametrize("pattern", ["random", "rising", "falling"])
@pytest.mark.parametrize("T", [1024, 320])
def test_attention_with_large_scores(T, pattern):
    """Scores whose spread (hundreds of nats inside a row) is far beyond what an exponential survives without the row's
    true running maximum: a reference point taken from only part of a key block, or one that lags, overflows here, where
    ordinary-sized inputs would still give the right answer. Forward output against the fp32 formulation
    (train_gpt2.c:271-345), every value finite. T = 1024 takes the direct-to-LDS kernel, T = 320 the register-staged one.
      random:  q and k scaled by 8, scores of +-60 nats rms.
      rising:  every row's scores grow along the keys by about 0.3 nats per key (plus noise), 19 nats per 64-key step,
               so every step of the key loop moves the reference point, by more than any slack it is allowed to lag.
      falling: the mirror image, the first keys dominate by up to 300 nats, the reference point settles in the first
               key tile and never moves again, and the probabilities of all later tiles underflow."""
    import torch
    L = G.lib("bf16")
    B, NH = 4, 6
    Cc = NH * 64
    gen = torch.Generator(device="cuda"); gen.manual_seed(T)
    qkv = torch.randn((B, T, 3 * Cc), generator=gen, device="cuda")
    if pattern == "random":
        qkv[:, :, :2 * Cc] *= 8.0                              # q and k: scores of +-60 nats rms, several hundred at the extremes
    else:
        # q = 8 u + noise, k_t = +-0.3 t u + noise with u a unit vector per head: score(q, k_t) = q.k_t / 8 = +-0.3 t + O(1)
        u = torch.randn((NH, 64), generator=gen, device="cuda")
        u = (u / u.norm(dim=1, keepdim=True)).view(1, 1, Cc)
        t = torch.arange(T, device="cuda", dtype=torch.float32).view(1, T, 1)
        qkv[:, :, :Cc] = 8.0 * u + 0.5 * qkv[:, :, :Cc]
        qkv[:, :, Cc:2 * Cc] = (0.3 if pattern == "rising" else -0.3) * t * u + 0.5 * qkv[:, :, Cc:2 * Cc]
    qkv = qkv.to(torch.bfloat16)
    out = torch.zeros((B, T, Cc), dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
    L.llmk_attention_forward(G.ptr(out), G.ptr(stats), G.ptr(qkv), B, T, NH, Cc, None)
    G.sync()
    assert torch.isfinite(out.float()).all() and torch.isfinite(stats).all()
    r_out, r_lse, _ = torch_attention(qkv, torch.zeros((B, T, Cc), dtype=torch.bfloat16, device="cuda"), NH)
    assert rel_fro(out, r_out) < 1e-2
    assert ((stats - r_lse).abs() / r_lse.abs().clamp_min(1.0)).max().item() < 1e-2
    if pattern == "rising":
        spread = (r_lse.max() - r_lse.min()).item()
        assert spread > 60.0, spread                           # the rows' reference points do span the range claimed
    G.check_no_error(L)


@pytest.mark.parametrize("zero", ["Q", "K"])
def test_attention_exact_zeros(zero):
    """Q = 0: all scores are 0, every row is the running mean of V, and dK = scale * dS^T Q is exactly zero;
    K = 0: the same probabilities, and dQ = scale * dS K is exactly zero. The other gradients against fp32."""
    import torch
    L = G.lib("bf16")
    B, T, NH = 4, 1024, 12
    Cc = NH * 64
    gen = torch.Generator(device="cuda"); gen.manual_seed(5)
    qkv = torch.randn((B, T, 3, Cc), generator=gen, device="cuda").to(torch.bfloat16)
    qkv[:, :, 0 if zero == "Q" else 1] = 0
    qkv = qkv.view(B, T, 3 * Cc).contiguous()
    dout = torch.randn((B, T, Cc), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.zeros((B, T, Cc), dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
    dqkv = torch.full((B, T, 3 * Cc), 3.0, dtype=torch.bfloat16, device="cuda")
    L.llmk_attention_forward(G.ptr(out), G.ptr(stats), G.ptr(qkv), B, T, NH, Cc, None)
    L.llmk_attention_backward(G.ptr(dqkv), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
    G.sync()
    v = qkv.view(B, T, 3, Cc)[:, :, 2].float()
    mean = v.cumsum(1) / torch.arange(1, T + 1, device="cuda", dtype=torch.float32).view(1, T, 1)
    assert (out.float() - mean).abs().max().item() <= 2.0 ** -8 * mean.abs().max().item() + 1e-3
    want_lse = torch.log(torch.arange(1, T + 1, device="cuda", dtype=torch.float32)).view(1, 1, T).expand(B, NH, T)
    assert (stats - want_lse).abs().max().item() < 1e-4
    d = dqkv.view(B, T, 3, Cc)
    assert (d[:, :, 1 if zero == "Q" else 0] == 0).all()
    _, _, r_d = torch_attention(qkv, dout, NH)
    rd = r_d.view(B, T, 3, Cc)
    for i in ((0, 2) if zero == "Q" else (1, 2)):
        assert rel_fro(d[:, :, i], rd[:, :, i]) < 1e-2, i
    G.check_no_error(L)


def test_row_wise_last_stage_variant_gives_the_same_bits():
    """The GEMM kernel's switched-off alternative schedule (LLMK_ROWWISE_LAST, a variant build that
    llm.c_amd/microbench.py --against rowwise times) changes the order of instructions, not of additions: where that
    build is present it must agree with the product library bit for bit, forward (bias and GELU epilogues) and dinp."""
    import os
    import torch
    pkg = G.package()
    path = os.path.join(os.path.dirname(pkg.lib_path("bf16")), "variants", "rowwise", "libllmk_bf16.so")
    if not os.path.exists(path):
        pytest.skip("no variant build: python llm.c_amd/build.py bf16 --variant rowwise -DLLMK_ROWWISE_LAST=1")
    L = G.lib("bf16")
    try:
        V = pkg.bind(CT.CDLL(path))
    except AttributeError as e:
        pytest.skip(f"the variant build is older than the library's interface ({e}): build it again")
    V.llmk_init(0)
    g = torch.Generator(device="cuda"); g.manual_seed(11)
    rn = lambda *s, scale=1.0: (torch.randn(*s, device="cuda", generator=g) * scale).to(torch.bfloat16)
    for C, OC in ((768, 3072), (3072, 768), (768, 2000)):          # the last one: tiles that reach past N
        M = N_ROWS // 2
        x, w, b = rn(M, C), rn(OC, C, scale=0.05), rn(OC)
        outs = []
        for lib in (L, V):
            out = torch.full((M, OC), 3.0, dtype=torch.bfloat16, device="cuda")
            pre = torch.full((M, OC), 5.0, dtype=torch.bfloat16, device="cuda")
            act = torch.full((M, OC), 5.0, dtype=torch.bfloat16, device="cuda")
            lib.llmk_matmul_forward(G.ptr(out), G.ptr(x), G.ptr(w), G.ptr(b), 1, M, C, OC, None, None, 1)
            lib.llmk_matmul_forward(G.ptr(act), G.ptr(x), G.ptr(w), G.ptr(b), 1, M, C, OC, None, G.ptr(pre), 2)
            dinp = torch.full((M, C), 3.0, dtype=torch.bfloat16, device="cuda")
            dw = torch.zeros((OC, C), dtype=torch.bfloat16, device="cuda")
            lib.llmk_matmul_backward(G.ptr(dinp), G.ptr(dw), None, G.ptr(out), G.ptr(x), G.ptr(w), None, 1, M, C, OC, None, None, 1)
            G.sync()
            outs.append((out, pre, act, dinp, dw))
        for a, c, what in zip(outs[0], outs[1], ("forward", "pre-activation", "activation", "dinp", "dweight")):
            assert torch.isfinite(a.float()).all()
            assert torch.equal(a, c), (C, OC, what)
    G.check_no_error(L)
    assert V.llmk_last_error() in (None, b"")
