"""Per-kernel parity: every entry point of include/llmk.h, called through the C ABI on the GPU,
against the CPU oracle (oracle/cpu_ref.c) on the same seeded inputs.

fp32 library: tolerances of the reference's own kernel harness (dev/cuda/*.cu, 1e-5 .. 1e-3).
bf16 library: the oracle is fed the bf16-rounded inputs; outputs may differ by bf16 rounding of the
result (relative 2^-8) plus fp32 accumulation-order noise.
"""
import ctypes as CT

import numpy as np
import pytest

import gpu_lib as G
import oracle_lib as ol

pytestmark = pytest.mark.gpu

PRECS = ["fp32", "bf16"]


def rnd(shape, seed, scale=1.0):
    return (np.random.RandomState(seed).standard_normal(shape) * scale).astype(np.float32)


def tol(precision, fp32_atol, bf16_rel=1.0 / 128, bf16_atol=None):
    if precision == "fp32":
        return dict(rtol=3e-5, atol=fp32_atol)
    return dict(rtol=bf16_rel, atol=bf16_atol if bf16_atol is not None else fp32_atol)


def rel_fro(actual, desired):
    a, d = np.asarray(actual, np.float64), np.asarray(desired, np.float64)
    return float(np.linalg.norm((a - d).ravel()) / max(np.linalg.norm(d.ravel()), 1e-30))


def close(actual, desired, rtol, atol, what=""):
    np.testing.assert_allclose(actual, desired, rtol=rtol, atol=atol, err_msg=what)


@pytest.fixture(scope="module", autouse=True)
def _cuda():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    yield
    torch.cuda.synchronize()


# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("B,T,C,V", [(2, 8, 64, 100), (4, 64, 768, 50257)])
def test_encoder_forward(precision, B, T, C, V):
    L = G.lib(precision)
    wte, wpe = G.rounded(rnd((V, C), 0), precision), G.rounded(rnd((T, C), 1), precision)
    inp = np.random.RandomState(2).randint(0, V, B * T).astype(np.int32)
    ref = np.zeros((B, T, C), np.float32)
    ol.cref().cref_encoder_forward(ref, inp, wte, wpe, B, T, C)
    d_out = G.dev(np.zeros((B, T, C), np.float32), precision)
    d_wte, d_wpe, d_inp = G.dev(wte, precision), G.dev(wpe, precision), G.dev(inp)
    L.llmk_encoder_forward(G.ptr(d_out), G.ptr(d_inp), G.ptr(d_wte), G.ptr(d_wpe), B, T, C, None)
    close(G.host(d_out), ref, **tol(precision, 1e-6, bf16_atol=1e-2))


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("B,T,C,V", [(2, 16, 64, 20), (8, 256, 768, 300), (3, 32, 1600, 50)])
def test_encoder_backward(precision, B, T, C, V):
    L = G.lib(precision)
    N = B * T
    rs = np.random.RandomState(3)
    inp = rs.randint(0, V, N).astype(np.int32)
    inp[rs.rand(N) < 0.3] = 7                       # one very frequent token: long bucket, all four waves busy
    dout = G.rounded(rnd((B, T, C), 4), precision)
    dwte0, dwpe0 = G.rounded(rnd((V, C), 5), precision), G.rounded(rnd((T, C), 6), precision)
    rwte, rwpe = dwte0.copy(), dwpe0.copy()
    ol.cref().cref_encoder_backward(rwte, rwpe, dout, inp, B, T, C)
    vn = 8 if precision == "bf16" else 4
    ncg = -(-C // (64 * vn))
    import torch
    scratch = torch.zeros(N * ncg * 20 + 64, dtype=torch.uint8, device="cuda")
    wl = np.zeros(N * ncg, np.int32); bk = np.zeros(4 * N * ncg, np.int32)
    d_wte, d_wpe, d_dout, d_inp = G.dev(dwte0, precision), G.dev(dwpe0, precision), G.dev(dout, precision), G.dev(inp)
    L.llmk_encoder_backward(G.ptr(d_wte), G.ptr(d_wpe), G.ptr(scratch), wl.ctypes.data_as(CT.c_void_p),
                            bk.ctypes.data_as(CT.c_void_p), G.ptr(d_dout), G.ptr(d_inp), inp.ctypes.data_as(CT.c_void_p),
                            B, T, C, 1234, None)
    # stochastic rounding lands on one of the two bf16 neighbours of the exact sum: 1 ulp = 2^-7 relative
    close(G.host(d_wte), rwte, **tol(precision, 1e-4, bf16_rel=1.0 / 64, bf16_atol=2e-2), what="dwte")
    close(G.host(d_wpe), rwpe, **tol(precision, 1e-4, bf16_rel=1.0 / 64, bf16_atol=2e-2), what="dwpe")
    # determinism: same call, same bits
    d_wte2, d_wpe2 = G.dev(dwte0, precision), G.dev(dwpe0, precision)
    L.llmk_encoder_backward(G.ptr(d_wte2), G.ptr(d_wpe2), G.ptr(scratch), wl.ctypes.data_as(CT.c_void_p),
                            bk.ctypes.data_as(CT.c_void_p), G.ptr(d_dout), G.ptr(d_inp), inp.ctypes.data_as(CT.c_void_p),
                            B, T, C, 1234, None)
    G.sync()
    assert torch.equal(d_wte, d_wte2) and torch.equal(d_wpe, d_wpe2)


# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("N,C", [(7, 64), (1024, 768), (300, 1600), (16, 4104)])
def test_layernorm_forward_and_fused_residual(precision, N, C):
    L = G.lib(precision)
    x, y = G.rounded(rnd((N, C), 0, 2.0) + 0.5, precision), G.rounded(rnd((N, C), 1), precision)
    w, b = G.rounded(rnd(C, 2), precision), G.rounded(rnd(C, 3), precision)
    ro = np.zeros((N, C), np.float32); rm = np.zeros(N, np.float32); rr = np.zeros(N, np.float32)
    ol.cref().cref_layernorm_forward(ro, rm.ctypes.data, rr.ctypes.data, x, w, b, N, C)
    d_o = G.dev(np.zeros((N, C), np.float32), precision)
    d_m, d_r = G.dev(np.zeros(N, np.float32)), G.dev(np.zeros(N, np.float32))
    d_x, d_y, d_w, d_b = (G.dev(a, precision) for a in (x, y, w, b))
    L.llmk_layernorm_forward(G.ptr(d_o), G.ptr(d_m), G.ptr(d_r), G.ptr(d_x), G.ptr(d_w), G.ptr(d_b), 1, N, C, None)
    close(G.host(d_m), rm, rtol=1e-5, atol=1e-5, what="mean")
    close(G.host(d_r), rr, rtol=2e-5, atol=1e-6, what="rstd")
    close(G.host(d_o), ro, **tol(precision, 2e-5, bf16_atol=2e-2), what="out")      # dev/cuda/layernorm_forward.cu:590
    # mean/rstd are optional
    d_o2 = G.dev(np.zeros((N, C), np.float32), precision)
    L.llmk_layernorm_forward(G.ptr(d_o2), None, None, G.ptr(d_x), G.ptr(d_w), G.ptr(d_b), 1, N, C, None)
    import torch
    G.sync()
    assert torch.equal(d_o, d_o2)
    # fused residual: residual = round(x + y), statistics of the rounded sum
    res = G.rounded(x + y, precision)
    ol.cref().cref_layernorm_forward(ro, rm.ctypes.data, rr.ctypes.data, res, w, b, N, C)
    d_res = G.dev(np.zeros((N, C), np.float32), precision)
    L.llmk_fused_residual_forward5(G.ptr(d_res), G.ptr(d_o), G.ptr(d_m), G.ptr(d_r), G.ptr(d_x), G.ptr(d_y), G.ptr(d_w),
                                   G.ptr(d_b), N, C, None)
    np.testing.assert_array_equal(G.host(d_res), res)
    close(G.host(d_m), rm, rtol=1e-5, atol=1e-5)
    close(G.host(d_o), ro, **tol(precision, 2e-5, bf16_atol=2e-2))
    # plain residual add
    d_sum = G.dev(np.zeros((N, C), np.float32), precision)
    L.llmk_residual_forward(G.ptr(d_sum), G.ptr(d_x), G.ptr(d_y), N * C, None)
    np.testing.assert_array_equal(G.host(d_sum), res)
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("N,C", [(9, 64), (2048, 768), (520, 1600), (300, 1024), (45, 2048), (70, 2560), (37, 4096),
                                 (300, 5120), (19, 12288)])      # past 8 vectors per lane: the workgroup-per-row kernel
def test_layernorm_backward(precision, N, C):
    L = G.lib(precision)
    x, g = G.rounded(rnd((N, C), 0, 1.5), precision), G.rounded(rnd((N, C), 1), precision)
    w = G.rounded(rnd(C, 2), precision)
    rm = np.zeros(N, np.float32); rr = np.zeros(N, np.float32); tmp = np.zeros((N, C), np.float32)
    ol.cref().cref_layernorm_forward(tmp, rm.ctypes.data, rr.ctypes.data, x, w, np.zeros(C, np.float32), N, C)
    dx0, dw0, db0 = G.rounded(rnd((N, C), 3), precision), G.rounded(rnd(C, 4), precision), G.rounded(rnd(C, 5), precision)
    rdx, rdw, rdb = dx0.copy(), dw0.copy(), db0.copy()
    ol.cref().cref_layernorm_backward(rdx, rdw, rdb, g, x, w, rm, rr, N, C)
    d_dx, d_dw, d_db = G.dev(dx0, precision), G.dev(dw0, precision), G.dev(db0, precision)
    d_g, d_x, d_w = G.dev(g, precision), G.dev(x, precision), G.dev(w, precision)
    d_m, d_r = G.dev(rm), G.dev(rr)
    import torch
    scratch = torch.empty(L.llmk_layernorm_backward_scratch_floats(C), dtype=torch.float32, device="cuda")
    L.llmk_layernorm_backward(G.ptr(d_dx), G.ptr(d_dw), G.ptr(d_db), G.ptr(scratch), G.ptr(d_g), G.ptr(d_x), G.ptr(d_w),
                              G.ptr(d_m), G.ptr(d_r), 1, N, C, None)
    # dev/cuda/layernorm_backward.cu:1506-1507: dinp 1e-3 / 1e-1, dweight/dbias 1e-3 / 5e-1
    close(G.host(d_dx), rdx, **tol(precision, 1e-4, bf16_atol=5e-2), what="dinp")
    s = np.sqrt(N)
    close(G.host(d_dw), rdw, **tol(precision, 1e-4 * s, bf16_rel=1.0 / 64, bf16_atol=1e-2 * s), what="dweight")
    close(G.host(d_db), rdb, **tol(precision, 1e-4 * s, bf16_rel=1.0 / 64, bf16_atol=1e-2 * s), what="dbias")
    G.check_no_error(L)


# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("precision", PRECS)
def test_gelu(precision):
    L = G.lib(precision)
    n = 8 * 1024 + 64
    x = G.rounded(np.concatenate([rnd(n - 8, 0, 3.0), np.array([0, -0.0, 20, -20, 1e-3, 5, -5, 0.5], np.float32)]), precision)
    g = G.rounded(rnd(n, 1), precision)
    ro = np.zeros(n, np.float32); ol.cref().cref_gelu_forward(ro, x, n)
    d_x, d_o = G.dev(x, precision), G.dev(np.zeros(n, np.float32), precision)
    L.llmk_gelu_forward(G.ptr(d_o), G.ptr(d_x), n, None)
    close(G.host(d_o), ro, **tol(precision, 1e-5, bf16_atol=1e-2))                # dev/cuda/gelu_forward.cu
    rd = np.zeros(n, np.float32); ol.cref().cref_gelu_backward(rd, x, g, n)
    d_g = G.dev(g, precision)
    L.llmk_gelu_backward_inplace(G.ptr(d_g), G.ptr(d_x), n, None)
    close(G.host(d_g), rd, **tol(precision, 1e-5, bf16_atol=1e-2))


@pytest.mark.parametrize("offset,nbytes", [(0, 0), (0, 16), (3, 5), (5, 11), (1, 64), (16, 4096), (7, 100003), (0, 50 * 1024 * 1024 + 9)])
def test_zero_touches_exactly_its_range(offset, nbytes):
    # any alignment and size: head and tail bytes around the 16-byte store kernel, neighbours left alone
    L = G.lib("bf16")
    total = offset + nbytes + 64
    base = (np.arange(total) % 251 + 1).astype(np.uint8)
    d = G.dev(base)
    L.llmk_zero(CT.c_void_p(d.data_ptr() + offset), nbytes, None)
    want = base.copy(); want[offset:offset + nbytes] = 0
    np.testing.assert_array_equal(G.host(d), want)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("N,OC", [(37, 64), (300, 3072), (2048, 264)])
def test_gelu_backward_bias_equals_the_two_separate_steps(precision, N, OC):
    """d *= gelu'(x) and dbias += colsum(d) in one pass: the GELU part against the oracle, the bias part against
    what llmk_matmul_backward's bias step gives on the stored result (same summation order: bit-identical in bf16)."""
    L = G.lib(precision)
    x = G.rounded(rnd((N, OC), 0, 2.0), precision)
    g = G.rounded(rnd((N, OC), 1), precision)
    b0 = G.rounded(rnd(OC, 2), precision)
    rd = np.zeros((N, OC), np.float32); ol.cref().cref_gelu_backward(rd, x, g, N * OC)
    nscr = L.llmk_matmul_backward_bias_scratch_floats(OC)
    d_x, d_g, d_b = G.dev(x, precision), G.dev(g, precision), G.dev(b0, precision)
    d_s = G.dev(np.zeros(nscr, np.float32), "fp32")
    L.llmk_gelu_backward_bias(G.ptr(d_g), G.ptr(d_x), G.ptr(d_b), G.ptr(d_s), 1, N, OC, None)
    got_d, got_b = G.host(d_g), G.host(d_b)
    close(got_d, rd, **tol(precision, 1e-5, bf16_atol=1e-2))
    # the two-step path: same elementwise kernel semantics, then the library's own bias reduction on that result
    d_g2, d_b2 = G.dev(g, precision), G.dev(b0, precision)
    L.llmk_gelu_backward_inplace(G.ptr(d_g2), G.ptr(d_x), N * OC, None)
    assert np.array_equal(G.host(d_g2), got_d)
    C_in = 8
    d_inp = G.dev(np.zeros((N, C_in), np.float32), precision); d_w = G.dev(np.zeros((OC, C_in), np.float32), precision)
    d_dinp = G.dev(np.zeros((N, C_in), np.float32), precision); d_dw = G.dev(np.zeros((OC, C_in), np.float32), precision)
    L.llmk_matmul_backward(G.ptr(d_dinp), G.ptr(d_dw), G.ptr(d_b2), G.ptr(d_g2), G.ptr(d_inp), G.ptr(d_w), G.ptr(d_s),
                           1, N, C_in, OC, None, None, 1)
    if precision == "bf16":
        assert np.array_equal(G.host(d_b2), got_b)
    else:                                   # fp32 storage: no rounding between product and sum, the compiler may fuse them
        close(got_b, G.host(d_b2), rtol=1e-5, atol=1e-5)
    # and against a float64 column sum
    ref_b = b0.astype(np.float64) + got_d.astype(np.float64).sum(0)
    close(got_b, ref_b.astype(np.float32), **tol(precision, 1e-4, bf16_rel=1e-2, bf16_atol=2e-2))


# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("N,V,P", [(5, 100, 128), (64, 50257, 50304), (3, 8003, 8064), (2, 130000, 130048),
                                   (3, 20000, 20032), (2, 55003, 55040), (2, 28001, 28032)])   # one shape per kernel variant
def test_fused_classifier(precision, N, V, P):
    L = G.lib(precision)
    z = rnd((N, P), 0, 2.0)
    rs = np.random.RandomState(1)
    for r in range(N):                                   # a few outliers per row (dev/cuda/classifier_fused.cu:689-696)
        z[r, rs.randint(0, V, 3)] *= 20
    z = G.rounded(z, precision)
    tg = rs.randint(0, V, N).astype(np.int32); tg[0] = V - 1
    probs = np.zeros((N, P), np.float32); rl = np.zeros(N, np.float32)
    ol.cref().cref_softmax_crossentropy_forward(probs, rl.ctypes.data, z, tg.ctypes.data, N, V, P)
    dloss = 1.0 / N
    rd = np.zeros((N, P), np.float32)
    ol.cref().cref_crossentropy_softmax_backward(rd, probs, tg, dloss, N, V, P)
    rd[:, V:] = z[:, V:]                                  # padded columns keep their logit values
    base = rnd(N, 5)
    d_z, d_l, d_t = G.dev(z, precision), G.dev(base.copy()), G.dev(tg)
    # losses only
    L.llmk_fused_classifier(G.ptr(d_z), G.ptr(d_l), dloss, G.ptr(d_t), 1, N, V, P, 0, None)
    close(G.host(d_l), base + rl, rtol=1e-5, atol=1e-4, what="losses accumulate")
    np.testing.assert_array_equal(G.host(d_z), z)
    # losses + dlogits in place
    d_l = G.dev(np.zeros(N, np.float32))
    L.llmk_fused_classifier(G.ptr(d_z), G.ptr(d_l), dloss, G.ptr(d_t), 1, N, V, P, 1, None)
    close(G.host(d_l), rl, rtol=1e-5, atol=1e-4)                                  # classifier_fused.cu:739
    out = G.host(d_z)
    # the oracle adds its 50k exponentials one after the other in fp32 (train_gpt2.c:468-472), which costs it up to
    # ~1e-4 relative; a float64 softmax shows which side is exact: oracle within 1e-3 of it, GPU within 2e-5
    z64 = z[:, :V].astype(np.float64)
    p64 = np.exp(z64 - z64.max(1, keepdims=True)); p64 /= p64.sum(1, keepdims=True)
    p64[np.arange(N), tg] -= 1.0
    close(rd[:, :V], p64 * dloss, rtol=1e-3, atol=1e-7, what="oracle vs float64")
    close(out[:, :V], p64 * dloss, **tol(precision, 1e-7, bf16_rel=1.0 / 64, bf16_atol=1e-5), what="dlogits")
    if precision == "fp32":
        close(out[:, :V], p64 * dloss, rtol=3e-5, atol=1e-7, what="dlogits vs float64")
    np.testing.assert_array_equal(out[:, V:], z[:, V:])
    G.check_no_error(L)


# ------------------------------------------------------------------------------------------------
def run_matmul_forward(L, precision, x, w, b, pre_gelu, fusion):
    M, Cc = x.shape
    OC = w.shape[0]
    d_x, d_w = G.dev(x, precision), G.dev(w, precision)
    d_b = G.dev(b, precision) if b is not None else None
    d_o = G.dev(np.zeros((M, OC), np.float32), precision)
    d_pre = G.dev(np.zeros((M, OC), np.float32), precision) if pre_gelu else None
    L.llmk_matmul_forward(G.ptr(d_o), G.ptr(d_x), G.ptr(d_w), G.ptr(d_b), 1, M, Cc, OC, None, G.ptr(d_pre), fusion)
    return G.host(d_o), (G.host(d_pre) if pre_gelu else None)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("M,Cc,OC,bias", [(64, 64, 64, True), (200, 72, 136, True), (256, 768, 2304, True),
                                           (512, 3072, 768, True), (128, 768, 50304, False),
                                           (4096, 256, 4096, True), (4100, 192, 4360, False),
                                           (4096, 1600, 4800, True),       # GPT-2 1558M qkv: 25 K stages, ragged N
                                           (32768, 768, 2304, True)])      # enough row panels for the XCD-private work list
def test_matmul_forward(precision, M, Cc, OC, bias):
    L = G.lib(precision)
    x, w = G.rounded(rnd((M, Cc), 0), precision), G.rounded(rnd((OC, Cc), 1, 0.1), precision)
    b = G.rounded(rnd(OC, 2), precision) if bias else None
    ref = x.astype(np.float64) @ w.astype(np.float64).T + (b if bias else 0)
    if M * Cc * OC <= 256 * 768 * 2304:                  # the oracle's loops, where they finish quickly
        r2 = np.zeros((M, OC), np.float32)
        ol.cref().cref_matmul_forward(r2, x, w, b.ctypes.data if bias else None, M, Cc, OC)
        close(r2, ref, rtol=1e-4, atol=1e-4)
    out, _ = run_matmul_forward(L, precision, x, w, b, False, 1)
    sc = np.sqrt(Cc) * 0.1
    close(out, ref, **tol(precision, 2e-5 * sc, bf16_atol=1e-2 * sc))
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("fusion", [0, 1])
@pytest.mark.parametrize("M,Cc,OC", [(192, 128, 512), (4096, 128, 4096)])
def test_matmul_forward_gelu(precision, fusion, M, Cc, OC):
    L = G.lib(precision)
    x, w, b = G.rounded(rnd((M, Cc), 0), precision), G.rounded(rnd((OC, Cc), 1, 0.1), precision), G.rounded(rnd(OC, 2), precision)
    pre = (x.astype(np.float64) @ w.astype(np.float64).T + b).astype(np.float32)
    out, got_pre = run_matmul_forward(L, precision, x, w, b, True, fusion)
    close(got_pre, pre, **tol(precision, 5e-5, bf16_atol=2e-2), what="pre_gelu")
    ref = np.zeros_like(got_pre)
    ol.cref().cref_gelu_forward(ref.reshape(-1), np.ascontiguousarray(got_pre).reshape(-1), got_pre.size)
    close(out, ref, **tol(precision, 1e-5, bf16_atol=1e-2), what="gelu(pre_gelu)")


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("M,Cc,OC,bias", [(64, 64, 64, True), (200, 72, 136, True), (256, 768, 2304, True),
                                           (1024, 3072, 768, True), (8192, 768, 768, True), (4096, 2048, 2048, False),
                                           (128, 256, 50304, False),
                                           (32768, 768, 768, True),        # dinp on the 256x256 kernel with XCD-private row panels
                                           (2048, 1600, 6400, True),       # GPT-2 1558M fc
                                           (4096, 1600, 1600, True),       # odd number of 64-wide K stages in dinp
                                           (16384, 832, 1600, False),      # odd stage counts on the 256x256 kernel
                                           (1024, 256, 384, True),         # bias gradient inside the dweight GEMM, 128x128 tiles
                                           (1024, 192, 136, True),         # ... with output rows past the matrix edge
                                           (4096, 768, 2440, True)])       # ... 256x256 tiles with a ragged last row of tiles
def test_matmul_backward(precision, M, Cc, OC, bias):
    L = G.lib(precision)
    x, w = G.rounded(rnd((M, Cc), 0), precision), G.rounded(rnd((OC, Cc), 1, 0.1), precision)
    g = G.rounded(rnd((M, OC), 2), precision)
    dw0, db0 = G.rounded(rnd((OC, Cc), 3), precision), G.rounded(rnd(OC, 4), precision)
    g64 = g.astype(np.float64)
    r_dx = g64 @ w.astype(np.float64)
    r_dw = dw0 + g64.T @ x.astype(np.float64)
    r_db = db0 + g64.sum(0)
    if M * Cc * OC <= 256 * 768 * 2304:
        c_dx = np.zeros((M, Cc), np.float32); c_dw = dw0.copy(); c_db = db0.copy()
        ol.cref().cref_matmul_backward(c_dx.ctypes.data, c_dw, c_db.ctypes.data, g, x, w, M, Cc, OC)
        close(c_dx, r_dx, rtol=1e-4, atol=1e-3); close(c_dw, r_dw, rtol=1e-4, atol=1e-3); close(c_db, r_db, rtol=1e-4, atol=1e-3)
    import torch
    d_dx = G.dev(np.full((M, Cc), 7.0, np.float32), precision)        # dinp is overwritten, not accumulated
    d_dw, d_db = G.dev(dw0, precision), (G.dev(db0, precision) if bias else None)
    d_g, d_x, d_w = G.dev(g, precision), G.dev(x, precision), G.dev(w, precision)
    scratch = torch.empty(max(1, L.llmk_matmul_backward_bias_scratch_floats(OC)), dtype=torch.float32, device="cuda")
    L.llmk_matmul_backward(G.ptr(d_dx), G.ptr(d_dw), G.ptr(d_db), G.ptr(d_g), G.ptr(d_x), G.ptr(d_w), G.ptr(scratch),
                           1, M, Cc, OC, None, None, 1)
    close(G.host(d_dx), r_dx, **tol(precision, 3e-5 * np.sqrt(OC), bf16_atol=1e-3 * np.sqrt(OC)), what="dinp")
    close(G.host(d_dw), r_dw, **tol(precision, 3e-5 * np.sqrt(M), bf16_atol=1e-2 * np.sqrt(M)), what="dweight")
    if bias:
        close(G.host(d_db), r_db, **tol(precision, 3e-5 * np.sqrt(M), bf16_atol=1e-2 * np.sqrt(M)), what="dbias")
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("fusion", [0, 2])
@pytest.mark.parametrize("M,Cc,OC", [(320, 512, 128),        # few tiles: GELU backward as a pass of its own
                                     (8192, 2048, 512),      # a tile per CU and more: in the GEMM's epilogue (bf16, fusion 2)
                                     (8448, 2056, 192)])     # ... with ragged last tiles in both directions
def test_matmul_backward_gelu(precision, fusion, M, Cc, OC):
    L = G.lib(precision)                # dinp has the 4C width: (M, Cc) with pre_gelu of the same shape
    x, w = G.rounded(rnd((M, Cc), 0), precision), G.rounded(rnd((OC, Cc), 1, 0.1), precision)
    g, pre = G.rounded(rnd((M, OC), 2), precision), G.rounded(rnd((M, Cc), 3, 2.0), precision)
    lin = G.rounded((g.astype(np.float64) @ w.astype(np.float64)).astype(np.float32), precision)
    ref = np.zeros((M, Cc), np.float32)
    ol.cref().cref_gelu_backward(ref.reshape(-1), pre.reshape(-1), lin.reshape(-1), M * Cc)
    import torch
    d_dx, d_dw = G.dev(np.zeros((M, Cc), np.float32), precision), G.dev(np.zeros((OC, Cc), np.float32), precision)
    d_g, d_x, d_w, d_pre = G.dev(g, precision), G.dev(x, precision), G.dev(w, precision), G.dev(pre, precision)
    L.llmk_matmul_backward(G.ptr(d_dx), G.ptr(d_dw), None, G.ptr(d_g), G.ptr(d_x), G.ptr(d_w), None, 1, M, Cc, OC, None,
                           G.ptr(d_pre), fusion)
    got = G.host(d_dx)
    close(got, ref, **tol(precision, 1e-4, bf16_rel=1.0 / 32, bf16_atol=3e-2))
    # element-wise bounds have to leave room for one bf16 rounding of the largest values; the error of the whole tensor
    # does not: relative Frobenius error of two bf16 roundings (2^-9 each, uniformly spread) is about 2e-3
    assert rel_fro(got, ref) < (1e-5 if precision == "fp32" else 4e-3), rel_fro(got, ref)
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("M,Cc,OC", [(320, 128, 512),        # few tiles: the two halves as passes of their own
                                     (8192, 512, 2048),      # a tile per CU and more: both in GEMM epilogues (bf16)
                                     (8448, 192, 2056)])     # ... with ragged last tiles in both directions
def test_gelu_fusion_3_keeps_the_derivative_for_backward(precision, M, Cc, OC):
    """gelu_fusion 3 (no counterpart in the reference): the forward pass leaves gelu'(pre-activation) where levels 0-2
    leave the pre-activation, and the backward pass multiplies by it. Against the oracle's GELU forward and backward
    (train_gpt2.c:407-433) applied to the pre-activation that level 2 reports: the output to the usual bound (it is
    the same bits as level 2's), the stored derivative to one rounding of the storage type, and dinp of the projection
    that follows (its contraction length is the fc width OC) to the bound of test_matmul_backward_gelu."""
    import torch
    L = G.lib(precision)
    x, w, b = G.rounded(rnd((M, Cc), 0), precision), G.rounded(rnd((OC, Cc), 1, 0.1), precision), G.rounded(rnd(OC, 2), precision)
    out2, pre = run_matmul_forward(L, precision, x, w, b, True, 2)
    out3, grad = run_matmul_forward(L, precision, x, w, b, True, 3)
    assert np.array_equal(out2, out3)
    ones = np.ones(pre.size, np.float32)
    want_grad = np.zeros(pre.size, np.float32)
    ol.cref().cref_gelu_backward(want_grad, np.ascontiguousarray(pre).reshape(-1), ones, pre.size)
    close(grad.reshape(-1), want_grad, **tol(precision, 2e-5, bf16_rel=1.0 / 128, bf16_atol=1e-2), what="stored gelu'")
    # backward of the projection that consumes gelu(pre): dinp (M, OC) = (dout (M, Cc2) . w2 (Cc2, OC)) * gelu'(pre)
    Cc2 = 128
    g, w2 = G.rounded(rnd((M, Cc2), 5), precision), G.rounded(rnd((Cc2, OC), 6, 0.1), precision)
    lin = G.rounded((g.astype(np.float64) @ w2.astype(np.float64)).astype(np.float32), precision)
    ref = np.zeros((M, OC), np.float32)
    ol.cref().cref_gelu_backward(ref.reshape(-1), np.ascontiguousarray(pre).reshape(-1), lin.reshape(-1), M * OC)
    d_dx, d_dw = G.dev(np.zeros((M, OC), np.float32), precision), G.dev(np.zeros((Cc2, OC), np.float32), precision)
    d_g, d_in, d_w2, d_grad = G.dev(g, precision), G.dev(out3, precision), G.dev(w2, precision), G.dev(grad, precision)
    L.llmk_matmul_backward(G.ptr(d_dx), G.ptr(d_dw), None, G.ptr(d_g), G.ptr(d_in), G.ptr(d_w2), None, 1, M, OC, Cc2, None,
                           G.ptr(d_grad), 3)
    got = G.host(d_dx)
    close(got, ref, **tol(precision, 1e-4, bf16_rel=1.0 / 32, bf16_atol=3e-2))
    # three bf16 roundings (the product, the derivative, the result) instead of level 2's two
    assert rel_fro(got, ref) < (1e-5 if precision == "fp32" else 5e-3), rel_fro(got, ref)
    G.check_no_error(L)


# ------------------------------------------------------------------------------------------------
def attention_case(precision, B, T, NH, seed=0, hs=64):
    Cc = NH * hs
    qkv = G.rounded(rnd((B, T, 3 * Cc), seed, 1.0), precision)
    g = G.rounded(rnd((B, T, Cc), seed + 1), precision)
    o = np.zeros((B, T, Cc), np.float32); lse = np.zeros((B, NH, T), np.float32)
    ol.cref().cref_attention_forward(o, None, lse.ctypes.data, qkv, B, T, Cc, NH)
    d = np.zeros((B, T, 3 * Cc), np.float32)
    ol.cref().cref_attention_backward(d, g, qkv, None, B, T, Cc, NH)
    return qkv, g, o, lse, d, Cc


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("B,T,NH", [(2, 64, 2), (1, 128, 3), (2, 200, 2), (1, 1, 2), (1, 1024, 2), (2, 384, 12), (4, 192, 2), (1, 320, 3)])
def test_attention_forward_backward(precision, B, T, NH):
    L = G.lib(precision)
    qkv, g, ro, rlse, rd, Cc = attention_case(precision, B, T, NH)
    d_qkv, d_g = G.dev(qkv, precision), G.dev(g, precision)
    d_o = G.dev(np.zeros((B, T, Cc), np.float32), precision)
    d_lse = G.dev(np.zeros((B, NH, T), np.float32))
    L.llmk_attention_forward(G.ptr(d_o), G.ptr(d_lse), G.ptr(d_qkv), B, T, NH, Cc, None)
    close(G.host(d_o), ro, **tol(precision, 1e-5, bf16_atol=2e-2), what="out")        # dev/cuda/attention_forward.cu:1330
    close(G.host(d_lse), rlse, rtol=1e-5, atol=(1e-4 if precision == "fp32" else 2e-2), what="stats")
    # inference mode: no statistics
    d_o2 = G.dev(np.zeros((B, T, Cc), np.float32), precision)
    L.llmk_attention_forward(G.ptr(d_o2), None, G.ptr(d_qkv), B, T, NH, Cc, None)
    import torch
    G.sync()
    assert torch.equal(d_o, d_o2)
    d_d = G.dev(np.full((B, T, 3 * Cc), 3.0, np.float32), precision)                  # overwritten, not accumulated
    L.llmk_attention_backward(G.ptr(d_d), G.ptr(d_g), G.ptr(d_qkv), G.ptr(d_o), G.ptr(d_lse), B, T, NH, Cc, None)
    scale = np.abs(rd).max()
    got = G.host(d_d)
    close(got, rd, **tol(precision, 1e-4 * scale, bf16_rel=1.0 / 32, bf16_atol=2e-2 * scale), what="dqkv")
    for i, name in enumerate(("dQ", "dK", "dV")):          # per gradient, over the whole tensor: bf16 operands and probabilities
        a, r = got[..., i * Cc:(i + 1) * Cc], rd[..., i * Cc:(i + 1) * Cc]
        joint = np.linalg.norm(rd.ravel())
        if np.linalg.norm(r.ravel()) < 1e-3 * joint:
            # T = 1: one key, probability 1, so dS = P (dP - D) is mathematically 0 and so are dQ and dK. The kernels
            # form dP - D from two fp32 sums of the same 64 products taken in different orders, which leaves a
            # rounding residue (1e-7 of the joint norm measured in fp32) instead of an exact zero; the oracle's loop
            # (train_gpt2.c:347-405) gives exact zeros. Held to: no more than fp32 / bf16 rounding of the joint norm.
            e = float(np.linalg.norm((a - r).ravel()) / joint)
            assert e < (1e-6 if precision == "fp32" else 2e-3), (name, "vanishing gradient", e)
            continue
        e = float(np.linalg.norm((a - r).ravel()) / np.linalg.norm(r.ravel()))
        assert e < (2e-5 if precision == "fp32" else 1e-2), (name, e)
    # causality at the kernel level: future tokens do not change earlier outputs
    if T >= 64:
        q2 = qkv.copy(); q2[:, T // 2:] += 1.0
        d_q2 = G.dev(G.rounded(q2, precision), precision)
        L.llmk_attention_forward(G.ptr(d_o2), None, G.ptr(d_q2), B, T, NH, Cc, None)
        G.sync()
        assert torch.equal(d_o[:, :T // 2], d_o2[:, :T // 2])
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("B,T,NH", [(2, 128, 3), (1, 200, 2)])
def test_attention_fallback_launchers(precision, B, T, NH):
    """The launcher pair of reference builds without cuDNN (llmc/attention.cuh:195, :239), in its argument order: same
    bits as the flash pair, from the buffers that signature provides (qkvr, att, scratch), against the oracle."""
    import torch
    L = G.lib(precision)
    dt = G.torch_dtype(precision)
    qkv, g, ro, rlse, rd, Cc = attention_case(precision, B, T, NH, seed=7)
    d_inp, d_g = G.dev(qkv, precision), G.dev(g, precision)
    d_o, d_stats = torch.zeros((B, T, Cc), dtype=dt, device="cuda"), torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
    L.llmk_attention_forward(G.ptr(d_o), G.ptr(d_stats), G.ptr(d_inp), B, T, NH, Cc, None)
    d_want = torch.zeros((B, T, 3 * Cc), dtype=dt, device="cuda")
    L.llmk_attention_backward(G.ptr(d_want), G.ptr(d_g), G.ptr(d_inp), G.ptr(d_o), G.ptr(d_stats), B, T, NH, Cc, None)
    d_qkvr = torch.zeros((B, T, 3 * Cc), dtype=dt, device="cuda")
    d_att = torch.full((B, NH, T, T), 9.0, dtype=dt, device="cuda")
    d_o2 = torch.zeros((B, T, Cc), dtype=dt, device="cuda")
    inp_copy = d_inp.clone()
    L.llmk_attention_forward_fallback(G.ptr(d_o2), G.ptr(d_qkvr), G.ptr(d_att), G.ptr(inp_copy), B, T, Cc, NH, None)
    inp_copy.fill_(5.0)                                     # the reference's driver reuses this buffer right away
    d_dinp = torch.full((B, T, 3 * Cc), 3.0, dtype=dt, device="cuda")
    d_dqkvr, d_datt = torch.zeros_like(d_qkvr), torch.zeros_like(d_att)
    d_scratch = torch.full((B, T, Cc), 7.0, dtype=dt, device="cuda")
    L.llmk_attention_backward_fallback(G.ptr(d_dinp), G.ptr(d_dqkvr), G.ptr(d_datt), G.ptr(d_scratch), G.ptr(d_g), G.ptr(d_qkvr),
                                       G.ptr(d_att), B, T, Cc, NH, None)
    G.sync()
    assert torch.equal(d_o2, d_o) and torch.equal(d_dinp, d_want)
    close(G.host(d_o2), ro, **tol(precision, 1e-5, bf16_atol=2e-2), what="out")
    scale = np.abs(rd).max()
    close(G.host(d_dinp), rd, **tol(precision, 1e-4 * scale, bf16_rel=1.0 / 32, bf16_atol=2e-2 * scale), what="dinp")
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("hs", [32, 80, 96, 128])
@pytest.mark.parametrize("B,T,NH", [(2, 96, 2), (1, 130, 3)])
def test_attention_other_head_sizes(precision, hs, B, T, NH):
    """Head sizes of the GPT-3 descriptors (train_gpt2.cu:538-559) and a small one: the one-wave-per-row kernels."""
    L = G.lib(precision)
    qkv, g, ro, rlse, rd, Cc = attention_case(precision, B, T, NH, seed=hs, hs=hs)
    d_qkv, d_g = G.dev(qkv, precision), G.dev(g, precision)
    d_o = G.dev(np.zeros((B, T, Cc), np.float32), precision)
    d_lse = G.dev(np.zeros((B, NH, T), np.float32))
    L.llmk_attention_forward(G.ptr(d_o), G.ptr(d_lse), G.ptr(d_qkv), B, T, NH, Cc, None)
    close(G.host(d_o), ro, **tol(precision, 1e-5, bf16_atol=2e-2), what="out")
    close(G.host(d_lse), rlse, rtol=1e-5, atol=1e-4, what="stats")                  # fp32 arithmetic in both builds
    d_d = G.dev(np.full((B, T, 3 * Cc), 3.0, np.float32), precision)
    L.llmk_attention_backward(G.ptr(d_d), G.ptr(d_g), G.ptr(d_qkv), G.ptr(d_o), G.ptr(d_lse), B, T, NH, Cc, None)
    scale = np.abs(rd).max()
    close(G.host(d_d), rd, **tol(precision, 1e-4 * scale, bf16_rel=1.0 / 32, bf16_atol=2e-2 * scale), what="dqkv")
    G.check_no_error(L)


# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("use_master", [True, False])
def test_adamw_update_multi_is_the_per_tensor_update(precision, use_master):
    """Sixteen tensors in one launch against sixteen launches: the same bits in every arena, including the noise words
    of the stochastic rounding (per slice, per element index inside the slice)."""
    import torch
    L = G.lib(precision)
    rs = np.random.RandomState(5)
    sizes = [int(x) * 8 for x in rs.randint(1, 700, 16)]
    sizes[0], sizes[5] = 300000, 8                         # one large tensor, one of a single vector
    slices = [1, 1] + [int(x) for x in rs.randint(1, 5, 12)] + [1, 1]
    wds = [0.1 if i in (0, 1, 4, 6, 10, 12) else 0.0 for i in range(16)]
    seeds = [int(x) for x in rs.randint(0, 2 ** 31, 16)]
    offsets = np.cumsum([0] + [sz * sl for sz, sl in zip(sizes, slices)])
    tot = int(offsets[-1])
    p0 = G.rounded(rnd(tot, 0, 0.05), precision); g = G.rounded(rnd(tot, 1, 0.01), precision)
    m0, v0 = rnd(tot, 2, 0.01), np.abs(rnd(tot, 3, 1e-4))
    master0 = (p0 + rnd(tot, 4, 1e-4)).astype(np.float32) if use_master else None
    hp = (1e-3, 0.9, 0.95, 3, 1e-8)
    gs = 0.5
    X = 2 if precision == "bf16" else 4

    def arenas():
        return [G.dev(p0, precision), (G.dev(master0) if use_master else None), G.dev(g, precision), G.dev(m0), G.dev(v0)]

    a = arenas()
    for i in range(16):
        o = int(offsets[i])
        ptrs = [None if t is None else CT.c_void_p(t.data_ptr() + o * (X if k in (0, 2) else 4)) for k, t in enumerate(a)]
        L.llmk_adamw_update(ptrs[0], ptrs[1], ptrs[2], ptrs[3], ptrs[4], sizes[i], sizes[i], sizes[i], sizes[i], slices[i],
                            hp[0], hp[1], hp[2], hp[3], hp[4], wds[i], gs, seeds[i], None)
    b = arenas()
    off_a, size_a = np.array(offsets[:16], np.uint64), np.array(sizes, np.uint64)
    sl_a, wd_a, seed_a = np.array(slices, np.int32), np.array(wds, np.float32), np.array(seeds, np.uint32)
    vp = lambda x: x.ctypes.data_as(CT.c_void_p)
    ran = L.llmk_adamw_update_multi(G.ptr(b[0]), G.ptr(b[1]), G.ptr(b[2]), G.ptr(b[3]), G.ptr(b[4]), 16, vp(off_a), vp(size_a),
                                    vp(sl_a), vp(wd_a), vp(seed_a), hp[0], hp[1], hp[2], hp[3], hp[4], gs, None)
    assert ran == 1
    G.sync()
    for x, y in zip(a, b):
        if x is not None:
            assert torch.equal(x, y)
    assert not torch.equal(a[0], G.dev(p0, precision))     # and something happened
    # tensors the single launch cannot take are refused, not mangled
    size_a[3] += 1
    assert L.llmk_adamw_update_multi(G.ptr(b[0]), G.ptr(b[1]), G.ptr(b[2]), G.ptr(b[3]), G.ptr(b[4]), 16, vp(off_a), vp(size_a),
                                     vp(sl_a), vp(wd_a), vp(seed_a), hp[0], hp[1], hp[2], hp[3], hp[4], gs, None) == 0
    G.sync()
    assert torch.equal(a[0], b[0])
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("use_master", [True, False])
def test_adamw_update(precision, use_master):
    L = G.lib(precision)
    n, slices, stride = 5000 * 8, 3, 5000 * 8 + 64
    tot = stride * slices
    p0 = G.rounded(rnd(tot, 0, 0.05), precision); g = G.rounded(rnd(tot, 1, 0.01), precision)
    m0, v0 = rnd(tot, 2, 0.01), np.abs(rnd(tot, 3, 1e-4))
    master0 = p0 + rnd(tot, 4, 1e-4) if use_master else None
    lr, b1, b2, t, eps, wd, gs, seed = 1e-3, 0.9, 0.95, 3, 1e-8, 0.1, 0.5, 42
    rp, rm, rv = p0.copy(), m0.copy(), v0.copy()
    rmaster = master0.copy() if use_master else None
    for s in range(slices):
        sl = slice(s * stride, s * stride + n)
        mm, vv = rm[sl].copy(), rv[sl].copy()
        ms = rmaster[sl].copy() if use_master else None
        if precision == "bf16":
            pb, gb = ol.to_bf16_bits(rp[sl]), ol.to_bf16_bits(g[sl])
            ol.cref().cref_adamw_mixed(pb, ms.ctypes.data if use_master else None, gb, mm, vv, n, lr, b1, b2, t, eps, wd, gs, seed, s)
            rp[sl] = ol.from_bf16_bits(pb)
        else:
            pp = rp[sl].copy()
            ol.cref().cref_adamw_f32(pp, ms.ctypes.data if use_master else None, g[sl].copy(), mm, vv, n, lr, b1, b2, t, eps, wd, gs)
            rp[sl] = pp
        rm[sl], rv[sl] = mm, vv
        if use_master:
            rmaster[sl] = ms
    d_p, d_g, d_m, d_v = G.dev(p0, precision), G.dev(g, precision), G.dev(m0), G.dev(v0)
    d_ms = G.dev(master0) if use_master else None
    L.llmk_adamw_update(G.ptr(d_p), G.ptr(d_ms), G.ptr(d_g), G.ptr(d_m), G.ptr(d_v), n, stride, stride, stride, slices,
                        lr, b1, b2, t, eps, wd, gs, seed, None)
    close(G.host(d_m), rm, rtol=1e-6, atol=1e-9, what="m")
    close(G.host(d_v), rv, rtol=1e-6, atol=1e-12, what="v")
    if use_master:
        close(G.host(d_ms), rmaster, rtol=1e-6, atol=1e-8, what="master")
    got = G.host(d_p)
    if precision == "fp32":
        close(got, rp, rtol=1e-6, atol=1e-8)
    else:
        # the low-precision parameter is the stochastic rounding of the fp32 result with the reference's noise word:
        # bit-exact given the GPU's own fp32 value (master), and equal to the oracle's wherever the fp32 values agree
        if use_master:
            gm = G.host(d_ms)
            for s in range(slices):
                for i in list(range(0, 64)) + list(range(n - 64, n)) + list(np.random.RandomState(s).randint(0, n, 200)):
                    k = s * stride + int(i)
                    want = ol.cref().cref_stochastic_round_bf16(float(gm[k]), ol.cref().cref_adamw_noise(int(i), s, seed))
                    assert ol.to_bf16_bits(got[k:k + 1])[0] == want, (s, i)
        close(got, rp, rtol=1.0 / 128, atol=1e-6)
        assert (got != rp).mean() < 1e-3
    # gaps between slices untouched
    for s in range(slices):
        np.testing.assert_array_equal(got[s * stride + n:(s + 1) * stride], p0[s * stride + n:(s + 1) * stride])
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
def test_adamw_unaligned_tail_and_init_from_master(precision):
    L = G.lib(precision)
    n = 1003                                         # not a multiple of the vector width: scalar path
    p0 = G.rounded(rnd(n, 0, 0.05), precision); g = G.rounded(rnd(n, 1, 0.01), precision)
    d_p, d_g = G.dev(p0, precision), G.dev(g, precision)
    d_m, d_v = G.dev(np.zeros(n, np.float32)), G.dev(np.zeros(n, np.float32))
    d_ms = G.dev(np.zeros(n, np.float32))
    L.llmk_copy_and_cast_to_f32(G.ptr(d_ms), G.ptr(d_p), n, 0, 0, 1, None)
    np.testing.assert_array_equal(G.host(d_ms), p0)
    L.llmk_adamw_update(G.ptr(d_p), G.ptr(d_ms), G.ptr(d_g), G.ptr(d_m), G.ptr(d_v), n, 0, 0, 0, 1,
                        1e-2, 0.9, 0.999, 1, 1e-8, 0.0, 1.0, 7, None)
    # first step from zero state is sign descent: p - lr * g/(|g|+eps)
    want = p0 - 1e-2 * g / (np.abs(g) + 1e-8)
    close(G.host(d_ms), want, rtol=1e-5, atol=1e-7)
    # init_from_master reproduces exactly the parameters the update wrote (same seed => same rounding)
    d_p2 = G.dev(np.zeros(n, np.float32), precision)
    L.llmk_init_from_master(G.ptr(d_p2), G.ptr(d_ms), n, 0, 0, 1, 7, None)
    import torch
    G.sync()
    assert torch.equal(d_p, d_p2)


@pytest.mark.parametrize("precision", PRECS)
def test_global_norm_and_sum(precision):
    L = G.lib(precision)
    import torch
    n, slices, stride = 100003, 4, 100003 + 5
    x = G.rounded(rnd(stride * slices, 0, 1e-3), precision)       # dev/cuda/global_norm.cu scales inputs by 1e-3
    d_x = G.dev(x, precision)
    ns = (CT.c_int * 2)(1, slices)
    mx = L.llmk_get_max_num_block_sums(ns, 2)
    out = torch.full((mx,), 5.0, dtype=torch.float32, device="cuda")
    L.llmk_global_norm_squared(G.ptr(out), G.ptr(d_x), n, stride, slices, mx, 1, None)
    L.llmk_global_norm_squared(G.ptr(out), G.ptr(d_x), 777, 0, 1, mx, 0, None)      # accumulates without reset
    res = torch.zeros(1, dtype=torch.float32, device="cuda")
    L.llmk_global_sum_deterministic(G.ptr(res), G.ptr(out), mx, None)
    want = sum(ol.cref().cref_sum_squares(np.ascontiguousarray(x[s * stride:s * stride + n]), n) for s in range(slices))
    want += ol.cref().cref_sum_squares(np.ascontiguousarray(x[:777]), 777)
    assert abs(G.host(res)[0] - want) <= 1e-5 * want                               # dev/cuda/global_norm.cu: 1e-2
    G.check_no_error(L)


@pytest.mark.parametrize("precision", PRECS)
def test_shape_preconditions_are_reported(precision):
    L = G.lib(precision)
    L.llmk_set_error_mode(1)
    try:
        import torch
        buf = torch.zeros(4096, dtype=G.torch_dtype(precision), device="cuda")
        L.llmk_layernorm_forward(G.ptr(buf), None, None, G.ptr(buf), G.ptr(buf), G.ptr(buf), 1, 2, 67, None)
        assert b"multiple" in L.llmk_last_error()
        L.llmk_clear_error()
        L.llmk_attention_forward(G.ptr(buf), None, G.ptr(buf), 1, 4, 3, 100, None)
        assert L.llmk_last_error() != b""
        L.llmk_clear_error()
        L.llmk_gelu_forward(G.ptr(buf), G.ptr(buf), 0, None)                       # empty input: no-op, no error
        assert L.llmk_last_error() == b""
    finally:
        L.llmk_clear_error()
        L.llmk_set_error_mode(0)
