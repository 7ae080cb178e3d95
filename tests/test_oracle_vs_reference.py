"""Pins the CPU restatement (oracle/cpu_ref.c) against the reference's own compiled code
(oracle/_ref, built from the reference's train_gpt2.c) and against what the mathematics fixes.

Runs without a GPU. Tests that need oracle/_ref skip when that library was not built."""
import ctypes as C
import os
import tempfile

import numpy as np
import pytest

import oracle_lib as ol
from oracle_lib import Config

needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="oracle/_ref not built (reference checkout absent)")

# llmc/rand.h:48-80 — values the reference documents for seed 137 (identical to torch's)
KAT_INTS = [4053805790, 2173880614, 380293709, 1237255315, 2986595568]
KAT_N8 = [0.7947664260864258, 1.4369317293167114, -0.2292192131280899, 0.47556325793266296,
          -0.6334410905838013, -0.5791953802108765, -0.0925704762339592, -0.8659197092056274]
KAT_MID = 2186503452
KAT_N16 = [-1.2813878059387207, -2.646395683288574, -0.06569503247737885, 0.2180829495191574,
           -0.46536165475845337, -0.33108410239219666, 2.5485482215881348, 0.10425379872322083,
           0.8460659980773926, 0.9462448358535767, -0.2913765013217926, 0.34313806891441345,
           -1.1186704635620117, -0.18305328488349915, -2.3153159618377686, 0.3961987793445587]
KAT_LAST = 2756748748


def _kat(fn):
    ints = np.zeros(5, np.uint32); n8 = np.zeros(8, np.float32); mid = np.zeros(1, np.uint32)
    n16 = np.zeros(16, np.float32); last = np.zeros(1, np.uint32)
    fn(137, ints, n8, mid, n16, last)
    return ints, n8, mid[0], n16, last[0]


def test_mt19937_known_answers():
    ints, n8, mid, n16, last = _kat(ol.cref().cref_mt_kat)
    assert list(ints) == KAT_INTS
    assert mid == KAT_MID and last == KAT_LAST
    np.testing.assert_allclose(n8, KAT_N8, rtol=2e-6, atol=1e-7)  # libm vs torch sin/cos: 1-2 ulp
    np.testing.assert_allclose(n16, KAT_N16, rtol=2e-6, atol=1e-7)


@needs_ref
def test_mt19937_matches_compiled_reference():
    a = _kat(ol.cref().cref_mt_kat)
    b = _kat(ol.ref().ref_mt_kat)
    assert list(a[0]) == list(b[0]) and a[2] == b[2] and a[4] == b[4]
    np.testing.assert_allclose(a[1], b[1], rtol=0, atol=1e-7)
    np.testing.assert_allclose(a[3], b[3], rtol=0, atol=1e-7)


def rnd(shape, seed, scale=1.0):
    return (np.random.RandomState(seed).standard_normal(shape) * scale).astype(np.float32)


@needs_ref
@pytest.mark.parametrize("B,T,C", [(2, 5, 48), (1, 8, 768)])
def test_layernorm_fwd_bwd(B, T, C):
    x, w, b, g = rnd((B, T, C), 0), rnd(C, 1), rnd(C, 2), rnd((B, T, C), 3)
    N = B * T
    o1 = np.zeros_like(x); m1 = np.zeros(N, np.float32); r1 = np.zeros(N, np.float32)
    o2 = np.zeros_like(x); m2 = np.zeros(N, np.float32); r2 = np.zeros(N, np.float32)
    ol.cref().cref_layernorm_forward(o1, m1.ctypes.data, r1.ctypes.data, x, w, b, N, C)
    ol.ref().layernorm_forward(o2, m2, r2, x, w, b, B, T, C)
    np.testing.assert_allclose(o1, o2, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(m1, m2, atol=1e-6); np.testing.assert_allclose(r1, r2, rtol=1e-5)
    dx1 = rnd((B, T, C), 4); dx2 = dx1.copy()   # backward accumulates: start from non-zero
    dw1 = rnd(C, 5); dw2 = dw1.copy(); db1 = rnd(C, 6); db2 = db1.copy()
    ol.cref().cref_layernorm_backward(dx1, dw1, db1, g, x, w, m1, r1, N, C)
    ol.ref().layernorm_backward(dx2, dw2, db2, g, x, w, m2, r2, B, T, C)
    np.testing.assert_allclose(dx1, dx2, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dw1, dw2, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(db1, db2, rtol=1e-4, atol=1e-4)


def test_layernorm_closed_forms():
    # constant rows normalise to zero => out == bias; w=1,b=0 => rows have mean 0, var = v/(v+eps)
    C_ = 64
    x = np.full((3, C_), 2.5, np.float32); w = rnd(C_, 1); b = rnd(C_, 2)
    o = np.zeros_like(x)
    ol.cref().cref_layernorm_forward(o, None, None, x, w, b, 3, C_)
    np.testing.assert_allclose(o, np.broadcast_to(b, o.shape), atol=1e-6)
    x = rnd((4, C_), 3); o = np.zeros_like(x)
    ol.cref().cref_layernorm_forward(o, None, None, x, np.ones(C_, np.float32), np.zeros(C_, np.float32), 4, C_)
    np.testing.assert_allclose(o.mean(1), 0, atol=1e-6)
    v = x.astype(np.float64).var(1)
    np.testing.assert_allclose(o.astype(np.float64).var(1), v / (v + 1e-5), rtol=1e-5)


@needs_ref
@pytest.mark.parametrize("N,C,OC,bias", [(8, 32, 48, True), (5, 16, 24, True), (16, 64, 128, False)])
def test_matmul_fwd_bwd(N, C, OC, bias):
    x, w, b, g = rnd((N, C), 0), rnd((OC, C), 1), rnd(OC, 2), rnd((N, OC), 3)
    bp = b.ctypes.data if bias else None
    o1 = np.zeros((N, OC), np.float32); o2 = np.zeros_like(o1)
    ol.cref().cref_matmul_forward(o1, x, w, bp, N, C, OC)
    ol.ref().matmul_forward(o2, x, w, bp, 1, N, C, OC)   # N%8!=0 falls back to the naive loop inside
    np.testing.assert_allclose(o1, o2, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(o1, x.astype(np.float64) @ w.astype(np.float64).T + (b if bias else 0), rtol=1e-4, atol=1e-4)
    dx1 = rnd((N, C), 4); dx2 = dx1.copy(); dw1 = rnd((OC, C), 5); dw2 = dw1.copy()
    db1 = rnd(OC, 6); db2 = db1.copy()
    ol.cref().cref_matmul_backward(dx1.ctypes.data, dw1, db1.ctypes.data if bias else None, g, x, w, N, C, OC)
    ol.ref().matmul_backward(dx2, dw2, db2.ctypes.data if bias else None, g, x, w, 1, N, C, OC)
    np.testing.assert_allclose(dx1, dx2, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(dw1, dw2, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(db1, db2, rtol=1e-4, atol=1e-4)


@needs_ref
@pytest.mark.parametrize("B,T,C,NH", [(2, 16, 32, 4), (1, 33, 128, 2)])
def test_attention_fwd_bwd_vs_cubic_reference(B, T, C, NH):
    qkv = rnd((B, T, 3 * C), 0); g = rnd((B, T, C), 1)
    o1 = np.zeros((B, T, C), np.float32); att1 = np.zeros((B, NH, T, T), np.float32); lse = np.zeros((B, NH, T), np.float32)
    o2 = np.zeros_like(o1); pre2 = np.zeros_like(att1); att2 = np.zeros_like(att1)
    ol.cref().cref_attention_forward(o1, att1.ctypes.data, lse.ctypes.data, qkv, B, T, C, NH)
    ol.ref().attention_forward(o2, pre2, att2, qkv, B, T, C, NH)
    np.testing.assert_allclose(o1, o2, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(att1, att2, rtol=1e-5, atol=1e-6)
    # lse against the reference's pre-softmax scores
    for t in range(T):
        ref_lse = np.log(np.exp(pre2[:, :, t, :t + 1].astype(np.float64)).sum(-1))
        np.testing.assert_allclose(lse[:, :, t], ref_lse, rtol=1e-5, atol=1e-5)
    d1 = rnd((B, T, 3 * C), 2); d2 = d1.copy()
    ol.cref().cref_attention_backward(d1, g, qkv, att1.ctypes.data, B, T, C, NH)
    dpre = np.zeros_like(att1); datt = np.zeros_like(att1)
    ol.ref().attention_backward(d2, dpre, datt, g, qkv, att2, B, T, C, NH)
    np.testing.assert_allclose(d1, d2, rtol=1e-4, atol=1e-5)
    # and with probabilities recomputed instead of stored
    d3 = rnd((B, T, 3 * C), 2)
    ol.cref().cref_attention_backward(d3, g, qkv, None, B, T, C, NH)
    np.testing.assert_allclose(d3, d2, rtol=1e-4, atol=1e-5)


def test_attention_closed_forms():
    # T=1: softmax over one key is 1 => out == V
    B, T, C_, NH = 3, 1, 32, 4
    qkv = rnd((B, T, 3 * C_), 0); o = np.zeros((B, T, C_), np.float32)
    ol.cref().cref_attention_forward(o, None, None, qkv, B, T, C_, NH)
    np.testing.assert_allclose(o, qkv[:, :, 2 * C_:], atol=1e-7)
    # causality: changing tokens after t leaves outputs up to t unchanged
    B, T = 1, 12
    qkv = rnd((B, T, 3 * C_), 1); o1 = np.zeros((B, T, C_), np.float32); o2 = np.zeros_like(o1)
    ol.cref().cref_attention_forward(o1, None, None, qkv, B, T, C_, NH)
    qkv2 = qkv.copy(); qkv2[:, 7:] += 1.0
    ol.cref().cref_attention_forward(o2, None, None, qkv2, B, T, C_, NH)
    np.testing.assert_array_equal(o1[:, :7], o2[:, :7])
    assert np.abs(o1[:, 7:] - o2[:, 7:]).max() > 1e-3


@needs_ref
def test_gelu_residual_encoder():
    n = 1000
    x = rnd(n, 0, 3.0); g = rnd(n, 1)
    o1 = np.zeros(n, np.float32); o2 = np.zeros(n, np.float32)
    ol.cref().cref_gelu_forward(o1, x, n); ol.ref().gelu_forward(o2, x, n)
    np.testing.assert_allclose(o1, o2, rtol=1e-5, atol=1e-6)
    d1 = rnd(n, 2); d2 = d1.copy()
    ol.cref().cref_gelu_backward(d1, x, g, n); ol.ref().gelu_backward(d2, x, g, n)
    np.testing.assert_allclose(d1, d2, rtol=1e-5, atol=1e-6)
    a, b = rnd(n, 3), rnd(n, 4)
    ol.cref().cref_residual_forward(o1, a, b, n)
    np.testing.assert_array_equal(o1, a + b)
    B, T, C_, V = 2, 6, 16, 50
    wte, wpe = rnd((V, C_), 5), rnd((T, C_), 6)
    inp = np.random.RandomState(7).randint(0, V, B * T).astype(np.int32)
    e1 = np.zeros((B, T, C_), np.float32); e2 = np.zeros_like(e1)
    ol.cref().cref_encoder_forward(e1, inp, wte, wpe, B, T, C_); ol.ref().encoder_forward(e2, inp, wte, wpe, B, T, C_)
    np.testing.assert_array_equal(e1, e2)
    dout = rnd((B, T, C_), 8)
    dwte1 = rnd((V, C_), 9); dwte2 = dwte1.copy(); dwpe1 = rnd((T, C_), 10); dwpe2 = dwpe1.copy()
    ol.cref().cref_encoder_backward(dwte1, dwpe1, dout, inp, B, T, C_)
    ol.ref().encoder_backward(dwte2, dwpe2, dout, inp, B, T, C_)
    np.testing.assert_allclose(dwte1, dwte2, atol=1e-6); np.testing.assert_allclose(dwpe1, dwpe2, atol=1e-6)


def test_gelu_closed_forms():
    x = np.array([0.0, 10.0, -10.0], np.float32); o = np.zeros(3, np.float32)
    ol.cref().cref_gelu_forward(o, x, 3)
    np.testing.assert_allclose(o, [0.0, 10.0, 0.0], atol=1e-6)
    d = np.zeros(3, np.float32)
    ol.cref().cref_gelu_backward(d, x, np.ones(3, np.float32), 3)
    np.testing.assert_allclose(d, [0.5, 1.0, 0.0], atol=1e-6)


@needs_ref
def test_softmax_crossentropy():
    N, V, Vp = 6, 50, 64
    z = rnd((N, Vp), 0, 2.0); tg = np.random.RandomState(1).randint(0, V, N).astype(np.int32)
    p1 = np.zeros((N, Vp), np.float32); l1 = np.zeros(N, np.float32)
    p2 = np.zeros_like(p1); l2 = np.zeros(N, np.float32)
    ol.cref().cref_softmax_crossentropy_forward(p1, l1.ctypes.data, z, tg.ctypes.data, N, V, Vp)
    ol.ref().softmax_forward(p2, z, 1, N, V, Vp); ol.ref().crossentropy_forward(l2, p2, tg, 1, N, Vp)
    np.testing.assert_allclose(p1, p2, rtol=1e-5, atol=1e-7); np.testing.assert_allclose(l1, l2, rtol=1e-5)
    d1 = rnd((N, Vp), 2); d2 = d1.copy()
    ol.cref().cref_crossentropy_softmax_backward(d1, p1, tg, 1.0 / N, N, V, Vp)
    ol.ref().crossentropy_softmax_backward(d2, np.full(N, 1.0 / N, np.float32), p2, tg, 1, N, V, Vp)
    np.testing.assert_allclose(d1, d2, rtol=1e-5, atol=1e-7)


def test_softmax_closed_forms():
    # uniform logits => loss = ln V; probabilities sum to 1; dlogits sum to 0 over the real vocabulary
    N, V, Vp = 2, 50257, 50304
    z = np.zeros((N, Vp), np.float32); tg = np.array([3, 50256], np.int32)
    p = np.zeros_like(z); l = np.zeros(N, np.float32)
    ol.cref().cref_softmax_crossentropy_forward(p, l.ctypes.data, z, tg.ctypes.data, N, V, Vp)
    np.testing.assert_allclose(l, np.log(V), rtol=1e-6)
    np.testing.assert_allclose(p[:, :V].sum(1, dtype=np.float64), 1.0, rtol=1e-5)
    assert (p[:, V:] == 0).all()
    d = np.zeros_like(z)
    ol.cref().cref_crossentropy_softmax_backward(d, p, tg, 1.0, N, V, Vp)
    np.testing.assert_allclose(d.sum(1, dtype=np.float64), 0.0, atol=1e-5)
    assert (d[:, V:] == 0).all()


def test_adamw_first_step_is_sign_descent():
    # t=1, m=v=0: m_hat=g, v_hat=g^2 => dp = -lr * (g/(|g|+eps) + wd*p)
    n = 257
    p = rnd(n, 0); g = rnd(n, 1); m = np.zeros(n, np.float32); v = np.zeros(n, np.float32)
    p0 = p.copy()
    ol.cref().cref_adamw(p, m, v, g, n, 1e-2, 0.9, 0.999, 1e-8, 0.1, 1)
    np.testing.assert_allclose(p, p0 - 1e-2 * (g / (np.abs(g) + 1e-8) + 0.1 * p0), rtol=1e-5, atol=1e-6)
    # the lerp form used on the GPU is the same update
    p2 = p0.copy(); m2 = np.zeros(n, np.float32); v2 = np.zeros(n, np.float32)
    ol.cref().cref_adamw_f32(p2, None, g, m2, v2, n, 1e-2, 0.9, 0.999, 1, 1e-8, 0.1, 1.0)
    np.testing.assert_allclose(p2, p, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(m2, m, rtol=1e-5, atol=1e-7)


def test_stochastic_rounding_properties():
    L = ol.cref()
    # SquirrelNoise5(0, 0): follow llmc/cuda_utils.cuh:238-256 by hand in Python integers
    def sq5(pos, seed):
        M = 0xffffffff
        x = (pos * 0xd2a80a3f) & M; x = (x + seed) & M; x ^= x >> 9
        x = (x + 0xa884f197) & M; x ^= x >> 11
        x = (x * 0x6C736F4B) & M; x ^= x >> 13
        x = (x + 0xB79F3ABB) & M; x ^= x >> 15
        x = (x * 0x1b56c4f5) & M; x ^= x >> 17
        return x
    for pos, seed in [(0, 0), (1, 2), (123456789, 987654321), (0xffffffff, 0xdeadbeef)]:
        assert L.cref_squirrel_noise5(pos, seed) == sq5(pos, seed)
    assert L.cref_noise_2d(5, 7, 11) == sq5((5 + 198491317 * 7) & 0xffffffff, 11)
    # rounding goes to one of the two bf16 neighbours, and is exact for representable values
    x = np.float32(1.0 + 2.0 ** -10)  # between bf16 1.0 and 1.0078125
    outs = {L.cref_stochastic_round_bf16(float(x), r) for r in range(0, 65536, 97)}
    assert outs == {0x3f80, 0x3f81}
    assert L.cref_stochastic_round_bf16(1.0, 12345) == 0x3f80
    # unbiased: P(round up) = low16/65536
    ups = sum(L.cref_stochastic_round_bf16(float(x), r) == 0x3f81 for r in range(65536))
    low = int(np.frombuffer(x.tobytes(), np.uint32)[0] & 0xffff)
    assert ups == low


TINY = dict(max_seq_len=32, vocab_size=100, padded_vocab_size=128, num_layers=2, num_heads=2, channels=32)


@needs_ref
def test_whole_model_matches_compiled_reference():
    cfg = Config(**TINY)
    B, T, steps = 2, 16, 5
    params = ol.init_params(cfg, 42)
    inp, tgt = ol.make_tokens(B, T, cfg.vocab_size, 7)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "tiny.bin")
        assert ol.cref().cref_write_checkpoint_fp32(path.encode(), params, C.byref(cfg)) == 0
        r = ol.ref_train(path, cfg, inp, tgt, B, T, steps, lr=1e-3, wd=0.01, want_logits=True)
    c = ol.cref_train(cfg, params, inp, tgt, B, T, steps, lr=1e-3, wd=0.01, want_logits=True)
    np.testing.assert_allclose(c["losses"], r["losses"], rtol=2e-6)
    np.testing.assert_allclose(c["logits"], r["logits"], rtol=1e-4, atol=1e-5)
    scale = np.abs(r["grads"]).max()
    assert np.abs(c["grads"] - r["grads"]).max() <= 1e-5 * scale
    # Adam divides by sqrt(v): coordinates whose gradient is at rounding-noise level move by a
    # noise-dependent fraction of lr, so parameters agree to a fraction of lr*steps, not to 1e-6
    np.testing.assert_allclose(c["params"], r["params"], rtol=1e-4, atol=1e-4)


def test_sampler_closed_forms():
    L = ol.cref()
    # four equally likely outcomes: the coin's quarter picks the index
    u = np.zeros(4, np.float32)
    assert [L.cref_sample_softmax(u, 4, c) for c in (0.0, 0.3, 0.5, 0.76, 0.999)] == [0, 1, 2, 3, 3]
    # one outcome far more likely than the rest takes (almost) every coin; softmax is shift-invariant
    z = np.array([0.0, 40.0, 0.0], np.float32)
    assert all(L.cref_sample_softmax(z, 3, c) == 1 for c in (1e-6, 0.5, 0.999999))
    assert L.cref_sample_softmax(z, 3, 0.0) == 0
    z = np.array([1.0, 2.0, 3.0, 0.5], np.float32)
    p = np.exp(z.astype(np.float64)); cdf = np.cumsum(p / p.sum())
    for c in (0.05, 0.2, 0.5, 0.9, 0.99):
        assert L.cref_sample_softmax(z, 4, c) == int(np.searchsorted(cdf, c, side="right"))
    # the generator: floats with 24 random bits in [0, 1), from the documented xorshift* recurrence
    st = C.c_uint64(1337)
    x = 1337
    for _ in range(5):
        x ^= x >> 12; x ^= (x << 25) & (2**64 - 1); x ^= x >> 27
        want = ((((x * 0x2545F4914F6CDD1D) & (2**64 - 1)) >> 32) >> 8) / 16777216.0
        assert L.cref_random_f32(C.byref(st)) == np.float32(want)
        assert st.value == x


@needs_ref
def test_sampler_matches_compiled_reference():
    L, R = ol.cref(), ol.ref()
    for seed in (1337, 1, 0xDEADBEEFCAFE):
        a, b = C.c_uint64(seed), C.c_uint64(seed)
        for _ in range(64):
            assert L.cref_random_f32(C.byref(a)) == R.random_f32(C.byref(b))
        assert a.value == b.value
    rs = np.random.RandomState(3)
    for n in (7, 100, 50257):
        z = (rs.randn(n) * 3).astype(np.float32)
        for coin in [0.0, 0.999999] + list(rs.rand(40).astype(np.float32)):
            assert L.cref_sample_softmax(z, n, coin) == R.sample_softmax(z, n, coin)


@needs_ref
def test_generation_matches_compiled_reference():
    cfg = Config(**TINY)
    params = ol.init_params(cfg, 42) * 8      # sharper distributions than the 0.02-scale init gives
    params = np.ascontiguousarray(params, np.float32)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "tiny.bin")
        assert ol.cref().cref_write_checkpoint_fp32(path.encode(), params, C.byref(cfg)) == 0
        rt, rstate = ol.ref_generate(path, cfg.max_seq_len, 32, cfg.vocab_size - 1)
    ct, cstate = ol.cref_generate(cfg, params, cfg.max_seq_len, 32, cfg.vocab_size - 1)
    np.testing.assert_array_equal(ct, rt)
    assert cstate == rstate
    assert len(set(ct[1:].tolist())) > 8      # a sequence, not one token over and over


def test_whole_model_gradient_by_finite_differences():
    # brute force: central differences of the oracle's own loss on a few coordinates of every tensor
    cfg = Config(max_seq_len=8, vocab_size=20, padded_vocab_size=32, num_layers=1, num_heads=2, channels=16)
    B, T = 1, 8
    params = ol.init_params(cfg, 3)
    params += (np.random.RandomState(0).standard_normal(params.size) * 0.05).astype(np.float32)  # biases != 0
    inp, tgt = ol.make_tokens(B, T, cfg.vocab_size, 1)
    base = ol.cref_train(cfg, params, inp, tgt, B, T, 1, lr=0.0)
    sizes, _ = ol.param_sizes(cfg)
    rng = np.random.RandomState(5)
    off = 0
    h = 1e-2
    for i, n in enumerate(sizes):
        lo = 0 if i != 0 else 0
        hi = n if i != 0 else cfg.vocab_size * cfg.channels
        for j in rng.randint(lo, hi, 3):
            k = off + j
            pp = params.copy(); pp[k] += h
            pm = params.copy(); pm[k] -= h
            lp = ol.cref_train(cfg, pp, inp, tgt, B, T, 1, lr=0.0)["losses"][0]
            lm = ol.cref_train(cfg, pm, inp, tgt, B, T, 1, lr=0.0)["losses"][0]
            fd = (float(lp) - float(lm)) / (2 * h)
            assert abs(fd - base["grads"][k]) <= 2e-3 + 2e-2 * abs(fd), (i, j, fd, base["grads"][k])
        off += n


def test_init_follows_descriptor_rules():
    cfg = Config(**TINY)
    p = ol.init_params(cfg, 42)
    sizes, tot = ol.param_sizes(cfg)
    offs = np.cumsum([0] + sizes)
    C_, V, Vp, L = cfg.channels, cfg.vocab_size, cfg.padded_vocab_size, cfg.num_layers
    wte = p[offs[0]:offs[1]].reshape(Vp, C_)
    assert (wte[V:] == 0).all() and wte[:V].std() > 0.015
    for i in (2, 8, 14):
        assert (p[offs[i]:offs[i + 1]] == 1).all()
    for i in (3, 5, 7, 9, 11, 13, 15):
        assert (p[offs[i]:offs[i + 1]] == 0).all()
    # residual projections are scaled by 1/sqrt(2L)
    r = p[offs[6]:offs[7]].std() / p[offs[4]:offs[5]].std()
    assert abs(r - 1 / np.sqrt(2 * L)) < 0.05
    # first draw of the stream is wte: same numbers as a bare normal_ of that length from the same seed
    ints = np.zeros(5, np.uint32)  # (KAT function draws 5 ints first, so compare through a second init instead)
    p2 = ol.init_params(cfg, 42)
    np.testing.assert_array_equal(p, p2)
    assert not np.array_equal(p, ol.init_params(cfg, 43))
