"""llmk_attention_backward_static - the entry point that allocates nothing - against llmk_attention_backward.

Both run the same kernels; the only difference is where the rowsum(dO*O) vector lives (a static device array instead of
the library's grow-only workspace), so the outputs must be the same bits. Two calls in a row, the second on a smaller
input: the array keeps the first call's contents, and nothing of them may leak into the second result. Sizes beyond
the array are rejected with an error instead of being run.
"""
import numpy as np
import pytest

import gpu_lib as G

pytestmark = pytest.mark.gpu


def _case(B, T, NH, seed):
    import torch
    Cc = NH * 64
    gen = torch.Generator(device="cuda"); gen.manual_seed(seed)
    qkv = torch.randn((B, T, 3 * Cc), generator=gen, device="cuda").to(torch.bfloat16)
    dout = torch.randn((B, T, Cc), generator=gen, device="cuda").to(torch.bfloat16)
    return qkv, dout, Cc


@pytest.mark.parametrize("precision", ["bf16", "fp32"])
def test_static_scratch_attention_backward_matches_the_allocating_one(precision):
    import torch
    L = G.lib(precision)
    dt = G.torch_dtype(precision)
    for B, T, NH, seed in ((8, 1024, 12, 1), (2, 192, 3, 2)):           # the second call is smaller than the first
        qkv, dout, Cc = _case(B, T, NH, seed)
        qkv, dout = qkv.to(dt), dout.to(dt)
        out = torch.zeros((B, T, Cc), dtype=dt, device="cuda")
        stats = torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
        L.llmk_attention_forward(G.ptr(out), G.ptr(stats), G.ptr(qkv), B, T, NH, Cc, None)
        want = torch.full((B, T, 3 * Cc), 3.0, dtype=dt, device="cuda")
        got = torch.full((B, T, 3 * Cc), 5.0, dtype=dt, device="cuda")
        L.llmk_attention_backward(G.ptr(want), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
        G.sync()
        before = torch.cuda.memory_allocated()
        L.llmk_attention_backward_static(G.ptr(got), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
        G.sync()
        assert torch.cuda.memory_allocated() == before
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got, want), (precision, B, T, NH)
    G.check_no_error(L)


def test_static_scratch_rejects_sizes_beyond_its_array():
    import torch
    L = G.lib("bf16")
    B, T, NH = 2, 64, 2
    qkv, dout, Cc = _case(B, T, NH, 3)
    L.llmk_set_error_mode(1)
    try:
        # B*NH*T = 2^20 + 64 floats; the check comes before any pointer is touched
        L.llmk_attention_backward_static(None, None, None, None, G.ptr(dout), 16385, 64, 1, 64, None)
        msg = L.llmk_last_error().decode()
        assert "exceeds" in msg and "static scratch" in msg, msg
    finally:
        L.llmk_clear_error()
        L.llmk_set_error_mode(0)
    # and the library still works afterwards
    out = torch.zeros((B, T, Cc), dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
    L.llmk_attention_forward(G.ptr(out), G.ptr(stats), G.ptr(qkv), B, T, NH, Cc, None)
    d = torch.zeros((B, T, 3 * Cc), dtype=torch.bfloat16, device="cuda")
    L.llmk_attention_backward_static(G.ptr(d), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
    G.sync()
    assert d.float().abs().sum().item() > 0
    G.check_no_error(L)
