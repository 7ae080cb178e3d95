"""llmk_attention_backward_static - the entry point that allocates nothing - against llmk_attention_backward.

Both run the same kernels; the only difference is where the rowsum(dO*O) vector lives (a static device array instead of
the library's grow-only workspace), so the outputs must be the same bits. Two calls in a row, the second on a smaller
input: the array keeps the first call's contents, and nothing of them may leak into the second result. Sizes beyond
the array are rejected with an error instead of being run.

That the static entry point allocates nothing is checked on what an allocation would move: the size of the library's
workspace (llmk_workspace_bytes), the device's free memory (hipMemGetInfo through torch.cuda.mem_get_info, which sees
every allocation of the process, not only torch's), torch's own allocator, and the library's timing events (with
profiling switched on the call must add no record). The static call runs BEFORE the allocating one, on a shape whose
rowsum(dO*O) vector is larger than the workspace is at that moment, so a static path that quietly took the workspace
would have to grow it.
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
    """bf16: T = 1024 and 192 take the direct-to-LDS kernels (the dQ kernel writes the vector), T = 200 the
    register-staged ones with the separate rowsum pass writing it. fp32: the one-wave-per-row kernels never touch the
    vector, so that leg only shows that the entry point dispatches and agrees."""
    import torch
    L = G.lib(precision)
    dt = G.torch_dtype(precision)
    # the second and third calls are smaller than the first
    for B, T, NH, seed in ((8, 1024, 12, 1), (2, 192, 3, 2), (2, 200, 3, 4)):
        qkv, dout, Cc = _case(B, T, NH, seed)
        qkv, dout = qkv.to(dt), dout.to(dt)
        out = torch.zeros((B, T, Cc), dtype=dt, device="cuda")
        stats = torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
        L.llmk_attention_forward(G.ptr(out), G.ptr(stats), G.ptr(qkv), B, T, NH, Cc, None)
        want = torch.full((B, T, 3 * Cc), 3.0, dtype=dt, device="cuda")
        got = torch.full((B, T, 3 * Cc), 5.0, dtype=dt, device="cuda")
        G.sync()
        # static first, so that nothing it could lean on has been made by the allocating call
        L.llmk_profile_reset()
        L.llmk_profile_enable(1)
        ws_before, free_before, torch_before = L.llmk_workspace_bytes(), torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
        L.llmk_attention_backward_static(G.ptr(got), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
        G.sync()
        assert L.llmk_workspace_bytes() == ws_before
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_allocated() == torch_before
        assert L.llmk_profile_count() == 0                                   # no timing events were taken or created
        L.llmk_profile_enable(0)
        L.llmk_attention_backward(G.ptr(want), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
        G.sync()
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got, want), (precision, B, T, NH)
    G.check_no_error(L)


def test_static_scratch_does_not_use_the_workspace():
    """In a process whose workspace is smaller than the vector of this shape (it is when this file runs alone; after
    other tests the workspace may already be large, and the check says so by being skipped), the static call must leave
    the workspace as small as it was."""
    import torch
    L = G.lib("bf16")
    B, T, NH = 16, 1024, 16                                                  # 262144 floats = 1 MiB of rowsum(dO*O)
    need = L.llmk_attention_backward_workspace_bytes(B, T, NH)
    assert need == B * T * NH * 4
    if L.llmk_workspace_bytes() >= need:
        pytest.skip("the workspace already exceeds this shape's vector: run this file alone for the check")
    qkv, dout, Cc = _case(B, T, NH, 9)
    out = torch.zeros((B, T, Cc), dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros((B, NH, T), dtype=torch.float32, device="cuda")
    d = torch.zeros((B, T, 3 * Cc), dtype=torch.bfloat16, device="cuda")
    L.llmk_attention_forward(G.ptr(out), G.ptr(stats), G.ptr(qkv), B, T, NH, Cc, None)
    G.sync()
    ws, free = L.llmk_workspace_bytes(), torch.cuda.mem_get_info()[0]
    L.llmk_attention_backward_static(G.ptr(d), G.ptr(dout), G.ptr(qkv), G.ptr(out), G.ptr(stats), B, T, NH, Cc, None)
    G.sync()
    assert L.llmk_workspace_bytes() == ws and torch.cuda.mem_get_info()[0] == free
    assert d.float().abs().sum().item() > 0
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
