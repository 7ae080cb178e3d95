"""Per-kernel microbenchmark at GPT-2 124M shapes (N = B*T = 65536 rows, bf16 storage, fp32 accumulation),
in the manner of the reference's dev/cuda/*.cu programs (timing loop dev/cuda/common.h:350-385: a cache flush
before every repetition, device events around the launch).

Every case is called through the C ABI (include/llmk.h); the library brackets each of its kernel launches with HIP
events on the launch stream (llmk_profile_*), so a case that launches several kernels (matmul_backward: dinp GEMM,
dweight GEMM, split-K reduce, bias gradient) reports each of them. Inputs are N(0,1) from a fixed seed, weights
N(0,0.02). Before each repetition 1 GiB is overwritten, which evicts the 8 x 4 MiB L2s and the 256 MiB Infinity Cache.

    python llm.c_amd/microbench.py [--reps 20] [--only gemm,attention,...] [--json out.json] [--variant NAME | --against NAME[,NAME...]]

--against loads the product library AND the named variant builds (lib/variants/NAME/, python llm.c_amd/build.py --variant
NAME -D...) into this one process and calls them in turn, repetition by repetition, on the same buffers: differences between
two builds of a kernel then show to about half a percent, where separate processes (or separate machines of the pool)
differ by several percent in clock, memory placement and temperature.

Prints, per kernel family and case: median and minimum milliseconds, the algorithmic TFLOP/s or GB/s at the median,
and the fraction of the roofline that bounds the family (2500 TFLOP/s bf16 MFMA, 8000 GB/s HBM). PyTorch is used
for device memory and random numbers only.
"""
import argparse
import ctypes as C
import importlib.util
import json
import os
import statistics
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("llmc_amd", os.path.join(HERE, "__init__.py"))
pkg = importlib.util.module_from_spec(spec)
sys.modules["llmc_amd"] = pkg
spec.loader.exec_module(pkg)

PEAK_TFLOPS, PEAK_GBS = 2500.0, 8000.0
MFMA_FAMILIES = ("gemm", "attention_forward", "attention_backward_dq", "attention_backward_dkdv")


class _InTurn:
    """Stands for whichever of several loaded libraries has the turn: the cases call through it."""

    def __init__(self, lib):
        self.cur = lib

    def __getattr__(self, name):
        return getattr(self.cur, name)


def run_cases(L, reps=20, only=(), emit=print, others=()):
    """Runs every case (or those whose tag contains one of `only`) on the loaded library L and returns the list of
    per-kernel records. `emit` receives the printed lines (None: silent). `others`: (tag, library) pairs timed in turn
    with L in every repetition; their medians go into each record's "against"."""
    only = list(only)
    turns = [("", L)] + list(others)
    L = _InTurn(L)
    dev = "cuda"
    p = lambda t: None if t is None else C.c_void_p(t.data_ptr())
    g = torch.Generator(device=dev); g.manual_seed(1234)
    randn = lambda *shape, scale=1.0: (torch.randn(*shape, device=dev, generator=g) * scale).bfloat16()
    flush_buf = torch.empty(1 << 30, dtype=torch.uint8, device=dev)

    name = C.create_string_buffer(64)
    calls, ms, fl, by = C.c_int(), C.c_double(), C.c_double(), C.c_double()

    def measure(fn, prepare=None):
        """-> {family: (list of ms per rep, flops per rep, bytes per rep, launches per rep, {tag: list of ms})}"""
        out = {}
        for _, lib in turns:
            L.cur = lib
            fn(); torch.cuda.synchronize()                    # warm-up (workspace growth, attribute setting)
        for _ in range(reps):
            for tag, lib in turns:
                L.cur = lib
                if prepare: prepare()
                flush_buf.zero_(); torch.cuda.synchronize()
                L.llmk_profile_reset(); L.llmk_profile_enable(1)
                fn()
                torch.cuda.synchronize(); L.llmk_profile_enable(0)
                for i in range(L.llmk_profile_count()):
                    L.llmk_profile_get(i, name, C.byref(calls), C.byref(ms), C.byref(fl), C.byref(by))
                    rec = out.setdefault(name.value.decode(), ([], fl.value, by.value, calls.value, {}))
                    (rec[4].setdefault(tag, []) if tag else rec[0]).append(ms.value)
        L.cur = turns[0][1]
        return out

    results = []

    def report(case, out):
        for fam, (times, flops, nbytes, ncalls, alt) in out.items():
            med, mn = statistics.median(times), min(times)
            mfma = fam.startswith(MFMA_FAMILIES)
            if mfma:
                rate, unit, frac = flops / med * 1e-9, "TFLOP/s", flops / med * 1e-9 / PEAK_TFLOPS
            else:
                rate, unit, frac = nbytes / med * 1e-6, "GB/s", nbytes / med * 1e-6 / PEAK_GBS
            against = {tag: statistics.median(t) for tag, t in alt.items()}
            if emit:
                versus = "".join(f"  | {tag} {m:8.4f} ms {100 * (m / med - 1):+5.1f} %" for tag, m in against.items())
                emit(f"{case:34s} {fam:26s} x{ncalls:<2d} median {med:8.4f} ms  min {mn:8.4f} ms  {rate:9.1f} {unit:8s} {100 * frac:5.1f} % of {'MFMA' if mfma else 'HBM'} peak{versus}")
            results.append({"case": case, "kernel": fam, "launches": ncalls, "median_ms": med, "min_ms": mn, "rate": rate, "unit": unit,
                            "bound": "mfma" if mfma else "hbm", "frac": frac, "flops": flops, "bytes": nbytes})
            if against:
                results[-1]["against"] = against

    def want(tag):
        return not only or any(o in tag for o in only)

    B, T, Cc, NH, V, Vp, NL = 64, 1024, 768, 12, 50257, 50304, 12
    N = B * T

    if want("gemm"):
        for nm, K, OC in [("qkv", 768, 2304), ("attproj", 768, 768), ("fc", 768, 3072), ("fcproj", 3072, 768), ("lm_head", 768, 50304)]:
            inp, w = randn(N, K), randn(OC, K, scale=0.02)
            bias = None if nm == "lm_head" else randn(OC, scale=0.02)
            out_t = torch.empty(N, OC, device=dev, dtype=torch.bfloat16)
            report(f"matmul_forward {nm} K={K} OC={OC}",
                   measure(lambda: L.llmk_matmul_forward(p(out_t), p(inp), p(w), p(bias), B, T, K, OC, None, None, 0)))
            if nm in ("attproj", "fcproj"):                     # the projections into the residual stream, with the add as their epilogue
                res = randn(N, OC)
                report(f"matmul_forward+residual {nm} K={K} OC={OC}",
                       measure(lambda: L.llmk_matmul_forward_residual(p(out_t), p(inp), p(w), p(bias), p(res), B, T, K, OC, None)))
                del res
            if nm == "fc":
                pre = torch.empty_like(out_t)
                report(f"matmul_forward+gelu {nm} K={K} OC={OC}",
                       measure(lambda: L.llmk_matmul_forward(p(out_t), p(inp), p(w), p(bias), B, T, K, OC, None, p(pre), 2)))
                # gelu_fusion 3: the second output is gelu'(pre-activation), kept for the backward epilogue
                report(f"matmul_forward+gelu3 {nm} K={K} OC={OC}",
                       measure(lambda: L.llmk_matmul_forward(p(out_t), p(inp), p(w), p(bias), B, T, K, OC, None, p(pre), 3)))
                del pre
            dout = out_t.normal_(generator=g)                  # reuse the output buffer as the upstream gradient
            dinp, dw = torch.empty_like(inp), torch.zeros_like(w)
            dbias = None if bias is None else torch.zeros_like(bias)
            scratch = torch.empty(max(L.llmk_matmul_backward_bias_scratch_floats(OC), 1), device=dev, dtype=torch.float32)
            report(f"matmul_backward {nm} K={K} OC={OC}",
                   measure(lambda: L.llmk_matmul_backward(p(dinp), p(dw), p(dbias), p(dout), p(inp), p(w), p(scratch), B, T, K, OC, None, None, 0)))
            if nm == "fcproj":                                 # the dinp GEMM with GELU backward in its epilogue (gelu_fusion 2)
                pre = randn(N, K)
                report(f"matmul_backward+dgelu {nm} K={K} OC={OC}",
                       measure(lambda: L.llmk_matmul_backward(p(dinp), p(dw), p(dbias), p(dout), p(inp), p(w), p(scratch), B, T, K, OC, None, p(pre), 2)))
                report(f"matmul_backward+dgelu3 {nm} K={K} OC={OC}",      # pre holds a stored derivative here (any values do for timing)
                       measure(lambda: L.llmk_matmul_backward(p(dinp), p(dw), p(dbias), p(dout), p(inp), p(w), p(scratch), B, T, K, OC, None, p(pre), 3)))
                del pre
            del inp, w, out_t, dout, dinp, dw, scratch
            torch.cuda.empty_cache()

    if want("layernorm"):
        x, y = randn(N, Cc), randn(N, Cc)
        w, b = randn(Cc), randn(Cc)
        o, r = torch.empty_like(x), torch.empty_like(x)
        mean, rstd = torch.empty(N, device=dev), torch.empty(N, device=dev)
        report("layernorm_forward 65536x768", measure(lambda: L.llmk_layernorm_forward(p(o), p(mean), p(rstd), p(x), p(w), p(b), B, T, Cc, None)))
        report("fused_residual_forward5 65536x768",
               measure(lambda: L.llmk_fused_residual_forward5(p(r), p(o), p(mean), p(rstd), p(x), p(y), p(w), p(b), N, Cc, None)))
        dinp, dw, db = torch.zeros_like(x), torch.zeros_like(w), torch.zeros_like(b)
        scratch = torch.empty(L.llmk_layernorm_backward_scratch_floats(Cc), device=dev, dtype=torch.float32)
        report("layernorm_backward 65536x768",
               measure(lambda: L.llmk_layernorm_backward(p(dinp), p(dw), p(db), p(scratch), p(y), p(x), p(w), p(mean), p(rstd), B, T, Cc, None)))
        del x, y, o, r, dinp

    if want("gelu"):
        n = N * 4 * Cc
        x, o = randn(N, 4 * Cc), torch.empty(N, 4 * Cc, device=dev, dtype=torch.bfloat16)
        report("gelu_forward 65536x3072", measure(lambda: L.llmk_gelu_forward(p(o), p(x), n, None)))
        report("gelu_backward_inplace 65536x3072", measure(lambda: L.llmk_gelu_backward_inplace(p(o), p(x), n, None)))
        db = torch.zeros(4 * Cc, device=dev, dtype=torch.bfloat16)
        scratch = torch.empty(max(L.llmk_matmul_backward_bias_scratch_floats(4 * Cc), 1), device=dev, dtype=torch.float32)
        report("gelu_backward_bias 65536x3072", measure(lambda: L.llmk_gelu_backward_bias(p(o), p(x), p(db), p(scratch), B, T, 4 * Cc, None)))
        del x, o

    if want("encoder"):
        tok = torch.randint(0, V, (N,), device=dev, dtype=torch.int32, generator=g)
        tok_host = np.ascontiguousarray(tok.cpu().numpy())
        wte, wpe = randn(Vp, Cc, scale=0.02), randn(T, Cc, scale=0.02)
        o = torch.empty(N, Cc, device=dev, dtype=torch.bfloat16)
        report("encoder_forward 65536x768", measure(lambda: L.llmk_encoder_forward(p(o), p(tok), p(wte), p(wpe), B, T, Cc, None)))
        dout = randn(N, Cc)
        dwte, dwpe = torch.zeros_like(wte), torch.zeros_like(wpe)
        ncg = -(-Cc // 512)
        scratch = torch.zeros(N * ncg * 20 + 64, dtype=torch.uint8, device=dev)
        wl, bk = np.zeros(N * ncg, np.int32), np.zeros(4 * N * ncg, np.int32)
        report("encoder_backward 65536x768 (device kernels; the host bucket sort is not in these figures)",
               measure(lambda: L.llmk_encoder_backward(p(dwte), p(dwpe), p(scratch), wl.ctypes.data_as(C.c_void_p), bk.ctypes.data_as(C.c_void_p),
                                                       p(dout), p(tok), tok_host.ctypes.data_as(C.c_void_p), B, T, Cc, 42, None)))
        del wte, dwte, o, dout

    if want("classifier"):
        logits = torch.empty(N, Vp, device=dev, dtype=torch.bfloat16)
        src = randn(2048, Vp)
        tgt = torch.randint(0, V, (N,), device=dev, dtype=torch.int32, generator=g)
        losses = torch.zeros(N, device=dev)

        def refill():                                           # the kernel works in place: give it logits again
            for i in range(0, N, 2048):
                logits[i:i + 2048].copy_(src)
        report("fused_classifier 65536x50304", measure(lambda: L.llmk_fused_classifier(p(logits), p(losses), 1.0 / N, p(tgt), B, T, V, Vp, 1, None), prepare=refill))
        del logits, src
        torch.cuda.empty_cache()

    if want("adamw"):
        P = 124475904
        params, grads = randn(P, scale=0.02), randn(P, scale=0.01)
        master = params.float()
        m, v = torch.zeros(P, device=dev), torch.zeros(P, device=dev)
        report("adamw_update 124475904 params",
               measure(lambda: L.llmk_adamw_update(p(params), p(master), p(grads), p(m), p(v), P, 0, 0, 0, 1, 6e-4, 0.9, 0.95, 1, 1e-8, 0.1, 1.0, 7, None)))
        nb = C.c_int(1)
        maxb = L.llmk_get_max_num_block_sums(C.byref(nb), 1)
        partial = torch.zeros(maxb, device=dev)
        report("global_norm_squared 124475904 grads", measure(lambda: L.llmk_global_norm_squared(p(partial), p(grads), P, 0, 1, maxb, 1, None)))
        del params, grads, master, m, v

    if want("attention"):
        qkv = randn(B, T, 3 * Cc, scale=0.5)
        o = torch.empty(B, T, Cc, device=dev, dtype=torch.bfloat16)
        stats = torch.empty(B * NH * T, device=dev)
        report("attention_forward B64 NH12 T1024 hs64", measure(lambda: L.llmk_attention_forward(p(o), p(stats), p(qkv), B, T, NH, Cc, None)))
        dout, dqkv = randn(B, T, Cc, scale=0.1), torch.empty_like(qkv)
        report("attention_backward B64 NH12 T1024 hs64",
               measure(lambda: L.llmk_attention_backward(p(dqkv), p(dout), p(qkv), p(o), p(stats), B, T, NH, Cc, None)))

    L.llmk_profile_reset()
    del flush_buf
    torch.cuda.empty_cache()
    return results


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--only", default="")
    ap.add_argument("--json", default="")
    ap.add_argument("--variant", default="", help="time lib/variants/NAME/libllmk_bf16.so (python llm.c_amd/build.py --variant NAME "
                    "-D...: a build with ablation switches set, whose results are wrong by design) instead of the product library")
    ap.add_argument("--against", default="", help="comma-separated variant names: time them in turn with the product library, in this process")
    args = ap.parse_args()
    if args.variant and args.against:
        ap.error("--variant replaces the product library, --against runs beside it: give one of them")
    product_dir = pkg.LIBDIR
    if args.variant:
        pkg.LIBDIR = os.path.join(product_dir, "variants", args.variant)
    L = pkg.load("bf16")          # raises LibraryMissing when the HIP library has not been built
    L.llmk_init(0)
    others = []
    for tag in [t for t in args.against.split(",") if t]:
        path = os.path.join(product_dir, "variants", tag, "libllmk_bf16.so")
        if not os.path.exists(path):
            raise pkg.LibraryMissing(f"{path} not found: python llm.c_amd/build.py --variant {tag} -D...")
        lib = pkg.bind(C.CDLL(path))
        lib.llmk_init(0)
        others.append((tag, lib))
    results = run_cases(L, args.reps, [s for s in args.only.split(",") if s], lambda line: print(line, flush=True), others)
    if args.json:
        with open(args.json, "w") as f:
            json.dump({"reps": args.reps, "peak_tflops": PEAK_TFLOPS, "peak_gbs": PEAK_GBS, "results": results}, f, indent=1)


if __name__ == "__main__":
    main()
