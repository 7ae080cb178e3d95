#!/usr/bin/env python3
"""Throughput of the GPT-2 124M training step (bf16, B=64, T=1024) on one MI355X through the C ABI,
with the reference's CPU trainer timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-kernel-events]

A step = gpt2_forward + gpt2_backward_and_reduce + gpt2_calculate_grad_norm (clip at 1.0) + gpt2_update
on one batch of synthetic tokens, exactly the work of one iteration of the reference's training loop
(train_gpt2.cu:1829-1852) with grad_accum_steps = 1. Prints one JSON line.
"""
import argparse
import ctypes as C
import importlib.util
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA, vendor figure
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E, vendor figure
METRIC = "train tokens/sec + MFU, GPT-2 124M bf16 B=64 T=1024, 1 MI355X"

# Bytes per launch (read + written, averaged over the launches of a step) that the GEMM families move between L2 and
# the memory side, from two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE) over this same workload, scaled by what
# the counters read for a copy kernel of known size (profiles/train_step_gpt2_124M_b64_t1024_hbm_traffic.txt has the
# commands and the table). Valid for the default workload only. FETCH_SIZE counts L2 fills whether the Infinity Cache
# or HBM served them.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {"gemm_nn": 933442355, "gemm_nn_dgelu": 1439589990, "gemm_tn_splitk": 824298433,
                                     "gemm_nt": 888288405, "gemm_nt_gelu": 1286917324}

# kernel families timed by the library -> roofline that bounds them
MFMA_BOUND = {"gemm_nt", "gemm_nt_gelu", "gemm_nn", "gemm_nn_dgelu", "gemm_tn", "gemm_tn_splitk",
              "attention_forward", "attention_backward_dkdv", "attention_backward_dq"}


def package():
    spec = importlib.util.spec_from_file_location("llmc_amd", os.path.join(ROOT, "llm.c_amd", "__init__.py"))
    m = importlib.util.module_from_spec(spec)
    sys.modules["llmc_amd"] = m
    spec.loader.exec_module(m)
    return m


def cpu_baseline(budget_s=14.0):
    """The reference's CPU trainer (oracle/_ref, compiled from train_gpt2.c; falls back to this repo's
    restatement) on the reference's own CPU-runnable case: 124M, B=4, T=64, 10-step recipe, bounded in time."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as ol
    cfg = ol.Config(1024, 50257, 50304, 12, 12, 768)
    B, T = 4, 64
    params = ol.init_params(cfg, 42)
    inp, tgt = ol.make_tokens(B, T, cfg.vocab_size, 1337)
    hyper = dict(lr=1e-4, b1=0.9, b2=0.999, eps=1e-8, wd=0.0)
    kind = "reference" if ol.have_ref() else "port"
    ms = []
    t_start = time.time()
    if kind == "reference":
        with tempfile.TemporaryDirectory() as d:
            path = os.path.join(d, "gpt2_124M_seed42.bin")
            assert ol.cref().cref_write_checkpoint_fp32(path.encode(), params, C.byref(cfg)) == 0
            # one call = checkpoint load + N steps; run 1 step first to size N
            r = ol.ref_train(path, cfg, inp, tgt, B, T, 2, **hyper)
            per = float(r["step_ms"][1]) / 1e3
            n = int(max(2, min(10, (budget_s - (time.time() - t_start)) / max(per, 1e-3))))
            r = ol.ref_train(path, cfg, inp, tgt, B, T, n, **hyper)
            ms = [float(x) for x in r["step_ms"][1:]]
        cores = ol.ref().ref_num_threads()
    else:
        r = ol.cref_train(cfg, params, inp, tgt, B, T, 2, **hyper)
        per = float(r["step_ms"][1]) / 1e3
        n = int(max(2, min(10, (budget_s - (time.time() - t_start)) / max(per, 1e-3))))
        r = ol.cref_train(cfg, params, inp, tgt, B, T, n, **hyper)
        ms = [float(x) for x in r["step_ms"][1:]]
        cores = ol.cref().cref_num_threads()
    mean_ms = float(np.mean(ms))
    return {"value": B * T / (mean_ms / 1e3), "unit": "tokens/s", "cores": int(cores), "kind": kind,
            "ms_per_step": mean_ms,
            "sample": f"GPT-2 124M fp32 train step B=4 T=64 (BASELINE config 0), {len(ms)} timed steps after 1 untimed, "
                      f"OpenMP threads={cores}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--model", default="d12")
    ap.add_argument("--recompute", type=int, default=0)   # the reference's 124M recipe runs with -r 0 (scripts/run_gpt2_124M.sh)
    ap.add_argument("--gelu-fusion", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-events", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first launch one copy kernel of known size (128 MiB read, 256 MiB written): the yardstick for "
                         "scaling FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this command")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the training step on ONE GPU only (no collectives are part of it); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)

    # the native driver and the reference's CPU trainer print their model headers with printf: send everything
    # written to file descriptor 1 to stderr until the result line, so stdout carries exactly one JSON line
    sys.stdout.flush()
    real_stdout = os.dup(1)
    os.dup2(2, 1)

    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    pkg = package()
    L = pkg.load("bf16")           # raises if the HIP library is not built: there is no other path
    L.llmk_init(0)
    B, T = args.batch, args.seq
    default_workload = (B, T, args.model, args.recompute, args.gelu_fusion) == (64, 1024, "d12", 0, 2)
    h = L.gpt2_create()
    L.gpt2_set_options(h, 1, args.recompute, args.gelu_fusion)
    L.gpt2_build_from_descriptor(h, args.model.encode())
    L.gpt2_allocate_state(h, B, T)
    cfg = (C.c_int * 6)()
    L.gpt2_get_config(h, cfg)
    V = cfg[1]
    nparams = L.gpt2_num_parameters(h)
    rng = np.random.RandomState(0)
    stream = rng.randint(0, V, size=B * T + 1).astype(np.int32)    # uint16-range tokens, targets = inputs shifted by one
    inp, tgt = np.ascontiguousarray(stream[:-1]), np.ascontiguousarray(stream[1:])
    ip, tp = inp.ctypes.data_as(C.c_void_p), tgt.ctypes.data_as(C.c_void_p)

    if args.calibrate_copy:
        n = 64 * 1024 * 1024
        src = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
        dst = torch.empty(n, dtype=torch.float32, device="cuda")
        L.llmk_copy_and_cast_to_f32(dst.data_ptr(), src.data_ptr(), n, 0, 0, 1, None)
        torch.cuda.synchronize()
        del src, dst

    def step(t):
        L.gpt2_forward(h, ip, B, T)
        L.gpt2_backward_and_reduce(h, ip, tp, 1, 0)
        loss = L.gpt2_mean_loss(h)
        norm = L.gpt2_calculate_grad_norm(h)
        scale = 1.0 / norm if norm > 1.0 else 1.0
        L.gpt2_update(h, 6e-4, 0.9, 0.95, 1e-8, 0.1, scale, t, 0)
        return loss, norm

    def read_profile(nsteps):
        recs = []
        name = C.create_string_buffer(64)
        calls, ms, fl, by = C.c_int(), C.c_double(), C.c_double(), C.c_double()
        for i in range(L.llmk_profile_count()):
            L.llmk_profile_get(i, name, C.byref(calls), C.byref(ms), C.byref(fl), C.byref(by))
            n = name.value.decode()
            rec = {"kernel": n, "launches_per_step": calls.value / nsteps, "ms_per_step": ms.value / nsteps,
                   "avg_launch_ms": ms.value / max(calls.value, 1), "bytes_per_launch": by.value / max(calls.value, 1)}
            if n in MFMA_BOUND:
                rec.update(bound="mfma", achieved=fl.value / (ms.value * 1e-3) / 1e12 if ms.value > 0 else 0.0,
                           peak=PEAK_BF16_TFLOPS, unit="TFLOP/s")
            else:
                rec.update(bound="hbm", achieved=by.value / (ms.value * 1e-3) / 1e9 if ms.value > 0 else 0.0,
                           peak=PEAK_HBM_GBS, unit="GB/s")
            rec["frac"] = rec["achieved"] / rec["peak"]
            recs.append(rec)
        recs.sort(key=lambda r: -r["ms_per_step"])
        return recs

    # Warmup. Its last step is run with every kernel launch bracketed by HIP events: that gives the per-family
    # table and names the dominant family. In the timed region only that family carries events (bracketing all
    # ~400 launches of a step costs about 1.7 % of the step; one family costs about 0.2 %).
    losses = []
    kernels = []
    for w in range(args.warmup):
        last = (w == args.warmup - 1) and not args.no_kernel_events
        if last:
            torch.cuda.synchronize()
            L.llmk_profile_reset()
            L.llmk_profile_only(None)
            L.llmk_profile_enable(1)
        losses.append(step(w + 1)[0])
        if last:
            torch.cuda.synchronize()
            L.llmk_profile_enable(0)
            kernels = read_profile(1)
    torch.cuda.synchronize()
    dominant = kernels[0]["kernel"] if kernels else None
    if not args.no_kernel_events:
        L.llmk_profile_reset()
        L.llmk_profile_only(dominant.encode() if dominant else None)   # without a warmup step: every family
        L.llmk_profile_enable(1)
    t0 = time.perf_counter()
    for s in range(args.steps):
        losses.append(step(args.warmup + s + 1)[0])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    L.llmk_profile_enable(0)

    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = B * T * args.steps / dt
    mfu = L.gpt2_estimate_mfu(h, B * T, ctypes_float(dt / args.steps))

    roofline = None
    if not args.no_kernel_events:
        timed = read_profile(args.steps)
        if not kernels:
            kernels = timed
        d = timed[0]                           # the dominant family, timed live inside the timed steps
        roofline = {"kernel": d["kernel"], "bound": d["bound"], "achieved": d["achieved"], "peak": d["peak"],
                    "unit": d["unit"], "frac": d["frac"],
                    "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(d["kernel"]) if default_workload else None,
                    "algorithmic_bytes_per_launch": d["bytes_per_launch"],
                    "avg_launch_ms": d["avg_launch_ms"], "launches_per_step": d["launches_per_step"],
                    "ms_per_step": d["ms_per_step"]}
    L.gpt2_free(h)

    out = {
        "metric": METRIC, "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"GPT-2 {args.model} ({nparams} params) full train step, bf16 + fp32 master weights/AdamW, "
                               f"flash attention, clip 1.0" +
                               {("d12", 64, 1024): " (BASELINE configs[2])", ("d24", 32, 1024): " (BASELINE configs[3])",
                                ("d48", 16, 1024): " (BASELINE configs[4])"}.get((args.model, B, T), ""),
                   "global_batch": B, "seq_len": T, "tokens_per_step": B * T, "recompute": args.recompute,
                   "gelu_fusion": args.gelu_fusion, "parallelism": "single GPU"},
        "mfu": float(mfu), "mfu_peak_tflops": PEAK_BF16_TFLOPS,
        "loss_first": float(losses[0]), "loss_last": float(losses[-1]),
        "roofline": roofline, "kernels_from_last_warmup_step": kernels,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    C.CDLL(None).fflush(None)
    sys.stdout.flush()
    os.dup2(real_stdout, 1)
    os.close(real_stdout)
    print(json.dumps(out), flush=True)


def ctypes_float(x):
    return C.c_float(x)


if __name__ == "__main__":
    main()
