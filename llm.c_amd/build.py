"""Builds the gfx950 shared libraries in-tree:  lib/libllmk_bf16.so  and  lib/libllmk_fp32.so, and the trainer
programs lib/train_gpt2_bf16 and lib/train_gpt2_fp32 linked against them.

Each library = the HIP kernels (csrc/*.hip) + the host GPT-2 driver and data path (driver/*.cpp) compiled for
one storage precision, the way the reference builds one binary per PRECISION (reference
Makefile:232-244). hipcc cross-compiles for gfx950, so this also runs on a machine without a GPU.

    python llm.c_amd/build.py            # both precisions
    python llm.c_amd/build.py bf16       # one
    python llm.c_amd/build.py --variant noloads -DLLMK_GEMM_ABL=1   # a measurement build beside the product library
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
DRIVER = os.path.join(HERE, "driver")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")

KERNEL_SOURCES = ["runtime.hip", "layernorm.hip", "gelu.hip", "encoder.hip", "classifier.hip", "optimizer.hip",
                  "gemm.hip", "gemm_tn.hip", "attention.hip"]
# options of single files: the weight-gradient GEMM kernels take the compiler's "max-ilp" instruction scheduling (measured
# per kernel family, each variant loaded beside the product in one process: these kernels -1.2 to -2.7 %, every other GEMM
# kernel +2 to +8 %, attention forward -1.5 %, dQ 0, dK/dV +9 %)
# The other GEMM kernels and attention: the pre-register-allocation scheduler working bottom-up only (same method: dinp
# GEMMs -2 to -3.7 % (K = 3072 and the LM head), forward GEMMs -0.4 to -2.2 %, the GELU epilogue kernels +0.5 %, attention
# dK/dV -1.5 %, forward and dQ unchanged; top-down only: every GEMM kernel +10 to +19 %).
FILE_FLAGS = {"gemm_tn.hip": ["-mllvm", "-amdgpu-sched-strategy=max-ilp"],
              "gemm.hip": ["-mllvm", "-misched-prera-direction=bottomup"],
              "attention.hip": ["-mllvm", "-misched-prera-direction=bottomup"]}
DRIVER_SOURCES = ["gpt2.cpp", "data.cpp"]

# -packed-fp32-ops off: this toolchain's packed fp32 instructions are not trusted on this hardware pool
# -amdgpu-mfma-vgpr-form: keep MFMA accumulators in ordinary VGPRs. The softmax between the two MFMA groups of the
# attention kernels works on accumulator values; with AGPR accumulators every value is copied out and back.
COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-mfma-vgpr-form=1"]
PREC_DEFS = {"bf16": [], "fp32": ["-DLLMK_FP32"]}


def lib_path(precision):
    return os.path.join(LIBDIR, f"libllmk_{precision}.so")


def trainer_path(precision):
    return os.path.join(LIBDIR, f"train_gpt2_{precision}")


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


def variant_dir(name):
    return os.path.join(LIBDIR, "variants", name)


def build(precisions=("bf16", "fp32"), jobs=8, verbose=False, variant=None, defines=()):
    """variant: build lib/variants/<variant>/libllmk_<precision>.so with the extra -D defines instead of the product
    library (measurement builds for microbench.py --variant: ablation switches of the kernels; nothing loads them by
    default and they are not part of what tests, bench.py or the trainer run)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIBDIR, exist_ok=True)
    if variant:
        return _build_variant(hipcc, precisions, variant, list(defines), jobs, verbose)
    tasks = []
    objs = {p: [] for p in precisions}
    for p in precisions:
        od = os.path.join(OBJDIR, p)
        os.makedirs(od, exist_ok=True)
        for src in KERNEL_SOURCES:
            o = os.path.join(od, src + ".o")
            objs[p].append(o)
            tasks.append([hipcc, *COMMON, *FILE_FLAGS.get(src, []), *PREC_DEFS[p], "-c", os.path.join(CSRC, src), "-o", o])
        for src in DRIVER_SOURCES:
            o = os.path.join(od, src + ".o")
            objs[p].append(o)
            tasks.append([hipcc, *COMMON, *PREC_DEFS[p], "-x", "hip", "-c", os.path.join(DRIVER, src), "-o", o])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for out in ex.map(_run, tasks):
            if verbose and out.strip():
                print(out)
    for p in precisions:
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path(p), *objs[p]])
        if verbose:
            print("built", lib_path(p))
        # the trainer program (the reference's main loop) against that library; found next to it at run time
        _run([hipcc, "-O2", "-std=c++17", "-Wall", "-x", "hip", "--offload-arch=gfx950", os.path.join(DRIVER, "train_gpt2.cpp"),
              "-o", trainer_path(p), "-L" + LIBDIR, f"-lllmk_{p}", "-Wl,-rpath,$ORIGIN"])
    return [lib_path(p) for p in precisions]


def _build_variant(hipcc, precisions, variant, defines, jobs, verbose):
    out = []
    for p in precisions:
        od = os.path.join(OBJDIR, f"{p}_{variant}")
        os.makedirs(od, exist_ok=True)
        os.makedirs(variant_dir(variant), exist_ok=True)
        tasks, objs = [], []
        for src in KERNEL_SOURCES:
            o = os.path.join(od, src + ".o")
            objs.append(o)
            tasks.append([hipcc, *COMMON, *FILE_FLAGS.get(src, []), *PREC_DEFS[p], *defines, "-c", os.path.join(CSRC, src), "-o", o])
        for src in DRIVER_SOURCES:
            o = os.path.join(od, src + ".o")
            objs.append(o)
            tasks.append([hipcc, *COMMON, *PREC_DEFS[p], *defines, "-x", "hip", "-c", os.path.join(DRIVER, src), "-o", o])
        with ThreadPoolExecutor(max_workers=jobs) as ex:
            for text in ex.map(_run, tasks):
                if verbose and text.strip():
                    print(text)
        path = os.path.join(variant_dir(variant), f"libllmk_{p}.so")
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", path, *objs])
        out.append(path)
    return out


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument("precisions", nargs="*", default=[])
    ap.add_argument("--variant", default=None, help="build lib/variants/NAME/ with the given -D switches instead of the product library")
    args, extra = ap.parse_known_args()
    defines = [a for a in extra if a.startswith("-D")]
    if [a for a in extra if not a.startswith("-D")]:
        ap.error("unknown arguments: " + " ".join(a for a in extra if not a.startswith("-D")))
    precs = tuple(args.precisions) or (("bf16",) if args.variant else ("bf16", "fp32"))
    for path in build(precs, verbose=True, variant=args.variant, defines=defines):
        print(path)
