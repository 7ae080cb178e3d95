"""Builds the gfx950 shared libraries in-tree:  lib/libllmk_bf16.so  and  lib/libllmk_fp32.so, and the trainer
programs lib/train_gpt2_bf16 and lib/train_gpt2_fp32 linked against them.

Each library = the HIP kernels (csrc/*.hip) + the host GPT-2 driver and data path (driver/*.cpp) compiled for
one storage precision, the way the reference builds one binary per PRECISION (reference
Makefile:232-244). hipcc cross-compiles for gfx950, so this also runs on a machine without a GPU.

    python llm.c_amd/build.py            # both precisions
    python llm.c_amd/build.py bf16       # one
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
                  "gemm.hip", "attention.hip"]
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


def build(precisions=("bf16", "fp32"), jobs=8, verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIBDIR, exist_ok=True)
    tasks = []
    objs = {p: [] for p in precisions}
    for p in precisions:
        od = os.path.join(OBJDIR, p)
        os.makedirs(od, exist_ok=True)
        for src in KERNEL_SOURCES:
            o = os.path.join(od, src + ".o")
            objs[p].append(o)
            tasks.append([hipcc, *COMMON, *PREC_DEFS[p], "-c", os.path.join(CSRC, src), "-o", o])
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


if __name__ == "__main__":
    precs = tuple(sys.argv[1:]) or ("bf16", "fp32")
    for path in build(precs, verbose=True):
        print(path)
