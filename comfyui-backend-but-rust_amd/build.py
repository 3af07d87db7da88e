"""Build libgpu_kernels.so (the C-ABI library of the gfx950 kernels) in-tree with hipcc.

hipcc cross-compiles for gfx950 without a GPU.  Objects are built in parallel, one per .hip file, then linked.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libgpu_kernels.so")
ARCH = os.environ.get("HIP_ARCH", "gfx950")
SOURCES = ["quant_rows.hip", "prologue_rows.hip", "weight_formats.hip", "act_tables.hip", "int8_gemm.hip", "w6.hip", "w6_requant.hip", "w6a8_group_gemm.hip", "attn_int8.hip"]
FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # exact arithmetic: no contraction except where fmaf is written, IEEE divide, no fast-math
    "-ffp-contract=off", "-fno-fast-math", "-fhip-fp32-correctly-rounded-divide-sqrt",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the DMA sequences name m0 as clobbered on purpose; the compiler remarks on every one
    "-Wno-inline-asm",
]
# Per-file additions.  The grouped W6A8 kernel reads every MFMA result with VALU instructions (int32 partial -> fp32),
# which cannot take accumulator registers as operands: keep its MFMA destinations in ordinary vector registers.
EXTRA = {"w6a8_group_gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _compile(src):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = ["hipcc", *FLAGS, *EXTRA.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


BLAS_OUT = os.path.join(HERE, "libgpu_blas.so")


def build_blas():
    """The dense-GEMM library over hipBLASLt: host code only."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    subprocess.check_call(["hipcc", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
                           os.path.join(CSRC, "blas_gemm.cpp"), "-o", BLAS_OUT, "-L" + os.path.join(rocm, "lib"), "-lhipblaslt",
                           "-Wl,-rpath," + os.path.join(rocm, "lib")])
    return BLAS_OUT


def stale():
    if not os.path.exists(OUT):
        return True
    t = os.path.getmtime(OUT)
    if not os.path.exists(BLAS_OUT):
        return True
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".hpp", ".cpp"))]
    deps.append(os.path.join(os.path.dirname(HERE), "include", "gpu_api.h"))
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=True):
    if not force and not stale():
        return OUT
    with concurrent.futures.ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        objs = list(ex.map(_compile, SOURCES))
    subprocess.check_call(["hipcc", "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", OUT, *objs])
    build_blas()
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
