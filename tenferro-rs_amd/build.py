"""Builds libtenferro_hip.so (the C-ABI library) in-tree with hipcc for gfx950.

    python tenferro-rs_amd/build.py [--force]

Every source is compiled to an object under csrc/build/ (in parallel) and linked into
tenferro-rs_amd/libtenferro_hip.so.  hipcc cross-compiles without a GPU.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libtenferro_hip.so")
SOURCES = ["errors.cpp", "plan.cpp", "prims.cpp", "einsum.cpp", "contract_cache.cpp", "runtime.cpp", "k_copy.hip", "k_reduce.hip", "k_gemm.hip", "k_gemm_skinny.hip", "k_gemm_wave.hip", "k_gemm_tiny.hip", "k_gemm_bfirst.hip", "k_gemm_thin.hip", "k_dot.hip", "static_scratch.hip",
           "k_gemm128_f32.hip", "k_gemm128_f64.hip", "k_gemm128_c64.hip", "k_gemm128_c128.hip",
           "k_gemm64_f32.hip", "k_gemm64_f64.hip", "k_gemm64_c64.hip", "k_gemm64_c128.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 instruction selection is switched off for all device code
FLAGS = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _newer(src, dst):
    if not os.path.exists(dst):
        return True
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    deps.append(os.path.join(HERE, "..", "include", "tenferro_hip.h"))
    return any(os.path.getmtime(d) > os.path.getmtime(dst) for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    if not force and not _newer(src, obj):
        return obj, ""
    cmd = [HIPCC] + FLAGS + ["-x", "hip", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, r.stderr[-8000:]))
    return obj, r.stderr


def build(force=False, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    with ThreadPoolExecutor(max_workers=min(12, len(srcs))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), srcs))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                sys.stderr.write(err)
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr[-8000:])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
