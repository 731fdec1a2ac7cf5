"""Build libmpsa.so (hand-written HIP kernels + C ABI) for gfx950 with plain hipcc.

    python mp-sparse-attn_amd/build.py

The library lands in ``mp-sparse-attn_amd/lib/libmpsa.so`` next to the sources (in-tree).
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libmpsa.so")
# measurement kernels that bench.py loads by itself; not part of the library or its header
BENCH_LIB = os.path.join(LIBDIR, "libmpsa_bench.so")
BENCH_SOURCES = ["bench/mfma_stream.hip"]

SOURCES = ["api.hip", "formats.hip", "quantize.hip", "v_tiles.hip", "prepare.hip", "gemm_mx.hip", "attn_fwd.hip", "attn_fwd_skip.hip", "attn_fwd_routed.hip", "attn_fwd_pp.hip", "route.hip", "skip_route.hip"]

# packed-fp32 instructions are switched off on purpose (the flag is for the device pass; the host
# pass warns that it does not know the feature, which is harmless)
COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# skip_route.hip: without -fno-honor-nans (device pass only: the host side tests its arguments for NaN) every two-input
# maximum of the row-maximum trees gets an instruction per operand that only quiets signalling NaNs (a fifth of the trees'
# instructions); scores are never NaN unless a scale byte is
PER_FILE = {"quantize.hip": ["-ffp-contract=off"], "formats.hip": ["-ffp-contract=off"], "prepare.hip": ["-ffp-contract=off"],
            "route.hip": ["-ffp-contract=off"], "skip_route.hip": ["-ffp-contract=off", "-Xarch_device", "-fno-honor-nans"]}


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_lib(verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    hipcc = _hipcc()

    def compile_one(src):
        obj = os.path.join(objdir, src.replace("/", "_").replace(".hip", ".o"))
        out = _run([hipcc] + COMMON + PER_FILE.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + len(BENCH_SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES + BENCH_SOURCES))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs[:len(SOURCES)])
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", BENCH_LIB] + objs[len(SOURCES):])
    return LIB


if __name__ == "__main__":
    print(build_lib(verbose="-v" in sys.argv))
