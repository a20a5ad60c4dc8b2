"""Build libhs_attn.so (hand-written HIP for gfx950) in-tree:  python -m hyprstream_amd.build

hipcc cross-compiles without a GPU.  Output: hyprstream_amd/lib/libhs_attn.so.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "libhs_attn.so")
HOST_LIB = os.path.join(LIBDIR, "libhs_kv_cache.so")

SOURCES = ["api.hip", "kv_quantize.hip", "decode_attn.hip", "prefill_attn.hip", "prefill_attn_wide.hip", "deltanet.hip", "deltanet_chunked.hip", "deltanet_glue.hip"]

COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math",
    # keep hipcc from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
# the quantizers must do exactly the fp32 operations written (bit-exact with the CPU oracle)
PER_FILE = {
    "kv_quantize.hip": ["-ffp-contract=off"],
}


def _compile(src, verbose):
    obj = os.path.join(OBJDIR, src.replace(".hip", ".o"))
    cmd = ["hipcc", "-c", os.path.join(CSRC, src), "-o", obj] + COMMON + PER_FILE.get(src, [])
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    if err.strip() and verbose:
        print(err)
    return obj


def build(verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # host-side LayerKVCache mirror: plain C++ over the C ABI above (it owns device memory, the kernels do not)
    hsrc = [os.path.join(HERE, "host", f) for f in ("kv_cache.cpp", "kv_cache_capi.cpp", "block_pool.cpp", "block_pool_capi.cpp", "kv_compat.cpp", "kv_compat_capi.cpp")]
    cmd = ["hipcc", "-shared", "-fPIC", "-O2", "-std=c++17", "-fvisibility=hidden", "-Wall", "-x", "hip", "--offload-arch=gfx950"]
    cmd += hsrc + ["-o", HOST_LIB, "-L" + LIBDIR, "-lhs_attn", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
