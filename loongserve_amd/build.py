"""Build recipe for liblsattn.so (hand-written HIP kernels + C ABI, gfx950 only).

`python -m loongserve_amd.build` compiles loongserve_amd/csrc/*.hip with hipcc into
loongserve_amd/liblsattn.so.  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "liblsattn.so")
CEILING_LIB_PATH = os.path.join(PKG_DIR, "libls_ceiling.so")  # measurement aids of bench.py (include/ls_ceiling.h)
SOURCES = ["prefill.hip", "prefill_small.hip", "decode.hip", "merge_scatter.hip", "elementwise.hip", "pool.hip"]
# elementwise.hip reproduces the reference's half arithmetic operation by operation: no fused multiply-adds
# other than the ones it writes
FILE_FLAGS = {
    "elementwise.hip": ["-ffp-contract=off"],
    # prefill.hip only: no NaN is ever produced on a valid path of its loop (infinities are, and stay honoured); this drops
    # the v_max x,x,x canonicalisation in front of every fmaxf of the softmax phase, the scarce one there
    "prefill.hip": ["-fno-honor-nans"],
}

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed-fp32 VALU forms are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    "-Wno-unused-result",
]


def _compile(src: str, extra) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *FILE_FLAGS.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr[-6000:]))
    # the host pass warns that it does not know the packed-fp32 feature; that is expected
    return obj


def build_all(verbose: bool = False, extra_flags=(), out: str = LIB_PATH) -> str:
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        objs = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-6000:]))
    if verbose:
        print("built", out)
    return out


def build_ceiling(verbose: bool = False, out: str = CEILING_LIB_PATH) -> str:
    """libls_ceiling.so: the MFMA stream and the streaming read that bench.py measures a box's sustained ceilings with."""
    obj = _compile("ceiling.hip", [])
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", obj, "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-6000:]))
    if verbose:
        print("built", out)
    return out


C_ABI_EXAMPLES = [os.path.join(ROOT, "tests", "c_abi", n) for n in ("decode_from_c", "prefill_from_c")]


def build_c_abi_example(verbose: bool = False):
    """The C ABI's consumers without Python or PyTorch (tests/c_abi/*.cpp), linked against the in-tree library and
    finding it relative to their own place; tests/test_gpu_c_abi.py runs them."""
    for out in C_ABI_EXAMPLES:
        cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-I" + os.path.join(ROOT, "include"), out + ".cpp",
               "-L" + PKG_DIR, "-llsattn", "-Wl,-rpath,$ORIGIN/../../loongserve_amd", "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for the C ABI example:\n%s\n%s" % (" ".join(cmd), r.stderr[-6000:]))
        if verbose:
            print("built", out)
    return C_ABI_EXAMPLES


if __name__ == "__main__":
    build_all(verbose=True, extra_flags=sys.argv[1:])
    build_ceiling(verbose=True)
    build_c_abi_example(verbose=True)
