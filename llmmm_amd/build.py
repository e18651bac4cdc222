"""Builds ``libllmmm.so`` (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

``python llmmm_amd/build.py`` (run as a script: importing the package needs the library this
builds).  hipcc cross-compiles without a GPU; the resulting library sits next to this file so
that it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libllmmm.so")

COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed fp32 VALU ops are kept off for every device file
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# per-file extras: the FP8 kernels promote MFMA results with VALU FMAs, so the MFMA must
# write architectural VGPRs rather than AGPRs
SOURCES = {
    "fp16_gemm.hip": [],
    "fp8_gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "fp8_skinny.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "quant_fp8.hip": [],
    "layout.hip": [],
    "probe.hip": [],
    "static_ws.hip": [],
    "capi.cpp": ["-x", "hip"],
}


def _compile(item):
    name, extra = item
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ, os.path.splitext(name)[0] + ".o")
    cmd = ["hipcc"] + COMMON + extra + ["-c", src, "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (name, out))
    return obj, out


def build(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        results = list(pool.map(_compile, SOURCES.items()))
    objs = [o for o, _ in results]
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    return LIB


def build_dropin_test():
    """Compile tests/cpp/dropin_test.cpp (the C++ drop-in shims of include/llmmm/mm) against the library."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "cpp", "dropin_test.cpp")
    out = os.path.join(root, "tests", "cpp", "dropin_test")
    cmd = ["hipcc", "-std=c++17", "-O1", "-Wno-unused-command-line-argument", "-I", os.path.join(root, "include"), "-o", out, src,
           "-L", HERE, "-lllmmm", "-Wl,-rpath,$ORIGIN/../../llmmm_amd"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for dropin_test.cpp:\n" + res.stdout)
    return out


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    print(build_dropin_test())
