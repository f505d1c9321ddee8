"""Builds libspargeattn_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m spargeattn_amd.build            # compile + link
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libspargeattn_amd.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

COMMON = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# translation unit -> extra flags.  The bit-exact stages forbid fused multiply-add contraction.
SOURCES = {
    "maskpred.hip": ["-ffp-contract=off"],
    "vquant.hip": ["-ffp-contract=off"],
    "attn.hip": [],
    "dense.hip": [],
    "capi.hip": ["-fvisibility=default"],
}


def _compile(item):
    src, extra = item
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [HIPCC, *COMMON, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{' '.join(cmd)}\n{err}")
    return obj, err


def build(verbose=True):
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as ex:
        results = list(ex.map(_compile, SOURCES.items()))
    objs = [o for o, _ in results]
    if verbose:
        for (_, err), src in zip(results, SOURCES):
            if err.strip():
                print(f"[{src}]\n{err}", file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build())
