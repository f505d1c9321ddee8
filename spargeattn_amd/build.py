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
# Translation units whose kernels read LDS through inline asm into registers the compiler believes are already
# written: a spill or a scratch copy between such a read and its wait would store stale data, so the build fails
# when any kernel of these files uses scratch memory or spills a vector register.  (Scalar registers parked in the
# lanes of a vector register - "SGPRs Spill" - never touch memory or the registers those reads write, and are allowed.)
NO_SPILL = {"attn.hip", "dense.hip"}
# Kernels of those files that issue EVERY inline-asm LDS read together with its wait (no window in which a register is
# in flight) may use scratch: the FP16-PV attention variants (template argument PV16 = true, "Lb1" in the mangled
# name), whose masked tail loop parks a few registers there.
SPILL_EXEMPT = ("block_sparse_attn_kernelILi128ELi0ELb1", "block_sparse_attn_kernelILi128ELi1ELb1",
                "block_sparse_attn_kernelILi64ELi0ELb1", "block_sparse_attn_kernelILi64ELi1ELb1")
RESOURCE_REMARKS = "-Rpass-analysis=kernel-resource-usage"
# The same kernels issue some LDS reads through inline asm and wait for them in a LATER asm statement (the reads run
# under matrix instructions).  In between, the compiler believes the destination registers are already written; the
# generated code of this compiler version was inspected for copies or live-range splits inside those windows and has
# none.  Another compiler may schedule differently: the build then says so, loudly, and asks for the check to be redone
# (SPARGEATTN_AMD_ALLOW_UNVALIDATED_COMPILER=1 silences the failure, not the warning).
VALIDATED_COMPILERS = ("roc-7.2.0",)


def _compiler_version():
    r = subprocess.run([HIPCC, "--version"], capture_output=True, text=True)
    return (r.stdout + r.stderr).strip()


def check_compiler():
    """Returns (ok, version text): ok when hipcc is one of the versions the inline-asm LDS windows were inspected with."""
    v = _compiler_version()
    return any(tag in v for tag in VALIDATED_COMPILERS), v


def _spill_report(stderr):
    """Kernel names of a -Rpass-analysis=kernel-resource-usage log that use scratch or spill vector registers."""
    bad, name = [], None
    for line in stderr.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        for key in ("ScratchSize [bytes/lane]:", "VGPRs Spill:"):
            if key in line:
                value = line.split(key)[1].split("[")[0].strip()
                if value != "0" and not any(tag in (name or "") for tag in SPILL_EXEMPT):
                    bad.append(f"{name}: {key} {value}")
    return bad


def _compile(item):
    src, extra = item
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    guard = [RESOURCE_REMARKS, "-fno-caret-diagnostics"] if src in NO_SPILL else []
    cmd = [HIPCC, *COMMON, *extra, *guard, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("is not a recognized feature for this target", RESOURCE_REMARKS)
    err = "\n".join(l for l in r.stderr.splitlines() if not any(n in l for n in noise))
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{' '.join(cmd)}\n{err}")
    if guard:
        bad = _spill_report(r.stderr)
        if bad:
            raise RuntimeError(f"{src}: kernels must not spill or use scratch memory:\n  " + "\n  ".join(bad))
    return obj, err


def build(verbose=True):
    ok, version = check_compiler()
    if not ok:
        msg = ("spargeattn_amd.build: hipcc is not a validated version (" + ", ".join(VALIDATED_COMPILERS) + "):\n  "
               + version.replace("\n", "\n  ") + "\nattn.hip / dense.hip read LDS through inline asm whose waits come "
               "later; re-inspect the generated code around those windows (or run the GPU parity tests) before trusting "
               "this build.")
        print("WARNING: " + msg, file=sys.stderr)
        if os.environ.get("SPARGEATTN_AMD_ALLOW_UNVALIDATED_COMPILER") != "1":
            raise RuntimeError(msg + "\nSet SPARGEATTN_AMD_ALLOW_UNVALIDATED_COMPILER=1 to build anyway.")
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


TORCH_EXT_LIB = os.path.join(HERE, "libspargeattn_amd_torch.so")


def build_torch_ext(verbose=True):
    """csrc/torch_ext.cpp -> libspargeattn_amd_torch.so: the torch.ops.spargeattn_amd.* registrations over the C ABI.
    Host code only (no kernel lives in the shim); links against libspargeattn_amd.so beside it and against torch."""
    import torch
    from torch.utils import cpp_extension as ce
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    obj = os.path.join(CSRC, "torch_ext.o")
    cmd = [HIPCC, "-x", "c++", "-O2", "-fPIC", "-std=c++17", "-fvisibility=hidden", "-Wno-unused-command-line-argument",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{p}" for p in ce.include_paths()], "-I/opt/rocm/include",
           "-c", os.path.join(CSRC, "torch_ext.cpp"), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"torch extension failed to compile:\n{' '.join(cmd)}\n{r.stderr[-6000:]}")
    cmd = [HIPCC, "-shared", "-fPIC", "-o", TORCH_EXT_LIB, obj, f"-L{HERE}", "-lspargeattn_amd", "-Wl,-rpath,$ORIGIN",
           f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"torch extension failed to link:\n{r.stderr[-6000:]}")
    return TORCH_EXT_LIB


if __name__ == "__main__":
    print(build())
    print(build_torch_ext())
