"""The argument validation of the C ABI under AddressSanitizer and UndefinedBehaviorSanitizer, on the host only.

capi.hip is compiled for the host (no device pass), linked with stand-ins for the kernel launchers
(tests/capi_host/stubs.cpp) and driven by tests/capi_host/check.cpp with bad arguments of every kind; a sanitizer report
or a wrong status / message fails the test.  Nothing here touches a GPU, and no GPU code is ever built with a sanitizer.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not found")
def test_capi_validation_under_asan_and_ubsan(tmp_path):
    csrc = os.path.join(ROOT, "spargeattn_amd", "csrc")
    host = os.path.join(ROOT, "tests", "capi_host")
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined"]
    common = [HIPCC, "--cuda-host-only", "-x", "hip", "-O1", "-g", "-std=c++17", "-fno-omit-frame-pointer",
              "-Wno-unused-command-line-argument", f"-I{csrc}"]
    objs = []
    for src in (os.path.join(csrc, "capi.hip"), os.path.join(host, "stubs.cpp"), os.path.join(host, "check.cpp")):
        obj = str(tmp_path / (os.path.basename(src) + ".o"))
        r = subprocess.run(common + san + ["-c", src, "-o", obj], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-4000:]
        objs.append(obj)
    exe = str(tmp_path / "capi_host_check")
    r = subprocess.run([HIPCC, "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-o", exe] + objs,
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=120)
    assert r.returncode == 0 and "capi host checks ok" in r.stdout, (r.stdout[-3000:], r.stderr[-3000:])
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr[-3000:]
    shutil.rmtree(tmp_path, ignore_errors=True)
