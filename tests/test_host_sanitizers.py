"""The library's host code (validators, planners, workspace sizing) under AddressSanitizer + UndefinedBehaviorSanitizer.

Host pass only: the sanitizer flags follow `-Xarch_host`, the device pass is compiled as always.  The instrumented
fa_rocm_api.cpp is linked with a driver that sweeps edge values through every integer field of the two argument
records (tests/native/host_sanitize_driver.cpp) and runs without a GPU; a sanitizer report aborts it."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
SAN = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host", "-fno-sanitize-recover=all",
       "-Xarch_host", "-fno-omit-frame-pointer"]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_validators_and_planners_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "host_sanitize_driver")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-x", "hip",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", *SAN,
           os.path.join(ROOT, "flash-attention-npu_amd", "csrc", "fa_rocm_api.cpp"),
           os.path.join(ROOT, "tests", "native", "host_sanitize_driver.cpp"),
           "-fsanitize=address", "-fsanitize=undefined", "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, f"sanitizer build failed:\n{r.stdout}\n{r.stderr[-4000:]}"
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, f"driver failed ({r.returncode}):\n{r.stdout[-2000:]}\n{r.stderr[-6000:]}"
    assert "host sanitizer sweep" in r.stdout
    shutil.rmtree(tmp_path, ignore_errors=True)
