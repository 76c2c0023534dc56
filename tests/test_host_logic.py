"""Host logic under AddressSanitizer and UBSan: descriptor gate, layout, repack round trips on exactly sized
buffers and the invariants of every launch plan (tests/host/plan_check.cpp), compiled here with g++ and run as a
child process.  No GPU is involved: the kernel launchers are stubs."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host compiler")
def test_plans_and_repacker_under_sanitizers(tmp_path):
    exe = str(tmp_path / "plan_check")
    src = [os.path.join(ROOT, "tests", "host", "plan_check.cpp"),
           os.path.join(ROOT, "openvino_amd", "csrc", "plan.cpp"), os.path.join(ROOT, "openvino_amd", "csrc", "repack.cpp")]
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-static-libasan", "-static-libubsan", "-pthread", "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(ROOT, "openvino_amd", "csrc"), "-o", exe] + src
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr[-4000:]
    env = {k: v for k, v in os.environ.items() if not k.startswith("OVFCC_")}
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0"
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, (run.stdout[-4000:], run.stderr[-4000:])
    assert "0 failures" in run.stdout
