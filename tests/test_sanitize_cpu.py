"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer (CPU only, g++).

The drivers in tests/sanitize/ are compiled together with the host core's sources; a sanitizer
report aborts the driver and fails the test.
"""

import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CORE = os.path.join(ROOT, "moodist_amd", "csrc", "core")
FLAGS = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
         "-I" + CORE, "-I" + os.path.join(ROOT, "include")]


def build_and_run(tmp_path, driver, sources):
    exe = str(tmp_path / "driver")
    cmd = ["g++"] + FLAGS + [os.path.join(HERE, "sanitize", driver)] + [os.path.join(CORE, s) for s in sources] + \
        ["-ldl", "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0")
    return subprocess.run([exe], cwd=str(tmp_path), env=env, capture_output=True, text=True, timeout=300)


def test_planner_and_plan_messages_under_sanitizers(tmp_path):
    r = build_and_run(tmp_path, "planner_driver.cc", ["planner.cc"])
    assert r.returncode == 0, r.stderr[-3000:]
    assert "message fuzz done" in r.stdout


def test_c_api_handle_lifetimes_under_sanitizers(tmp_path):
    r = build_and_run(tmp_path, "c_api_driver.cc", ["planner.cc", "processgroup.cc", "c_api.cc", "hip_loader.cc"])
    assert r.returncode == 0, r.stderr[-3000:]
    assert "c api driver done" in r.stdout
