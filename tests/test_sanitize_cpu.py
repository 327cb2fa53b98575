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
FLAGS = ["-std=c++20", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
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


def test_plugin_entry_and_reference_lifetimes_under_sanitizers(tmp_path):
    # moodistGetApi -> CoreApi table with a fake WrapperApi: handshake, off-path slots, handle
    # ownership, and tensor references held from a rank's post until the collective's launch
    r = build_and_run(tmp_path, "plugin_driver.cc",
                      ["planner.cc", "processgroup.cc", "c_api.cc", "hip_loader.cc", "plugin.cc"])
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-3000:])
    assert "plugin driver done" in r.stdout


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="the driver's tensors are fake addresses: on a machine with a "
                    "GPU the launch it provokes would really run and fault")
def test_plugin_entry_of_the_built_library_through_dlsym(tmp_path):
    # the same walk against the shipped libmoodist.so: dlopen + dlsym("moodistGetApi"), the
    # driver's own destroy() going back through the table
    import ctypes

    lib = os.path.join(ROOT, "moodist_amd", "libmoodist.so")
    exe = str(tmp_path / "driver")
    # the driver checks the table's magic against its own: compiled with the built library's
    L = ctypes.CDLL(lib)
    L.moodist_build_magic.restype = ctypes.c_uint64
    subprocess.run(["g++", "-std=c++20", "-O1", "-g", "-DMOODIST_DRIVER_DLOPEN",
                    "-DMOODIST_BUILD_MAGIC=0x%xULL" % L.moodist_build_magic(), "-I" + os.path.join(ROOT, "include"),
                    os.path.join(HERE, "sanitize", "plugin_driver.cc"), "-ldl", "-o", exe],
                   check=True, capture_output=True, text=True)
    r = subprocess.run([exe, lib], cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-3000:])
    assert "plugin driver done" in r.stdout
