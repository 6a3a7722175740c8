"""CPU: the library's host-side occupancy code (habitat_amd/csrc/occupancy.h
compiled as plain C++) under AddressSanitizer and UndefinedBehaviorSanitizer,
fuzzed against the CPU oracle and its own two formulations
(tests/native/occupancy_fuzz.cpp)."""
import os
import shutil
import subprocess

import pytest

from conftest import ROOT


def test_occupancy_host_code_is_clean_under_asan_and_ubsan(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++")
    exe = str(tmp_path / "occupancy_fuzz")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=all", "-Wall", "-Wextra", "-o", exe,
           os.path.join(ROOT, "tests", "native", "occupancy_fuzz.cpp"),
           "-x", "c", os.path.join(ROOT, "oracle", "occupancy.c")]
    built = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert built.returncode == 0, built.stdout
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)      # the sanitizer runtime must come first in the process
    run = subprocess.run([exe, "400", "2000"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True, env=env, timeout=300)
    assert run.returncode == 0, run.stdout[-3000:]
    assert run.stdout.startswith("ok:"), run.stdout
