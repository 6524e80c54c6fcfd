"""The loop that runs a step's command buffer (kllm_amd/csrc/executor.hpp), built for the CPU
with stand-in entry points and run under AddressSanitizer and UndefinedBehaviorSanitizer."""

import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "kllm_amd", "csrc")


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host compiler")
def test_command_loop_under_sanitizers(tmp_path):
    exe = str(tmp_path / "executor_host_check")
    build = subprocess.run(
        ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-Wall",
         "-Werror", "-I", CSRC, os.path.join(HERE, "executor_host_check.cpp"), "-o", exe],
        capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0 and "executor host check: ok" in run.stdout, run.stdout[-2000:] + run.stderr[-3000:]
