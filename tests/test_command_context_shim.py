"""include/guffin_hip_command_context.hpp compiles against the reference's public headers with every method
the reference's engine calls, in the reference's argument types (syntax only: the reference's own sources
need Objective-C++ to link).  Skipped where the reference checkout or the HIP headers are absent."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = "/root/reference/include"
ROCM = "/opt/rocm/include"


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference checkout is not present")
@pytest.mark.skipif(not os.path.exists(os.path.join(ROCM, "hip", "hip_runtime_api.h")), reason="no HIP headers")
@pytest.mark.skipif(shutil.which("g++") is None, reason="no g++")
def test_the_shim_compiles_against_the_reference_headers():
    cmd = ["g++", "-std=c++20", "-fsyntax-only", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(ROOT, "include"), "-I", REFERENCE, "-I", ROCM,
           os.path.join(ROOT, "tests", "shim", "command_context_probe.cpp")]
    run = subprocess.run(cmd, capture_output=True, text=True)
    assert run.returncode == 0, run.stderr[-4000:]
