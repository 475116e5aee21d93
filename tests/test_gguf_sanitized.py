"""The GGUF reader and the weight binding (host code: guffin_amd/csrc/gguf.cpp) compiled with g++ under
AddressSanitizer and UndefinedBehaviorSanitizer and driven over 20 000 damaged copies of a small model image
(tests/sanitize/gguf_damage_run.cpp): no report, every image either parsed or refused."""
import os
import shutil
import subprocess
from dataclasses import replace

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_reader_and_binding_under_sanitizers(tmp_path):
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    from guffin_amd import model
    from gguf_image import write_gguf
    binary = str(tmp_path / "gguf_damage_run")
    build = subprocess.run(["g++", "-std=c++20", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                            "-fno-omit-frame-pointer", "-I", os.path.join(ROOT, "include"),
                            os.path.join(HERE, "sanitize", "gguf_damage_run.cpp"),
                            os.path.join(ROOT, "guffin_amd", "csrc", "gguf.cpp"), "-o", binary], capture_output=True, text=True)
    if build.returncode != 0 and "asan" in build.stderr.lower():
        pytest.skip("this g++ has no sanitizer runtime")
    assert build.returncode == 0, build.stderr
    shape = replace(model.GEMMA3_270M, layers=1, vocab=256, hidden=64, ffn=128)
    image = str(tmp_path / "image.gguf")
    np.array(write_gguf(model.HostModel(shape, seed=1, position=0))).tofile(image)
    run = subprocess.run([binary, image, "20000"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "ERROR" not in run.stderr and "runtime error" not in run.stderr, run.stderr
    words = run.stdout.split()
    parsed, refused, bound = int(words[1]), int(words[3]), int(words[5])
    assert parsed + refused == 20000 and parsed > 1000 and refused > 1000 and bound > 1000
