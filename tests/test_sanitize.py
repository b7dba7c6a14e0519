"""Host AddressSanitizer / UBSan runs of the CPU-side code: the oracle and the library's pruned-weight
format code with its container parser (et_amd/csrc/formats.cpp), each through a small driver of
tests/sanitize/.  CPU only - sanitizers never run on the GPU box's device code."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def san_dir():
    if shutil.which("gcc") is None or shutil.which("g++") is None or shutil.which("make") is None:
        pytest.skip("no host compiler here")
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "asan"], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return os.path.join(ROOT, "oracle", "_san")


def test_formats_and_container_parser_under_asan_ubsan(san_dir, tmp_path):
    """generators, validator, packer, pruner, container round trips, and the damaged files (every
    truncation of the header, flipped bits, trailing bytes, absurd counts, sizes other than the caller's)"""
    res = subprocess.run([os.path.join(san_dir, "formats_san"), str(tmp_path)], capture_output=True, text=True)
    assert res.returncode == 0, (res.stdout + res.stderr)[-3000:]
    assert "formats_san: ok" in res.stdout


def test_oracle_under_asan_ubsan(san_dir):
    """one small pass through every exported oracle function with arrays of exactly the documented sizes
    (the driver frees nothing, so leak checking is off for it)"""
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    res = subprocess.run([os.path.join(san_dir, "oracle_san")], capture_output=True, text=True, env=env)
    assert res.returncode == 0, (res.stdout + res.stderr)[-3000:]
    assert "oracle_san: ok" in res.stdout
