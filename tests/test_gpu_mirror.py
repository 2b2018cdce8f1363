"""The C++ mirror of the reference surface (include/p100e_fast_attn.hpp), driven by a standalone executable the way
the reference's own tests are: paged == contiguous, rows == single, refusals, all bitwise."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "mirror_check")


@pytest.mark.gpu
def test_cpp_mirror_harness():
    assert os.path.exists(EXE), "tests/cpp/mirror_check is built by __graft_entry__.build()"
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=170)
    print(r.stdout[-3000:])
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "0 failed" in r.stdout
