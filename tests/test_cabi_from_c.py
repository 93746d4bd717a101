"""The C-ABI called from a C++ program with no Python or torch in the process.

``tests/cabi/host_check.cpp`` is linked against the built library by the package's build
step; these tests only run it.  Its own checks are self-contained (host arithmetic on the
bytes the library produced), so it is a third opinion beside the oracle.
"""

import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi", "host_check")


def _run(*args):
    if not os.path.exists(BIN):
        # a tree whose library was built by an older build step: link the program now
        from deepfold_amd import build_ext
        build_ext.build_host_check()
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built; run `python -m deepfold_amd.build_ext` "
                    "(or __graft_entry__.build()) first")
    if not os.access(BIN, os.X_OK):
        os.chmod(BIN, 0o755)
    proc = subprocess.run([BIN, *args], capture_output=True, text=True, timeout=100)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.strip().endswith("host_check: OK"), proc.stdout
    return proc.stdout


def test_plan_and_argument_checks_from_c():
    _run("--host-only")


@pytest.mark.gpu
def test_codec_gemv_gemm_from_c():
    out = _run()
    assert "gemv max-rel" in out
