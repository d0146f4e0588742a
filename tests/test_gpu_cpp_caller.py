"""A C++ program written against the host layer's headers the way the reference's micro-benchmark drives HEMMer
(examples/bert-matmul.cpp:159-208, 292-338), built by build.py as plain C++ and linked with libhemm.so only: it has
to run on the GPU and land within 2^-12 of the float64 products."""
import os
import subprocess

import pytest

from __graft_entry__ import PKG_DIR

pytestmark = pytest.mark.gpu


def test_cpp_caller_runs_the_matmul_path():
    exe = os.path.join(PKG_DIR, "examples", "matmul_projection")
    assert os.path.exists(exe), "examples/matmul_projection is missing: run __graft_entry__.build() first"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = dict(l.split() for l in r.stdout.splitlines() if "_max_abs_err" in l)
    assert set(lines) == {"pcmm_pre_reuse_max_abs_err", "ccmm_max_abs_err", "pcmm_single_max_abs_err"}
    assert all(float(v) < 2.0 ** -12 for v in lines.values()), lines
