"""The C++ mirror of the engine's operator interface (include/vmath_hip.h, csrc/vmath_hip.hip), called from
compiled engine-style code: tests/vmath_mirror_driver.cpp is linked against libkai_hip.so and calls
VMath::matmul, add_bias, activate, dense_forward, mult_on_heads, mem_alloc / mem_free and calls that must
raise KaiMathError with the reference's numeric codes (VERR_CONDITIONAL_STATEMENT = 8,
VERR_INVALID_ARGUMENT = 510, VERR_INVALID_POINTER = 523; vmath.cu:64-87, 3159-3161).  Expected values come
from the CPU oracle through files."""
import os
import subprocess

import numpy as np
import pytest

from util import ROOT, ko

HERE = os.path.join(ROOT, "tests")
DRIVER = os.path.join(HERE, "vmath_mirror_driver")


def driver():
    """The built driver; built here when missing (host compiler, a second or two)."""
    if not os.path.exists(DRIVER):
        subprocess.check_call(["make", "-C", HERE, "-s", "vmath_mirror_driver"])
    return DRIVER


def run(args):
    r = subprocess.run([driver()] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=110)
    print(r.stdout)
    return r


def test_mirror_links_and_raises_the_reference_error_codes():
    r = run(["cpu"])
    assert r.returncode == 0, r.stdout
    for line in ("matmul on device -1: KaiMathError 510", "activate with code 10: KaiMathError 8",
                 "matmul with a null output: KaiMathError 523", "host memory helpers", "all checks passed"):
        assert line in r.stdout, line
    assert "FAIL" not in r.stdout


@pytest.mark.gpu
def test_mirror_results_match_the_oracle(tmp_path):
    ndat, xvec, yvec = 70, 200, 130
    nbat, ntimes, nhead, npiece = 2, 50, 4, 8
    rng = np.random.default_rng(7)
    x = rng.standard_normal((ndat, xvec)).astype(np.float32)
    w = rng.uniform(-0.07, 0.07, (yvec, xvec)).astype(np.float32)
    b = rng.standard_normal(yvec).astype(np.float32)
    q = rng.standard_normal((nbat, ntimes, nhead * npiece)).astype(np.float32)
    k = rng.standard_normal((nbat, ntimes, nhead * npiece)).astype(np.float32)
    y_ref = ko.matmul(w, x)
    act_ref = ko.activate(ko.add_bias(y_ref, b), "relu")
    p_ref = ko.mult_on_heads(k, q, nhead, float(np.float32(1.0) / np.sqrt(np.float32(npiece))))
    for name, a in dict(x=x, w=w, b=b, q=q, k=k, y_ref=y_ref, act_ref=act_ref, p_ref=p_ref).items():
        np.ascontiguousarray(a, np.float32).tofile(str(tmp_path / (name + ".bin")))
    r = run(["gpu", tmp_path, ndat, xvec, yvec, nbat, ntimes, nhead, npiece])
    assert r.returncode == 0, r.stdout
    assert "FAIL" not in r.stdout and "all checks passed" in r.stdout
    assert r.stdout.count("ok  ") >= 9
