"""Shared helpers of the test-suite: seeded inputs of the five benchmark configurations,
the error metric, and access to the oracle (oracle/oracle.py, test infrastructure)."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

import oracle as ko  # noqa: E402  (oracle/oracle.py)

# relative Frobenius tolerance of the path: fp32, differences of summation order only
REL_FRO_TOL = 1e-5


def rel_fro(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    den = np.linalg.norm(ref.ravel())
    num = np.linalg.norm((got - ref).ravel())
    return num / den if den > 0 else num


def xavier_uniform(rng, out_w, in_w):
    """The engine's "xavier" init: uniform in +-sqrt(1/in_width) (api_objects/vmodule.cpp:1390)."""
    a = np.sqrt(1.0 / in_w)
    return rng.uniform(-a, a, size=(out_w, in_w)).astype(np.float32)


def cfg1(seed=0):
    """Single dense layer forward: X[64,784]~N(0,1), W'[784,512] Xavier-uniform, b = 0, ReLU."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((64, 784)).astype(np.float32)
    w = xavier_uniform(rng, 512, 784)        # engine layout [out, in]; W' = w.T
    b = np.zeros(512, np.float32)
    return x, w, b


def cfg2(seed=2):
    """Dense forward+backward, batch 256, 1024 -> 1024."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((256, 1024)).astype(np.float32)
    w = xavier_uniform(rng, 1024, 1024)
    b = xavier_uniform(rng, 1, 1024).reshape(1024)
    gy = (0.01 * rng.standard_normal((256, 1024))).astype(np.float32)
    return x, w, b, gy


def cfg3(n=8192, seed=3):
    """Large square GEMM: A, B ~ U(-1,1), bias ~ N(0,1); B is [K,N] row-major."""
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1, 1, size=(n, n)).astype(np.float32)
    b = rng.uniform(-1, 1, size=(n, n)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    return a, b, bias


def cfg4(nbat=32, ntimes=512, nvec=64, seed=4):
    """Attention: Q, K, V [nbat, ntimes, nvec] ~ N(0,1)."""
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    k = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    v = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    return q, k, v


def cfg5(m, k=4096, n=4096, seed=5):
    """Skinny / ragged: W[n,k] ~ U(-0.05,0.05), X[m,k] ~ N(0,1)."""
    rng = np.random.default_rng(seed)
    w = rng.uniform(-0.05, 0.05, size=(n, k)).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    return w, x
