"""ctypes binding of the CPU oracle (oracle/kai_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by
the ``cpu_baseline`` leg of ``bench.py``.  The product package never imports it.

Each wrapper takes and returns C-contiguous float32 numpy arrays and keeps the
argument order of the reference's ``VMath`` methods
(source/engine/support/vmath.h:65-66, 137-143, 234-241) without ``device``.
"""
import ctypes
import os
import subprocess
import threading

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkai_oracle.so")
_lib = None

_F = ctypes.POINTER(ctypes.c_float)
_I64 = ctypes.c_int64
_INT = ctypes.c_int

ACT = {"none": 0, "relu": 1, "leaky": 2, "sigmoid": 3, "tanh": 4, "gelu": 5, "selu": 6, "mish": 7, "swish": 8,
       "softmax": 9}


def build(force=False):
    """Compile the C restatement with the reference's strict-FP flags."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libkai_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        sig = {
            "ko_matmul": [_F, _F, _F, _I64, _I64, _I64, _INT],
            "ko_matmul_rows": [_F, _F, _F, _I64, _I64, _I64, _I64, _INT],
            "ko_matmul_backward_x": [_F, _F, _F, _I64, _I64, _I64, _INT],
            "ko_matmul_backward_w": [_F, _F, _F, _I64, _I64, _I64, _INT],
            "ko_add_bias": [_F, _F, _F, _I64, _I64],
            "ko_add_bias_backward_b": [_F, _F, _I64, _I64, _INT],
            "ko_activate": [_F, _F, _I64, _I64, _INT, _F],
            "ko_activate_backward": [_F, _F, _F, _I64, _I64, _INT, _F],
            "ko_activate_backward_with_y": [_F, _F, _F, _I64, _I64, _INT, _F],
            "ko_mult_on_heads": [_F, _F, _F, _I64, _I64, _I64, _I64, _I64, _F],
            "ko_mult_on_heads_backward": [_F, _F, _F, _I64, _I64, _I64, _I64, _I64],
            "ko_set_mh_attention_mask": [_F, _I64, _I64, _I64, _INT],
            "ko_softmax_direct_on_axis": [_F, _I64, _I64, _I64],
            "ko_softmax_direct_on_axis_backward": [_F, _F, _I64, _I64, _I64, _F],
            "ko_mix_values": [_F, _F, _F, _I64, _I64, _I64, _I64, _I64],
            "ko_mix_values_backward_prop": [_F, _F, _F, _I64, _I64, _I64, _I64, _I64],
            "ko_mix_values_backward_value": [_F, _F, _F, _I64, _I64, _I64, _I64, _I64],
            "ko_transpose": [_F, _F, ctypes.c_void_p, _I64, _I64],
            "ko_transpose_backward": [_F, _F, ctypes.c_void_p, _I64, _I64],
            "ko_transpose_bin": [_F, _F, _I64, _I64],
            "ko_cosinesim": [_F, _F, _F, _I64, _I64, _I64],
            "ko_copy": [_F, _F, _I64],
            "ko_add": [_F, _F, _F, _I64],
            "ko_lstm_process": [_F, _F, _F, _F, _I64, _I64],
            "ko_lstm_process_backward": [_F, _F, _F, _F, _F, _I64, _I64],
            "ko_gru_process": [_F, _F, _F, _I64, _I64, _I64],
            "ko_gru_process_backward": [_F, _F, _F, _F, _F, _F, _I64, _I64, _I64],
            "ko_accumulate_grad": [_F, _F, _I64],
            "ko_subtract_param_grad": [_F, _F, _I64, _F],
            "ko_apply_decay": [_F, _F, _F, _I64, _F, _F],
            "ko_eval_adam_delta": [_F, _F, _F, _F, _F, _I64, _F, _F, _F],
        }
        for name, args in sig.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _INT
        _lib = L
    return _lib


class OracleError(RuntimeError):
    def __init__(self, code):
        super().__init__("oracle returned error code %d" % code)
        self.code = code


def _p(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_F)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _hyper(v):
    """float or None -> (keepalive, pointer); None is the reference's null HYPER (reads as 0)."""
    if v is None:
        return None, None
    c = ctypes.c_float(v)
    return c, ctypes.pointer(c)


def _check(rc):
    if rc != 0:
        raise OracleError(rc)


def matmul(w, x, acc_into=None):
    """y[ndat,yvec] (+)= x[ndat,xvec] . w[yvec,xvec]^T"""
    w, x = _f32(w), _f32(x)
    yvec, xvec = w.shape
    ndat = x.size // xvec
    y = np.zeros((ndat, yvec), np.float32) if acc_into is None else _f32(acc_into).copy().reshape(ndat, yvec)
    _check(lib().ko_matmul(_p(y), _p(w), _p(x), yvec, ndat, xvec, int(acc_into is not None)))
    return y


def matmul_rows(w, x, rows):
    """Oracle rows ``rows`` (a list of row indices) of matmul(w, x); used to sample a big product."""
    w, x = _f32(w), _f32(x)
    yvec, xvec = w.shape
    xs = np.ascontiguousarray(x.reshape(-1, xvec)[rows])
    y = np.zeros((xs.shape[0], yvec), np.float32)
    _check(lib().ko_matmul(_p(y), _p(w), _p(xs), yvec, xs.shape[0], xvec, 0))
    return y


def matmul_parallel(w, x, threads):
    """matmul(w, x) with the rows spread over ``threads`` host threads (ctypes drops the GIL);
    each element's summation order is unchanged, so the result is bit-identical."""
    w, x = _f32(w), _f32(x)
    yvec, xvec = w.shape
    ndat = x.size // xvec
    y = np.zeros((ndat, yvec), np.float32)
    bounds = np.linspace(0, ndat, threads + 1).astype(np.int64)
    L = lib()

    def work(i):
        L.ko_matmul_rows(_p(y), _p(w), _p(x), yvec, int(bounds[i]), int(bounds[i + 1]), xvec, 0)

    ts = [threading.Thread(target=work, args=(i,)) for i in range(threads)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    return y


def matmul_backward_x(gy, w, acc_into=None):
    gy, w = _f32(gy), _f32(w)
    yvec, xvec = w.shape
    ndat = gy.size // yvec
    gx = np.zeros((ndat, xvec), np.float32) if acc_into is None else _f32(acc_into).copy().reshape(ndat, xvec)
    _check(lib().ko_matmul_backward_x(_p(gx), _p(gy), _p(w), yvec, ndat, xvec, int(acc_into is not None)))
    return gx


def matmul_backward_w(gy, x, yvec, xvec, acc_into=None):
    gy, x = _f32(gy), _f32(x)
    ndat = x.size // xvec
    gw = np.zeros((yvec, xvec), np.float32) if acc_into is None else _f32(acc_into).copy().reshape(yvec, xvec)
    _check(lib().ko_matmul_backward_w(_p(gw), _p(gy), _p(x), yvec, ndat, xvec, int(acc_into is not None)))
    return gw


def add_bias(a, b):
    a, b = _f32(a), _f32(b)
    ncol = b.size
    y = np.empty_like(a)
    _check(lib().ko_add_bias(_p(y), _p(a), _p(b), a.size // ncol, ncol))
    return y


def add_bias_backward_b(gy, ncol, acc_into=None):
    gy = _f32(gy)
    gb = np.zeros(ncol, np.float32) if acc_into is None else _f32(acc_into).copy()
    _check(lib().ko_add_bias_backward_b(_p(gb), _p(gy), gy.size // ncol, ncol, int(acc_into is not None)))
    return gb


def activate(x, act, leaky_alpha=None):
    x = _f32(x)
    ncol = x.shape[-1]
    y = np.empty_like(x)
    keep, h = _hyper(leaky_alpha)
    _check(lib().ko_activate(_p(y), _p(x), x.size // ncol, ncol, ACT[act] if isinstance(act, str) else act, h))
    return y


def activate_backward(gy, x, act, leaky_alpha=None):
    gy, x = _f32(gy), _f32(x)
    ncol = x.shape[-1]
    gx = np.empty_like(x)
    keep, h = _hyper(leaky_alpha)
    _check(lib().ko_activate_backward(_p(gx), _p(gy), _p(x), x.size // ncol, ncol,
                                      ACT[act] if isinstance(act, str) else act, h))
    return gx


def activate_backward_with_y(gy, y, act, leaky_alpha=None):
    gy, y = _f32(gy), _f32(y)
    ncol = y.shape[-1]
    gx = np.empty_like(y)
    keep, h = _hyper(leaky_alpha)
    _check(lib().ko_activate_backward_with_y(_p(gx), _p(gy), _p(y), y.size // ncol, ncol,
                                             ACT[act] if isinstance(act, str) else act, h))
    return gx


def mult_on_heads(K, Q, nhead, coef):
    """K, Q: [nbat, ntimes, nvec] -> scores [nbat, ntimes, ntimes, nhead]"""
    K, Q = _f32(K), _f32(Q)
    nbat, ntimes, nvec = K.shape
    p = np.empty((nbat, ntimes, ntimes, nhead), np.float32)
    keep, h = _hyper(coef)
    _check(lib().ko_mult_on_heads(_p(p), _p(K), _p(Q), nbat, ntimes, nvec, nhead, nvec // nhead, h))
    return p


def mult_on_heads_backward(gp, KQ, nhead):
    gp, KQ = _f32(gp), _f32(KQ)
    nbat, ntimes, nvec = KQ.shape
    g = np.empty_like(KQ)
    _check(lib().ko_mult_on_heads_backward(_p(g), _p(gp), _p(KQ), nbat, ntimes, nvec, nhead, nvec // nhead))
    return g


def set_mh_attention_mask(p, forward=True):
    p = _f32(p).copy()
    nbat, ntimes, _, nhead = p.shape
    _check(lib().ko_set_mh_attention_mask(_p(p), nbat, ntimes, nhead, int(forward)))
    return p


def softmax_direct_on_axis(p, nrow, nvec, ncol):
    p = _f32(p).copy()
    _check(lib().ko_softmax_direct_on_axis(_p(p), nrow, nvec, ncol))
    return p


def softmax_direct_on_axis_backward(gp, p, coef):
    gp, p = _f32(gp).copy(), _f32(p)
    nbat, ntimes, _, nhead = p.shape
    keep, h = _hyper(coef)
    _check(lib().ko_softmax_direct_on_axis_backward(_p(gp), _p(p), nbat, ntimes, nhead, h))
    return gp


def mix_values(p, V, nhead):
    p, V = _f32(p), _f32(V)
    nbat, ntimes, nvec = V.shape
    y = np.empty((nbat, ntimes, nvec), np.float32)
    _check(lib().ko_mix_values(_p(y), _p(p), _p(V), nbat, ntimes, nvec, nhead, nvec // nhead))
    return y


def mix_values_backward_prop(gy, V, nhead):
    gy, V = _f32(gy), _f32(V)
    nbat, ntimes, nvec = V.shape
    gp = np.empty((nbat, ntimes, ntimes, nhead), np.float32)
    _check(lib().ko_mix_values_backward_prop(_p(gp), _p(gy), _p(V), nbat, ntimes, nvec, nhead, nvec // nhead))
    return gp


def mix_values_backward_value(gy, p, nhead):
    gy, p = _f32(gy), _f32(p)
    nbat, ntimes, nvec = gy.shape
    gV = np.empty((nbat, ntimes, nvec), np.float32)
    _check(lib().ko_mix_values_backward_value(_p(gV), _p(gy), _p(p), nbat, ntimes, nvec, nhead, nvec // nhead))
    return gV


def accumulate_grad(y, x):
    """y + x elementwise (returns the new y)."""
    y = _f32(y).copy()
    x = _f32(x)
    _check(lib().ko_accumulate_grad(_p(y), _p(x), y.size))
    return y


def subtract_param_grad(p, g, learning_rate):
    p = _f32(p).copy()
    g = _f32(g)
    keep, h = _hyper(learning_rate)
    _check(lib().ko_subtract_param_grad(_p(p), _p(g), p.size, h))
    return p


def apply_decay(p, g, l1_decay, l2_decay):
    p, g = _f32(p), _f32(g)
    d = np.zeros_like(g)
    k1, h1 = _hyper(l1_decay)
    k2, h2 = _hyper(l2_decay)
    _check(lib().ko_apply_decay(_p(d), _p(p), _p(g), g.size, h1, h2))
    return d


def eval_adam_delta(g, s, t, n, ro1, ro2, epsilon):
    """One Adam step: returns (delta, s', t', n'); s, t, n are the moment and step-count tensors."""
    g = _f32(g)
    s, t, n = _f32(s).copy(), _f32(t).copy(), _f32(n).copy()
    a = np.zeros_like(g)
    k1, h1 = _hyper(ro1)
    k2, h2 = _hyper(ro2)
    k3, h3 = _hyper(epsilon)
    _check(lib().ko_eval_adam_delta(_p(a), _p(g), _p(s), _p(t), _p(n), g.size, h1, h2, h3))
    return a, s, t, n


def transpose_axinfo(shape, axes):
    """The [axis_size, 3] int32 table VTensor::transpose builds (vtensor.cpp:5391-5417): per output axis n the
    source axis, the output elements per step of axis n, and the SOURCE elements per step of source axis n."""
    shape = [int(v) for v in shape]
    total = int(np.prod(shape))
    rest, prod = total, total
    info = np.zeros((len(shape), 3), np.int32)
    for n, axis in enumerate(axes):
        rest //= shape[axis]
        prod //= shape[n]
        info[n] = (axis, rest, prod)
    return info


def transpose(x, axes):
    x = _f32(x)
    info = transpose_axinfo(x.shape, axes)
    y = np.zeros([x.shape[a] for a in axes], np.float32)
    _check(lib().ko_transpose(_p(y), _p(x), info.ctypes.data, x.ndim, x.size))
    return y


def transpose_backward(gy, xshape, axes):
    gy = _f32(gy)
    info = transpose_axinfo(xshape, axes)
    gx = np.zeros(xshape, np.float32)
    _check(lib().ko_transpose_backward(_p(gx), _p(gy), info.ctypes.data, len(xshape), gy.size))
    return gx


def transpose_bin(x, nrow, ncol):
    """x is [ncol, nrow]; returns [nrow, ncol]."""
    x = _f32(x)
    y = np.zeros((nrow, ncol), np.float32)
    _check(lib().ko_transpose_bin(_p(y), _p(x), nrow, ncol))
    return y


def cosinesim(x1, x2):
    """y[nrow1, nrow2]: cosine of every row of x1 with every row of x2 (last axis = the vector)."""
    x1, x2 = _f32(x1), _f32(x2)
    ncol = x1.shape[-1]
    nrow1, nrow2 = x1.size // ncol, x2.size // ncol
    y = np.zeros((nrow1, nrow2), np.float32)
    _check(lib().ko_cosinesim(_p(y), _p(x1), _p(x2), nrow1, nrow2, ncol))
    return y


# ---- recurrent cells -------------------------------------------------------------------------------

def copy(a):
    a = _f32(a)
    y = np.zeros_like(a)
    _check(lib().ko_copy(_p(y), _p(a), a.size))
    return y


def add(a, b):
    a, b = _f32(a), _f32(b)
    y = np.zeros_like(a)
    _check(lib().ko_add(_p(y), _p(a), _p(b), a.size))
    return y


def lstm_process(affine, prev_state=None):
    """affine [ndat, 4*nrec] (input, forget, block, output); returns (recurrent, state), each [ndat, nrec]."""
    affine = _f32(affine)
    ndat, nrec = affine.shape[0], affine.shape[1] // 4
    r = np.zeros((ndat, nrec), np.float32)
    st = np.zeros((ndat, nrec), np.float32)
    ps1 = None if prev_state is None else _p(_f32(prev_state))
    _check(lib().ko_lstm_process(_p(r), _p(st), ps1, _p(affine), ndat, nrec))
    return r, st


def lstm_process_backward(gr, gs, affine, prev_state=None):
    """Gradient of one LSTM cell step, the reference's device kernel.  gr, gs [ndat, nrec]: gradients of this
    step's output and state; affine [ndat, 4*nrec]: this step's gate sums; prev_state: the state the step
    started from (None: 0).  Returns (gradient of the previous state, gate-sum gradients [ndat, 4*nrec])."""
    gr, gs, affine = _f32(gr), _f32(gs).copy(), _f32(affine)
    ndat, nrec = affine.shape[0], affine.shape[1] // 4
    ga = np.zeros_like(affine)
    ps = None if prev_state is None else _p(_f32(prev_state))
    _check(lib().ko_lstm_process_backward(_p(gr), _p(gs), _p(ga), ps, _p(affine), ndat, nrec))
    return gs, ga


def gru_process(recurs, pai, par, nt):
    """recurs [ntimes, ndat, nrec] is updated in place at step nt (reads step nt-1 when nt > 0)."""
    assert recurs.dtype == np.float32 and recurs.flags["C_CONTIGUOUS"]
    pai, par = _f32(pai), _f32(par)
    _, ndat, nrec = recurs.shape
    _check(lib().ko_gru_process(_p(recurs[nt]), _p(pai), _p(par), nt, ndat, nrec))
    return recurs


def gru_process_backward(gr, recurs, pai, par, nt):
    """gr [ndat, nrec] is replaced by the gradient of the previous step's output; returns (gr, gai, gar)."""
    gr = _f32(gr).copy()
    pai, par = _f32(pai), _f32(par)
    _, ndat, nrec = recurs.shape
    gai, gar = np.zeros_like(pai), np.zeros_like(par)
    _check(lib().ko_gru_process_backward(_p(gr), _p(gai), _p(gar), _p(recurs[nt]), _p(pai), _p(par), nt, ndat, nrec))
    return gr, gai, gar
