"""ctypes binding of libkai_hip.so (the C-ABI declared in include/kai_hip.h).

The library is the product; this module is the thin Python harness over it used by the
tests, the smoke check and the benchmark.  It fails loudly when the shared library is
missing: there is no CPU fallback.

``VMath`` mirrors the reference's ``class VMath`` (source/engine/support/vmath.h:10-332):
same method names, argument order and meaning, raw device pointers (``DeviceBuffer`` or
int addresses).  A non-zero status raises ``KaiError`` with the reference's numeric
error code, where the reference throws ``VException``.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkai_hip.so")

_F = ctypes.c_void_p       # device pointers travel as plain addresses
_I64 = ctypes.c_int64
_INT = ctypes.c_int

# name -> argument types; every function returns int except kai_last_error
SIGNATURES = {
    "kai_device_count": [ctypes.POINTER(_INT)],
    "kai_set_device": [_INT],
    "kai_device_synchronize": [],
    "kai_set_stream": [ctypes.c_void_p],
    "kai_arch_info": [ctypes.c_char_p, ctypes.c_char_p, _INT],
    "kai_shutdown": [],
    "kai_reserve_scratch": [_I64],
    "kai_scratch_info": [ctypes.POINTER(_I64), ctypes.POINTER(_I64), ctypes.POINTER(_I64)],
    "kai_mem_alloc": [_INT, _I64, ctypes.POINTER(ctypes.c_void_p)],
    "kai_mem_free": [_INT, ctypes.c_void_p],
    "kai_memcpy_host_to_host": [ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_memcpy_host_to_device": [ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_memcpy_device_to_host": [ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_memcpy_device_to_device": [ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_copy_data": [_INT, _INT, ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_fill_int": [_INT, _F, _I64, _INT],
    "kai_fill_float": [_INT, _F, _I64, ctypes.c_float],
    "kai_set_zero": [_INT, ctypes.c_void_p, _I64],
    "kai_memcpy_from_host": [_INT, ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_memcpy_to_host": [_INT, ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_memcpy_to_device": [_INT, ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_get_slice": [_INT, ctypes.c_void_p, ctypes.c_void_p, _I64],
    "kai_matmul": [_INT, _F, _F, _F, _I64, _I64, _I64, _INT],
    "kai_matmul_noalloc": [_INT, _F, _F, _F, _I64, _I64, _I64, _INT],
    "kai_matmul_backward_x": [_INT, _F, _F, _F, _I64, _I64, _I64, _INT],
    "kai_matmul_backward_w": [_INT, _F, _F, _F, _I64, _I64, _I64, _INT],
    "kai_add_bias": [_INT, _F, _F, _F, _I64, _I64],
    "kai_add_bias_backward_b": [_INT, _F, _F, _I64, _I64, _INT],
    "kai_activate": [_INT, _F, _F, _I64, _I64, _INT, _F],
    "kai_activate_backward": [_INT, _F, _F, _F, _I64, _I64, _INT, _F],
    "kai_activate_backward_with_y": [_INT, _F, _F, _F, _I64, _I64, _INT, _F],
    "kai_mult_on_heads": [_INT, _F, _F, _F, _I64, _I64, _I64, _I64, _I64, _F],
    "kai_mult_on_heads_backward": [_INT, _F, _F, _F, _I64, _I64, _I64, _I64, _I64],
    "kai_set_mh_attention_mask": [_INT, _F, _I64, _I64, _I64, _INT],
    "kai_softmax_direct_on_axis": [_INT, _F, _I64, _I64, _I64],
    "kai_softmax_direct_on_axis_backward": [_INT, _F, _F, _I64, _I64, _I64, _F],
    "kai_mix_values": [_INT, _F, _F, _F, _I64, _I64, _I64, _I64, _I64],
    "kai_mix_values_backward_prop": [_INT, _F, _F, _F, _I64, _I64, _I64, _I64, _I64],
    "kai_mix_values_backward_value": [_INT, _F, _F, _F, _I64, _I64, _I64, _I64, _I64],
    "kai_gemm_f32": [_INT, _INT, _INT, _I64, _I64, _I64, _F, _I64, _F, _I64, _F, _I64, _F, _INT, _F, _INT],
    "kai_gemm_plan": [_INT, _INT, _I64, _I64, _I64, _I64, _I64, _I64, _INT, _INT, _INT, ctypes.c_char_p, _INT],
    "kai_dense_forward": [_INT, _F, _F, _F, _F, _F, _I64, _I64, _I64, _INT, _F],
    "kai_attention_forward": [_INT, _F, _F, _F, _F, _I64, _I64, _I64, _I64, _I64, _F, _INT],
    "kai_gemm_force_plan": [ctypes.c_char_p],
    "kai_attention_plan": [_INT, _I64, _I64, _I64, _I64, _I64, ctypes.c_char_p, _INT],
    "kai_attention_forward_train": [_INT, _F, _F, _F, _F, _F, _I64, _I64, _I64, _I64, _I64, _F, _INT],
    "kai_attention_backward": [_INT, _F, _F, _F, _F, _F, _F, _F, _F, _F, _I64, _I64, _I64, _I64, _I64, _F, _INT],
    "kai_cosinesim": [_INT, _F, _F, _F, _I64, _I64, _I64],
    "kai_copy": [_INT, _F, _F, _I64],
    "kai_add": [_INT, _F, _F, _F, _I64],
    "kai_lstm_process": [_INT, _F, _F, _F, _F, _I64, _I64, _I64],
    "kai_lstm_process_backward": [_INT, _F, _F, _F, _F, _F, _I64, _I64, _I64],
    "kai_gru_process": [_INT, _F, _F, _F, _I64, _I64, _I64, _I64],
    "kai_gru_process_backward": [_INT, _F, _F, _F, _F, _F, _F, _I64, _I64, _I64, _I64],
    "kai_lstm_step": [_INT, _F, _F, _F, _F, _F, _F, _F, _F, _I64, _I64],
    "kai_gru_step": [_INT, _F, _F, _F, _F, _F, _F, _F, _F, _I64, _I64],
    "kai_transpose": [_INT, _F, _F, _F, _I64, _I64],
    "kai_transpose_backward": [_INT, _F, _F, _F, _I64, _I64],
    "kai_transpose_bin": [_INT, _F, _F, _I64, _I64],
    "kai_accumulate_grad": [_INT, _F, _F, _I64],
    "kai_subtract_param_grad": [_INT, _F, _F, _I64, _F],
    "kai_apply_decay": [_INT, _F, _F, _F, _I64, _F, _F],
    "kai_eval_adam_delta": [_INT, _F, _F, _F, _F, _F, _I64, _F, _F, _F],
    "kai_dense_backward": [_INT, _F, _F, _F, _F, _F, _F, _F, _F, _I64, _I64, _I64, _INT, _F, _INT],
}

ACT = {"none": 0, "relu": 1, "leaky": 2, "sigmoid": 3, "tanh": 4, "gelu": 5, "selu": 6, "mish": 7, "swish": 8,
       "softmax": 9}

_lib = None


class KaiError(RuntimeError):
    """A non-zero status of the C-ABI; ``code`` is the reference's numeric error code."""

    def __init__(self, code, message):
        super().__init__("kai error %d: %s" % (code, message))
        self.code = code
        self.message = message


def load():
    """Load libkai_hip.so from the package directory; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `make -C %s/csrc` (or __graft_entry__.build()); "
                "there is no CPU fallback" % (LIB_PATH, _HERE))
        L = ctypes.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _INT
        L.kai_last_error.argtypes = []
        L.kai_last_error.restype = ctypes.c_char_p
        L.kai_matmul_noalloc_scratch_bytes.argtypes = []
        L.kai_matmul_noalloc_scratch_bytes.restype = _I64
        _lib = L
    return _lib


def _ck(rc):
    if rc != 0:
        raise KaiError(rc, load().kai_last_error().decode("utf-8", "replace"))


def _addr(p):
    if p is None:
        return None
    if isinstance(p, DeviceBuffer):
        return p.ptr
    return int(p)


class DeviceBuffer:
    """Device memory owned through VMath::mem_alloc / mem_free semantics (kai_mem_alloc)."""

    def __init__(self, nbytes, device=0):
        self.device = device
        self.nbytes = int(nbytes)
        out = ctypes.c_void_p()
        _ck(load().kai_mem_alloc(device, self.nbytes, ctypes.byref(out)))
        self.ptr = out.value

    @classmethod
    def from_numpy(cls, a, device=0):
        a = np.ascontiguousarray(a)
        buf = cls(max(a.nbytes, 1), device)
        if a.nbytes:
            _ck(load().kai_memcpy_from_host(device, buf.ptr, a.ctypes.data, a.nbytes))
        return buf

    def to_numpy(self, shape, dtype=np.float32):
        out = np.empty(shape, dtype)
        if out.nbytes:
            _ck(load().kai_memcpy_to_host(self.device, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def offset(self, nbytes):
        """Raw address inside the buffer (sub-buffer pointers, as the engine's RNN driver passes)."""
        return self.ptr + int(nbytes)

    def free(self):
        if self.ptr:
            _ck(load().kai_mem_free(self.device, self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            if getattr(self, "ptr", None) and _lib is not None:
                _lib.kai_mem_free(self.device, self.ptr)
                self.ptr = None
        except Exception:
            pass


def hyper(value, device=0):
    """A device-resident float cell, as VHyperManager::fetch hands to kernels
    (source/engine/local_objects/vhypermanager.cpp:79-88); None stays a null HYPER."""
    if value is None:
        return None
    return DeviceBuffer.from_numpy(np.array([value], np.float32), device)


def device_count():
    n = _INT(0)
    _ck(load().kai_device_count(ctypes.byref(n)))
    return n.value


def set_device(device):
    _ck(load().kai_set_device(device))


def synchronize():
    _ck(load().kai_device_synchronize())


def set_stream(stream_handle):
    _ck(load().kai_set_stream(stream_handle))


def shutdown():
    """Release the library's own scratch memory (it is re-created on demand)."""
    _ck(load().kai_shutdown())


def reserve_scratch(nbytes):
    """Size the current device's scratch now, so that later calls allocate nothing."""
    _ck(load().kai_reserve_scratch(nbytes))


def scratch_info():
    """(bytes, growths since the last shutdown, bytes of replaced buffers still held) of the current device."""
    b, g, r = _I64(), _I64(), _I64()
    _ck(load().kai_scratch_info(ctypes.byref(b), ctypes.byref(g), ctypes.byref(r)))
    return b.value, g.value, r.value


def arch_info():
    a = ctypes.create_string_buffer(64)
    b = ctypes.create_string_buffer(256)
    _ck(load().kai_arch_info(a, b, 64))
    return a.value.decode(), b.value.decode()


class VMath:
    """The hot subset of the reference's ``VMath`` static methods over raw device pointers."""

    @staticmethod
    def matmul(device, py, pw, px, yvec, ndat, xvec, acc):
        _ck(load().kai_matmul(device, _addr(py), _addr(pw), _addr(px), yvec, ndat, xvec, int(acc)))

    @staticmethod
    def matmul_noalloc(device, py, pw, px, yvec, ndat, xvec, acc):
        """kai_matmul without any allocation: partial sums go to a fixed array inside the library."""
        _ck(load().kai_matmul_noalloc(device, _addr(py), _addr(pw), _addr(px), yvec, ndat, xvec, int(acc)))

    @staticmethod
    def matmul_backward_x(device, pgx, pgy, pw, yvec, ndat, xvec, acc):
        _ck(load().kai_matmul_backward_x(device, _addr(pgx), _addr(pgy), _addr(pw), yvec, ndat, xvec, int(acc)))

    @staticmethod
    def matmul_backward_w(device, pgw, pgy, px, yvec, ndat, xvec, acc):
        _ck(load().kai_matmul_backward_w(device, _addr(pgw), _addr(pgy), _addr(px), yvec, ndat, xvec, int(acc)))

    @staticmethod
    def add_bias(device, py, pa, pb, nrow, ncol):
        _ck(load().kai_add_bias(device, _addr(py), _addr(pa), _addr(pb), nrow, ncol))

    @staticmethod
    def add_bias_backward_b(device, pgb, pgy, nrow, ncol, acc):
        _ck(load().kai_add_bias_backward_b(device, _addr(pgb), _addr(pgy), nrow, ncol, int(acc)))

    @staticmethod
    def activate(device, py, px, nrow, ncol, actFunc, hLeakyAlpha):
        _ck(load().kai_activate(device, _addr(py), _addr(px), nrow, ncol, actFunc, _addr(hLeakyAlpha)))

    @staticmethod
    def activate_backward(device, pgx, pgy, px, nrow, ncol, actFunc, hLeakyAlpha):
        _ck(load().kai_activate_backward(device, _addr(pgx), _addr(pgy), _addr(px), nrow, ncol, actFunc,
                                         _addr(hLeakyAlpha)))

    @staticmethod
    def activate_backward_with_y(device, pgx, pgy, py, nrow, ncol, actFunc, hLeakyAlpha):
        _ck(load().kai_activate_backward_with_y(device, _addr(pgx), _addr(pgy), _addr(py), nrow, ncol, actFunc,
                                                _addr(hLeakyAlpha)))

    @staticmethod
    def mult_on_heads(device, pp, pK, pQ, nbat, ntimes, nvec, nhead, npiece, hCoef):
        _ck(load().kai_mult_on_heads(device, _addr(pp), _addr(pK), _addr(pQ), nbat, ntimes, nvec, nhead, npiece,
                                     _addr(hCoef)))

    @staticmethod
    def mult_on_heads_backward(device, pgQKV, pgp, pQKV, nbat, ntimes, nvec, nhead, npiece):
        _ck(load().kai_mult_on_heads_backward(device, _addr(pgQKV), _addr(pgp), _addr(pQKV), nbat, ntimes, nvec,
                                              nhead, npiece))

    @staticmethod
    def set_mh_attention_mask(device, pp, ndat, ntimes, nhead, forward):
        _ck(load().kai_set_mh_attention_mask(device, _addr(pp), ndat, ntimes, nhead, int(forward)))

    @staticmethod
    def softmax_direct_on_axis(device, pp, nrow, nvec, ncol):
        _ck(load().kai_softmax_direct_on_axis(device, _addr(pp), nrow, nvec, ncol))

    @staticmethod
    def softmax_direct_on_axis_backward(device, pgp, pp, nbat, ntimes, nhead, hCoef):
        _ck(load().kai_softmax_direct_on_axis_backward(device, _addr(pgp), _addr(pp), nbat, ntimes, nhead,
                                                       _addr(hCoef)))

    @staticmethod
    def mix_values(device, py, pp, pV, nbat, ntimes, nvec, nhead, npiece):
        _ck(load().kai_mix_values(device, _addr(py), _addr(pp), _addr(pV), nbat, ntimes, nvec, nhead, npiece))

    @staticmethod
    def mix_values_backward_prop(device, pgp, pgy, pV, nbat, ntimes, nvec, nhead, npiece):
        _ck(load().kai_mix_values_backward_prop(device, _addr(pgp), _addr(pgy), _addr(pV), nbat, ntimes, nvec,
                                                nhead, npiece))

    @staticmethod
    def mix_values_backward_value(device, pgV, pgy, pp, nbat, ntimes, nvec, nhead, npiece):
        _ck(load().kai_mix_values_backward_value(device, _addr(pgV), _addr(pgy), _addr(pp), nbat, ntimes, nvec,
                                                 nhead, npiece))

    # memory and fills
    @staticmethod
    def fill_float(device, ptr, size, value):
        _ck(load().kai_fill_float(device, _addr(ptr), size, value))

    @staticmethod
    def fill_int(device, ptr, size, value):
        _ck(load().kai_fill_int(device, _addr(ptr), size, value))

    @staticmethod
    def set_zero(device, ptr, size):
        _ck(load().kai_set_zero(device, _addr(ptr), size))

    @staticmethod
    def copy_data(dest_device, src_device, py, px, nbytes):
        _ck(load().kai_copy_data(dest_device, src_device, _addr(py), _addr(px), nbytes))

    @staticmethod
    def get_slice(device, py, px, nbytes):
        _ck(load().kai_get_slice(device, _addr(py), _addr(px), nbytes))

    @staticmethod
    def memcpy_to_device(device, py, px, size):
        _ck(load().kai_memcpy_to_device(device, _addr(py), _addr(px), size))

    # fused, additive entry points
    @staticmethod
    def gemm_f32(device, transA, transB, M, N, K, A, lda, B, ldb, C, ldc, bias, actFunc, hLeakyAlpha, acc):
        _ck(load().kai_gemm_f32(device, int(transA), int(transB), M, N, K, _addr(A), lda, _addr(B), ldb, _addr(C),
                                ldc, _addr(bias), actFunc, _addr(hLeakyAlpha), int(acc)))

    @staticmethod
    def gemm_plan(transA, transB, M, N, K, lda=None, ldb=None, ldc=None, has_bias=False, actFunc=0, acc=False):
        """Text naming the kernel kai_gemm_f32 would launch for aligned operands of this shape (no GPU needed)."""
        lda = (M if transA else K) if lda is None else lda
        ldb = (K if transB else N) if ldb is None else ldb
        ldc = N if ldc is None else ldc
        buf = ctypes.create_string_buffer(128)
        _ck(load().kai_gemm_plan(int(transA), int(transB), M, N, K, lda, ldb, ldc, int(has_bias), actFunc, int(acc),
                                 buf, 128))
        return buf.value.decode()

    @staticmethod
    def cosinesim(device, py, px1, px2, nrow1, nrow2, ncol):
        _ck(load().kai_cosinesim(device, _addr(py), _addr(px1), _addr(px2), nrow1, nrow2, ncol))

    @staticmethod
    def copy(device, py, pa, ndat):
        _ck(load().kai_copy(device, _addr(py), _addr(pa), ndat))

    @staticmethod
    def add(device, py, pa, pb, ndat):
        _ck(load().kai_add(device, _addr(py), _addr(pa), _addr(pb), ndat))

    @staticmethod
    def lstm_process(device, pr, ps, ps1, pa, ndat, nrec, ninp):
        _ck(load().kai_lstm_process(device, _addr(pr), _addr(ps), _addr(ps1), _addr(pa), ndat, nrec, ninp))

    @staticmethod
    def lstm_process_backward(device, pgr, pgs, pga, ps, pa, ndat, nrec, ninp):
        _ck(load().kai_lstm_process_backward(device, _addr(pgr), _addr(pgs), _addr(pga), _addr(ps), _addr(pa), ndat,
                                             nrec, ninp))

    @staticmethod
    def gru_process(device, pr, pai, par, nt, ntimes, ndat, nrec):
        _ck(load().kai_gru_process(device, _addr(pr), _addr(pai), _addr(par), nt, ntimes, ndat, nrec))

    @staticmethod
    def gru_process_backward(device, pgr, pgai, pgar, pr, pai, par, nt, ntimes, ndat, nrec):
        _ck(load().kai_gru_process_backward(device, _addr(pgr), _addr(pgai), _addr(pgar), _addr(pr), _addr(pai),
                                            _addr(par), nt, ntimes, ndat, nrec))

    @staticmethod
    def lstm_step(device, pr, ps, ps_prev, pa, pwr, pr_prev, pbi, pbr, ndat, nrec):
        _ck(load().kai_lstm_step(device, _addr(pr), _addr(ps), _addr(ps_prev), _addr(pa), _addr(pwr), _addr(pr_prev),
                                 _addr(pbi), _addr(pbr), ndat, nrec))

    @staticmethod
    def gru_step(device, pr, pai, par, pwr, pr_prev, ph_prev, pbi, pbr, ndat, nrec):
        _ck(load().kai_gru_step(device, _addr(pr), _addr(pai), _addr(par), _addr(pwr), _addr(pr_prev), _addr(ph_prev),
                                _addr(pbi), _addr(pbr), ndat, nrec))

    @staticmethod
    def transpose(device, py, px, pn, axis_size, data_size):
        _ck(load().kai_transpose(device, _addr(py), _addr(px), _addr(pn), axis_size, data_size))

    @staticmethod
    def transpose_backward(device, pgx, pgy, pn, axis_size, data_size):
        _ck(load().kai_transpose_backward(device, _addr(pgx), _addr(pgy), _addr(pn), axis_size, data_size))

    @staticmethod
    def transpose_bin(device, py, px, nrow, ncol):
        _ck(load().kai_transpose_bin(device, _addr(py), _addr(px), nrow, ncol))

    @staticmethod
    def accumulate_grad(device, py, px, nrow):
        _ck(load().kai_accumulate_grad(device, _addr(py), _addr(px), nrow))

    @staticmethod
    def subtract_param_grad(device, pp, pg, nrow, hLearningRate):
        _ck(load().kai_subtract_param_grad(device, _addr(pp), _addr(pg), nrow, _addr(hLearningRate)))

    @staticmethod
    def apply_decay(device, pd, pp, pg, nrow, hL1Decay, hL2Decay):
        _ck(load().kai_apply_decay(device, _addr(pd), _addr(pp), _addr(pg), nrow, _addr(hL1Decay), _addr(hL2Decay)))

    @staticmethod
    def eval_adam_delta(device, pa, pg, ps, pt, pn, nrow, hRo1, hRo2, hEpsilon):
        _ck(load().kai_eval_adam_delta(device, _addr(pa), _addr(pg), _addr(ps), _addr(pt), _addr(pn), nrow,
                                       _addr(hRo1), _addr(hRo2), _addr(hEpsilon)))

    @staticmethod
    def attention_forward(device, py, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef, masked):
        _ck(load().kai_attention_forward(device, _addr(py), _addr(pQ), _addr(pK), _addr(pV), nbat, ntimes, nvec,
                                         nhead, npiece, _addr(hCoef), int(bool(masked))))

    @staticmethod
    def gemm_force_plan(text):
        """Override the dispatcher's choice for later single products ("small split 4", "wavesplit 32", ...); "auto" or
        None clears it.  For audits of the dispatch rules only."""
        _ck(load().kai_gemm_force_plan((text or "auto").encode()))

    @staticmethod
    def attention_plan(which, nbat, ntimes, nvec, nhead, npiece):
        """How an attention entry point would run this geometry (host arithmetic only): which = "forward",
        "forward_train", "backward", "value_gradient" or "mix_values" (also mult_on_heads_backward)."""
        buf = ctypes.create_string_buffer(128)
        code = {"forward": 0, "forward_train": 1, "backward": 2, "value_gradient": 3, "mix_values": 4}[which]
        _ck(load().kai_attention_plan(code, nbat, ntimes, nvec, nhead, npiece, buf, 128))
        return buf.value.decode()

    @staticmethod
    def attention_forward_train(device, py, pp, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef, masked):
        _ck(load().kai_attention_forward_train(device, _addr(py), _addr(pp), _addr(pQ), _addr(pK), _addr(pV), nbat,
                                               ntimes, nvec, nhead, npiece, _addr(hCoef), int(bool(masked))))

    @staticmethod
    def attention_backward(device, pgQ, pgK, pgV, pgm, pp, pm, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef,
                           masked):
        _ck(load().kai_attention_backward(device, _addr(pgQ), _addr(pgK), _addr(pgV), _addr(pgm), _addr(pp), _addr(pm),
                                          _addr(pQ), _addr(pK), _addr(pV), nbat, ntimes, nvec, nhead, npiece,
                                          _addr(hCoef), int(bool(masked))))

    @staticmethod
    def dense_forward(device, py, ppre, pw, pb, px, yvec, ndat, xvec, actFunc, hLeakyAlpha):
        _ck(load().kai_dense_forward(device, _addr(py), _addr(ppre), _addr(pw), _addr(pb), _addr(px), yvec, ndat,
                                     xvec, actFunc, _addr(hLeakyAlpha)))

    @staticmethod
    def dense_backward(device, pgx, pgw, pgb, pga_work, pgy, pw, px, ppre, yvec, ndat, xvec, actFunc, hLeakyAlpha,
                       acc):
        _ck(load().kai_dense_backward(device, _addr(pgx), _addr(pgw), _addr(pgb), _addr(pga_work), _addr(pgy),
                                      _addr(pw), _addr(px), _addr(ppre), yvec, ndat, xvec, actFunc,
                                      _addr(hLeakyAlpha), int(acc)))
