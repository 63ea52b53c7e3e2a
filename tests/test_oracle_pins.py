"""Pins the CPU oracle (oracle/kai_oracle.c) without the reference, which holds no golden
vectors and cannot be built here: closed forms in float64, exact small-integer cases whose
fp32 result does not depend on the order of summation, brute force on tiny shapes written
from the index formulas, adjoint identities and special values.  Each check is chosen so that
a dropped term, a swapped operand, a wrong stride or a transposed index fails it."""
import numpy as np
import pytest
from scipy import special

from util import ko, rel_fro

RNG = np.random.default_rng(1234)


def ints(shape, lo=-4, hi=5):
    return RNG.integers(lo, hi, size=shape).astype(np.float32)


# ---- matmul family -----------------------------------------------------------------------------

@pytest.mark.parametrize("ndat,xvec,yvec", [(3, 5, 7), (1, 1, 1), (8, 16, 4), (13, 2, 9)])
def test_matmul_family_exact_on_small_integers(ndat, xvec, yvec):
    x, w, gy = ints((ndat, xvec)), ints((yvec, xvec)), ints((ndat, yvec))
    # non-square shapes with distinct sizes: any index mix-up changes the result or the shape
    assert np.array_equal(ko.matmul(w, x), (x.astype(np.int64) @ w.astype(np.int64).T).astype(np.float32))
    assert np.array_equal(ko.matmul_backward_x(gy, w), (gy.astype(np.int64) @ w.astype(np.int64)).astype(np.float32))
    assert np.array_equal(ko.matmul_backward_w(gy, x, yvec, xvec),
                          (gy.astype(np.int64).T @ x.astype(np.int64)).astype(np.float32))


def test_matmul_brute_force_index_formula():
    ndat, xvec, yvec = 3, 5, 7
    x = RNG.standard_normal((ndat, xvec)).astype(np.float32)
    w = RNG.standard_normal((yvec, xvec)).astype(np.float32)
    gy = RNG.standard_normal((ndat, yvec)).astype(np.float32)
    y = np.zeros((ndat, yvec), np.float32)
    gx = np.zeros((ndat, xvec), np.float32)
    gw = np.zeros((yvec, xvec), np.float32)
    for nd in range(ndat):
        for ny in range(yvec):
            s = np.float32(0)
            for nx in range(xvec):
                s = np.float32(s + np.float32(w[ny, nx] * x[nd, nx]))
            y[nd, ny] = s
    for nd in range(ndat):
        for nx in range(xvec):
            s = np.float32(0)
            for ny in range(yvec):
                s = np.float32(s + np.float32(w[ny, nx] * gy[nd, ny]))
            gx[nd, nx] = s
    for ny in range(yvec):
        for nx in range(xvec):
            s = np.float32(0)
            for nd in range(ndat):
                s = np.float32(s + np.float32(x[nd, nx] * gy[nd, ny]))
            gw[ny, nx] = s
    # sequential, separately rounded multiply and add: bit-exact
    assert np.array_equal(ko.matmul(w, x), y)
    assert np.array_equal(ko.matmul_backward_x(gy, w), gx)
    assert np.array_equal(ko.matmul_backward_w(gy, x, yvec, xvec), gw)


def test_matmul_is_not_contracted_into_fma():
    # a*b + c with a*b rounded first differs from fma(a,b,c) for these values
    a, b = np.float32(1 + 2 ** -12), np.float32(1 + 2 ** -12)
    c = -np.float32(a * b)
    w = np.array([[a, 1.0]], np.float32)
    x = np.array([[b, c]], np.float32)
    # sequential: (0 + a*b) + 1*c = round(a*b) - round(a*b) = 0 exactly; an FMA would leave the rounding error
    assert ko.matmul(w, x)[0, 0] == 0.0


def test_matmul_closed_form_float64_and_special_cases():
    x = RNG.standard_normal((64, 300)).astype(np.float32)
    w = RNG.standard_normal((50, 300)).astype(np.float32)
    gy = RNG.standard_normal((64, 50)).astype(np.float32)
    assert rel_fro(ko.matmul(w, x), x.astype(np.float64) @ w.astype(np.float64).T) < 1e-6
    assert rel_fro(ko.matmul_backward_x(gy, w), gy.astype(np.float64) @ w.astype(np.float64)) < 1e-6
    assert rel_fro(ko.matmul_backward_w(gy, x, 50, 300), gy.astype(np.float64).T @ x.astype(np.float64)) < 1e-6
    eye = np.eye(300, dtype=np.float32)
    assert np.array_equal(ko.matmul(eye, x), x)                     # W = I
    ones = np.ones((4, 300), np.float32)
    assert np.array_equal(ko.matmul(ones, ones), np.full((4, 4), 300, np.float32))   # all ones -> K
    # transposed-layout equivalence: NT(X, W) == NN(X, W^T)
    assert np.array_equal(ko.matmul(w, x), ko.matmul_backward_x(x, np.ascontiguousarray(w.T)))


def test_matmul_acc_and_row_range_and_threads():
    x, w = ints((6, 9)), ints((5, 9))
    y = ko.matmul(w, x)
    assert np.array_equal(ko.matmul(w, x, acc_into=y), 2 * y)        # acc adds to what is there
    gy = ints((6, 5))
    gx = ko.matmul_backward_x(gy, w)
    assert np.array_equal(ko.matmul_backward_x(gy, w, acc_into=gx), 2 * gx)
    gw = ko.matmul_backward_w(gy, x, 5, 9)
    assert np.array_equal(ko.matmul_backward_w(gy, x, 5, 9, acc_into=gw), 2 * gw)
    xf = RNG.standard_normal((40, 33)).astype(np.float32)
    wf = RNG.standard_normal((21, 33)).astype(np.float32)
    full = ko.matmul(wf, xf)
    assert np.array_equal(ko.matmul_rows(wf, xf, [3, 17, 39]), full[[3, 17, 39]])
    assert np.array_equal(ko.matmul_parallel(wf, xf, 4), full)       # bit-identical across threads


def test_adjoint_identities():
    x = RNG.standard_normal((12, 20)).astype(np.float32)
    w = RNG.standard_normal((15, 20)).astype(np.float32)
    gy = RNG.standard_normal((12, 15)).astype(np.float32)
    a = np.vdot(gy.astype(np.float64), ko.matmul(w, x))
    b = np.vdot(ko.matmul_backward_x(gy, w).astype(np.float64), x)
    c = np.vdot(ko.matmul_backward_w(gy, x, 15, 20).astype(np.float64), w)
    assert abs(a - b) < 1e-4 * abs(a) and abs(a - c) < 1e-4 * abs(a)


# ---- bias ------------------------------------------------------------------------------------------

def test_bias_ops():
    a, b = ints((7, 5)), ints((5,))
    assert np.array_equal(ko.add_bias(a, b), a + b[None, :])
    assert np.array_equal(ko.add_bias_backward_b(a, 5), a.sum(axis=0))
    g0 = ints((5,))
    assert np.array_equal(ko.add_bias_backward_b(a, 5, acc_into=g0), g0 + a.sum(axis=0))
    f = RNG.standard_normal((300, 17)).astype(np.float32)
    assert rel_fro(ko.add_bias_backward_b(f, 17), np.ones(300) @ f.astype(np.float64)) < 1e-6
    # sequential order of the column sum: row-ascending, bit-exact
    s = np.zeros(17, np.float32)
    for r in range(300):
        s = (s + f[r]).astype(np.float32)
    assert np.array_equal(ko.add_bias_backward_b(f, 17), s)


# ---- activations -----------------------------------------------------------------------------------

def test_relu_and_leaky_special_values():
    x = np.array([[-0.0, 0.0, np.nan, np.inf, -np.inf, -2.0, 3.0]], np.float32)
    y = ko.activate(x, "relu")
    assert np.array_equal(y, np.array([[0, 0, 0, np.inf, 0, 0, 3]], np.float32))
    assert not np.signbit(y[0, 0])                                    # -0 -> +0, NaN -> 0
    yl = ko.activate(x, "leaky", 0.25)
    assert yl[0, 5] == -0.5 and yl[0, 6] == 3.0 and np.isnan(yl[0, 2]) and yl[0, 4] == -np.inf
    y0 = ko.activate(x, "leaky", None)                                # null hyper-parameter reads as 0
    assert y0[0, 5] == 0.0 and y0[0, 6] == 3.0


def test_activation_closed_forms():
    x = np.linspace(-6, 6, 241, dtype=np.float32).reshape(1, -1)
    x64 = x.astype(np.float64)
    sig = 1 / (1 + np.exp(-x64))
    softplus = np.log1p(np.exp(x64))
    lam, alp = 1.0507009, 1.6732632
    want = {
        "none": x64,
        "sigmoid": sig,
        "tanh": np.tanh(x64),
        "gelu": x64 * 0.5 * (1 + special.erf(x64 / np.sqrt(2))),
        "selu": np.where(x64 > 0, lam * x64, lam * alp * (np.exp(x64) - 1)),
        "mish": x64 * np.tanh(softplus),
        "swish": x64 * sig,
    }
    for name, ref in want.items():
        np.testing.assert_allclose(ko.activate(x, name), ref, rtol=3e-6, atol=3e-7, err_msg=name)
    rows = (4 * RNG.standard_normal((5, 11))).astype(np.float32)
    np.testing.assert_allclose(ko.activate(rows, "softmax"), special.softmax(rows.astype(np.float64), axis=1),
                               rtol=2e-6, atol=1e-8)


@pytest.mark.parametrize("name", ["none", "relu", "leaky", "sigmoid", "tanh", "gelu", "selu", "mish", "swish"])
def test_activation_derivative_matches_finite_difference_of_float64_function(name):
    x = np.array([[-3.1, -1.2, -0.4, 0.3, 0.9, 2.2, 4.5]], np.float32)
    alpha = 0.2 if name == "leaky" else None
    f = {
        "none": lambda t: t,
        "relu": lambda t: np.maximum(t, 0),
        "leaky": lambda t: np.where(t > 0, t, 0.2 * t),
        "sigmoid": lambda t: 1 / (1 + np.exp(-t)),
        "tanh": np.tanh,
        "gelu": lambda t: t * 0.5 * (1 + special.erf(t / np.sqrt(2))),
        "selu": lambda t: np.where(t > 0, 1.0507009 * t, 1.0507009 * 1.6732632 * (np.exp(t) - 1)),
        "mish": lambda t: t * np.tanh(np.log1p(np.exp(t))),
        "swish": lambda t: t / (1 + np.exp(-t)),
    }[name]
    x64 = x.astype(np.float64)
    h = 1e-6
    deriv = (f(x64 + h) - f(x64 - h)) / (2 * h)
    gy = np.array([[2.0, -1.0, 0.5, 3.0, -2.0, 1.0, 0.25]], np.float32)
    np.testing.assert_allclose(ko.activate_backward(gy, x, name, alpha), deriv * gy, rtol=2e-5, atol=2e-6)
    if name in ("none", "relu", "leaky", "sigmoid", "tanh"):
        y = ko.activate(x, name, alpha)
        np.testing.assert_allclose(ko.activate_backward_with_y(gy, y, name, alpha), deriv * gy, rtol=2e-5, atol=2e-6)


def test_activation_error_codes():
    x = np.zeros((1, 4), np.float32)
    for fn, args, bad in [(ko.activate, (x, 10), None), (ko.activate, (x, -1), None),
                          (ko.activate_backward, (x, x, 9), None), (ko.activate_backward_with_y, (x, x, 5), None)]:
        with pytest.raises(ko.OracleError) as e:
            fn(*args)
        assert e.value.code == 8          # VERR_CONDITIONAL_STATEMENT


# ---- attention -------------------------------------------------------------------------------------

def heads(a, nhead):
    """[B,T,H*D] -> [B,H,T,D] float64"""
    b, t, v = a.shape
    return a.astype(np.float64).reshape(b, t, nhead, v // nhead).transpose(0, 2, 1, 3)


@pytest.mark.parametrize("nbat,ntimes,nhead,npiece", [(2, 5, 3, 4), (1, 7, 1, 6), (3, 4, 2, 1)])
def test_attention_forward_reduces_to_per_head_matmul(nbat, ntimes, nhead, npiece):
    nvec = nhead * npiece
    q = RNG.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    k = RNG.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    v = RNG.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    coef = 0.37
    s = ko.mult_on_heads(k, q, nhead, coef)                      # [B,Tq,Tk,H]
    ref_s = np.einsum("bhqd,bhkd->bqkh", heads(q, nhead), heads(k, nhead)) * coef
    np.testing.assert_allclose(s, ref_s, rtol=1e-5, atol=1e-6)
    # asymmetric in q and k: swapping the operands must transpose the time axes
    np.testing.assert_allclose(ko.mult_on_heads(q, k, nhead, coef), ref_s.transpose(0, 2, 1, 3), rtol=1e-5, atol=1e-6)
    assert np.array_equal(ko.mult_on_heads(k, q, nhead, None), np.zeros_like(s))   # null coef reads as 0
    p = ko.softmax_direct_on_axis(s, nbat * ntimes, ntimes, nhead)
    np.testing.assert_allclose(p, special.softmax(ref_s, axis=2), rtol=1e-5, atol=1e-7)
    o = ko.mix_values(p, v, nhead)                               # [B,T,H*D]
    ref_o = np.einsum("bqkh,bhkd->bqhd", p.astype(np.float64), heads(v, nhead)).reshape(nbat, ntimes, nvec)
    np.testing.assert_allclose(o, ref_o, rtol=1e-5, atol=1e-6)
    # uniform probabilities: the output is the mean of V over the keys
    u = np.full_like(p, 1.0 / ntimes)
    np.testing.assert_allclose(ko.mix_values(u, v, nhead), np.repeat(v.mean(axis=1, keepdims=True), ntimes, axis=1),
                               rtol=1e-5, atol=1e-6)


def test_softmax_axis_properties():
    s = (3 * RNG.standard_normal((6, 9, 4))).astype(np.float32)
    p = ko.softmax_direct_on_axis(s, 6, 9, 4)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, atol=1e-6)
    shifted = ko.softmax_direct_on_axis(s + np.float32(8.0), 6, 9, 4)
    np.testing.assert_allclose(shifted, p, rtol=1e-5, atol=1e-7)             # shift invariance
    # strided layout equals transposing and taking the plain row softmax
    rows = np.ascontiguousarray(s.transpose(0, 2, 1)).reshape(24, 9, 1)
    pr = ko.softmax_direct_on_axis(rows, 24, 9, 1).reshape(6, 4, 9).transpose(0, 2, 1)
    assert np.array_equal(pr, p)
    m = s.copy()
    m[:, 5:, :] = -np.inf
    pm = ko.softmax_direct_on_axis(m, 6, 9, 4)
    assert (pm[:, 5:, :] == 0).all() and np.allclose(pm[:, :5, :].sum(axis=1), 1.0, atol=1e-6)


def test_mask():
    p = RNG.standard_normal((2, 4, 4, 3)).astype(np.float32)
    f = ko.set_mh_attention_mask(p, True)
    b = ko.set_mh_attention_mask(p, False)
    for q in range(4):
        for k in range(4):
            if k > q:
                assert (f[:, q, k, :] == -np.inf).all() and (b[:, q, k, :] == 0).all()
            else:
                assert np.array_equal(f[:, q, k, :], p[:, q, k, :]) and np.array_equal(b[:, q, k, :], p[:, q, k, :])


@pytest.mark.parametrize("nbat,ntimes,nhead,npiece", [(2, 5, 3, 4), (1, 6, 1, 3)])
def test_attention_backward_closed_forms(nbat, ntimes, nhead, npiece):
    nvec = nhead * npiece
    v = RNG.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    kq = RNG.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    gy = RNG.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    p = special.softmax(RNG.standard_normal((nbat, ntimes, ntimes, nhead)), axis=2).astype(np.float32)
    gp = RNG.standard_normal((nbat, ntimes, ntimes, nhead)).astype(np.float32)
    gyh = heads(gy, nhead)                                                   # [B,H,T,D]
    np.testing.assert_allclose(ko.mix_values_backward_prop(gy, v, nhead),
                               np.einsum("bhqd,bhkd->bqkh", gyh, heads(v, nhead)), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(ko.mix_values_backward_value(gy, p, nhead),
                               np.einsum("bqkh,bhqd->bkhd", p.astype(np.float64), gyh).reshape(nbat, ntimes, nvec),
                               rtol=1e-5, atol=1e-6)
    # the score gradient is read as [b, t, k, h] with t the OUTPUT row for key and query alike
    np.testing.assert_allclose(ko.mult_on_heads_backward(gp, kq, nhead),
                               np.einsum("btkh,bhkd->bthd", gp.astype(np.float64), heads(kq, nhead)).reshape(
                                   nbat, ntimes, nvec), rtol=1e-5, atol=1e-6)
    coef = 0.5
    p64, g64 = p.astype(np.float64), gp.astype(np.float64)
    ref = coef * p64 * (g64 - (p64 * g64).sum(axis=2, keepdims=True))
    np.testing.assert_allclose(ko.softmax_direct_on_axis_backward(gp, p, coef), ref, rtol=1e-5, atol=1e-6)
    # adjoint pairs: <gy, mix(p, v)> = <backward_prop(gy, v), p> = <backward_value(gy, p), v>
    a = np.vdot(gy.astype(np.float64), ko.mix_values(p, v, nhead))
    b = np.vdot(ko.mix_values_backward_prop(gy, v, nhead).astype(np.float64), p)
    c = np.vdot(ko.mix_values_backward_value(gy, p, nhead).astype(np.float64), v)
    assert abs(a - b) < 1e-4 * abs(a) + 1e-5 and abs(a - c) < 1e-4 * abs(a) + 1e-5


# ---- parameter update (vmath.cu:364-490) --------------------------------------------------------------------------

def test_accumulate_subtract_and_decay_exact_cases():
    y = np.array([1, -2, 3.5, 0], np.float32)
    x = np.array([4, 2, -0.5, -0.0], np.float32)
    np.testing.assert_array_equal(ko.accumulate_grad(y, x), np.array([5, 0, 3, 0], np.float32))
    # powers of two keep every product and difference exact
    np.testing.assert_array_equal(ko.subtract_param_grad(y, x, 0.5), np.array([-1, -3, 3.75, 0], np.float32))
    np.testing.assert_array_equal(ko.subtract_param_grad(y, x, None), y)          # null HYPER reads as 0
    p = np.array([2, -4, 0, 1], np.float32)
    g = np.array([1, 1, 1, -1], np.float32)
    np.testing.assert_array_equal(ko.apply_decay(p, g, None, None), g)            # no decay: delta = g
    np.testing.assert_array_equal(ko.apply_decay(p, g, 0.0, 0.25), g + 0.25 * p)  # L2 only
    np.testing.assert_array_equal(ko.apply_decay(p, g, 0.5, 0.0), g + 0.5 * np.sign(p))   # L1 only: sign(0) = 0
    np.testing.assert_array_equal(ko.apply_decay(p, g, 0.5, 0.25), g + 0.25 * p + 0.5 * np.sign(p))
    np.testing.assert_array_equal(ko.apply_decay(p, g, -1.0, -1.0), g)            # non-positive coefficients are skipped


def test_subtract_rounds_the_product_before_the_difference():
    # p - g * lr with separately rounded product (no FMA): brute force in explicit fp32 steps
    rng = np.random.default_rng(5)
    p = rng.standard_normal(1000).astype(np.float32)
    g = rng.standard_normal(1000).astype(np.float32)
    lr = np.float32(0.0123)
    want = (p - (g * lr).astype(np.float32)).astype(np.float32)
    np.testing.assert_array_equal(ko.subtract_param_grad(p, g, float(lr)), want)


def test_adam_first_step_closed_form_and_float64_recurrence():
    rng = np.random.default_rng(6)
    g = rng.standard_normal(500).astype(np.float32)
    z = np.zeros(500, np.float32)
    ro1, ro2, eps = 0.9, 0.999, 1e-8
    a, s, t, n = ko.eval_adam_delta(g, z, z, z, ro1, ro2, eps)
    # step 1: s / (1 - ro1) = g and t / (1 - ro2) = g^2, so the update direction is g / (|g| + eps)
    np.testing.assert_allclose(a, g / (np.abs(g) + eps), rtol=2e-6)
    np.testing.assert_array_equal(n, np.ones(500, np.float32))
    # three more steps against a float64 recurrence
    s64, t64 = s.astype(np.float64), t.astype(np.float64)
    for step in range(2, 5):
        g2 = rng.standard_normal(500).astype(np.float32)
        a, s, t, n = ko.eval_adam_delta(g2, s, t, n, ro1, ro2, eps)
        s64 = ro1 * s64 + (1 - ro1) * g2
        t64 = ro2 * t64 + (1 - ro2) * g2.astype(np.float64) ** 2
        want = (s64 / (1 - ro1 ** step)) / (np.sqrt(t64 / (1 - ro2 ** step)) + eps)
        np.testing.assert_allclose(a, want, rtol=2e-5, atol=1e-6)
        np.testing.assert_array_equal(n, np.full(500, step, np.float32))


# ---- transposes (vmath.cu:9384-9510) --------------------------------------------------------------------------------

def test_transposes_equal_numpy():
    rng = np.random.default_rng(8)
    for shape, axes in [((5,), (0,)), ((3, 7), (1, 0)), ((2, 3, 4), (2, 0, 1)), ((2, 3, 4), (0, 2, 1)),
                        ((3, 1, 5, 2), (3, 2, 1, 0)), ((4, 3, 2, 5), (0, 1, 2, 3))]:
        x = rng.standard_normal(shape).astype(np.float32)
        y = ko.transpose(x, axes)
        np.testing.assert_array_equal(y, np.transpose(x, axes))
        # the backward pass scatters a gradient of y's shape back to x's positions: the inverse permutation
        gy = rng.standard_normal(y.shape).astype(np.float32)
        np.testing.assert_array_equal(ko.transpose_backward(gy, shape, axes), np.transpose(gy, np.argsort(axes)))
    x = rng.standard_normal((37, 53)).astype(np.float32)            # [ncol, nrow]
    np.testing.assert_array_equal(ko.transpose_bin(x, 53, 37), x.T)


# ---- recurrent cells (vmath.cu:732-778, 4807-4826, 4946-5033) --------------------------------------------------------

def _sig64(v):
    return 1.0 / (1.0 + np.exp(-np.asarray(v, np.float64)))


def _gru64(ai, ar, hprev):
    nrec = hprev.shape[1]
    r = _sig64(ai[:, :nrec] + ar[:, :nrec])
    z = _sig64(ai[:, nrec:2 * nrec] + ar[:, nrec:2 * nrec])
    cand = np.tanh(ai[:, 2 * nrec:] + r * ar[:, 2 * nrec:])
    return (1 - z) * cand + z * hprev


def test_copy_and_add_exact():
    a = np.arange(-5, 6, dtype=np.float32)
    b = np.arange(11, dtype=np.float32) * 3
    np.testing.assert_array_equal(ko.copy(a), a)
    np.testing.assert_array_equal(ko.add(a, b), a + b)


def test_lstm_cell_equals_textbook_float64():
    rng = np.random.default_rng(9)
    ndat, nrec = 5, 7
    a = (rng.standard_normal((ndat, 4 * nrec)) * 2).astype(np.float32)
    s0 = rng.standard_normal((ndat, nrec)).astype(np.float32)
    i, f, g, o = (a[:, k * nrec:(k + 1) * nrec].astype(np.float64) for k in range(4))
    for prev in (s0, None):
        r, s = ko.lstm_process(a, prev)
        want_s = (0 if prev is None else prev) * _sig64(f) + np.tanh(g) * _sig64(i)
        np.testing.assert_allclose(s, want_s, rtol=0, atol=5e-7)
        np.testing.assert_allclose(r, np.tanh(want_s) * _sig64(o), rtol=0, atol=5e-7)
    # a gate order mistake would show here: only the forget gate open keeps the state, output gate shut gives 0
    a2 = np.full((1, 4), -40.0, np.float32)
    a2[0, 1] = 40.0
    r, s = ko.lstm_process(a2, np.array([[0.75]], np.float32))
    assert s[0, 0] == 0.75 and abs(r[0, 0]) < 1e-12


def _lstm64(a, prev):
    """Textbook LSTM cell in float64; gate order input, forget, block, output.  Returns (output, state)."""
    nrec = a.shape[1] // 4
    i, f, g, o = (a[:, k * nrec:(k + 1) * nrec] for k in range(4))
    s = prev * _sig64(f) + np.tanh(g) * _sig64(i)
    return np.tanh(s) * _sig64(o), s


def test_lstm_cell_backward_against_central_differences():
    # The reference's device kernel (vmath.cu:4899-4937): given gr = dL/d(output) and gs = dL/d(state) of THIS
    # step it returns dL/d(gate sums) and dL/d(previous state).  L = <output, gr> + <state, gs> in float64.
    rng = np.random.default_rng(11)
    ndat, nrec = 3, 5                                 # nrec > 4: the host loop's index expression would leave the buffer
    a = (rng.standard_normal((ndat, 4 * nrec)) * 1.5).astype(np.float32)
    s0 = rng.standard_normal((ndat, nrec)).astype(np.float32)
    gr = rng.standard_normal((ndat, nrec)).astype(np.float32)
    gs = rng.standard_normal((ndat, nrec)).astype(np.float32)

    def loss(a_, prev_):
        r, s = _lstm64(a_, prev_)
        return float((r * gr).sum() + (s * gs).sum())

    got_gs, got_ga = ko.lstm_process_backward(gr, gs, a, s0)
    eps = 1e-6
    base = (a.astype(np.float64), s0.astype(np.float64))
    for which, got in ((0, got_ga), (1, got_gs)):
        num = np.zeros_like(base[which])
        for idx in np.ndindex(num.shape):
            hi = [b.copy() for b in base]
            lo = [b.copy() for b in base]
            hi[which][idx] += eps
            lo[which][idx] -= eps
            num[idx] = (loss(*hi) - loss(*lo)) / (2 * eps)
        np.testing.assert_allclose(got, num, rtol=0, atol=2e-6)
    # no previous state (first processed step): same as a zero state, and its gradient is still forget * g_state
    z_gs, z_ga = ko.lstm_process_backward(gr, gs, a, None)
    w_gs, w_ga = ko.lstm_process_backward(gr, gs, a, np.zeros_like(s0))
    np.testing.assert_array_equal(z_ga, w_ga)
    np.testing.assert_array_equal(z_gs, w_gs)
    assert np.all(z_ga[:, nrec:2 * nrec] == 0)        # forget gate's gradient = old_state * ... = 0
    # gate-order trap: forget gate wide open, the others shut: the state passes through, so does its gradient,
    # and nothing reaches the gate sums (every sigmoid/tanh derivative is ~0 or multiplied by ~0)
    a2 = np.full((1, 4), -40.0, np.float32)
    a2[0, 1] = 40.0
    p_gs, p_ga = ko.lstm_process_backward(np.array([[0.3]], np.float32), np.array([[0.7]], np.float32), a2,
                                          np.array([[0.75]], np.float32))
    assert p_gs[0, 0] == np.float32(0.7) and np.all(np.abs(p_ga) < 1e-12)
    # the output's gradient is an input only
    gr_before = gr.copy()
    ko.lstm_process_backward(gr, gs, a, s0)
    np.testing.assert_array_equal(gr, gr_before)


def test_gru_cell_and_its_backward():
    rng = np.random.default_rng(10)
    ntimes, ndat, nrec = 3, 4, 6
    ai = rng.standard_normal((ndat, 3 * nrec)).astype(np.float32)
    ar = rng.standard_normal((ndat, 3 * nrec)).astype(np.float32)
    recurs = np.zeros((ntimes, ndat, nrec), np.float32)
    recurs[0] = rng.standard_normal((ndat, nrec)).astype(np.float32)
    # step 0 sees no previous output, step 1 reads step 0
    first = ko.gru_process(np.zeros_like(recurs), ai, ar, 0)[0]
    np.testing.assert_allclose(first, _gru64(ai, ar, np.zeros((ndat, nrec))), rtol=0, atol=5e-7)
    ko.gru_process(recurs, ai, ar, 1)
    np.testing.assert_allclose(recurs[1], _gru64(ai, ar, recurs[0]), rtol=0, atol=5e-7)
    # backward against central differences of the float64 closed form
    gh = rng.standard_normal((ndat, nrec)).astype(np.float32)
    gprev, gai, gar = ko.gru_process_backward(gh, recurs, ai, ar, 1)
    loss = lambda ai_, ar_, hp_: float((_gru64(ai_, ar_, hp_) * gh).sum())
    eps = 1e-6
    base = (ai.astype(np.float64), ar.astype(np.float64), recurs[0].astype(np.float64))
    for which, got in ((0, gai), (1, gar), (2, gprev)):
        num = np.zeros_like(base[which])
        for idx in np.ndindex(num.shape):
            hi = [b.copy() for b in base]
            lo = [b.copy() for b in base]
            hi[which][idx] += eps
            lo[which][idx] -= eps
            num[idx] = (loss(*hi) - loss(*lo)) / (2 * eps)
        np.testing.assert_allclose(got, num, rtol=0, atol=2e-6)


# ---- cosinesim (vmath.cu:6459-6480) ----------------------------------------------------------------------------------

def test_cosinesim_against_float64_and_special_rows():
    rng = np.random.default_rng(12)
    a = rng.standard_normal((6, 33)).astype(np.float32)
    b = rng.standard_normal((4, 33)).astype(np.float32)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    want = (a64 @ b64.T) / (np.linalg.norm(a64, axis=1)[:, None] * np.linalg.norm(b64, axis=1)[None, :])
    np.testing.assert_allclose(ko.cosinesim(a, b), want, rtol=0, atol=1e-6)
    # a row with itself is 1, with its negative -1, with an orthogonal one 0; a zero row gives 0 (the 1e-20 guard)
    e = np.array([[3, 4, 0], [-3, -4, 0], [0, 0, 2], [0, 0, 0]], np.float32)
    got = ko.cosinesim(e[:1], e)
    np.testing.assert_array_equal(got, np.array([[1, -1, 0, 0]], np.float32))
    # leading axes fold into rows (vtensor.cpp:5878-5880)
    assert ko.cosinesim(a.reshape(2, 3, 33), b).shape == (6, 4)
