"""Parity of the HIP path with the CPU oracle, through the C-ABI, on the five benchmark
configurations and on the edge cases of the path.  Bar: relative Frobenius error <= 1e-5
(fp32, differences of summation order only); exact where no arithmetic is involved."""
import numpy as np
import pytest

from util import REL_FRO_TOL, cfg1, cfg2, cfg3, cfg4, cfg5, ko, rel_fro

pytestmark = pytest.mark.gpu

kai = None
VMath = None
DB = None


@pytest.fixture(scope="module", autouse=True)
def _lib():
    global kai, VMath, DB
    from deep_learning_framework_amd import kai as _kai
    kai = _kai
    VMath = _kai.VMath
    DB = _kai.DeviceBuffer
    kai.load()
    kai.set_device(0)
    yield
    kai.synchronize()


def dev(a):
    return DB.from_numpy(np.ascontiguousarray(a, np.float32))


def check(got, ref, tol=REL_FRO_TOL, what=""):
    err = rel_fro(got, ref)
    assert np.isfinite(got).all(), what + ": non-finite output"
    assert err <= tol, "%s: rel Frobenius error %.3e > %.1e" % (what, err, tol)


# ---- configuration 1: dense forward 64 x 784 -> 512, ReLU ------------------------------------------

def test_cfg1_dense_forward_unfused_and_fused():
    x, w, b = cfg1()
    ref_pre = ko.add_bias(ko.matmul(w, x), b)
    ref = ko.activate(ref_pre, "relu")
    dx, dw, db = dev(x), dev(w), dev(b)
    # the engine's three calls: matmul -> add_bias -> activate (api/vconst.cpp:11)
    y = DB(64 * 512 * 4)
    VMath.matmul(0, y, dw, dx, 512, 64, 784, False)
    VMath.add_bias(0, y, y, db, 64, 512)
    VMath.activate(0, y, y, 64, 512, kai.ACT["relu"], None)
    check(y.to_numpy((64, 512)), ref, what="cfg1 unfused")
    # one launch
    y2, pre = DB(64 * 512 * 4), DB(64 * 512 * 4)
    VMath.dense_forward(0, y2, pre, dw, db, dx, 512, 64, 784, kai.ACT["relu"], None)
    check(y2.to_numpy((64, 512)), ref, what="cfg1 fused")
    check(pre.to_numpy((64, 512)), ref_pre, what="cfg1 fused pre-activation")
    # BASELINE layout W'[784,512] = w.T as a row-major [K,N] operand
    wt = dev(np.ascontiguousarray(w.T))
    y3 = DB(64 * 512 * 4)
    VMath.gemm_f32(0, 0, 0, 64, 512, 784, dx, 784, wt, 512, y3, 512, db, kai.ACT["relu"], None, False)
    check(y3.to_numpy((64, 512)), ref, what="cfg1 [K,N] weight layout")


# ---- configuration 2: dense forward + backward 256 x 1024 -> 1024 ---------------------------------------

def test_cfg2_dense_forward_backward():
    x, w, b, gy = cfg2()
    ref_y = ko.add_bias(ko.matmul(w, x), b)
    ref_gx = ko.matmul_backward_x(gy, w)
    ref_gw = ko.matmul_backward_w(gy, x, 1024, 1024)
    ref_gb = ko.add_bias_backward_b(gy, 1024)
    dx, dw, db, dgy = dev(x), dev(w), dev(b), dev(gy)
    y = DB(256 * 1024 * 4)
    VMath.matmul(0, y, dw, dx, 1024, 256, 1024, False)
    VMath.add_bias(0, y, y, db, 256, 1024)
    check(y.to_numpy((256, 1024)), ref_y, what="cfg2 Y")
    gx, gw, gb = DB(256 * 1024 * 4), DB(1024 * 1024 * 4), DB(1024 * 4)
    VMath.matmul_backward_x(0, gx, dgy, dw, 1024, 256, 1024, False)
    VMath.matmul_backward_w(0, gw, dgy, dx, 1024, 256, 1024, False)
    VMath.add_bias_backward_b(0, gb, dgy, 256, 1024, False)
    check(gx.to_numpy((256, 1024)), ref_gx, what="cfg2 dX")
    check(gw.to_numpy((1024, 1024)), ref_gw, what="cfg2 dW")
    check(gb.to_numpy((1024,)), ref_gb, what="cfg2 db")
    # fused backward entry point, no activation
    gx2, gw2, gb2 = DB(256 * 1024 * 4), DB(1024 * 1024 * 4), DB(1024 * 4)
    VMath.dense_backward(0, gx2, gw2, gb2, None, dgy, dw, dx, None, 1024, 256, 1024, kai.ACT["none"], None, False)
    check(gx2.to_numpy((256, 1024)), ref_gx, what="cfg2 fused dX")
    check(gw2.to_numpy((1024, 1024)), ref_gw, what="cfg2 fused dW")
    check(gb2.to_numpy((1024,)), ref_gb, what="cfg2 fused db")


def test_cfg2_relu_backward_chain():
    x, w, b, gy = cfg2()
    pre = ko.add_bias(ko.matmul(w, x), b)
    ga = ko.activate_backward(gy, pre, "relu")
    ref_gx = ko.matmul_backward_x(ga, w)
    ref_gw = ko.matmul_backward_w(ga, x, 1024, 1024)
    ref_gb = ko.add_bias_backward_b(ga, 1024)
    dx, dw, dgy, dpre = dev(x), dev(w), dev(gy), dev(pre)
    gx, gw, gb, work = DB(256 * 1024 * 4), DB(1024 * 1024 * 4), DB(1024 * 4), DB(256 * 1024 * 4)
    VMath.dense_backward(0, gx, gw, gb, work, dgy, dw, dx, dpre, 1024, 256, 1024, kai.ACT["relu"], None, False)
    check(gx.to_numpy((256, 1024)), ref_gx, what="relu chain dX")
    check(gw.to_numpy((1024, 1024)), ref_gw, what="relu chain dW")
    check(gb.to_numpy((1024,)), ref_gb, what="relu chain db")


# the bias gradient rides on the weight-gradient product where that runs on the small or medium tile (whole
# tiles, edges in every dimension, a tile column count above one) and is a separate kernel elsewhere (reduction
# long enough to be split, 256-wide tiles)
@pytest.mark.parametrize("ndat,yvec,xvec,acc", [(256, 1024, 1024, True), (100, 130, 70, False), (37, 200, 333, True),
                                                (64, 2048, 1024, False), (1024, 64, 64, False),
                                                (160, 2304, 2560, True), (5, 64, 64, False), (16, 4096, 4096, False)])
def test_dense_backward_bias_gradient_fused_or_not(ndat, yvec, xvec, acc):
    rng = np.random.default_rng(ndat + 3 * yvec + 7 * xvec)
    x = rng.standard_normal((ndat, xvec)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, (yvec, xvec)).astype(np.float32)
    gy = rng.standard_normal((ndat, yvec)).astype(np.float32)
    gx0 = rng.standard_normal((ndat, xvec)).astype(np.float32)
    gw0 = rng.standard_normal((yvec, xvec)).astype(np.float32)
    gb0 = rng.standard_normal(yvec).astype(np.float32)
    gx, gw, gb = dev(gx0), dev(gw0), dev(gb0)
    VMath.dense_backward(0, gx, gw, gb, None, dev(gy), dev(w), dev(x), None, yvec, ndat, xvec, kai.ACT["none"], None,
                         acc)
    a = dict(acc_into=gx0) if acc else {}
    check(gx.to_numpy((ndat, xvec)), ko.matmul_backward_x(gy, w, **a), what="dX")
    a = dict(acc_into=gw0) if acc else {}
    check(gw.to_numpy((yvec, xvec)), ko.matmul_backward_w(gy, x, yvec, xvec, **a), what="dW")
    a = dict(acc_into=gb0) if acc else {}
    check(gb.to_numpy((yvec,)), ko.add_bias_backward_b(gy, yvec, **a), what="db")


# The whole backward of a dense layer through kai_dense_backward with an activation and NO work buffer: shapes that
# run as one launch (both products, the derivative of relu / leaky relu on the loads, the bias gradient from the
# staged tiles; gx's reduction whole or cut into parts) and shapes that run the separate kernels with ga in the
# library scratch.  The bias gradient sums in the order of a sequential loop: bit-identical to the oracle.
@pytest.mark.parametrize("ndat,yvec,xvec,act,acc,one_launch", [
    (256, 1024, 1024, "relu", False, True),      # configuration 2: gx cut into 4 parts of 256 steps
    (256, 1024, 1024, "leaky", True, True),
    (128, 1024, 1024, "relu", True, True),       # 128-column tiles, 8 parts of 4 tiles: one tile staged at a time
    (64, 512, 128, "relu", True, True),          # gx cut into 4 parts of 128
    (128, 256, 320, "none", False, True),        # two parts of 128
    (512, 512, 512, "leaky", False, True),       # no cut: a part would be shorter than gw's reduction
    (1024, 1024, 1024, "relu", False, True),     # 512 workgroups, no cut
    (64, 2048, 64, "relu", True, True),          # one tile of gx, 16 parts
    (192, 1024, 1024, "relu", False, False),      # separate kernels from here on: 192 is no whole number of 64s
    (100, 130, 70, "leaky", True, False),
    (2048, 2048, 1024, "relu", False, False),     # too many workgroups for the paired launch
    (256, 1024, 1024, "gelu", False, False),      # a derivative that is no select
])
def test_dense_backward_with_activation_and_no_work_buffer(ndat, yvec, xvec, act, acc, one_launch):
    rng = np.random.default_rng(ndat + 3 * yvec + 7 * xvec + len(act))
    x = rng.standard_normal((ndat, xvec)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, (yvec, xvec)).astype(np.float32)
    pre = rng.standard_normal((ndat, yvec)).astype(np.float32)
    pre[0, :7] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-30, -1e-30][:min(7, yvec)]
    gy = rng.standard_normal((ndat, yvec)).astype(np.float32)
    gx0 = rng.standard_normal((ndat, xvec)).astype(np.float32)
    gw0 = rng.standard_normal((yvec, xvec)).astype(np.float32)
    gb0 = rng.standard_normal(yvec).astype(np.float32)
    alpha = 0.1 if act == "leaky" else None
    if act == "gelu":
        pre[0, 2:5] = 0.5                                   # keep the transcendental derivative finite
    ga = gy if act == "none" else ko.activate_backward(gy, pre, act, alpha)
    a = lambda base: dict(acc_into=base) if acc else {}
    want_gx = ko.matmul_backward_x(ga, w, **a(gx0))
    want_gw = ko.matmul_backward_w(ga, x, yvec, xvec, **a(gw0))
    want_gb = ko.add_bias_backward_b(ga, yvec, **a(gb0))
    gx, gw, gb = dev(gx0), dev(gw0), dev(gb0)
    dgy, dpre = dev(gy), dev(pre)
    VMath.dense_backward(0, gx, gw, gb, None, dgy, dev(w), dev(x), dpre, yvec, ndat, xvec, kai.ACT[act], kai.hyper(alpha), acc)
    what = "dense backward %dx%dx%d %s acc=%s " % (ndat, yvec, xvec, act, acc)
    check(gx.to_numpy((ndat, xvec)), want_gx, what=what + "dX")
    check(gw.to_numpy((yvec, xvec)), want_gw, what=what + "dW")
    got_gb = gb.to_numpy((yvec,))
    check(got_gb, want_gb, what=what + "db")
    if one_launch:      # summed in the order of a sequential loop (the separate column-sum kernel folds in a tree)
        np.testing.assert_array_equal(got_gb, want_gb, err_msg=what + "db bit for bit")
    np.testing.assert_array_equal(dgy.to_numpy(gy.shape), gy)        # the inputs are read only
    # only some of the outputs requested (separate kernels; same values)
    gx2 = dev(gx0)
    VMath.dense_backward(0, gx2, None, None, None, dgy, dev(w), dev(x), dpre, yvec, ndat, xvec, kai.ACT[act], kai.hyper(alpha), acc)
    check(gx2.to_numpy((ndat, xvec)), want_gx, what=what + "dX alone")


# ---- configuration 3: 8192^3 GEMM + bias + ReLU -------------------------------------------------------------

def test_cfg3_large_gemm_bias_relu_row_sample():
    n = 8192
    a, b, bias = cfg3(n)
    da, dbm, dbias = dev(a), dev(b), dev(bias)
    c = DB(n * n * 4)
    # row-major A.B: B is a [K,N] operand
    VMath.gemm_f32(0, 0, 0, n, n, n, da, n, dbm, n, c, n, dbias, kai.ACT["relu"], None, False)
    got = c.to_numpy((n, n))
    rows = np.sort(np.random.default_rng(33).choice(n, 48, replace=False))
    bt = np.ascontiguousarray(b.T)
    ref = ko.activate(ko.add_bias(ko.matmul_rows(bt, a, rows), bias), "relu")
    check(got[rows], ref, what="cfg3 NN sampled rows")
    # engine layout: the same product with B pre-stored [N,K], fused dense entry point
    dbt = dev(bt)
    c2 = DB(n * n * 4)
    VMath.dense_forward(0, c2, None, dbt, dbias, da, n, n, n, kai.ACT["relu"], None)
    got2 = c2.to_numpy((n, n))
    check(got2[rows], ref, what="cfg3 NT sampled rows")
    # whole matrix: the two operand forms must agree with each other far inside the tolerance
    check(got2, got, tol=2e-6, what="cfg3 NN vs NT full matrix")
    # linearity over the full size: relu(A.B + bias) has no negative entry and the share of
    # positive entries of a symmetric product is one half
    assert (got >= 0).all()
    assert abs((got > 0).mean() - 0.5) < 0.01


def test_cfg3_size_backward_products_sampled_and_adjoint():
    """The backward pair at the size of configuration 3 (8192^3, the engine's NN and TN forms): sampled rows of dX
    and sampled rows of dW against the oracle, and the adjoint identities <dY, X.W^T> = <dY.W, X> = <dY^T.X, W>
    over the whole matrices (float64 sums), which tie the three products together at a size the oracle cannot
    compute in full."""
    n = 8192
    rng = np.random.default_rng(33)
    x = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    w = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    gy = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    dx, dw, dgy = dev(x), dev(w), dev(gy)
    out = DB(n * n * 4)
    VMath.matmul(0, out, dw, dx, n, n, n, False)
    y = out.to_numpy((n, n))
    VMath.matmul_backward_x(0, out, dgy, dw, n, n, n, False)
    gx = out.to_numpy((n, n))
    VMath.matmul_backward_w(0, out, dgy, dx, n, n, n, False)
    gw = out.to_numpy((n, n))
    rows = np.array([0, 4095, 4096, 8191] + list(rng.integers(0, n, 4)))
    # dX rows are independent: gx[r] = gy[r] . w
    check(gx[rows], ko.matmul_backward_x(gy[rows], w), what="8192^3 dX sampled rows")
    # dW rows belong to columns of gy: gw[c] = sum_m gy[m, c] * x[m]
    check(gw[rows], ko.matmul_backward_w(np.ascontiguousarray(gy[:, rows]), x, len(rows), n), what="8192^3 dW sampled rows")
    check(y[rows], ko.matmul_rows(w, x, rows), what="8192^3 Y sampled rows")
    dot = lambda a, b: float(np.einsum("ij,ij->", a, b, dtype=np.float64))
    s_y, s_x, s_w = dot(gy, y), dot(gx, x), dot(gw, w)
    scale = np.sqrt(dot(gy, gy) * dot(y, y))
    assert abs(s_y - s_x) <= 1e-5 * scale and abs(s_y - s_w) <= 1e-5 * scale, (s_y, s_x, s_w, scale)


def test_product_beyond_the_last_level_cache_row_sample():
    # 16384 x 16384 x 4096: operands and output (1.5 GiB) exceed the 256 MB last-level cache, so every tile's
    # operands come from HBM; sampled rows against the oracle, bias + ReLU fused
    m, n, k = 16384, 16384, 4096
    rng = np.random.default_rng(16)
    x = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    w = rng.uniform(-1, 1, (n, k)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    dx, dw, db = dev(x), dev(w), dev(b)
    y = DB(m * n * 4)
    VMath.dense_forward(0, y, None, dw, db, dx, n, m, k, kai.ACT["relu"], None)
    got = y.to_numpy((m, n))
    rows = np.unique(np.concatenate([[0, m - 1, 255, 256], rng.integers(0, m, 12)]))
    ref = ko.activate(ko.add_bias(ko.matmul_rows(w, x, rows), b), "relu")
    check(got[rows], ref, what="16384 x 16384 x 4096 sampled rows")
    assert (got >= 0).all()


# ---- configuration 4: attention batched matmul ---------------------------------------------------------------

@pytest.mark.parametrize("nbat,nhead,nvec", [(32, 1, 64), (4, 8, 512)])
def test_cfg4_attention_forward(nbat, nhead, nvec):
    ntimes = 512
    npiece = nvec // nhead
    q, k, v = cfg4(nbat, ntimes, nvec)
    coef = 1.0 / np.sqrt(npiece)
    ref_s = ko.mult_on_heads(k, q, nhead, coef)
    ref_p = ko.softmax_direct_on_axis(ref_s, nbat * ntimes, ntimes, nhead)
    ref_o = ko.mix_values(ref_p, v, nhead)
    dq, dk, dv = dev(q), dev(k), dev(v)
    hcoef = kai.hyper(coef)
    p = DB(nbat * ntimes * ntimes * nhead * 4)
    VMath.mult_on_heads(0, p, dk, dq, nbat, ntimes, nvec, nhead, npiece, hcoef)
    check(p.to_numpy(ref_s.shape), ref_s, what="cfg4 scores")
    VMath.softmax_direct_on_axis(0, p, nbat * ntimes, ntimes, nhead)
    got_p = p.to_numpy(ref_p.shape)
    check(got_p, ref_p, what="cfg4 softmax")
    np.testing.assert_allclose(got_p.sum(axis=2), 1.0, atol=1e-5)
    o = DB(nbat * ntimes * nvec * 4)
    VMath.mix_values(0, o, p, dv, nbat, ntimes, nvec, nhead, npiece)
    check(o.to_numpy((nbat, ntimes, nvec)), ref_o, what="cfg4 output")


# ---- configuration 5: skinny and ragged ------------------------------------------------------------------------

@pytest.mark.parametrize("m", [1, 4, 16])
def test_cfg5_skinny(m):
    w, x = cfg5(m)
    ref = ko.matmul(w, x)
    dw, dx = dev(w), dev(x)
    y = DB(m * 4096 * 4)
    VMath.matmul(0, y, dw, dx, 4096, m, 4096, False)
    check(y.to_numpy((m, 4096)), ref, what="cfg5 M=%d" % m)
    # [K,N] weight layout of the same product
    wt = dev(np.ascontiguousarray(w.T))
    y2 = DB(m * 4096 * 4)
    VMath.gemm_f32(0, 0, 0, m, 4096, 4096, dx, 4096, wt, 4096, y2, 4096, None, kai.ACT["none"], None, False)
    check(y2.to_numpy((m, 4096)), ref, what="cfg5 M=%d [K,N] layout" % m)


def test_cfg5_ragged():
    m, k, n = 1000, 777, 333
    w, x = cfg5(m, k, n)
    gy = (0.01 * np.random.default_rng(55).standard_normal((m, n))).astype(np.float32)
    dw, dx, dgy = dev(w), dev(x), dev(gy)
    y, gx, gw = DB(m * n * 4), DB(m * k * 4), DB(n * k * 4)
    VMath.matmul(0, y, dw, dx, n, m, k, False)
    VMath.matmul_backward_x(0, gx, dgy, dw, n, m, k, False)
    VMath.matmul_backward_w(0, gw, dgy, dx, n, m, k, False)
    check(y.to_numpy((m, n)), ko.matmul(w, x), what="ragged Y")
    check(gx.to_numpy((m, k)), ko.matmul_backward_x(gy, w), what="ragged dX")
    check(gw.to_numpy((n, k)), ko.matmul_backward_w(gy, x, n, k), what="ragged dW")


# ---- shapes around the tile edges, every operand form, acc, unaligned pointers ---------------------------------

SHAPES = [(1, 1, 1), (3, 5, 7), (17, 33, 9), (64, 64, 64), (65, 63, 66), (100, 300, 50), (128, 128, 32),
          (129, 257, 40), (256, 256, 16), (300, 520, 128), (31, 1000, 4), (513, 64, 260), (40, 24, 1000),
          # split along K (few output tiles, long reduction), with and without whole tiles
          (64, 64, 1024), (100, 300, 4096), (256, 512, 2048), (20, 130, 4000), (20, 130, 4100), (3, 5, 1000),
          # 128-wide tiles: pipelined whole-tile kernel, then its edge variant
          (1024, 2048, 256), (1000, 2000, 130),
          # 256-wide tiles with edges in every dimension
          (1500, 3000, 100),
          # at most 32 rows against many columns, too long for the one-launch kernel: the 32 x 128 tile, whole and ragged
          (32, 2048, 2304), (20, 1030, 2100),
          # short reductions: the tiled kernel below 4M outputs, the panel-resident kernel (K-contiguous form)
          # above: odd K, ragged rows and columns
          (200, 130, 61), (513, 700, 64), (64, 1000, 8), (2050, 2100, 61), (2048, 2048, 64), (4100, 1030, 24),
          # tile and number of parts from the cost model: the pipelined 64 x 64, 64 x 128 and 128 x 128 tiles, whole and
          # with edges, the reduction in equal parts and in parts with a shorter last one
          (300, 200, 5003), (130, 260, 3001), (192, 384, 2048), (100, 1000, 4100), (640, 512, 1024), (333, 444, 2222),
          (64, 128, 31), (65, 129, 33), (500, 1000, 1000)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_all_operand_forms(m, n, k):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    bt = np.ascontiguousarray(b.T)
    at = np.ascontiguousarray(a.T)
    ref = ko.matmul(bt, a)                       # a . b
    ref_acc = ko.matmul(bt, a, acc_into=c0)
    ref_full = ko.activate(ko.add_bias(ref_acc, bias), "leaky", 0.1)
    da, dat, dbm, dbt, dbias = dev(a), dev(at), dev(b), dev(bt), dev(bias)
    alpha = kai.hyper(0.1)
    for ta, tb, A, lda, B, ldb in [(0, 1, da, k, dbt, k), (0, 0, da, k, dbm, n), (1, 0, dat, m, dbm, n),
                                   (1, 1, dat, m, dbt, k)]:
        c = DB(m * n * 4)
        VMath.gemm_f32(0, ta, tb, m, n, k, A, lda, B, ldb, c, n, None, 0, None, False)
        check(c.to_numpy((m, n)), ref, what="gemm form (%d,%d) %dx%dx%d" % (ta, tb, m, n, k))
        c = dev(c0)
        VMath.gemm_f32(0, ta, tb, m, n, k, A, lda, B, ldb, c, n, dbias, kai.ACT["leaky"], alpha, True)
        check(c.to_numpy((m, n)), ref_full, what="gemm form (%d,%d) acc+bias+leaky" % (ta, tb))


def test_engine_calls_with_acc_and_unaligned_subbuffers():
    # the RNN driver passes base + t*size pointers and acc = true (vtensor.cpp:2462-2474)
    rng = np.random.default_rng(7)
    ndat, xvec, yvec = 37, 53, 29
    x = rng.standard_normal((ndat, xvec)).astype(np.float32)
    w = rng.standard_normal((yvec, xvec)).astype(np.float32)
    y0 = rng.standard_normal((ndat, yvec)).astype(np.float32)
    pad = 3   # floats: shifts every pointer off 16-byte alignment
    bx = dev(np.concatenate([np.zeros(pad, np.float32), x.ravel()]))
    bw = dev(np.concatenate([np.zeros(pad, np.float32), w.ravel()]))
    by = dev(np.concatenate([np.zeros(pad, np.float32), y0.ravel()]))
    VMath.matmul(0, by.offset(4 * pad), bw.offset(4 * pad), bx.offset(4 * pad), yvec, ndat, xvec, True)
    got = by.to_numpy((pad + ndat * yvec,))[pad:].reshape(ndat, yvec)
    check(got, ko.matmul(w, x, acc_into=y0), what="acc + unaligned matmul")
    gy = rng.standard_normal((ndat, yvec)).astype(np.float32)
    bgy = dev(np.concatenate([np.zeros(pad, np.float32), gy.ravel()]))
    gx0 = rng.standard_normal((ndat, xvec)).astype(np.float32)
    gw0 = rng.standard_normal((yvec, xvec)).astype(np.float32)
    bgx = dev(np.concatenate([np.zeros(pad, np.float32), gx0.ravel()]))
    bgw = dev(np.concatenate([np.zeros(pad, np.float32), gw0.ravel()]))
    VMath.matmul_backward_x(0, bgx.offset(4 * pad), bgy.offset(4 * pad), bw.offset(4 * pad), yvec, ndat, xvec, True)
    VMath.matmul_backward_w(0, bgw.offset(4 * pad), bgy.offset(4 * pad), bx.offset(4 * pad), yvec, ndat, xvec, True)
    check(bgx.to_numpy((pad + ndat * xvec,))[pad:].reshape(ndat, xvec), ko.matmul_backward_x(gy, w, acc_into=gx0),
          what="acc + unaligned backward_x")
    check(bgw.to_numpy((pad + yvec * xvec,))[pad:].reshape(yvec, xvec),
          ko.matmul_backward_w(gy, x, yvec, xvec, acc_into=gw0), what="acc + unaligned backward_w")


@pytest.mark.parametrize("m,k,n", [(1, 4096, 4096), (2, 1000, 300), (7, 130, 1024), (16, 4100, 257), (16, 3, 5),
                                   (5, 8192, 256), (9, 68, 300), (13, 1028, 1000), (3, 4096, 1024), (4, 260, 256),
                                   (1, 5000, 300), (2, 4100, 513), (1, 12292, 300), (1, 8192, 1030),
                                   # batch 1 at K = 4096 (the straight-line kernel) with rows that do not fill the last wave
                                   (1, 4096, 1027), (1, 4096, 257),
                                   # 2..4 rows with X shared through LDS: K in (3072, 4096], N >= 1024
                                   (3, 3080, 1030), (2, 4096, 1024), (4, 3588, 2050),
                                   # rows a multiple of 32 KiB apart: every wave starts at a place of its own in its
                                   # rows / slices and wraps round
                                   (16, 8192, 512), (12, 16384, 272), (1, 16384, 260), (2, 8192, 4112), (1, 24576, 130),
                                   # 17..32 rows on the streaming kernel: two blocks of 16 rows of X per tile of W
                                   (17, 4096, 4096), (24, 8192, 4112), (25, 4096, 4096), (32, 4096, 4096),
                                   # workgroups of 8 rows of W where those of 16 would not cover the compute units
                                   (8, 4096, 2048), (16, 8192, 1024), (3, 4096, 1544), (2, 4096, 2048), (9, 12288, 1032),
                                   # workgroups of 48 and 32 rows of W where they fill the compute units (the last one
                                   # of 11008 and of 7184 owns 16 rows)
                                   (32, 4096, 11008), (16, 4096, 11008), (9, 4096, 12288), (24, 4096, 7184), (17, 4096, 6144),
                                   # 33..64 rows: three and four blocks of X rows
                                   (48, 4096, 8192), (64, 4096, 11008), (33, 4096, 6160),
                                   # rows of 8192 steps against a 256 MB matrix, and two rounds of 32-row workgroups
                                   (12, 8192, 8192), (40, 8192, 8192), (25, 4096, 16384),
                                   # 2..4 rows against 9..15 rows of W per compute unit: the streaming kernel, except
                                   # the rolled loop over long rows (the slice kernel keeps 3072 x 11008)
                                   (3, 4096, 2304), (4, 5120, 3072), (4, 12288, 3840), (2, 8192, 2560), (3, 2048, 2048),
                                   (4, 1024, 2320), (4, 11008, 3072), (2, 12288, 3072),
                                   # one row with K not in whole chunks of 4096: the slice kernel, short rows the
                                   # streaming kernel
                                   (1, 2048, 5120), (1, 11008, 4096), (1, 512, 2048), (1, 1024, 1024), (1, 1024, 4100),
                                   (1, 3072, 1031), (1, 260, 300), (1, 5124, 4096),
                                   # 17..32 rows through the rolled loop (K in whole tiles, not in whole slices), and
                                   # K = 4096 against 9..15 rows of W per compute unit
                                   (17, 2048, 4096), (32, 1024, 3072), (24, 3072, 4096), (25, 4096, 3072), (17, 4096, 2304),
                                   (32, 2048, 11008), (20, 1056, 2320), (8, 2080, 4096), (5, 11008, 4096),
                                   # a last round of 16-row workgroups that is mostly empty: one round of wider ones
                                   (5, 4096, 4352), (16, 4096, 8704), (4, 8192, 5120), (24, 4096, 12800), (3, 4096, 8448),
                                   (2, 4096, 4352), (12, 11008, 1024), (5, 13824, 256),
                                   # widths that are not a multiple of the workgroup's rows of W: whole tiles all the same
                                   (8, 4096, 4100), (16, 2048, 5003), (24, 4096, 4100), (32, 4096, 11001), (3, 4096, 4099),
                                   (12, 4096, 8707), (5, 1024, 4353),
                                   # K a multiple of 4 but not of 32: whole-tile loads, the last tile's lanes past K read zeros
                                   (8, 4100, 4096), (16, 5004, 4100), (24, 2052, 4096), (32, 1028, 3000), (3, 4100, 4352),
                                   (12, 1060, 4099), (5, 68, 4096),
                                   # many short rows (a vocabulary against a narrow model): slices up to 4 rows, tiles beyond
                                   (1, 768, 30522), (4, 768, 30522), (8, 768, 30522), (16, 1280, 20000)])
def test_skinny_shapes_bias_act_acc(m, k, n):
    if n % 16 != 0:
        pass
    elif n >= 6144 and k % 4096 == 0:
        want = "skinny stream %d" % (48 if n in (11008, 12288, 8704, 8448) else 32)
        assert VMath.gemm_plan(0, 1, m, n, k) == want
    elif n in (4352, 5120) and m >= 2 and k % 4096 == 0:
        assert VMath.gemm_plan(0, 1, m, n, k) == "skinny stream 32"
    elif m > 16 and k % 4096 != 0 and k % 32 == 0:
        assert VMath.gemm_plan(0, 1, m, n, k) == "skinny"      # 16-row workgroups, rolled loop
    rng = np.random.default_rng(m + k + n)
    w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    y0 = rng.standard_normal((m, n)).astype(np.float32)
    dw, dx, db = dev(w), dev(x), dev(b)
    y, pre = DB(m * n * 4), DB(m * n * 4)
    VMath.dense_forward(0, y, pre, dw, db, dx, n, m, k, kai.ACT["relu"], None)
    ref_pre = ko.add_bias(ko.matmul(w, x), b)
    check(pre.to_numpy((m, n)), ref_pre, what="skinny pre")
    check(y.to_numpy((m, n)), ko.activate(ref_pre, "relu"), what="skinny relu")
    ya = dev(y0)
    VMath.matmul(0, ya, dw, dx, n, m, k, True)
    check(ya.to_numpy((m, n)), ko.matmul(w, x, acc_into=y0), what="skinny acc")


@pytest.mark.parametrize("m,k,n,padw,padx", [(1, 4095, 4096, 0, 0), (1, 4097, 1000, 0, 0), (4, 4098, 300, 0, 0), (16, 4095, 1030, 0, 0),
                                            (8, 1001, 513, 0, 0), (3, 769, 5000, 0, 0), (16, 37, 256, 0, 0), (5, 4096, 700, 3, 0),
                                            (5, 4096, 700, 0, 1), (2, 999, 999, 5, 7), (13, 130, 2000, 1, 2), (1, 5, 256, 0, 0)])
def test_few_rows_rows_off_16_byte_lines(m, k, n, padw, padx):
    """Rows of W or X that do not start on 16-byte lines (K or a leading dimension not a multiple of 4): 128-bit buffer
    loads at 4-byte alignment.  The last rows end with the buffers, NaN lies between the rows."""
    rng = np.random.default_rng(m * 7 + k + n)
    w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    wp = np.full(n * (k + padw) - padw, np.nan, np.float32)       # the last row is not padded: the buffer ends with it
    xp = np.full(m * (k + padx) - padx, np.nan, np.float32)
    for r in range(n):
        wp[r * (k + padw): r * (k + padw) + k] = w[r]
    for r in range(m):
        xp[r * (k + padx): r * (k + padx) + k] = x[r]
    b = rng.standard_normal(n).astype(np.float32)
    y0 = rng.standard_normal((m, n)).astype(np.float32)
    for acc in (0, 1):
        dy = dev(y0)
        VMath.gemm_f32(0, 0, 1, m, n, k, dev(xp), k + padx, dev(wp), k + padw, dy, n, dev(b), kai.ACT["tanh"], None, acc)
        ref = ko.activate(ko.add_bias(ko.matmul(w, x, acc_into=y0 if acc else None), b), "tanh")
        got = dy.to_numpy((m, n))
        assert np.isfinite(got).all()
        check(got, ref, what="rows off 16-byte lines, acc=%d, plan %s" % (acc, VMath.gemm_plan(0, 1, m, n, k, k + padx, k + padw, n)))


@pytest.mark.parametrize("seed", list(range(1, 13)))
def test_few_rows_random_shapes(seed):
    """1..33 rows against weight matrices of random width, length and row padding (multiples of 4, on and off the
    streaming kernels' tile grid and the 128-byte lines), with and without accumulation: whatever kernel the
    dispatcher's rules pick must give the oracle's product."""
    rng = np.random.default_rng(1000 + seed)
    for _ in range(10):
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 13, 16, 17, 24, 33]))
        k = int(rng.choice([68, 768, 1028, 2048, 2052, 4096, 4100, 5004])) if rng.integers(0, 2) else 4 * int(rng.integers(16, 1500))
        n = int(rng.choice([256, 1000, 2304, 4099, 4352, 5120])) if rng.integers(0, 2) else int(rng.integers(256, 6000))
        n = min(n, max(256, int(6e6 // k)))
        padw = int(rng.choice([0, 4, 32]))
        w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
        wp = np.full((n, k + padw), np.nan, np.float32); wp[:, :k] = w
        x = rng.standard_normal((m, k)).astype(np.float32)
        y0 = rng.standard_normal((m, n)).astype(np.float32)
        acc = int(rng.integers(0, 2))
        dwp, dx, dy = dev(wp), dev(x), dev(y0)
        plan = VMath.gemm_plan(0, 1, m, n, k, k, k + padw, n)
        VMath.gemm_f32(0, 0, 1, m, n, k, dx, k, dwp, k + padw, dy, n, None, 0, None, acc)
        check(dy.to_numpy((m, n)), ko.matmul(w, x, acc_into=y0 if acc else None),
              what="%d x %d x %d, rows of W %d floats apart, acc %d (%s)" % (m, n, k, k + padw, acc, plan))


@pytest.mark.parametrize("rows", [32, 48])
def test_skinny_stream_with_wide_workgroups_forced(rows):
    # every variant of the streaming kernel with 32 / 48 rows of W per workgroup (one or two loads of X per tile, one
    # or two blocks of X rows), on a matrix whose last workgroup owns fewer blocks, with padded rows, bias,
    # activation and acc; the override is the audit hook, the dispatcher's own rule is asserted elsewhere
    rng = np.random.default_rng(rows)
    n, k, padw, padx = 4112, 4096, 32, 8    # (rows of W on 128-byte lines: off them 13 and more rows run on the tiles)
    w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
    wp = np.full((n, k + padw), np.nan, np.float32); wp[:, :k] = w
    bias = rng.standard_normal(n).astype(np.float32)
    dwp, dbias = dev(wp), dev(bias)
    try:
        VMath.gemm_force_plan("stream %d" % rows)
        for m in (2, 8, 9, 16, 17, 24, 25, 32, 33, 40, 47, 48, 49, 56, 64):
            assert VMath.gemm_plan(0, 1, m, n, k, k + padx, k + padw, n) == "skinny stream %d" % rows
            x = rng.standard_normal((m, k)).astype(np.float32)
            xp = np.full((m, k + padx), np.nan, np.float32); xp[:, :k] = x
            y0 = rng.standard_normal((m, n)).astype(np.float32)
            acc, act = bool(m % 2), ("tanh" if m % 3 == 0 else "relu")
            y = dev(y0)
            VMath.gemm_f32(0, 0, 1, m, n, k, dev(xp), k + padx, dwp, k + padw, y, n, dbias, kai.ACT[act], None, acc)
            ref = ko.activate(ko.add_bias(ko.matmul(w, x, acc_into=y0 if acc else None), bias), act)
            got = y.to_numpy((m, n))
            assert np.isfinite(got).all(), m
            check(got, ref, what="%d rows of X, workgroups of %d rows of W" % (m, rows))
    finally:
        VMath.gemm_force_plan("auto")


@pytest.mark.parametrize("m,k,n", [(1, 4096, 4096), (4, 2500, 4100), (5, 2100, 1500), (9, 9000, 1024), (16, 3000, 1028),
                                   (13, 4096, 2048), (2, 8200, 1100)])
def test_skinny_products_against_a_row_major_k_by_n_matrix(m, k, n):
    # at most 16 rows against b[K, N]: matmul_backward_x at small batches (reduction over yvec = k here) and the
    # forward product in the transposed weight layout; K beyond one LDS chunk per part, ragged column slices
    rng = np.random.default_rng(m * 31 + k + n)
    gy = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.uniform(-0.05, 0.05, (k, n)).astype(np.float32)        # the engine's w[yvec, xvec]
    gx0 = rng.standard_normal((m, n)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    dgy, dw = dev(gy), dev(w)
    gx = DB(m * n * 4)
    VMath.matmul_backward_x(0, gx, dgy, dw, k, m, n, False)
    check(gx.to_numpy((m, n)), ko.matmul_backward_x(gy, w), what="backward_x")
    gxa = dev(gx0)
    VMath.matmul_backward_x(0, gxa, dgy, dw, k, m, n, True)
    check(gxa.to_numpy((m, n)), ko.matmul_backward_x(gy, w, acc_into=gx0), what="backward_x acc")
    y = dev(gx0)
    VMath.gemm_f32(0, 0, 0, m, n, k, dgy, k, dw, n, y, n, dev(b), kai.ACT["leaky"], kai.hyper(0.1), True)
    ref = ko.activate(ko.add_bias(ko.matmul_backward_x(gy, w, acc_into=gx0), b), "leaky", 0.1)
    check(y.to_numpy((m, n)), ref, what="[K,N] layout, acc + bias + leaky")
    # leading dimensions beyond the row lengths and operands that start 4 bytes past a 16-byte boundary
    lda, ldb, ldc = k + 3, n + 5, n + 2
    ap = np.full((m, lda), np.nan, np.float32); ap[:, :k] = gy
    bp = np.full((k, ldb), np.nan, np.float32); bp[:, :n] = w
    cp0 = rng.standard_normal((m, ldc)).astype(np.float32)
    ba = dev(np.concatenate([np.zeros(1, np.float32), ap.ravel()]))
    bb = dev(np.concatenate([np.zeros(1, np.float32), bp.ravel()]))
    bc = dev(np.concatenate([np.zeros(1, np.float32), cp0.ravel()]))
    VMath.gemm_f32(0, 0, 0, m, n, k, ba.offset(4), lda, bb.offset(4), ldb, bc.offset(4), ldc, None, 0, None, False)
    got = bc.to_numpy((1 + m * ldc,))[1:].reshape(m, ldc)
    check(got[:, :n], ko.matmul_backward_x(gy, w), what="[K,N] layout, padded rows, unaligned operands")
    assert np.array_equal(got[:, n:], cp0[:, n:]), "wrote between the rows of C"


def test_empty_and_degenerate_sizes():
    d = dev(np.ones(16, np.float32))
    out = dev(np.full(16, 7.0, np.float32))
    VMath.matmul(0, out, d, d, 4, 0, 4, False)          # no rows: nothing written
    VMath.matmul(0, out, d, d, 0, 4, 4, False)
    np.testing.assert_array_equal(out.to_numpy((16,)), 7.0)
    VMath.matmul(0, out, d, d, 4, 4, 0, False)          # empty reduction: zeros
    np.testing.assert_array_equal(out.to_numpy((16,)), 0.0)
    VMath.add_bias(0, out, d, d, 0, 4)
    VMath.add_bias_backward_b(0, out, d, 0, 4, False)   # column sum over no rows: zeros
    np.testing.assert_array_equal(out.to_numpy((16,))[:4], 0.0)
    VMath.softmax_direct_on_axis(0, out, 0, 4, 1)
    VMath.activate(0, out, d, 0, 0, 1, None)


# ---- bias, activations ----------------------------------------------------------------------------------------------

@pytest.mark.parametrize("nrow,ncol", [(1, 1), (7, 13), (256, 1024), (33, 4), (1000, 333), (5000, 64),
                                       # few columns under many rows: the rows are cut into runs, two launches
                                       (100000, 12), (32768, 10), (6144, 1), (20001, 100), (8193, 2000)])
def test_add_bias_and_column_sum(nrow, ncol):
    rng = np.random.default_rng(nrow * 31 + ncol)
    a = rng.standard_normal((nrow, ncol)).astype(np.float32)
    b = rng.standard_normal(ncol).astype(np.float32)
    da, db = dev(a), dev(b)
    y = DB(nrow * ncol * 4)
    VMath.add_bias(0, y, da, db, nrow, ncol)
    np.testing.assert_array_equal(y.to_numpy((nrow, ncol)), ko.add_bias(a, b))
    VMath.add_bias(0, da, da, db, nrow, ncol)   # in place, as the attention layer calls it
    np.testing.assert_array_equal(da.to_numpy((nrow, ncol)), ko.add_bias(a, b))
    gb0 = rng.standard_normal(ncol).astype(np.float32)
    gb = dev(gb0)
    dgy = dev(a)
    VMath.add_bias_backward_b(0, gb, dgy, nrow, ncol, False)
    check(gb.to_numpy((ncol,)), ko.add_bias_backward_b(a, ncol), what="colsum")
    gb = dev(gb0)
    VMath.add_bias_backward_b(0, gb, dgy, nrow, ncol, True)
    check(gb.to_numpy((ncol,)), ko.add_bias_backward_b(a, ncol, acc_into=gb0), what="colsum acc")


ACT_NAMES = ["none", "relu", "leaky", "sigmoid", "tanh", "gelu", "selu", "mish", "swish"]


@pytest.mark.parametrize("act", ACT_NAMES)
def test_activate_and_backward(act):
    rng = np.random.default_rng(11)
    x = (3 * rng.standard_normal((37, 101))).astype(np.float32)
    x[0, :6] = [0.0, -0.0, np.inf, -np.inf, 1e-30, -1e-30]
    gy = rng.standard_normal(x.shape).astype(np.float32)
    alpha = 0.1 if act == "leaky" else None
    h = kai.hyper(alpha)
    dx, dgy = dev(x), dev(gy)
    y, gx = DB(x.nbytes), DB(x.nbytes)
    VMath.activate(0, y, dx, 37, 101, kai.ACT[act], h)
    ref = ko.activate(x, act, alpha)
    got = y.to_numpy(x.shape)
    finite = np.isfinite(ref)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(ref))
    # device expf/logf/erff differ from the host libm in the last ulp; cancellation in the
    # exp-based forms magnifies that for small outputs, hence the absolute term
    np.testing.assert_allclose(got[finite], ref[finite], rtol=1e-5, atol=1e-6)
    check(got[finite], ref[finite], what="activate " + act)
    xs = x.copy()
    xs[0, :6] = [0.0, -0.0, 50.0, -50.0, 1e-30, -1e-30]
    dxs = dev(xs)
    VMath.activate_backward(0, gx, dgy, dxs, 37, 101, kai.ACT[act], h)
    np.testing.assert_allclose(gx.to_numpy(x.shape), ko.activate_backward(gy, xs, act, alpha), rtol=1e-5, atol=1e-6)
    if act in ("none", "relu", "leaky", "sigmoid", "tanh"):
        yv = ko.activate(xs, act, alpha)
        dy = dev(yv)
        VMath.activate_backward_with_y(0, gx, dgy, dy, 37, 101, kai.ACT[act], h)
        np.testing.assert_allclose(gx.to_numpy(x.shape), ko.activate_backward_with_y(gy, yv, act, alpha), rtol=1e-5,
                                   atol=1e-6)
    # in place (vtensor.cpp:2480)
    VMath.activate(0, dx, dx, 37, 101, kai.ACT[act], h)
    np.testing.assert_array_equal(dx.to_numpy(x.shape), got)


def test_relu_special_values_and_null_leaky_alpha():
    x = np.array([[-0.0, 0.0, np.nan, np.inf, -np.inf, -1.5, 2.5, 1e-45]], np.float32)
    dx = dev(x)
    y = DB(x.nbytes)
    VMath.activate(0, y, dx, 1, 8, kai.ACT["relu"], None)
    got = y.to_numpy(x.shape)
    np.testing.assert_array_equal(got, ko.activate(x, "relu"))
    assert not np.signbit(got[0, 0]) and got[0, 2] == 0.0   # -0 -> +0, NaN -> 0
    VMath.activate(0, y, dx, 1, 8, kai.ACT["leaky"], None)   # null HYPER reads as alpha = 0
    ref = ko.activate(x, "leaky", None)
    got = y.to_numpy(x.shape)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(ref))
    np.testing.assert_array_equal(got[~np.isnan(ref)], ref[~np.isnan(ref)])


# several short rows per wave, rows in a wave's registers (up to 4096 columns, every register depth), a workgroup per row (longer rows, and few
# rows of 1024 columns and more), one element, in place (the three-pass kernel)
@pytest.mark.parametrize("nrow,ncol", [(50, 77), (3000, 10), (300, 64), (300, 65), (500, 130), (300, 300), (300, 600),
                                       (2100, 1000), (2100, 2048), (40, 1500), (300, 2049), (2100, 3000), (2060, 4096), (64, 4097), (7, 50257), (5, 1),
                                       # a workgroup's registers: every depth, and the first length beyond them
                                       (40, 4096), (33, 8192), (20, 8193), (20, 12289), (16, 16384), (9, 16385), (5, 20000), (4, 32769), (3, 60000), (2, 70000),
                                       # several short rows per wave
                                       (100001, 12), (1001, 2), (1001, 3), (999, 5), (777, 17), (501, 32), (501, 33)])
def test_softmax_activation_rows(nrow, ncol):
    rng = np.random.default_rng(5 + nrow + ncol)
    x = (4 * rng.standard_normal((nrow, ncol))).astype(np.float32)
    gy = rng.standard_normal(x.shape).astype(np.float32)
    dx, dgy = dev(x), dev(gy)
    y, gx = DB(x.nbytes), DB(x.nbytes)
    VMath.activate(0, y, dx, nrow, ncol, kai.ACT["softmax"], None)
    if ncol <= 4096 and nrow * ncol <= 1000000:
        ref = ko.activate(x, "softmax")
    else:
        # the large cases against the exact value (the oracle's row loop would take minutes, and it agrees with the
        # exact value to 1e-6 at these lengths, as the smaller cases show); beyond 4096 columns the exact value is the
        # better check anyway: the reference adds the 50257 exponentials of a row one after the other in float, which
        # alone is worth 7e-5 of the sum, while the kernel's tree of partial sums is closer to the exact value
        e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
        ref = e / e.sum(axis=1, keepdims=True)
    check(y.to_numpy(x.shape), ref, what="softmax activation")
    VMath.activate_backward(0, gx, dgy, dx, nrow, ncol, kai.ACT["softmax"], None)
    p = np.asarray(ref, np.float64)
    ref_g = p * (gy - (p * gy).sum(axis=1, keepdims=True))
    check(gx.to_numpy(x.shape), ref_g, what="softmax activation backward")
    if nrow * ncol < 100000:
        VMath.activate(0, dx, dx, nrow, ncol, kai.ACT["softmax"], None)     # in place
        check(dx.to_numpy(x.shape), ref, what="softmax activation in place")


# ---- attention ops at small sizes, masks, backward --------------------------------------------------------------------

# the last three are large enough (4M scores) for the panel-resident kernels: four heads of a (q, k) pair written
# as one word, ragged lengths, head sizes that are not multiples of 8 or of 4; one head per batch entry
@pytest.mark.parametrize("nbat,ntimes,nhead,npiece", [(2, 5, 1, 3), (3, 17, 4, 8), (1, 64, 2, 64), (2, 33, 3, 5),
                                                      (1, 130, 1, 64), (1, 7, 200, 2), (2, 100, 4, 16),
                                                      (1, 130, 8, 64), (1, 70, 4, 6), (1, 96, 12, 24),
                                                      (2, 700, 8, 24), (1, 1100, 4, 6), (3, 1200, 1, 40), (1, 608, 12, 8),
                                                      # several heads per batch entry, lengths and head sizes in whole
                                                      # 32s: the kernels that take four heads per workgroup
                                                      (2, 64, 4, 32), (1, 96, 8, 64), (3, 32, 12, 32), (4, 128, 4, 96),
                                                      # whole 128-query tiles of four heads, one workgroup per compute unit
                                                      (4, 512, 4, 64),
                                                      # rows of the scores longer than 8192 floats: the deepest
                                                      # register-resident softmax variants (12 and 16 heads)
                                                      (1, 1000, 12, 16), (1, 900, 16, 16)])
def test_attention_ops_small(nbat, ntimes, nhead, npiece):
    nvec = nhead * npiece
    rng = np.random.default_rng(nbat * 100 + ntimes * 10 + nhead)
    q = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    k = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    v = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    gy = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    coef = 1.0 / np.sqrt(npiece)
    hcoef = kai.hyper(coef)
    dq, dk, dv, dgy = dev(q), dev(k), dev(v), dev(gy)
    pshape = (nbat, ntimes, ntimes, nhead)
    p = DB(int(np.prod(pshape)) * 4)
    VMath.mult_on_heads(0, p, dk, dq, nbat, ntimes, nvec, nhead, npiece, hcoef)
    ref_s = ko.mult_on_heads(k, q, nhead, coef)
    check(p.to_numpy(pshape), ref_s, what="scores")
    VMath.set_mh_attention_mask(0, p, nbat, ntimes, nhead, True)
    ref_m = ko.set_mh_attention_mask(ref_s, True)
    np.testing.assert_array_equal(np.isinf(p.to_numpy(pshape)), np.isinf(ref_m))
    VMath.softmax_direct_on_axis(0, p, nbat * ntimes, ntimes, nhead)
    ref_p = ko.softmax_direct_on_axis(ref_m, nbat * ntimes, ntimes, nhead)
    got_p = p.to_numpy(pshape)
    check(got_p, ref_p, what="masked softmax")
    assert (got_p[np.isinf(ref_m)] == 0).all()          # masked entries are exactly 0
    o = DB(nbat * ntimes * nvec * 4)
    dp = dev(ref_p)
    VMath.mix_values(0, o, dp, dv, nbat, ntimes, nvec, nhead, npiece)
    check(o.to_numpy((nbat, ntimes, nvec)), ko.mix_values(ref_p, v, nhead), what="mix_values")
    # backward ops, fed with oracle intermediates so that each op is compared on equal inputs
    gp = DB(int(np.prod(pshape)) * 4)
    VMath.mix_values_backward_prop(0, gp, dgy, dv, nbat, ntimes, nvec, nhead, npiece)
    ref_gp = ko.mix_values_backward_prop(gy, v, nhead)
    check(gp.to_numpy(pshape), ref_gp, what="mix_values_backward_prop")
    gv = DB(nbat * ntimes * nvec * 4)
    VMath.mix_values_backward_value(0, gv, dgy, dp, nbat, ntimes, nvec, nhead, npiece)
    check(gv.to_numpy((nbat, ntimes, nvec)), ko.mix_values_backward_value(gy, ref_p, nhead),
          what="mix_values_backward_value")
    dgp = dev(ref_gp)
    VMath.softmax_direct_on_axis_backward(0, dgp, dp, nbat, ntimes, nhead, hcoef)
    ref_gs = ko.softmax_direct_on_axis_backward(ref_gp, ref_p, coef)
    check(dgp.to_numpy(pshape), ref_gs, what="softmax backward")
    VMath.set_mh_attention_mask(0, dgp, nbat, ntimes, nhead, False)
    ref_gs = ko.set_mh_attention_mask(ref_gs, False)
    dgs = dev(ref_gs)
    gk = DB(nbat * ntimes * nvec * 4)
    VMath.mult_on_heads_backward(0, gk, dgs, dq, nbat, ntimes, nvec, nhead, npiece)
    check(gk.to_numpy((nbat, ntimes, nvec)), ko.mult_on_heads_backward(ref_gs, q, nhead), what="mult_on_heads_backward")


# ---- the attention block caller: VTensor::mh_attention and its backprop (vtensor.cpp:2978-3052, 3054-3195) -------

def _oracle_mh_attention(key, query, value, W, nhead, mask, coef):
    """The 11 (12) math calls of vtensor.cpp:3026-3043 issued against the oracle."""
    nbat, ntimes, nvec = key.shape
    n = nbat * ntimes
    flat = lambda a: a.reshape(n, nvec)
    K = ko.add_bias(ko.matmul(W["Kw"], flat(key)), W["Kb"]).reshape(key.shape)
    Q = ko.add_bias(ko.matmul(W["Qw"], flat(query)), W["Qb"]).reshape(key.shape)
    V = ko.add_bias(ko.matmul(W["Vw"], flat(value)), W["Vb"]).reshape(key.shape)
    s = ko.mult_on_heads(K, Q, nhead, coef)
    if mask:
        s = ko.set_mh_attention_mask(s, True)
    probs = ko.softmax_direct_on_axis(s, n, ntimes, nhead)
    mixed = ko.mix_values(probs, V, nhead)
    y = ko.add_bias(ko.matmul(W["Ow"], flat(mixed)), W["Ob"]).reshape(key.shape)
    return y, dict(K=K, Q=Q, V=V, probs=probs, mixed=mixed)


def _oracle_mh_attention_backprop(gy, key, query, value, W, fw, nhead, mask, coef, same):
    """The 17 (18) math calls of vtensor.cpp:3142-3166 and the operand's own gradient (3168-3195)."""
    nbat, ntimes, nvec = key.shape
    n = nbat * ntimes
    flat = lambda a: a.reshape(n, nvec)
    g = {}
    g["Ob"] = ko.add_bias_backward_b(flat(gy), nvec)
    g["Ow"] = ko.matmul_backward_w(flat(gy), flat(fw["mixed"]), nvec, nvec)
    g["mixed"] = ko.matmul_backward_x(flat(gy), W["Ow"]).reshape(key.shape)
    gp = ko.mix_values_backward_prop(g["mixed"], fw["V"], nhead)
    g["V"] = ko.mix_values_backward_value(g["mixed"], fw["probs"], nhead)
    gp = ko.softmax_direct_on_axis_backward(gp, fw["probs"], coef)
    if mask:
        gp = ko.set_mh_attention_mask(gp, False)
    g["probs"] = gp
    g["K"] = ko.mult_on_heads_backward(gp, fw["Q"], nhead)
    g["Q"] = ko.mult_on_heads_backward(gp, fw["K"], nhead)
    for name, src in (("K", key), ("Q", query), ("V", value)):
        g[name + "b"] = ko.add_bias_backward_b(flat(g[name]), nvec)
        g[name + "w"] = ko.matmul_backward_w(flat(g[name]), flat(src), nvec, nvec)
    g["key"] = ko.matmul_backward_x(flat(g["K"]), W["Kw"]).reshape(key.shape)
    g["query"] = ko.matmul_backward_x(flat(g["Q"]), W["Qw"]).reshape(key.shape)
    g["value"] = ko.matmul_backward_x(flat(g["V"]), W["Vw"]).reshape(key.shape)
    gx = np.zeros_like(key)
    for name in ("key", "query", "value"):
        if name in same:
            gx = ko.add(gx, g[name])
    g["x"] = gx
    return g


@pytest.mark.parametrize("nbat,ntimes,nvec,nhead,mask,same", [
    (2, 40, 32, 4, False, ("key", "query", "value")),     # self-attention: all three gradients meet in x
    (2, 40, 32, 4, True, ("key",)),                      # masked; query and value come from other tensors
    (1, 130, 64, 1, True, ("key", "query", "value")),    # one head, ragged length
    (3, 64, 96, 8, False, ()),                           # head size 12: the per-head tiled kernels
    (2, 128, 256, 4, True, ("query", "value")),          # head size 64, four heads per workgroup kernels
    (1, 33, 20, 5, False, ("value",)),                   # unaligned rows everywhere
    (2, 200, 192, 6, True, ("key", "value")),            # head size 32, six heads, ragged length
    (1, 96, 256, 2, False, ()),                          # head size 128
])
@pytest.mark.parametrize("fused", [False, True])          # the reference's calls one by one / the one-call middles
def test_mh_attention_block_and_backprop(nbat, ntimes, nvec, nhead, mask, same, fused):
    from deep_learning_framework_amd import tensor_ops as T
    rng = np.random.default_rng(nbat * 1000 + ntimes * 10 + nvec + nhead)
    tn = T.Tensor.from_numpy
    act = lambda: rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    x = act()
    inputs = {name: (x if name in same else act()) for name in ("key", "query", "value")}
    W = {}
    for name in ("Kw", "Qw", "Vw", "Ow"):
        W[name] = (rng.standard_normal((nvec, nvec)) / np.sqrt(nvec)).astype(np.float32)
    for name in ("Kb", "Qb", "Vb", "Ob"):
        W[name] = (rng.standard_normal(nvec) * 0.1).astype(np.float32)
    gy = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    coef = float(1.0 / np.sqrt(nvec / nhead))

    want_y, fw = _oracle_mh_attention(inputs["key"], inputs["query"], inputs["value"], W, nhead, mask, coef)
    want_g = _oracle_mh_attention_backprop(gy, inputs["key"], inputs["query"], inputs["value"], W, fw, nhead, mask,
                                           coef, same)

    tx = tn(x)
    tin = {name: (tx if name in same else tn(inputs[name])) for name in ("key", "query", "value")}
    tw = {name: tn(a) for name, a in W.items()}
    y = tx.mh_attention(tin["key"], tin["query"], tin["value"], tw["Kw"], tw["Kb"], tw["Qw"], tw["Qb"], tw["Vw"],
                        tw["Vb"], tw["Ow"], tw["Ob"], nhead, mask=mask, fused=fused)
    check(y.numpy(), want_y, what="mh_attention output")
    for name in ("K", "Q", "V", "probs", "mixed"):
        check(y.saved[name].numpy(), fw[name], what="mh_attention saved " + name)
    if mask:
        upper = np.triu(np.ones((ntimes, ntimes), bool), 1)
        assert (y.saved["probs"].numpy()[:, upper] == 0).all()       # keys after the query: exactly 0
    got_g = y.mh_attention_backprop(tn(gy), fused=fused)
    if fused:
        del want_g["probs"]      # never formed by the one-call backward
    assert set(got_g) == set(want_g)
    for name in sorted(want_g):
        # gradients run through up to eight chained products: the bar of a whole layer
        check(got_g[name].numpy(), want_g[name], tol=2e-5, what="mh_attention backprop " + name)


# the backward ops at the two benchmark mappings of configuration 4 (what bench.py times is what is tested)
@pytest.mark.parametrize("nbat,nhead,nvec", [(32, 1, 64), (4, 8, 512)])
def test_cfg4_attention_backward(nbat, nhead, nvec):
    ntimes, npiece = 512, 64
    q, k, v = cfg4(nbat, ntimes, nvec)
    rng = np.random.default_rng(44)
    gy = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    coef = 1.0 / np.sqrt(npiece)
    hcoef = kai.hyper(coef)
    pshape = (nbat, ntimes, ntimes, nhead)
    ref_p = ko.softmax_direct_on_axis(ko.mult_on_heads(k, q, nhead, coef), nbat * ntimes, ntimes, nhead)
    dq, dk, dv, dgy, dp = dev(q), dev(k), dev(v), dev(gy), dev(ref_p)
    gp = DB(ref_p.nbytes)
    VMath.mix_values_backward_prop(0, gp, dgy, dv, nbat, ntimes, nvec, nhead, npiece)
    ref_gp = ko.mix_values_backward_prop(gy, v, nhead)
    check(gp.to_numpy(pshape), ref_gp, what="cfg4 mix_values_backward_prop")
    gv = DB(v.nbytes)
    VMath.mix_values_backward_value(0, gv, dgy, dp, nbat, ntimes, nvec, nhead, npiece)
    check(gv.to_numpy(v.shape), ko.mix_values_backward_value(gy, ref_p, nhead), what="cfg4 mix_values_backward_value")
    dgp = dev(ref_gp)
    VMath.softmax_direct_on_axis_backward(0, dgp, dp, nbat, ntimes, nhead, hcoef)
    ref_gs = ko.softmax_direct_on_axis_backward(ref_gp, ref_p, coef)
    check(dgp.to_numpy(pshape), ref_gs, what="cfg4 softmax backward")
    dgs = dev(ref_gs)
    for src, dsrc, name in ((q, dq, "gK"), (k, dk, "gQ")):
        g = DB(q.nbytes)
        VMath.mult_on_heads_backward(0, g, dgs, dsrc, nbat, ntimes, nvec, nhead, npiece)
        check(g.to_numpy(q.shape), ko.mult_on_heads_backward(ref_gs, src, nhead), what="cfg4 mult_on_heads_backward " + name)


# the backward middle of the block in one call (kai_attention_backward) against the oracle's chain of the six calls
# it replaces: both cfg4 mappings, the small geometries of test_attention_ops_small (most of them fall back to the
# separate kernels: head sizes that are no multiple of 16), head sizes 16 .. 128, ragged lengths, masked and not,
# with the mixed output given (row sums as one dot product) and without it (a first pass over the keys)
ATTENTION_BACKWARD_SHAPES = [(32, 512, 1, 64), (4, 512, 8, 64),
                             (2, 5, 1, 3), (3, 17, 4, 8), (1, 64, 2, 64), (2, 33, 3, 5), (1, 130, 1, 64), (1, 7, 200, 2),
                             (2, 100, 4, 16), (1, 130, 8, 64), (1, 70, 4, 6), (1, 96, 12, 24), (2, 700, 8, 24),
                             (1, 1100, 4, 6), (3, 1200, 1, 40), (1, 608, 12, 8), (2, 64, 4, 32), (1, 96, 8, 64),
                             (3, 32, 12, 32), (4, 128, 4, 96), (4, 512, 4, 64),
                             (2, 384, 12, 64), (1, 500, 16, 96), (2, 1024, 8, 128), (3, 200, 6, 32), (1, 77, 2, 16),
                             (2, 129, 3, 48), (1, 257, 2, 80), (1, 100, 1, 112), (1, 1, 1, 16), (2, 66, 1, 128)]


@pytest.mark.parametrize("nbat,ntimes,nhead,npiece", ATTENTION_BACKWARD_SHAPES)
def test_attention_backward_one_call(nbat, ntimes, nhead, npiece):
    nvec = nhead * npiece
    plan = VMath.attention_plan("backward", nbat, ntimes, nvec, nhead, npiece)
    if npiece % 16 == 0 and npiece <= 128:
        streamed = VMath.attention_plan("value_gradient", nbat, ntimes, nvec, nhead, npiece).startswith("streamed")
        assert plan == ("fused rows and value gradient in one launch" if streamed else "fused rows + value gradient")
    else:
        assert plan == "separate"
    rng = np.random.default_rng(nbat * 1000 + ntimes * 10 + nhead + npiece)
    q, k, v, gm = (rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32) for _ in range(4))
    coef = 1.0 / np.sqrt(npiece)
    hcoef = kai.hyper(coef)
    dq, dk, dv, dgm = dev(q), dev(k), dev(v), dev(gm)
    big = nbat * ntimes * ntimes * nhead >= (1 << 22)
    for masked in ((False,) if big and ntimes != 512 else (False, True)):
        s = ko.mult_on_heads(k, q, nhead, coef)
        if masked:
            s = ko.set_mh_attention_mask(s, True)
        p = ko.softmax_direct_on_axis(s, nbat * ntimes, ntimes, nhead)
        m = ko.mix_values(p, v, nhead)
        ref_gv = ko.mix_values_backward_value(gm, p, nhead)
        gs = ko.softmax_direct_on_axis_backward(ko.mix_values_backward_prop(gm, v, nhead), p, coef)
        if masked:
            gs = ko.set_mh_attention_mask(gs, False)
        ref_gk = ko.mult_on_heads_backward(gs, q, nhead)     # the key gradient is formed with Q, by the output row
        ref_gq = ko.mult_on_heads_backward(gs, k, nhead)
        dp, dm = dev(p), dev(m)
        for with_m in (True, False):
            gq, gk, gv = (dev(np.full(q.shape, np.nan, np.float32)) for _ in range(3))
            VMath.attention_backward(0, gq, gk, gv, dgm, dp, dm if with_m else None, dq, dk, dv, nbat, ntimes, nvec,
                                     nhead, npiece, hcoef, masked)
            what = " (%d x %d x %d heads of %d, masked %s, mixed output %s)" % (nbat, ntimes, nhead, npiece, masked, with_m)
            check(gq.to_numpy(q.shape), ref_gq, what="query gradient" + what)
            check(gk.to_numpy(q.shape), ref_gk, what="key gradient" + what)
            check(gv.to_numpy(q.shape), ref_gv, what="value gradient" + what)


def test_attention_backward_one_call_when_the_heads_do_not_fill_the_vector():
    # nhead * npiece < nvec: the gradients of the mixed output are compact, those of the projections are not; the
    # separate kernels take it (columns of the outputs beyond the heads are not written, as with the reference)
    nbat, ntimes, nvec, nhead, npiece = 2, 70, 80, 2, 32
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32) for _ in range(3))
    gm = rng.standard_normal((nbat, ntimes, nhead * npiece)).astype(np.float32)
    coef = 1.0 / np.sqrt(npiece)
    used = slice(0, nhead * npiece)
    qc, kc, vc = (np.ascontiguousarray(t[:, :, used]) for t in (q, k, v))
    p = ko.softmax_direct_on_axis(ko.mult_on_heads(kc, qc, nhead, coef), nbat * ntimes, ntimes, nhead)
    gs = ko.softmax_direct_on_axis_backward(ko.mix_values_backward_prop(gm, vc, nhead), p, coef)
    gq, gk, gv = (dev(np.zeros(q.shape, np.float32)) for _ in range(3))
    VMath.attention_backward(0, gq, gk, gv, dev(gm), dev(p), None, dev(q), dev(k), dev(v), nbat, ntimes, nvec, nhead,
                             npiece, kai.hyper(coef), False)
    check(gq.to_numpy(q.shape)[:, :, used], ko.mult_on_heads_backward(gs, kc, nhead), what="query gradient")
    check(gk.to_numpy(q.shape)[:, :, used], ko.mult_on_heads_backward(gs, qc, nhead), what="key gradient")
    check(gv.to_numpy(q.shape)[:, :, used], ko.mix_values_backward_value(gm, p, nhead), what="value gradient")
    assert (gq.to_numpy(q.shape)[:, :, nhead * npiece:] == 0).all()


# the value gradient on the kernel that streams P straight into the matrix cores' operand layout: every head size with
# one head per workgroup, every head size up to 64 with four, lengths that leave the last block of keys and the last
# step of four rows partly empty, a vector wider than the heads (columns beyond them stay untouched)
@pytest.mark.parametrize("nbat,ntimes,nhead,npiece,extra", [
    (2, 128, 1, 16, 0), (1, 200, 1, 32, 0), (2, 64, 1, 48, 0), (32, 512, 1, 64, 0), (1, 132, 1, 80, 0), (1, 260, 1, 96, 0),
    (1, 96, 1, 112, 0), (2, 320, 1, 128, 0), (1, 100, 1, 64, 64),
    (1, 77, 4, 16, 0), (2, 130, 8, 32, 0), (1, 97, 12, 48, 0), (4, 512, 8, 64, 0), (2, 384, 12, 64, 0), (1, 50, 4, 64, 32),
    (1, 1030, 4, 32, 0)])
def test_value_gradient_streamed(nbat, ntimes, nhead, npiece, extra):
    nvec = nhead * npiece + extra
    want = "streamed, %s per workgroup" % ("one head" if nhead == 1 else "four heads")
    assert VMath.attention_plan("value_gradient", nbat, ntimes, nvec, nhead, npiece) == want
    rng = np.random.default_rng(nbat * 1000 + ntimes + nhead + npiece)
    p = rng.random((nbat, ntimes, ntimes, nhead), dtype=np.float32)
    p /= p.sum(axis=2, keepdims=True)
    gy = rng.standard_normal((nbat, ntimes, nhead * npiece)).astype(np.float32)
    start = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    gv = dev(start)
    VMath.mix_values_backward_value(0, gv, dev(gy), dev(p), nbat, ntimes, nvec, nhead, npiece)
    got = gv.to_numpy((nbat, ntimes, nvec))
    if nbat * ntimes * ntimes * nhead * npiece <= 1 << 28:
        ref = ko.mix_values_backward_value(gy, p, nhead)
        check(got[:, :, :nhead * npiece], ref, what="value gradient")
    else:   # the large cases: the oracle on the first and the last batch entry
        for b in (0, nbat - 1):
            ref = ko.mix_values_backward_value(gy[b:b + 1], p[b:b + 1], nhead)
            check(got[b:b + 1, :, :nhead * npiece], ref, what="value gradient, batch entry %d" % b)
        f64 = np.matmul(p.astype(np.float64).transpose(0, 3, 2, 1),
                        gy.reshape(nbat, ntimes, nhead, npiece).astype(np.float64).transpose(0, 2, 1, 3))   # [b, h, k, d]
        assert rel_fro(got[:, :, :nhead * npiece], f64.transpose(0, 2, 1, 3).reshape(nbat, ntimes, -1)) <= REL_FRO_TOL
    np.testing.assert_array_equal(got[:, :, nhead * npiece:], start[:, :, nhead * npiece:])


# mix_values and mult_on_heads_backward on the same kernel with the roles of P's middle indices exchanged (head counts
# in whole fours, head sizes up to 64): lengths that leave the last block of rows and the last step of four keys partly
# empty (a key past the end must not bring the next row's values in), a vector wider than the heads
@pytest.mark.parametrize("nbat,ntimes,nhead,npiece,extra", [
    (1, 77, 4, 16, 0), (2, 130, 8, 32, 0), (1, 97, 12, 48, 0), (4, 512, 8, 64, 0), (2, 384, 12, 64, 0), (1, 50, 4, 64, 32),
    (1, 1030, 4, 32, 0), (3, 33, 16, 16, 0)])
def test_heads_products_streamed(nbat, ntimes, nhead, npiece, extra):
    nvec = nhead * npiece + extra
    assert VMath.attention_plan("mix_values", nbat, ntimes, nvec, nhead, npiece) == "streamed, four heads per workgroup"
    rng = np.random.default_rng(nbat * 1000 + ntimes + nhead + npiece)
    # no zeros, and large values right behind every row's end, so that a read past the row shows
    p = rng.standard_normal((nbat, ntimes, ntimes, nhead)).astype(np.float32) * 0.1 + 1.0
    p[:, :, 0, :] += 100.0
    v = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    used = slice(0, nhead * npiece)
    vc = np.ascontiguousarray(v[:, :, used])
    small = nbat * ntimes * ntimes * nhead * npiece <= 1 << 28
    batches = range(nbat) if small else (0, nbat - 1)
    # mix_values: Y [nbat, ntimes, nhead, npiece]
    y = DB(nbat * ntimes * nhead * npiece * 4)
    VMath.mix_values(0, y, dev(p), dev(v), nbat, ntimes, nvec, nhead, npiece)
    got = y.to_numpy((nbat, ntimes, nhead * npiece))
    for b in batches:
        check(got[b:b + 1], ko.mix_values(p[b:b + 1], vc[b:b + 1], nhead), what="mix_values, batch entry %d" % b)
    # mult_on_heads_backward: G [nbat, ntimes, nvec], columns beyond the heads untouched
    start = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    gq = dev(start)
    VMath.mult_on_heads_backward(0, gq, dev(p), dev(v), nbat, ntimes, nvec, nhead, npiece)
    got = gq.to_numpy((nbat, ntimes, nvec))
    for b in batches:
        check(got[b:b + 1, :, used], ko.mult_on_heads_backward(p[b:b + 1], vc[b:b + 1], nhead),
              what="mult_on_heads_backward, batch entry %d" % b)
    np.testing.assert_array_equal(got[:, :, nhead * npiece:], start[:, :, nhead * npiece:])
    f64 = np.matmul(p.astype(np.float64).transpose(0, 3, 1, 2),
                    vc.reshape(nbat, ntimes, nhead, npiece).astype(np.float64).transpose(0, 2, 1, 3))   # [b, h, t, d]
    assert rel_fro(got[:, :, used], f64.transpose(0, 2, 1, 3).reshape(nbat, ntimes, -1)) <= REL_FRO_TOL


# one case per kernel variant: rows in registers (1 head; 2..128 heads, short and long axis), rows through
# LDS (long axis, odd lengths), one thread per head (more than 128 heads)
SOFTMAX_AXIS_SHAPES = [(5, 1, 1), (3, 1000, 1), (4, 3000, 1), (7, 33, 3), (2, 512, 8), (3, 20, 128), (2, 9, 129),
                       (2, 5, 300), (300, 512, 1), (3, 2048, 1), (2, 2052, 1), (2, 700, 8), (1, 2000, 8),
                       (2, 1030, 2), (40, 64, 16),
                       # many rows with 4, 8, 16 or 128 heads: a whole head-interleaved row per wave
                       (1100, 33, 8), (2048, 512, 8), (1030, 100, 4), (1200, 30, 128), (1024, 1024, 4), (1500, 7, 16),
                       # one head, rows off 16-byte lines: every register depth of the buffer-access variant and its bounds
                       (37, 65, 1), (1031, 77, 1), (300, 255, 1), (300, 257, 1), (1200, 511, 1), (50, 513, 1), (20, 1001, 1),
                       (9, 2047, 1), (9, 2049, 1), (33, 63, 1), (5, 66, 1)]


# fused forward attention against the oracle's four separate steps: both cfg4 mappings, ragged lengths, the three
# fused head sizes, the causal mask, and shapes that fall back to the separate kernels (head size 24, unaligned nvec)
@pytest.mark.parametrize("nbat,ntimes,nhead,npiece,masked", [(32, 512, 1, 64, False), (4, 512, 8, 64, False),
                                                             (2, 130, 4, 32, True), (3, 77, 2, 16, False),
                                                             (1, 1000, 2, 64, True), (2, 64, 3, 64, True),
                                                             (2, 100, 2, 24, True), (1, 50, 3, 7, False),
                                                             (1, 1, 1, 16, True),
                                                             # BERT-style geometries: 12 heads of 64, heads of 96 and
                                                             # 128, lengths that are no multiple of 32, six heads
                                                             (2, 384, 12, 64, False), (1, 500, 16, 96, True),
                                                             (2, 1024, 8, 128, False), (3, 200, 6, 32, True),
                                                             (1, 70, 2, 48, False), (1, 90, 3, 80, True),
                                                             (2, 65, 1, 112, False)])
def test_attention_forward_fused(nbat, ntimes, nhead, npiece, masked):
    nvec = nhead * npiece
    # head sizes in whole 16s up to 128 run the one-launch kernel, whatever the length and the head count
    assert VMath.attention_plan("forward", nbat, ntimes, nvec, nhead, npiece) == ("fused" if npiece % 16 == 0 else "separate")
    rng = np.random.default_rng(nbat * 1000 + ntimes * 10 + nhead + npiece)
    q = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    k = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    v = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    coef = 1.0 / np.sqrt(npiece)
    s = ko.mult_on_heads(k, q, nhead, coef)
    if masked:
        s = ko.set_mh_attention_mask(s, True)
    pr = ko.softmax_direct_on_axis(s, nbat * ntimes, ntimes, nhead).reshape(nbat, ntimes, ntimes, nhead)
    ref = ko.mix_values(pr, v, nhead)
    o = DB(nbat * ntimes * nvec * 4)
    VMath.attention_forward(0, o, dev(q), dev(k), dev(v), nbat, ntimes, nvec, nhead, npiece, kai.hyper(coef), masked)
    check(o.to_numpy((nbat, ntimes, nvec)), ref, what="fused attention")


# the training form of the block in one call (kai_attention_forward_train): mixed output AND probabilities against
# the oracle's four steps; both cfg4 mappings, the three register depths (lengths up to 256 / 512 / 1024), ragged
# lengths, masked and not (masked keys must be exactly 0), and shapes that fall back to the separate kernels
@pytest.mark.parametrize("nbat,ntimes,nhead,npiece", [(32, 512, 1, 64), (4, 512, 8, 64), (2, 130, 4, 32), (3, 77, 2, 16),
                                                      (1, 1000, 2, 64), (2, 64, 3, 64), (2, 100, 2, 24), (1, 50, 3, 7),
                                                      (1, 1, 1, 16), (2, 300, 1, 32), (1, 1024, 1, 16), (1, 1030, 2, 32),
                                                      (2, 257, 1, 64), (1, 640, 4, 64), (3, 33, 5, 16),
                                                      (2, 384, 12, 64), (1, 500, 16, 96), (1, 1024, 8, 128),
                                                      (3, 200, 6, 32), (1, 300, 4, 48), (1, 100, 1, 128), (1, 512, 2, 128),
                                                      (1, 700, 2, 96), (1, 600, 1, 128),
                                                      (4, 640, 4, 64), (2, 1024, 8, 128), (16, 600, 1, 128)])
def test_attention_forward_train(nbat, ntimes, nhead, npiece):
    nvec = nhead * npiece
    plan = VMath.attention_plan("forward_train", nbat, ntimes, nvec, nhead, npiece)
    four = nhead % 4 == 0 and npiece <= 64 and not (npiece == 64 and ntimes > 512)
    # more than 512 keys, one head per workgroup and workgroups for at most half of the compute units: the three
    # separate calls are the faster ones for one head of 96 and more, several heads of 64 and more
    few = ntimes > 512 and not four and nbat * nhead * ((ntimes + 63) // 64) <= 128 and (
        (nhead == 1 and npiece >= 96) or (nhead >= 2 and npiece >= 64))
    if npiece % 16 != 0 or ntimes > 1024 or few:
        assert plan == "separate"
    elif four:
        assert plan == "fused, four heads per workgroup"
    else:
        assert plan == "fused"
    rng = np.random.default_rng(nbat * 1000 + ntimes * 10 + nhead + npiece)
    q, k, v = (rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32) for _ in range(3))
    coef = 1.0 / np.sqrt(npiece)
    dq, dk, dv = dev(q), dev(k), dev(v)
    pshape = (nbat, ntimes, ntimes, nhead)
    for masked in (False, True):
        s = ko.mult_on_heads(k, q, nhead, coef)
        if masked:
            s = ko.set_mh_attention_mask(s, True)
        pr = ko.softmax_direct_on_axis(s, nbat * ntimes, ntimes, nhead).reshape(pshape)
        ref = ko.mix_values(pr, v, nhead)
        o = dev(np.full((nbat, ntimes, nvec), np.nan, np.float32))
        pp = dev(np.full(pshape, np.nan, np.float32))
        VMath.attention_forward_train(0, o, pp, dq, dk, dv, nbat, ntimes, nvec, nhead, npiece, kai.hyper(coef), masked)
        what = " (%d x %d x %d heads of %d, masked %s)" % (nbat, ntimes, nhead, npiece, masked)
        got_p = pp.to_numpy(pshape)
        check(got_p, pr, what="probabilities" + what)
        check(o.to_numpy((nbat, ntimes, nvec)), ref, what="mixed output" + what)
        np.testing.assert_allclose(got_p.sum(axis=2), 1.0, rtol=0, atol=2e-6)
        if masked:
            upper = np.triu(np.ones((ntimes, ntimes), bool), 1)
            assert (got_p[:, upper] == 0).all()       # keys after the query: exactly 0


def test_attention_forward_when_the_heads_do_not_fill_the_vector():
    # nhead * npiece < nvec: the engine never does this, the interface allows it.  The output is the compact
    # [nbat, ntimes, nhead, npiece] of mix_values whatever the head size (the one-launch kernel steps aside).
    nbat, ntimes, nvec, nhead = 2, 70, 80, 2
    for npiece in (32, 24):
        rng = np.random.default_rng(npiece)
        q, k, v = (rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32) for _ in range(3))
        coef = 1.0 / np.sqrt(npiece)
        used = slice(0, nhead * npiece)
        # the oracle on the used part of the vectors, packed: same values, compact layout
        qc, kc, vc = (np.ascontiguousarray(t[:, :, used]) for t in (q, k, v))
        probs = ko.softmax_direct_on_axis(ko.mult_on_heads(kc, qc, nhead, coef), nbat * ntimes, ntimes, nhead)
        ref = ko.mix_values(probs, vc, nhead)
        o = DB(nbat * ntimes * nhead * npiece * 4)
        VMath.attention_forward(0, o, dev(q), dev(k), dev(v), nbat, ntimes, nvec, nhead, npiece, kai.hyper(coef), False)
        check(o.to_numpy((nbat, ntimes, nhead * npiece)), ref, what="attention, heads of %d in vectors of %d" % (npiece, nvec))


@pytest.mark.parametrize("nrow,nvec,ncol", SOFTMAX_AXIS_SHAPES)
def test_softmax_axis_layouts(nrow, nvec, ncol):
    rng = np.random.default_rng(nrow + nvec + ncol)
    s = (5 * rng.standard_normal((nrow, nvec, ncol))).astype(np.float32)
    d = dev(s)
    VMath.softmax_direct_on_axis(0, d, nrow, nvec, ncol)
    check(d.to_numpy(s.shape), ko.softmax_direct_on_axis(s, nrow, nvec, ncol), what="softmax axis")


@pytest.mark.parametrize("nbat,ntimes,nhead", [(3, 512, 1), (1, 512, 8), (2, 700, 8), (1, 2000, 4), (1, 300, 130), (3, 400, 4), (9, 130, 16),
                                               (2, 2052, 1)])
def test_softmax_axis_backward_layouts(nbat, ntimes, nhead):
    _softmax_axis_backward_case(nbat, ntimes, nhead, 0)


@pytest.mark.parametrize("nbat,ntimes,shift", [(3, 511, 0), (2, 257, 0), (40, 65, 0), (1, 1001, 0), (1, 2047, 0), (2, 77, 0),
                                               (3, 512, 1), (2, 128, 3)])
def test_softmax_axis_one_head_rows_off_16_byte_lines(nbat, ntimes, shift):
    """One head with an odd number of keys, or a tensor that does not start on a 16-byte line: forward in place and
    backward, the words behind the tensor untouched."""
    rng = np.random.default_rng(nbat + ntimes + shift)
    n = nbat * ntimes * ntimes
    buf = np.full(shift + n + 8, 7.0, np.float32)
    logits = (4 * rng.standard_normal(n)).astype(np.float32)
    buf[shift:shift + n] = logits
    d = dev(buf)
    VMath.softmax_direct_on_axis(0, d.offset(4 * shift), nbat * ntimes, ntimes, 1)
    got = d.to_numpy((shift + n + 8,))
    assert (got[:shift] == 7.0).all() and (got[shift + n:] == 7.0).all()
    check(got[shift:shift + n].reshape(nbat * ntimes, ntimes),
          ko.softmax_direct_on_axis(logits.reshape(nbat * ntimes, ntimes, 1), nbat * ntimes, ntimes, 1).reshape(nbat * ntimes, ntimes),
          what="softmax axis, one head, shift %d" % shift)
    _softmax_axis_backward_case(nbat, ntimes, 1, shift)


def _softmax_axis_backward_case(nbat, ntimes, nhead, shift):
    rng = np.random.default_rng(nbat + ntimes + nhead)
    shape = (nbat, ntimes, ntimes, nhead)
    logits = (3 * rng.standard_normal(shape)).astype(np.float32)
    probs = ko.softmax_direct_on_axis(logits, nbat * ntimes, ntimes, nhead).reshape(shape)
    gp = rng.standard_normal(shape).astype(np.float32)
    coef = 0.125
    n = gp.size
    gbuf, pbuf = np.full(shift + n + 8, 7.0, np.float32), np.full(shift + n + 8, np.nan, np.float32)
    gbuf[shift:shift + n] = gp.reshape(-1)
    pbuf[shift:shift + n] = probs.reshape(-1)
    dgp, dp, hcoef = dev(gbuf), dev(pbuf), kai.hyper(coef)
    VMath.softmax_direct_on_axis_backward(0, dgp.offset(4 * shift), dp.offset(4 * shift), nbat, ntimes, nhead, hcoef)
    got = dgp.to_numpy((shift + n + 8,))
    assert (got[:shift] == 7.0).all() and (got[shift + n:] == 7.0).all()
    check(got[shift:shift + n].reshape(shape), ko.softmax_direct_on_axis_backward(gp, probs, coef), what="softmax axis backward")


def test_split_k_scratch_survives_shutdown_and_growth():
    # a product cut along K over workgroups (reductions too long for the single-launch small-product kernel) uses
    # scratch memory of the library; an attention forward with a head size outside the fused kernel's keeps its
    # probabilities there and needs more of it (the buffer grows); then it is released and created again
    rng = np.random.default_rng(99)

    def split_k(m, n, k):
        x = rng.standard_normal((m, k)).astype(np.float32)
        w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
        y = DB(m * n * 4)
        VMath.matmul(0, y, dev(w), dev(x), n, m, k, False)
        rows = list(range(0, m, max(1, m // 64)))
        check(y.to_numpy((m, n))[rows], ko.matmul_rows(w, x, rows), what="split-K %dx%dx%d" % (m, n, k))

    def attention_with_scratch():
        nbat, T, nhead, npiece = 2, 384, 4, 24            # 2 * 384 * 384 * 4 floats = 4.5 MiB of probabilities
        q, k, v = (rng.standard_normal((nbat, T, nhead * npiece)).astype(np.float32) for _ in range(3))
        coef = 1.0 / np.sqrt(npiece)
        o = DB(nbat * T * nhead * npiece * 4)
        VMath.attention_forward(0, o, dev(q), dev(k), dev(v), nbat, T, nhead * npiece, nhead, npiece, kai.hyper(coef), False)
        probs = ko.softmax_direct_on_axis(ko.mult_on_heads(k, q, nhead, coef), nbat * T, T, nhead)
        check(o.to_numpy((nbat, T, nhead * npiece)), ko.mix_values(probs, v, nhead), what="attention through the scratch")

    kai.shutdown()
    assert kai.scratch_info() == (0, 0, 0)
    split_k(64, 64, 4096)
    split_k(256, 512, 4096)
    assert kai.scratch_info() == (4 << 20, 1, 0)          # first need: 4 MiB, enough for both products
    attention_with_scratch()                              # 4.5 MiB of probabilities: the buffer grows
    size, growths, retired = kai.scratch_info()
    assert size >= 4718592 and growths == 2 and retired == 4 << 20    # the smaller buffer is kept, not freed
    split_k(64, 128, 8192)
    assert kai.scratch_info()[1] == 2
    kai.shutdown()
    assert kai.scratch_info() == (0, 0, 0)
    split_k(64, 128, 8192)
    attention_with_scratch()
    # sizing ahead of time: afterwards nothing grows
    kai.reserve_scratch(48 << 20)
    n_growths = kai.scratch_info()[1]
    split_k(1024, 1024, 8192)
    attention_with_scratch()
    assert kai.scratch_info()[1] == n_growths and kai.scratch_info()[0] >= 48 << 20


def test_split_k_products_on_two_streams_at_once_and_retired_scratch_returns():
    # Each stream that calls are enqueued on has a scratch buffer of its own: products cut along K that run on two
    # streams of the device at the same time do not share partial sums.  Buffers that grown ones replaced go back
    # when the device is idle at kai_device_synchronize, without kai_shutdown.
    import ctypes
    kai.load()
    hip = ctypes.CDLL("libamdhip64.so.7")        # the runtime the library itself is linked to, already loaded
    hip.hipStreamCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]

    def new_stream():
        h = ctypes.c_void_p()
        assert hip.hipStreamCreateWithFlags(ctypes.byref(h), 1) == 0      # hipStreamNonBlocking
        return h.value

    rng = np.random.default_rng(123)
    kai.synchronize()
    kai.shutdown()
    s1, s2 = new_stream(), new_stream()
    shapes = {s1: (256, 512, 16384), s2: (192, 384, 12288)}
    data, outs = {}, {}
    for st, (m, n, k) in shapes.items():
        x = rng.standard_normal((m, k)).astype(np.float32)
        w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
        data[st] = (x, w, dev(x), dev(w))
        outs[st] = [DB(m * n * 4) for _ in range(6)]
        assert int(VMath.gemm_plan(0, 1, m, n, k).rsplit(" ", 1)[1]) >= 8       # many parts: a long second launch each
    kai.synchronize()
    try:
        for i in range(6):                      # alternating: the two streams' kernels overlap on the device
            for st, (m, n, k) in shapes.items():
                kai.set_stream(st)
                x, w, dx, dw = data[st]
                VMath.matmul(0, outs[st][i], dw, dx, n, m, k, False)
        sizes = {}
        for st in shapes:
            kai.set_stream(st)
            sizes[st] = kai.scratch_info()[0]
        assert all(v >= 4 << 20 for v in sizes.values())     # a buffer per stream
        # a larger product on the first stream: its buffer grows, the old one is retired, nothing waits
        kai.set_stream(s1)
        big = DB(1024 * 1024 * 4)
        xb = rng.standard_normal((1024, 8192)).astype(np.float32)
        wb = rng.uniform(-0.05, 0.05, (1024, 8192)).astype(np.float32)
        VMath.matmul(0, big, dev(wb), dev(xb), 1024, 1024, 8192, False)
        assert kai.scratch_info()[2] == sizes[s1]            # retired, not freed
    finally:
        kai.set_stream(None)
    kai.synchronize()                                        # the device is idle: the retired buffer goes back
    assert kai.scratch_info()[2] == 0
    for st, (m, n, k) in shapes.items():
        x, w, _, _ = data[st]
        rows = list(range(0, m, 16))
        ref = ko.matmul_rows(w, x, rows)
        for i in range(6):
            check(outs[st][i].to_numpy((m, n))[rows], ref, what="split-K on its own stream, call %d, %dx%dx%d" % (i, m, n, k))
    rows = list(range(0, 1024, 64))
    check(big.to_numpy((1024, 1024))[rows], ko.matmul_rows(wb, xb, rows), what="split-K after the growth")
    kai.shutdown()
    for st in (s1, s2):
        assert hip.hipStreamDestroy(st) == 0


# products cut along K whose outputs are larger than one capped element-wise grid covers (4096 workgroups x 256
# threads: 4 Mi outputs with 128-bit accesses, 1 Mi without): the pass that sums the parts covers all of them
@pytest.mark.parametrize("m,n,k,bias_act", [(1152, 4096, 4096, False), (1280, 5120, 5120, True), (1030, 1031, 8000, False), (1025, 1027, 6001, True),
                                            (1100, 1023, 3000, True)])
def test_split_k_with_a_large_output(m, n, k, bias_act):
    plan = VMath.gemm_plan(0, 1, m, n, k)
    assert int(plan.rsplit(" ", 1)[1]) > 1, plan
    rng = np.random.default_rng(m + n + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    y = DB(m * n * 4)
    VMath.fill_float(0, y, m * n, 123.0)
    if bias_act:
        VMath.dense_forward(0, y, None, dev(w), dev(b), dev(x), n, m, k, kai.ACT["relu"], None)
    else:
        VMath.matmul(0, y, dev(w), dev(x), n, m, k, False)
    got = y.to_numpy((m, n))
    # sampled rows against the oracle (first, last and a spread in between), the whole output against float64
    rows = sorted(set([0, 1, m // 2, m - 2, m - 1] + list(range(0, m, max(1, m // 24)))))
    ref_rows = ko.matmul_rows(w, x, rows)
    ref_all = x.astype(np.float64) @ w.astype(np.float64).T
    if bias_act:
        ref_rows = ko.activate(ko.add_bias(ref_rows, b), "relu")
        ref_all = np.maximum(ref_all + b, 0.0)
    check(got[rows], ref_rows, what="split-K %dx%dx%d sampled rows" % (m, n, k))
    check(got, ref_all.astype(np.float32), what="split-K %dx%dx%d whole output" % (m, n, k))


# The pipelined kernels keep one, two or four tiles on their way in registers; the loop over the tiles is
# unrolled over those sets, with whole rounds and a remainder.  One case per (tile, variant, depth) and, across
# the reduction lengths, every remainder of the tile count, with and without a masked last tile.
STAGED = [
    ((1024, 1024, 512), "small whole pipelined staged 4"), ((1024, 1024, 544), "small whole pipelined staged 4"),
    ((1024, 1024, 576), "small whole pipelined staged 4"), ((1024, 1024, 608), "small whole pipelined staged 4"),
    ((1000, 1000, 1013), "small ragged pipelined staged 4"), ((1000, 1000, 1050), "small ragged pipelined staged 4"),
    ((999, 1001, 1090), "small ragged pipelined staged 4"), ((1001, 999, 1120), "small ragged pipelined staged 4"),
    ((1024, 2048, 512), "wide whole pipelined staged 2"), ((1024, 2048, 544), "wide whole pipelined staged 2"),
    ((512, 4096, 4096), "wide whole pipelined staged 4"), ((512, 4096, 4128), "wide whole pipelined staged 4"),
    ((512, 4096, 4160), "wide whole pipelined staged 4"), ((512, 4096, 4192), "wide whole pipelined staged 4"),
    ((1000, 2000, 1111), "wide ragged pipelined staged 2"), ((1000, 2000, 1150), "wide ragged pipelined staged 2"),
    ((2048, 2048, 1024), "medium whole pipelined staged 2"), ((2048, 2048, 1056), "medium whole pipelined staged 2"),
    ((2000, 2000, 1050), "medium ragged pipelined staged 2"), ((2000, 2000, 1100), "medium ragged pipelined staged 2"),
    ((4096, 4096, 512), "large whole pipelined staged 2"), ((4096, 4096, 528), "large whole pipelined staged 2"),
    ((4000, 4000, 530), "large ragged pipelined staged 2"), ((4000, 4000, 550), "large ragged pipelined staged 2"),
    ((24, 8192, 4100), "flat ragged pipelined staged 2"), ((31, 16384, 2100), "flat ragged pipelined staged 2"),
    # several rows of 32 x 128 tiles: 129..160 rows with parts of unequal length, whole tiles in equal parts,
    # steps after the last whole tile of 32
    ((144, 4096, 4096), "flat ragged pipelined staged 2 split 3"), ((160, 2048, 2048), "flat ragged pipelined split 3"),
    ((96, 2048, 2048), "flat ragged pipelined split 4"), ((130, 3072, 2100), "flat ragged pipelined staged 2 split 2"),
    ((150, 1100, 2500), "flat ragged pipelined split 5"),
    ((200, 3072, 4096), "flat ragged pipelined staged 2 split 3"), ((224, 4608, 2304), "flat ragged pipelined staged 2 split 1"),
]


@pytest.mark.parametrize("shape,variant", STAGED, ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else v.replace(" ", "_"))
def test_staged_tiles_every_remainder(shape, variant):
    m, n, k = shape
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    bias = rng.standard_normal(n).astype(np.float32)
    sample = sorted(set([0, 1, m // 3, m - 2, m - 1] + list(range(5, m, max(1, m // 12)))))
    sample = sample[:max(3, int(1.5e8 // (n * k)))]          # keeps the oracle's scalar loops to seconds
    for ta, tb in ((0, 1), (0, 0), (1, 0)):
        assert variant in VMath.gemm_plan(ta, tb, m, n, k), VMath.gemm_plan(ta, tb, m, n, k)
        a = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
        b = rng.uniform(-0.05, 0.05, (n, k) if tb else (k, n)).astype(np.float32)
        c = DB(m * n * 4)
        VMath.fill_float(0, c, m * n, 77.0)
        VMath.gemm_f32(0, ta, tb, m, n, k, dev(a), a.shape[1], dev(b), b.shape[1], c, n, dev(bias), kai.ACT["relu"], None, False)
        got = c.to_numpy((m, n))
        a64 = (a.T if ta else a).astype(np.float64)
        b64 = (b.T if tb else b).astype(np.float64)
        ref_all = np.maximum(a64 @ b64 + bias, 0.0).astype(np.float32)
        if (ta, tb) == (0, 1):
            ref_rows = ko.matmul_rows(b, a, sample)
        elif (ta, tb) == (0, 0):
            ref_rows = ko.matmul_backward_x(np.ascontiguousarray(a[sample]), b)
        else:
            ref_rows = ko.matmul_backward_w(np.ascontiguousarray(a[:, sample]), b, len(sample), n)
        ref_rows = ko.activate(ko.add_bias(ref_rows, bias), "relu")
        what = "%dx%dx%d form %d%d" % (m, n, k, ta, tb)
        check(got[sample], ref_rows, what=what + " sampled rows")
        check(got, ref_all, what=what + " whole output")


def test_scratch_growth_does_not_wait_for_the_device():
    # Growth allocates the larger buffer and keeps the old one: no device-wide wait, no free.  Shown by
    # queueing ~0.1 s of products, then issuing a call that makes the scratch grow: it returns while the queue
    # is still busy (the wait afterwards takes most of the queued time), and its result is right.
    import time
    rng = np.random.default_rng(5)
    n = 4096
    a, b, c = dev(rng.standard_normal((n, n)).astype(np.float32)), dev(rng.standard_normal((n, n)).astype(np.float32)), DB(n * n * 4)
    m, nn, k = 1024, 1024, 4096                        # gx = gy . w, cut into parts: 8 MiB of partial sums
    plan = VMath.gemm_plan(0, 0, m, nn, k)
    assert int(plan.rsplit(" ", 1)[1]) * m * nn * 4 >= 8 << 20, plan
    gy = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.uniform(-0.05, 0.05, (k, nn)).astype(np.float32)
    dgy, dw, y = dev(gy), dev(w), DB(m * nn * 4)
    VMath.gemm_f32(0, 0, 0, n, n, n, a, n, b, n, c, n, None, 0, None, False)     # code objects loaded, clocks up
    kai.shutdown()
    kai.reserve_scratch(1 << 20)                       # the smallest buffer (4 MiB), which the product below outgrows
    before = kai.scratch_info()
    kai.synchronize()
    t0 = time.perf_counter()
    for _ in range(100):                               # ~1 ms each
        VMath.gemm_f32(0, 0, 0, n, n, n, a, n, b, n, c, n, None, 0, None, False)
    t_queued = time.perf_counter()
    VMath.matmul_backward_x(0, y, dgy, dw, k, m, nn, False)
    t_call = time.perf_counter()
    grown = kai.scratch_info()                         # host bookkeeping only: does not wait either
    kai.synchronize()
    t_done = time.perf_counter()
    after = kai.scratch_info()
    print("queueing %.1f ms, growing call %.2f ms, drain %.1f ms, scratch %s -> %s -> %s"
          % ((t_queued - t0) * 1e3, (t_call - t_queued) * 1e3, (t_done - t_call) * 1e3, before, grown, after))
    # the old buffer is only retired while the queue may still use it, and goes back once the device is idle
    assert grown[1] == before[1] + 1 and grown[0] >= 8 << 20 and grown[2] == before[0]
    assert after[:2] == grown[:2] and after[2] == 0
    rows = list(range(0, m, 32))
    check(y.to_numpy((m, nn))[rows], ko.matmul_backward_x(gy[rows], w), what="product after growth")
    if (t_done - t_call) > 0.02:                       # the queue was still busy when the call returned
        assert (t_call - t_queued) < 0.5 * (t_done - t_call)
    else:
        pytest.skip("the queued products had drained before the call: nothing to observe")


# the fallback of kai_attention_forward keeps its probabilities in the scratch while its own products cut their
# reductions into parts and need scratch, too: the partial sums must land behind the probabilities
@pytest.mark.parametrize("ntimes,npiece,masked", [(1536, 128, False), (1536, 96, True), (2048, 128, True)])
def test_attention_fallback_with_one_long_head(ntimes, npiece, masked):
    nbat = nhead = 1
    nvec = npiece
    # the product P . V of this geometry is one that cuts its reduction into parts
    assert int(VMath.gemm_plan(0, 0, ntimes, npiece, ntimes).rsplit(" ", 1)[1]) > 1
    rng = np.random.default_rng(ntimes + npiece)
    q, k, v = (rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32) for _ in range(3))
    coef = 1.0 / np.sqrt(npiece)
    s = ko.mult_on_heads(k, q, nhead, coef)
    if masked:
        s = ko.set_mh_attention_mask(s, True)
    probs = ko.softmax_direct_on_axis(s, nbat * ntimes, ntimes, nhead)
    ref = ko.mix_values(probs, v, nhead)
    kai.shutdown()                                     # start from no scratch: the inner products make it grow
    o = DB(nbat * ntimes * nvec * 4)
    VMath.attention_forward(0, o, dev(q), dev(k), dev(v), nbat, ntimes, nvec, nhead, npiece, kai.hyper(coef), masked)
    check(o.to_numpy((nbat, ntimes, nvec)), ref, what="attention fallback, one head of %d" % npiece)
    VMath.attention_forward(0, o, dev(q), dev(k), dev(v), nbat, ntimes, nvec, nhead, npiece, kai.hyper(coef), masked)
    check(o.to_numpy((nbat, ntimes, nvec)), ref, what="attention fallback again, scratch in place")


# ---- small products: the reduction cut over the waves of one workgroup ---------------------------------------

WAVE_SPLIT = [
    # M, N, K: 16 x 16 blocks (few workgroups) and 32 x 32 blocks (more of them), whole and ragged blocks, K with and
    # without a rest after the last round, K shorter than one round
    (64, 512, 784), (256, 1024, 1024), (100, 300, 1000), (17, 33, 44), (31, 77, 1001), (300, 300, 300),
    (16, 16, 2048), (50, 70, 4), (33, 17, 1), (512, 1024, 512), (192, 1000, 1000), (9, 200, 1030), (128, 512, 260),
    # rows that start at odd float addresses (128-bit loads at 4-byte alignment) and one to three k after the rounds
    (64, 512, 783), (256, 1024, 1023), (1000, 333, 777), (130, 70, 2),
    # one round of eight groups per wave (16 x 16 blocks: 1792 < K <= 2048; 32 x 32 blocks: 640 <= K <= 1024)
    (40, 100, 1901), (64, 512, 2000), (256, 512, 650),
]


@pytest.mark.parametrize("m,n,k", WAVE_SPLIT)
def test_small_products_every_form_and_epilogue(m, n, k):
    rng = np.random.default_rng(m * 7919 + n * 31 + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    bt, at = np.ascontiguousarray(b.T), np.ascontiguousarray(a.T)
    ref = ko.matmul(bt, a)
    ref_pre = ko.add_bias(ko.matmul(bt, a, acc_into=c0), bias)
    da, dat, dbm, dbt, dbias = dev(a), dev(at), dev(b), dev(bt), dev(bias)
    alpha = kai.hyper(0.1)
    for ta, tb, A, lda, B, ldb in [(0, 1, da, k, dbt, k), (0, 0, da, k, dbm, n), (1, 0, dat, m, dbm, n),
                                   (1, 1, dat, m, dbt, k)]:
        what = "form (%d,%d) %dx%dx%d" % (ta, tb, m, n, k)
        c = DB.from_numpy(np.full((m, n), np.nan, np.float32))
        VMath.gemm_f32(0, ta, tb, m, n, k, A, lda, B, ldb, c, n, None, 0, None, False)
        check(c.to_numpy((m, n)), ref, what=what)
        for act in ("leaky", "sigmoid", "gelu"):
            c = dev(c0)
            VMath.gemm_f32(0, ta, tb, m, n, k, A, lda, B, ldb, c, n, dbias, kai.ACT[act], alpha, True)
            check(c.to_numpy((m, n)), ko.activate(ref_pre, act, 0.1), what=what + " acc+bias+" + act)
    # the engine's calls, the fused forward with its pre-activation output, a padded output row
    w, x = bt, a
    y, pre = DB(m * n * 4), DB(m * n * 4)
    VMath.dense_forward(0, y, pre, dev(w), dbias, dev(x), n, m, k, kai.ACT["relu"], None)
    ref_pre2 = ko.add_bias(ko.matmul(w, x), bias)
    check(pre.to_numpy((m, n)), ref_pre2, what="pre-activation")
    check(y.to_numpy((m, n)), ko.activate(ref_pre2, "relu"), what="relu")
    gy = rng.standard_normal((m, n)).astype(np.float32)
    gx, gw = DB(m * k * 4), DB(n * k * 4)
    VMath.matmul_backward_x(0, gx, dev(gy), dev(w), n, m, k, False)
    VMath.matmul_backward_w(0, gw, dev(gy), dev(x), n, m, k, False)
    check(gx.to_numpy((m, k)), ko.matmul_backward_x(gy, w), what="backward_x")
    check(gw.to_numpy((n, k)), ko.matmul_backward_w(gy, x, n, k), what="backward_w")
    ldc = n + 5
    cp0 = rng.standard_normal((m, ldc)).astype(np.float32)
    cp = DB.from_numpy(cp0)
    VMath.gemm_f32(0, 0, 1, m, n, k, da, k, dbt, k, cp, ldc, None, 0, None, False)
    got = cp.to_numpy((m, ldc))
    check(got[:, :n], ref, what="padded output rows")
    assert np.array_equal(got[:, n:], cp0[:, n:]), "wrote between the rows of C"


# ---- operands whose tiles span 2 GiB: the flat-load fallback of the buffer-load kernels ---------------------------

def test_matmul_with_a_two_gib_tile_span():
    """64 x 64 outputs over K = 8.6M: 64 rows of either operand span 2.2 GB, more than the 31-bit lane offsets of
    the buffer-load variants, so dispatch must take the general kernel with flat loads (cut along K as usual).
    Inputs are -1 / 0 / 1: every partial sum is an integer below 2^24, so any summation order is exact and the
    comparison with float64 is bit for bit."""
    m = n = 64
    k = 8_600_064
    rng = np.random.default_rng(77)
    x = rng.integers(-1, 2, (m, k), dtype=np.int8).astype(np.float32)
    w = rng.integers(-1, 2, (n, k), dtype=np.int8).astype(np.float32)
    y = DB(m * n * 4)
    dx, dw = dev(x), dev(w)
    VMath.matmul(0, y, dw, dx, n, m, k, False)
    got = y.to_numpy((m, n))
    rows = [0, 17, 63]
    want = np.stack([w.astype(np.float64) @ x[r].astype(np.float64) for r in rows])
    np.testing.assert_array_equal(got[rows], want.astype(np.float32))
    # and the whole matrix against the oracle's own (sequential, equally exact) sums on one more row
    np.testing.assert_array_equal(got[40], ko.matmul_rows(w, x, [40])[0])


@pytest.mark.parametrize("nbat,ntimes,nhead", [(1, 1, 1), (2, 2, 1), (3, 7, 3), (2, 33, 5), (1, 130, 4), (2, 64, 12), (1, 257, 1), (4, 100, 2)])
def test_attention_mask_exact(nbat, ntimes, nhead):
    """The masked run of every row filled, nothing else touched: both fill values, a buffer that starts on a 16-byte
    line and one that does not, a guard behind the tensor."""
    rng = np.random.default_rng(nbat + ntimes + nhead)
    shape = (nbat, ntimes, ntimes, nhead)
    n = int(np.prod(shape))
    for shift in (0, 1, 3):
        for forward in (True, False):
            buf = rng.standard_normal(shift + n + 8).astype(np.float32)
            d = dev(buf)
            VMath.set_mh_attention_mask(0, d.offset(4 * shift), nbat, ntimes, nhead, forward)
            got = d.to_numpy((shift + n + 8,))
            want = buf.copy()
            want[shift:shift + n] = ko.set_mh_attention_mask(buf[shift:shift + n].reshape(shape), forward).reshape(-1)
            np.testing.assert_array_equal(got, want)


# ---- cosinesim ----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("nrow1,nrow2,ncol", [(1, 1, 1), (6, 4, 33), (64, 512, 784), (300, 70, 1000), (2048, 2048, 64), (5, 4100, 128),
                                              # up to four rows against many: one pass over the many (and just outside its conditions)
                                              (1, 100000, 256), (4, 5001, 2048), (3, 513, 4), (2, 1000, 36), (1, 600, 8192),
                                              (4, 515, 100), (1, 600, 8196), (2, 700, 30), (4, 511, 64)])
def test_cosinesim(nrow1, nrow2, ncol):
    rng = np.random.default_rng(nrow1 + ncol)
    a = rng.standard_normal((nrow1, ncol)).astype(np.float32)
    b = rng.standard_normal((nrow2, ncol)).astype(np.float32)
    if nrow2 > 2:
        b[1] = 0                                           # a zero row: 0 through the 1e-20 guard
    y = DB(nrow1 * nrow2 * 4)
    VMath.cosinesim(0, y, dev(a), dev(b), nrow1, nrow2, ncol)
    got = y.to_numpy((nrow1, nrow2))
    check(got, ko.cosinesim(a, b), what="cosinesim")
    if nrow2 > 2:
        assert (got[:, 1] == 0).all()


# ---- recurrent layers: cells and the per-time-step loop ---------------------------------------------------------

def test_recurrent_cells():
    rng = np.random.default_rng(21)
    for ndat, nrec in ((3, 5), (64, 256), (1, 1)):
        n = ndat * nrec
        a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        y = dev(a)
        VMath.add(0, y, y, dev(b), n)                       # in place, as the engine's gradient sum does
        np.testing.assert_array_equal(y.to_numpy(n), ko.add(a, b))
        c = DB(n * 4)
        VMath.copy(0, c, y, n)
        np.testing.assert_array_equal(c.to_numpy(n), a + b)
        aff = (rng.standard_normal((ndat, 4 * nrec)) * 2).astype(np.float32)
        s0 = rng.standard_normal((ndat, nrec)).astype(np.float32)
        for prev in (s0, None):
            r, st = DB(n * 4), DB(n * 4)
            VMath.lstm_process(0, r, st, None if prev is None else dev(prev), dev(aff), ndat, nrec, 7)
            want_r, want_s = ko.lstm_process(aff, prev)
            check(st.to_numpy((ndat, nrec)), want_s, what="lstm state")
            check(r.to_numpy((ndat, nrec)), want_r, what="lstm recurrent")
            # the cell's gradient (the reference's device kernel): gate-sum gradients, previous-state gradient
            gr = rng.standard_normal((ndat, nrec)).astype(np.float32)
            gs = rng.standard_normal((ndat, nrec)).astype(np.float32)
            want_gs, want_ga = ko.lstm_process_backward(gr, gs, aff, prev)
            dgr, dgs, dga = dev(gr), dev(gs), DB(aff.nbytes)
            VMath.lstm_process_backward(0, dgr, dgs, dga, None if prev is None else dev(prev), dev(aff), ndat, nrec, 7)
            check(dga.to_numpy(aff.shape), want_ga, what="lstm backward gate gradients")
            check(dgs.to_numpy(gs.shape), want_gs, what="lstm backward state gradient")
            np.testing.assert_array_equal(dgr.to_numpy(gr.shape), gr)     # the output's gradient is only read
        ai = rng.standard_normal((ndat, 3 * nrec)).astype(np.float32)
        ar = rng.standard_normal((ndat, 3 * nrec)).astype(np.float32)
        recurs = np.zeros((3, ndat, nrec), np.float32)
        recurs[0] = rng.standard_normal((ndat, nrec)).astype(np.float32)
        for nt in (0, 1):
            rbuf = dev(recurs)
            VMath.gru_process(0, rbuf.offset(nt * n * 4), dev(ai), dev(ar), nt, 3, ndat, nrec)
            check(rbuf.to_numpy(recurs.shape), ko.gru_process(recurs.copy(), ai, ar, nt), what="gru step %d" % nt)
            gh = rng.standard_normal((ndat, nrec)).astype(np.float32)
            want = ko.gru_process_backward(gh, recurs, ai, ar, nt)
            g, gai, gar, rsrc = dev(gh), DB(ai.nbytes), DB(ar.nbytes), dev(recurs)
            VMath.gru_process_backward(0, g, gai, gar, rsrc.offset(nt * n * 4), dev(ai), dev(ar), nt, 3, ndat, nrec)
            for got, ref, name in ((g.to_numpy(gh.shape), want[0], "gH"), (gai.to_numpy(ai.shape), want[1], "gai"),
                                   (gar.to_numpy(ar.shape), want[2], "gar")):
                check(got, ref, what="gru backward %s step %d" % (name, nt))


def _oracle_rnn(x, wi, wr, bi, br, cell, nrec, forward, act="tanh"):
    """The reference's per-step loop (vtensor.cpp:2455-2492) issued against the oracle."""
    ntimes, ndat, _ = x.shape
    ngates = {"rnn": 1, "lstm": 4, "gru": 3}[cell]
    recurs = np.zeros((ntimes, ndat, nrec), np.float32)
    states = np.zeros((ntimes, ndat, nrec), np.float32)
    ia = np.zeros((ntimes, ndat, ngates * nrec), np.float32)
    ra = np.zeros_like(ia) if cell == "gru" else ia
    for n in range(ntimes):
        nt = n if forward else ntimes - n - 1
        prev = nt - 1 if forward else nt + 1
        if n > 0:
            ra[nt] = ko.matmul(wr, recurs[prev])
        ia[nt] = ko.matmul(wi, x[nt], acc_into=ia[nt].copy())
        if bi is not None:
            ra[nt] = ko.add_bias(ra[nt], br)
            ia[nt] = ko.add_bias(ia[nt], bi)
        if cell == "rnn":
            recurs[nt] = ko.activate(ko.add(ko.copy(ia[nt]), ia[nt]), act)
        elif cell == "lstm":
            recurs[nt], states[nt] = ko.lstm_process(ia[nt], states[prev] if n > 0 else None)
        else:
            ko.gru_process(recurs, ia[nt], ra[nt], nt)
    return recurs, ia, ra, states


def _oracle_rnn_backprop(x, wi, wr, use_bias, cell, recurs, ia, ra, gy, gyt, forward, act="tanh", states=None,
                         use_state=False):
    """vtensor.cpp:2614-2631, 2657-2701 issued against the oracle."""
    ntimes, ndat, nrec = gyt.shape
    gx, gwi, gwr = np.zeros_like(x), np.zeros_like(wi), np.zeros_like(wr)
    gbi = np.zeros(wi.shape[0], np.float32)
    gbr = np.zeros(wi.shape[0], np.float32)
    gr = gy.copy()
    gs = np.zeros_like(gy)
    if cell == "lstm" and use_state:
        gs, gr = gy.copy(), np.zeros_like(gy)
    for n in range(ntimes):
        nt = ntimes - n - 1 if forward else n
        prev = nt - 1 if forward else nt + 1
        if cell == "lstm" and use_state:
            gs = ko.add(gs, gyt[nt])
        else:
            gr = ko.add(gr, gyt[nt])
        if cell == "rnn":
            gai = ko.activate_backward_with_y(gr, recurs[nt], act)
            gar = gai
        elif cell == "lstm":
            gs, gai = ko.lstm_process_backward(gr, gs, ia[nt], states[prev] if n < ntimes - 1 else None)
            gar = gai
        else:
            gr, gai, gar = ko.gru_process_backward(gr, recurs, ia[nt], ra[nt], nt)
        if use_bias:
            gbi = ko.add_bias_backward_b(gai, gai.shape[1], acc_into=gbi)
            gbr = ko.add_bias_backward_b(gar, gar.shape[1], acc_into=gbr)
        gwi = ko.matmul_backward_w(gai, x[nt], wi.shape[0], wi.shape[1], acc_into=gwi)
        if n < ntimes - 1:
            gwr = ko.matmul_backward_w(gar, recurs[prev], wr.shape[0], wr.shape[1], acc_into=gwr)
        gx[nt] = ko.matmul_backward_x(gai, wi)
        gr = ko.matmul_backward_x(gar, wr, acc_into=gr if cell == "gru" else None)
    return {"x": gx, "wi": gwi, "wr": gwr, "bi": gbi, "br": gbr}


@pytest.mark.parametrize("cell", ["rnn", "lstm", "gru"])
@pytest.mark.parametrize("ntimes,ndat,ninp,nrec,forward,bias", [(4, 3, 7, 5, True, True),       # sub-buffers at odd offsets
                                                                (6, 16, 64, 32, False, False),
                                                                (5, 64, 96, 128, True, True),
                                                                (3, 40, 32, 100, True, True)])       # ragged tiles
def test_rnn_layer_loop(cell, ntimes, ndat, ninp, nrec, forward, bias):
    from deep_learning_framework_amd import tensor_ops as T
    rng = np.random.default_rng(ntimes * 100 + ndat)
    ngates = {"rnn": 1, "lstm": 4, "gru": 3}[cell]
    x = rng.standard_normal((ntimes, ndat, ninp)).astype(np.float32)
    wi = (rng.standard_normal((ngates * nrec, ninp)) / np.sqrt(ninp) * 0.5).astype(np.float32)
    wr = (rng.standard_normal((ngates * nrec, nrec)) / np.sqrt(nrec) * 0.5).astype(np.float32)
    bi = (rng.standard_normal(ngates * nrec) * 0.1).astype(np.float32) if bias else None
    br = (rng.standard_normal(ngates * nrec) * 0.1).astype(np.float32) if bias else None
    recurs, ia, ra, states = _oracle_rnn(x, wi, wr, bi, br, cell, nrec, forward)
    tn = lambda a: None if a is None else T.Tensor.from_numpy(a)
    for batched, fused in ((True, True), (False, False), (True, False)):
        y, saved = T.rnn(tn(x), tn(wi), tn(wr), tn(bi), tn(br), cell, nrec, forward=forward,
                         batch_input_projection=batched, fused_step=fused)
        mode = "batched=%s fused=%s" % (batched, fused)
        check(saved["recurs"].numpy(), recurs, what="%s recurrent outputs (%s)" % (cell, mode))
        check(saved["iaffines"].numpy(), ia, what="%s gate pre-activations (%s)" % (cell, mode))
        if cell == "gru":
            check(saved["raffines"].numpy(), ra, what="gru recurrent gate sums (%s)" % mode)
        check(y.numpy(), recurs[-1 if forward else 0], what="%s output (%s)" % (cell, mode))
    if cell == "lstm":
        check(saved["states"].numpy(), states, what="lstm cell states")
    gy = rng.standard_normal((ndat, nrec)).astype(np.float32)
    gyt = (rng.standard_normal((ntimes, ndat, nrec)) * 0.5).astype(np.float32)
    for use_state in ((False, True) if cell == "lstm" else (False,)):
        want = _oracle_rnn_backprop(x, wi, wr, bias, cell, recurs, ia, ra, gy, gyt, forward, states=states,
                                    use_state=use_state)
        got = T.rnn_backprop(saved, tn(gy), tn(gyt), use_state=use_state)
        for name in got:
            check(got[name].numpy(), want[name], tol=2e-5,
                  what="%s backprop %s (use_state=%s)" % (cell, name, use_state))


# ---- transposes ---------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("shape,axes", [((5,), (0,)), ((33, 70), (1, 0)), ((2, 3, 4), (2, 0, 1)), ((4, 512, 8, 64), (0, 2, 1, 3)),
                                        ((3, 1, 5, 2), (3, 2, 1, 0)), ((2, 2, 2, 2, 3, 2, 2, 5), (7, 0, 6, 1, 5, 2, 4, 3)),
                                        # the innermost axis changes: tiles through LDS, every tile shape, edges, axes of one
                                        ((1000, 777), (1, 0)), ((257, 1025), (1, 0)), ((8, 3, 50, 60), (0, 2, 3, 1)),
                                        ((8, 50, 60, 3), (0, 3, 1, 2)), ((4, 70, 5, 33), (0, 2, 3, 1)), ((3, 40, 7, 9, 2), (4, 0, 3, 1, 2)),
                                        ((2, 1, 100, 37), (3, 1, 0, 2)), ((37, 1), (1, 0)), ((1, 37), (1, 0)), ((6, 300, 10), (2, 0, 1)),
                                        ((5, 2000, 2), (2, 1, 0)), ((2, 9, 1200), (2, 0, 1)), ((2, 1200, 13), (2, 1, 0)),
                                        ((4, 64, 12, 16), (0, 2, 3, 1)), ((3, 5, 1, 1), (3, 1, 0, 2)), ((40, 6, 1), (1, 2, 0))])
def test_transpose_axes(shape, axes):
    rng = np.random.default_rng(len(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    info = DB.from_numpy(ko.transpose_axinfo(shape, axes))            # raw int32 table, as the engine holds it
    y = DB(x.size * 4)
    VMath.transpose(0, y, dev(x), info, len(shape), x.size)
    yshape = [shape[a] for a in axes]
    np.testing.assert_array_equal(y.to_numpy(yshape), ko.transpose(x, axes))
    gy = rng.standard_normal(yshape).astype(np.float32)
    gx = DB(x.size * 4)
    VMath.transpose_backward(0, gx, dev(gy), info, len(shape), x.size)
    np.testing.assert_array_equal(gx.to_numpy(shape), ko.transpose_backward(gy, shape, axes))


@pytest.mark.parametrize("nrow,ncol", [(1, 1), (32, 32), (33, 31), (5, 1000), (1000, 5), (1024, 4096)])
def test_transpose_bin(nrow, ncol):
    x = np.random.default_rng(nrow + ncol).standard_normal((ncol, nrow)).astype(np.float32)
    y = DB(x.size * 4)
    VMath.transpose_bin(0, y, dev(x), nrow, ncol)
    np.testing.assert_array_equal(y.to_numpy((nrow, ncol)), ko.transpose_bin(x, nrow, ncol))


# ---- parameter update: accumulate_grad, subtract_param_grad, apply_decay, eval_adam_delta ------------------------------

@pytest.mark.parametrize("n", [1, 7, 1024, 4099, 1 << 20])
def test_parameter_update_ops(n):
    rng = np.random.default_rng(n)
    p = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    p[:: 5] = 0.0                                  # sign(0) = 0 in the L1 term
    y = dev(p)
    VMath.accumulate_grad(0, y, dev(g), n)
    np.testing.assert_array_equal(y.to_numpy((n,)), ko.accumulate_grad(p, g))
    y = dev(p)
    VMath.subtract_param_grad(0, y, dev(g), n, kai.hyper(0.0123))
    np.testing.assert_array_equal(y.to_numpy((n,)), ko.subtract_param_grad(p, g, 0.0123))   # product rounded first
    y = dev(p)
    VMath.subtract_param_grad(0, y, dev(g), n, None)                                        # null learning rate = 0
    np.testing.assert_array_equal(y.to_numpy((n,)), p)
    for l1, l2 in ((0.01, 0.02), (None, 0.5), (0.25, None), (None, None), (-1.0, -1.0)):
        d = DB(n * 4)
        VMath.apply_decay(0, d, dev(p), dev(g), n, kai.hyper(l1), kai.hyper(l2))
        np.testing.assert_array_equal(d.to_numpy((n,)), ko.apply_decay(p, g, l1, l2))
    # Adam: four steps, state carried on the device and in the oracle side by side
    s, t, cnt = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.float32)
    ds, dt, dn, da = dev(s), dev(t), dev(cnt), DB(n * 4)
    h1, h2, he = kai.hyper(0.9), kai.hyper(0.999), kai.hyper(1e-8)
    for step in range(4):
        gs = rng.standard_normal(n).astype(np.float32)
        VMath.eval_adam_delta(0, da, dev(gs), ds, dt, dn, n, h1, h2, he)
        a, s, t, cnt = ko.eval_adam_delta(gs, s, t, cnt, 0.9, 0.999, 1e-8)
        np.testing.assert_array_equal(dn.to_numpy((n,)), cnt)
        np.testing.assert_array_equal(ds.to_numpy((n,)), s)        # the moments use only +, * (rounded as in the oracle)
        np.testing.assert_array_equal(dt.to_numpy((n,)), t)
        np.testing.assert_allclose(da.to_numpy((n,)), a, rtol=2e-6, atol=1e-7)   # powf and sqrtf of two libraries
    # step counts that differ from element to element (parts of a tensor updated at different times)
    cnt = (np.arange(n) % 3 + (np.arange(n) // 8) % 2 * 5).astype(np.float32)
    dn = dev(cnt)
    gs = rng.standard_normal(n).astype(np.float32)
    VMath.eval_adam_delta(0, da, dev(gs), ds, dt, dn, n, h1, h2, he)
    a, s, t, cnt = ko.eval_adam_delta(gs, s, t, cnt, 0.9, 0.999, 1e-8)
    np.testing.assert_array_equal(dn.to_numpy((n,)), cnt)
    np.testing.assert_array_equal(ds.to_numpy((n,)), s)
    np.testing.assert_allclose(da.to_numpy((n,)), a, rtol=2e-6, atol=1e-7)


# ---- memory helpers and errors ----------------------------------------------------------------------------------------

def test_memory_helpers():
    a = np.arange(1000, dtype=np.float32)
    d = dev(a)
    e = DB(a.nbytes)
    VMath.copy_data(0, 0, e, d, a.nbytes)
    np.testing.assert_array_equal(e.to_numpy(a.shape), a)
    VMath.set_zero(0, e, 400)
    got = e.to_numpy(a.shape)
    assert (got[:100] == 0).all() and (got[100:] == a[100:]).all()
    VMath.fill_float(0, e, 10, 2.5)
    assert (e.to_numpy(a.shape)[:10] == 2.5).all()
    VMath.fill_int(0, e, 3, 7)
    assert (e.to_numpy(a.shape, np.int32)[:3] == 7).all()
    VMath.get_slice(0, e, d.offset(400), 400)
    np.testing.assert_array_equal(e.to_numpy(a.shape)[:100], a[100:200])
    assert kai.arch_info()[0] == "gfx950" and "gfx950" in kai.arch_info()[1]


def test_errors_do_not_poison_the_stream():
    d = dev(np.ones(4, np.float32))
    with pytest.raises(kai.KaiError) as e:
        VMath.activate(0, d, d, 1, 4, 42, None)
    assert e.value.code == 8
    with pytest.raises(kai.KaiError) as e:
        VMath.matmul(-1, d, d, d, 1, 1, 1, False)
    assert e.value.code == 510
    VMath.activate(0, d, d, 1, 4, 1, None)   # the library still works afterwards
    np.testing.assert_array_equal(d.to_numpy((4,)), 1.0)
