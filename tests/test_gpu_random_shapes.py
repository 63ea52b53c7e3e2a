"""Seeded sweeps over shapes, operand forms, leading dimensions and epilogue flags: kai_gemm_f32 against the
oracle's loops (and float64 for the one form the engine never issues), and the attention entry points against
the oracle at random geometries.  The fixed cases of test_gpu_parity.py aim at kernel variants one by one; this
walks the dispatch at large."""
import numpy as np
import pytest

from util import REL_FRO_TOL, ko, rel_fro

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 96, 100, 127, 128, 129, 200, 255, 256, 257,
         300, 384, 500, 512, 513, 640, 777, 1000, 1024, 1030, 2048]


def _kai():
    from deep_learning_framework_amd import kai
    from deep_learning_framework_amd.kai import DeviceBuffer, VMath
    kai.load()
    kai.set_device(0)
    return kai, DeviceBuffer, VMath


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_gemm_f32_random_shapes(seed):
    kai, DB, VMath = _kai()
    rng = np.random.default_rng(seed)
    leaky = kai.hyper(0.1)
    for _ in range(60):
        M, N = int(rng.choice(SIZES)), int(rng.choice(SIZES))
        K = int(rng.choice(SIZES + [3000, 4096]))
        if M * N * K > 4e7:                                   # keeps the oracle's scalar loops to seconds
            K = max(1, int(4e7 // (M * N)))
        tA, tB = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        pads = [int(rng.choice([0, 0, 1, 3, 4, 8])) for _ in range(3)]
        acc, use_bias, act = int(rng.integers(0, 2)), int(rng.integers(0, 2)), int(rng.choice([0, 0, 1, 2]))
        A = rng.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
        B = rng.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
        lda, ldb, ldc = A.shape[1] + pads[0], B.shape[1] + pads[1], N + pads[2]
        Ap = np.full((A.shape[0], lda), np.nan, np.float32)      # what lies between the rows must never be read as data
        Ap[:, :A.shape[1]] = A
        Bp = np.full((B.shape[0], ldb), np.nan, np.float32)
        Bp[:, :B.shape[1]] = B
        C0 = rng.standard_normal((M, ldc)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        dC = DB.from_numpy(C0)
        VMath.gemm_f32(0, tA, tB, M, N, K, DB.from_numpy(Ap), lda, DB.from_numpy(Bp), ldb, dC, ldc,
                       DB.from_numpy(bias) if use_bias else None, act, leaky, acc)
        got = dC.to_numpy((M, ldc))
        start = np.ascontiguousarray(C0[:, :N]) if acc else None
        if (tA, tB) == (0, 1):
            ref = ko.matmul(B, A, acc_into=start)
        elif (tA, tB) == (0, 0):
            ref = ko.matmul_backward_x(A, B, acc_into=start)
        elif (tA, tB) == (1, 0):
            ref = ko.matmul_backward_w(A, B, M, N, acc_into=start)
        else:
            ref = (A.T.astype(np.float64) @ B.T.astype(np.float64) + (start if acc else 0)).astype(np.float32)
        if use_bias:
            ref = ko.add_bias(ref, bias)
        ref = ko.activate(ref, ["none", "relu", "leaky"][act], 0.1)
        what = "M=%d N=%d K=%d tA=%d tB=%d ld=%d/%d/%d acc=%d bias=%d act=%d" % (M, N, K, tA, tB, lda, ldb, ldc, acc,
                                                                                use_bias, act)
        assert np.isfinite(got[:, :N]).all(), what
        assert rel_fro(got[:, :N], ref) <= 2 * REL_FRO_TOL, what      # K up to 4096 with unit-variance inputs
        assert np.array_equal(got[:, N:], C0[:, N:]), what + ": wrote between the rows of C"


# Products big enough for the 256x256 and 128x128 tiles whose sides are no multiples of the tile: the pipelined
# kernels then read past the last row (never stored) and finish K with one masked tile.  Leading dimensions that
# are multiples of 4 keep the 128-bit loads; the cases with other ones take the element-wise variant of the same tile.
BIG_RAGGED = [
    # M, N, K, tA, tB, pads (A, B, C), acc, bias, act
    (3000, 4200, 36, 0, 1, (0, 0, 0), 0, 1, 1),     # large tile, two whole K-tiles and a rest of 4
    (3100, 4100, 8, 0, 0, (0, 0, 0), 1, 0, 0),      # large tile, K shorter than one K-tile
    (3001, 4204, 32, 1, 0, (3, 0, 0), 0, 0, 2),     # large tile, whole K-tiles, 128-bit chunks that straddle the last row
    (2900, 4400, 20, 1, 1, (0, 0, 1), 0, 1, 0),     # large tile, the form the engine never issues
    (3000, 4200, 18, 0, 1, (1, 0, 0), 0, 0, 0),     # large tile, unaligned rows of A: element-wise loads
    (1000, 3000, 200, 0, 1, (0, 0, 0), 0, 1, 1),    # medium tile, six whole K-tiles and a rest of 8
    (1001, 2999, 77, 0, 0, (3, 1, 0), 1, 1, 0),     # medium tile, K no multiple of 4 behind aligned rows
    (1500, 1300, 44, 1, 0, (0, 0, 3), 0, 0, 1),     # medium tile
    (1100, 1900, 20, 1, 1, (0, 0, 0), 0, 0, 0),     # medium tile, only the masked K-tile
]


@pytest.mark.parametrize("case", BIG_RAGGED, ids=lambda c: "%dx%dx%d-%d%d" % c[:5])
def test_gemm_f32_big_ragged_tiles(case):
    kai, DB, VMath = _kai()
    M, N, K, tA, tB, pads, acc, use_bias, act = case
    rng = np.random.default_rng(M + N + K)
    leaky = kai.hyper(0.1)
    A = rng.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
    B = rng.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
    lda, ldb, ldc = A.shape[1] + pads[0], B.shape[1] + pads[1], N + pads[2]
    Ap = np.full((A.shape[0], lda), np.nan, np.float32)
    Ap[:, :A.shape[1]] = A
    Bp = np.full((B.shape[0], ldb), np.nan, np.float32)
    Bp[:, :B.shape[1]] = B
    C0 = rng.standard_normal((M, ldc)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    dC = DB.from_numpy(C0)
    VMath.gemm_f32(0, tA, tB, M, N, K, DB.from_numpy(Ap), lda, DB.from_numpy(Bp), ldb, dC, ldc,
                   DB.from_numpy(bias) if use_bias else None, act, leaky, acc)
    got = dC.to_numpy((M, ldc))
    start = np.ascontiguousarray(C0[:, :N]) if acc else None
    if (tA, tB) == (0, 1):
        ref = ko.matmul(B, A, acc_into=start)
    elif (tA, tB) == (0, 0):
        ref = ko.matmul_backward_x(A, B, acc_into=start)
    elif (tA, tB) == (1, 0):
        ref = ko.matmul_backward_w(A, B, M, N, acc_into=start)
    else:
        ref = (A.T.astype(np.float64) @ B.T.astype(np.float64) + (start if acc else 0)).astype(np.float32)
    if use_bias:
        ref = ko.add_bias(ref, bias)
    ref = ko.activate(ref, ["none", "relu", "leaky"][act], 0.1)
    assert np.isfinite(got[:, :N]).all()
    assert rel_fro(got[:, :N], ref) <= REL_FRO_TOL
    assert np.array_equal(got[:, N:], C0[:, N:]), "wrote between the rows of C"


def test_attention_random_geometries():
    kai, DB, VMath = _kai()
    rng = np.random.default_rng(21)
    dev = lambda a: DB.from_numpy(np.ascontiguousarray(a, np.float32))
    done = 0
    while done < 24:
        nhead = int(rng.choice([1, 2, 3, 4, 8, 12]))
        npiece = int(rng.choice([4, 6, 16, 24, 32, 64, 96]))
        T = int(rng.choice([5, 32, 33, 64, 96, 100, 128, 160, 256, 300, 512]))
        nbat = int(rng.choice([1, 2, 3, 5]))
        if nbat * T * T * nhead > 4e6:
            nbat = 1
        if nbat * T * T * nhead * npiece > 2e8:
            continue
        done += 1
        nvec = nhead * npiece
        q, k, v, gy = (rng.standard_normal((nbat, T, nvec)).astype(np.float32) for _ in range(4))
        coef = 1.0 / np.sqrt(npiece)
        hc = kai.hyper(coef)
        masked = bool(rng.integers(0, 2))
        ps = (nbat, T, T, nhead)
        what = "nbat=%d T=%d nhead=%d npiece=%d masked=%s: " % (nbat, T, nhead, npiece, masked)
        p = DB(int(np.prod(ps)) * 4)
        VMath.mult_on_heads(0, p, dev(k), dev(q), nbat, T, nvec, nhead, npiece, hc)
        ref_s = ko.mult_on_heads(k, q, nhead, coef)
        assert rel_fro(p.to_numpy(ps), ref_s) <= REL_FRO_TOL, what + "scores"
        if masked:
            VMath.set_mh_attention_mask(0, p, nbat, T, nhead, True)
            ref_s = ko.set_mh_attention_mask(ref_s, True)
        VMath.softmax_direct_on_axis(0, p, nbat * T, T, nhead)
        ref_p = ko.softmax_direct_on_axis(ref_s, nbat * T, T, nhead)
        assert rel_fro(p.to_numpy(ps), ref_p) <= REL_FRO_TOL, what + "softmax"
        dp, o = dev(ref_p), DB(nbat * T * nvec * 4)
        VMath.mix_values(0, o, dp, dev(v), nbat, T, nvec, nhead, npiece)
        ref_o = ko.mix_values(ref_p, v, nhead)
        assert rel_fro(o.to_numpy((nbat, T, nvec)), ref_o) <= REL_FRO_TOL, what + "mix_values"
        VMath.attention_forward(0, o, dev(q), dev(k), dev(v), nbat, T, nvec, nhead, npiece, hc, masked)
        assert rel_fro(o.to_numpy((nbat, T, nvec)), ref_o) <= REL_FRO_TOL, what + "attention_forward"
        g = DB(nbat * T * nvec * 4)
        VMath.mix_values_backward_value(0, g, dev(gy), dp, nbat, T, nvec, nhead, npiece)
        assert rel_fro(g.to_numpy((nbat, T, nvec)), ko.mix_values_backward_value(gy, ref_p, nhead)) <= REL_FRO_TOL, what + "gV"
        gp = DB(int(np.prod(ps)) * 4)
        VMath.mix_values_backward_prop(0, gp, dev(gy), dev(v), nbat, T, nvec, nhead, npiece)
        ref_gp = ko.mix_values_backward_prop(gy, v, nhead)
        assert rel_fro(gp.to_numpy(ps), ref_gp) <= REL_FRO_TOL, what + "gP"
        VMath.mult_on_heads_backward(0, g, dev(ref_gp), dev(k), nbat, T, nvec, nhead, npiece)
        assert rel_fro(g.to_numpy((nbat, T, nvec)), ko.mult_on_heads_backward(ref_gp, k, nhead)) <= REL_FRO_TOL, what + "gQ"


@pytest.mark.parametrize("seed", [21, 22])
def test_dense_backward_random_shapes(seed):
    """kai_dense_backward over random layer sizes, activations, acc and subsets of the outputs: multiples of 64 (the
    one-launch kernel, with gx's reduction whole or cut) mixed with ragged sizes (the separate kernels)."""
    kai, DB, VMath = _kai()
    rng = np.random.default_rng(seed)
    sizes = [64, 64, 128, 192, 256, 320, 512, 576, 1024, 100, 37, 130, 1000]
    for it in range(14):
        ndat, yvec, xvec = (int(rng.choice(sizes)) for _ in range(3))
        while ndat * yvec * xvec > 6e7:                       # keeps the oracle's scalar loops to a second
            if yvec > 64:
                yvec //= 2
            elif ndat > 64:
                ndat //= 2
            else:
                xvec //= 2
        act = str(rng.choice(["none", "relu", "leaky", "relu", "sigmoid"]))
        acc = bool(rng.integers(0, 2))
        alpha = float(rng.choice([0.1, 0.3])) if act == "leaky" else None
        x = rng.standard_normal((ndat, xvec)).astype(np.float32)
        w = rng.uniform(-0.1, 0.1, (yvec, xvec)).astype(np.float32)
        pre = rng.standard_normal((ndat, yvec)).astype(np.float32)
        gy = rng.standard_normal((ndat, yvec)).astype(np.float32)
        gx0, gw0, gb0 = (rng.standard_normal(s).astype(np.float32) for s in ((ndat, xvec), (yvec, xvec), (yvec,)))
        ga = gy if act == "none" else ko.activate_backward(gy, pre, act, alpha)
        a = lambda base: dict(acc_into=base) if acc else {}
        want = {"gx": ko.matmul_backward_x(ga, w, **a(gx0)), "gw": ko.matmul_backward_w(ga, x, yvec, xvec, **a(gw0)),
                "gb": ko.add_bias_backward_b(ga, yvec, **a(gb0))}
        ask = {"gx": True, "gw": True, "gb": bool(rng.integers(0, 4))} if it % 3 else \
              {k: bool(rng.integers(0, 2)) for k in ("gx", "gw", "gb")}
        bufs = {"gx": DB.from_numpy(gx0), "gw": DB.from_numpy(gw0), "gb": DB.from_numpy(gb0)}
        work = DB(ndat * yvec * 4) if rng.integers(0, 2) else None
        VMath.dense_backward(0, bufs["gx"] if ask["gx"] else None, bufs["gw"] if ask["gw"] else None,
                             bufs["gb"] if ask["gb"] else None, work, DB.from_numpy(gy), DB.from_numpy(w), DB.from_numpy(x),
                             DB.from_numpy(pre), yvec, ndat, xvec, kai.ACT[act], kai.hyper(alpha), acc)
        what = "seed %d case %d: %dx%dx%d %s acc=%s ask=%s work=%s" % (seed, it, ndat, yvec, xvec, act, acc, ask, work is not None)
        for name, shape, start in (("gx", (ndat, xvec), gx0), ("gw", (yvec, xvec), gw0), ("gb", (yvec,), gb0)):
            got = bufs[name].to_numpy(shape)
            if ask[name]:
                assert np.isfinite(got).all(), what + " " + name
                assert rel_fro(got, want[name]) <= REL_FRO_TOL, "%s %s: %.3e" % (what, name, rel_fro(got, want[name]))
            else:
                np.testing.assert_array_equal(got, start, err_msg=what + " " + name + " must stay untouched")


def test_skinny_whole_tile_shapes_random():
    """At most 16 rows against weight matrices whose sides are whole tiles of the streaming kernel (N % 16 == 0,
    K % 32 == 0) and just beside them, with padded rows, bias, activation and acc."""
    kai, DB, VMath = _kai()
    rng = np.random.default_rng(31)
    for it in range(16):
        m = int(rng.integers(1, 17))
        n = int(rng.choice([256, 272, 1024, 4096, 4112, 1000]))
        k = int(rng.choice([64, 96, 512, 1056, 4096, 4128, 1000]))
        padw, padx = int(rng.choice([0, 0, 4, 32])), int(rng.choice([0, 0, 4]))
        w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
        x = rng.standard_normal((m, k)).astype(np.float32)
        wp = np.full((n, k + padw), np.nan, np.float32); wp[:, :k] = w
        xp = np.full((m, k + padx), np.nan, np.float32); xp[:, :k] = x
        bias = rng.standard_normal(n).astype(np.float32)
        y0 = rng.standard_normal((m, n)).astype(np.float32)
        acc, use_bias, act = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), str(rng.choice(["none", "relu", "tanh"]))
        y = DB.from_numpy(y0)
        # B stored [N, K] (transB), lda / ldb carry the padding
        VMath.gemm_f32(0, 0, 1, m, n, k, DB.from_numpy(xp), k + padx, DB.from_numpy(wp), k + padw, y, n,
                       DB.from_numpy(bias) if use_bias else None, kai.ACT[act], None, acc)
        ref = ko.matmul(w, x, acc_into=y0 if acc else None)
        if use_bias:
            ref = ko.add_bias(ref, bias)
        ref = ko.activate(ref, act)
        got = y.to_numpy((m, n))
        what = "case %d: %dx%dx%d pad %d/%d acc=%s bias=%s %s" % (it, m, n, k, padw, padx, acc, use_bias, act)
        assert np.isfinite(got).all(), what
        assert rel_fro(got, ref) <= REL_FRO_TOL, "%s: %.3e" % (what, rel_fro(got, ref))


@pytest.mark.parametrize("seed", [41, 42])
def test_transpose_random_permutations(seed):
    """Random shapes of 1 to 6 axes (axes of one position among them, short and long innermost axes on either side)
    under random permutations: every path of the general transpose kernel (128-bit words, tiles through LDS, element
    by element), forward and backward, bit for bit against the oracle."""
    kai, DB, VMath = _kai()
    rng = np.random.default_rng(seed)
    for it in range(60):
        rank = int(rng.integers(1, 7))
        shape = [int(rng.choice([1, 2, 3, 4, 5, 7, 8, 12, 16, 31, 32, 33, 64, 100, 257])) for _ in range(rank)]
        while int(np.prod(shape)) > 3_000_000:
            shape[int(np.argmax(shape))] = max(1, max(shape) // 2)
        axes = [int(a) for a in rng.permutation(rank)]
        x = rng.standard_normal(shape).astype(np.float32)
        info = DB.from_numpy(ko.transpose_axinfo(tuple(shape), tuple(axes)))
        what = "case %d: %s under %s" % (it, shape, axes)
        y = DB(x.size * 4)
        VMath.transpose(0, y, DB.from_numpy(x), info, rank, x.size)
        yshape = [shape[a] for a in axes]
        assert np.array_equal(y.to_numpy(yshape), ko.transpose(x, axes)), what
        gy = rng.standard_normal(yshape).astype(np.float32)
        gx = DB(x.size * 4)
        VMath.transpose_backward(0, gx, DB.from_numpy(gy), info, rank, x.size)
        assert np.array_equal(gx.to_numpy(shape), ko.transpose_backward(gy, tuple(shape), tuple(axes))), what + " (backward)"


@pytest.mark.parametrize("seed", [51, 52, 53])
def test_few_rows_odd_lengths_random(seed):
    """1..16 rows against matrices whose reduction length and leading dimensions are NOT multiples of 4 (rows off
    16-byte lines: 128-bit buffer loads in chunks of 4, 8 or 16 steps), NaN between the rows, the buffers ending with
    their last rows; bias, activation and accumulation at random."""
    kai, DB, VMath = _kai()
    rng = np.random.default_rng(seed)
    for it in range(24):
        m = int(rng.integers(1, 17))
        k = int(rng.choice([5, 37, 63, 65, 130, 511, 513, 769, 1001, 1027, 2049, 4095, 4097, 6001]))
        n = int(rng.choice([256, 257, 300, 1000, 1030, 2500, 4099]))
        n = min(n, max(256, int(4e6 // k)))
        padw, padx = int(rng.choice([0, 1, 2, 3, 5])), int(rng.choice([0, 1, 3]))
        w = rng.uniform(-0.05, 0.05, (n, k)).astype(np.float32)
        x = rng.standard_normal((m, k)).astype(np.float32)
        wp = np.full(n * (k + padw) - padw, np.nan, np.float32)
        xp = np.full(m * (k + padx) - padx, np.nan, np.float32)
        for r in range(n):
            wp[r * (k + padw): r * (k + padw) + k] = w[r]
        for r in range(m):
            xp[r * (k + padx): r * (k + padx) + k] = x[r]
        bias = rng.standard_normal(n).astype(np.float32)
        y0 = rng.standard_normal((m, n)).astype(np.float32)
        acc, use_bias, act = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), str(rng.choice(["none", "relu", "tanh"]))
        y = DB.from_numpy(y0)
        VMath.gemm_f32(0, 0, 1, m, n, k, DB.from_numpy(xp), k + padx, DB.from_numpy(wp), k + padw, y, n,
                       DB.from_numpy(bias) if use_bias else None, kai.ACT[act], None, acc)
        ref = ko.matmul(w, x, acc_into=y0 if acc else None)
        if use_bias:
            ref = ko.add_bias(ref, bias)
        ref = ko.activate(ref, act)
        got = y.to_numpy((m, n))
        what = "case %d: %dx%dx%d pad %d/%d acc=%s bias=%s %s" % (it, m, n, k, padw, padx, acc, use_bias, act)
        assert np.isfinite(got).all(), what
        assert rel_fro(got, ref) <= REL_FRO_TOL, "%s: %.3e" % (what, rel_fro(got, ref))
