"""The committed fixture tests/golden/matmul_path_small.npz (made by tests/golden/make_golden.py
from the pinned oracle): the oracle must still reproduce it bit for bit on the CPU, and the HIP
path must match it within the path's tolerance on the GPU."""
import os

import numpy as np
import pytest

from util import REL_FRO_TOL, ROOT, ko, rel_fro

G = np.load(os.path.join(ROOT, "tests", "golden", "matmul_path_small.npz"), allow_pickle=False)
ACTS = ["none", "relu", "leaky", "sigmoid", "tanh", "gelu", "selu", "mish", "swish"]


def test_oracle_reproduces_the_fixture_bit_for_bit():
    x, w, b, gy = G["dense_x"], G["dense_w"], G["dense_b"], G["dense_gy"]
    yvec, xvec = w.shape
    assert np.array_equal(ko.matmul(w, x), G["dense_matmul"])
    assert np.array_equal(ko.add_bias(G["dense_matmul"], b), G["dense_pre"])
    assert np.array_equal(ko.matmul_backward_x(gy, w), G["dense_gx"])
    assert np.array_equal(ko.matmul_backward_w(gy, x, yvec, xvec), G["dense_gw"])
    assert np.array_equal(ko.add_bias_backward_b(gy, yvec), G["dense_gb"])
    assert np.array_equal(ko.matmul(w, x, acc_into=G["dense_pre"]), G["dense_matmul_acc"])
    for name in ACTS + ["softmax"]:
        alpha = 0.1 if name == "leaky" else None
        assert np.array_equal(ko.activate(G["dense_pre"], name, alpha), G["act_" + name]), name
    nbat, ntimes, nhead, npiece = (int(v) for v in G["att_dims"])
    coef = float(G["att_coef"][0])
    assert np.array_equal(ko.mult_on_heads(G["att_k"], G["att_q"], nhead, coef), G["att_scores"])
    assert np.array_equal(ko.softmax_direct_on_axis(G["att_scores"], nbat * ntimes, ntimes, nhead), G["att_probs"])
    assert np.array_equal(ko.mix_values(G["att_probs"], G["att_v"], nhead), G["att_out"])
    assert np.array_equal(ko.mult_on_heads_backward(G["att_gscores"], G["att_q"], nhead), G["att_gk"])


def test_fixture_satisfies_closed_forms():
    # the frozen numbers themselves agree with float64 algebra (guards the fixture, not the oracle)
    x, w, b = (G[k].astype(np.float64) for k in ("dense_x", "dense_w", "dense_b"))
    assert rel_fro(G["dense_pre"], x @ w.T + b) < 1e-6
    assert rel_fro(G["dense_gw"], G["dense_gy"].astype(np.float64).T @ x) < 1e-6
    assert np.allclose(G["att_probs"].sum(axis=2), 1.0, atol=1e-6)
    assert (G["att_probs_masked"][np.isinf(G["att_masked"])] == 0).all()


@pytest.mark.gpu
def test_hip_path_matches_the_fixture():
    from deep_learning_framework_amd import kai
    from deep_learning_framework_amd.kai import DeviceBuffer as DB, VMath
    kai.load()
    kai.set_device(0)
    dev = lambda a: DB.from_numpy(np.ascontiguousarray(a, np.float32))
    x, w, b, gy = G["dense_x"], G["dense_w"], G["dense_b"], G["dense_gy"]
    ndat, xvec = x.shape
    yvec = w.shape[0]
    dx, dw, db, dgy = dev(x), dev(w), dev(b), dev(gy)
    y = DB(ndat * yvec * 4)
    VMath.matmul(0, y, dw, dx, yvec, ndat, xvec, False)
    assert rel_fro(y.to_numpy((ndat, yvec)), G["dense_matmul"]) <= REL_FRO_TOL
    VMath.add_bias(0, y, y, db, ndat, yvec)
    assert rel_fro(y.to_numpy((ndat, yvec)), G["dense_pre"]) <= REL_FRO_TOL
    VMath.matmul(0, y, dw, dx, yvec, ndat, xvec, True)
    assert rel_fro(y.to_numpy((ndat, yvec)), G["dense_matmul_acc"]) <= REL_FRO_TOL
    gx, gw, gb = DB(x.nbytes), DB(w.nbytes), DB(b.nbytes)
    VMath.matmul_backward_x(0, gx, dgy, dw, yvec, ndat, xvec, False)
    VMath.matmul_backward_w(0, gw, dgy, dx, yvec, ndat, xvec, False)
    VMath.add_bias_backward_b(0, gb, dgy, ndat, yvec, False)
    assert rel_fro(gx.to_numpy(x.shape), G["dense_gx"]) <= REL_FRO_TOL
    assert rel_fro(gw.to_numpy(w.shape), G["dense_gw"]) <= REL_FRO_TOL
    assert rel_fro(gb.to_numpy(b.shape), G["dense_gb"]) <= REL_FRO_TOL
    dpre = dev(G["dense_pre"])
    for name in ACTS + ["softmax"]:
        h = kai.hyper(0.1 if name == "leaky" else None)
        out = DB(ndat * yvec * 4)
        VMath.activate(0, out, dpre, ndat, yvec, kai.ACT[name], h)
        assert rel_fro(out.to_numpy((ndat, yvec)), G["act_" + name]) <= REL_FRO_TOL, name
        if name != "softmax":
            VMath.activate_backward(0, out, dgy, dpre, ndat, yvec, kai.ACT[name], h)
            assert rel_fro(out.to_numpy((ndat, yvec)), G["actbwd_" + name]) <= REL_FRO_TOL, name
        if name in ("none", "relu", "leaky", "sigmoid", "tanh"):
            dyv = dev(G["act_" + name])
            VMath.activate_backward_with_y(0, out, dgy, dyv, ndat, yvec, kai.ACT[name], h)
            assert rel_fro(out.to_numpy((ndat, yvec)), G["actbwdy_" + name]) <= REL_FRO_TOL, name
    nbat, ntimes, nhead, npiece = (int(v) for v in G["att_dims"])
    nvec = nhead * npiece
    hc = kai.hyper(float(G["att_coef"][0]))
    dq, dk, dv, dgo = dev(G["att_q"]), dev(G["att_k"]), dev(G["att_v"]), dev(G["att_go"])
    p = DB(G["att_scores"].nbytes)
    VMath.mult_on_heads(0, p, dk, dq, nbat, ntimes, nvec, nhead, npiece, hc)
    assert rel_fro(p.to_numpy(G["att_scores"].shape), G["att_scores"]) <= REL_FRO_TOL
    pm = dev(G["att_scores"])
    VMath.set_mh_attention_mask(0, pm, nbat, ntimes, nhead, True)
    assert np.array_equal(pm.to_numpy(G["att_masked"].shape), G["att_masked"])
    VMath.softmax_direct_on_axis(0, pm, nbat * ntimes, ntimes, nhead)
    assert rel_fro(pm.to_numpy(G["att_probs"].shape), G["att_probs_masked"]) <= REL_FRO_TOL
    VMath.softmax_direct_on_axis(0, p, nbat * ntimes, ntimes, nhead)
    assert rel_fro(p.to_numpy(G["att_probs"].shape), G["att_probs"]) <= REL_FRO_TOL
    dp = dev(G["att_probs"])
    o = DB(G["att_out"].nbytes)
    VMath.mix_values(0, o, dp, dv, nbat, ntimes, nvec, nhead, npiece)
    assert rel_fro(o.to_numpy(G["att_out"].shape), G["att_out"]) <= REL_FRO_TOL
    gp = DB(G["att_gprobs"].nbytes)
    VMath.mix_values_backward_prop(0, gp, dgo, dv, nbat, ntimes, nvec, nhead, npiece)
    assert rel_fro(gp.to_numpy(G["att_gprobs"].shape), G["att_gprobs"]) <= REL_FRO_TOL
    gv = DB(G["att_gv"].nbytes)
    VMath.mix_values_backward_value(0, gv, dgo, dp, nbat, ntimes, nvec, nhead, npiece)
    assert rel_fro(gv.to_numpy(G["att_gv"].shape), G["att_gv"]) <= REL_FRO_TOL
    dgp = dev(G["att_gprobs"])
    VMath.softmax_direct_on_axis_backward(0, dgp, dp, nbat, ntimes, nhead, hc)
    assert rel_fro(dgp.to_numpy(G["att_gscores"].shape), G["att_gscores"]) <= REL_FRO_TOL
    dgs = dev(G["att_gscores"])
    gk, gq = DB(G["att_gk"].nbytes), DB(G["att_gq"].nbytes)
    VMath.mult_on_heads_backward(0, gk, dgs, dq, nbat, ntimes, nvec, nhead, npiece)
    VMath.mult_on_heads_backward(0, gq, dgs, dk, nbat, ntimes, nvec, nhead, npiece)
    assert rel_fro(gk.to_numpy(G["att_gk"].shape), G["att_gk"]) <= REL_FRO_TOL
    assert rel_fro(gq.to_numpy(G["att_gq"].shape), G["att_gq"]) <= REL_FRO_TOL
