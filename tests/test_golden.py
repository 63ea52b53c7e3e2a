"""The committed fixture tests/golden/matmul_path_small.npz (made by tests/golden/make_golden.py
from the pinned oracle): the oracle must still reproduce it bit for bit on the CPU, and the HIP
path must match it within the path's tolerance on the GPU."""
import os

import numpy as np
import pytest

from util import REL_FRO_TOL, ROOT, ko, rel_fro

G = np.load(os.path.join(ROOT, "tests", "golden", "matmul_path_small.npz"), allow_pickle=False)
G2 = np.load(os.path.join(ROOT, "tests", "golden", "next_to_path_small.npz"), allow_pickle=False)
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


# ---- the operators either side of the path: tests/golden/next_to_path_small.npz ----------------------------------

def test_oracle_reproduces_the_second_fixture_bit_for_bit():
    p, g, s, t, steps = (G2[k] for k in ("upd_p", "upd_g", "upd_s", "upd_t", "upd_steps"))
    lr, l1, l2, ro1, ro2, eps = (float(v) for v in G2["upd_hyper"])
    assert np.array_equal(ko.accumulate_grad(p, g), G2["upd_accumulate"])
    assert np.array_equal(ko.subtract_param_grad(p, g, lr), G2["upd_subtract"])
    assert np.array_equal(ko.apply_decay(p, g, l1, l2), G2["upd_decay"])
    for got, name in zip(ko.eval_adam_delta(g, s, t, steps, ro1, ro2, eps), ("adam_delta", "adam_s", "adam_t", "adam_steps")):
        assert np.array_equal(got, G2[name]), name
    axes = tuple(int(a) for a in G2["tr_axes"])
    assert np.array_equal(ko.transpose_axinfo(G2["tr_x"].shape, axes), G2["tr_table"])
    assert np.array_equal(ko.transpose(G2["tr_x"], axes), G2["tr_y"])
    assert np.array_equal(ko.transpose_backward(G2["tr_gy"], G2["tr_x"].shape, axes), G2["tr_gx"])
    assert np.array_equal(ko.transpose_bin(G2["trbin_x"], 13, 7), G2["trbin_y"])
    r, st = ko.lstm_process(G2["lstm_affine"], G2["lstm_prev_state"])
    assert np.array_equal(r, G2["lstm_recur"]) and np.array_equal(st, G2["lstm_state"])
    for prev, tag in ((G2["lstm_prev_state"], ""), (None, "_first")):
        gs, ga = ko.lstm_process_backward(G2["lstm_gr"], G2["lstm_gs"], G2["lstm_affine"], prev)
        assert np.array_equal(gs, G2["lstm_gprev_state" + tag]) and np.array_equal(ga, G2["lstm_gaffine" + tag])
    assert np.array_equal(ko.gru_process(G2["gru_recurs_in"].copy(), G2["gru_ai"], G2["gru_ar"], 1), G2["gru_recurs_out"])
    for got, name in zip(ko.gru_process_backward(G2["gru_gh"], G2["gru_recurs_out"], G2["gru_ai"], G2["gru_ar"], 1),
                         ("gru_gprev", "gru_gai", "gru_gar")):
        assert np.array_equal(got, G2[name]), name


def test_second_fixture_satisfies_closed_forms():
    axes = tuple(int(a) for a in G2["tr_axes"])
    assert np.array_equal(G2["tr_y"], np.transpose(G2["tr_x"], axes))
    assert np.array_equal(G2["trbin_y"], G2["trbin_x"].T)
    lr = np.float32(G2["upd_hyper"][0])
    assert np.array_equal(G2["upd_subtract"], G2["upd_p"] - G2["upd_g"] * lr)
    assert np.array_equal(G2["adam_steps"], G2["upd_steps"] + 1)
    sig = lambda v: 1 / (1 + np.exp(-v.astype(np.float64)))
    i, f, g, o = (G2["lstm_affine"][:, k * 5:(k + 1) * 5] for k in range(4))
    assert np.allclose(G2["lstm_state"], G2["lstm_prev_state"] * sig(f) + np.tanh(g.astype(np.float64)) * sig(i), atol=1e-6)


@pytest.mark.gpu
def test_hip_path_matches_the_second_fixture():
    from deep_learning_framework_amd import kai
    from deep_learning_framework_amd.kai import DeviceBuffer as DB, VMath
    kai.load()
    kai.set_device(0)
    dev = lambda a: DB.from_numpy(np.ascontiguousarray(a))
    p, g, s, t, steps = (G2[k] for k in ("upd_p", "upd_g", "upd_s", "upd_t", "upd_steps"))
    n = p.size
    lr, l1, l2, ro1, ro2, eps = (kai.hyper(float(v)) for v in G2["upd_hyper"])
    y = dev(p)
    VMath.accumulate_grad(0, y, dev(g), n)
    assert np.array_equal(y.to_numpy(n), G2["upd_accumulate"])
    y = dev(p)
    VMath.subtract_param_grad(0, y, dev(g), n, lr)
    assert np.array_equal(y.to_numpy(n), G2["upd_subtract"])
    d = DB(n * 4)
    VMath.apply_decay(0, d, dev(p), dev(g), n, l1, l2)
    assert np.array_equal(d.to_numpy(n), G2["upd_decay"])
    a, ds, dt, dn = DB(n * 4), dev(s), dev(t), dev(steps)
    VMath.eval_adam_delta(0, a, dev(g), ds, dt, dn, n, ro1, ro2, eps)
    assert np.array_equal(ds.to_numpy(n), G2["adam_s"]) and np.array_equal(dt.to_numpy(n), G2["adam_t"])
    assert np.array_equal(dn.to_numpy(n), G2["adam_steps"])
    assert rel_fro(a.to_numpy(n), G2["adam_delta"]) <= REL_FRO_TOL
    x = G2["tr_x"]
    table = dev(G2["tr_table"])
    out = DB(x.nbytes)
    VMath.transpose(0, out, dev(x), table, x.ndim, x.size)
    assert np.array_equal(out.to_numpy(G2["tr_y"].shape), G2["tr_y"])
    VMath.transpose_backward(0, out, dev(G2["tr_gy"]), table, x.ndim, x.size)
    assert np.array_equal(out.to_numpy(x.shape), G2["tr_gx"])
    ob = DB(G2["trbin_x"].nbytes)
    VMath.transpose_bin(0, ob, dev(G2["trbin_x"]), 13, 7)
    assert np.array_equal(ob.to_numpy((13, 7)), G2["trbin_y"])
    ndat, nrec = G2["lstm_prev_state"].shape
    r, st = DB(ndat * nrec * 4), DB(ndat * nrec * 4)
    VMath.lstm_process(0, r, st, dev(G2["lstm_prev_state"]), dev(G2["lstm_affine"]), ndat, nrec, 0)
    assert rel_fro(r.to_numpy((ndat, nrec)), G2["lstm_recur"]) <= REL_FRO_TOL
    assert rel_fro(st.to_numpy((ndat, nrec)), G2["lstm_state"]) <= REL_FRO_TOL
    VMath.lstm_process(0, r, st, None, dev(G2["lstm_affine"]), ndat, nrec, 0)
    assert rel_fro(r.to_numpy((ndat, nrec)), G2["lstm_recur_first"]) <= REL_FRO_TOL
    for prev, tag in ((G2["lstm_prev_state"], ""), (None, "_first")):
        gs, ga = dev(G2["lstm_gs"]), DB(G2["lstm_affine"].nbytes)
        VMath.lstm_process_backward(0, dev(G2["lstm_gr"]), gs, ga, None if prev is None else dev(prev),
                                    dev(G2["lstm_affine"]), ndat, nrec, 0)
        assert rel_fro(gs.to_numpy((ndat, nrec)), G2["lstm_gprev_state" + tag]) <= REL_FRO_TOL
        assert rel_fro(ga.to_numpy(G2["lstm_affine"].shape), G2["lstm_gaffine" + tag]) <= REL_FRO_TOL
    rec = dev(G2["gru_recurs_in"])
    ai, ar = dev(G2["gru_ai"]), dev(G2["gru_ar"])
    VMath.gru_process(0, rec.offset(ndat * nrec * 4), ai, ar, 1, 2, ndat, nrec)
    assert rel_fro(rec.to_numpy(G2["gru_recurs_out"].shape), G2["gru_recurs_out"]) <= REL_FRO_TOL
    gh, gai, gar, rec2 = dev(G2["gru_gh"]), DB(G2["gru_ai"].nbytes), DB(G2["gru_ar"].nbytes), dev(G2["gru_recurs_out"])
    VMath.gru_process_backward(0, gh, gai, gar, rec2.offset(ndat * nrec * 4), ai, ar, 1, 2, ndat, nrec)
    assert rel_fro(gh.to_numpy((ndat, nrec)), G2["gru_gprev"]) <= REL_FRO_TOL
    assert rel_fro(gai.to_numpy(G2["gru_ai"].shape), G2["gru_gai"]) <= REL_FRO_TOL
    assert rel_fro(gar.to_numpy(G2["gru_ar"].shape), G2["gru_gar"]) <= REL_FRO_TOL
    s2 = DB(n * 4)
    VMath.add(0, s2, dev(p), dev(g), n)
    assert np.array_equal(s2.to_numpy(n), G2["add"])
