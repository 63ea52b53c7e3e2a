#!/usr/bin/env python3
"""Writes tests/golden/matmul_path_small.npz: inputs and expected outputs of every operator of
the matmul path at small shapes, and tests/golden/next_to_path_small.npz: the same for the operators
either side of it (parameter update, transposes, recurrent cells).

The reference ships no golden vectors, known-answer tests or fixtures for this path and cannot be
built or run here, so the expected outputs are produced by the CPU oracle (oracle/kai_oracle.c),
which tests/test_oracle_pins.py pins against closed forms.  The fixture freezes those outputs so
that a later change of the oracle, of its compiler flags or of the host libm shows up as a diff,
and gives the GPU tests a fixed data set.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import oracle as ko  # noqa: E402


def main():
    rng = np.random.default_rng(20240607)
    f = {}
    # dense layer: ndat 19, xvec 23, yvec 11 (all distinct, none a multiple of 4)
    ndat, xvec, yvec = 19, 23, 11
    x = rng.standard_normal((ndat, xvec)).astype(np.float32)
    w = rng.uniform(-0.2, 0.2, (yvec, xvec)).astype(np.float32)
    b = rng.standard_normal(yvec).astype(np.float32)
    gy = rng.standard_normal((ndat, yvec)).astype(np.float32)
    f.update(dense_x=x, dense_w=w, dense_b=b, dense_gy=gy)
    f["dense_matmul"] = ko.matmul(w, x)
    f["dense_pre"] = ko.add_bias(f["dense_matmul"], b)
    f["dense_gx"] = ko.matmul_backward_x(gy, w)
    f["dense_gw"] = ko.matmul_backward_w(gy, x, yvec, xvec)
    f["dense_gb"] = ko.add_bias_backward_b(gy, yvec)
    f["dense_matmul_acc"] = ko.matmul(w, x, acc_into=f["dense_pre"])
    for name in ["none", "relu", "leaky", "sigmoid", "tanh", "gelu", "selu", "mish", "swish", "softmax"]:
        alpha = 0.1 if name == "leaky" else None
        f["act_" + name] = ko.activate(f["dense_pre"], name, alpha)
        if name != "softmax":
            f["actbwd_" + name] = ko.activate_backward(gy, f["dense_pre"], name, alpha)
        if name in ("none", "relu", "leaky", "sigmoid", "tanh"):
            f["actbwdy_" + name] = ko.activate_backward_with_y(gy, f["act_" + name], name, alpha)
    # attention: nbat 2, ntimes 9, nhead 3, npiece 5
    nbat, ntimes, nhead, npiece = 2, 9, 3, 5
    nvec = nhead * npiece
    q = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    k = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    v = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    go = rng.standard_normal((nbat, ntimes, nvec)).astype(np.float32)
    coef = np.float32(1.0 / np.sqrt(npiece))
    f.update(att_q=q, att_k=k, att_v=v, att_go=go, att_coef=np.array([coef], np.float32),
             att_dims=np.array([nbat, ntimes, nhead, npiece], np.int64))
    s = ko.mult_on_heads(k, q, nhead, float(coef))
    f["att_scores"] = s
    f["att_masked"] = ko.set_mh_attention_mask(s, True)
    f["att_probs"] = ko.softmax_direct_on_axis(s, nbat * ntimes, ntimes, nhead)
    f["att_probs_masked"] = ko.softmax_direct_on_axis(f["att_masked"], nbat * ntimes, ntimes, nhead)
    f["att_out"] = ko.mix_values(f["att_probs"], v, nhead)
    f["att_gprobs"] = ko.mix_values_backward_prop(go, v, nhead)
    f["att_gv"] = ko.mix_values_backward_value(go, f["att_probs"], nhead)
    f["att_gscores"] = ko.softmax_direct_on_axis_backward(f["att_gprobs"], f["att_probs"], float(coef))
    f["att_gk"] = ko.mult_on_heads_backward(f["att_gscores"], q, nhead)
    f["att_gq"] = ko.mult_on_heads_backward(f["att_gscores"], k, nhead)
    out = os.path.join(HERE, "matmul_path_small.npz")
    np.savez_compressed(out, **f)
    print("wrote", out, os.path.getsize(out), "bytes,", len(f), "arrays")
    next_to_path()


def next_to_path():
    rng = np.random.default_rng(20240608)
    f = {}
    # parameter update on 37 elements
    n = 37
    p = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    s = (rng.standard_normal(n) * 0.1).astype(np.float32)
    t = (rng.random(n) * 0.01).astype(np.float32)
    steps = np.full(n, 3, np.float32)
    f.update(upd_p=p, upd_g=g, upd_s=s, upd_t=t, upd_steps=steps,
             upd_hyper=np.array([0.01, 0.001, 0.0005, 0.9, 0.999, 1e-8], np.float32))   # lr, l1, l2, ro1, ro2, eps
    f["upd_accumulate"] = ko.accumulate_grad(p, g)
    f["upd_subtract"] = ko.subtract_param_grad(p, g, 0.01)
    f["upd_decay"] = ko.apply_decay(p, g, 0.001, 0.0005)
    f["adam_delta"], f["adam_s"], f["adam_t"], f["adam_steps"] = ko.eval_adam_delta(g, s, t, steps, 0.9, 0.999, 1e-8)
    # transposes
    x = rng.standard_normal((2, 3, 4, 5)).astype(np.float32)
    axes = (2, 0, 3, 1)
    f.update(tr_x=x, tr_axes=np.array(axes, np.int64), tr_table=ko.transpose_axinfo(x.shape, axes))
    f["tr_y"] = ko.transpose(x, axes)
    gy = rng.standard_normal(f["tr_y"].shape).astype(np.float32)
    f.update(tr_gy=gy, tr_gx=ko.transpose_backward(gy, x.shape, axes))
    xb = rng.standard_normal((7, 13)).astype(np.float32)          # [ncol, nrow]
    f.update(trbin_x=xb, trbin_y=ko.transpose_bin(xb, 13, 7))
    # recurrent cells: ndat 3, nrec 5
    ndat, nrec = 3, 5
    a4 = (rng.standard_normal((ndat, 4 * nrec)) * 2).astype(np.float32)
    st = rng.standard_normal((ndat, nrec)).astype(np.float32)
    f.update(lstm_affine=a4, lstm_prev_state=st)
    f["lstm_recur"], f["lstm_state"] = ko.lstm_process(a4, st)
    f["lstm_recur_first"], f["lstm_state_first"] = ko.lstm_process(a4, None)
    ai = rng.standard_normal((ndat, 3 * nrec)).astype(np.float32)
    ar = rng.standard_normal((ndat, 3 * nrec)).astype(np.float32)
    recurs = np.zeros((2, ndat, nrec), np.float32)
    recurs[0] = rng.standard_normal((ndat, nrec)).astype(np.float32)
    gh = rng.standard_normal((ndat, nrec)).astype(np.float32)
    f.update(gru_ai=ai, gru_ar=ar, gru_recurs_in=recurs.copy(), gru_gh=gh)
    f["gru_recurs_out"] = ko.gru_process(recurs, ai, ar, 1).copy()
    f["gru_gprev"], f["gru_gai"], f["gru_gar"] = ko.gru_process_backward(gh, f["gru_recurs_out"], ai, ar, 1)
    f["add"] = ko.add(p, g)
    # lstm cell gradient (drawn after everything above, so the earlier arrays keep their values)
    lgr = rng.standard_normal((ndat, nrec)).astype(np.float32)
    lgs = rng.standard_normal((ndat, nrec)).astype(np.float32)
    f.update(lstm_gr=lgr, lstm_gs=lgs)
    f["lstm_gprev_state"], f["lstm_gaffine"] = ko.lstm_process_backward(lgr, lgs, a4, st)
    f["lstm_gprev_state_first"], f["lstm_gaffine_first"] = ko.lstm_process_backward(lgr, lgs, a4, None)
    out = os.path.join(HERE, "next_to_path_small.npz")
    np.savez_compressed(out, **f)
    print("wrote", out, os.path.getsize(out), "bytes,", len(f), "arrays")


if __name__ == "__main__":
    main()
