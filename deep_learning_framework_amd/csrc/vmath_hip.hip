// class VMath (include/vmath_hip.h): the engine's operator names over the C-ABI.
#include "../../include/vmath_hip.h"

#include "../../include/kai_hip.h"

static void raise_on(int rc) {
    if (rc != KAI_OK) throw KaiMathError(rc, kai_last_error());
}

void* VMath::mem_alloc(int device, int64 size) {
    void* p = nullptr;
    raise_on(kai_mem_alloc(device, size, &p));
    return p;
}
void VMath::mem_free(int device, void* ptr) { raise_on(kai_mem_free(device, ptr)); }

void VMath::memcpy_host_to_host(void* d, void* s, int64 n) { raise_on(kai_memcpy_host_to_host(d, s, n)); }
void VMath::memcpy_host_to_device(void* d, void* s, int64 n) { raise_on(kai_memcpy_host_to_device(d, s, n)); }
void VMath::memcpy_device_to_host(void* d, void* s, int64 n) { raise_on(kai_memcpy_device_to_host(d, s, n)); }
void VMath::memcpy_device_to_device(void* d, void* s, int64 n) { raise_on(kai_memcpy_device_to_device(d, s, n)); }

void VMath::copy_data(int dd, int sd, void* py, void* px, int64 n) { raise_on(kai_copy_data(dd, sd, py, px, n)); }

void VMath::fill_int(int device, int* p, int64 n, int v) { raise_on(kai_fill_int(device, p, n, v)); }
void VMath::fill_float(int device, float* p, int64 n, float v) { raise_on(kai_fill_float(device, p, n, v)); }
void VMath::set_zero(int device, void* p, int64 n) { raise_on(kai_set_zero(device, p, n)); }

void VMath::memcpy_from_host(int device, void* py, void* px, int64 n) { raise_on(kai_memcpy_from_host(device, py, px, n)); }
void VMath::memcpy_to_host(int device, void* py, void* px, int64 n) { raise_on(kai_memcpy_to_host(device, py, px, n)); }
void VMath::memcpy_to_device(int device, void* py, void* px, int64 n) { raise_on(kai_memcpy_to_device(device, py, px, n)); }
void VMath::get_slice(int device, void* py, void* px, int64 n) { raise_on(kai_get_slice(device, py, px, n)); }

void VMath::add_bias(int device, float* py, float* pa, float* pb, int64 nrow, int64 ncol) {
    raise_on(kai_add_bias(device, py, pa, pb, nrow, ncol));
}
void VMath::add_bias_backward_b(int device, float* pgb, float* pgy, int64 nrow, int64 ncol, bool acc) {
    raise_on(kai_add_bias_backward_b(device, pgb, pgy, nrow, ncol, acc));
}

void VMath::matmul(int device, float* py, float* pw, float* px, int64 yvec, int64 ndat, int64 xvec, bool acc) {
    raise_on(kai_matmul(device, py, pw, px, yvec, ndat, xvec, acc));
}
void VMath::matmul_backward_x(int device, float* pgx, float* pgy, float* pw, int64 yvec, int64 ndat, int64 xvec, bool acc) {
    raise_on(kai_matmul_backward_x(device, pgx, pgy, pw, yvec, ndat, xvec, acc));
}
void VMath::matmul_backward_w(int device, float* pgw, float* pgy, float* px, int64 yvec, int64 ndat, int64 xvec, bool acc) {
    raise_on(kai_matmul_backward_w(device, pgw, pgy, px, yvec, ndat, xvec, acc));
}

void VMath::activate(int device, float* py, float* px, int64 nrow, int64 ncol, int actFunc, HYPER h) {
    raise_on(kai_activate(device, py, px, nrow, ncol, actFunc, h));
}
void VMath::activate_backward(int device, float* pgx, float* pgy, float* px, int64 nrow, int64 ncol, int actFunc, HYPER h) {
    raise_on(kai_activate_backward(device, pgx, pgy, px, nrow, ncol, actFunc, h));
}
void VMath::activate_backward_with_y(int device, float* pgx, float* pgy, float* py, int64 nrow, int64 ncol, int actFunc, HYPER h) {
    raise_on(kai_activate_backward_with_y(device, pgx, pgy, py, nrow, ncol, actFunc, h));
}

void VMath::mult_on_heads(int device, float* pp, float* pK, float* pQ, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef) {
    raise_on(kai_mult_on_heads(device, pp, pK, pQ, nbat, ntimes, nvec, nhead, npiece, hCoef));
}
void VMath::mult_on_heads_backward(int device, float* pg, float* pgp, float* pQKV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece) {
    raise_on(kai_mult_on_heads_backward(device, pg, pgp, pQKV, nbat, ntimes, nvec, nhead, npiece));
}
void VMath::set_mh_attention_mask(int device, float* pp, int64 ndat, int64 ntimes, int64 nhead, bool forward) {
    raise_on(kai_set_mh_attention_mask(device, pp, ndat, ntimes, nhead, forward));
}
void VMath::softmax_direct_on_axis(int device, float* pp, int64 nrow, int64 nvec, int64 ncol) {
    raise_on(kai_softmax_direct_on_axis(device, pp, nrow, nvec, ncol));
}
void VMath::softmax_direct_on_axis_backward(int device, float* pgp, float* pp, int64 nbat, int64 ntimes, int64 nhead, HYPER hCoef) {
    raise_on(kai_softmax_direct_on_axis_backward(device, pgp, pp, nbat, ntimes, nhead, hCoef));
}
void VMath::mix_values(int device, float* py, float* pp, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece) {
    raise_on(kai_mix_values(device, py, pp, pV, nbat, ntimes, nvec, nhead, npiece));
}
void VMath::mix_values_backward_prop(int device, float* pgp, float* pgy, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece) {
    raise_on(kai_mix_values_backward_prop(device, pgp, pgy, pV, nbat, ntimes, nvec, nhead, npiece));
}
void VMath::mix_values_backward_value(int device, float* pgV, float* pgy, float* pp, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece) {
    raise_on(kai_mix_values_backward_value(device, pgV, pgy, pp, nbat, ntimes, nvec, nhead, npiece));
}

void VMath::cosinesim(int device, float* py, float* px1, float* px2, int64 nrow1, int64 nrow2, int64 ncol) {
    raise_on(kai_cosinesim(device, py, px1, px2, nrow1, nrow2, ncol));
}
void VMath::copy(int device, float* py, float* pa, int64 ndat) { raise_on(kai_copy(device, py, pa, ndat)); }
void VMath::add(int device, float* py, float* pa, float* pb, int64 ndat) { raise_on(kai_add(device, py, pa, pb, ndat)); }
void VMath::lstm_process(int device, float* pr, float* ps, float* ps1, float* pa, int64 ndat, int64 nrec, int64 ninp) {
    raise_on(kai_lstm_process(device, pr, ps, ps1, pa, ndat, nrec, ninp));
}
void VMath::lstm_process_backward(int device, float* pgr, float* pgs, float* pga, float* ps, float* pa, int64 ndat,
                                  int64 nrec, int64 ninp) {
    raise_on(kai_lstm_process_backward(device, pgr, pgs, pga, ps, pa, ndat, nrec, ninp));
}
void VMath::gru_process(int device, float* pr, float* pai, float* par, int64 nt, int64 ntimes, int64 ndat, int64 nrec) {
    raise_on(kai_gru_process(device, pr, pai, par, nt, ntimes, ndat, nrec));
}
void VMath::gru_process_backward(int device, float* pgr, float* pgai, float* pgar, float* pr, float* pai, float* par,
                                 int64 nt, int64 ntimes, int64 ndat, int64 nrec) {
    raise_on(kai_gru_process_backward(device, pgr, pgai, pgar, pr, pai, par, nt, ntimes, ndat, nrec));
}
void VMath::lstm_step(int device, float* pr, float* ps, float* ps_prev, float* pa, float* pwr, float* pr_prev, float* pbi,
                      float* pbr, int64 ndat, int64 nrec) {
    raise_on(kai_lstm_step(device, pr, ps, ps_prev, pa, pwr, pr_prev, pbi, pbr, ndat, nrec));
}
void VMath::gru_step(int device, float* pr, float* pai, float* par, float* pwr, float* pr_prev, float* ph_prev, float* pbi,
                     float* pbr, int64 ndat, int64 nrec) {
    raise_on(kai_gru_step(device, pr, pai, par, pwr, pr_prev, ph_prev, pbi, pbr, ndat, nrec));
}
void VMath::transpose(int device, float* py, float* px, int* pn, int64 axis_size, int64 data_size) {
    raise_on(kai_transpose(device, py, px, pn, axis_size, data_size));
}
void VMath::transpose_backward(int device, float* pgx, float* pgy, int* pn, int64 axis_size, int64 data_size) {
    raise_on(kai_transpose_backward(device, pgx, pgy, pn, axis_size, data_size));
}
void VMath::transpose_bin(int device, float* py, float* px, int64 nrow, int64 ncol) {
    raise_on(kai_transpose_bin(device, py, px, nrow, ncol));
}
void VMath::accumulate_grad(int device, float* py, float* px, int64 nrow) {
    raise_on(kai_accumulate_grad(device, py, px, nrow));
}
void VMath::subtract_param_grad(int device, float* pp, float* pg, int64 nrow, HYPER h) {
    raise_on(kai_subtract_param_grad(device, pp, pg, nrow, h));
}
void VMath::apply_decay(int device, float* pd, float* pp, float* pg, int64 nrow, HYPER h1, HYPER h2) {
    raise_on(kai_apply_decay(device, pd, pp, pg, nrow, h1, h2));
}
void VMath::eval_adam_delta(int device, float* pa, float* pg, float* ps, float* pt, float* pn, int64 nrow, HYPER hRo1, HYPER hRo2, HYPER hEpsilon) {
    raise_on(kai_eval_adam_delta(device, pa, pg, ps, pt, pn, nrow, hRo1, hRo2, hEpsilon));
}

void VMath::attention_forward(int device, float* py, float* pQ, float* pK, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef, bool masked) {
    raise_on(kai_attention_forward(device, py, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef, masked ? 1 : 0));
}

void VMath::dense_forward(int device, float* py, float* ppre, float* pw, float* pb, float* px, int64 yvec, int64 ndat, int64 xvec, int actFunc, HYPER h) {
    raise_on(kai_dense_forward(device, py, ppre, pw, pb, px, yvec, ndat, xvec, actFunc, h));
}
void VMath::attention_forward_train(int device, float* py, float* pp, float* pQ, float* pK, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef, bool masked) {
    raise_on(kai_attention_forward_train(device, py, pp, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef, masked ? 1 : 0));
}

void VMath::attention_backward(int device, float* pgQ, float* pgK, float* pgV, float* pgm, float* pp, float* pm, float* pQ, float* pK, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef, bool masked) {
    raise_on(kai_attention_backward(device, pgQ, pgK, pgV, pgm, pp, pm, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef, masked ? 1 : 0));
}

void VMath::dense_backward(int device, float* pgx, float* pgw, float* pgb, float* pga_work, float* pgy, float* pw, float* px, float* ppre, int64 yvec, int64 ndat, int64 xvec, int actFunc, HYPER h, bool acc) {
    raise_on(kai_dense_backward(device, pgx, pgw, pgb, pga_work, pgy, pw, px, ppre, yvec, ndat, xvec, actFunc, h, acc));
}
