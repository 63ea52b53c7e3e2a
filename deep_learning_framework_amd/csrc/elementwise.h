// Launchers of the bandwidth-bound kernels in elementwise.hip and attention_ops.hip.
#pragma once

#include "kai_common.h"

namespace kai {

int launch_add_bias(float* y, const float* a, const float* b, int64_t nrow, int64_t ncol, hipStream_t stream);
// parts: the number colsum_row_parts() gives; with two and more, parts_buf holds parts * ncol floats of scratch
int colsum_row_parts(int64_t nrow, int64_t ncol);
int launch_colsum(float* gb, const float* gy, int64_t nrow, int64_t ncol, int acc, hipStream_t stream,
                  float* parts_buf = nullptr, int parts = 1);
int launch_activate(float* y, const float* x, int64_t total, int act, const float* hleaky, hipStream_t stream);
int launch_activate_backward(float* gx, const float* gy, const float* x, int64_t total, int act, const float* hleaky,
                             hipStream_t stream);
int launch_activate_backward_with_y(float* gx, const float* gy, const float* y, int64_t total, int act,
                                    const float* hleaky, hipStream_t stream);
int launch_softmax_rows(float* y, const float* x, int64_t nrow, int64_t ncol, hipStream_t stream);
int launch_softmax_rows_backward(float* gx, const float* gy, const float* x, int64_t nrow, int64_t ncol,
                                 hipStream_t stream);
int launch_fill_float(float* p, int64_t n, float value, hipStream_t stream);
int launch_fill_int(int* p, int64_t n, int value, hipStream_t stream);

// parameter update: VMath::accumulate_grad / subtract_param_grad / apply_decay / eval_adam_delta
// (vmath.cu:364-490 of the reference); hyper-parameters are device scalars, null reads as 0
int launch_accumulate_grad(float* y, const float* x, int64_t n, hipStream_t stream);
int launch_subtract_param_grad(float* p, const float* g, int64_t n, const float* hlr, hipStream_t stream);
int launch_apply_decay(float* d, const float* p, const float* g, int64_t n, const float* hl1, const float* hl2,
                       hipStream_t stream);
int launch_eval_adam_delta(float* a, const float* g, float* s, float* t, float* nstep, int64_t n, const float* hro1,
                           const float* hro2, const float* heps, hipStream_t stream);

// VMath::transpose / transpose_backward / transpose_bin (vmath.cu:9384-9510 of the reference); pn is the
// engine's device table of axis_size x 3 ints
int launch_transpose(float* y, const float* x, const int* pn, int64_t axis_size, int64_t n, bool backward,
                     hipStream_t stream);
int launch_transpose_bin(float* y, const float* x, int64_t nrow, int64_t ncol, hipStream_t stream);

// VMath::add, lstm_process, lstm_process_backward, gru_process, gru_process_backward (vmath.cu:774-800,
// 4807-4857, 4899-4943, 4946-5080 of the reference): the element-wise steps between the gate products of a
// recurrent layer
int launch_add(float* y, const float* a, const float* b, int64_t n, hipStream_t stream);
int launch_lstm_process(float* r, float* s, const float* s1, const float* a, int64_t ndat, int64_t nrec,
                        hipStream_t stream);
int launch_lstm_process_backward(const float* gr, float* gs, float* ga, const float* s_prev, const float* a,
                                 int64_t ndat, int64_t nrec, hipStream_t stream);
int launch_gru_process(float* r, const float* ai, const float* ar, int64_t nt, int64_t ndat, int64_t nrec,
                       hipStream_t stream);
int launch_gru_process_backward(float* gr, float* gai, float* gar, const float* r, const float* ai, const float* ar,
                                int64_t nt, int64_t ndat, int64_t nrec, hipStream_t stream);

// One LSTM / GRU time step in one launch (recurrent_step.hip): recurrent gate product + biases + cell.
// r_prev null: no recurrent product (first step).  recurrent_step_applies: operand alignment and the sizes up
// to which the single launch beats the separate calls.
constexpr int64_t kRecStepMaxRows = 256, kRecStepMaxUnits = 1024;
bool recurrent_step_applies(const float* wr, const float* r_prev, int64_t ndat, int64_t nrec);
int launch_lstm_step(float* r, float* s, const float* s1, float* a, const float* wr, const float* r_prev,
                     const float* bi, const float* br, int64_t ndat, int64_t nrec, hipStream_t stream);
int launch_gru_step(float* r, float* ai, float* ar, const float* wr, const float* r_prev, const float* h_prev,
                    const float* bi, const float* br, int64_t ndat, int64_t nrec, hipStream_t stream);
// gru_process with the previous output given by pointer (null: 0) instead of by position
int launch_gru_process_from(float* r, const float* h_prev, const float* ai, const float* ar, int64_t ndat, int64_t nrec,
                            hipStream_t stream);

// VMath::cosinesim (vmath.cu:6459-6513 of the reference) after the row-pair products are in y: the norms of
// the nrow1 + nrow2 rows go to norms, then y[i,j] /= norms[i] * norms[nrow1 + j] + 1e-20
int launch_cosine_norms_and_scale(float* y, float* norms, const float* x1, const float* x2, int64_t nrow1,
                                  int64_t nrow2, int64_t ncol, hipStream_t stream);
// up to four rows of x1 against 512 and more of x2: both in one pass over x2
bool cosine_few_rows_applies(const float* x1, const float* x2, int64_t nrow1, int64_t nrow2, int64_t ncol);
int launch_cosine_few_rows(float* y, const float* x1, const float* x2, int64_t nrow1, int64_t nrow2, int64_t ncol,
                           hipStream_t stream);

// Final pass of a split-K product: C(m,n) (=|+=) act(alpha * sum_s part[s][m][n] + bias[n]), the
// pre-activation value also to C2 when given.  `part` holds nsplit dense [M,N] matrices.
struct SplitReduceParams {
    const float* part;
    float* C;
    float* C2;
    const float* bias;
    const float* alpha;   // device scalar or null
    const float* leaky;   // device scalar or null
    int64_t M, N, c_rs, c_cs;
    int nsplit, act, accflag, has_alpha;   // has_alpha with a null alpha multiplies by 0
};
int launch_splitk_reduce(const SplitReduceParams& p, hipStream_t stream);

// attention_ops.hip
int launch_attention_mask(float* pp, int64_t ndat, int64_t ntimes, int64_t nhead, int forward, hipStream_t stream);
int launch_softmax_axis(float* pp, int64_t nrow, int64_t nvec, int64_t ncol, hipStream_t stream);
int launch_softmax_axis_backward(float* pgp, const float* pp, int64_t nrow, int64_t nvec, int64_t ncol,
                                 const float* hcoef, hipStream_t stream);


// attention_fused.hip
bool attention_fused_applies(const float* q, const float* k, const float* v, const float* o, int64_t ntimes,
                             int64_t nvec, int64_t nhead, int64_t npiece);
int launch_attention_fused(float* o, const float* q, const float* k, const float* v, int64_t nbat, int64_t ntimes,
                           int64_t nvec, int64_t nhead, int64_t npiece, const float* hcoef, int masked,
                           hipStream_t stream);

// the same block with the probabilities stored as well (training): lengths up to 1024
bool attention_probs_applies(const float* q, const float* k, const float* v, const float* o, const float* pp,
                             int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece);
bool attention_probs_four_heads(const float* pp, int64_t ntimes, int64_t nhead, int64_t npiece);
// whether the one-launch training forward is expected to beat the three separate calls for this geometry
bool attention_probs_pays(const float* pp, int64_t nbat, int64_t ntimes, int64_t nhead, int64_t npiece);
int launch_attention_probs(float* o, float* pp, const float* q, const float* k, const float* v, int64_t nbat,
                           int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, const float* hcoef, int masked,
                           hipStream_t stream);

// attention_value_grad.hip: gV = P^T.gY per (batch entry, head) without LDS passes of the operands; 0 = geometry not
// served, else the heads a workgroup owns (1 or 4)
int attention_value_grad_heads(const float* gv, const float* gy, const float* pp, int64_t ntimes, int64_t nvec,
                               int64_t nhead, int64_t npiece);
int launch_attention_value_grad(float* gv, const float* gy, const float* pp, int64_t nbat, int64_t ntimes, int64_t nvec,
                                int64_t nhead, int64_t npiece, hipStream_t stream);
// the same kernel with the roles of P's middle indices exchanged: Y[b,t,h,:] = sum_k P[b,t,k,h] * B[b,k,h,:] (mix_values,
// mult_on_heads_backward) for head counts in whole fours and head sizes up to 64
bool attention_heads_mix_applies(const float* out, int64_t out_rs, const float* pp, const float* other, int64_t other_rs,
                                 int64_t ntimes, int64_t nhead, int64_t npiece);
int launch_attention_heads_mix(float* out, int64_t out_rs, const float* pp, const float* other, int64_t other_rs, int64_t nbat,
                               int64_t ntimes, int64_t nhead, int64_t npiece, hipStream_t stream);
// attention_backward.hip: gQ and gK of the attention block from gM, P (and M) without storing gP or gS
bool attention_backward_applies(const float* gq, const float* gk, const float* gm, const float* m, const float* pp,
                                const float* q, const float* k, const float* v, int64_t ntimes, int64_t nvec,
                                int64_t nhead, int64_t npiece);
bool attention_backward_one_launch(const float* gv, const float* gm, const float* pp, int64_t nbat, int64_t ntimes,
                                   int64_t nvec, int64_t nhead, int64_t npiece);
// gv null: gQ and gK only; else gV in the same launch (where attention_backward_one_launch says so)
int launch_attention_backward_rows(float* gq, float* gk, float* gv, const float* gm, const float* m, const float* pp,
                                   const float* q, const float* k, const float* v, int64_t nbat, int64_t ntimes,
                                   int64_t nvec, int64_t nhead, int64_t npiece, const float* hcoef, int masked,
                                   hipStream_t stream);

}  // namespace kai
