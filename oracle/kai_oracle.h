/*
 * kai_oracle.h -- CPU restatement of the KONAN AI engine's host math loops for
 * the matrix-multiplication path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the cpu_baseline leg of the benchmark may link or load it.
 * The shipped library never calls into it and has no CPU fallback.
 *
 * Every function follows, loop for loop, one `*_host` function of the
 * reference engine (file source/engine/support/vmath.cu, cited per function):
 * the same index order, a `float` accumulator that starts at 0.0f, a separately
 * rounded multiply and add (build with -ffp-contract=off, no fast-math), and the
 * `acc` flag applied after the dot product.  Argument order and meaning are
 * those of the reference's VMath methods (source/engine/support/vmath.h:65-66,
 * 137-143, 234-241) minus the leading `device` argument.
 *
 * Hyper-parameters (`hLeakyAlpha`, `hCoef`) are pointers to one float; a null
 * pointer reads as 0, as the reference's HYPER_ACCESS does
 * (source/engine/local_objects/vhypermanager.h:9).
 *
 * Return value: 0 on success, KO_ERR_CONDITIONAL_STATEMENT (8) where the
 * reference throws VERR_CONDITIONAL_STATEMENT (unknown activation code).
 *
 * Parity status: every function here is pinned by tests/test_oracle_pins.py
 * (closed forms in float64, exact small-integer cases, brute force on tiny
 * shapes, adjoint identities and special values).  The reference holds no golden
 * vectors and cannot be compiled in this image (it needs the CUDA toolkit,
 * curand and OpenCV), so those checks are the whole pin; nothing is left
 * "parity unpinned" except the libm-level rounding of expf/erff/logf, which the
 * tolerance covers.
 */
#ifndef KAI_ORACLE_H
#define KAI_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KO_OK 0
#define KO_ERR_CONDITIONAL_STATEMENT 8

/* activation codes: source/engine/include/vtypes.h:37-39 */
enum {
    KO_ACT_NONE = 0, KO_ACT_RELU = 1, KO_ACT_LEAKY = 2, KO_ACT_SIGMOID = 3, KO_ACT_TANH = 4,
    KO_ACT_GELU = 5, KO_ACT_SELU = 6, KO_ACT_MISH = 7, KO_ACT_SWISH = 8, KO_ACT_SOFTMAX = 9
};

/* vmath.cu:2961-2977  y[nd,ny] (=|+=) sum_nx w[ny,nx]*x[nd,nx] */
int ko_matmul(float* py, const float* pw, const float* px, int64_t yvec, int64_t ndat, int64_t xvec, int acc);
/* same loop restricted to rows nd in [nd_begin, nd_end): lets callers sample rows of a
 * large product or spread rows over threads; each element's sum order is unchanged. */
int ko_matmul_rows(float* py, const float* pw, const float* px, int64_t yvec, int64_t nd_begin, int64_t nd_end,
                   int64_t xvec, int acc);
/* vmath.cu:3007-3022  gx[nd,nx] (=|+=) sum_ny w[ny,nx]*gy[nd,ny] */
int ko_matmul_backward_x(float* pgx, const float* pgy, const float* pw, int64_t yvec, int64_t ndat, int64_t xvec, int acc);
/* vmath.cu:3051-3067  gw[ny,nx] (=|+=) sum_nd x[nd,nx]*gy[nd,ny] */
int ko_matmul_backward_w(float* pgw, const float* pgy, const float* px, int64_t yvec, int64_t ndat, int64_t xvec, int acc);

/* vmath.cu:875-881 */
int ko_add_bias(float* py, const float* pa, const float* pb, int64_t nrow, int64_t ncol);
/* vmath.cu:901-911 */
int ko_add_bias_backward_b(float* pgb, const float* pgy, int64_t nrow, int64_t ncol, int acc);

/* vmath.cu:3097-3167 (helpers :297-307) */
int ko_activate(float* py, const float* px, int64_t nrow, int64_t ncol, int actFunc, const float* hLeakyAlpha);
/* vmath.cu:3247-3308 */
int ko_activate_backward(float* pgx, const float* pgy, const float* px, int64_t nrow, int64_t ncol, int actFunc,
                         const float* hLeakyAlpha);
/* vmath.cu:3411-3444 */
int ko_activate_backward_with_y(float* pgx, const float* pgy, const float* py, int64_t nrow, int64_t ncol, int actFunc,
                                const float* hLeakyAlpha);

/* vmath.cu:6729-6750 */
int ko_mult_on_heads(float* pp, const float* pK, const float* pQ, int64_t nbat, int64_t ntimes, int64_t nvec,
                     int64_t nhead, int64_t npiece, const float* hCoef);
/* vmath.cu:6783-6802 */
int ko_mult_on_heads_backward(float* pgQK, const float* pgp, const float* pKQ, int64_t nbat, int64_t ntimes,
                              int64_t nvec, int64_t nhead, int64_t npiece);
/* vmath.cu:6833-6844 */
int ko_set_mh_attention_mask(float* pp, int64_t ndat, int64_t ntimes, int64_t nhead, int forward);
/* vmath.cu:6864-6885 */
int ko_softmax_direct_on_axis(float* pp, int64_t nrow, int64_t nvec, int64_t ncol);
/* vmath.cu:6920-6942 */
int ko_softmax_direct_on_axis_backward(float* pgp, const float* pp, int64_t nbat, int64_t ntimes, int64_t nhead,
                                       const float* hCoef);
/* vmath.cu:6977-6997 */
int ko_mix_values(float* py, const float* pp, const float* pV, int64_t nbat, int64_t ntimes, int64_t nvec,
                  int64_t nhead, int64_t npiece);
/* vmath.cu:7029-7049 */
int ko_mix_values_backward_prop(float* pgp, const float* pgy, const float* pV, int64_t nbat, int64_t ntimes,
                                int64_t nvec, int64_t nhead, int64_t npiece);
/* vmath.cu:7081-7101 */
int ko_mix_values_backward_value(float* pgV, const float* pgy, const float* pp, int64_t nbat, int64_t ntimes,
                                 int64_t nvec, int64_t nhead, int64_t npiece);

/* vmath.cu:364-368, 385-390, 408-421, 449-468: what consumes the weight and bias gradients */
int ko_accumulate_grad(float* py, const float* px, int64_t ndat);
int ko_subtract_param_grad(float* pp, const float* pg, int64_t nrow, const float* hLearningRate);
int ko_apply_decay(float* pd, const float* pp, const float* pg, int64_t nrow, const float* hL1Decay,
                   const float* hL2Decay);
int ko_eval_adam_delta(float* pa, const float* pg, float* ps, float* pt, float* pn, int64_t nrow, const float* hRo1,
                       const float* hRo2, const float* hEpsilon);

/* vmath.cu:9384-9403, 9436-9455, 9487-9494 */
int ko_transpose(float* py, const float* px, const int* pn, int64_t axis_size, int64_t data_size);
int ko_transpose_backward(float* pgx, const float* pgy, const int* pn, int64_t axis_size, int64_t data_size);
int ko_transpose_bin(float* py, const float* px, int64_t nrow, int64_t ncol);

/* cosine similarity of every row of x1[nrow1, ncol] with every row of x2[nrow2, ncol] (vmath.cu:6459-6480) */
int ko_cosinesim(float* py, const float* px1, const float* px2, int64_t nrow1, int64_t nrow2, int64_t ncol);

/* recurrent cells (vmath.cu:732-736, 774-778, 4807-4826, 4899-4937, 4946-4965, 4999-5033).
 * lstm_process_backward follows the reference's DEVICE kernel (vmath.cu:4899-4937, gate gradients at
 * apos + g * nrec): the host loop (vmath.cu:4860-4897) has the same arithmetic but its index expression
 * (apos * g + n * nrec) leaves the [ndat, 4*nrec] buffer. */
int ko_copy(float* py, const float* pa, int64_t ndat);
int ko_add(float* py, const float* pa, const float* pb, int64_t ndat);
int ko_lstm_process(float* pr, float* ps, const float* ps1, const float* pa, int64_t ndat, int64_t nrec);
int ko_lstm_process_backward(const float* pgr, float* pgs, float* pga, const float* ps, const float* pa,
                             int64_t ndat, int64_t nrec);
int ko_gru_process(float* pr, const float* pai, const float* par, int64_t nt, int64_t ndat, int64_t nrec);
int ko_gru_process_backward(float* pgr, float* pgai, float* pgar, const float* pr, const float* pai,
                            const float* par, int64_t nt, int64_t ndat, int64_t nrec);

#ifdef __cplusplus
}
#endif
#endif
