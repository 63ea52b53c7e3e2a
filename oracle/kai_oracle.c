/*
 * kai_oracle.c -- CPU restatement of the reference engine's host loops for the
 * matrix-multiplication path.  TEST INFRASTRUCTURE ONLY (see kai_oracle.h).
 *
 * Build: gcc -O2 -ffp-contract=off -fPIC -shared (oracle/Makefile); the flags
 * mirror the reference's Linux build, which forbids contraction of a*b+c into an
 * FMA (source/engine/CMakeLists.txt:189-208).
 *
 * One deliberate deviation, documented at ko_activate(): the reference's softmax
 * activation case computes its row pointer from the array base instead of from
 * the current element and so reads outside the buffer for every element but
 * those of column 0 (vmath.cu:3146); the restatement uses the row the element
 * belongs to, which is what the surrounding code evidently intends.
 */
#include "kai_oracle.h"

#include <float.h>
#include <math.h>

#define KO_PI 3.14159265358979323846

static float hyper_value(const float* h) { return h ? *h : 0.0f; }

/* ---- dense matmul family ------------------------------------------------------------------- */

int ko_matmul_rows(float* py, const float* pw, const float* px, int64_t yvec, int64_t nd_begin, int64_t nd_end,
                   int64_t xvec, int acc) {
    /* vmath.cu:2961-2977, outer loop cut to a row range */
    for (int64_t nd = nd_begin; nd < nd_end; nd++) {
        const float* xrow = px + nd * xvec;
        float* yrow = py + nd * yvec;
        for (int64_t ny = 0; ny < yvec; ny++) {
            const float* wrow = pw + ny * xvec;
            float dot = 0.0f;
            for (int64_t nx = 0; nx < xvec; nx++) {
                dot += wrow[nx] * xrow[nx];
            }
            if (acc) yrow[ny] += dot;
            else yrow[ny] = dot;
        }
    }
    return KO_OK;
}

int ko_matmul(float* py, const float* pw, const float* px, int64_t yvec, int64_t ndat, int64_t xvec, int acc) {
    return ko_matmul_rows(py, pw, px, yvec, 0, ndat, xvec, acc);
}

int ko_matmul_backward_x(float* pgx, const float* pgy, const float* pw, int64_t yvec, int64_t ndat, int64_t xvec,
                         int acc) {
    /* vmath.cu:3007-3022 */
    for (int64_t nd = 0; nd < ndat; nd++) {
        for (int64_t nx = 0; nx < xvec; nx++) {
            float dot = 0.0f;
            for (int64_t ny = 0; ny < yvec; ny++) {
                dot += pw[ny * xvec + nx] * pgy[nd * yvec + ny];
            }
            float* out = pgx + nd * xvec + nx;
            if (acc) *out += dot;
            else *out = dot;
        }
    }
    return KO_OK;
}

int ko_matmul_backward_w(float* pgw, const float* pgy, const float* px, int64_t yvec, int64_t ndat, int64_t xvec,
                         int acc) {
    /* vmath.cu:3051-3067 */
    for (int64_t ny = 0; ny < yvec; ny++) {
        for (int64_t nx = 0; nx < xvec; nx++) {
            float dot = 0.0f;
            for (int64_t nd = 0; nd < ndat; nd++) {
                dot += px[nd * xvec + nx] * pgy[nd * yvec + ny];
            }
            float* out = pgw + ny * xvec + nx;
            if (acc) *out += dot;
            else *out = dot;
        }
    }
    return KO_OK;
}

/* ---- bias ---------------------------------------------------------------------------------- */

int ko_add_bias(float* py, const float* pa, const float* pb, int64_t nrow, int64_t ncol) {
    /* vmath.cu:875-881; py may alias pa */
    for (int64_t nr = 0; nr < nrow; nr++) {
        for (int64_t nc = 0; nc < ncol; nc++) {
            py[nr * ncol + nc] = pa[nr * ncol + nc] + pb[nc];
        }
    }
    return KO_OK;
}

int ko_add_bias_backward_b(float* pgb, const float* pgy, int64_t nrow, int64_t ncol, int acc) {
    /* vmath.cu:901-911 */
    for (int64_t nc = 0; nc < ncol; nc++) {
        float sum = 0.0f;
        for (int64_t nr = 0; nr < nrow; nr++) {
            sum += pgy[nr * ncol + nc];
        }
        if (acc) pgb[nc] += sum;
        else pgb[nc] = sum;
    }
    return KO_OK;
}

/* ---- activations ---------------------------------------------------------------------------- */

static float ko_sigmoid(float x) {
    /* vmath.cu:297-299 */
    return (x > 0) ? (1.0f / (1.0f + expf(-x))) : (expf(x) / (expf(x) + 1.0f));
}

static float ko_tanh(float x) {
    /* vmath.cu:305-307 */
    return 2 * ko_sigmoid(2 * x) - 1;
}

int ko_activate(float* py, const float* px, int64_t nrow, int64_t ncol, int actFunc, const float* hLeakyAlpha) {
    /* vmath.cu:3097-3167 */
    const float leaky_alpha = hyper_value(hLeakyAlpha);
    if (actFunc < KO_ACT_NONE || actFunc > KO_ACT_SOFTMAX) return KO_ERR_CONDITIONAL_STATEMENT;

    for (int64_t nr = 0; nr < nrow; nr++) {
        const float* xrow = px + nr * ncol;
        for (int64_t nc = 0; nc < ncol; nc++) {
            const float x = xrow[nc];
            float y, t;
            switch (actFunc) {
            case KO_ACT_NONE:
                y = x;
                break;
            case KO_ACT_RELU:
                y = (x > 0) ? x : 0;
                break;
            case KO_ACT_LEAKY:
                y = (x > 0) ? x : x * leaky_alpha;
                break;
            case KO_ACT_SIGMOID:
                y = ko_sigmoid(x);
                break;
            case KO_ACT_TANH:
                y = ko_tanh(x);
                break;
            case KO_ACT_GELU:
                y = x * 0.5f * (1.0f + erff(x / sqrtf(2.0f)));
                break;
            case KO_ACT_SELU: {
                const float lambda = 1.0507009f;
                const float alpha = 1.6732632f;
                y = (x > 0) ? lambda * x : lambda * alpha * (expf(x) - 1);
                break;
            }
            case KO_ACT_MISH:
                t = logf(1.0f + expf(x)) * 2;
                t = (float)((t > 0) ? ((1.0f - expf(-t)) / (1.0f + expf(-t))) : ((expf(t) - 1.0f) / (expf(t) + 1.0f)));
                y = x * t;
                break;
            case KO_ACT_SWISH:
                t = (float)((x > 0) ? (1.0f / (1.0f + expf(-x))) : (expf(x) / (expf(x) + 1.0f)));
                y = x * t;
                break;
            default: { /* KO_ACT_SOFTMAX */
                /* vmath.cu:3140-3157, with the row taken from the element's own row (the reference
                 * subtracts the column index from the array base, an out-of-bounds read). */
                float max_term = -FLT_MAX;
                float exp_sum = 0.0f;
                for (int64_t nn = 0; nn < ncol; nn++) {
                    if (xrow[nn] > max_term) max_term = xrow[nn];
                }
                for (int64_t nn = 0; nn < ncol; nn++) {
                    exp_sum += expf(xrow[nn] - max_term);
                }
                y = expf(x - max_term) / exp_sum;
                break;
            }
            }
            py[nr * ncol + nc] = y;
        }
    }
    return KO_OK;
}

int ko_activate_backward(float* pgx, const float* pgy, const float* px, int64_t nrow, int64_t ncol, int actFunc,
                         const float* hLeakyAlpha) {
    /* vmath.cu:3247-3308; the host twin has no softmax case (it throws) */
    const float leaky_alpha = hyper_value(hLeakyAlpha);
    if (actFunc < KO_ACT_NONE || actFunc > KO_ACT_SWISH) return KO_ERR_CONDITIONAL_STATEMENT;

    const int64_t total = nrow * ncol;
    for (int64_t n = 0; n < total; n++) {
        const float gy = pgy[n];
        const float x = px[n];
        float gx, y, s, t, u, v;
        switch (actFunc) {
        case KO_ACT_NONE:
            gx = 1.0f;
            break;
        case KO_ACT_RELU:
            gx = (x > 0) ? 1.0f : 0.0f;
            break;
        case KO_ACT_LEAKY:
            gx = (x > 0) ? 1.0f : leaky_alpha;
            break;
        case KO_ACT_SIGMOID:
            y = ko_sigmoid(x);
            gx = y * (1.0f - y);
            break;
        case KO_ACT_TANH:
            y = ko_tanh(x);
            gx = 1.0f - y * y;
            break;
        case KO_ACT_GELU:
            s = 0.5f * (1.0f + erff(x / sqrtf(2.0f)));
            t = 0.5f * x * sqrtf(2.0f / (float)KO_PI) * expf(-x * x / 2.0f);
            gx = s + t;
            break;
        case KO_ACT_SELU: {
            const float lambda = 1.0507009f;
            const float alpha = 1.6732632f;
            gx = (x > 0) ? lambda : lambda * alpha * expf(x);
            break;
        }
        case KO_ACT_MISH:
            s = logf(1.0f + expf(x));
            t = (x > 0) ? (1.0f / (1.0f + expf(-x))) : (expf(x) / (1.0f + expf(x)));
            s = s * 2.0f;
            u = (float)((s > 0) ? ((1.0f - expf(-s)) / (1.0f + expf(-s))) : ((expf(s) - 1.0f) / (expf(s) + 1.0f)));
            v = (1.0f - u * u);
            gx = u + x * v * t;
            break;
        default: /* KO_ACT_SWISH */
            s = ko_sigmoid(x);
            t = s * (1.0f - s);
            gx = s + x * t;
            break;
        }
        pgx[n] = gx * gy;
    }
    return KO_OK;
}

int ko_activate_backward_with_y(float* pgx, const float* pgy, const float* py, int64_t nrow, int64_t ncol,
                                int actFunc, const float* hLeakyAlpha) {
    /* vmath.cu:3411-3444; only none/relu/leaky/sigmoid/tanh exist */
    const float leaky_alpha = hyper_value(hLeakyAlpha);
    if (actFunc < KO_ACT_NONE || actFunc > KO_ACT_TANH) return KO_ERR_CONDITIONAL_STATEMENT;

    const int64_t total = nrow * ncol;
    for (int64_t n = 0; n < total; n++) {
        const float gy = pgy[n];
        const float y = py[n];
        float gx;
        switch (actFunc) {
        case KO_ACT_NONE:
            gx = 1.0f;
            break;
        case KO_ACT_RELU:
            gx = (y > 0) ? 1.0f : 0;
            break;
        case KO_ACT_LEAKY:
            gx = (y > 0) ? 1.0f : leaky_alpha;
            break;
        case KO_ACT_SIGMOID:
            gx = y * (1 - y);
            break;
        default: /* KO_ACT_TANH */
            gx = 1 - y * y;
            break;
        }
        pgx[n] = gx * gy;
    }
    return KO_OK;
}

/* ---- attention ------------------------------------------------------------------------------ */

int ko_mult_on_heads(float* pp, const float* pK, const float* pQ, int64_t nbat, int64_t ntimes, int64_t nvec,
                     int64_t nhead, int64_t npiece, const float* hCoef) {
    /* vmath.cu:6729-6750; probabilities laid out [nbat, ntimes(q), ntimes(k), nhead] */
    const float coef = hyper_value(hCoef);
    int64_t n = 0;
    for (int64_t nb = 0; nb < nbat; nb++) {
        for (int64_t nq = 0; nq < ntimes; nq++) {
            for (int64_t nk = 0; nk < ntimes; nk++) {
                for (int64_t nh = 0; nh < nhead; nh++, n++) {
                    const float* krow = pK + (nb * ntimes + nk) * nvec + nh * npiece;
                    const float* qrow = pQ + (nb * ntimes + nq) * nvec + nh * npiece;
                    float sum = 0.0f;
                    for (int64_t np = 0; np < npiece; np++) {
                        sum += krow[np] * qrow[np];
                    }
                    pp[n] = sum * coef;
                }
            }
        }
    }
    return KO_OK;
}

int ko_mult_on_heads_backward(float* pgQK, const float* pgp, const float* pKQ, int64_t nbat, int64_t ntimes,
                              int64_t nvec, int64_t nhead, int64_t npiece) {
    /* vmath.cu:6783-6802; the score gradient is always indexed [b, t, k, h] with t the row of
     * the output, for the key call and the query call alike */
    for (int64_t nb = 0; nb < nbat; nb++) {
        for (int64_t nt = 0; nt < ntimes; nt++) {
            for (int64_t nh = 0; nh < nhead; nh++) {
                for (int64_t np = 0; np < npiece; np++) {
                    float sum = 0.0f;
                    for (int64_t nk = 0; nk < ntimes; nk++) {
                        const int64_t kpos = (nb * ntimes + nk) * nvec + nh * npiece + np;
                        const int64_t ypos = ((nb * ntimes + nt) * ntimes + nk) * nhead + nh;
                        sum += pgp[ypos] * pKQ[kpos];
                    }
                    pgQK[(nb * ntimes + nt) * nvec + nh * npiece + np] = sum;
                }
            }
        }
    }
    return KO_OK;
}

int ko_set_mh_attention_mask(float* pp, int64_t ndat, int64_t ntimes, int64_t nhead, int forward) {
    /* vmath.cu:6833-6844 */
    for (int64_t nd = 0; nd < ndat; nd++) {
        for (int64_t nh = 0; nh < nhead; nh++) {
            for (int64_t nq = 0; nq < ntimes; nq++) {
                for (int64_t nk = nq + 1; nk < ntimes; nk++) {
                    pp[((nd * ntimes + nq) * ntimes + nk) * nhead + nh] = forward ? -INFINITY : 0;
                }
            }
        }
    }
    return KO_OK;
}

int ko_softmax_direct_on_axis(float* pp, int64_t nrow, int64_t nvec, int64_t ncol) {
    /* vmath.cu:6864-6885; in place, softmax over the middle axis of [nrow, nvec, ncol] */
    for (int64_t nr = 0; nr < nrow; nr++) {
        for (int64_t nc = 0; nc < ncol; nc++) {
            float* base = pp + nr * nvec * ncol + nc;
            float max_term = -FLT_MAX;
            float exp_sum = 0.0f;
            for (int64_t nv = 0; nv < nvec; nv++) {
                if (base[nv * ncol] > max_term) max_term = base[nv * ncol];
            }
            for (int64_t nv = 0; nv < nvec; nv++) {
                exp_sum += expf(base[nv * ncol] - max_term);
            }
            for (int64_t nv = 0; nv < nvec; nv++) {
                base[nv * ncol] = expf(base[nv * ncol] - max_term) / exp_sum;
            }
        }
    }
    return KO_OK;
}

int ko_softmax_direct_on_axis_backward(float* pgp, const float* pp, int64_t nbat, int64_t ntimes, int64_t nhead,
                                       const float* hCoef) {
    /* vmath.cu:6920-6942; in place on pgp */
    const float coef = hyper_value(hCoef);
    for (int64_t nb = 0; nb < nbat; nb++) {
        for (int64_t nq = 0; nq < ntimes; nq++) {
            for (int64_t nh = 0; nh < nhead; nh++) {
                const int64_t base = (nb * ntimes + nq) * ntimes * nhead + nh;
                float sum = 0.0f;
                for (int64_t nk = 0; nk < ntimes; nk++) {
                    sum += pp[base + nk * nhead] * pgp[base + nk * nhead];
                }
                for (int64_t nk = 0; nk < ntimes; nk++) {
                    const int64_t pos = base + nk * nhead;
                    pgp[pos] = coef * pp[pos] * (pgp[pos] - sum);
                }
            }
        }
    }
    return KO_OK;
}

int ko_mix_values(float* py, const float* pp, const float* pV, int64_t nbat, int64_t ntimes, int64_t nvec,
                  int64_t nhead, int64_t npiece) {
    /* vmath.cu:6977-6997 */
    for (int64_t nb = 0; nb < nbat; nb++) {
        for (int64_t nq = 0; nq < ntimes; nq++) {
            for (int64_t nh = 0; nh < nhead; nh++) {
                for (int64_t np = 0; np < npiece; np++) {
                    float sum = 0.0f;
                    for (int64_t nk = 0; nk < ntimes; nk++) {
                        const int64_t ppos = ((nb * ntimes + nq) * ntimes + nk) * nhead + nh;
                        const int64_t vpos = (nb * ntimes + nk) * nvec + nh * npiece + np;
                        sum += pp[ppos] * pV[vpos];
                    }
                    py[((nb * ntimes + nq) * nhead + nh) * npiece + np] = sum;
                }
            }
        }
    }
    return KO_OK;
}

int ko_mix_values_backward_prop(float* pgp, const float* pgy, const float* pV, int64_t nbat, int64_t ntimes,
                                int64_t nvec, int64_t nhead, int64_t npiece) {
    /* vmath.cu:7029-7049 */
    for (int64_t nb = 0; nb < nbat; nb++) {
        for (int64_t nq = 0; nq < ntimes; nq++) {
            for (int64_t nk = 0; nk < ntimes; nk++) {
                for (int64_t nh = 0; nh < nhead; nh++) {
                    float sum = 0.0f;
                    for (int64_t np = 0; np < npiece; np++) {
                        const int64_t ypos = ((nb * ntimes + nq) * nhead + nh) * npiece + np;
                        const int64_t vpos = (nb * ntimes + nk) * nvec + nh * npiece + np;
                        sum += pgy[ypos] * pV[vpos];
                    }
                    pgp[((nb * ntimes + nq) * ntimes + nk) * nhead + nh] = sum;
                }
            }
        }
    }
    return KO_OK;
}

int ko_mix_values_backward_value(float* pgV, const float* pgy, const float* pp, int64_t nbat, int64_t ntimes,
                                 int64_t nvec, int64_t nhead, int64_t npiece) {
    /* vmath.cu:7081-7101 */
    for (int64_t nb = 0; nb < nbat; nb++) {
        for (int64_t nk = 0; nk < ntimes; nk++) {
            for (int64_t nh = 0; nh < nhead; nh++) {
                for (int64_t np = 0; np < npiece; np++) {
                    float sum = 0.0f;
                    for (int64_t nq = 0; nq < ntimes; nq++) {
                        const int64_t ppos = ((nb * ntimes + nq) * ntimes + nk) * nhead + nh;
                        const int64_t ypos = ((nb * ntimes + nq) * nhead + nh) * npiece + np;
                        sum += pp[ppos] * pgy[ypos];
                    }
                    pgV[(nb * ntimes + nk) * nvec + nh * npiece + np] = sum;
                }
            }
        }
    }
    return KO_OK;
}

/* ---- parameter update (next to the path: what consumes dW and db) ------------------------------ */

#define KO_HYPER(h) ((h) ? *(h) : 0.0f)   /* HYPER_ACCESS, local_objects/vhypermanager.h:9 */

int ko_accumulate_grad(float* py, const float* px, int64_t ndat) {
    /* vmath.cu:364-368 */
    for (int64_t nd = 0; nd < ndat; nd++) {
        py[nd] += px[nd];
    }
    return KO_OK;
}

int ko_subtract_param_grad(float* pp, const float* pg, int64_t nrow, const float* hLearningRate) {
    /* vmath.cu:385-390 */
    float learningRate = KO_HYPER(hLearningRate);
    for (int64_t n = 0; n < nrow; n++) {
        pp[n] -= pg[n] * learningRate;
    }
    return KO_OK;
}

int ko_apply_decay(float* pd, const float* pp, const float* pg, int64_t nrow, const float* hL1Decay,
                   const float* hL2Decay) {
    /* vmath.cu:408-421 */
    float l1Decay = KO_HYPER(hL1Decay);
    float l2Decay = KO_HYPER(hL2Decay);
    for (int64_t n = 0; n < nrow; n++) {
        float delta = pg[n];
        if (l2Decay > 0) delta += l2Decay * pp[n];
        if (l1Decay > 0) delta += l1Decay * ((pp[n] > 0) ? 1 : ((pp[n] < 0) ? -1 : 0));
        pd[n] = delta;
    }
    return KO_OK;
}

int ko_eval_adam_delta(float* pa, const float* pg, float* ps, float* pt, float* pn, int64_t nrow, const float* hRo1,
                       const float* hRo2, const float* hEpsilon) {
    /* vmath.cu:449-468 */
    float ro1 = KO_HYPER(hRo1);
    float ro2 = KO_HYPER(hRo2);
    float epsilon = KO_HYPER(hEpsilon);
    for (int64_t n = 0; n < nrow; n++) {
        float delta = pg[n];
        float nstep = pn[n] + 1;
        ps[n] = ro1 * ps[n] + (1 - ro1) * delta;
        pt[n] = ro2 * pt[n] + (1 - ro2) * delta * delta;
        float sterm = ps[n] / (1 - powf(ro1, nstep));
        float tterm = pt[n] / (1 - powf(ro2, nstep));
        pa[n] = sterm / (sqrtf(tterm) + epsilon);
        pn[n] = nstep;
    }
    return KO_OK;
}

/* ---- transposes (next to the path) ------------------------------------------------------------------ */

int ko_transpose(float* py, const float* px, const int* pn, int64_t axis_size, int64_t data_size) {
    /* vmath.cu:9384-9403.  pn[m*3] = source axis of output axis m, pn[m*3+1] = elements per step of output
       axis m, pn[a*3+2] = elements per step of SOURCE axis a (vtensor.cpp:5399-5417) */
    for (int64_t n = 0; n < data_size; n++) {
        int64_t xpos = 0;
        int64_t ypos = n;
        int64_t cood;
        for (int64_t m = 0; m < axis_size; m++) {
            int64_t y_block_size = pn[m * 3 + 1];
            int64_t x_block_size = pn[pn[m * 3] * 3 + 2];
            cood = ypos / y_block_size;
            ypos = ypos % y_block_size;
            xpos += cood * x_block_size;
        }
        py[n] = px[xpos];
    }
    return KO_OK;
}

int ko_transpose_backward(float* pgx, const float* pgy, const int* pn, int64_t axis_size, int64_t data_size) {
    /* vmath.cu:9436-9455 */
    for (int64_t n = 0; n < data_size; n++) {
        int64_t xpos = 0;
        int64_t ypos = n;
        int64_t cood;
        for (int64_t m = 0; m < axis_size; m++) {
            int64_t y_block_size = pn[m * 3 + 1];
            int64_t x_block_size = pn[pn[m * 3] * 3 + 2];
            cood = ypos / y_block_size;
            ypos = ypos % y_block_size;
            xpos += cood * x_block_size;
        }
        pgx[xpos] = pgy[n];
    }
    return KO_OK;
}

int ko_transpose_bin(float* py, const float* px, int64_t nrow, int64_t ncol) {
    /* vmath.cu:9487-9494 */
    for (int64_t nr = 0, n = 0; nr < nrow; nr++) {
        for (int64_t nc = 0; nc < ncol; nc++, n++) {
            int64_t xpos = nc * nrow + nr;
            py[n] = px[xpos];
        }
    }
    return KO_OK;
}

/* ---- recurrent cells: what runs between the gate products of an RNN/LSTM/GRU step ----------- */

int ko_copy(float* py, const float* pa, int64_t ndat) {
    /* vmath.cu:732-736 */
    for (int64_t n = 0; n < ndat; n++) py[n] = pa[n];
    return KO_OK;
}

int ko_add(float* py, const float* pa, const float* pb, int64_t ndat) {
    /* vmath.cu:774-778 */
    for (int64_t nd = 0; nd < ndat; nd++) py[nd] = pa[nd] + pb[nd];
    return KO_OK;
}

int ko_lstm_process(float* pr, float* ps, const float* ps1, const float* pa, int64_t ndat, int64_t nrec) {
    /* vmath.cu:4807-4826; gate order in pa[ndat, 4*nrec]: input, forget, block, output */
    for (int64_t nd = 0, n = 0; nd < ndat; nd++) {
        for (int64_t nr = 0; nr < nrec; nr++, n++) {
            int64_t apos = nd * 4 * nrec + nr;
            float state = ps1 ? ps1[n] : 0;
            float input_gate = ko_sigmoid(pa[apos + 0 * nrec]);
            float forget_gate = ko_sigmoid(pa[apos + 1 * nrec]);
            float input_block = ko_tanh(pa[apos + 2 * nrec]);
            float output_gate = ko_sigmoid(pa[apos + 3 * nrec]);
            float new_state = state * forget_gate + input_block * input_gate;
            float new_recur = ko_tanh(new_state) * output_gate;
            ps[n] = new_state;
            pr[n] = new_recur;
        }
    }
    return KO_OK;
}

int ko_lstm_process_backward(const float* pgr, float* pgs, float* pga, const float* ps, const float* pa,
                             int64_t ndat, int64_t nrec) {
    /* vmath.cu:4899-4937, the DEVICE twin: gate gradients at pga[apos + g * nrec].  The host twin
     * (vmath.cu:4860-4897) has the same arithmetic but writes them at pga[apos * g + n * nrec], which
     * leaves the [ndat, 4*nrec] buffer; the library replaces the device branch, so that is the one
     * restated.  ps is the state of the step processed BEFORE this one (null: 0), pa the gate sums of
     * this step, pgr the gradient of this step's output (read only), pgs the gradient of this step's
     * state on entry and of the previous state on return. */
    for (int64_t nd = 0, n = 0; nd < ndat; nd++) {
        for (int64_t nr = 0; nr < nrec; nr++, n++) {
            int64_t apos = nd * 4 * nrec + nr;
            float old_state = ps ? ps[n] : 0;
            float input_gate = ko_sigmoid(pa[apos + 0 * nrec]);
            float forget_gate = ko_sigmoid(pa[apos + 1 * nrec]);
            float input_block = ko_tanh(pa[apos + 2 * nrec]);
            float output_gate = ko_sigmoid(pa[apos + 3 * nrec]);
            float new_state = old_state * forget_gate + input_block * input_gate;
            float g_new_recur = pgr[n];
            float g_output_gate = ko_tanh(new_state) * g_new_recur;
            float g_tanh_state = output_gate * g_new_recur;
            float th = ko_tanh(new_state);                       /* _tanh_derv_with_x, vmath.cu:336-339 */
            float g_new_state = (1.0f - th * th) * g_tanh_state + pgs[n];
            float g_forget_gate = old_state * g_new_state;
            float g_old_state = forget_gate * g_new_state;
            float g_input_block = input_gate * g_new_state;
            float g_input_gate = input_block * g_new_state;
            /* _sigmoid_derv_with_y: y * (1 - y); _tanh_derv_with_y: 1 - y * y (vmath.cu:327-347) */
            pga[apos + 0 * nrec] = input_gate * (1.0f - input_gate) * g_input_gate;
            pga[apos + 1 * nrec] = forget_gate * (1.0f - forget_gate) * g_forget_gate;
            pga[apos + 2 * nrec] = (1.0f - input_block * input_block) * g_input_block;
            pga[apos + 3 * nrec] = output_gate * (1.0f - output_gate) * g_output_gate;
            pgs[n] = g_old_state;
        }
    }
    return KO_OK;
}

int ko_gru_process(float* pr, const float* pai, const float* par, int64_t nt, int64_t ndat, int64_t nrec) {
    /* vmath.cu:4946-4965; pr points at time step nt of [ntimes, ndat, nrec], the previous step lies ndat*nrec
     * floats before it; gate order in pai/par[ndat, 3*nrec]: reset, update, candidate */
    for (int64_t nd = 0; nd < ndat; nd++) {
        for (int64_t ny = 0; ny < nrec; ny++) {
            int64_t rpos = nd * nrec + ny;
            int64_t rgpos = nd * 3 * nrec + ny;
            int64_t zgpos = nd * 3 * nrec + nrec + ny;
            int64_t ngpos = nd * 3 * nrec + 2 * nrec + ny;
            float Rt = ko_sigmoid(pai[rgpos] + par[rgpos]);
            float Zt = ko_sigmoid(pai[zgpos] + par[zgpos]);
            float Nt = ko_tanh(pai[ngpos] + Rt * par[ngpos]);
            float Ht = (nt > 0) ? pr[rpos - ndat * nrec] : 0;
            pr[rpos] = (1.0f - Zt) * Nt + Zt * Ht;
        }
    }
    return KO_OK;
}

int ko_gru_process_backward(float* pgr, float* pgai, float* pgar, const float* pr, const float* pai,
                            const float* par, int64_t nt, int64_t ndat, int64_t nrec) {
    /* vmath.cu:4999-5033 */
    for (int64_t nd = 0; nd < ndat; nd++) {
        for (int64_t ny = 0; ny < nrec; ny++) {
            int64_t rpos = nd * nrec + ny;
            int64_t rgpos = nd * 3 * nrec + ny;
            int64_t zgpos = nd * 3 * nrec + nrec + ny;
            int64_t ngpos = nd * 3 * nrec + 2 * nrec + ny;
            float Rt = ko_sigmoid(pai[rgpos] + par[rgpos]);
            float Zt = ko_sigmoid(pai[zgpos] + par[zgpos]);
            float Nt = ko_tanh(pai[ngpos] + Rt * par[ngpos]);
            float Ht_1 = (nt > 0) ? pr[rpos - ndat * nrec] : 0;
            float gHt = pgr[rpos];
            float gNt = (1 - Zt) * gHt;
            float gZt = (Ht_1 - Nt) * gHt;
            float gHt_1 = Zt * gHt;
            float gNt_seed = (1 + Nt) * (1 - Nt) * gNt;
            float gRt = par[ngpos] * gNt_seed;
            pgai[rgpos] = pgar[rgpos] = Rt * (1 - Rt) * gRt;
            pgai[zgpos] = pgar[zgpos] = Zt * (1 - Zt) * gZt;
            pgai[ngpos] = gNt_seed;
            pgar[ngpos] = Rt * gNt_seed;
            pgr[rpos] = gHt_1;
        }
    }
    return KO_OK;
}

/* ---- cosine similarity of every row pair ------------------------------------------------------ */

int ko_cosinesim(float* py, const float* px1, const float* px2, int64_t nrow1, int64_t nrow2, int64_t ncol) {
    /* vmath.cu:6459-6480 */
    for (int64_t nr1 = 0, n = 0; nr1 < nrow1; nr1++) {
        for (int64_t nr2 = 0; nr2 < nrow2; nr2++, n++) {
            float aa_sum = 0;
            float bb_sum = 0;
            float ab_sum = 0;
            for (int64_t nc = 0; nc < ncol; nc++) {
                float a = px1[nr1 * ncol + nc];
                float b = px2[nr2 * ncol + nc];
                aa_sum += a * a;
                bb_sum += b * b;
                ab_sum += a * b;
            }
            py[n] = ab_sum / (sqrtf(aa_sum) * sqrtf(bb_sum) + 1e-20f);
        }
    }
    return KO_OK;
}
