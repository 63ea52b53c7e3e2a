// Skinny products (at most 16 rows of X): bandwidth-bound wavefront-reduction GEMV.
//
//   y[m,n] (=|+=) act( sum_k x[m,k] * w[n,k] + bias[n] ),   m < M <= 16
//
// This is VMath::matmul (vmath.cu:2961-3003 of the reference) at batch sizes where
// the weight matrix is read once and everything else is noise: the kernel is a
// stream over W.  Each wave owns R rows of W and walks them with 128-bit loads, 64
// lanes wide (1 KiB per row per step, fully coalesced); the M rows of X for the
// current K chunk sit in LDS ([m][k], conflict-free 128-bit reads); every lane keeps
// M*R partial sums that are folded across the wave at the end.  No MFMA: at
// M <= 16 the matrix cores would idle behind HBM anyway.
#include "gemv_skinny.h"

#include "act_funcs.h"

namespace kai {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSkinnyLdsFloats = 16384;   // 64 KiB of X per block
constexpr int kSkinnyThreads = 256;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <int MT, int R, bool VEC>
__global__ void __launch_bounds__(kSkinnyThreads) skinny_nt_kernel(const SkinnyParams p) {
    constexpr int KCH = kSkinnyLdsFloats / MT;   // K chunk held in LDS
    constexpr int STEP = VEC ? 256 : 64;         // k covered by one wave step
    __shared__ __attribute__((aligned(16))) float xs[kSkinnyLdsFloats];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t n0 = ((int64_t)blockIdx.x * (kSkinnyThreads / 64) + wave) * R;

    float acc[MT][R];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[m][r] = 0.f;

    const float* __restrict__ wrow[R];
    bool rvalid[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        rvalid[r] = (n0 + r) < p.N;
        wrow[r] = p.W + (rvalid[r] ? (n0 + r) : 0) * p.ldw;
    }

    for (int kc0 = 0; kc0 < p.K; kc0 += KCH) {
        const int kc_len = min(KCH, p.K - kc0);
        if (kc0 > 0) __syncthreads();
        // stage x[:, kc0 : kc0+kc_len] (rows beyond M as zeros)
        if (VEC) {
            for (int m = 0; m < MT; m++) {
                for (int k = tid * 4; k < kc_len; k += kSkinnyThreads * 4) {
                    f32x4 v = {0.f, 0.f, 0.f, 0.f};
                    if (m < p.M) v = *reinterpret_cast<const f32x4*>(p.X + (int64_t)m * p.ldx + kc0 + k);
                    *reinterpret_cast<f32x4*>(&xs[m * KCH + k]) = v;
                }
            }
        } else {
            for (int m = 0; m < MT; m++)
                for (int k = tid; k < kc_len; k += kSkinnyThreads)
                    xs[m * KCH + k] = (m < p.M) ? p.X[(int64_t)m * p.ldx + kc0 + k] : 0.f;
        }
        __syncthreads();

        if (VEC) {
#pragma unroll 4
            for (int k = lane * 4; k < kc_len; k += STEP) {
                f32x4 w[R];
#pragma unroll
                for (int r = 0; r < R; r++) w[r] = *reinterpret_cast<const f32x4*>(wrow[r] + kc0 + k);
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const f32x4 x = *reinterpret_cast<const f32x4*>(&xs[m * KCH + k]);
#pragma unroll
                    for (int r = 0; r < R; r++)
                        acc[m][r] += w[r][0] * x[0] + w[r][1] * x[1] + w[r][2] * x[2] + w[r][3] * x[3];
                }
            }
        } else {
#pragma unroll 4
            for (int k = lane; k < kc_len; k += STEP) {
                float w[R];
#pragma unroll
                for (int r = 0; r < R; r++) w[r] = wrow[r][kc0 + k];
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const float x = xs[m * KCH + k];
#pragma unroll
                    for (int r = 0; r < R; r++) acc[m][r] += w[r] * x;
                }
            }
        }
    }

    const float leaky = p.leaky ? *p.leaky : 0.f;
#pragma unroll
    for (int m = 0; m < MT; m++) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            float v = wave_sum(acc[m][r]);
            if (lane == ((m * R + r) & 63) && m < p.M && rvalid[r]) {
                const int64_t n = n0 + r;
                const int64_t idx = (int64_t)m * p.ldy + n;
                if (p.accflag) v += p.Y[idx];
                if (p.bias) v += p.bias[n];
                if (p.Y2) p.Y2[idx] = v;
                p.Y[idx] = apply_act(v, p.act, leaky);
            }
        }
    }
}

template <int MT, bool VEC>
static int launch_mt(const SkinnyParams& p, hipStream_t stream) {
    constexpr int R = 2;
    const int64_t rows_per_block = (kSkinnyThreads / 64) * R;
    const int64_t blocks = (p.N + rows_per_block - 1) / rows_per_block;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: too many output columns");
    skinny_nt_kernel<MT, R, VEC><<<dim3((unsigned)blocks), dim3(kSkinnyThreads), 0, stream>>>(p);
    return check_launch("skinny_nt_kernel");
}

template <bool VEC>
static int launch_vec(const SkinnyParams& p, hipStream_t stream) {
    if (p.M <= 1) return launch_mt<1, VEC>(p, stream);
    if (p.M <= 2) return launch_mt<2, VEC>(p, stream);
    if (p.M <= 4) return launch_mt<4, VEC>(p, stream);
    if (p.M <= 8) return launch_mt<8, VEC>(p, stream);
    return launch_mt<16, VEC>(p, stream);
}

int launch_skinny_nt(const SkinnyParams& p, hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0) return KAI_OK;
    if (p.M > kSkinnyMaxRows) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: more than 16 rows");
    const bool vec = p.K % 4 == 0 && p.ldw % 4 == 0 && p.ldx % 4 == 0 && aligned16(p.W) && aligned16(p.X);
    return vec ? launch_vec<true>(p, stream) : launch_vec<false>(p, stream);
}

}  // namespace kai
