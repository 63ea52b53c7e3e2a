// Bandwidth-bound pieces of the attention layer: causal mask, softmax over the key
// axis of the head-interleaved score tensor [nrow, nvec, ncol] (ncol = heads, innermost), and
// its backward.  Reference: VMath::set_mh_attention_mask (vmath.cu:6833-6860),
// softmax_direct_on_axis (vmath.cu:6864-6916), softmax_direct_on_axis_backward
// (vmath.cu:6920-6973).
//
// The data of one outer row (nvec*ncol floats) is contiguous.  Three access plans keep every
// global access coalesced whatever the head count:
//   ncol == 1        one wave per row, lanes stride the row
//   2..128 heads     one workgroup per outer row; thread t walks elements t, t+TB, ... with TB a
//                    multiple of ncol, so a thread always sees the same head; per-head partials
//                    meet in LDS
//   > 128 heads      one thread per (row, head); neighbouring threads touch neighbouring heads
// The row stays in L1/L2 between the max, sum and write passes, so HBM sees one read and one
// write per element.
#include <float.h>

#include "elementwise.h"

namespace kai {

constexpr int kTB = 256;
typedef float f32x4s __attribute__((ext_vector_type(4)));

// Wave-wide reductions through the DPP data path (result in every lane); see gemv_skinny.hip for
// the sequence.  For the maximum, lanes that a row-masked broadcast step does not write keep their
// own value (old = v), which leaves the maximum unchanged.
#define KAI_DPP(old, v, ctrl, rmask) \
    __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, (old)), __builtin_bit_cast(int, (v)), (ctrl), (rmask), 0xf, false))
__device__ __forceinline__ float wmax(float v) {
    v = fmaxf(v, KAI_DPP(v, v, 0xB1, 0xf));
    v = fmaxf(v, KAI_DPP(v, v, 0x4E, 0xf));
    v = fmaxf(v, KAI_DPP(v, v, 0x141, 0xf));
    v = fmaxf(v, KAI_DPP(v, v, 0x140, 0xf));
    v = fmaxf(v, KAI_DPP(v, v, 0x142, 0xa));
    v = fmaxf(v, KAI_DPP(v, v, 0x143, 0xc));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wsum(float v) {
    v += KAI_DPP(0.f, v, 0xB1, 0xf);
    v += KAI_DPP(0.f, v, 0x4E, 0xf);
    v += KAI_DPP(0.f, v, 0x141, 0xf);
    v += KAI_DPP(0.f, v, 0x140, 0xf);
    v += KAI_DPP(0.f, v, 0x142, 0xa);
    v += KAI_DPP(0.f, v, 0x143, 0xc);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// ---- mask -------------------------------------------------------------------------------------

// The masked elements of a query's row are one contiguous run: keys q + 1 .. T - 1 of every head.  A wave per row
// fills it, 128-bit words between its unaligned ends (one thread per element of the WHOLE tensor with two 64-bit
// divisions each took 20 us for 32 x 512 x 512, of which half is written).
__global__ void __launch_bounds__(kTB) attention_mask_kernel(float* __restrict__ pp, int64_t nrows, int64_t ntimes,
                                                             int64_t nhead, int forward, int aligned) {
    const float fillv = forward ? -INFINITY : 0.f;
    const int lane = threadIdx.x & 63;
    const int64_t nwaves = (int64_t)gridDim.x * (kTB / 64);
    for (int64_t row = (int64_t)blockIdx.x * (kTB / 64) + (threadIdx.x >> 6); row < nrows; row += nwaves) {
        const int64_t q = row % ntimes;
        const int64_t start = (row * ntimes + q + 1) * nhead, end = (row + 1) * ntimes * nhead;
        if (!aligned) {
            for (int64_t i = start + lane; i < end; i += 64) pp[i] = fillv;
            continue;
        }
        const int64_t first = min(end, (start + 3) & ~(int64_t)3), last = max(first, end & ~(int64_t)3);
        if (start + lane < first) pp[start + lane] = fillv;
        const f32x4s w = {fillv, fillv, fillv, fillv};
        for (int64_t i = first + 4 * lane; i < last; i += 256) *reinterpret_cast<f32x4s*>(pp + i) = w;
        if (last + lane < end) pp[last + lane] = fillv;
    }
}

int launch_attention_mask(float* pp, int64_t ndat, int64_t ntimes, int64_t nhead, int forward, hipStream_t stream) {
    const int64_t nrows = ndat * ntimes;
    if (nrows <= 0 || ntimes * nhead <= 0) return KAI_OK;
    int64_t blocks = (nrows + kTB / 64 - 1) / (kTB / 64);
    if (blocks > 256 * 32) blocks = 256 * 32;
    const int aligned = (reinterpret_cast<uintptr_t>(pp) & 15u) == 0;
    attention_mask_kernel<<<dim3((unsigned)blocks), kTB, 0, stream>>>(pp, nrows, ntimes, nhead, forward, aligned);
    return check_launch("attention_mask_kernel");
}

// ---- softmax over the middle axis ---------------------------------------------------------------
// BACKWARD = false: p <- softmax(p) in place.
// BACKWARD = true : g <- coef * p * (g - sum_k p*g) in place on g.

template <bool BACKWARD>
__global__ void __launch_bounds__(kTB) softmax_axis_wave_kernel(float* __restrict__ io, const float* __restrict__ pp,
                                                                int64_t nrow, int64_t nvec,
                                                                const float* __restrict__ hcoef) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kTB / 64) + (threadIdx.x >> 6);
    if (row >= nrow) return;
    float* __restrict__ r = io + row * nvec;
    if (!BACKWARD) {
        float mx = -FLT_MAX;
        for (int64_t v = lane; v < nvec; v += 64) mx = fmaxf(mx, r[v]);
        mx = wmax(mx);
        float sum = 0.f;
        for (int64_t v = lane; v < nvec; v += 64) sum += expf(r[v] - mx);
        sum = wsum(sum);
        for (int64_t v = lane; v < nvec; v += 64) r[v] = expf(r[v] - mx) / sum;
    } else {
        const float coef = hcoef ? *hcoef : 0.f;
        const float* __restrict__ p = pp + row * nvec;
        float dot = 0.f;
        for (int64_t v = lane; v < nvec; v += 64) dot += p[v] * r[v];
        dot = wsum(dot);
        for (int64_t v = lane; v < nvec; v += 64) r[v] = coef * p[v] * (r[v] - dot);
    }
}

template <bool BACKWARD>
__global__ void __launch_bounds__(kTB) softmax_axis_block_kernel(float* __restrict__ io,
                                                                 const float* __restrict__ pp, int64_t nvec,
                                                                 int ncol, int tb, const float* __restrict__ hcoef) {
    __shared__ float red[kTB];
    const int t = threadIdx.x;
    const int64_t len = nvec * ncol;
    float* __restrict__ r = io + (int64_t)blockIdx.x * len;
    const bool active = t < tb;   // tb = ncol * floor(kTB / ncol): a thread keeps one head
    const int c = t % ncol;

    // folds the per-thread values of all threads that own head c, in thread order
    auto fold = [&](float mine, bool is_max) -> float {
        __syncthreads();
        red[t] = mine;
        __syncthreads();
        float a = is_max ? -FLT_MAX : 0.f;
        for (int u = c; u < tb; u += ncol) a = is_max ? fmaxf(a, red[u]) : a + red[u];
        return a;
    };

    if (!BACKWARD) {
        float mx = -FLT_MAX;
        if (active)
            for (int64_t e = t; e < len; e += tb) mx = fmaxf(mx, r[e]);
        mx = fold(mx, true);
        float sum = 0.f;
        if (active)
            for (int64_t e = t; e < len; e += tb) sum += expf(r[e] - mx);
        sum = fold(sum, false);
        if (active)
            for (int64_t e = t; e < len; e += tb) r[e] = expf(r[e] - mx) / sum;
    } else {
        const float coef = hcoef ? *hcoef : 0.f;
        const float* __restrict__ p = pp + (int64_t)blockIdx.x * len;
        float dot = 0.f;
        if (active)
            for (int64_t e = t; e < len; e += tb) dot += p[e] * r[e];
        dot = fold(dot, false);
        if (active)
            for (int64_t e = t; e < len; e += tb) r[e] = coef * p[e] * (r[e] - dot);
    }
}

// ncol == 1, row length a multiple of 4 and at most 64*4*NV4: the whole row lives in registers
// (NV4 float4 per lane), so HBM sees exactly one 128-bit read and one 128-bit write per element.

// v where keep, else `other` in every element.  Bitwise on purpose: with a select the compiler moves
// the load that produced v under the condition, and a conditional load is waited for before the next
// load is issued.
__device__ __forceinline__ f32x4s keep_or(f32x4s v, bool keep, float other) {
    const int m = keep ? -1 : 0;
    const int o = __float_as_int(other) & ~m;
    f32x4s r;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float e = v[j];
        r[j] = __int_as_float((__float_as_int(e) & m) | o);
    }
    return r;
}

// exp(d) for d <= 0 in the register-resident row kernels: one multiply and the hardware's 2^x.  The rounding of
// d * log2(e) costs a relative 6e-8 * |d| in the result, i.e. nothing for the entries that carry the row's
// weight (d near 0); the library routine's range reduction and the eight full divisions per lane were a third
// of these kernels' run time.  -inf gives 0, results below the normal range are flushed to 0.
__device__ __forceinline__ float exp_nonpositive(float d) { return __builtin_amdgcn_exp2f(d * 1.44269504088896341f); }

// the same element by element (a word that straddles the end of its row)
__device__ __forceinline__ f32x4s keep_each_or(f32x4s v, int k, int nvec, float other) {
    f32x4s r;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int m = k + j < nvec ? -1 : 0;
        const float e = v[j];
        r[j] = __int_as_float((__float_as_int(e) & m) | (__float_as_int(other) & ~m));
    }
    return r;
}

// UNAL: rows of any length at any 4-byte alignment (511 keys).  The 128-bit loads are buffer loads, which need no
// more than that; the word that straddles the end of a row brings the next row's first elements (zeros behind the
// last row: the buffer ends with the tensor), masked element by element, and is stored element by element, the
// words before it as 128-bit buffer stores.  (Three passes of 32-bit accesses before: 32 x 511 x 511 20.8 us where
// 512 keys take 8.3.)
template <bool BACKWARD, int NV4, bool UNAL = false>
__global__ void __launch_bounds__(kTB) softmax_axis_wave_reg_kernel(float* __restrict__ io,
                                                                    const float* __restrict__ pp, int64_t nrow,
                                                                    int nvec, const float* __restrict__ hcoef) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kTB / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (kTB / 64);
    const float coef = (BACKWARD && hcoef) ? *hcoef : 0.f;
    auto row_resource = [&](const float* base, int64_t row) -> __amdgpu_buffer_rsrc_t {
        const uint64_t a = reinterpret_cast<uint64_t>(base + row * nvec);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        const int64_t bytes = (nrow - row) * nvec * 4;
        const int ext = __builtin_amdgcn_readfirstlane((int)(bytes < 0x7FFFFFFF ? bytes : 0x7FFFFFFF));
        return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<float*>(((uint64_t)hi << 32) | lo), 0, ext, 0x00020000);
    };
    for (int64_t row = wave; row < nrow; row += nwaves) {
        float* __restrict__ r = io + row * nvec;
        f32x4s v[NV4];
        __amdgpu_buffer_rsrc_t rs_io;
        if (UNAL) rs_io = row_resource(io, row);
#pragma unroll
        for (int i = 0; i < NV4; i++) {
            const int k = 4 * lane + 256 * i;   // loads are unconditional (clamped), padding is masked below
            if (UNAL) {
                v[i] = __builtin_bit_cast(f32x4s, __builtin_amdgcn_raw_buffer_load_b128(rs_io, k * 4, 0, 0));
                continue;
            }
            // forward: rows that come straight from HBM gain 7 % from the non-temporal hint (14.5 -> 13.5 us for
            // 16384 rows of 512), rows still in the last-level cache lose nothing; backward it costs 1 us there
            const f32x4s* src = reinterpret_cast<const f32x4s*>(r + min(k, nvec - 4));
            v[i] = BACKWARD ? *src : __builtin_nontemporal_load(src);
        }
        f32x4s q[NV4];   // backward only
        if (BACKWARD) {
            const float* __restrict__ pr = pp + row * nvec;
            __amdgpu_buffer_rsrc_t rs_p;
            if (UNAL) rs_p = row_resource(pp, row);
#pragma unroll
            for (int i = 0; i < NV4; i++) {
                const int k = 4 * lane + 256 * i;
                if (UNAL) q[i] = __builtin_bit_cast(f32x4s, __builtin_amdgcn_raw_buffer_load_b128(rs_p, k * 4, 0, 0));
                else q[i] = *reinterpret_cast<const f32x4s*>(pr + min(k, nvec - 4));
            }
        }
        // a word of the row: 128 bits at once, or element by element where it straddles the row's end
        auto store_word = [&](int k, f32x4s w) {
            if (!UNAL) {
                if (k < nvec) *reinterpret_cast<f32x4s*>(r + k) = w;
            } else if (k + 4 <= nvec) {
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int, w), rs_io, k * 4, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j < 3; j++)
                    if (k + j < nvec) r[k + j] = w[j];
            }
        };
#pragma unroll
        for (int i = 0; i < NV4; i++)
            v[i] = UNAL ? keep_each_or(v[i], 4 * lane + 256 * i, nvec, BACKWARD ? 0.f : -INFINITY)
                        : keep_or(v[i], 4 * lane + 256 * i < nvec, BACKWARD ? 0.f : -INFINITY);
        if (!BACKWARD) {
            float mx = -FLT_MAX;
#pragma unroll
            for (int i = 0; i < NV4; i++) mx = fmaxf(mx, fmaxf(fmaxf(v[i][0], v[i][1]), fmaxf(v[i][2], v[i][3])));
            mx = wmax(mx);
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < NV4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    v[i][j] = exp_nonpositive(v[i][j] - mx);   // padding lanes hold -inf: exp gives 0
                    sum += v[i][j];
                }
            const float inv = 1.0f / wsum(sum);
#pragma unroll
            for (int i = 0; i < NV4; i++) store_word(4 * lane + 256 * i, v[i] * inv);
        } else {
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < NV4; i++) {
                q[i] = UNAL ? keep_each_or(q[i], 4 * lane + 256 * i, nvec, 0.f) : keep_or(q[i], 4 * lane + 256 * i < nvec, 0.f);
                dot += q[i][0] * v[i][0] + q[i][1] * v[i][1] + q[i][2] * v[i][2] + q[i][3] * v[i][3];
            }
            dot = wsum(dot);
#pragma unroll
            for (int i = 0; i < NV4; i++) store_word(4 * lane + 256 * i, coef * q[i] * (v[i] - dot));
        }
    }
}

// 2..128 heads, outer row (nvec*ncol floats) at most kTB*EMAX long: each thread keeps its EMAX
// elements (all of one head) in registers between the passes.
template <bool BACKWARD, int EMAX>
__global__ void __launch_bounds__(kTB) softmax_axis_block_reg_kernel(float* __restrict__ io,
                                                                     const float* __restrict__ pp, int64_t nvec,
                                                                     int ncol, int tb,
                                                                     const float* __restrict__ hcoef) {
    __shared__ float red[kTB];
    const int t = threadIdx.x;
    const int len = (int)(nvec * ncol);
    float* __restrict__ r = io + (int64_t)blockIdx.x * len;
    const bool active = t < tb;
    const int c = t % ncol;
    auto fold = [&](float mine, bool is_max) -> float {
        __syncthreads();
        red[t] = mine;
        __syncthreads();
        float a = is_max ? -FLT_MAX : 0.f;
        for (int u = c; u < tb; u += ncol) a = is_max ? fmaxf(a, red[u]) : a + red[u];
        return a;
    };
    float v[EMAX];
#pragma unroll
    for (int i = 0; i < EMAX; i++) {
        const int e = t + i * tb;
        v[i] = (active && e < len) ? r[e] : -INFINITY;
    }
    if (!BACKWARD) {
        float mx = -FLT_MAX;
#pragma unroll
        for (int i = 0; i < EMAX; i++) mx = fmaxf(mx, v[i]);
        mx = fold(mx, true);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < EMAX; i++) {
            v[i] = expf(v[i] - mx);
            sum += v[i];
        }
        sum = fold(sum, false);
#pragma unroll
        for (int i = 0; i < EMAX; i++) {
            const int e = t + i * tb;
            if (active && e < len) r[e] = v[i] / sum;
        }
    } else {
        const float coef = hcoef ? *hcoef : 0.f;
        const float* __restrict__ p = pp + (int64_t)blockIdx.x * len;
        float q[EMAX];
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < EMAX; i++) {
            const int e = t + i * tb;
            q[i] = (active && e < len) ? p[e] : 0.f;
            if (active && e < len) dot += q[i] * v[i];
        }
        dot = fold(dot, false);
#pragma unroll
        for (int i = 0; i < EMAX; i++) {
            const int e = t + i * tb;
            if (active && e < len) r[e] = coef * q[i] * (v[i] - dot);
        }
    }
}

// 4, 8, 16, ... 128 heads (a multiple of 4 whose quarter is a power of two), outer row (nvec*ncol
// floats) at most 4*kTB*VN long: a thread keeps VN 128-bit chunks, each the same four heads of one
// position, so that HBM sees one 128-bit read and one 128-bit write per four elements.  The four heads
// are four independent reductions per thread; threads of one head group (t % G, G = ncol / 4) meet by
// a butterfly over the lanes of a wave and one exchange through LDS.
template <bool BACKWARD, int VN>
__global__ void __launch_bounds__(kTB) softmax_axis_heads4_kernel(float* __restrict__ io,
                                                                  const float* __restrict__ pp, int64_t nvec,
                                                                  int ncol, const float* __restrict__ hcoef) {
    __shared__ f32x4s red[2][kTB / 64][32];
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = t >> 6;
    const int G = ncol >> 2;        // head groups: a power of two, at most 32
    const int g = t & (G - 1);
    const int len4 = (int)(nvec * ncol) >> 2;   // chunks in the row
    float* __restrict__ r = io + (int64_t)blockIdx.x * (nvec * ncol);

    // reduction over the threads of a head group, per component; `which` alternates the LDS buffer
    auto fold = [&](f32x4s mine, bool is_max, int which) -> f32x4s {
        for (int m = G; m < 64; m <<= 1) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float o = __shfl_xor(mine[j], m);
                mine[j] = is_max ? fmaxf(mine[j], o) : mine[j] + o;
            }
        }
        if (lane < G) red[which][wave][lane] = mine;
        __syncthreads();
        f32x4s a = red[which][0][g];
#pragma unroll
        for (int w = 1; w < kTB / 64; w++) {
            const f32x4s b = red[which][w][g];
#pragma unroll
            for (int j = 0; j < 4; j++) a[j] = is_max ? fmaxf(a[j], b[j]) : a[j] + b[j];
        }
        return a;
    };

    f32x4s v[VN], q[VN];
#pragma unroll
    for (int i = 0; i < VN; i++) v[i] = *reinterpret_cast<const f32x4s*>(r + 4 * min(t + i * kTB, len4 - 1));
    if (BACKWARD) {
        const float* __restrict__ p = pp + (int64_t)blockIdx.x * (nvec * ncol);
#pragma unroll
        for (int i = 0; i < VN; i++) q[i] = *reinterpret_cast<const f32x4s*>(p + 4 * min(t + i * kTB, len4 - 1));
    }
#pragma unroll
    for (int i = 0; i < VN; i++) v[i] = keep_or(v[i], t + i * kTB < len4, BACKWARD ? 0.f : -INFINITY);

    if (!BACKWARD) {
        f32x4s mx = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
#pragma unroll
        for (int i = 0; i < VN; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) mx[j] = fmaxf(mx[j], v[i][j]);
        mx = fold(mx, true, 0);
        f32x4s sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VN; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[i][j] = exp_nonpositive(v[i][j] - mx[j]);   // padding holds -inf: exp gives 0
                sum[j] += v[i][j];
            }
        sum = fold(sum, false, 1);
        f32x4s inv;
#pragma unroll
        for (int j = 0; j < 4; j++) inv[j] = 1.0f / sum[j];
#pragma unroll
        for (int i = 0; i < VN; i++)
            if (t + i * kTB < len4) *reinterpret_cast<f32x4s*>(r + 4 * (t + i * kTB)) = v[i] * inv;
    } else {
        const float coef = hcoef ? *hcoef : 0.f;
        f32x4s dot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VN; i++) {
            q[i] = keep_or(q[i], t + i * kTB < len4, 0.f);
            dot += q[i] * v[i];
        }
        dot = fold(dot, false, 0);
#pragma unroll
        for (int i = 0; i < VN; i++)
            if (t + i * kTB < len4) *reinterpret_cast<f32x4s*>(r + 4 * (t + i * kTB)) = coef * q[i] * (v[i] - dot);
    }
}

// The same layout with a whole outer row per WAVE (rows of at most 64 * VN chunks, i.e. 4096 floats for VN = 16):
// lane l keeps chunks l, l + 64, ..., which all belong to head group l % G because G divides 64, so the four
// reductions of a lane meet their partners by a butterfly over the lanes alone: no LDS, no barrier.  With many
// rows (the attention block has nbat * ntimes of them) this beats the workgroup-per-row kernel above, whose two
// block-wide folds each cost a barrier round trip: 16.5 -> 12.3 us for [4, 512, 512, 8] read from HBM.
template <bool BACKWARD, int VN>
__global__ void __launch_bounds__(kTB) softmax_axis_heads4_wave_kernel(float* __restrict__ io,
                                                                       const float* __restrict__ pp, int64_t nrow,
                                                                       int64_t nvec, int ncol,
                                                                       const float* __restrict__ hcoef) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kTB / 64) + (threadIdx.x >> 6);
    if (row >= nrow) return;   // whole waves leave; there is no barrier below
    const int G = ncol >> 2;
    const int len4 = (int)(nvec * ncol) >> 2;
    float* __restrict__ r = io + row * (nvec * ncol);
    auto fold = [&](f32x4s mine, bool is_max) -> f32x4s {
        for (int m = G; m < 64; m <<= 1) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float o = __shfl_xor(mine[j], m);
                mine[j] = is_max ? fmaxf(mine[j], o) : mine[j] + o;
            }
        }
        return mine;
    };
    f32x4s v[VN], q[VN];
#pragma unroll
    for (int i = 0; i < VN; i++) {
        const f32x4s* src = reinterpret_cast<const f32x4s*>(r + 4 * min(lane + 64 * i, len4 - 1));
        v[i] = BACKWARD ? *src : __builtin_nontemporal_load(src);
    }
    if (BACKWARD) {
        const float* __restrict__ p = pp + row * (nvec * ncol);
#pragma unroll
        for (int i = 0; i < VN; i++) q[i] = *reinterpret_cast<const f32x4s*>(p + 4 * min(lane + 64 * i, len4 - 1));
    }
#pragma unroll
    for (int i = 0; i < VN; i++) v[i] = keep_or(v[i], lane + 64 * i < len4, BACKWARD ? 0.f : -INFINITY);
    if (!BACKWARD) {
        f32x4s mx = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
#pragma unroll
        for (int i = 0; i < VN; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) mx[j] = fmaxf(mx[j], v[i][j]);
        mx = fold(mx, true);
        f32x4s sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VN; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[i][j] = exp_nonpositive(v[i][j] - mx[j]);   // padding holds -inf: exp gives 0
                sum[j] += v[i][j];
            }
        sum = fold(sum, false);
        f32x4s inv;
#pragma unroll
        for (int j = 0; j < 4; j++) inv[j] = 1.0f / sum[j];
#pragma unroll
        for (int i = 0; i < VN; i++)
            if (lane + 64 * i < len4) *reinterpret_cast<f32x4s*>(r + 4 * (lane + 64 * i)) = v[i] * inv;
    } else {
        const float coef = hcoef ? *hcoef : 0.f;
        f32x4s dot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VN; i++) {
            q[i] = keep_or(q[i], lane + 64 * i < len4, 0.f);
            dot += q[i] * v[i];
        }
        dot = fold(dot, false);
#pragma unroll
        for (int i = 0; i < VN; i++)
            if (lane + 64 * i < len4) *reinterpret_cast<f32x4s*>(r + 4 * (lane + 64 * i)) = coef * q[i] * (v[i] - dot);
    }
}

template <bool BACKWARD>
__global__ void __launch_bounds__(kTB) softmax_axis_thread_kernel(float* __restrict__ io,
                                                                  const float* __restrict__ pp, int64_t nrow,
                                                                  int64_t nvec, int64_t ncol,
                                                                  const float* __restrict__ hcoef) {
    const int64_t n = (int64_t)blockIdx.x * kTB + threadIdx.x;
    if (n >= nrow * ncol) return;
    const int64_t base = (n / ncol) * nvec * ncol + n % ncol;
    float* __restrict__ r = io + base;
    if (!BACKWARD) {
        float mx = -FLT_MAX;
        for (int64_t v = 0; v < nvec; v++) mx = fmaxf(mx, r[v * ncol]);
        float sum = 0.f;
        for (int64_t v = 0; v < nvec; v++) sum += expf(r[v * ncol] - mx);
        for (int64_t v = 0; v < nvec; v++) r[v * ncol] = expf(r[v * ncol] - mx) / sum;
    } else {
        const float coef = hcoef ? *hcoef : 0.f;
        const float* __restrict__ p = pp + base;
        float dot = 0.f;
        for (int64_t v = 0; v < nvec; v++) dot += p[v * ncol] * r[v * ncol];
        for (int64_t v = 0; v < nvec; v++) r[v * ncol] = coef * p[v * ncol] * (r[v * ncol] - dot);
    }
}

// Any head count up to 32, a whole outer row per wave, E elements per lane: the first A = H * (64 / H) lanes of a wave
// walk the row A floats at a time, so a lane's elements all belong to head lane % H and consecutive lanes read
// consecutive floats; the 64 / H lanes of a head meet by reading each other's partial result (one ds_bpermute per
// member): no LDS, no barrier.  For the head counts the four-heads layout does not take (2, 3, 6, 12, ...) and rows
// short enough for a wave's registers the workgroup-per-row kernels above spend their time in two block-wide folds:
// [64, 128, 128, 12] forward 33.5 us there, [64, 128, 128, 2] 79.7.
template <bool BACKWARD, int E>
__global__ void __launch_bounds__(kTB) softmax_axis_wave_heads_kernel(float* __restrict__ io,
                                                                      const float* __restrict__ pp, int64_t nrow,
                                                                      int64_t nvec, int ncol,
                                                                      const float* __restrict__ hcoef) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kTB / 64) + (threadIdx.x >> 6);
    if (row >= nrow) return;   // whole waves leave; there is no barrier below
    const int members = 64 / ncol;           // lanes per head
    const int active = members * ncol;       // lanes that hold elements
    const int len = (int)(nvec * ncol);
    const int head = lane % ncol;
    const bool on = lane < active;
    float* __restrict__ r = io + row * (int64_t)len;
    // every lane ends up with the result of its head (lanes past `active` hold the neutral element and are never read)
    auto fold = [&](float mine, bool is_max) -> float {
        float a = is_max ? -FLT_MAX : 0.f;
        for (int j = 0; j < members; j++) {
            const float o = __shfl(mine, head + ncol * j);
            a = is_max ? fmaxf(a, o) : a + o;
        }
        return a;
    };
    float v[E], q[E];
#pragma unroll
    for (int i = 0; i < E; i++) {
        const int idx = lane + active * i;
        v[i] = r[min(idx, len - 1)];
        if (BACKWARD) q[i] = pp[row * (int64_t)len + min(idx, len - 1)];
    }
#pragma unroll
    for (int i = 0; i < E; i++) {
        const bool in = on && lane + active * i < len;
        v[i] = in ? v[i] : (BACKWARD ? 0.f : -INFINITY);
        if (BACKWARD) q[i] = in ? q[i] : 0.f;
    }
    if (!BACKWARD) {
        float mx = -FLT_MAX;
#pragma unroll
        for (int i = 0; i < E; i++) mx = fmaxf(mx, v[i]);
        mx = fold(mx, true);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < E; i++) {
            v[i] = exp_nonpositive(v[i] - mx);   // padding holds -inf: exp gives 0
            sum += v[i];
        }
        const float inv = 1.0f / fold(sum, false);
#pragma unroll
        for (int i = 0; i < E; i++)
            if (on && lane + active * i < len) r[lane + active * i] = v[i] * inv;
    } else {
        const float coef = hcoef ? *hcoef : 0.f;
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < E; i++) dot += q[i] * v[i];
        dot = fold(dot, false);
#pragma unroll
        for (int i = 0; i < E; i++)
            if (on && lane + active * i < len) r[lane + active * i] = coef * q[i] * (v[i] - dot);
    }
}

template <bool BACKWARD>
static int launch_softmax_axis_impl(float* io, const float* pp, int64_t nrow, int64_t nvec, int64_t ncol,
                                    const float* hcoef, hipStream_t stream) {
    if (nrow <= 0 || nvec <= 0 || ncol <= 0) return KAI_OK;
    if (ncol == 1) {
        const int64_t blocks = (nrow + kTB / 64 - 1) / (kTB / 64);
        if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "softmax_direct_on_axis: too many rows");
        const bool vec = nvec % 4 == 0 && nvec <= 2048 && aligned16(io) && (!BACKWARD || aligned16(pp));
        if (vec) {
            const unsigned g = (unsigned)(blocks < 256 * 8 ? blocks : 256 * 8);   // grid-stride over rows
            const int nv = (int)nvec;
            if (nvec <= 256) softmax_axis_wave_reg_kernel<BACKWARD, 1><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
            else if (nvec <= 512) softmax_axis_wave_reg_kernel<BACKWARD, 2><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
            else if (nvec <= 1024) softmax_axis_wave_reg_kernel<BACKWARD, 4><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
            else softmax_axis_wave_reg_kernel<BACKWARD, 8><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
        } else if (nvec >= 64 && nvec <= 2048) {
            // rows off 16-byte lines: the same kernels through buffer accesses
            const unsigned g = (unsigned)(blocks < 256 * 8 ? blocks : 256 * 8);
            const int nv = (int)nvec;
            if (nvec <= 256) softmax_axis_wave_reg_kernel<BACKWARD, 1, true><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
            else if (nvec <= 512) softmax_axis_wave_reg_kernel<BACKWARD, 2, true><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
            else if (nvec <= 1024) softmax_axis_wave_reg_kernel<BACKWARD, 4, true><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
            else softmax_axis_wave_reg_kernel<BACKWARD, 8, true><<<g, kTB, 0, stream>>>(io, pp, nrow, nv, hcoef);
        } else {
            softmax_axis_wave_kernel<BACKWARD><<<dim3((unsigned)blocks), kTB, 0, stream>>>(io, pp, nrow, nvec, hcoef);
        }
    } else if (ncol <= 128) {
        if (nrow > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "softmax_direct_on_axis: too many rows");
        const int tb = (int)ncol * (kTB / (int)ncol);
        const int64_t len = nvec * ncol;
        const int64_t quarter = ncol / 4;
        const bool heads4 = ncol % 4 == 0 && (quarter & (quarter - 1)) == 0 && aligned16(io) &&
                            (pp == nullptr || aligned16(pp)) && len <= 4 * kTB * 16;
        // forward, many rows that each fit a wave's registers: one wave per row, no barrier (at least four waves
        // per compute unit; fewer rows keep the workgroup-per-row kernel, which puts more threads on each).  The
        // backward pass holds two rows per wave and measured slower this way (17.4 -> 19.6 us): it stays.
        if (!BACKWARD && heads4 && len <= 4 * 64 * 16 && nrow >= 4 * (int64_t)compute_units()) {
            const dim3 g((unsigned)((nrow + kTB / 64 - 1) / (kTB / 64)));
            const int nc = (int)ncol;
            if (len <= 4 * 64 * 4) softmax_axis_heads4_wave_kernel<BACKWARD, 4><<<g, kTB, 0, stream>>>(io, pp, nrow, nvec, nc, hcoef);
            else if (len <= 4 * 64 * 8) softmax_axis_heads4_wave_kernel<BACKWARD, 8><<<g, kTB, 0, stream>>>(io, pp, nrow, nvec, nc, hcoef);
            else softmax_axis_heads4_wave_kernel<BACKWARD, 16><<<g, kTB, 0, stream>>>(io, pp, nrow, nvec, nc, hcoef);
        } else if (!heads4 && ncol <= 32 && nrow >= 4 * (int64_t)compute_units() &&
                   len <= (int64_t)(64 / ncol) * ncol * (BACKWARD ? 16 : 32)) {
            // many rows that each fit a wave's registers, any head count: [64, 128, 128, 12] forward 33.5 -> 17.3 us, 6 heads
            // 39.5 -> 9.0, 2 heads 79.7 -> 10.2 (backward 37.8 -> 6.9), [256, 64, 64, 12] 53.7 -> 16.4
            const dim3 g((unsigned)((nrow + kTB / 64 - 1) / (kTB / 64)));
            const int nc = (int)ncol;
            const int64_t per_lane = (len + (64 / ncol) * ncol - 1) / ((64 / ncol) * ncol);
            if (per_lane <= 4) softmax_axis_wave_heads_kernel<BACKWARD, 4><<<g, kTB, 0, stream>>>(io, pp, nrow, nvec, nc, hcoef);
            else if (per_lane <= 8) softmax_axis_wave_heads_kernel<BACKWARD, 8><<<g, kTB, 0, stream>>>(io, pp, nrow, nvec, nc, hcoef);
            else if (per_lane <= 16) softmax_axis_wave_heads_kernel<BACKWARD, 16><<<g, kTB, 0, stream>>>(io, pp, nrow, nvec, nc, hcoef);
            else softmax_axis_wave_heads_kernel<BACKWARD, 32><<<g, kTB, 0, stream>>>(io, pp, nrow, nvec, nc, hcoef);
        } else if (heads4) {
            const dim3 g((unsigned)nrow);
            if (len <= 4 * kTB * 2) softmax_axis_heads4_kernel<BACKWARD, 2><<<g, kTB, 0, stream>>>(io, pp, nvec, (int)ncol, hcoef);
            else if (len <= 4 * kTB * 4) softmax_axis_heads4_kernel<BACKWARD, 4><<<g, kTB, 0, stream>>>(io, pp, nvec, (int)ncol, hcoef);
            else if (len <= 4 * kTB * 8) softmax_axis_heads4_kernel<BACKWARD, 8><<<g, kTB, 0, stream>>>(io, pp, nvec, (int)ncol, hcoef);
            // (16 heads x 1000 keys: 71.9 us with the three passes over memory)
            else softmax_axis_heads4_kernel<BACKWARD, 16><<<g, kTB, 0, stream>>>(io, pp, nvec, (int)ncol, hcoef);
        } else if (len <= (int64_t)tb * 16)
            softmax_axis_block_reg_kernel<BACKWARD, 16><<<dim3((unsigned)nrow), kTB, 0, stream>>>(io, pp, nvec, (int)ncol,
                                                                                                 tb, hcoef);
        else if (len <= (int64_t)tb * 32)
            softmax_axis_block_reg_kernel<BACKWARD, 32><<<dim3((unsigned)nrow), kTB, 0, stream>>>(io, pp, nvec, (int)ncol,
                                                                                                 tb, hcoef);
        // (12 heads x 1000 keys: 56.0 us with the three passes over memory, 26.3 here; the backward pass would hold two
        // rows, 256 registers: 85 us against 40 with the three passes)
        else if (!BACKWARD && len <= (int64_t)tb * 64)
            softmax_axis_block_reg_kernel<BACKWARD, 64><<<dim3((unsigned)nrow), kTB, 0, stream>>>(io, pp, nvec, (int)ncol,
                                                                                                 tb, hcoef);
        else
            softmax_axis_block_kernel<BACKWARD><<<dim3((unsigned)nrow), kTB, 0, stream>>>(io, pp, nvec, (int)ncol, tb,
                                                                                         hcoef);
    } else {
        const int64_t blocks = (nrow * ncol + kTB - 1) / kTB;
        if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "softmax_direct_on_axis: too many rows");
        softmax_axis_thread_kernel<BACKWARD><<<dim3((unsigned)blocks), kTB, 0, stream>>>(io, pp, nrow, nvec, ncol,
                                                                                        hcoef);
    }
    return check_launch("softmax_axis_kernel");
}

int launch_softmax_axis(float* pp, int64_t nrow, int64_t nvec, int64_t ncol, hipStream_t stream) {
    return launch_softmax_axis_impl<false>(pp, nullptr, nrow, nvec, ncol, nullptr, stream);
}

int launch_softmax_axis_backward(float* pgp, const float* pp, int64_t nrow, int64_t nvec, int64_t ncol,
                                 const float* hcoef, hipStream_t stream) {
    return launch_softmax_axis_impl<true>(pgp, pp, nrow, nvec, ncol, hcoef, stream);
}

}  // namespace kai
