// Attention for inference in one kernel: O = softmax(coef * Q.K^T [causal mask]) . V per (batch, head),
// i.e. VMath::mult_on_heads -> set_mh_attention_mask -> softmax_direct_on_axis -> mix_values
// (vmath.cu:6729-6779, 6833-6860, 6864-6916, 6977-7025 of the reference, driven by
// VTensor::mh_attention, vtensor.cpp:3036-3043) without the [batch, T, T, heads] tensor ever reaching
// memory.  The engine's training path needs that tensor for the backward pass and keeps using the
// separate entry points; this one is for forward-only use.
//
// A workgroup owns 64 query rows of one (batch, head) and walks the keys in tiles of 64
// with a running maximum and sum per query (the softmax is renormalised tile by tile, so the result
// differs from the three-pass form only by rounding).  Everything is computed transposed, queries
// along the lanes: S^T = K.Q^T puts the 32 scores of a query into 8 registers of 4 lanes, so the
// row maximum and sum cost two cross-lane steps, and the registers that hold exp(S^T) are, as they
// are, the B operand of O^T += V^T.P^T.  v_mfma_f32_16x16x4_f32: lane = (row or column l % 16, k
// group l / 16); element e of a 128-bit LDS read at k offset 16*s + 4*(l/16) feeds step (s, e) of both
// operands.  K and V tiles lie in LDS as in memory.
#include <float.h>

#include "elementwise.h"

namespace kai {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kFaQGroups = 4;          // waves along the queries, 16 rows each
constexpr int kFaKGroups = 2;          // waves along the keys: each takes 32 of a tile's 64 keys
constexpr int kFaWaves = kFaQGroups * kFaKGroups;
constexpr int kFaThreads = 64 * kFaWaves;
constexpr int kFaQ = 16 * kFaQGroups;  // query rows per workgroup
constexpr int kFaKeys = 32 * kFaKGroups;   // keys per tile

struct FusedParams {
    const float* Q;
    const float* K;
    const float* V;
    float* O;
    const float* coef;   // device scalar, null reads as 0
    int64_t nvec;        // row stride of Q, K, V and O
    int64_t batch_stride;   // ntimes * nvec
    int ntimes, nhead, npiece;
    int masked;
};

// DB = npiece / 16.  Two sets of four waves share a tile of 64 keys, 32 keys each, and keep separate
// running maxima, sums and outputs that are merged once at the end: a SIMD then holds two waves of
// the workgroup, and the softmax arithmetic and LDS waits of one run under the MFMAs of the other.
template <int DB>
__global__ void __launch_bounds__(kFaThreads) attention_fused_kernel(const FusedParams p) {
    constexpr int D = 16 * DB;
    constexpr int kKStride = D + 4;          // K tile [64 keys][D]
    constexpr int kVStride = D + 4;          // V tile [64 keys][D]
    constexpr int kChunksPerKey = D / 4;
    constexpr int kTileChunks = kFaKeys * kChunksPerKey;
    constexpr int NCH = (kTileChunks + kFaThreads - 1) / kFaThreads;   // 128-bit chunks per thread and tile
    constexpr bool kPartial = kTileChunks % kFaThreads != 0;           // head size 16: half of the threads load
    __shared__ __attribute__((aligned(16))) float lds_k[2][kFaKeys * kKStride];
    __shared__ __attribute__((aligned(16))) float lds_v[2][kFaKeys * kVStride];
    static_assert((2 + 4 * DB) * 64 * kFaQGroups <= 2 * kFaKeys * kKStride, "merge buffer must fit the K tiles");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qg = wave % kFaQGroups;     // which 16 query rows
    const int kgp = wave / kFaQGroups;    // which half of every key tile
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int T = p.ntimes;
    const int b = blockIdx.y / p.nhead, h = blockIdx.y % p.nhead;
    const int q0 = blockIdx.x * kFaQ;
    const int64_t base = (int64_t)b * p.batch_stride + (int64_t)h * p.npiece;
    const float* __restrict__ Qb = p.Q + base;
    const float* __restrict__ Kb = p.K + base;
    const float* __restrict__ Vb = p.V + base;
    const float coef = p.coef ? *p.coef : 0.f;
    const float c2 = coef * 1.44269504088896340736f;   // scores are scaled straight into the base-2 domain

    // this lane's query row and its operand fragments of Q (rows past the end are clamped, never stored)
    const int q = q0 + 16 * qg + r16;
    const int qc = min(q, T - 1);
    f32x4 qf[DB];
#pragma unroll
    for (int s = 0; s < DB; s++) qf[s] = c2 * *reinterpret_cast<const f32x4*>(Qb + (int64_t)qc * p.nvec + 16 * s + 4 * g);

    // key tiles that hold an unmasked key for some query of this workgroup
    const int q_last = min(q0 + kFaQ, T) - 1;
    const int nkt = p.masked ? q_last / kFaKeys + 1 : (T + kFaKeys - 1) / kFaKeys;

    // tile loads: chunk c of a thread = (key c / (D/4), d 4 * (c % (D/4))), the same for K and V.  Buffer loads:
    // resource = this (batch entry, head)'s rows of K / V up to the last key, lane offset constant, tile offset
    // scalar, so a tile costs no vector instruction for addresses, and keys past the end read as zeros (their
    // scores are masked) without a clamp or a mask.  Vector instructions take their time from the fp32 MFMAs.
    auto uniform_ptr = [](const float* q) -> float* {
        const uint64_t a = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
    };
    const int extent = (int)(((int64_t)(T - 1) * p.nvec + D) * 4);   // bytes; the host keeps it below 2 GiB
    const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(Kb), 0, extent, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(Vb), 0, extent, 0x00020000);
    const int tile_bytes = kFaKeys * (int)p.nvec * 4;
    int choff[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * kFaThreads;
        choff[i] = ((c / kChunksPerKey) * (int)p.nvec + (c % kChunksPerKey) * 4) * 4;
    }
    f32x4 rk[NCH], rv[NCH];
    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * kFaThreads;
            if (!kPartial || c < kTileChunks) {
                rk[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_k, choff[i], kt * tile_bytes, 0));
                rv[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_v, choff[i], kt * tile_bytes, 0));
            }
        }
    };
    auto store_tile = [&](int kt, int buf) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * kFaThreads;
            const int kl = c / kChunksPerKey;
            const int d = (c % kChunksPerKey) * 4;
            if (!kPartial || c < kTileChunks) {
                *reinterpret_cast<f32x4*>(&lds_k[buf][kl * kKStride + d]) = rk[i];
                *reinterpret_cast<f32x4*>(&lds_v[buf][kl * kVStride + d]) = rv[i];
            }
        }
    };

    float m_run = -INFINITY;   // running maximum of this lane's query (equal in the 4 lanes that share it)
    float l_run = 0.f;         // running sum over this lane's own keys
    f32x4 acc_o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++) acc_o[db] = f32x4{0.f, 0.f, 0.f, 0.f};

    load_tile(0);
    store_tile(0, 0);
    __syncthreads();

    for (int kt = 0; kt < nkt; kt++) {
        const int buf = kt & 1;
        load_tile(min(kt + 1, nkt - 1));   // in flight during the work below; the surplus load is never stored
        const int key0 = kt * kFaKeys + 32 * kgp;   // first key of this wave's half
        // a half tile past the end, or entirely above the diagonal of the workgroup's last query, adds nothing
        if (key0 < T && !(p.masked && key0 > q_last)) {
            const float* lk = lds_k[buf] + 32 * kgp * kKStride;
            const float* lv = lds_v[buf] + 32 * kgp * kVStride;
            // S^T: 2 blocks of 16 keys x 16 queries
            f32x4 sc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
            // the two key blocks alternate, so that no MFMA waits for the one before it
#pragma unroll
            for (int s = 0; s < DB; s++) {
                f32x4 kf[2];
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
                    kf[kb] = *reinterpret_cast<const f32x4*>(lk + (16 * kb + r16) * kKStride + 16 * s + 4 * g);
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int kb = 0; kb < 2; kb++)
                        sc[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[kb][e], qf[s][e], sc[kb], 0, 0, 0);
            }
            // sc[kb][v] = score of (query q, key key0 + 16*kb + 4*g + v) in the base-2 domain (Q was scaled by
            // c2 = coef * log2(e) when it was loaded): exp(coef * s - m) = 2^(c2 * s - m2), one v_exp_f32 per element
            const bool edge_tile = key0 + 32 > T || (p.masked && key0 + 31 > q0 + 16 * qg);   // wave-uniform
            // fp32 MFMAs and vector ALU instructions take turns on a SIMD (measured: their times add up), so the
            // 16 compares and selects of the mask are kept off the tiles that do not need them by a real branch
            if (edge_tile) {   // keys past the end or above the diagonal of some query of this wave
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const int key = key0 + 16 * kb + 4 * g + v;
                        if (key >= T || (p.masked && key > q)) sc[kb][v] = -INFINITY;
                    }
                __builtin_amdgcn_sched_barrier(0);
            }
            float m_tile = fmaxf(fmaxf(fmaxf(sc[0][0], sc[0][1]), fmaxf(sc[0][2], sc[0][3])),
                                 fmaxf(fmaxf(sc[1][0], sc[1][1]), fmaxf(sc[1][2], sc[1][3])));
            m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16));
            m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32));
            const float m_new = fmaxf(m_run, m_tile);
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;   // nothing unmasked for this query so far
            const float rescale = __builtin_amdgcn_exp2f(m_run - m_safe);   // 2^-inf = 0 on the first tile
            float l_tile = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    sc[kb][v] = __builtin_amdgcn_exp2f(sc[kb][v] - m_safe);
                    l_tile += sc[kb][v];
                }
            l_run = l_run * rescale + l_tile;
            m_run = m_new;
            // O^T[d, q] = O^T * rescale + sum_key V[key, d] * P[q, key]
            // the running maximum rarely moves after the first tiles: skip the 4*DB multiplies when no lane needs them
            if (__builtin_amdgcn_ballot_w64(rescale != 1.0f) != 0) {
#pragma unroll
                for (int db = 0; db < DB; db++) acc_o[db] *= rescale;
            }
            // V^T[d = 16*db + r16][key = 16*kb + 4*g + e]: 32-bit reads down a column of the tile (consecutive
            // lanes, consecutive d: no bank conflict); a transposed tile would allow 128-bit reads but costs
            // element-wise LDS stores with 8-way conflicts on the way in.  The DB output blocks alternate.
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float* vp = lv + (16 * kb + 4 * g + e) * kVStride + r16;
#pragma unroll
                    for (int db = 0; db < DB; db++)
                        acc_o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(vp[16 * db], sc[kb][e], acc_o[db], 0, 0, 0);
                }
        }
        if (kt + 1 < nkt) store_tile(kt + 1, buf ^ 1);
        __syncthreads();
    }

    // merge the two key halves: the second set of waves hands (m, l, O) over through LDS
    float* mg = &lds_k[0][0] + (qg * 64 + lane);
    constexpr int kMergeStride = 64 * kFaQGroups;
    if (kgp == 1) {
        mg[0] = m_run;
        mg[kMergeStride] = l_run;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int v = 0; v < 4; v++) mg[(2 + 4 * db + v) * kMergeStride] = acc_o[db][v];
    }
    __syncthreads();
    if (kgp == 1) return;
    {
        const float m1 = mg[0], l1 = mg[kMergeStride];
        const float m = fmaxf(m_run, m1);
        const float m_safe = m == -INFINITY ? 0.f : m;
        const float f0 = __builtin_amdgcn_exp2f(m_run - m_safe), f1 = __builtin_amdgcn_exp2f(m1 - m_safe);
        l_run = l_run * f0 + l1 * f1;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int v = 0; v < 4; v++) acc_o[db][v] = acc_o[db][v] * f0 + mg[(2 + 4 * db + v) * kMergeStride] * f1;
    }
    // the four lanes of a query add their partial sums; acc_o[db][v] = O[q, 16*db + 4*g + v]
    l_run += __shfl_xor(l_run, 16);
    l_run += __shfl_xor(l_run, 32);
    if (q < T) {
        float* out = p.O + base + (int64_t)q * p.nvec;
#pragma unroll
        for (int db = 0; db < DB; db++) *reinterpret_cast<f32x4*>(out + 16 * db + 4 * g) = acc_o[db] / l_run;
    }
}

}  // namespace

bool attention_fused_applies(const float* q, const float* k, const float* v, const float* o, int64_t ntimes,
                             int64_t nvec, int64_t nhead, int64_t npiece) {
    // the kernel writes its output with the row stride of the inputs; the output of the separate calls is
    // [nbat, ntimes, nhead, npiece], which is the same thing only when the heads fill the vector
    return nhead * npiece == nvec &&
           (npiece == 16 || npiece == 32 || npiece == 64) && nvec % 4 == 0 && ntimes >= 1 && ntimes <= kMaxDim &&
           ntimes * nvec * 4 < (1ll << 31) &&
           nhead >= 1 && aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o);
}

int launch_attention_fused(float* o, const float* q, const float* k, const float* v, int64_t nbat, int64_t ntimes,
                           int64_t nvec, int64_t nhead, int64_t npiece, const float* hcoef, int masked,
                           hipStream_t stream) {
    FusedParams p{};
    p.Q = q; p.K = k; p.V = v; p.O = o; p.coef = hcoef;
    p.nvec = nvec; p.batch_stride = ntimes * nvec;
    p.ntimes = (int)ntimes; p.nhead = (int)nhead; p.npiece = (int)npiece;
    p.masked = masked;
    const int64_t qtiles = (ntimes + kFaQ - 1) / kFaQ;
    if (qtiles > kMaxDim || nbat * nhead > 65535) return fail(KAI_ERR_INVALID_ARGUMENT, "attention: grid too large");
    const dim3 grid((unsigned)qtiles, (unsigned)(nbat * nhead));
    if (npiece == 16) attention_fused_kernel<1><<<grid, dim3(kFaThreads), 0, stream>>>(p);
    else if (npiece == 32) attention_fused_kernel<2><<<grid, dim3(kFaThreads), 0, stream>>>(p);
    else attention_fused_kernel<4><<<grid, dim3(kFaThreads), 0, stream>>>(p);
    return check_launch("attention_fused_kernel");
}

}  // namespace kai
