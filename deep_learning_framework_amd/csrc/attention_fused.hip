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

#include <type_traits>

#include "elementwise.h"

namespace kai {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// loop with compile-time indices (register arrays must never be indexed by a run-time value)
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// Workgroup id -> (batch entry, head, row tile).  Hardware deals consecutive workgroup ids round-robin over the 8
// XCDs, so ids congruent mod 8 share an L2.  They are renumbered so that each XCD gets a contiguous run of the
// order (batch entry, row tile, head): the workgroups that read the same K and V rows (all row tiles of a batch
// entry and head) and, with several heads, the same lines of the head-interleaved probabilities (all heads of a
// batch entry and row tile) then sit behind one L2 instead of fetching them into all eight.
__device__ __forceinline__ void attention_block_of(int bid, int total, int ntiles, int nhead, int& b, int& h, int& tile) {
    int id = bid;
    if ((total & 7) == 0) id = (bid & 7) * (total >> 3) + (bid >> 3);
    h = id % nhead;
    const int r = id / nhead;
    tile = r % ntiles;
    b = r / ntiles;
}

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
    int b, h, qtile;
    attention_block_of(blockIdx.x, gridDim.x, (T + kFaQ - 1) / kFaQ, p.nhead, b, h, qtile);
    const int q0 = qtile * kFaQ;
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

    // The schedule of a tile is written out (as in attention_backward.hip): its products are dealt with in NG groups
    // -- DB groups of 8 (S^T, one 16-wide slice of the head dimension each), then 8 groups of DB (O^T, one key column
    // of one block each) -- with fences between them.  The LDS reads of group i + 1 are issued before the products of
    // group i (operands double buffered by group parity), the global loads of the next tile are dealt out over the
    // first groups and its LDS stores over the last, and the barrier sits before the last group, whose products
    // cover the first reads of the next tile.  A half tile past the end or above the diagonal is not skipped: its
    // scores are masked to -inf and add nothing.
    constexpr int NA = DB, NC = 8, NG = NA + NC;
    constexpr int NLOAD = 2 * NCH;    // K chunks, then V chunks
    constexpr int kLoadsPerGroup = (NLOAD + (NG - 3) - 1) / (NG - 3);
    constexpr int kStoresPerGroup = 2;
    constexpr int kStoreGroups = (NLOAD + kStoresPerGroup - 1) / kStoresPerGroup;
    constexpr int kFirstStoreGroup = NG - 1 - kStoreGroups;     // the last store is in group NG - 2
    static_assert(kFirstStoreGroup >= 1 && kLoadsPerGroup * (kFirstStoreGroup) >= 1, "too many chunks for this schedule");
    auto load_one = [&](auto jc, int kt) {
        constexpr int jj = decltype(jc)::value;
        constexpr int i = jj % NCH;
        const int c = tid + i * kFaThreads;
        if (!kPartial || c < kTileChunks) {
            if constexpr (jj / NCH == 0) rk[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_k, choff[i], kt * tile_bytes, 0));
            else rv[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_v, choff[i], kt * tile_bytes, 0));
        }
    };
    auto store_one = [&](auto jc, int buf) {
        constexpr int jj = decltype(jc)::value;
        constexpr int i = jj % NCH;
        const int c = tid + i * kFaThreads;
        if (!kPartial || c < kTileChunks) {
            const int off = (c / kChunksPerKey) * kKStride + (c % kChunksPerKey) * 4;
            if constexpr (jj / NCH == 0) *reinterpret_cast<f32x4*>(&lds_k[buf][off]) = rk[i];
            else *reinterpret_cast<f32x4*>(&lds_v[buf][off]) = rv[i];
        }
    };
    static_assert(kKStride == kVStride, "one chunk offset for both tiles");
    // operand registers of the groups, double buffered by group parity
    f32x4 kf[2][2];
    float vf[2][DB];
    auto stage = [&](auto ic, int buf) {
        constexpr int i = decltype(ic)::value;
        constexpr int par = i & 1;
        if constexpr (i < NA) {
            const float* lk = lds_k[buf] + 32 * kgp * kKStride;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
                kf[par][kb] = *reinterpret_cast<const f32x4*>(lk + (16 * kb + r16) * kKStride + 16 * i + 4 * g);
        } else {
            // V^T[d = 16*db + r16][key = 16*kb + 4*g + e]: 32-bit reads down a column of the tile (consecutive
            // lanes, consecutive d: no bank conflict); a transposed tile would allow 128-bit reads but costs
            // element-wise LDS stores with 8-way conflicts on the way in.
            constexpr int kb = (i - NA) / 4, e = (i - NA) % 4;
            const float* vp = lds_v[buf] + 32 * kgp * kVStride + (16 * kb + 4 * g + e) * kVStride + r16;
#pragma unroll
            for (int db = 0; db < DB; db++) vf[par][db] = vp[16 * db];
        }
    };

    load_tile(0);
    store_tile(0, 0);
    __syncthreads();
    stage(std::integral_constant<int, 0>{}, 0);

    for (int kt = 0; kt < nkt; kt++) {
        const int buf = kt & 1;
        const int nxt = min(kt + 1, nkt - 1);       // the surplus loads and stores of the last tile are never used
        const int key0 = kt * kFaKeys + 32 * kgp;   // first key of this wave's half
        // S^T: 2 blocks of 16 keys x 16 queries; the two key blocks alternate, so that no MFMA waits for the one before it
        f32x4 sc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
        static_for<0, NG>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            constexpr int par = i & 1;
            // -- the next group's operands
            if constexpr (i + 1 < NG) {
                stage(std::integral_constant<int, i + 1>{}, buf);
            } else {
                __syncthreads();     // the next tile is in LDS, and every wave has read this one
                if (kt + 1 < nkt) stage(std::integral_constant<int, 0>{}, buf ^ 1);
            }
            // -- this group's share of the next tile's traffic
            static_for<0, kLoadsPerGroup>([&](auto lc) {
                constexpr int jj = i * kLoadsPerGroup + decltype(lc)::value;
                if constexpr (jj < NLOAD) load_one(std::integral_constant<int, jj>{}, nxt);
            });
            if constexpr (i >= kFirstStoreGroup && i < NG - 1) {
                static_for<0, kStoresPerGroup>([&](auto sc_) {
                    constexpr int jj = (i - kFirstStoreGroup) * kStoresPerGroup + decltype(sc_)::value;
                    if constexpr (jj < NLOAD) store_one(std::integral_constant<int, jj>{}, buf ^ 1);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
            // -- this group's products
            if constexpr (i < NA) {
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int kb = 0; kb < 2; kb++)
                        sc[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[par][kb][e], qf[i][e], sc[kb], 0, 0, 0);
                if constexpr (i == NA - 1) {
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
                }
            } else {
                // the DB output blocks alternate
                constexpr int kb = (i - NA) / 4, e = (i - NA) % 4;
#pragma unroll
                for (int db = 0; db < DB; db++)
                    acc_o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[par][db], sc[kb][e], acc_o[db], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
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


// ---- the same block for TRAINING: the probabilities are also stored, as the backward pass needs them -------------
//
// With the probabilities to be written normalised, the running renormalisation of the kernel above does not apply:
// a query's maximum and sum must be known before its first probability is stored.  Here a wave keeps ALL of its
// scores in registers (8 per tile of 64 keys: lengths up to 64 * NT) -- first every key tile of K passes through
// LDS and leaves its scores, then maximum, exponentials and sum are formed in registers (the two key halves exchange
// theirs through LDS), then every tile of V passes through the same LDS buffers while the finished probabilities
// are stored and multiplied into the output.  Each product is computed once; P is written once and never read.
struct ProbsParams {
    FusedParams f;
    float* P;                 // [nbat, ntimes, ntimes, nhead]
    int64_t p_batch_stride;   // ntimes * ntimes * nhead
};

// HG = heads per workgroup.  1: the eight waves are 4 groups of 16 queries x 2 halves of every key tile, all of one
// head; a lane stores the probabilities of 4 consecutive keys of its query (one 128-bit store with one head in
// all, PVEC, else four 32-bit stores nhead floats apart).  4 (head counts that are multiples of 4): the waves are
// 4 HEADS x 2 key halves of the same 16 queries, the K / V tiles hold the rows of the four heads side by side as
// they lie in memory, and the probabilities of a tile meet in LDS so that a lane stores the four heads of one
// (query, key) as one 128-bit word: written head by head, 4 bytes every 4 * nhead, the stores of the probabilities
// alone took longer than everything else together (cfg4 with 8 heads: 58 us against 29 with one head).
template <int DB, int NT, int HG, bool PVEC>
__global__ void __launch_bounds__(kFaThreads) attention_probs_kernel(const ProbsParams pp) {
    const FusedParams& p = pp.f;
    constexpr int D = 16 * DB;
    constexpr int kRows = HG == 1 ? kFaQ : 16;        // queries per workgroup
    constexpr int kStride = HG * D + 4;               // tile [64 keys][HG heads x D]
    constexpr int kChunksPerKey = HG * D / 4;
    constexpr int kTileChunks = kFaKeys * kChunksPerKey;
    constexpr int NCH = (kTileChunks + kFaThreads - 1) / kFaThreads;
    constexpr bool kPartial = kTileChunks % kFaThreads != 0;
    constexpr int kPStride = kFaKeys + 4;             // exchange buffer [4 heads][16 queries][64 keys]: a plane per head
    constexpr int kPPlane = 16 * kPStride;
    __shared__ __attribute__((aligned(16))) float lds_t[2][kFaKeys * kStride];   // K tiles, then V tiles
    __shared__ float lds_x[2][64 * kFaQGroups];                                   // exchange of maxima and sums
    __shared__ __attribute__((aligned(16))) float lds_p[HG == 4 ? 4 * kPPlane : 4];
    static_assert(HG == 1 || HG == 4, "one head or four heads per workgroup");
    static_assert(!(HG == 4 && PVEC), "PVEC is the one-head store");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int w4 = wave % kFaQGroups;
    const int kgp = wave / kFaQGroups;
    const int qg = HG == 1 ? w4 : 0;      // which 16 queries of the workgroup
    const int hd = HG == 1 ? 0 : w4;      // which head of the workgroup
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int T = p.ntimes;
    const int H = p.nhead;
    int b, hgrp, qtile;
    attention_block_of(blockIdx.x, gridDim.x, (T + kRows - 1) / kRows, H / HG, b, hgrp, qtile);
    const int h0 = hgrp * HG;             // first head of the workgroup
    const int q0 = qtile * kRows;
    const int64_t base = (int64_t)b * p.batch_stride + (int64_t)h0 * p.npiece;   // the workgroup's heads, side by side
    const float* __restrict__ Qb = p.Q + base + hd * D;
    const float coef = p.coef ? *p.coef : 0.f;
    const float c2 = coef * 1.44269504088896340736f;

    const int q = q0 + 16 * qg + r16;
    const int qc = min(q, T - 1);
    f32x4 qf[DB];
#pragma unroll
    for (int s = 0; s < DB; s++) qf[s] = c2 * *reinterpret_cast<const f32x4*>(Qb + (int64_t)qc * p.nvec + 16 * s + 4 * g);

    const int nkt_all = (T + kFaKeys - 1) / kFaKeys;
    const int q_last = min(q0 + kRows, T) - 1;
    // key tiles that hold an unmasked key for some query of this workgroup; the others hold zeros only
    const int nkt = p.masked ? min(q_last / kFaKeys + 1, nkt_all) : nkt_all;

    auto uniform_ptr = [](const float* ptr) -> float* {
        const uint64_t a = reinterpret_cast<uint64_t>(ptr);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
    };
    const int extent = (int)(((int64_t)(T - 1) * p.nvec + HG * D) * 4);
    const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.K + base), 0, extent, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.V + base), 0, extent, 0x00020000);
    const int tile_bytes = kFaKeys * (int)p.nvec * 4;
    int choff[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * kFaThreads;
        choff[i] = ((c / kChunksPerKey) * (int)p.nvec + (c % kChunksPerKey) * 4) * 4;
    }
    // Staging registers of the tiles on their way, two sets: while tile kt is at work, tile kt + 1 (requested a tile
    // earlier) moves to LDS and tile kt + 2 is requested.  The loads are dealt out over the groups of products of a
    // tile instead of being issued together (issued together they fill the address unit's queue and every wave
    // waits at its next load), the LDS stores sit in the group before the last, the barrier before the last group,
    // whose operands are in registers by then and whose products cover the first LDS reads of the next tile; the
    // LDS reads of a group are issued before the products of the group before it.  Fences keep the order.
    f32x4 rt[2][NCH];
    auto load_one = [&](auto setc, auto jc, const __amdgpu_buffer_rsrc_t& rsrc, int kt) {
        constexpr int set = decltype(setc)::value, j = decltype(jc)::value;
        const int c = tid + j * kFaThreads;
        if (!kPartial || c < kTileChunks)
            rt[set][j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, choff[j], kt * tile_bytes, 0));
    };
    auto store_one = [&](auto setc, auto jc, int buf) {
        constexpr int set = decltype(setc)::value, j = decltype(jc)::value;
        const int c = tid + j * kFaThreads;
        if (!kPartial || c < kTileChunks)
            *reinterpret_cast<f32x4*>(&lds_t[buf][(c / kChunksPerKey) * kStride + (c % kChunksPerKey) * 4]) = rt[set][j];
    };
    auto load_all = [&](auto setc, const __amdgpu_buffer_rsrc_t& rsrc, int kt) {
        static_for<0, NCH>([&](auto jc) { load_one(setc, jc, rsrc, kt); });
    };
    auto store_all = [&](auto setc, int buf) {
        static_for<0, NCH>([&](auto jc) { store_one(setc, jc, buf); });
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    // ---- scores of every key tile into registers: sc[kt][kb][v] = (query q, key 64*kt + 32*kgp + 16*kb + 4*g + v) -----
    // groups of 8 products: one 16-wide slice s of the head dimension, both key blocks
    f32x4 sc[NT][2];
    f32x4 kf[2][2];      // operands of a group, double buffered by group parity
    auto stage_k = [&](auto parc, int s, int buf) {
        constexpr int par = decltype(parc)::value;
        const float* lk = lds_t[buf] + 32 * kgp * kStride + hd * D;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
            kf[par][kb] = *reinterpret_cast<const f32x4*>(lk + (16 * kb + r16) * kStride + 16 * s + 4 * g);
    };
    constexpr int kLoadGroups1 = DB > 1 ? DB - 1 : 1;                      // groups that carry the loads of tile kt + 2
    constexpr int kLPG1 = (NCH + kLoadGroups1 - 1) / kLoadGroups1;
    constexpr int kStoreGroup1 = DB > 1 ? DB - 2 : 0;                       // the group that moves tile kt + 1 to LDS
    load_all(I0{}, rsrc_k, 0);
    load_all(I1{}, rsrc_k, min(1, nkt - 1));
    store_all(I0{}, 0);
    __syncthreads();
    stage_k(I0{}, 0, 0);
    static_for<0, NT>([&](auto ktc) {
        constexpr int kt = decltype(ktc)::value;
        if (kt < nkt) {
            constexpr int buf = kt & 1;
            using SetNow = std::integral_constant<int, kt & 1>;          // held tile kt, free now: receives tile kt + 2
            using SetNext = std::integral_constant<int, (kt + 1) & 1>;   // holds tile kt + 1
            const int key0 = kt * kFaKeys + 32 * kgp;
            const int kt2 = min(kt + 2, nkt - 1);                         // past the end: a surplus load, never stored
            sc[kt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
            sc[kt][1] = f32x4{0.f, 0.f, 0.f, 0.f};
            static_for<0, DB>([&](auto sc_) {
                constexpr int s = decltype(sc_)::value;
                constexpr int par = (kt * DB + s) & 1;
                using ParNext = std::integral_constant<int, par ^ 1>;
                if constexpr (s == kStoreGroup1) store_all(SetNext{}, buf ^ 1);
                if constexpr (s + 1 < DB) {
                    stage_k(ParNext{}, s + 1, buf);
                } else {
                    __syncthreads();     // tile kt + 1 is in LDS, and every wave has read tile kt
                    if (kt + 1 < nkt) stage_k(ParNext{}, 0, buf ^ 1);
                }
                static_for<0, kLPG1>([&](auto lc) {
                    constexpr int j = s * kLPG1 + decltype(lc)::value;
                    if constexpr (j < NCH && (s < kLoadGroups1)) load_one(SetNow{}, std::integral_constant<int, j>{}, rsrc_k, kt2);
                });
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int kb = 0; kb < 2; kb++)
                        sc[kt][kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[par][kb][e], qf[s][e], sc[kt][kb], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            });
            const bool edge_tile = key0 + 32 > T || (p.masked && key0 + 31 > q0 + 16 * qg);   // wave-uniform
            if (edge_tile) {
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const int key = key0 + 16 * kb + 4 * g + v;
                        if (key >= T || (p.masked && key > q)) sc[kt][kb][v] = -INFINITY;
                    }
            }
        } else {
            sc[kt][0] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            sc[kt][1] = sc[kt][0];
        }
    });
    // the first two tiles of V are on their way while the softmax runs
    load_all(I0{}, rsrc_v, 0);
    load_all(I1{}, rsrc_v, min(1, nkt - 1));

    // ---- maximum, exponentials, sum: in registers; the two key halves exchange through LDS ---------------------------
    float m = -INFINITY;
    static_for<0, NT>([&](auto ktc) {
        constexpr int kt = decltype(ktc)::value;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
            m = fmaxf(m, fmaxf(fmaxf(sc[kt][kb][0], sc[kt][kb][1]), fmaxf(sc[kt][kb][2], sc[kt][kb][3])));
    });
    m = fmaxf(m, __shfl_xor(m, 16));
    m = fmaxf(m, __shfl_xor(m, 32));
    lds_x[kgp][w4 * 64 + lane] = m;
    __syncthreads();
    m = fmaxf(m, lds_x[kgp ^ 1][w4 * 64 + lane]);   // key 0 is never masked: the maximum is finite
    float l = 0.f;
    static_for<0, NT>([&](auto ktc) {
        constexpr int kt = decltype(ktc)::value;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                sc[kt][kb][v] = __builtin_amdgcn_exp2f(sc[kt][kb][v] - m);
                l += sc[kt][kb][v];
            }
    });
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    __syncthreads();                                  // every wave has read the maxima
    lds_x[kgp][w4 * 64 + lane] = l;
    store_all(I0{}, 0);                               // V tile 0 (the K tiles are done with)
    __syncthreads();
    l += lds_x[kgp ^ 1][w4 * 64 + lane];
    const float rl = 1.0f / l;

    // ---- probabilities stored, and multiplied into the output tile by tile -------------------------------------------
    // groups of 2 * DB products: two key columns e of one key block kb
    f32x4 acc_o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++) acc_o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float vfl[2][2][DB];
    auto stage_v = [&](auto parc, int gi, int buf) {
        constexpr int par = decltype(parc)::value;
        const float* lv = lds_t[buf] + 32 * kgp * kStride + hd * D;
        const int kb = gi >> 1, e0 = 2 * (gi & 1);
#pragma unroll
        for (int ee = 0; ee < 2; ee++) {
            const float* vp = lv + (16 * kb + 4 * g + e0 + ee) * kStride + r16;
#pragma unroll
            for (int db = 0; db < DB; db++) vfl[par][ee][db] = vp[16 * db];
        }
    };
    constexpr int kLPG2 = (NCH + 1) / 2;     // the loads of tile kt + 2 over groups 0 and 1, the stores of tile kt + 1 in group 2
    float* Pq = pp.P + (int64_t)b * pp.p_batch_stride + ((int64_t)qc * T) * H + h0 + hd;   // P[b, q, 0, h]
    // the probabilities of a tile: masked keys hold exp(-inf) = 0 exactly, also in the tiles above the diagonal
    auto store_p_direct = [&](const f32x4 (&pr)[2], int key0) {
        if (q < T) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                const int key = key0 + 16 * kb + 4 * g;
                if (PVEC) {
                    if (key < T) __builtin_nontemporal_store(pr[kb], reinterpret_cast<f32x4*>(Pq + key));
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (key + v < T) Pq[(int64_t)(key + v) * H] = pr[kb][v];
                }
            }
        }
    };
    // four heads per workgroup: this wave's head of (query r16, keys 32*kgp + 16*kb + 4*g + 0..3) into its plane of the
    // exchange buffer, one 128-bit write per key block (written as the fourth part of 4-float groups, the 64 lanes
    // of a write would share 8 banks); after a barrier a lane stores the four heads of a (query, key) as one word
    auto exchange_write = [&](const f32x4 (&pr)[2]) {
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
            *reinterpret_cast<f32x4*>(&lds_p[hd * kPPlane + r16 * kPStride + 32 * kgp + 16 * kb + 4 * g]) = pr[kb];
    };
    auto exchange_store = [&](int kt) {
#pragma unroll
        for (int i = 0; i < 16 * kFaKeys / kFaThreads; i++) {
            const int idx = tid + i * kFaThreads;
            const int qq = idx / kFaKeys, kk = idx % kFaKeys;
            const int key = kt * kFaKeys + kk;
            const float* src = &lds_p[qq * kPStride + kk];
            const f32x4 w = {src[0], src[kPPlane], src[2 * kPPlane], src[3 * kPPlane]};
            if (q0 + qq < T && key < T)
                __builtin_nontemporal_store(w, reinterpret_cast<f32x4*>(pp.P + (int64_t)b * pp.p_batch_stride + (((int64_t)(q0 + qq) * T + key) * H + h0)));
        }
    };
    stage_v(I0{}, 0, 0);
    static_for<0, NT>([&](auto ktc) {
        constexpr int kt = decltype(ktc)::value;
        if (kt < nkt_all) {
            constexpr int buf = kt & 1;
            using SetNow = std::integral_constant<int, kt & 1>;
            using SetNext = std::integral_constant<int, (kt + 1) & 1>;
            const int key0 = kt * kFaKeys + 32 * kgp;
            f32x4 pr[2];
#pragma unroll
            for (int kb = 0; kb < 2; kb++) pr[kb] = sc[kt][kb] * rl;
            if (kt < nkt) {
                const int kt2 = min(kt + 2, nkt - 1);
                static_for<0, 4>([&](auto gc) {
                    constexpr int gi = decltype(gc)::value;
                    constexpr int par = gi & 1;
                    using ParNext = std::integral_constant<int, par ^ 1>;
                    if constexpr (gi == 0) {
                        if (HG == 4) exchange_write(pr);
                        else store_p_direct(pr, key0);
                    }
                    if constexpr (gi == 2) {
                        store_all(SetNext{}, buf ^ 1);
                        if (HG == 4) {
                            __syncthreads();   // the four heads of every (query, key) of the tile are in the exchange buffer
                            exchange_store(kt);
                        }
                    }
                    if constexpr (gi < 3) {
                        stage_v(ParNext{}, gi + 1, buf);
                    } else {
                        __syncthreads();       // tile kt + 1 is in LDS, every wave has read tile kt (and the exchange buffer)
                        if (kt + 1 < nkt) stage_v(ParNext{}, 0, buf ^ 1);
                    }
                    if constexpr (gi < 2) {
                        static_for<0, kLPG2>([&](auto lc) {
                            constexpr int j = gi * kLPG2 + decltype(lc)::value;
                            if constexpr (j < NCH) load_one(SetNow{}, std::integral_constant<int, j>{}, rsrc_v, kt2);
                        });
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    constexpr int kb = gi >> 1, e0 = 2 * (gi & 1);
#pragma unroll
                    for (int ee = 0; ee < 2; ee++)
#pragma unroll
                        for (int db = 0; db < DB; db++)
                            acc_o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(vfl[par][ee][db], pr[kb][e0 + ee], acc_o[db], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                });
            } else if (HG == 4) {
                exchange_write(pr);
                __syncthreads();
                exchange_store(kt);
                __syncthreads();   // the exchange buffer is free again
            } else {
                store_p_direct(pr, key0);
            }
        }
    });

    // merge the two key halves of the output
    float* mg = &lds_t[0][0] + (w4 * 64 + lane);
    constexpr int kMergeStride = 64 * kFaQGroups;
    static_assert(4 * DB * 64 * kFaQGroups <= 2 * kFaKeys * kStride, "merge buffer must fit the tiles");
    if (kgp == 1) {
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int v = 0; v < 4; v++) mg[(4 * db + v) * kMergeStride] = acc_o[db][v];
    }
    __syncthreads();
    if (kgp == 1) return;
    if (q < T) {
        float* out = p.O + base + hd * D + (int64_t)q * p.nvec;
#pragma unroll
        for (int db = 0; db < DB; db++) {
            f32x4 o = acc_o[db];
#pragma unroll
            for (int v = 0; v < 4; v++) o[v] += mg[(4 * db + v) * kMergeStride];
            *reinterpret_cast<f32x4*>(out + 16 * db + 4 * g) = o;
        }
    }
}

}  // namespace

bool attention_fused_applies(const float* q, const float* k, const float* v, const float* o, int64_t ntimes,
                             int64_t nvec, int64_t nhead, int64_t npiece) {
    // the kernel writes its output with the row stride of the inputs; the output of the separate calls is
    // [nbat, ntimes, nhead, npiece], which is the same thing only when the heads fill the vector
    return nhead * npiece == nvec &&
           npiece % 16 == 0 && npiece >= 16 && npiece <= 128 && nvec % 4 == 0 && ntimes >= 1 && ntimes <= kMaxDim &&
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
    if (qtiles * nbat * nhead > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "attention: grid too large");
    const dim3 grid((unsigned)(qtiles * nbat * nhead));
    switch (npiece / 16) {
    case 1: attention_fused_kernel<1><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    case 2: attention_fused_kernel<2><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    case 3: attention_fused_kernel<3><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    case 4: attention_fused_kernel<4><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    case 5: attention_fused_kernel<5><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    case 6: attention_fused_kernel<6><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    case 7: attention_fused_kernel<7><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    default: attention_fused_kernel<8><<<grid, dim3(kFaThreads), 0, stream>>>(p); break;
    }
    return check_launch("attention_fused_kernel");
}

bool attention_probs_applies(const float* q, const float* k, const float* v, const float* o, const float* pp,
                             int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece) {
    return attention_fused_applies(q, k, v, o, ntimes, nvec, nhead, npiece) && ntimes <= 1024 &&
           (reinterpret_cast<uintptr_t>(pp) & 3u) == 0;
}

template <int DB, int HG>
static void launch_probs(const ProbsParams& p, bool pvec, int64_t ntimes, dim3 grid, hipStream_t stream) {
    const dim3 block(kFaThreads);
    constexpr bool kVecOk = HG == 1;
    if (ntimes <= 256) {
        if (kVecOk && pvec) attention_probs_kernel<DB, 4, HG, kVecOk><<<grid, block, 0, stream>>>(p);
        else attention_probs_kernel<DB, 4, HG, false><<<grid, block, 0, stream>>>(p);
    } else if (ntimes <= 512) {
        if (kVecOk && pvec) attention_probs_kernel<DB, 8, HG, kVecOk><<<grid, block, 0, stream>>>(p);
        else attention_probs_kernel<DB, 8, HG, false><<<grid, block, 0, stream>>>(p);
    } else if constexpr (!(HG == 4 && DB == 4)) {
        // (head sizes above 96 with more than 512 keys: the variant with 128-bit stores of P does not fit its
        // registers; one head per batch entry stores its probabilities element by element there)
        if (kVecOk && pvec && DB <= 6) attention_probs_kernel<DB, 16, HG, (kVecOk && DB <= 6)><<<grid, block, 0, stream>>>(p);
        else attention_probs_kernel<DB, 16, HG, false><<<grid, block, 0, stream>>>(p);
    }
}

// four heads per workgroup: head counts in whole fours and rows of the probabilities that allow 128-bit stores
// (head sizes up to 64: the tiles of four heads side by side must fit LDS twice)
// (and not head size 64 beyond 512 keys: 128 score registers next to the staging registers of the wide tiles do not fit)
static bool probs_four_heads(const float* pp, int64_t nhead, int64_t npiece, int64_t ntimes) {
    return nhead % 4 == 0 && npiece <= 64 && !(npiece == 64 && ntimes > 512) && aligned16(pp);
}

bool attention_probs_four_heads(const float* pp, int64_t ntimes, int64_t nhead, int64_t npiece) {
    return probs_four_heads(pp, nhead, npiece, ntimes);
}

// Beyond 512 keys a wave keeps 128 score registers, and with one head per workgroup and few workgroups (a batch of
// one or two) the launch neither fills the compute units nor hides its latencies: the three separate calls, whose
// kernels spread the same work over more workgroups, are faster there.  Measured at 1000 keys, one launch | three
// calls, us: 8 x 1 head of 128 100.0 | 61.7, of 96 61.3 | 57.1 (of 64: 45.0 | 52.6, stays); 2 x 4 heads of 64 82.0 | 60.9,
// 1 x 8 heads of 64 83.1 | 53.8, of 96 97.5 | 85.3, of 128 110.0 | 88.9; 4 x 2 heads of 128 98.1 | 73.7, 1 x 6 heads of 128
// 105.2 | 80.9; with workgroups for more than half of the compute units the one launch stays (1 x 12 heads of 64:
// 91.7 | 102.7, 3 x 3 heads of 128: 102.6 | 115.4).
bool attention_probs_pays(const float* pp, int64_t nbat, int64_t ntimes, int64_t nhead, int64_t npiece) {
    if (ntimes <= 512 || probs_four_heads(pp, nhead, npiece, ntimes)) return true;
    if (nbat * nhead * ((ntimes + kFaQ - 1) / kFaQ) > compute_units() / 2) return true;
    return !((nhead == 1 && npiece >= 96) || (nhead >= 2 && npiece >= 64));
}

int launch_attention_probs(float* o, float* pp, const float* q, const float* k, const float* v, int64_t nbat,
                           int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, const float* hcoef, int masked,
                           hipStream_t stream) {
    ProbsParams p{};
    p.f.Q = q; p.f.K = k; p.f.V = v; p.f.O = o; p.f.coef = hcoef;
    p.f.nvec = nvec; p.f.batch_stride = ntimes * nvec;
    p.f.ntimes = (int)ntimes; p.f.nhead = (int)nhead; p.f.npiece = (int)npiece;
    p.f.masked = masked;
    p.P = pp; p.p_batch_stride = ntimes * ntimes * nhead;
    const bool four = probs_four_heads(pp, nhead, npiece, ntimes);
    const int64_t qtiles = four ? (ntimes + 15) / 16 : (ntimes + kFaQ - 1) / kFaQ;
    const int64_t wgs = qtiles * nbat * (four ? nhead / 4 : nhead);
    if (wgs > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "attention: grid too large");
    const dim3 grid((unsigned)wgs);
    const bool pvec = nhead == 1 && ntimes % 4 == 0 && aligned16(pp);
    if (four) {
        switch (npiece / 16) {
        case 1: launch_probs<1, 4>(p, false, ntimes, grid, stream); break;
        case 2: launch_probs<2, 4>(p, false, ntimes, grid, stream); break;
        case 3: launch_probs<3, 4>(p, false, ntimes, grid, stream); break;
        default: launch_probs<4, 4>(p, false, ntimes, grid, stream); break;
        }
    } else {
        switch (npiece / 16) {
        case 1: launch_probs<1, 1>(p, pvec, ntimes, grid, stream); break;
        case 2: launch_probs<2, 1>(p, pvec, ntimes, grid, stream); break;
        case 3: launch_probs<3, 1>(p, pvec, ntimes, grid, stream); break;
        case 4: launch_probs<4, 1>(p, pvec, ntimes, grid, stream); break;
        case 5: launch_probs<5, 1>(p, pvec, ntimes, grid, stream); break;
        case 6: launch_probs<6, 1>(p, pvec, ntimes, grid, stream); break;
        case 7: launch_probs<7, 1>(p, pvec, ntimes, grid, stream); break;
        default: launch_probs<8, 1>(p, pvec, ntimes, grid, stream); break;
        }
    }
    return check_launch("attention_probs_kernel");
}

}  // namespace kai
