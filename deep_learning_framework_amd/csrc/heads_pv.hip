// Products of the head-interleaved attention tensor P[nbat, T, T, H] (head index innermost) with a
// [nbat, T, H*D] tensor, for several heads per batch entry:
//
//   plain       C[b,q,h,:] = sum_k P[b,q,k,h] * X[b,k,h,:]   (mix_values, mult_on_heads_backward)
//   transposed  C[b,k,h,:] = sum_q P[b,q,k,h] * X[b,q,h,:]   (mix_values_backward_value)
//
// One head at a time, P is a matrix whose elements lie H floats apart in both directions: the tiled kernel
// loads it 4 bytes at a time, and the workgroups of the H heads fetch every 32-byte sector H times.  Here
// a workgroup owns 32 output rows, 32 output columns and FOUR heads, one per wave: a P tile of 32 x 32
// positions is loaded as 128-bit pieces (the four heads of a position) and split into four planes in LDS,
// the matching X tile (32 reduction rows x 4 heads x 32 columns) goes into four planes as well, and each
// wave runs v_mfma_f32_32x32x2_f32 on its own pair of planes.  Tiles are staged through registers four
// deep (a tile computes for ~0.4 us, a global load takes 1-2 us) and two LDS buffers.
//
// Workgroups that read the same P sectors (the other head groups and column blocks of the same rows) are
// numbered so that they land on one XCD and share its L2.
#include "gemm_host.h"

namespace kai {
namespace {

constexpr int kHpTile = 32;       // output rows = reduction steps per tile = output columns
constexpr int kHpHeads = 4;       // heads per workgroup, one per wave
constexpr int kHpDepth = 4;       // tiles in flight in registers
constexpr int kHpPStride = 36;    // floats per row of a P plane (128-bit rows, conflict-free reads along the row)
constexpr int kHpXStride = 32;
constexpr int kHpThreads = 64 * kHpHeads;
constexpr int kHpChunks = kHpTile * kHpTile / kHpThreads;   // 128-bit pieces per thread, tile and operand

struct HeadsPvParams {
    const float* P;
    const float* X;
    float* C;
    int T, H, D;
    int row_tiles;    // T / 32
    int share;        // workgroups per (batch entry, row tile): head groups x column blocks
    int col_blocks;   // D / 32
    int remap;        // nbat * row_tiles is a multiple of 8: the XCD-aware numbering applies
};

template <bool TRANS>
__global__ void __launch_bounds__(kHpThreads) heads_pv_kernel(HeadsPvParams p) {
    __shared__ float lds_p[2][kHpHeads][kHpTile * kHpPStride];
    __shared__ float lds_x[2][kHpHeads][kHpTile * kHpXStride];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;

    // consecutive workgroup numbers go round the XCDs: the `share` workgroups of one unit (batch entry,
    // row tile) take consecutive slots of ONE XCD
    int unit, member;
    if (p.remap) {
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        unit = (slot / p.share) * 8 + xcd;
        member = slot % p.share;
    } else {
        unit = blockIdx.x / p.share;
        member = blockIdx.x % p.share;
    }
    const int b = unit / p.row_tiles, o0 = (unit % p.row_tiles) * kHpTile;
    const int g = member / p.col_blocks, db = member % p.col_blocks;
    const int64_t T = p.T, H = p.H, HD = (int64_t)p.H * p.D;
    const float* Pb = p.P + (int64_t)b * T * T * H + kHpHeads * g;
    const float* Xb = p.X + (int64_t)b * T * HD + (int64_t)(kHpHeads * g) * p.D + kHpTile * db;
    const int nkt = p.T / kHpTile;

    // per-thread coordinates of the 128-bit pieces: P piece c = position (second axis pq, third axis pk),
    // X piece c = (reduction row xr, head xh, four columns from 4 * xd).  Buffer loads: resource = this batch
    // entry's part of P / X from the workgroup's heads on, lane offsets constant, tile offset scalar, so that a
    // tile costs no vector instruction for addresses (they would take their time from the fp32 MFMAs).
    int poff[kHpChunks], xoff[kHpChunks];   // bytes
    int plds[kHpChunks], xlds[kHpChunks];
#pragma unroll
    for (int c = 0; c < kHpChunks; c++) {
        const int idx = tid + kHpThreads * c;
        const int pk = idx & 31, pq = idx >> 5;
        // plain: rows pq are the workgroup's output rows, pk walks the reduction; transposed: the other way round
        poff[c] = (int)((TRANS ? ((int64_t)pq * T + (o0 + pk)) * H : ((int64_t)(o0 + pq) * T + pk) * H) * 4);
        plds[c] = pq * kHpPStride + pk;
        const int xd = idx & 7, xh = (idx >> 3) & 3, xr = idx >> 5;
        xoff[c] = (int)(((int64_t)xr * HD + (int64_t)xh * p.D + 4 * xd) * 4);
        xlds[c] = xh * (kHpTile * kHpXStride) + xr * kHpXStride + 4 * xd;
    }
    const int pstep = (int)((TRANS ? (int64_t)kHpTile * T * H : (int64_t)kHpTile * H) * 4);   // one tile along the reduction
    const int xstep = (int)((int64_t)kHpTile * HD * 4);
    auto uniform_ptr = [](const float* q) -> float* {
        const uint64_t a = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
    };
    // (the host keeps a batch entry of P and of X below 2 GiB)
    const __amdgpu_buffer_rsrc_t rsrc_p =
        __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(Pb), 0, (int)(T * T * H * 4 - kHpHeads * g * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
        uniform_ptr(Xb), 0, (int)(T * HD * 4 - ((int64_t)(kHpHeads * g) * p.D + kHpTile * db) * 4), 0x00020000);

    f32x4 rp[kHpDepth][kHpChunks], rx[kHpDepth][kHpChunks];
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;

    // every load is unconditional: a tile index past the end repeats the last tile, which is never stored
    auto load_into = [&](int kt, f32x4(&dp)[kHpChunks], f32x4(&dx)[kHpChunks]) {
        const int ktc = kt < nkt ? kt : nkt - 1;
#pragma unroll
        for (int c = 0; c < kHpChunks; c++)
            dp[c] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_p, poff[c], ktc * pstep, 0));
#pragma unroll
        for (int c = 0; c < kHpChunks; c++)
            dx[c] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, xoff[c], ktc * xstep, 0));
    };
    auto store_lds = [&](int buf, const f32x4(&sp)[kHpChunks], const f32x4(&sx)[kHpChunks]) {
#pragma unroll
        for (int c = 0; c < kHpChunks; c++) {
            const f32x4 v = sp[c];
#pragma unroll
            for (int hh = 0; hh < kHpHeads; hh++) lds_p[buf][hh][plds[c]] = v[hh];
            *reinterpret_cast<f32x4*>(&lds_x[buf][0][0] + xlds[c]) = sx[c];
        }
    };
    // prologue: tiles 0 .. depth-1 into the register slots, tile 0 on to LDS, its slot refilled
    static_for<0, kHpDepth>([&](auto dc) {
        constexpr int d = decltype(dc)::value;
        load_into(d, rp[d], rx[d]);
    });
    store_lds(0, rp[0], rx[0]);
    load_into(kHpDepth, rp[0], rx[0]);
    __syncthreads();
    // At the top of tile kt: LDS[kt & 1] holds tile kt, slot (kt + j) % depth holds tile kt + j, j = 1 .. depth.
    // The next tile goes to the free LDS buffer between the MFMAs of this one, its slot is refilled behind them.
    // One tile: the MFMAs of tile kt (LDS[cur]) with everything else between them -- a wave issues its 16
    // dependent MFMAs 64 cycles apart and has those gaps to spend: the operands of step s + 1 are read while
    // step s multiplies, and piece s of the next tile goes from its register slot to the other LDS buffer behind
    // the MFMAs of step s (written as one block before the MFMAs, the 12 LDS stores of a tile and their waits
    // were a phase of their own: 1.2 us per tile against 0.43 us of MFMAs).
    auto read_ops = [&](const float* pl, const float* xl, int s, float (&a)[4], float (&bq)[4]) {
        if (!TRANS) {
            const f32x4 av = *reinterpret_cast<const f32x4*>(pl + l32 * kHpPStride + 8 * s + 4 * half);
#pragma unroll
            for (int e = 0; e < 4; e++) a[e] = av[e];
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) a[e] = pl[(8 * s + 4 * half + e) * kHpPStride + l32];
        }
#pragma unroll
        for (int e = 0; e < 4; e++) bq[e] = xl[(8 * s + 4 * half + e) * kHpXStride + l32];
    };
    static_assert(kHpChunks == kHpTile / 8, "one piece of the next tile per group of four MFMAs");
    auto stage = [&](auto dc, int kt, bool guard) {
        constexpr int d = decltype(dc)::value;
        constexpr int nslot = (d + 1) % kHpDepth;
        const int cur = kt & 1;
        const bool st = !guard || kt + 1 < nkt;   // the same for every thread
        const float* pl = lds_p[cur][wave];
        const float* xl = lds_x[cur][wave];
        float a[2][4], bq[2][4];
        read_ops(pl, xl, 0, a[0], bq[0]);
        static_for<0, kHpChunks>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            constexpr int o = s & 1;
            if constexpr (s + 1 < kHpChunks) read_ops(pl, xl, s + 1, a[o ^ 1], bq[o ^ 1]);
            const f32x4 v = rp[nslot][s];
            __builtin_amdgcn_sched_barrier(0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[o][0], bq[o][0], acc, 0, 0, 0);
            if (st) {
                lds_p[cur ^ 1][0][plds[s]] = v[0];
                lds_p[cur ^ 1][1][plds[s]] = v[1];
            }
            __builtin_amdgcn_sched_barrier(0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[o][1], bq[o][1], acc, 0, 0, 0);
            if (st) {
                lds_p[cur ^ 1][2][plds[s]] = v[2];
                lds_p[cur ^ 1][3][plds[s]] = v[3];
            }
            __builtin_amdgcn_sched_barrier(0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[o][2], bq[o][2], acc, 0, 0, 0);
            if (st) *reinterpret_cast<f32x4*>(&lds_x[cur ^ 1][0][0] + xlds[s]) = rx[nslot][s];
            __builtin_amdgcn_sched_barrier(0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[o][3], bq[o][3], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        load_into(kt + 1 + kHpDepth, rp[nslot], rx[nslot]);
        __syncthreads();
    };
    int kt0 = 0;
    for (; kt0 + kHpDepth <= nkt; kt0 += kHpDepth)
        static_for<0, kHpDepth>([&](auto dc) { stage(dc, kt0 + decltype(dc)::value, false); });
    static_for<0, kHpDepth>([&](auto dc) {
        if (kt0 + decltype(dc)::value < nkt) stage(dc, kt0 + decltype(dc)::value, true);
    });

    // acc[r] = C[row 8 * (r / 4) + 4 * half + r % 4][column l32] of this wave's head
    float* Cb = p.C + ((int64_t)b * T + o0) * HD + (int64_t)(kHpHeads * g + wave) * p.D + kHpTile * db + l32;
#pragma unroll
    for (int r = 0; r < 16; r++) Cb[(int64_t)(8 * (r >> 2) + 4 * half + (r & 3)) * HD] = acc[r];
}

}  // namespace

// d describes one head's product with the batch index running over (batch entry, head): see the callers in
// kai_abi.hip.  Recognised: P as A with element stride H in one direction and T*H in the other, X as B with
// unit column stride, C laid out like X, square P.
bool heads_pv_applies(const GemmDesc& d) {
    const int64_t H = d.bdiv, T = d.M, D = d.N;
    if (H < kHpHeads || H % kHpHeads != 0 || d.nbatch % H != 0 || d.K != T || T % kHpTile != 0 || D % kHpTile != 0)
        return false;
    const bool plain = d.a_ks == H && d.a_rs == T * H, trans = d.a_rs == H && d.a_ks == T * H;
    if (!plain && !trans) return false;
    if (d.a_bs1 != 1 || d.a_bs0 != T * T * H) return false;
    if (d.b_rs != 1 || d.b_ks != H * D || d.b_bs1 != D || d.b_bs0 != T * H * D) return false;
    if (d.c_cs != 1 || d.c_rs != H * D || d.c_bs1 != D || d.c_bs0 != T * H * D) return false;
    if (d.acc || d.bias || d.C2 || d.act != kActNone || d.has_alpha || d.rowsum || d.k_part != 0) return false;
    if (!aligned16(d.A) || !aligned16(d.B)) return false;
    return T * T * H * 4 < (1ll << 31) && T * H * D * 4 < (1ll << 31);
}

int launch_heads_pv(const GemmDesc& d, hipStream_t stream) {
    const int64_t H = d.bdiv, T = d.M, D = d.N, nbat = d.nbatch / H;
    HeadsPvParams p;
    p.P = d.A; p.X = d.B; p.C = d.C;
    p.T = (int)T; p.H = (int)H; p.D = (int)D;
    p.row_tiles = (int)(T / kHpTile);
    p.col_blocks = (int)(D / kHpTile);
    p.share = (int)((H / kHpHeads) * p.col_blocks);
    const int64_t units = nbat * p.row_tiles, blocks = units * p.share;
    if (blocks <= 0) return KAI_OK;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: grid too large");
    p.remap = units % 8 == 0;
    if (d.a_ks == H) heads_pv_kernel<false><<<dim3((unsigned)blocks), dim3(kHpThreads), 0, stream>>>(p);
    else heads_pv_kernel<true><<<dim3((unsigned)blocks), dim3(kHpThreads), 0, stream>>>(p);
    return check_launch("heads_pv_kernel");
}

}  // namespace kai
