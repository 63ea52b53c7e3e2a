// Products with a short reduction (K <= 64) and both operands K-contiguous:
// C[M,N] = A[M,K] . B[N,K]^T, the shape of attention scores (K = head size) and of the gradient
// of attention probabilities.
//
// Such a product writes 4 bytes for every 2K <= 128 flops: it is bound by how fast C streams
// out, not by the matrix cores, and a tiled kernel that loads, computes and then stores runs its
// three phases one after the other.  Here a workgroup keeps a panel of 128 rows of B in LDS for its
// whole life and streams row tiles of A (128 rows, all of K) past it through two LDS buffers:
// while the matrix cores work on tile t the loads of tile t+1 are in flight, and the stores of
// tile t drain under the work on tile t+1.  The host picks the run of tiles per workgroup so that
// the grid still covers the compute units.
//
// B is held column-contiguous in LDS (transposed on the way in) so that one 128-bit read yields the
// same row of four interleaved 32-column blocks; a lane then owns four consecutive columns of C
// and stores them as one 128-bit word, 512 contiguous bytes per row and half wave.
#include "gemm_host.h"

namespace kai {

namespace {

constexpr int kSkWaves = 4;
constexpr int kSkThreads = 64 * kSkWaves;
constexpr int kSkBM = 32 * kSkWaves;   // rows of A per tile: one 32-row block per wave
constexpr int kSkBN = 128;             // 4 interleaved blocks of 32 columns
constexpr int kSkK = 64;               // longest reduction
constexpr int kSkMaxRun = 8;           // most row tiles one workgroup walks

using TileA = TileShape<true, kSkBM, kSkK>;    // [128][68]
using TileB = TileShape<false, kSkBN, kSkK>;   // [64][132]

// Loads a panel of `ROWS` rows x K (K-contiguous in memory, row stride ld) into registers: chunk c
// of a thread covers row c / 16, k = 4 * (c % 16) .. +3.  Every address is clamped into the matrix,
// so the loads carry no branches and all of them are in flight together; mask_panel() then zeroes
// what lies beyond the matrix.
template <int ROWS, bool VEC>
__device__ __forceinline__ void load_panel(f32x4 (&reg)[ROWS * kSkK / 4 / kSkThreads], const float* __restrict__ base,
                                           int64_t ld, int rows_left, int K, int tid) {
    constexpr int NCH = ROWS * kSkK / 4 / kSkThreads;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * kSkThreads;
        const int r = c >> 4;
        const int k = (c & 15) * 4;
        const float* row = base + (int64_t)min(r, rows_left - 1) * ld;
        if (VEC) {   // K % 4 == 0: a chunk is inside or outside as a whole
            reg[i] = *reinterpret_cast<const f32x4*>(row + (k < K ? k : 0));
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) reg[i][j] = row[min(k + j, K - 1)];
        }
    }
}

template <int ROWS>
__device__ __forceinline__ void mask_panel(f32x4 (&reg)[ROWS * kSkK / 4 / kSkThreads], int rows_left, int K, int tid) {
    constexpr int NCH = ROWS * kSkK / 4 / kSkThreads;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * kSkThreads;
        const int r = c >> 4;
        const int k = (c & 15) * 4;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // bitwise, so that the compiler keeps the loads unconditional
            const int keep = (r < rows_left && k + j < K) ? -1 : 0;
            const float x = reg[i][j];
            reg[i][j] = __int_as_float(__float_as_int(x) & keep);
        }
    }
}

// NG: groups of 8 reduction steps that are computed (K <= 8 * NG; the panels are zero beyond K).
// The epilogue only scales and stores (no accumulation into C, bias, second output or activation: products that
// ask for those run the tiled kernels), so nothing in the loop waits on a load issued after a store.
// Grid: one dimension over (batch, column panel, run), where a run is p.group_m consecutive row
// tiles.  Hardware deals consecutive workgroup ids round-robin over the 8 XCDs; ids are renumbered
// so that each XCD walks a contiguous range, which keeps the workgroups of one batch entry (they
// share its A and B) behind one L2.
// WHOLE: row and column counts in whole tiles, K = 64, 128-bit loads and stores: no clamp, mask or branch is left.
template <int NG, bool WHOLE>
__global__ void __launch_bounds__(kSkThreads) shortk_nt_kernel(const GemmParams p) {
    static_assert(!WHOLE || NG * 8 == kSkK, "whole panels: all 64 reduction steps");
    __shared__ __attribute__((aligned(16))) float lds_a[2][TileA::kFloats];
    __shared__ __attribute__((aligned(16))) float lds_b[TileB::kFloats];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const int wm0 = wave * 32;

    const int run_len = p.group_m;
    const int runs = (p.tiles_m + run_len - 1) / run_len;
    const int per_batch = runs * p.tiles_n;
    const int total = gridDim.x;
    int id = blockIdx.x;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    const int z = id / per_batch;
    const int in_batch = id - z * per_batch;
    const int tn = in_batch / runs;
    const int tm_first = (in_batch - tn * runs) * run_len;
    const int ntile = min(run_len, p.tiles_m - tm_first);
    const int n0 = tn * kSkBN;
    const int zq = z / p.bdiv, zr = z % p.bdiv;
    const float* __restrict__ Az = p.A + zq * p.a_bs0 + zr * p.a_bs1;
    const float* __restrict__ Bb = p.B + zq * p.b_bs0 + zr * p.b_bs1 + (int64_t)n0 * p.b_rs;
    const int64_t c_off = zq * p.c_bs0 + zr * p.c_bs1;

    // the two scalars of the epilogue are fetched before any store is in flight
    float alpha = p.has_alpha ? (p.alpha ? *p.alpha : 0.f) : 1.f;
    float leaky = p.leaky ? *p.leaky : 0.f;
    // this batch entry's C as a buffer (used where p.c_buf says so; the host has checked that it spans less than 2 GiB)
    // (the halves as unsigned 32-bit values before they are joined: readfirstlane returns a signed int, and a low
    // half with its top bit set would otherwise fill the high half with ones)
    const uint64_t c_addr = reinterpret_cast<uint64_t>(p.C + c_off);
    const uint32_t c_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)c_addr);
    const uint32_t c_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(c_addr >> 32));
    const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<float*>(((uint64_t)c_hi << 32) | c_lo), 0,
        p.c_buf ? (int)((((int64_t)p.M - 1) * p.c_rs + p.N) * 4) : 0, 0x00020000);

    constexpr int NCHA = kSkBM * kSkK / 4 / kSkThreads;
    constexpr int NCHB = kSkBN * kSkK / 4 / kSkThreads;
    const bool vec = WHOLE || (p.a_vec && p.b_vec && (p.K & 3) == 0);
    f32x4 ra[NCHA];

    auto load_a = [&](int tm) {
        const int m0 = tm * kSkBM;
        const float* ab = Az + (int64_t)m0 * p.a_rs;
        if (WHOLE) load_panel<kSkBM, true>(ra, ab, p.a_rs, kSkBM, kSkK, tid);
        else if (vec) load_panel<kSkBM, true>(ra, ab, p.a_rs, p.M - m0, p.K, tid);
        else load_panel<kSkBM, false>(ra, ab, p.a_rs, p.M - m0, p.K, tid);
    };
    auto stage_a = [&](int tm, int buf) {
        const int m0 = tm * kSkBM;
        if (!WHOLE && (p.M - m0 < kSkBM || p.K < kSkK)) mask_panel<kSkBM>(ra, p.M - m0, p.K, tid);
        store_tile_lds<true, kSkBM, kSkK, kSkThreads>(lds_a[buf], ra, tid);
    };

    {
        f32x4 rb[NCHB];
        if (WHOLE) load_panel<kSkBN, true>(rb, Bb, p.b_rs, kSkBN, kSkK, tid);
        else if (vec) load_panel<kSkBN, true>(rb, Bb, p.b_rs, p.N - n0, p.K, tid);
        else load_panel<kSkBN, false>(rb, Bb, p.b_rs, p.N - n0, p.K, tid);
        load_a(tm_first);
        __builtin_amdgcn_sched_barrier(0);
        if (!WHOLE && (p.N - n0 < kSkBN || p.K < kSkK)) mask_panel<kSkBN>(rb, p.N - n0, p.K, tid);
        // B goes in transposed: element (row n, k) to [k][n]
#pragma unroll
        for (int i = 0; i < NCHB; i++) {
            const int c = tid + i * kSkThreads;
            const int n = c >> 4;
            const int k = (c & 15) * 4;
#pragma unroll
            // plain epilogue: the scale goes into the panel once per workgroup instead of into every output (64
            // multiplies per lane and tile, which would take their time from the MFMAs)
            for (int j = 0; j < 4; j++) lds_b[(k + j) * TileB::kStride + n] = rb[i][j] * alpha;
        }
        stage_a(tm_first, 0);
    }
    alpha = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(alpha)));
    leaky = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(leaky)));
    __syncthreads();

#pragma nounroll
    for (int it = 0; it < ntile; it++) {
        const int tm = tm_first + it;
        const int m0 = tm * kSkBM;
        const bool more = it + 1 < ntile;
        // in flight during the matrix work below (whole tiles: unconditional, after the last tile it comes again)
        if (WHOLE) load_a(min(tm + 1, tm_first + ntile - 1));
        else if (more) load_a(tm + 1);
        const float* la = lds_a[it & 1];

        f32x16 acc[1][4];
        const bool rows_inside = WHOLE || m0 + wm0 < p.M;   // wave-uniform
        if (rows_inside) {
            static_for<0, NG>([&](auto kgc) {
                constexpr int kg = decltype(kgc)::value;
                Frag<true, 1> fa;
                Frag<false, 4> fb;
                read_frag<true, 1, kSkBM, kSkK>(fa, la, wm0, kg, l32, half);
                read_frag<false, 4, kSkBN, kSkK>(fb, lds_b, 0, kg, l32, half);
                static_for<0, 4>([&](auto tc) {
                    constexpr int t = decltype(tc)::value;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        // the first product of an accumulator starts from a zero constant: no 64 moves to clear them
                        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                        acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.get(0, t), fb.get(j, t),
                                                                        (kg == 0 && t == 0) ? zero : acc[0][j], 0, 0, 0);
                    }
                });
            });
        }
        // the next tile moves to LDS before this tile's stores are issued: the wait for its loads
        // then never includes a store
        if (WHOLE || more) stage_a(min(tm + 1, tm_first + ntile - 1), (it + 1) & 1);

        if (rows_inside) {
            {
                float* C = p.C + c_off;
                const int col = n0 + 4 * l32;
                static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    const int row = m0 + wm0 + 8 * (r >> 2) + 4 * half + (r & 3);
                    const f32x4 o = {acc[0][0][r], acc[0][1][r], acc[0][2][r], acc[0][3][r]};   // scaled through B
                    float* out = C + (int64_t)row * p.c_rs + col;
                    if (WHOLE) {
                        __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(out));
                    } else if (row < p.M) {
                        if (p.c_vec) {   // N % 4 == 0: the four columns are inside or outside together
                            // streaming: whole 512-byte rows that this kernel never reads again; otherwise the
                            // dirty lines pile up in L2 and are written back after the last wave has ended
                            if (col < p.N) __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(out));
                        } else if (p.c_buf && col + 4 <= p.N) {
                            // rows of C off 16-byte lines (511 keys): a buffer store needs 4-byte alignment only
                            __builtin_amdgcn_raw_buffer_store_b128(
                                __builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int, o),
                                rsrc_c, (int)(((int64_t)row * p.c_rs + col) * 4), 0, 0);
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; j++)
                                if (col + j < p.N) out[j] = o[j];
                        }
                    }
                });
            }
        }
        __syncthreads();
    }
}


// ---- the same product for several heads interleaved in C -------------------------------------------
//
// The engine keeps attention scores as P[batch, q, k, head] with the head index innermost
// (vtensor.cpp:3005 of the reference), so the product of one head writes 4 bytes at a stride of
// 4 * heads.  Here the four accumulators of a wave are four HEADS of the same 32 x 32 block of
// (q, k): a lane then holds P[b, q, k, h .. h+3] and stores it as one 128-bit word.  A workgroup keeps
// the rows of B (keys) of its 32-column panel for the four heads in LDS and streams the rows of A
// (queries), one head slice of a 128-row tile at a time, through two LDS buffers; the stores of a
// tile drain under the work on the next one.
//
// Batch index z = outer * bdiv + head (bdiv heads): A and B of head h start h * a_bs1 / h * b_bs1 past
// the outer entry, C at + h (c_bs1 == 1) with element stride c_cs == bdiv.
constexpr int kShHeads = 4;     // heads per workgroup
constexpr int kShBN = 32;       // keys per workgroup

using TileBh = TileShape<true, kShBN, kSkK>;   // [32][68]

// WHOLE: query and key counts in whole tiles, K = 64, 128-bit loads: no clamp, mask or branch is left in the
// loop, which lets the compiler count the loads and stores in flight exactly (behind a branch it waits for all).
// PAIR: one LDS buffer for the A slices instead of two, so that two workgroups share a compute unit and one
// computes while the other waits for its stores (a second barrier per step lets the buffer be overwritten).
// ONE: the workgroup has one query tile (four steps): no slice is requested or staged beyond the fourth, at
// compile time (the unconditional form would request three surplus slices, 96 KB per workgroup, for the four it needs).
template <int NG, bool WHOLE, bool PAIR, bool ONE = false>
__global__ void __launch_bounds__(kSkThreads, PAIR ? 2 : 1) shortk_heads_kernel(const GemmParams p) {
    static_assert(!WHOLE || NG * 8 == kSkK, "whole panels hold all 64 reduction steps");
    static_assert(!ONE || WHOLE, "the one-tile form exists for whole tiles");
    __shared__ __attribute__((aligned(16))) float lds_a[PAIR ? 1 : 2][TileA::kFloats];
    __shared__ __attribute__((aligned(16))) float lds_b[kShHeads][TileBh::kFloats];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const int wm0 = wave * 32;

    // grid: (outer batch, key panel, head group, run of query tiles), renumbered XCD-contiguous
    const int run_len = p.group_m;
    const int runs = (p.tiles_m + run_len - 1) / run_len;
    const int hgroups = p.bdiv / kShHeads;
    const int per_batch = runs * p.tiles_n * hgroups;
    const int total = gridDim.x;
    int id = blockIdx.x;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    const int zq = id / per_batch;
    int rest = id - zq * per_batch;
    const int tn = rest / (runs * hgroups);
    rest -= tn * runs * hgroups;
    const int hg = rest / runs;
    const int tm_first = (rest - hg * runs) * run_len;
    const int ntile = min(run_len, p.tiles_m - tm_first);
    const int n0 = tn * kShBN;
    const int h0 = hg * kShHeads;
    const float* __restrict__ Az = p.A + zq * p.a_bs0 + h0 * p.a_bs1;
    const float* __restrict__ Bz = p.B + zq * p.b_bs0 + h0 * p.b_bs1 + (int64_t)n0 * p.b_rs;
    float* __restrict__ Cz = p.C + zq * p.c_bs0 + h0;

    float alpha = p.has_alpha ? (p.alpha ? *p.alpha : 0.f) : 1.f;

    constexpr int NCHA = kSkBM * kSkK / 4 / kSkThreads;   // 8
    constexpr int NCHB = kShBN * kSkK / 4 / kSkThreads;   // 2
    const bool vec = WHOLE || (p.a_vec && p.b_vec && (p.K & 3) == 0);
    // Whole tiles: the slices are requested three steps ahead into a ring of four register sets, set s % 4 for
    // step s.  The counter a wave waits on for its loads also counts its stores, in order: a slice requested
    // after a tile's stores is waited for only after those stores have drained, and the matrix cores idle
    // meanwhile; this way the slices of the next tile's first three steps are requested before the stores.
    // (With the edge handling in the loop the compiler waits for everything in flight at every step anyway, and
    // the extra requests only cost: those variants stay one step ahead.)
    f32x4 ra[WHOLE ? kShHeads : 1][NCHA];
    static_assert(kShHeads == 4, "the ring of staged slices has one set per head of the group");
    constexpr int AHEAD = WHOLE ? 3 : 1;

    // step s = tile * 4 + head: the A slice of head (s & 3) of query tile tm_first + (s >> 2)
    auto load_a = [&](int s, auto setc) {
        const int m0 = (tm_first + (s >> 2)) * kSkBM;
        const float* ab = Az + (s & 3) * p.a_bs1 + (int64_t)m0 * p.a_rs;
        if (WHOLE) load_panel<kSkBM, true>(ra[decltype(setc)::value], ab, p.a_rs, kSkBM, kSkK, tid);
        else if (vec) load_panel<kSkBM, true>(ra[decltype(setc)::value], ab, p.a_rs, p.M - m0, p.K, tid);
        else load_panel<kSkBM, false>(ra[decltype(setc)::value], ab, p.a_rs, p.M - m0, p.K, tid);
    };
    auto stage_a = [&](int s, int buf, auto setc) {
        const int m0 = (tm_first + (s >> 2)) * kSkBM;
        if (!WHOLE && (p.M - m0 < kSkBM || p.K < kSkK)) mask_panel<kSkBM>(ra[decltype(setc)::value], p.M - m0, p.K, tid);
        store_tile_lds<true, kSkBM, kSkK, kSkThreads>(lds_a[PAIR ? 0 : buf], ra[decltype(setc)::value], tid);
    };

    {
        f32x4 rb[kShHeads][NCHB];
#pragma unroll
        for (int j = 0; j < kShHeads; j++) {
            if (WHOLE) load_panel<kShBN, true>(rb[j], Bz + j * p.b_bs1, p.b_rs, kShBN, kSkK, tid);
            else if (vec) load_panel<kShBN, true>(rb[j], Bz + j * p.b_bs1, p.b_rs, p.N - n0, p.K, tid);
            else load_panel<kShBN, false>(rb[j], Bz + j * p.b_bs1, p.b_rs, p.N - n0, p.K, tid);
        }
        // a workgroup has at least the four steps of one query tile
        static_for<0, AHEAD>([&](auto dc) { load_a(decltype(dc)::value, dc); });
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kShHeads; j++) {
            if (!WHOLE && (p.N - n0 < kShBN || p.K < kSkK)) mask_panel<kShBN>(rb[j], p.N - n0, p.K, tid);
            // whole tiles: the scale goes into the key panel once per workgroup instead of into every output (64
            // multiplies per lane and tile, which would take their time from the MFMAs)
            if (WHOLE) {
#pragma unroll
                for (int c = 0; c < NCHB; c++) rb[j][c] *= alpha;
            }
            store_tile_lds<true, kShBN, kSkK, kSkThreads>(lds_b[j], rb[j], tid);
        }
        stage_a(0, 0, std::integral_constant<int, 0>{});
    }
    alpha = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(alpha)));
    __syncthreads();

    const int nstep = ntile * kShHeads;
#pragma nounroll
    for (int it = 0; it < ntile; it++) {
        const int m0 = (tm_first + it) * kSkBM;
        const bool rows_inside = WHOLE || m0 + wm0 < p.M;   // wave-uniform
        f32x16 acc[kShHeads];
        if (!WHOLE) {
#pragma unroll
            for (int j = 0; j < kShHeads; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[j][r] = 0.f;
        }

        static_for<0, kShHeads>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int s = it * kShHeads + j;
            constexpr bool loads = !ONE || j + AHEAD < kShHeads, stages = !ONE || j + 1 < kShHeads;
            // whole tiles: every load and LDS store is unconditional (behind a branch the compiler waits for
            // everything in flight where the paths join): past the last step the last slice comes again and a
            // surplus copy goes to LDS that nobody reads any more
            if (loads && (WHOLE || s + 1 < nstep))
                load_a(min(s + AHEAD, nstep - 1), std::integral_constant<int, WHOLE ? (j + AHEAD) % kShHeads : 0>{});
            const float* la = lds_a[PAIR ? 0 : s & 1];
            if (rows_inside) {
#pragma unroll
                for (int kg = 0; kg < NG; kg++) {
                    Frag<true, 1> fa, fb;
                    read_frag<true, 1, kSkBM, kSkK>(fa, la, wm0, kg, l32, half);
                    read_frag<true, 1, kShBN, kSkK>(fb, lds_b[j], 0, kg, l32, half);
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        // whole tiles: the first product of an accumulator starts from a zero constant (no 64 moves)
                        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.get(0, t), fb.get(0, t),
                                                                     (WHOLE && kg == 0 && t == 0) ? zero : acc[j], 0, 0, 0);
                    }
                }
            }
            // the next slice moves to LDS before this tile's stores are issued
            if (PAIR && stages) __syncthreads();   // every wave has read this step's slice
            if (stages && (WHOLE || s + 1 < nstep))
                stage_a(min(s + 1, nstep - 1), (s + 1) & 1, std::integral_constant<int, WHOLE ? (j + 1) % kShHeads : 0>{});
            if (j + 1 < kShHeads) __syncthreads();
        });

        if (rows_inside) {
            const int col = n0 + l32;
            static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                const int row = m0 + wm0 + 8 * (r >> 2) + 4 * half + (r & 3);
                f32x4 o = {acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
                if (!WHOLE) o *= alpha;
                if (WHOLE || (row < p.M && col < p.N))
                    *reinterpret_cast<f32x4*>(Cz + (int64_t)row * p.c_rs + (int64_t)col * p.c_cs) = o;
            });
        }
        __syncthreads();
    }
}

}  // namespace

// These kernels pay for their panel set-up; below about 16 MiB of output the tiled kernel is faster
// (measured: 64x64x64 6.1 against 9.2 us, 1024x1024x64 7.3 against 9.8 us, 32x512x512x64 24.3 against 19.6 us).
constexpr int64_t kSkMinOutputs = 1ll << 22;

bool shortk_nt_applies(const GemmDesc& d) {
    return d.a_ks == 1 && d.b_ks == 1 && d.c_cs == 1 && d.K >= 1 && d.K <= kSkK && d.rowsum == nullptr &&
           // (tiles of 128 x 128: a 64 x 64 product fills a quarter of one, and 2048 of them, 32 MB of scores, took
           // 69.5 us here against 23.2 on the batched 64 x 64 tiles; 96 x 96: 37.9 against 29.7 at 95)
           d.k_part == 0 && d.M >= 112 && d.N >= 112 && d.M * d.N * d.nbatch >= kSkMinOutputs &&
           // plain epilogue only (scale and store): with accumulate / bias / second output / activation the kernel
           // needed more registers than a wave has and spilled; no call of the engine's path asks for them here
           !d.acc && d.bias == nullptr && d.C2 == nullptr && d.act == 0;
}

int launch_gemm_shortk_nt(GemmParams p, int64_t nbatch, hipStream_t stream) {
    p.tiles_m = (p.M + kSkBM - 1) / kSkBM;
    p.tiles_n = (p.N + kSkBN - 1) / kSkBN;
    if (p.tiles_m <= 0 || p.tiles_n <= 0 || nbatch <= 0) return KAI_OK;
    // longest run of row tiles per workgroup that still leaves one workgroup per compute unit
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n * nbatch;
    int64_t run = tiles / compute_units();
    if (run > kSkMaxRun) run = kSkMaxRun;
    if (run > p.tiles_m) run = p.tiles_m;
    if (run < 1) run = 1;
    p.group_m = (int)run;
    const int64_t runs = (p.tiles_m + run - 1) / run;
    const int64_t blocks = runs * p.tiles_n * nbatch;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: grid too large");
    const dim3 grid((unsigned)blocks, 1, 1);
    if (p.accflag || p.bias || p.C2 || p.act != kActNone)
        return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: the short-reduction kernel has no accumulate / bias / activation epilogue");
    const bool whole = p.M % kSkBM == 0 && p.N % kSkBN == 0 && p.K == kSkK && p.a_vec && p.b_vec && p.c_vec;
    p.c_buf = !p.c_vec && ((int64_t)p.M * p.c_rs + 4) * 4 < (1ll << 31);
    if (whole) {
        shortk_nt_kernel<8, true><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    } else if (p.K <= 32) {
        shortk_nt_kernel<4, false><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    } else {
        shortk_nt_kernel<8, false><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    }
    return check_launch("shortk_nt_kernel");
}

bool shortk_heads_applies(const GemmDesc& d) {
    return d.a_ks == 1 && d.b_ks == 1 && d.K >= 1 && d.K <= kSkK && d.bdiv >= kShHeads && d.bdiv % kShHeads == 0 &&
           d.nbatch % d.bdiv == 0 && d.c_bs1 == 1 && d.c_cs == d.bdiv && d.c_rs % 4 == 0 && d.c_bs0 % 4 == 0 &&
           aligned16(d.C) && !d.acc && !d.bias && !d.C2 && d.act == kActNone && d.rowsum == nullptr &&
           d.k_part == 0 && d.M >= 64 && d.N >= kShBN && d.M * d.N * d.nbatch >= kSkMinOutputs;
}

int launch_gemm_shortk_heads(GemmParams p, int64_t nbatch, hipStream_t stream) {
    p.tiles_m = (p.M + kSkBM - 1) / kSkBM;
    p.tiles_n = (p.N + kShBN - 1) / kShBN;
    const int64_t outer = nbatch / p.bdiv;
    const int64_t hgroups = p.bdiv / kShHeads;
    if (p.tiles_m <= 0 || p.tiles_n <= 0 || outer <= 0) return KAI_OK;
    // longest run of query tiles per workgroup that still leaves one workgroup per compute unit
    const int64_t units = (int64_t)p.tiles_m * p.tiles_n * hgroups * outer;
    // whole tiles with two workgroups or more per compute unit: the kernel that runs two of them side by side
    // (4 x 512 x 512 x 8 heads x 64: 20.9 -> 20.3 us, 16 entries: 64.2 -> 56.8)
    const bool whole = p.M % kSkBM == 0 && p.N % kShBN == 0 && p.K == kSkK && p.a_vec && p.b_vec;
    const bool pair = whole && units >= 2 * (int64_t)compute_units();
    int64_t run = units / (compute_units() * (pair ? 2 : 1));
    if (run > kSkMaxRun) run = kSkMaxRun;
    if (run > p.tiles_m) run = p.tiles_m;
    if (run < 1) run = 1;
    p.group_m = (int)run;
    const int64_t runs = (p.tiles_m + run - 1) / run;
    const int64_t blocks = runs * p.tiles_n * hgroups * outer;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: grid too large");
    const dim3 grid((unsigned)blocks, 1, 1);
    if (whole && pair && run == 1) shortk_heads_kernel<8, true, true, true><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    else if (whole && pair) shortk_heads_kernel<8, true, true><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    else if (whole) shortk_heads_kernel<8, true, false><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    else if (p.K <= 32) shortk_heads_kernel<4, false, false><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    else shortk_heads_kernel<8, false, false><<<grid, dim3(kSkThreads), 0, stream>>>(p);
    return check_launch("shortk_heads_kernel");
}

}  // namespace kai
