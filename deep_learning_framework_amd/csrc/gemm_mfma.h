// fp32 MFMA GEMM for gfx950 (MI355X): C[M,N] (=|+=) act(alpha * A.B + bias)
//
// One kernel template covers the three operand forms of the engine's dense layer
// (VMath::matmul / matmul_backward_x / matmul_backward_w, vmath.cu:2961-3093 of the
// reference) and the strided, batched products of its attention layer
// (mult_on_heads / mix_values and their backward twins, vmath.cu:6729-7129)
// without ever materialising a transpose:
//
//  * Each operand tile is staged in LDS in the orientation in which it is
//    contiguous in global memory: "KC" = [rows][BK+4] when the reduction index is
//    contiguous, "MC" = [BK][rows+4] when the output index is.  Both orientations
//    are read back with 128-bit LDS loads.  A KC read hands a lane four
//    consecutive k of one row (used by four successive MFMAs); an MC read hands a
//    lane one k of four consecutive rows (used by the four 32-row MFMA blocks of
//    the wave).  The k-slot a lane feeds is the same for both operands:
//        k = 8*group + 4*(lane/32) + step,    step = 0..3
//    so products always pair equal k, whatever the orientation mix.
//  * v_mfma_f32_32x32x2_f32: every wave owns NBM x NBN blocks of 32x32 outputs held
//    in accumulator registers (16 per lane per block).
//  * Global -> register -> LDS staging, LDS double buffered, one barrier per K-tile.
//    Two schedules (template parameter PIPE, described at the kernel): a simple one
//    that keeps DEPTH tiles in flight in staging registers, for small tiles and
//    general shapes, and a slot schedule that interleaves LDS reads, LDS stores and
//    global loads with the MFMAs one by one, for large whole-tile products.
//  * Shapes that are whole multiples of the tile with 16-byte aligned operands
//    run a kernel variant with predicate-free 128-bit loads (EDGE = false).  The
//    general variant loads through buffer resources that end with the operand:
//    128 bits at a time for an operand with a unit stride (any 4-byte aligned
//    address will do, and the range is checked dword by dword), element-wise for
//    one that is strided both ways, as chosen once per workgroup; it zeroes what
//    lies outside the matrix when the tile moves to LDS: no load in any loop sits
//    behind a branch.  With the slot schedule it masks only the last, partial
//    K-tile: rows past the operand never reach a stored output.  (A tile that
//    spans 2 GiB or more falls back to flat, clamped, element-wise loads.)
//  * A single product can be cut along K over the batch dimension (k_part) and can
//    sum the rows of A on the side (ROWSUM, the bias gradient of a dense layer).
//  * Workgroup ids are remapped so that the workgroups that share one XCD (and its
//    L2) cover a compact patch of C.
//  * Epilogue in registers: alpha, C += (acc), bias add, optional store of the
//    pre-activation, activation, store (128-bit stores when the B operand is MC).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "act_funcs.h"

namespace kai {

// Loop with compile-time indices: f(std::integral_constant<int, B>), ..., f(<E-1>).  Used where a
// register array must never be indexed by a run-time value, whatever the unroller decides.
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct GemmParams {
    const float* A;
    const float* B;
    float* C;
    float* C2;            // optional second output: value before the activation
    const float* bias;    // optional, indexed by output column
    const float* alpha;   // optional device scalar multiplied into the product (null pointer semantics in has_alpha)
    const float* leaky;   // optional device scalar for leaky relu
    int M, N, K;
    int64_t a_rs, a_ks;   // A(m,k) = A[m*a_rs + k*a_ks]
    int64_t b_rs, b_ks;   // B(n,k) = B[n*b_rs + k*b_ks]
    int64_t c_rs, c_cs;   // C(m,n) = C[m*c_rs + n*c_cs]
    // batch z = blockIdx.z is split as (z / bdiv, z % bdiv); offset = q*bs0 + r*bs1
    int64_t a_bs0, a_bs1, b_bs0, b_bs1, c_bs0, c_bs1;
    int bdiv;
    int a_vec, b_vec, c_vec;  // 16-byte aligned 128-bit access along the contiguous index is legal
    int c_buf;                // short-reduction kernel: rows of C off 16-byte lines take 128-bit buffer stores
    int a_cont, b_cont;       // the operand has a unit stride (then buffer loads may fetch 128 bits at 4-byte alignment)
    int edge_buf;             // general kernels: a tile of either operand spans less than 2 GiB (buffer loads)
    int act;
    int accflag;
    int has_alpha;        // 1: multiply by (*alpha, or 0 if alpha is null)
    int tiles_m, tiles_n;
    int group_m;          // tile rows per column sweep of the XCD-local ordering
    // ROWSUM kernels only: rowsum[m] (=|+=) sum_k A(m,k), summed in ascending k (the bias gradient
    // when A is the transposed output gradient of a dense layer); null switches it off
    float* rowsum;
    int rowsum_acc;
    // EDGE kernels only: when > 0 the batch index also cuts the reduction: batch z covers the
    // k_part steps from z*k_part on (fewer in the last batch), K being the whole length
    int k_part;
    // AMASK bodies only: the A operand is the output gradient of a dense layer and A2, laid out like A, its
    // pre-activation: the product uses A(m,k) * f'(A2(m,k)) with f = relu (a_mask 1) or leaky relu (a_mask 2,
    // slope *leaky, 0 if null); a_mask 0 uses A as it is
    const float* A2;
    int a_mask;
};

constexpr int kLdsPad = 4;

template <bool KC, int ROWS, int BK>
struct TileShape {
    // KC: [ROWS][BK+pad], MC: [BK][ROWS+pad]
    static constexpr int kStride = KC ? (BK + kLdsPad) : (ROWS + kLdsPad);
    static constexpr int kFloats = KC ? ROWS * (BK + kLdsPad) : BK * (ROWS + kLdsPad);
    static constexpr int kChunks = ROWS * BK / 4;
    // chunk c -> (row, k) of its first element
    static constexpr int kChunksPerLine = KC ? BK / 4 : ROWS / 4;
};

// Predicate-free load of one operand tile: every chunk is a 16-byte aligned float4 inside the matrix.
// `base` (wave-uniform) points at element (row0, k0); `ld` is the stride of the non-contiguous index;
// `toff` is the calling thread's element offset of its first chunk, line0*ld + off0, which does not
// change along K.  Chunk i of a thread lies a uniform i*(NT/chunks-per-line)*ld further on, so the
// address is a scalar base plus one 32-bit vector offset.
template <bool KC, int ROWS, int BK, int NT>
__device__ __forceinline__ void load_tile_fast(f32x4 (&reg)[ROWS * BK / 4 / NT], const float* __restrict__ base,
                                               int64_t ld, uint32_t toff) {
    using TS = TileShape<KC, ROWS, BK>;
    constexpr int NCH = TS::kChunks / NT;
    static_assert(NT % TS::kChunksPerLine == 0, "threads must cover whole lines");
    constexpr int kLinesPerPass = NT / TS::kChunksPerLine;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const float* bi = base + (int64_t)(i * kLinesPerPass) * ld;
        reg[i] = *reinterpret_cast<const f32x4*>(bi + toff);
    }
}

// The same chunk through a buffer load: address = resource base + a uniform byte offset (scalar registers) +
// the thread's constant byte offset.  In the pipelined loop this leaves NO vector instruction per load; with
// flat addresses the compiler keeps a 64-bit pointer per load in vector registers and advances each of them
// every tile, and vector instructions take their time from the fp32 MFMAs.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <bool KC, int ROWS, int BK, int NT>
__device__ __forceinline__ void load_tile_chunk_buf(f32x4 (&reg)[ROWS * BK / 4 / NT], __amdgpu_buffer_rsrc_t rsrc,
                                                    int tile_off, int ld_bytes, int toff_bytes, int i) {
    using TS = TileShape<KC, ROWS, BK>;
    constexpr int kLinesPerPass = NT / TS::kChunksPerLine;
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, toff_bytes, tile_off + i * kLinesPerPass * ld_bytes, 0);
    reg[i] = __builtin_bit_cast(f32x4, v);
}

// One chunk of the predicate-free load (chunk i of the calling thread).
template <bool KC, int ROWS, int BK, int NT>
__device__ __forceinline__ void load_tile_chunk(f32x4 (&reg)[ROWS * BK / 4 / NT], const float* __restrict__ base,
                                                int64_t ld, uint32_t toff, int i) {
    using TS = TileShape<KC, ROWS, BK>;
    constexpr int kLinesPerPass = NT / TS::kChunksPerLine;
    const float* bi = base + (int64_t)(i * kLinesPerPass) * ld;
    reg[i] = *reinterpret_cast<const f32x4*>(bi + toff);
}

// General load of one operand tile: rows_left / k_left (both >= 1) are the numbers of valid rows / k
// from the tile origin, rs / ks the element strides of the row index and the reduction index.
// Every address is clamped into the matrix, so that no branch separates the loads of a tile (a load
// under a condition makes the compiler wait for it before it issues the next one); what lies
// outside the matrix is zeroed by mask_tile_edge() when the tile moves on to LDS, not here: a mask
// right behind the load would bring the wait for it along.
template <bool KC, int ROWS, int BK, int NT, bool VEC>
__device__ __forceinline__ void load_tile_edge(f32x4 (&reg)[ROWS * BK / 4 / NT], const float* __restrict__ base,
                                               int64_t rs, int64_t ks, int rows_left, int k_left, int tid) {
    using TS = TileShape<KC, ROWS, BK>;
    constexpr int NCH = TS::kChunks / NT;
    const int r_last = rows_left - 1, k_last = k_left - 1;
    const int64_t klks = (int64_t)k_last * ks;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * NT;
        const int line = c / TS::kChunksPerLine;
        const int off = (c % TS::kChunksPerLine) * 4;
        const int r = KC ? line : off;   // first row of the chunk
        const int k = KC ? off : line;   // first k of the chunk
        if (VEC) {
            const int rc = KC ? min(r, r_last) : (r < rows_left ? r : 0);
            const int kc = KC ? (k < k_left ? k : 0) : min(k, k_last);
            reg[i] = *reinterpret_cast<const f32x4*>(base + (int64_t)rc * rs + (int64_t)kc * ks);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int rj = KC ? r : r + j, kj = KC ? k + j : k;
                // products of per-thread constants: they do not change from tile to tile, only the
                // choice between them and the (uniform) offset of the last valid k does
                const int64_t roff = (int64_t)min(rj, r_last) * rs;
                const int64_t koff = kj <= k_last ? (int64_t)kj * ks : klks;
                reg[i][j] = base[roff + koff];
            }
        }
    }
}

// Zeroes the elements of a tile loaded by load_tile_edge() that lie outside the matrix (bitwise, so
// that the compiler cannot turn the mask back into a conditional load).
template <bool KC, int ROWS, int BK, int NT>
__device__ __forceinline__ void mask_tile_edge(f32x4 (&reg)[ROWS * BK / 4 / NT], int rows_left, int k_left, int tid) {
    using TS = TileShape<KC, ROWS, BK>;
    constexpr int NCH = TS::kChunks / NT;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * NT;
        const int line = c / TS::kChunksPerLine;
        const int off = (c % TS::kChunksPerLine) * 4;
        const int r = KC ? line : off;
        const int k = KC ? off : line;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int rj = KC ? r : r + j, kj = KC ? k + j : k;
            const int keep = (rj < rows_left && kj < k_left) ? -1 : 0;
            const float e = reg[i][j];
            reg[i][j] = __int_as_float(__float_as_int(e) & keep);
        }
    }
}

// The general tile through buffer loads.  A thread's byte offsets inside a tile do not change from tile to tile
// (edge_offsets, computed once); the tile itself is addressed by a resource that starts at the tile and ends with
// the operand (edge_resource, scalar arithmetic), so nothing is clamped: an address past the end of the operand
// returns zero instead of faulting, an address that wraps into a neighbouring row returns data that mask_tile_edge
// removes.  No vector instruction per load is left in the loop, where they would take their time from the MFMAs;
// the flat version above spends about six per element on clamps and 64-bit sums.
template <bool KC, int ROWS, int BK, int NT, bool VEC>
__device__ __forceinline__ void edge_offsets(int (&voff)[ROWS * BK / 4 / NT][VEC ? 1 : 4], int64_t rs, int64_t ks, int tid) {
    using TS = TileShape<KC, ROWS, BK>;
    constexpr int NCH = TS::kChunks / NT;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * NT;
        const int line = c / TS::kChunksPerLine;
        const int off = (c % TS::kChunksPerLine) * 4;
        const int r = KC ? line : off;
        const int k = KC ? off : line;
#pragma unroll
        for (int j = 0; j < (VEC ? 1 : 4); j++) {
            const int rj = KC ? r : r + j, kj = KC ? k + j : k;
            voff[i][j] = (int)(((int64_t)rj * rs + (int64_t)kj * ks) * 4);   // the host has checked the tile's span
        }
    }
}

// base: address of element (row 0 of the workgroup's rows, k = 0) as an integer known to be uniform;
// rows_total: rows from there to the end of the operand; k_total: reduction length from k = 0
__device__ __forceinline__ __amdgpu_buffer_rsrc_t edge_resource(uint64_t base, int64_t rs, int64_t ks, int rows_total,
                                                                int k_total, int k0) {
    const uint64_t addr = base + (uint64_t)((int64_t)k0 * ks * 4);
    int64_t ext = ((int64_t)(rows_total - 1) * rs + (int64_t)(k_total - k0 - 1) * ks + 1) * 4;
    if (ext > 0xFFFFFFFFll) ext = 0xFFFFFFFFll;   // a tile's own span is below 2 GiB: then all of it is inside
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(addr), 0, (int)(uint32_t)ext, 0x00020000);
}

template <int NCH, bool VEC>
__device__ __forceinline__ void load_tile_edge_buf(f32x4 (&reg)[NCH], __amdgpu_buffer_rsrc_t rsrc,
                                                   const int (&voff)[NCH][VEC ? 1 : 4]) {
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        if (VEC) {
            reg[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff[i][0], 0, 0));
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                reg[i][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff[i][j], 0, 0));
        }
    }
}

template <bool KC, int ROWS, int BK, int NT>
__device__ __forceinline__ void store_tile_lds(float* __restrict__ lds, const f32x4 (&reg)[ROWS * BK / 4 / NT],
                                               int tid) {
    using TS = TileShape<KC, ROWS, BK>;
    constexpr int NCH = TS::kChunks / NT;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * NT;
        const int line = c / TS::kChunksPerLine;
        const int off = (c % TS::kChunksPerLine) * 4;
        *reinterpret_cast<f32x4*>(lds + line * TS::kStride + off) = reg[i];
    }
}

// Fragments of one operand for one group of 8 k (4 MFMA steps), NB 32-row blocks.
template <bool KC, int NB>
struct Frag {
    // KC: v[b] holds k-steps 0..3 of block b.  MC: v[t][b] holds block b of step t.
    f32x4 v[KC ? NB : 4];
    __device__ __forceinline__ float get(int b, int t) const { return KC ? v[b][t] : v[t][b]; }
};

template <bool KC, int NB, int ROWS, int BK>
__device__ __forceinline__ void read_frag(Frag<KC, NB>& f, const float* __restrict__ lds, int w_r0, int kg, int l32,
                                          int half) {
    using TS = TileShape<KC, ROWS, BK>;
    if (KC) {
#pragma unroll
        for (int b = 0; b < NB; b++)
            f.v[b] = *reinterpret_cast<const f32x4*>(lds + (w_r0 + 32 * b + l32) * TS::kStride + kg * 8 + 4 * half);
    } else {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const float* p = lds + (kg * 8 + 4 * half + t) * TS::kStride + w_r0 + NB * l32;
            if (NB == 4) {
                f.v[t] = *reinterpret_cast<const f32x4*>(p);
            } else if (NB == 2) {
                const f32x2 q = *reinterpret_cast<const f32x2*>(p);
                f.v[t][0] = q[0];
                f.v[t][1] = q[1];
            } else {
                f.v[t][0] = p[0];
            }
        }
    }
}

// One LDS read of a fragment: piece < (KC ? NB : 4).
template <bool KC, int NB, int ROWS, int BK>
__device__ __forceinline__ void read_frag_piece(Frag<KC, NB>& f, const float* __restrict__ lds, int w_r0, int kg,
                                                int l32, int half, int piece) {
    using TS = TileShape<KC, ROWS, BK>;
    if (KC) {
        f.v[piece] =
            *reinterpret_cast<const f32x4*>(lds + (w_r0 + 32 * piece + l32) * TS::kStride + kg * 8 + 4 * half);
    } else {
        const float* p = lds + (kg * 8 + 4 * half + piece) * TS::kStride + w_r0 + NB * l32;
        if (NB == 4) {
            f.v[piece] = *reinterpret_cast<const f32x4*>(p);
        } else if (NB == 2) {
            const f32x2 q = *reinterpret_cast<const f32x2*>(p);
            f.v[piece][0] = q[0];
            f.v[piece][1] = q[1];
        } else {
            f.v[piece][0] = p[0];
        }
    }
}

// One 128-bit LDS store of a staged tile: chunk i of the calling thread.
template <bool KC, int ROWS, int BK, int NT>
__device__ __forceinline__ void store_tile_chunk(float* __restrict__ lds, const f32x4 (&reg)[ROWS * BK / 4 / NT],
                                                 int tid, int i) {
    using TS = TileShape<KC, ROWS, BK>;
    const int c = tid + i * NT;
    const int line = c / TS::kChunksPerLine;
    const int off = (c % TS::kChunksPerLine) * 4;
    *reinterpret_cast<f32x4*>(lds + line * TS::kStride + off) = reg[i];
}

// Workgroup id -> (tile_m, tile_n).  Hardware deals consecutive workgroup ids round-robin over
// the 8 XCDs; ids congruent mod 8 therefore share an L2.  They are renumbered so that each XCD
// walks a contiguous run of tiles, and the run is ordered in column sweeps of `group_m` tile rows
// so that tiles that are live together share A row panels and B column panels.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    int id = bid;
    if ((total & 7) == 0) id = (bid & 7) * (total >> 3) + (bid >> 3);
    const int per_group = group_m * tiles_n;
    const int g = id / per_group;
    const int first_m = g * group_m;
    const int rows = min(group_m, tiles_m - first_m);
    const int in_g = id - g * per_group;
    tm = first_m + in_g % rows;
    tn = in_g / rows;
}

// Epilogue of one output tile.  In registers: alpha, += C (acc), bias, optional store of the
// pre-activation, the activation, one store.  none / relu / leaky relu are written out per element; the
// transcendental codes run in a rolled loop over the 16 rows of a block (see there), so that the kernel
// holds one copy of their code per block and the accumulators stay in registers for the whole kernel.
template <int NBM, int NBN, bool A_KC, bool B_KC>
__device__ __forceinline__ void gemm_epilogue(const GemmParams& p, f32x16 (&acc)[NBM][NBN], int m0, int n0,
                                              int64_t c_off, int wm0, int wn0, int l32, int half, float alpha,
                                              float leaky) {
    float* C = p.C + c_off;
    float* C2 = p.C2 ? p.C2 + c_off : nullptr;
    const int act = p.act;
    const bool slow_act = act > kActLeaky;

    auto row_of = [&](int i, int r) -> int {
        const int mi = 8 * (r >> 2) + 4 * half + (r & 3);   // row inside the 32x32 block
        return m0 + (A_KC ? wm0 + 32 * i + mi : wm0 + NBM * mi + i);
    };
    auto col_of = [&](int j) -> int { return n0 + (B_KC ? wn0 + 32 * j + l32 : wn0 + NBN * l32 + j); };
    auto cheap_act = [&](float v) -> float {
        if (act == kActRelu) return (v > 0) ? v : 0.0f;
        if (act == kActLeaky) return (v > 0) ? v : v * leaky;
        return v;
    };
    const bool vec_store = !B_KC && (NBN == 4 || NBN == 2) && p.c_vec;
    // Per 32-row block: everything that has to be loaded (the old C for acc, the bias) is loaded first, at
    // clamped addresses and under workgroup-uniform conditions only, then all stores follow back to back.
    // Written element by element (load, wait, store, next load ...) every store waited for the one before it:
    // the 16 stores of a 64x64 tile took 2.7 us.
    const bool has_alpha = p.has_alpha != 0, accf = p.accflag != 0, has_bias = p.bias != nullptr;
    auto activate_cheap = [&](float& v) {   // act is uniform: the branch is taken once per call site by all lanes
        v = cheap_act(v);
    };

    // Row r of a lane's 16 accumulator rows lies dr(r) rows below its row 0, a compile-time number, so a row's
    // offset in C is the lane's 64-bit offset of row 0 plus a wave-uniform product dr(r) * c_rs: no per-row
    // address is kept in vector registers (sixteen 64-bit offsets next to 128 accumulators did not fit).
    auto dr = [](int r) constexpr -> int { return (A_KC ? 1 : NBM) * (8 * (r >> 2) + (r & 3)); };
    static_for<0, NBM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const int row0 = row_of(i, 0);
        const int64_t base0 = (int64_t)row0 * p.c_rs;
        // where a load must not leave the matrix: rows past the end read the lane's row 0, or the last row
        const int64_t base0_c = (int64_t)(row0 < p.M ? row0 : p.M - 1) * p.c_rs;
        auto row_ok = [&](int r) -> bool { return row0 + dr(r) < p.M; };
        auto rowoff = [&](int r) -> int64_t { return base0 + (int64_t)dr(r) * p.c_rs; };
        auto rowoff_c = [&](int r) -> int64_t { return row_ok(r) ? rowoff(r) : base0_c; };
        if (vec_store) {
            // the NBN columns of a lane are adjacent in memory: one store of NBN floats per row
            constexpr int VW = (NBN == 2 || NBN == 4) ? NBN : 4;
            typedef float vecw __attribute__((ext_vector_type(VW)));
            const int col = col_of(0);
            const bool col_ok = col < p.N;       // N % 4 == 0 under c_vec: a chunk is inside or outside as a whole
            const int colc = col_ok ? col : 0;
            vecw o[16];
            static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                static_for<0, VW>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    o[r][j] = acc[i][j % NBN][r];
                });
            });
            if (has_alpha) {
#pragma unroll
                for (int r = 0; r < 16; r++) o[r] *= alpha;
            }
            if (accf) {
                vecw cin[16];
#pragma unroll
                for (int r = 0; r < 16; r++) cin[r] = *reinterpret_cast<const vecw*>(C + rowoff_c(r) + colc);
#pragma unroll
                for (int r = 0; r < 16; r++) o[r] += cin[r];
            }
            if (has_bias) {
                const vecw bv = *reinterpret_cast<const vecw*>(p.bias + colc);
#pragma unroll
                for (int r = 0; r < 16; r++) o[r] += bv;
            }
            if (C2) {
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (row_ok(r) && col_ok) *reinterpret_cast<vecw*>(C2 + rowoff(r) + col) = o[r];
            }
            if (slow_act) {
                // The values go back into the accumulator vectors (compile-time indices) and a ROLLED loop picks
                // row r out of them with a run-time index (a register-indexed move, the index is wave-uniform):
                // one copy of the transcendental code per 32-row block instead of one per element, every value
                // transformed in registers and stored once.
                static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    static_for<0, NBN>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        acc[i][j][r] = o[r][j];
                    });
                });
#pragma nounroll
                for (int r = 0; r < 16; r++) {
                    vecw x;
                    static_for<0, VW>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        x[j] = apply_act(acc[i][j % NBN][r], act, leaky);
                    });
                    const int d = (A_KC ? 1 : NBM) * (8 * (r >> 2) + (r & 3));
                    if (row0 + d < p.M && col_ok) *reinterpret_cast<vecw*>(C + base0 + (int64_t)d * p.c_rs + col) = x;
                }
            } else {
                if (act != kActNone) {
#pragma unroll
                    for (int r = 0; r < 16; r++)
#pragma unroll
                        for (int j = 0; j < VW; j++) {
                            float v = o[r][j];
                            activate_cheap(v);
                            o[r][j] = v;
                        }
                }
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (row_ok(r) && col_ok) *reinterpret_cast<vecw*>(C + rowoff(r) + col) = o[r];
            }
        } else {
            float v[NBN][16];
            int cols[NBN];
            int64_t coloff[NBN], coloff_c[NBN];
#pragma unroll
            for (int j = 0; j < NBN; j++) {
                cols[j] = col_of(j);
                coloff[j] = (int64_t)cols[j] * p.c_cs;
                coloff_c[j] = (int64_t)(cols[j] < p.N ? cols[j] : 0) * p.c_cs;
            }
            static_for<0, NBN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    v[j][r] = acc[i][j][r];
                });
            });
            if (has_alpha) {
#pragma unroll
                for (int j = 0; j < NBN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) v[j][r] *= alpha;
            }
            if (accf) {
                float cin[NBN][16];
#pragma unroll
                for (int j = 0; j < NBN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) cin[j][r] = C[rowoff_c(r) + coloff_c[j]];
#pragma unroll
                for (int j = 0; j < NBN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) v[j][r] += cin[j][r];
            }
            if (has_bias) {
#pragma unroll
                for (int j = 0; j < NBN; j++) {
                    const float bv = p.bias[cols[j] < p.N ? cols[j] : 0];
#pragma unroll
                    for (int r = 0; r < 16; r++) v[j][r] += bv;
                }
            }
            if (C2) {
#pragma unroll
                for (int j = 0; j < NBN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        if (row_ok(r) && cols[j] < p.N) C2[rowoff(r) + coloff[j]] = v[j][r];
            }
            if (slow_act) {
                // as above: back into the accumulator vectors, then one rolled loop over the 16 rows of the block
                static_for<0, NBN>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    static_for<0, 16>([&](auto rc) {
                        constexpr int r = decltype(rc)::value;
                        acc[i][j][r] = v[j][r];
                    });
                });
#pragma nounroll
                for (int r = 0; r < 16; r++) {
                    const int d = (A_KC ? 1 : NBM) * (8 * (r >> 2) + (r & 3));
                    const bool ok = row0 + d < p.M;
                    const int64_t ro = base0 + (int64_t)d * p.c_rs;
                    static_for<0, NBN>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        const float x = apply_act(acc[i][j][r], act, leaky);
                        if (ok && cols[j] < p.N) C[ro + coloff[j]] = x;
                    });
                }
            } else {
                if (act != kActNone) {
#pragma unroll
                    for (int j = 0; j < NBN; j++)
#pragma unroll
                        for (int r = 0; r < 16; r++) activate_cheap(v[j][r]);
                }
#pragma unroll
                for (int j = 0; j < NBN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        if (row_ok(r) && cols[j] < p.N) C[rowoff(r) + coloff[j]] = v[j][r];
            }
        }
    });
}

// EDGE = false: the host has checked that M, N, K are multiples of the tile, that both operands
// allow aligned 128-bit loads and that a tile's offsets fit 32 bits; the kernel then holds no
// predicated load code at all (fewer registers).  EDGE = true: general shapes (with PIPE 1: any
// M, N, K, but operands that allow aligned 128-bit loads and 32-bit offsets, checked by the host).
//
// PIPE selects the schedule of the main loop:
//   0  per K-tile: all fragment reads of a group, then its MFMAs; LDS stores and the barrier at the
//      end of the tile.
//   1  fragments double buffered: the reads of group g+1 are issued with the MFMAs of group g and
//      spread between them, so the waves of a workgroup do not hit LDS in one burst and no MFMA
//      waits for an LDS round trip.  The next tile is stored to LDS while the second-to-last group
//      computes; the barrier sits before the last group, whose MFMAs (operands already in
//      registers) cover the first fragment reads of the next tile.
//
// MINW is the number of waves per SIMD the register allocation must leave room for (2 lets two
// independent workgroups of four waves share a compute unit, so that one computes while the other
// waits at its barrier).
//
// DEPTH (PIPE 0 only) is the number of K-tiles kept in flight in staging registers: small tiles
// compute for far less time than a global load takes to return, so they run several tiles ahead.
//
// ROWSUM (PIPE 0 only): the workgroups of the first tile column also sum every row of their A tile
// over K, one thread per row reading the tile from LDS, k ascending across tiles: a fixed order
// that is the order of a sequential loop.
//
// AMASK (whole tiles only): the A tile is multiplied element by element with the derivative of
// relu / leaky relu at a second tensor A2 of the same layout on its way to LDS (GemmParams::a_mask): the
// backward products of a dense layer read the output gradient and the pre-activation directly.
//
// The body is a device function over (workgroup id, batch index, the two LDS tile pairs) so that one launch
// can hold the workgroups of two different products (dense_backward.hip); gemm_mfma_kernel is one product.
template <int WM, int WN, int NBM, int NBN, int BK, bool A_KC, bool B_KC, bool EDGE, int PIPE, int DEPTH,
          bool ROWSUM, bool AMASK>
__device__ __forceinline__ void gemm_tile_body(
    const GemmParams& p, const int bid, const int z,
    float (*lds_a)[TileShape<A_KC, WM * NBM * 32, BK>::kFloats],
    float (*lds_b)[TileShape<B_KC, WN * NBN * 32, BK>::kFloats]) {
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = WM * NBM * 32;
    constexpr int BN = WN * NBN * 32;
    using TA = TileShape<A_KC, BM, BK>;
    using TB = TileShape<B_KC, BN, BK>;
    constexpr int NCHA = TA::kChunks / NT;
    constexpr int NCHB = TB::kChunks / NT;
    static_assert(TA::kChunks % NT == 0 && TB::kChunks % NT == 0, "tile must divide over the threads");
    static_assert(BK % 8 == 0, "BK must hold whole groups of 8 k");
    static_assert(!AMASK || !EDGE, "the masked A operand exists for whole tiles only");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const int wm0 = (wave / WN) * (NBM * 32);
    const int wn0 = (wave % WN) * (NBN * 32);

    int tm, tn;
    tile_of_block(bid, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const int zq = z / p.bdiv, zr = z % p.bdiv;
    const float* __restrict__ Ab = p.A + zq * p.a_bs0 + zr * p.a_bs1 + (int64_t)m0 * p.a_rs;
    const float* __restrict__ Bb = p.B + zq * p.b_bs0 + zr * p.b_bs1 + (int64_t)n0 * p.b_rs;
    const int64_t c_off = zq * p.c_bs0 + zr * p.c_bs1;

    const int rows_a = p.M - m0;
    const int rows_b = p.N - n0;
    const int64_t a_ld = A_KC ? p.a_rs : p.a_ks;
    const int64_t b_ld = B_KC ? p.b_rs : p.b_ks;
    // per-thread element offsets of the predicate-free loads (whole-tile kernels: they fit 32 bits)
    const uint32_t toff_a =
        (uint32_t)(tid / TA::kChunksPerLine) * (uint32_t)a_ld + (uint32_t)(tid % TA::kChunksPerLine) * 4u;
    const uint32_t toff_b =
        (uint32_t)(tid / TB::kChunksPerLine) * (uint32_t)b_ld + (uint32_t)(tid % TB::kChunksPerLine) * 4u;

    f32x16 acc[NBM][NBN];
#pragma unroll
    for (int i = 0; i < NBM; i++)
#pragma unroll
        for (int j = 0; j < NBN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    static_assert(DEPTH >= 1, "at least one tile is staged in registers");
    static_assert(!ROWSUM || (PIPE == 0 && BM <= NT), "row sums: PIPE 0 schedule, one thread per tile row");
    const bool do_rowsum = ROWSUM && p.rowsum != nullptr && tn == 0 && z == 0 && tid < BM;
    float rowsum = 0.f;
    f32x4 rax[DEPTH][NCHA], rbx[DEPTH][NCHB];
    f32x4 rax2[AMASK ? DEPTH : 1][NCHA];   // AMASK: the pre-activation tile that belongs to rax
    f32x4(&ra)[NCHA] = rax[0];
    f32x4(&rb)[NCHB] = rbx[0];
    // reduction length of this workgroup
    const int Kz = (EDGE && p.k_part > 0) ? min(p.k_part, p.K - z * p.k_part) : p.K;
    // steps from this workgroup's first one to the end of the operand (the bound of its buffer resources)
    const int Krem = (EDGE && p.k_part > 0) ? p.K - z * p.k_part : p.K;
    const int nkt = (Kz + BK - 1) / BK;

    constexpr int NKG = BK / 8;
    auto mfma_group = [&](const Frag<A_KC, NBM>& fa, const Frag<B_KC, NBN>& fb) {
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
            for (int i = 0; i < NBM; i++)
#pragma unroll
                for (int j = 0; j < NBN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.get(i, t), fb.get(j, t), acc[i][j], 0, 0, 0);
    };
    // predicate-free load of tile kt (whole-tile kernels)
    auto load_global = [&](int kt) {
        load_tile_fast<A_KC, BM, BK, NT>(ra, Ab + (int64_t)kt * BK * p.a_ks, a_ld, toff_a);
        load_tile_fast<B_KC, BN, BK, NT>(rb, Bb + (int64_t)kt * BK * p.b_ks, b_ld, toff_b);
    };

    // Whole-tile kernels read their operand tiles with buffer loads: resources over the two operands from this
    // workgroup's tile rows on (the host has checked that every offset of the tile row block fits 31 bits); stride 0,
    // no bounds below 4 GiB, raw 32-bit data format.  The bases are the same in every lane; saying so keeps the
    // compiler from looping over "distinct" resources.
    auto uniform_ptr = [](const float* q) -> float* {
        const uint64_t a = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
    };
    // The pipelined schedule on general shapes (PIPE 1 with EDGE): the resources end with the operand, so a
    // row past the last one reads as zero or as other rows' data of the same operand; either only ever reaches
    // output rows and columns that are not stored.  The loop then runs over the whole K-tiles without any
    // predicate, and the rest of K follows as one masked tile.
    constexpr bool RAGGED_PIPE = EDGE && PIPE == 1;
    const __amdgpu_buffer_rsrc_t rsrc_a =
        RAGGED_PIPE ? edge_resource(reinterpret_cast<uint64_t>(uniform_ptr(Ab)), p.a_rs, p.a_ks, p.M - m0, Krem, 0)
                    : __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(Ab), 0, (int)0xFFFFFFFFu, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        RAGGED_PIPE ? edge_resource(reinterpret_cast<uint64_t>(uniform_ptr(Bb)), p.b_rs, p.b_ks, p.N - n0, Krem, 0)
                    : __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(Bb), 0, (int)0xFFFFFFFFu, 0x00020000);
    // AMASK: the second tensor behind the A operand, addressed exactly like A
    const bool a_masked = AMASK && p.a_mask != 0;
    const __amdgpu_buffer_rsrc_t rsrc_a2 = __builtin_amdgcn_make_buffer_rsrc(
        uniform_ptr(a_masked ? p.A2 + (Ab - p.A) : Ab), 0, (int)0xFFFFFFFFu, 0x00020000);
    const float a_mask_slope = (AMASK && p.a_mask == 2 && p.leaky) ? *p.leaky : 0.f;

    if (PIPE == 0) {
        // The whole loop exists once per combination of 128-bit / element-wise loads of A and B.  The
        // choice is made once per workgroup: a loop body that holds both kinds of load behind a branch
        // makes the compiler wait for every load before the next tile's are issued, which turns the
        // register staging into one memory round trip per tile.  For the same reason every load in the
        // loop is unconditional: a tile index past the end is clamped (that tile is never stored).
        auto pipe0 = [&](auto va_c, auto vb_c, auto buf_c) {
            constexpr bool VA = decltype(va_c)::value, VB = decltype(vb_c)::value;
            constexpr bool BUF = EDGE && decltype(buf_c)::value;   // general tiles through buffer loads
            int voa[NCHA][VA ? 1 : 4], vob[NCHB][VB ? 1 : 4];
            uint64_t a_base = 0, b_base = 0;
            if (BUF) {
                edge_offsets<A_KC, BM, BK, NT, VA>(voa, p.a_rs, p.a_ks, tid);
                edge_offsets<B_KC, BN, BK, NT, VB>(vob, p.b_rs, p.b_ks, tid);
                a_base = reinterpret_cast<uint64_t>(uniform_ptr(Ab));
                b_base = reinterpret_cast<uint64_t>(uniform_ptr(Bb));
            }
            // AMASK: da2 receives the pre-activation tile that goes with da; amask_tile turns da into
            // da * f'(da2) when the tile leaves the staging registers
            auto load_a2 = [&](int kt, f32x4(&da2)[NCHA]) {
                if constexpr (AMASK) {
                    const int k0 = min(kt, nkt - 1) * BK;
#pragma unroll
                    for (int i = 0; i < NCHA; i++)
                        load_tile_chunk_buf<A_KC, BM, BK, NT>(da2, rsrc_a2, k0 * (int)p.a_ks * 4, (int)a_ld * 4, (int)toff_a * 4, i);
                }
            };
            auto amask_tile = [&](f32x4(&da)[NCHA], const f32x4(&da2)[NCHA]) {
                if constexpr (AMASK) {
                    if (a_masked) {   // uniform
#pragma unroll
                        for (int i = 0; i < NCHA; i++)
#pragma unroll
                            for (int j = 0; j < 4; j++) da[i][j] = ((da2[i][j] > 0) ? 1.0f : a_mask_slope) * da[i][j];
                    }
                }
            };
            auto load_into = [&](int kt, f32x4(&da)[NCHA], f32x4(&db)[NCHB]) {
                const int ktc = min(kt, nkt - 1);
                const int k0 = ktc * BK;
                const float* ap = Ab + (int64_t)k0 * p.a_ks;
                const float* bp = Bb + (int64_t)k0 * p.b_ks;
                if (BUF) {
                    load_tile_edge_buf<NCHA, VA>(da, edge_resource(a_base, p.a_rs, p.a_ks, p.M - m0, Kz, k0), voa);
                    load_tile_edge_buf<NCHB, VB>(db, edge_resource(b_base, p.b_rs, p.b_ks, p.N - n0, Kz, k0), vob);
                } else if (!EDGE) {
#pragma unroll
                    for (int i = 0; i < NCHA; i++)
                        load_tile_chunk_buf<A_KC, BM, BK, NT>(da, rsrc_a, k0 * (int)p.a_ks * 4, (int)a_ld * 4, (int)toff_a * 4, i);
#pragma unroll
                    for (int i = 0; i < NCHB; i++)
                        load_tile_chunk_buf<B_KC, BN, BK, NT>(db, rsrc_b, k0 * (int)p.b_ks * 4, (int)b_ld * 4, (int)toff_b * 4, i);
                } else {
                    load_tile_edge<A_KC, BM, BK, NT, VA>(da, ap, p.a_rs, p.a_ks, rows_a, Kz - k0, tid);
                    load_tile_edge<B_KC, BN, BK, NT, VB>(db, bp, p.b_rs, p.b_ks, rows_b, Kz - k0, tid);
                }
            };
            // a tile loaded by the general path still holds whatever the clamped addresses gave
            auto mask_tile = [&](int kt, f32x4(&da)[NCHA], f32x4(&db)[NCHB]) {
                const int k_left = Kz - kt * BK;
                if (EDGE && (rows_a < BM || rows_b < BN || k_left < BK)) {
                    mask_tile_edge<A_KC, BM, BK, NT>(da, rows_a, k_left, tid);
                    mask_tile_edge<B_KC, BN, BK, NT>(db, rows_b, k_left, tid);
                }
            };

            // prologue: tiles 0 .. DEPTH-1 go to the staging slots, tile 0 on to LDS, its slot is refilled
            static_for<0, DEPTH>([&](auto dc) {
                constexpr int d = decltype(dc)::value;
                load_into(d, rax[d], rbx[d]);
                load_a2(d, rax2[AMASK ? d : 0]);
            });
            mask_tile(0, ra, rb);
            amask_tile(ra, rax2[0]);
            store_tile_lds<A_KC, BM, BK, NT>(lds_a[0], ra, tid);
            store_tile_lds<B_KC, BN, BK, NT>(lds_b[0], rb, tid);
            if (DEPTH > 1) {
                load_into(DEPTH, ra, rb);
                load_a2(DEPTH, rax2[0]);
            }
            __syncthreads();

            // At the top of tile kt: LDS[kt & 1] holds tile kt; slot (kt + j) % DEPTH holds tile kt + j for
            // j = 1 .. DEPTH (slot kt % DEPTH was refilled with tile kt + DEPTH when tile kt left it).
            // With DEPTH == 1 the single slot is refilled before the MFMAs of the tile instead.
            auto stage = [&](auto dc, int kt, bool last_tiles) {
                constexpr int d = decltype(dc)::value;
                constexpr int nslot = (d + 1) % DEPTH;
                const int cur = kt & 1;
                if (DEPTH == 1) {
                    load_into(kt + 1, ra, rb);
                    load_a2(kt + 1, rax2[0]);
                }
                // With DEPTH > 1 the next tile has been in registers for a while: it goes to the free LDS
                // buffer first, so that the store's latency runs under this tile's MFMAs instead of between
                // them and the barrier.  (Every wave left that buffer before the last barrier.)  In the main
                // loop the store is unconditional: past the last tile it moves a surplus copy of the last
                // tile into the buffer nobody reads any more.
                auto store_next = [&]() {
                    if (!last_tiles || kt + 1 < nkt) {
                        mask_tile(kt + 1, rax[nslot], rbx[nslot]);
                        amask_tile(rax[nslot], rax2[AMASK ? nslot : 0]);
                        store_tile_lds<A_KC, BM, BK, NT>(lds_a[cur ^ 1], rax[nslot], tid);
                        store_tile_lds<B_KC, BN, BK, NT>(lds_b[cur ^ 1], rbx[nslot], tid);
                    }
                    if (DEPTH > 1) {
                        load_into(kt + 1 + DEPTH, rax[nslot], rbx[nslot]);
                        load_a2(kt + 1 + DEPTH, rax2[AMASK ? nslot : 0]);
                    }
                };
                if (DEPTH > 1) store_next();
                const float* la = lds_a[cur];
                const float* lb = lds_b[cur];
                if (ROWSUM && do_rowsum) {   // rows and k beyond the matrix were stored as zeros
#pragma unroll
                    for (int kk = 0; kk < BK; kk++) rowsum += la[A_KC ? tid * TA::kStride + kk : kk * TA::kStride + tid];
                }
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    Frag<A_KC, NBM> fa;
                    Frag<B_KC, NBN> fb;
                    read_frag<A_KC, NBM, BM, BK>(fa, la, wm0, kg, l32, half);
                    read_frag<B_KC, NBN, BN, BK>(fb, lb, wn0, kg, l32, half);
                    mfma_group(fa, fb);
                }
                if (DEPTH == 1) store_next();
                __syncthreads();
            };
            // Main loop: whole rounds of DEPTH tiles with no branch in the body, so that the compiler can
            // count the loads in flight exactly across the back edge; with a conditional stage inside it
            // waited for every load once per round.  The last, partial round follows.
            int kt0 = 0;
            for (; kt0 + DEPTH <= nkt; kt0 += DEPTH)
                static_for<0, DEPTH>([&](auto dc) { stage(dc, kt0 + decltype(dc)::value, false); });
            static_for<0, DEPTH>([&](auto dc) {
                if (kt0 + decltype(dc)::value < nkt) stage(dc, kt0 + decltype(dc)::value, true);
            });
        };
        using yes = std::integral_constant<bool, true>;
        using no = std::integral_constant<bool, false>;
        if (nkt > 0) {
            if (!EDGE) {
                pipe0(yes{}, yes{}, no{});
            } else if (!p.edge_buf) {
                pipe0(no{}, no{}, no{});   // a tile spans 2 GiB or more: flat element-wise loads
            } else {
                // Buffer loads fetch 128 bits at any 4-byte aligned address, a chunk that runs past the end of
                // its row or of the operand brings data that the mask removes or zeros: a unit stride is enough.
                const bool va = p.a_cont != 0, vb = p.b_cont != 0;
                if (va && vb) pipe0(yes{}, yes{}, yes{});
                else if (va) pipe0(yes{}, no{}, yes{});
                else if (vb) pipe0(no{}, yes{}, yes{});
                else pipe0(no{}, no{}, yes{});
            }
        }
    } else {
        static_assert(PIPE == 0 || NKG % 2 == 0, "the pipelined schedule needs an even number of groups per tile");
        // whole K-tiles of the pipelined loop; a general shape's last, partial tile follows it
        const int nkt_all = nkt;
        const int nkt = RAGGED_PIPE ? Kz / BK : nkt_all;
        constexpr int kReadsA = A_KC ? NBM : 4;
        constexpr int kReads = kReadsA + (B_KC ? NBN : 4);   // LDS reads per group
        constexpr int kWrites = NCHA + NCHB;                  // LDS stores per tile and thread
        constexpr int kMfma = 4 * NBM * NBN;                  // MFMAs per group
        Frag<A_KC, NBM> fa[2];
        Frag<B_KC, NBN> fb[2];
        auto load_whole = [&](int kt) {
            if (RAGGED_PIPE) {   // flat loads could fault on the rows past the operand
#pragma unroll
                for (int i = 0; i < NCHA; i++)
                    load_tile_chunk_buf<A_KC, BM, BK, NT>(ra, rsrc_a, kt * BK * (int)p.a_ks * 4, (int)a_ld * 4, (int)toff_a * 4, i);
#pragma unroll
                for (int i = 0; i < NCHB; i++)
                    load_tile_chunk_buf<B_KC, BN, BK, NT>(rb, rsrc_b, kt * BK * (int)p.b_ks * 4, (int)b_ld * 4, (int)toff_b * 4, i);
            } else {
                load_global(kt);
            }
        };
        // AMASK: the pre-activation tile kt into the registers beside staging set `set`; mask_chunk turns chunk i
        // of that set into A * f'(A2) on its way to LDS
        auto load_a2_chunk = [&](int kt, auto setc, int i) {
            if constexpr (AMASK)
                load_tile_chunk_buf<A_KC, BM, BK, NT>(rax2[decltype(setc)::value], rsrc_a2, kt * BK * (int)p.a_ks * 4,
                                                      (int)a_ld * 4, (int)toff_a * 4, i);
        };
        auto mask_chunk = [&](auto setc, int i) {
            if constexpr (AMASK) {
                constexpr int set = decltype(setc)::value;
                if (a_masked) {   // uniform
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        rax[set][i][j] = ((rax2[set][i][j] > 0) ? 1.0f : a_mask_slope) * rax[set][i][j];
                }
            }
        };
        constexpr std::integral_constant<int, 0> set0{};
        if (nkt > 0) {
            load_whole(0);
            if constexpr (AMASK) {
#pragma unroll
                for (int i = 0; i < NCHA; i++) load_a2_chunk(0, set0, i);
#pragma unroll
                for (int i = 0; i < NCHA; i++) mask_chunk(set0, i);
            }
            store_tile_lds<A_KC, BM, BK, NT>(lds_a[0], ra, tid);
            store_tile_lds<B_KC, BN, BK, NT>(lds_b[0], rb, tid);
        }
        __syncthreads();

        // One group of the schedule: the MFMAs of the fragments in `use`, cut into slots; slot s is
        // preceded by the s-th LDS read of the fragments for the next group (into `fill`, from
        // tile buffer `rbuf`, group `rkg`) and, when `store` is set, by the s-th LDS store of the
        // staged next tile (into buffer `wbuf`).  Scheduling fences pin that interleaving, so the
        // waves of a workgroup never hit LDS in one burst and no MFMA waits for an LDS round trip.
        auto group = [&](int use, int fill, bool read, int rbuf, int rkg, bool store, int wbuf, bool gload, int gkt,
                         auto setc) {
            constexpr int set = decltype(setc)::value;   // the staging registers that `store` empties / `gload` fills
            f32x4(&ra)[NCHA] = rax[set];
            f32x4(&rb)[NCHB] = rbx[set];
            const int memops = (store || gload) ? kWrites : 0;
            const int slots = (read ? kReads : 0) > memops ? (read ? kReads : 0) : memops;
            const int ga_off = gkt * BK * (int)p.a_ks * 4, gb_off = gkt * BK * (int)p.b_ks * 4;   // bytes, uniform
            const int per = slots > 0 ? kMfma / slots : kMfma;
            int q = 0;
#pragma unroll
            for (int sl = 0; sl < (kReads > kWrites ? kReads : kWrites); sl++) {
                if (sl < slots) {
                    if (read && sl < kReads) {
                        if (sl < kReadsA)
                            read_frag_piece<A_KC, NBM, BM, BK>(fa[fill], lds_a[rbuf], wm0, rkg, l32, half, sl);
                        else
                            read_frag_piece<B_KC, NBN, BN, BK>(fb[fill], lds_b[rbuf], wn0, rkg, l32, half, sl - kReadsA);
                    }
                    if (store && sl < kWrites) {
                        if (sl < NCHA) {
                            if constexpr (AMASK) mask_chunk(setc, sl);
                            store_tile_chunk<A_KC, BM, BK, NT>(lds_a[wbuf], ra, tid, sl);
                        } else {
                            store_tile_chunk<B_KC, BN, BK, NT>(lds_b[wbuf], rb, tid, sl - NCHA);
                        }
                    }
                    if (gload && sl < kWrites) {
                        if (sl < NCHA) {
                            load_tile_chunk_buf<A_KC, BM, BK, NT>(ra, rsrc_a, ga_off, (int)a_ld * 4, (int)toff_a * 4, sl);
                            if constexpr (AMASK) load_a2_chunk(gkt, setc, sl);
                        } else {
                            load_tile_chunk_buf<B_KC, BN, BK, NT>(rb, rsrc_b, gb_off, (int)b_ld * 4, (int)toff_b * 4, sl - NCHA);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    // fewer MFMAs than slots (one block per wave and an operand whose fragments take four reads):
                    // they are spread evenly over the slots instead
                    const int cnt = per > 0 ? per : ((sl + 1) * kMfma) / slots - (sl * kMfma) / slots;
#pragma unroll
                    for (int u = 0; u < kMfma; u++) {
                        if (u < cnt) {
                            const int t = q / (NBM * NBN), i = (q / NBN) % NBM, j = q % NBN;
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[use].get(i, t), fb[use].get(j, t),
                                                                            acc[i][j], 0, 0, 0);
                            q++;
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int u = 0; u < kMfma; u++) {
                if (q < kMfma) {
                    const int t = q / (NBM * NBN), i = (q / NBN) % NBM, j = q % NBN;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[use].get(i, t), fb[use].get(j, t), acc[i][j],
                                                                    0, 0, 0);
                    q++;
                }
            }
        };

        // The staging registers run one tile ahead of LDS: at the top of tile kt they hold tile
        // kt+1 (loaded during the last group of tile kt-1, or by the prologue).  Group NKG-2 moves
        // them into the free LDS buffer, one store per slot; the last group refills them with tile
        // kt+2, one global load per slot, so that the waves of a workgroup never queue all their
        // loads on the address unit at once and every load has most of a tile to land.
        if constexpr (DEPTH == 1) {
            if (nkt > 1) {
                load_whole(1);
                if constexpr (AMASK) {
#pragma unroll
                    for (int i = 0; i < NCHA; i++) load_a2_chunk(1, set0, i);
                }
            }
        } else if (nkt > 0) {
            // DEPTH > 1: tile t waits in staging set t % DEPTH, requested DEPTH tiles before its turn -- the
            // workgroups that have a compute unit to themselves and stream an operand from HBM need that much
            // (a load has a tile's time to land otherwise: 0.4 us for the 64x64 tile).  Tiles 1 .. DEPTH now
            // (tile DEPTH into set 0, which tile 0 has left); past the end: the last tile again, never stored.
            static_for<1, DEPTH + 1>([&](auto dc) {
                constexpr int d = decltype(dc)::value;
                const int kt = min(d, nkt - 1);
#pragma unroll
                for (int i = 0; i < NCHA; i++)
                    load_tile_chunk_buf<A_KC, BM, BK, NT>(rax[d % DEPTH], rsrc_a, kt * BK * (int)p.a_ks * 4, (int)a_ld * 4, (int)toff_a * 4, i);
                if constexpr (AMASK) {
#pragma unroll
                    for (int i = 0; i < NCHA; i++) load_a2_chunk(kt, std::integral_constant<int, d % DEPTH>{}, i);
                }
#pragma unroll
                for (int i = 0; i < NCHB; i++)
                    load_tile_chunk_buf<B_KC, BN, BK, NT>(rbx[d % DEPTH], rsrc_b, kt * BK * (int)p.b_ks * 4, (int)b_ld * 4, (int)toff_b * 4, i);
            });
        }
        if (nkt > 0) {
            read_frag<A_KC, NBM, BM, BK>(fa[0], lds_a[0], wm0, 0, l32, half);
            read_frag<B_KC, NBN, BN, BK>(fb[0], lds_b[0], wn0, 0, l32, half);
        }
        if constexpr (DEPTH == 1) {
            for (int kt = 0; kt + 1 < nkt; kt++) {
                const int cur = kt & 1;
                const int gkt = min(kt + 2, nkt - 1);   // clamped: the surplus load of the last round is never stored
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    if (kg + 1 < NKG) {
                        group(kg & 1, (kg + 1) & 1, true, cur, kg + 1, kg == NKG - 2, cur ^ 1, false, 0, set0);
                    } else {
                        // last group: everyone's stores are in LDS after the barrier; its MFMAs (operands
                        // already in registers) cover the first fragment reads of the next tile
                        __syncthreads();
                        group(kg & 1, (kg + 1) & 1, true, cur ^ 1, 0, false, 0, true, gkt, set0);
                    }
                }
            }
        } else {
            static_assert(DEPTH % 2 == 0, "an even number of staging sets keeps the LDS buffer of a tile a constant");
            // tile kt (in LDS buffer `curc`): group NKG-2 moves tile kt+1 from staging set `setc` into the other LDS
            // buffer, the last group refills that set with tile kt+1+DEPTH
            auto tile_round = [&](int kt, auto setc, auto curc) {
                constexpr int cur = decltype(curc)::value;
                const int gkt = min(kt + 1 + DEPTH, nkt - 1);   // clamped: a surplus load is never stored
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    if (kg + 1 < NKG) {
                        group(kg & 1, (kg + 1) & 1, true, cur, kg + 1, kg == NKG - 2, cur ^ 1, false, 0, setc);
                    } else {
                        __syncthreads();
                        group(kg & 1, (kg + 1) & 1, true, cur ^ 1, 0, false, 0, true, gkt, setc);
                    }
                }
            };
            // whole rounds over the staging sets without a condition inside, then a guarded remainder
            int kt0 = 0;
            for (; kt0 + DEPTH < nkt; kt0 += DEPTH)
                static_for<0, DEPTH>([&](auto dc) {
                    constexpr int d = decltype(dc)::value;
                    tile_round(kt0 + d, std::integral_constant<int, (d + 1) % DEPTH>{}, std::integral_constant<int, d & 1>{});
                });
            static_for<0, DEPTH>([&](auto dc) {
                constexpr int d = decltype(dc)::value;
                if (kt0 + d + 1 < nkt)   // uniform
                    tile_round(kt0 + d, std::integral_constant<int, (d + 1) % DEPTH>{}, std::integral_constant<int, d & 1>{});
            });
        }
        if (nkt > 0) {
            const int cur = (nkt - 1) & 1;
#pragma unroll
            for (int kg = 0; kg < NKG; kg++) group(kg & 1, (kg + 1) & 1, kg + 1 < NKG, cur, kg + 1, false, 0, false, 0, set0);
        }
        if constexpr (RAGGED_PIPE) {
            const int k0 = nkt * BK, k_left = Kz - k0;
            if (k_left > 0) {   // uniform
                int voa[NCHA][4], vob[NCHB][4];
                edge_offsets<A_KC, BM, BK, NT, false>(voa, p.a_rs, p.a_ks, tid);
                edge_offsets<B_KC, BN, BK, NT, false>(vob, p.b_rs, p.b_ks, tid);
                load_tile_edge_buf<NCHA, false>(
                    ra, edge_resource(reinterpret_cast<uint64_t>(uniform_ptr(Ab)), p.a_rs, p.a_ks, p.M - m0, Krem, k0), voa);
                load_tile_edge_buf<NCHB, false>(
                    rb, edge_resource(reinterpret_cast<uint64_t>(uniform_ptr(Bb)), p.b_rs, p.b_ks, p.N - n0, Krem, k0), vob);
                mask_tile_edge<A_KC, BM, BK, NT>(ra, rows_a, k_left, tid);
                mask_tile_edge<B_KC, BN, BK, NT>(rb, rows_b, k_left, tid);
                __syncthreads();   // every wave has read its last fragments of the whole tiles
                store_tile_lds<A_KC, BM, BK, NT>(lds_a[0], ra, tid);
                store_tile_lds<B_KC, BN, BK, NT>(lds_b[0], rb, tid);
                __syncthreads();
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    Frag<A_KC, NBM> ta;
                    Frag<B_KC, NBN> tb;
                    read_frag<A_KC, NBM, BM, BK>(ta, lds_a[0], wm0, kg, l32, half);
                    read_frag<B_KC, NBN, BN, BK>(tb, lds_b[0], wn0, kg, l32, half);
                    mfma_group(ta, tb);
                }
            }
        }
    }

    if (ROWSUM && do_rowsum && m0 + tid < p.M) {
        float* g = p.rowsum + m0 + tid;
        *g = p.rowsum_acc ? *g + rowsum : rowsum;
    }
    const float alpha = p.has_alpha ? (p.alpha ? *p.alpha : 0.f) : 1.f;
    const float leaky = p.leaky ? *p.leaky : 0.f;
    gemm_epilogue<NBM, NBN, A_KC, B_KC>(p, acc, m0, n0, c_off, wm0, wn0, l32, half, alpha, leaky);
}

template <int WM, int WN, int NBM, int NBN, int BK, bool A_KC, bool B_KC, bool EDGE, int PIPE = 0, int MINW = 1,
          int DEPTH = 1, bool ROWSUM = false>
__global__ void __launch_bounds__(64 * WM * WN, MINW) gemm_mfma_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) float lds_a[2][TileShape<A_KC, WM * NBM * 32, BK>::kFloats];
    __shared__ __attribute__((aligned(16))) float lds_b[2][TileShape<B_KC, WN * NBN * 32, BK>::kFloats];
    gemm_tile_body<WM, WN, NBM, NBN, BK, A_KC, B_KC, EDGE, PIPE, DEPTH, ROWSUM, false>(p, blockIdx.x, blockIdx.z, lds_a,
                                                                                       lds_b);
}

}  // namespace kai
