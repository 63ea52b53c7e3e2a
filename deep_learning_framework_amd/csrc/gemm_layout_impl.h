// Instantiates the tile configurations of the MFMA GEMM for one pair of operand
// orientations.  Included by one translation unit per pair so that they compile in
// parallel.
//
//   large  256x256 tile, 8 waves of 128x64 (2 waves per SIMD)  -- big, compute-bound products
//   medium 128x128 tile, 4 waves of 64x64, 2 workgroups per CU -- fills the chip at mid sizes
//   small   64x64  tile, 4 waves of 32x32                      -- small or very ragged products
//   wide    64x128 tile, 4 waves of 32x64                      -- whole tiles, fewer workgroups than the small tile
//   flat    32x128 tile, 4 waves of 32x32 side by side         -- at most 32 rows against many columns
// On the two bigger tiles, operands that allow 128-bit loads run the pipelined kernel: predicate-free
// when the shape is a whole multiple of the tile, else with range-checked buffer resources and one
// masked K-tile at the end.  The wide tile and the small tile run the pipelined kernel too, each with one to four
// tiles on their way in registers (staging_depth).  Everything else runs the general kernel with the simple
// schedule.
#pragma once

#include "gemm_host.h"

namespace kai {

constexpr int kGroupM = 4;

// the variants that also sum the rows of A (medium and small tiles, simple schedule)
template <bool A_KC, bool B_KC>
int launch_gemm_layout_rowsum(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream) {
    if (tile == kTileMedium)
        return launch_gemm_config<2, 2, 2, 2, 16, A_KC, B_KC, true, 0, 1, 1, true>(p, nbatch, kGroupM, stream);
    if (fits_without_edges(p, A_KC, B_KC, 64, 64, 16) && fits_buffer_offsets(p, A_KC, B_KC, 64, 64))
        return launch_gemm_config<2, 2, 1, 1, 16, A_KC, B_KC, false, 0, 2, 8, true>(p, nbatch, kGroupM, stream);
    return launch_gemm_config<2, 2, 1, 1, 16, A_KC, B_KC, true, 0, 1, 1, true>(p, nbatch, kGroupM, stream);
}

// How many tiles the pipelined kernels keep on their way in registers (their DEPTH).  A load has that many tiles'
// time to land; one tile's time is little for a workgroup that has a compute unit to itself, and too little when
// the operand comes from HBM or the last-level cache instead of L2 (64 x 4096 x 4096 with the matrix from HBM,
// one 64x64 workgroup per unit: 0.73 us per tile against 0.48; 512 x 4096 x 4096 on the wide tile: 139 -> 120 us
// with four tiles in flight).  Measured over 1..8 workgroups per unit x 4..128 tiles per workgroup, both operand
// forms, operands in L2: below 16 tiles the requests for tiles that do not exist cost 2-9 %; the small tile gains
// 1-9 % with four tiles up to four workgroups per unit and loses 8-13 % with six or eight; the wide tile gains
// 1-5 % with two tiles up to three workgroups per unit (and loses 14 % at four with a [K, N] operand); the two
// big tiles gain 1-5 % with two on long reductions.
inline int staging_depth(int tile, const GemmParams& p, int64_t groups, int64_t nbatch, int bk) {
    const int64_t k_len = p.k_part > 0 ? p.k_part : p.K;
    const int64_t tiles_k = k_len / bk;
    const int64_t cus = compute_units();
    const bool streamed = (int64_t)(p.M > p.N ? p.M : p.N) * k_len * nbatch * 4 >= (32ll << 20);
    switch (tile) {
    case kTileSmall:
        return (tiles_k >= 32 && groups <= 4 * cus) || (tiles_k >= 16 && groups <= 2 * cus) ? 4 : 1;
    case kTileWide:
        if (streamed && tiles_k >= 32 && groups <= 2 * cus) return 4;
        return tiles_k >= 16 && groups <= 3 * cus ? 2 : 1;
    case kTileMedium:
        return tiles_k >= 32 && groups <= 2 * cus ? 2 : 1;
    default:   // large (256 x 256 x 16), flat with edges
        return tiles_k >= 32 ? 2 : 1;
    }
}

template <bool A_KC, bool B_KC>
int launch_gemm_layout(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream) {
    switch (tile) {
    case kTileLarge:
        if (fits_without_edges(p, A_KC, B_KC, 256, 256, 16) && fits_buffer_offsets(p, A_KC, B_KC, 256, 256)) {
            if (staging_depth(tile, p, 0, nbatch, 16) == 2)
                return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, false, 1, 1, 2>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, false, 1, 1, 1>(p, nbatch, kGroupM, stream);
        }
        if (fits_ragged_pipe(p, A_KC, B_KC, 256, 256)) {
            if (staging_depth(tile, p, 0, nbatch, 16) == 2)
                return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, true, 1, 1, 2>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, true, 1, 1, 1>(p, nbatch, kGroupM, stream);
        }
        return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, true>(p, nbatch, kGroupM, stream);
    case kTileMedium:
        if (fits_without_edges(p, A_KC, B_KC, 128, 128, 32) && fits_buffer_offsets(p, A_KC, B_KC, 128, 128)) {
            if (staging_depth(tile, p, (int64_t)(p.M / 128) * (p.N / 128) * nbatch, nbatch, 32) == 2)
                return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, false, 1, 2, 2>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, false, 1, 2, 1>(p, nbatch, kGroupM, stream);
        }
        if (fits_ragged_pipe(p, A_KC, B_KC, 128, 128)) {
            if (staging_depth(tile, p, (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * nbatch, nbatch, 32) == 2)
                return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, true, 1, 2, 2>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
        }
        return launch_gemm_config<2, 2, 2, 2, 16, A_KC, B_KC, true>(p, nbatch, kGroupM, stream);
    case kTileFlat:
        // at most 32 rows against many columns (a batch of 17..32 rows against a weight matrix): four waves side
        // by side, so that the matrix cores do not spend half their time on rows that do not exist
        if (fits_without_edges(p, A_KC, B_KC, 32, 128, 32) && fits_buffer_offsets(p, A_KC, B_KC, 32, 128))
            return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, false, 0, 2, 4>(p, nbatch, kGroupM, stream);
        // with edges the pipelined schedule is the faster one (80 x 4096 x 4096: 41.2 -> 36.6 us, 72 x 4096 x 11008:
        // 88.6 -> 79.9, 17 and 24 rows 22.9 -> 22.4); whole tiles lose with it (32 x 11008 x 4096: 50 -> 65: the
        // stream of the other operand wants the four tiles in flight that the simple schedule keeps)
        if (fits_ragged_pipe(p, A_KC, B_KC, 32, 128)) {
            if (staging_depth(tile, p, 0, nbatch, 32) == 2)
                return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, true, 1, 2, 2>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
        }
        return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, true, 0, 1, 4>(p, nbatch, kGroupM, stream);
    case kTileWide:
        if (fits_without_edges(p, A_KC, B_KC, 64, 128, 32) && fits_buffer_offsets(p, A_KC, B_KC, 64, 128)) {
            const int depth = staging_depth(kTileWide, p, (int64_t)(p.M / 64) * (p.N / 128) * nbatch, nbatch, 32);
            if (depth == 4) return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, false, 1, 2, 4>(p, nbatch, kGroupM, stream);
            if (depth == 2) return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, false, 1, 2, 2>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, false, 1, 2, 1>(p, nbatch, kGroupM, stream);
        }
        if (fits_ragged_pipe(p, A_KC, B_KC, 64, 128)) {
            const int depth = staging_depth(kTileWide, p, (int64_t)((p.M + 63) / 64) * ((p.N + 127) / 128) * nbatch, nbatch, 32);
            if (depth >= 2) return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, true, 1, 2, 2>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
        }
        [[fallthrough]];
    default:
        // The pipelined schedule (fragment reads and LDS stores dealt between the MFMAs).  Both operands
        // K-contiguous: a 32-step tile takes 0.48 us whether the workgroup has the compute unit to itself or not,
        // the simple schedule below 0.53-0.70 (1024^3: 22.6 -> 18.9 us, 512 x 2048 x 2048: 41.0 -> 34.2,
        // 64 x 4096 x 4096: 27.2 -> 22.8).  An operand that is not K-contiguous takes four LDS reads per fragment
        // instead of one: the pipelined schedule still wins while at most three workgroups share a unit
        // (1024^3 23.7 -> 21.8, 128 x 2048 x 2048 18.0 -> 16.5) and loses beyond (3072^3: 420 -> 432).
        {
            const int64_t small_tiles = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * nbatch;
            const bool pipelined = (A_KC && B_KC) || small_tiles <= 3 * (int64_t)compute_units();
            if (pipelined && fits_without_edges(p, A_KC, B_KC, 64, 64, 32) && fits_buffer_offsets(p, A_KC, B_KC, 64, 64)) {
                if (staging_depth(kTileSmall, p, small_tiles, nbatch, 32) == 4)
                    return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, false, 1, 2, 4>(p, nbatch, kGroupM, stream);
                return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, false, 1, 2, 1>(p, nbatch, kGroupM, stream);
            }
        }
        // a 64x64x16 tile computes for ~0.25 us, a global load takes ~1-2 us: 128 reduction steps in flight
        // (measured with whole tiles of 32 steps against 16 and 64: 15.5 / 16.9 / 16.0 us for 256x1024x1024)
        if (fits_without_edges(p, A_KC, B_KC, 64, 64, 32) && fits_buffer_offsets(p, A_KC, B_KC, 64, 64))
            return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, false, 0, 2, 4>(p, nbatch, kGroupM, stream);
        // shapes with edges: the pipelined schedule in every operand form (777^3 with a [K, N] operand 24.2 -> 19.1 us,
        // 200 x 200 x 8192 20.5 -> 16.5)
        if (fits_ragged_pipe(p, A_KC, B_KC, 64, 64)) {
            const int64_t groups = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * nbatch;
            if (staging_depth(kTileSmall, p, groups, nbatch, 32) == 4)
                return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, true, 1, 2, 4>(p, nbatch, kGroupM, stream);
            return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
        }
        if (fits_without_edges(p, A_KC, B_KC, 64, 64, 16) && fits_buffer_offsets(p, A_KC, B_KC, 64, 64))
            return launch_gemm_config<2, 2, 1, 1, 16, A_KC, B_KC, false, 0, 2, 8>(p, nbatch, kGroupM, stream);
        // 32-step tiles halve the number of rounds; with an operand that is strided in both directions (one
        // head of an interleaved tensor) the element-wise loads of a tile cost more than the round saves
        // (measured: 1000x777x333 28.8 -> 26.7 us, head-strided 512x512x64 26 -> 32 us)
        if (p.K >= 128 && (p.a_ks == 1 || p.a_rs == 1) && (p.b_ks == 1 || p.b_rs == 1))
            return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, true, 0, 1, 4>(p, nbatch, kGroupM, stream);
        return launch_gemm_config<2, 2, 1, 1, 16, A_KC, B_KC, true, 0, 1, 4>(p, nbatch, kGroupM, stream);
    }
}

}  // namespace kai
