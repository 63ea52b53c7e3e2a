// Instantiates the tile configurations of the MFMA GEMM for one pair of operand
// orientations.  Included by one translation unit per pair so that they compile in
// parallel.
//
//   large  256x256 tile, 8 waves of 128x64 (2 waves per SIMD)  -- big, compute-bound products
//   medium 128x128 tile, 4 waves of 64x64, 2 workgroups per CU -- fills the chip at mid sizes
//   small   64x64  tile, 4 waves of 32x32                      -- small or very ragged products
//   wide    64x128 tile, 4 waves of 32x64                      -- whole tiles, fewer workgroups than the small tile
//   flat    32x128 tile, 4 waves of 32x32 side by side         -- 17..32 rows against many columns, and row counts that
//                                                                 fill an odd number of 32-row tiles (65..96, 129..160, 193..224)
// On the two bigger tiles, operands that allow 128-bit loads run the pipelined kernel: predicate-free
// when the shape is a whole multiple of the tile, else with range-checked buffer resources and one
// masked K-tile at the end.  The wide tile and the small tile run the pipelined kernel too, each with one to four
// tiles on their way in registers (staging_depth).  Everything else runs the general kernel with the simple
// schedule.  pick_gemm_variant (gemm_host.h) chooses; this file turns its answer into the instantiation.
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

template <bool A_KC, bool B_KC>
int launch_gemm_layout(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream) {
    const GemmVariant v = pick_gemm_variant(p, A_KC, B_KC, nbatch, tile);
    const bool whole = v.kind == kKindWholePipelined, ragged = v.kind == kKindRaggedPipelined;
    switch (v.tile) {
    case kTileLarge:
        if (whole && v.depth == 2) return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, false, 1, 1, 2>(p, nbatch, kGroupM, stream);
        if (whole) return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, false, 1, 1, 1>(p, nbatch, kGroupM, stream);
        if (ragged && v.depth == 2) return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, true, 1, 1, 2>(p, nbatch, kGroupM, stream);
        if (ragged) return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, true, 1, 1, 1>(p, nbatch, kGroupM, stream);
        return launch_gemm_config<2, 4, 4, 2, 16, A_KC, B_KC, true>(p, nbatch, kGroupM, stream);
    case kTileMedium:
        if (whole && v.depth == 2) return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, false, 1, 2, 2>(p, nbatch, kGroupM, stream);
        if (whole) return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, false, 1, 2, 1>(p, nbatch, kGroupM, stream);
        if (ragged && v.depth == 2) return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, true, 1, 2, 2>(p, nbatch, kGroupM, stream);
        if (ragged) return launch_gemm_config<2, 2, 2, 2, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
        return launch_gemm_config<2, 2, 2, 2, 16, A_KC, B_KC, true>(p, nbatch, kGroupM, stream);
    case kTileFlat:
        if (v.kind == kKindWhole) return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, false, 0, 2, 4>(p, nbatch, kGroupM, stream);
        if (ragged && v.depth == 2) return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, true, 1, 2, 2>(p, nbatch, kGroupM, stream);
        if (ragged) return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
        return launch_gemm_config<1, 4, 1, 1, 32, A_KC, B_KC, true, 0, 1, 4>(p, nbatch, kGroupM, stream);
    case kTileWide:
        if (whole && v.depth == 4) return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, false, 1, 2, 4>(p, nbatch, kGroupM, stream);
        if (whole && v.depth == 2) return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, false, 1, 2, 2>(p, nbatch, kGroupM, stream);
        if (whole) return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, false, 1, 2, 1>(p, nbatch, kGroupM, stream);
        if (v.depth == 2) return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, true, 1, 2, 2>(p, nbatch, kGroupM, stream);
        return launch_gemm_config<2, 2, 1, 2, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
    default:
        if (whole && v.depth == 4) return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, false, 1, 2, 4>(p, nbatch, kGroupM, stream);
        if (whole) return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, false, 1, 2, 1>(p, nbatch, kGroupM, stream);
        if (ragged && v.depth == 4) return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, true, 1, 2, 4>(p, nbatch, kGroupM, stream);
        if (ragged) return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, true, 1, 2, 1>(p, nbatch, kGroupM, stream);
        if (v.kind == kKindWhole && v.bk == 32) return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, false, 0, 2, 4>(p, nbatch, kGroupM, stream);
        if (v.kind == kKindWhole) return launch_gemm_config<2, 2, 1, 1, 16, A_KC, B_KC, false, 0, 2, 8>(p, nbatch, kGroupM, stream);
        if (v.bk == 32) return launch_gemm_config<2, 2, 1, 1, 32, A_KC, B_KC, true, 0, 1, 4>(p, nbatch, kGroupM, stream);
        return launch_gemm_config<2, 2, 1, 1, 16, A_KC, B_KC, true, 0, 1, 4>(p, nbatch, kGroupM, stream);
    }
}

}  // namespace kai
