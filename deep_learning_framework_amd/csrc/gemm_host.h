// Host-side description of one (batched) GEMM and the launcher of one kernel
// configuration.  Used by gemm_dispatch.hip, which picks the configuration.
#pragma once

#include <string>

#include "gemm_mfma.h"
#include "kai_common.h"

namespace kai {

// C(m,n) (=|+=) act(alpha * sum_k A(m,k)*B(n,k) + bias[n]) with arbitrary element strides.
struct GemmDesc {
    const float* A = nullptr;
    const float* B = nullptr;
    float* C = nullptr;
    float* C2 = nullptr;
    const float* bias = nullptr;
    const float* alpha = nullptr;
    const float* leaky = nullptr;
    int64_t M = 0, N = 0, K = 0;
    int64_t a_rs = 0, a_ks = 1, b_rs = 0, b_ks = 1, c_rs = 0, c_cs = 1;
    int64_t nbatch = 1, bdiv = 1;
    int64_t a_bs0 = 0, a_bs1 = 0, b_bs0 = 0, b_bs1 = 0, c_bs0 = 0, c_bs1 = 0;
    int act = 0;
    int acc = 0;
    int has_alpha = 0;
    // optional: rowsum[m] (=|+=) sum_k A(m,k) computed by the same launch; only products for which
    // gemm_fuses_rowsum() holds may set it
    float* rowsum = nullptr;
    int rowsum_acc = 0;
    // > 0: the nbatch batches are consecutive parts of k_part reduction steps of ONE product of length K
    // (the last part may be shorter); the batch strides of A and B must then be k_part steps
    int64_t k_part = 0;
    // where a reduction cut into parts puts its partial sums: null = the library's own scratch (allocated and
    // grown on demand); otherwise this buffer of scratch_bytes, and a product that needs more is refused
    float* scratch = nullptr;
    int64_t scratch_bytes = 0;
};

// LDS orientation of an operand: reduction index contiguous (KC) or output index contiguous (MC).
// A strided operand (neither stride is 1) goes to the orientation of its smaller stride.
inline bool operand_is_kc(int64_t rs, int64_t ks) { return ks == 1 || (rs != 1 && ks <= rs); }

inline GemmParams make_params(const GemmDesc& d, bool a_kc, bool b_kc) {
    GemmParams p{};
    p.A = d.A; p.B = d.B; p.C = d.C; p.C2 = d.C2; p.bias = d.bias; p.alpha = d.alpha; p.leaky = d.leaky;
    p.M = (int)d.M; p.N = (int)d.N; p.K = (int)d.K;
    p.a_rs = d.a_rs; p.a_ks = d.a_ks; p.b_rs = d.b_rs; p.b_ks = d.b_ks; p.c_rs = d.c_rs; p.c_cs = d.c_cs;
    p.a_bs0 = d.a_bs0; p.a_bs1 = d.a_bs1; p.b_bs0 = d.b_bs0; p.b_bs1 = d.b_bs1; p.c_bs0 = d.c_bs0; p.c_bs1 = d.c_bs1;
    p.bdiv = (int)d.bdiv;
    // 128-bit loads need: unit stride along the LDS-contiguous index, the other stride and every
    // batch stride a multiple of 4 elements, and a 16-byte aligned base
    const int64_t a_cont = a_kc ? d.a_ks : d.a_rs, a_ld = a_kc ? d.a_rs : d.a_ks;
    const int64_t b_cont = b_kc ? d.b_ks : d.b_rs, b_ld = b_kc ? d.b_rs : d.b_ks;
    p.a_vec = a_cont == 1 && a_ld % 4 == 0 && d.a_bs0 % 4 == 0 && d.a_bs1 % 4 == 0 && aligned16(d.A);
    p.b_vec = b_cont == 1 && b_ld % 4 == 0 && d.b_bs0 % 4 == 0 && d.b_bs1 % 4 == 0 && aligned16(d.B);
    p.a_cont = a_cont == 1;
    p.b_cont = b_cont == 1;
    p.c_vec = d.c_cs == 1 && d.c_rs % 4 == 0 && d.N % 4 == 0 && d.c_bs0 % 4 == 0 && d.c_bs1 % 4 == 0 &&
              aligned16(d.C) && (d.C2 == nullptr || aligned16(d.C2)) && (d.bias == nullptr || aligned16(d.bias));
    p.act = d.act;
    p.accflag = d.acc;
    p.has_alpha = d.has_alpha;
    p.rowsum = d.rowsum;
    p.rowsum_acc = d.rowsum_acc;
    p.k_part = (int)d.k_part;
    return p;
}

// true when the predicate-free kernel variant may run this problem with tile BM x BN x BK
inline bool fits_without_edges(const GemmParams& p, bool a_kc, bool b_kc, int BM, int BN, int BK) {
    const int64_t a_ld = a_kc ? p.a_rs : p.a_ks, b_ld = b_kc ? p.b_rs : p.b_ks;
    return p.k_part == 0 && p.a_vec && p.b_vec && p.M % BM == 0 && p.N % BN == 0 && p.K % BK == 0 && p.K > 0 &&
           a_ld * BM < (1ll << 30) && b_ld * BN < (1ll << 30);
}

// The pipelined kernels address their operands as a 32-bit byte offset from the first row of the workgroup's
// tile (buffer loads): the whole extent of a tile row block must stay below 2 GiB.
inline bool fits_buffer_offsets(const GemmParams& p, bool a_kc, bool b_kc, int BM, int BN) {
    const int64_t a_span = a_kc ? (BM - 1) * p.a_rs + p.K : (p.K - 1) * p.a_ks + BM;
    const int64_t b_span = b_kc ? (BN - 1) * p.b_rs + p.K : (p.K - 1) * p.b_ks + BN;
    return a_span * 4 < (1ll << 31) && b_span * 4 < (1ll << 31);
}

// true when the pipelined kernel's general variant may run the problem: both operands have a unit stride (its
// buffer loads fetch 128 bits at any 4-byte aligned address; M, N, K and the leading dimensions are arbitrary:
// rows past the end are never stored, the last partial K-tile is masked; a reduction cut over the batch index
// into parts of k_part steps is fine, too)
inline bool fits_ragged_pipe(const GemmParams& p, bool a_kc, bool b_kc, int BM, int BN) {
    const int64_t a_ld = a_kc ? p.a_rs : p.a_ks, b_ld = b_kc ? p.b_rs : p.b_ks;
    return p.a_cont && p.b_cont && p.K > 0 && a_ld * BM < (1ll << 30) && b_ld * BN < (1ll << 30) &&
           fits_buffer_offsets(p, a_kc, b_kc, BM, BN);
}

template <int WM, int WN, int NBM, int NBN, int BK, bool A_KC, bool B_KC, bool EDGE, int PIPE = 0, int MINW = 1,
          int DEPTH = 1, bool ROWSUM = false>
int launch_gemm_config(GemmParams p, int64_t nbatch, int group_m, hipStream_t stream) {
    constexpr int BM = WM * NBM * 32, BN = WN * NBN * 32;
    {
        // byte span of one tile of each operand (its lane offsets are 32-bit in the buffer-load variants)
        const int64_t a_span = ((BM - 1) * p.a_rs + (BK - 1) * p.a_ks + 1) * 4;
        const int64_t b_span = ((BN - 1) * p.b_rs + (BK - 1) * p.b_ks + 1) * 4;
        p.edge_buf = a_span < (1ll << 31) && b_span < (1ll << 31);
    }
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    p.group_m = group_m < 1 ? 1 : group_m;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    if (tiles <= 0 || nbatch <= 0) return KAI_OK;
    if (tiles > kMaxDim || nbatch > 65535) return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: grid too large");
    dim3 grid((unsigned)tiles, 1, (unsigned)nbatch);
    gemm_mfma_kernel<WM, WN, NBM, NBN, BK, A_KC, B_KC, EDGE, PIPE, MINW, DEPTH, ROWSUM>
        <<<grid, dim3(64 * WM * WN), 0, stream>>>(p);
    return check_launch("gemm_mfma_kernel");
}

// picks kernel family, tile and variant; defined in gemm_dispatch.hip
int launch_gemm(const GemmDesc& d, hipStream_t stream);
// a maintainer's override of that choice (kai_gemm_force_plan); "auto" clears it
int set_forced_gemm_plan(const char* text);
// the decision of launch_gemm as text (host arithmetic only)
std::string describe_gemm(const GemmDesc& d);
// true when launch_gemm would compute GemmDesc::rowsum inside the product's own launch (d.rowsum is
// not looked at); otherwise the caller runs a separate column-sum kernel and leaves rowsum null
bool gemm_fuses_rowsum(const GemmDesc& d);

// short reductions (K <= 64) with both operands K-contiguous and a contiguous output row: gemm_shortk.hip
bool shortk_nt_applies(const GemmDesc& d);
int launch_gemm_shortk_nt(GemmParams p, int64_t nbatch, hipStream_t stream);
// the same with the inner batch index (heads) interleaved in C: element stride = number of heads
bool shortk_heads_applies(const GemmDesc& d);
int launch_gemm_shortk_heads(GemmParams p, int64_t nbatch, hipStream_t stream);

// small products with a long reduction, both operands K-contiguous: the reduction is cut over the waves of a
// workgroup (gemm_wavesplit.hip); block_edge is 32 or 16
bool wavesplit_applies(const GemmDesc& d);
int launch_gemm_wavesplit(const GemmDesc& d, int block_edge, hipStream_t stream);

// at most 16 rows against a matrix stored [K, N] (skinny_rows.hip; uses the library's scratch memory)
bool skinny_rows_applies(const GemmDesc& d);
int launch_skinny_rows(const GemmDesc& d, hipStream_t stream);

// products of the head-interleaved attention tensor with several heads per batch entry: heads_pv.hip
bool heads_pv_applies(const GemmDesc& d);
int launch_heads_pv(const GemmDesc& d, hipStream_t stream);

// the two products and the bias gradient of a dense layer's backward pass in one launch: dense_backward.hip
int dense_backward_pair_split(const float* pgx, const float* pgw, const float* pgy, const float* pw, const float* px,
                              const float* ppre, int64_t yvec, int64_t ndat, int64_t xvec, int act);
int launch_dense_backward_pair(float* pgx, float* pgw, float* pgb, const float* pgy, const float* pw, const float* px,
                               const float* ppre, int64_t yvec, int64_t ndat, int64_t xvec, int act,
                               const float* leaky, bool acc, int split, hipStream_t stream);

// per-layout entry points (one translation unit each, to compile in parallel)
// flat: 32 rows x 128 columns; wide: 64 rows x 128 columns (pipelined kernels only, else the small tile runs)
enum GemmTile { kTileLarge = 0, kTileMedium = 1, kTileSmall = 2, kTileFlat = 3, kTileWide = 4 };

// Which kernel of a tile runs a product.  whole: predicate-free (the shape is a whole multiple of the tile, 128-bit
// loads); ragged pipelined: range-checked buffer resources and one masked K-tile at the end; general: any strides.
enum GemmKind { kKindGeneral = 0, kKindWhole = 1, kKindWholePipelined = 2, kKindRaggedPipelined = 3 };
struct GemmVariant {
    int tile;    // the tile that runs (the wide tile gives way to the small one where it has no kernel)
    int kind;
    int bk;      // reduction steps per tile
    int depth;   // tiles on their way in registers (pipelined kernels: 1, 2 or 4; the others: their fixed ring)
};

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

// The kernel that launch_gemm_layout starts for a tile choice (host arithmetic only).
inline GemmVariant pick_gemm_variant(const GemmParams& p, bool a_kc, bool b_kc, int64_t nbatch, int tile) {
    auto whole = [&](int bm, int bn, int bk) {
        return fits_without_edges(p, a_kc, b_kc, bm, bn, bk) && fits_buffer_offsets(p, a_kc, b_kc, bm, bn);
    };
    auto groups = [&](int bm, int bn) { return (int64_t)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * nbatch; };
    switch (tile) {
    case kTileLarge:
        if (whole(256, 256, 16)) return {tile, kKindWholePipelined, 16, staging_depth(tile, p, 0, nbatch, 16)};
        if (fits_ragged_pipe(p, a_kc, b_kc, 256, 256))
            return {tile, kKindRaggedPipelined, 16, staging_depth(tile, p, 0, nbatch, 16)};
        return {tile, kKindGeneral, 16, 1};
    case kTileMedium:
        if (whole(128, 128, 32))
            return {tile, kKindWholePipelined, 32, staging_depth(tile, p, groups(128, 128), nbatch, 32)};
        if (fits_ragged_pipe(p, a_kc, b_kc, 128, 128))
            return {tile, kKindRaggedPipelined, 32, staging_depth(tile, p, groups(128, 128), nbatch, 32)};
        return {tile, kKindGeneral, 16, 1};
    case kTileFlat:
        // 17..32 rows against many columns (a batch against a weight matrix), or several rows of such tiles where
        // 64-row tiles would pad more (65..96, 129..160, 193..224 rows): four waves side by side, so that the matrix
        // cores do not spend half their time on rows that do not exist.  With edges
        // the pipelined schedule is the faster one (80 x 4096 x 4096: 41.2 -> 36.6 us, 72 x 4096 x 11008:
        // 88.6 -> 79.9, 17 and 24 rows 22.9 -> 22.4), and so it is with whole tiles in several rows of tiles
        // (96 x 4096 x 4096: 35.7 -> 33.1 us, 96 x 2048 x 2048 17.9 -> 15.9, 96 x 4096 x 11008 76.2 -> 72.6,
        // 160 x 4096 x 4096 56.4 -> 52.0; the variant without range checks measured the same as the one with
        // them, so there is only the latter); one row of whole tiles loses with it (32 x 11008 x 4096:
        // 50 -> 65: the stream of the other operand wants the four tiles in flight that the simple schedule keeps)
        if (whole(32, 128, 32) && p.M <= 32) return {tile, kKindWhole, 32, 4};
        if (fits_ragged_pipe(p, a_kc, b_kc, 32, 128))
            return {tile, kKindRaggedPipelined, 32, staging_depth(tile, p, 0, nbatch, 32)};
        return {tile, kKindGeneral, 32, 4};
    case kTileWide:
        if (whole(64, 128, 32))
            return {tile, kKindWholePipelined, 32, staging_depth(tile, p, groups(64, 128), nbatch, 32)};
        if (fits_ragged_pipe(p, a_kc, b_kc, 64, 128))
            return {tile, kKindRaggedPipelined, 32, staging_depth(tile, p, groups(64, 128), nbatch, 32) >= 2 ? 2 : 1};
        [[fallthrough]];
    default: {
        // The pipelined schedule (fragment reads and LDS stores dealt between the MFMAs).  Both operands
        // K-contiguous: a 32-step tile takes 0.48 us whether the workgroup has the compute unit to itself or not,
        // the simple schedule 0.53-0.70 (1024^3: 22.6 -> 18.9 us, 512 x 2048 x 2048: 41.0 -> 34.2,
        // 64 x 4096 x 4096: 27.2 -> 22.8).  An operand that is not K-contiguous takes four LDS reads per fragment
        // instead of one: the pipelined schedule still wins while at most three workgroups share a unit
        // (1024^3 23.7 -> 21.8, 128 x 2048 x 2048 18.0 -> 16.5) and loses beyond (3072^3: 420 -> 432).
        const int64_t small_tiles = groups(64, 64);
        const bool pipelined = (a_kc && b_kc) || small_tiles <= 3 * (int64_t)compute_units();
        if (whole(64, 64, 32)) {
            if (pipelined) return {kTileSmall, kKindWholePipelined, 32, staging_depth(kTileSmall, p, small_tiles, nbatch, 32)};
            // a 64x64x16 tile computes for ~0.25 us, a global load takes ~1-2 us: 128 reduction steps in flight
            // (measured with whole tiles of 32 steps against 16 and 64: 15.5 / 16.9 / 16.0 us for 256x1024x1024)
            return {kTileSmall, kKindWhole, 32, 4};
        }
        // shapes with edges: the pipelined schedule in every operand form (777^3 with a [K, N] operand
        // 24.2 -> 19.1 us, 200 x 200 x 8192 20.5 -> 16.5)
        if (fits_ragged_pipe(p, a_kc, b_kc, 64, 64))
            return {kTileSmall, kKindRaggedPipelined, 32, staging_depth(kTileSmall, p, small_tiles, nbatch, 32)};
        if (whole(64, 64, 16)) return {kTileSmall, kKindWhole, 16, 8};
        // 32-step tiles halve the number of rounds; with an operand that is strided in both directions (one
        // head of an interleaved tensor) the element-wise loads of a tile cost more than the round saves
        // (measured: 1000x777x333 28.8 -> 26.7 us, head-strided 512x512x64 26 -> 32 us)
        if (p.K >= 128 && (p.a_ks == 1 || p.a_rs == 1) && (p.b_ks == 1 || p.b_rs == 1))
            return {kTileSmall, kKindGeneral, 32, 4};
        return {kTileSmall, kKindGeneral, 16, 4};
    }
    }
}

int launch_gemm_kc_kc(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream);
int launch_gemm_kc_mc(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream);
int launch_gemm_mc_mc(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream);
int launch_gemm_mc_kc(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream);

}  // namespace kai
