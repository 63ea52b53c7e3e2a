// Chooses the kernel for one (batched) product: the bandwidth-bound skinny kernel for at
// most 16 rows against a K-contiguous weight matrix, the wave-split kernel for small products that
// one launch can finish in a few microseconds, otherwise the MFMA kernel in the LDS orientation
// pair that matches how the operands lie in memory, with the tile that needs the fewest rounds
// over the compute units.
#include <algorithm>
#include <cstdlib>
#include <string>

#include "elementwise.h"
#include "gemm_host.h"
#include "gemv_skinny.h"

namespace kai {

static int64_t tiles_of(int64_t M, int64_t N, int64_t nbatch, int64_t t) {
    return ((M + t - 1) / t) * ((N + t - 1) / t) * nbatch;
}

// Only reductions of at least kSplitFromK steps are cut (a shorter one does not repay the second
// launch), into at most kSplitMax parts of at least kSplitMinK steps each.
constexpr int64_t kSplitFromK = 512;
constexpr int64_t kSplitMinK = 64;
constexpr int64_t kSplitMax = 16;
constexpr int64_t kSplitScratchMax = 64ll << 20;   // bytes of partial sums a product may ask of the library scratch

static int launch_layout(const GemmParams& p, bool a_kc, bool b_kc, int64_t nbatch, int tile, hipStream_t stream) {
    if (a_kc && b_kc) return launch_gemm_kc_kc(p, nbatch, tile, stream);
    if (a_kc && !b_kc) return launch_gemm_kc_mc(p, nbatch, tile, stream);
    if (!a_kc && !b_kc) return launch_gemm_mc_mc(p, nbatch, tile, stream);
    return launch_gemm_mc_kc(p, nbatch, tile, stream);
}

namespace {

// A maintainer's override of the choice below (kai_gemm_force_plan): the tile and / or the number of parts of the
// reduction, or the one-launch kernel for small products.  Process-wide, meant for audits of the fitted rules
// (bench.py --plan-audit times the chosen plan against every alternative), never set in production.
struct ForcedPlan {
    bool active = false;
    int tile = -1;          // kTile* or -1: keep the chosen tile
    int64_t split = 0;      // >= 1: this many parts; 0: keep the chosen number
    int wavesplit = 0;      // 16 or 32: the wave-split kernel with blocks of that edge
    int stream_rows = 0;    // 16, 32 or 48: rows of W per workgroup of the skinny streaming kernel (does not force a tile)
};
ForcedPlan g_forced;

struct GemmPlan {
    bool skinny = false;
    bool a_kc = false, b_kc = false;
    int tile = kTileSmall;
    int64_t split = 1;      // >= 2: cut the reduction into this many parts of k_part steps
    int64_t k_part = 0;
    bool ragged_parts = false;   // the last part is shorter than k_part
    GemmDesc dn;   // the product with batch strides normalised
    int wavesplit_edge = 0;   // 16 or 32: the product runs on the kernel that cuts K over the waves of a workgroup
    bool forced = false;      // set by an override: the tiled kernel (or the wave-split kernel) whatever else applies
};

// Expected duration in microseconds of the wave-split kernel with T x T blocks, or a negative value outside the
// measured range; fitted to sweeps over 64..768 rows x 256..2048 columns x 64..2048 steps in the three operand
// forms.  Up to one workgroup per compute unit the time is one workgroup's: a floor of 3.9 us, then 2.5 ns per step
// with 16 x 16 blocks (3.2 ns with both operands K-contiguous, the slowest form there) and 6.4 ns with 32 x 32
// blocks.  Beyond that, every further 256 workgroups add a round that overlaps the end of the one before.
double wavesplit_estimate(const GemmDesc& d, int T) {
    const int64_t wgs = ((d.M + T - 1) / T) * ((d.N + T - 1) / T);
    const int64_t cus = compute_units();
    const double K = (double)d.K;
    if (wgs > 1024) return -1.0;
    const double more_rounds = (double)((wgs + cus - 1) / cus - 1);
    if (T == 16) {
        if (d.K > 2048) return -1.0;
        const double per_step = (d.a_ks == 1 && d.b_ks == 1) ? 3.2e-3 : 2.5e-3;
        // one row of blocks against a matrix whose rows run along the output index: a block reads 64 bytes of each
        // row, and beyond one workgroup per compute unit the rounds cost more than twice the fit (16 x 8192 x 1024:
        // 13.9 us, 16 x 11008 x 1024: 19.9; 32 x 32 blocks 9.8, the tiles 15.8)
        // (the fit holds up to 768 steps, up to 512 from two full rounds on: 16 x 8192 x 768 9.7 against 7.7 us)
        const double per_round = (d.M <= 16 && d.b_ks != 1 && (d.K > 768 || (d.K > 512 && wgs >= 2 * cus))) ? 7.5e-3 : 3.2e-3;
        return std::max(3.9, 2.9 + per_step * K) + more_rounds * per_round * K;
    }
    if (d.K > 1024) return -1.0;
    return std::max(3.9, 2.7 + 6.4e-3 * K) + 1.0e-3 * (double)std::min(wgs, cus) + more_rounds * (0.2 + 8.0e-3 * K);
}

// Number of parts for a long reduction on the 64x64 tile.  A compute unit that holds one workgroup spends
// 0.53 us per 32 reduction steps (store to LDS, barrier, read, 16 dependent MFMAs: a chain), one that holds two
// or more 0.43 us per 32 steps of any of them (the MFMA rate); the parts cost a second launch and their
// traffic (5 us + 0.5 us per part, measured).  So cutting K pays twice where it turns a partly filled round over
// the compute units into full ones or brings a second workgroup onto each (768^2 x 4096: 76 -> 59 us with 4
// parts, 1536^2 x 4096: 190 -> 158, 1024^2 x 8192: 154 -> 134), and not where the tiles already do both.
int64_t small_tile_split(int64_t tiles, int64_t K, int64_t cus) {
    int64_t best = 1;
    double best_cost = 0.0;
    for (int64_t s = 1; s <= kSplitMax; s *= 2) {
        if (s > 1 && K / s < 256) break;
        const int64_t per_cu = (tiles * s + cus - 1) / cus;
        const double cost = (double)per_cu * ((double)K / (double)s / 32.0) * (per_cu >= 2 ? 0.43 : 0.53) +
                            (s > 1 ? 5.0 + 0.5 * (double)s : 0.0);
        if (s == 1 || cost < 0.97 * best_cost) {
            best = s;
            best_cost = cost;
        }
    }
    return best;
}

// Expected duration in microseconds of a single product on `tile` (small, wide or medium) with the reduction cut
// into `parts` parts of `k_len` steps, fitted to sweeps of 380 whole-tile and 75 ragged shapes (M 40..3000, N and K
// 250..11008, the three operand forms, every tile and part count; the choice made from it is within 1 % of the
// best measured one on average, 8 % at worst).  A workgroup takes a fixed time per 32 reduction steps whatever
// shares its compute unit -- small 0.48 us with both operands K-contiguous, else 0.57 / 0.54 / 0.52 with one / two /
// three workgroups per unit and 0.49 with more (the simple schedule), wide 0.95, medium 1.8 (two resident at
// most); edge tiles cost a twentieth more (not on the small tile with two K-contiguous operands) -- so the kernel takes
// rounds x steps x that, plus 3.5 us of launch, first loads and epilogue; the parts cost a second launch
// (3.5 us + 0.1 per part) and their traffic (each part written and read once, at about 6 TB/s).
double tiled_cost(int tile, bool both_kc, bool whole, int64_t M, int64_t N, int64_t k_len, int64_t parts, int64_t cus) {
    bool pipelined = true;
    const int64_t bm = tile == kTileMedium ? 128 : 64, bn = tile == kTileSmall ? 64 : 128;
    const int64_t groups = ((M + bm - 1) / bm) * ((N + bn - 1) / bn) * parts;
    const int64_t per_cu = (groups + cus - 1) / cus;
    const double steps = (double)k_len / 32.0;
    double t;
    if (tile == kTileMedium) {
        const double one = (both_kc ? 1.79 : 1.86) * (whole ? 1.0 : 1.05);
        t = per_cu == 1 ? steps * one : steps * 1.02 * one * (double)(2 * (per_cu / 2)) + steps * one * (double)(per_cu % 2);
    } else if (tile == kTileWide) {
        t = (double)per_cu * steps * (both_kc ? 0.95 : 0.96) * (whole ? 1.0 : 1.05);
    } else if (whole && per_cu >= 4 && !both_kc) {
        pipelined = false;   // the simple schedule
        t = (double)per_cu * steps * 0.49;
    } else {
        // (the surcharge for edge tiles applies to the forms with an operand that is not K-contiguous only: the
        // sweeps this was fitted to were run with exactly this expression, and with both operands K-contiguous the
        // edge variant's range-checked loads measured like the whole-tile ones)
        // (16 rounds and more of edge-checked tiles with both operands K-contiguous measured 0.52 .. 0.57: 5000^3 2020 us
        // where the 64 x 128 tile takes 1889, 7000 x 3000 x 3000 1057 against 990, 5000 x 5000 x 1000 445 against 418)
        const double c = both_kc ? (!whole && per_cu >= 16 ? 0.52 : 0.48)
                                 : (per_cu == 1 ? 0.57 : per_cu == 2 ? 0.54 : 0.52) * (whole ? 1.0 : 1.05);
        t = (double)per_cu * steps * c;
    }
    // the pipelined kernels run the steps after the last whole tile of 32 as a tile of their own, loaded, masked
    // and multiplied with nothing else in flight
    if (pipelined && k_len % 32 != 0) t += 1.5 * (double)per_cu;
    return t + 3.5 + (parts > 1 ? 3.5 + 0.1 * (double)parts + (double)(2 * parts + 1) * (double)(M * N) * 4.0 / 6.0e6 : 0.0);
}

GemmPlan plan_gemm(const GemmDesc& d) {
    GemmPlan plan;
    // skinny: y = x . w^T with both operands K-contiguous, a contiguous output row, no scaling
    plan.skinny = d.M <= kSkinnyMaxRows && d.nbatch == 1 && d.a_ks == 1 && d.b_ks == 1 && d.c_cs == 1 &&
                  !d.has_alpha && d.K > 0 && d.N >= 256;
    // 5..16 rows against few and long rows that the streaming kernel walks in its rolled loop (K > 8192, not a multiple
    // of 4096; up to four rows of W per compute unit): its 64 workgroups stream 11008 steps each, and the 64 x 64 tiles
    // with 16 parts of K are faster (1024 x 11008 with W from HBM, 5 / 8 / 12 / 16 rows: 21.9 / 24.0 / 27.6 / 30.1 us ->
    // 20.5 .. 21.0; 256 x 13824 at 5 rows 24.5 -> 19.5; rows of 8192 steps: 13.0 / 14.6 / 15.9 against 17)
    if (plan.skinny && d.M >= 5 && d.N <= 4 * compute_units() && d.K > 8192 && d.K % 4096 != 0) plan.skinny = false;
    // 5..16 rows against long rows of W that do not start on 128-byte lines (the streaming kernel's 128-byte pieces
    // straddle two lines each): the tiles from 8192 steps on (4100 x 11012 at 8 / 16 rows 62.2 / 78.4 us against 46.4 at
    // 17 rows; 4100 x 8200 45.6 / 55.1 against 33.7; at 5004 steps and fewer the streaming kernel holds up to 12 rows)
    // (8..16 rows from 5000 steps on: 8200 x 5004 at 8 / 16 rows 52.8 / 64.3 against 46.5; 13..16 rows from 4096 steps
    // on: 5000 x 4100 at 16 rows 38.3 against 32.2)
    if (plan.skinny && d.M >= 5 && d.b_rs % 32 != 0 &&
        (d.K >= 8192 || (d.M >= 8 && d.K > 4608) || (d.M >= 13 && d.K >= 4096)))
        plan.skinny = false;
    // 5..16 rows against many short rows (50257 x 768: 43 / 55 us at 8 / 16 rows on the streaming kernel, whose 3142
    // workgroups of 48 KB are all prologue and epilogue; 29 us on the tiles at 17 rows)
    // (9..16 rows up to 1536 steps: 16 x 50257 x 1280 60.2 against 45.2, 16 x 20000 x 1536 32.5 against 24.7, matrices
    // of up to 257 MB multiplied again and again; at 2048 steps the streaming kernel wins from 400 MB on and loses 20 % at 262)
    if (plan.skinny && d.N >= 64 * compute_units() && ((d.M >= 5 && d.K <= 1024) || (d.M >= 9 && d.K <= 1536))) plan.skinny = false;
    // 17..32 rows where the streaming kernel's two-block variant applies (whole tiles, K a multiple of 4096, enough
    // columns for one workgroup per compute unit, a matrix of at most 192 MB): W streams once in one launch
    // (4096 x 4096 from HBM: 17 rows 21.2 -> 15.0 us, 32 rows 21.3 -> 17.9, on a row of 32 x 128 tiles with eight
    // parts of K and their second launch before)
    if (!plan.skinny && d.M > kSkinnyMaxRows && d.M <= 4 * kSkinnyMaxRows && d.nbatch == 1 && d.a_ks == 1 && d.b_ks == 1 &&
        d.c_cs == 1 && !d.has_alpha && d.rowsum == nullptr) {
        SkinnyParams sp{};
        sp.W = d.B; sp.X = d.A; sp.ldw = d.b_rs; sp.ldx = d.a_rs; sp.N = d.N; sp.M = (int)d.M; sp.K = (int)d.K;
        plan.skinny = skinny_stream32_applies(sp);
    }
    // batch strides that are never multiplied by a non-zero index must not spoil the alignment checks
    GemmDesc& dn = plan.dn;
    dn = d;
    if (dn.bdiv <= 1) { dn.bdiv = 1; dn.a_bs1 = dn.b_bs1 = dn.c_bs1 = 0; }
    if (dn.nbatch <= dn.bdiv) dn.a_bs0 = dn.b_bs0 = dn.c_bs0 = 0;
    plan.a_kc = operand_is_kc(dn.a_rs, dn.a_ks);
    plan.b_kc = operand_is_kc(dn.b_rs, dn.b_ks);

    // Largest tile that still yields about one workgroup per compute unit and is not mostly padding.  Between
    // the two big tiles the number of rounds decides: both run at the same rate per compute unit (measured:
    // 149 TFLOP/s either way at 8192^3), a compute unit works through its 256x256 tiles one at a time and
    // through 128x128 tiles at a quarter of that each (two resident ones share its rate), so the last, partly
    // filled round costs four times less with the medium tile (4100^3: 1.85 ms against 1.19 ms).  On a tie the
    // large tile wins: it moves half as much through LDS per flop (8000^3: 7.1 against 7.5 ms).
    const int64_t short_side = d.M < d.N ? d.M : d.N;
    const int64_t cus = compute_units();
    // bytes of partial sums this product may use: the library scratch grows up to kSplitScratchMax, a caller's
    // fixed buffer (the allocation-free entry point) may be smaller, and the part count is then chosen to fit it
    const int64_t scratch_cap = d.scratch ? std::min(kSplitScratchMax, d.scratch_bytes) : kSplitScratchMax;
    const int64_t t256 = tiles_of(d.M, d.N, d.nbatch, 256), t128 = tiles_of(d.M, d.N, d.nbatch, 128);
    // A single round of them must also be well filled, padding counted: 196 .. 210 tiles on 256 units lost 8 .. 15 % to
    // the smaller tiles (3584^3 796 us against 693 on 64 x 64 tiles, 3600 x 3400 x 4096 912 against 814, 3200 x 4000 x
    // 2500 564 against 522: M N / (65536 units) = 0.73 .. 0.77), 3840 x 3700 x 2048 1 .. 6 % at 0.85; from 0.88 on
    // (3840^3, 3712 x 3968 x 3000, 4000^2) the large tile is the fastest.  Two rounds and more only get here with
    // fills of 0.875 and more.
    const int64_t rounds256 = (t256 + cus - 1) / cus;
    const bool fills256 = rounds256 > 1 || d.nbatch > 1 || 100 * d.M * d.N >= 86 * 65536 * cus;
    if (short_side > 128 && t256 >= (3 * cus) / 4 && 4 * rounds256 <= (t128 + cus - 1) / cus && fills256)
        plan.tile = kTileLarge;
    else if (short_side > 64 && t128 >= cus / 2) {
        // The same count between the 128- and the 64-wide tile, which runs at about 0.88 of the medium tile's
        // rate per compute unit (2048^3: 134 against 123 us): the small tile wins where its finer grain saves
        // a round (1024x2048x512, 128 medium tiles on 256 units: 36 -> 24 us; 1536^3 91 -> 77; 3000^3 540 -> 485).
        const int64_t t64 = tiles_of(d.M, d.N, d.nbatch, 64);
        const int64_t rounds_m = (t128 + cus - 1) / cus, rounds_s = (t64 + cus - 1) / cus;
        if (100 * rounds_s >= 340 * rounds_m) plan.tile = kTileMedium;
    }
    // 17..32 rows against at least 256 columns: a 64-row tile would spend half of its MFMAs on padding, and these
    // products are bound by the stream of the other operand (32 x 4096 x 4096: 30.6 -> 21.5 us).  65..96 rows
    // likewise: three row tiles of 32 instead of two of 64 (96 x 4096 x 4096: 55 -> 43 us; 144 rows: 67 against 73)
    // One row of them needs enough column tiles: while the 64 x 64 tile's column tiles with the most parts of K (16)
    // still find a compute unit each (1024 columns at 256 units), that tile is the faster one although half of its
    // MFMAs multiply padding -- the flat row has half as many workgroups (17 x 1024 x 11008: 23.4 -> 20.0 us with the
    // matrix in the last-level cache, 31 -> 21 from HBM; 32 x 256 x 8192 17.0 -> 14.7; 32 x 1024 x 4096 13.0 -> 12.1);
    // beyond that it has to take fewer parts and the flat row wins (17 x 1280 x 8192: 15.8 against 21.5).
    const bool flat_row_fills = d.M > 32 || ((d.N + 63) / 64) * kSplitMax > cus || d.K < kSplitFromK;
    if (plan.tile == kTileSmall && (d.M <= 32 || (d.M > 64 && d.M <= 96)) && d.N >= 256 && flat_row_fills) plan.tile = kTileFlat;

    // Small products: one launch of the wave-split kernel where it is expected to finish before the tiled
    // kernel (plus, for long K, its second launch) could: measured, it wins wherever its estimate stays below
    // ~12.5 us (64x512x784 9.8 -> 4.9 us, 256x1024x1024 14.3 -> 11.0, its backward_x form 14.3 -> 12.4,
    // 300^3 11.1 -> 4.9), and against the skinny kernels for 5..16 rows below ~7 us (16x1024x1024 7.8 -> 5.9).
    // (and where the cost model below expects no less of the tiled kernels: 1000 x 333 x 777 19.4 -> 14.6 us,
    // 512 x 1024 x 256 11.6 -> 7.0)
    int ws_edge = 0;
    double ws_cost = 0.0;
    if (wavesplit_applies(dn)) {
        const double e16 = wavesplit_estimate(dn, 16), e32 = wavesplit_estimate(dn, 32);
        const bool take16 = e16 > 0 && (e32 < 0 || e16 <= e32);
        const double best = take16 ? e16 : e32;
        const double limit = plan.skinny ? (d.M <= 4 ? 0.0 : 7.0) : 12.5;
        if (best > 0 && best <= limit) {
            ws_edge = take16 ? 16 : 32;
            ws_cost = best;
        }
    }

    // A single product of more than 32 rows whose operands the pipelined kernels can load (unit strides): tile and
    // number of parts together, from the model above.  Everything else keeps the rules above and below.
    bool modelled = false;
    // (The 32 x 128 tile keeps 65..96 rows where it wastes nothing or both operands are K-contiguous: 96 x 4096 x 4096
    // 36 us against 37-39 with the tiles below, but 72 x 4096 x 11008 with a [K, N] matrix 101 -> 90.)
    const bool keep_flat = plan.tile == kTileFlat && (d.M <= 32 || d.M % 32 == 0 || (plan.a_kc && plan.b_kc));
    double tiles_cost = 0.0;
    if (!plan.skinny && d.nbatch == 1 && plan.tile != kTileLarge && !keep_flat && d.M > 32 &&
        d.N >= 64 && d.K >= 32 && !skinny_rows_applies(dn) && !shortk_nt_applies(dn)) {
        const GemmParams pp = make_params(dn, plan.a_kc, plan.b_kc);
        const bool both_kc = plan.a_kc && plan.b_kc;
        const bool vec = pp.a_vec && pp.b_vec && fits_buffer_offsets(pp, plan.a_kc, plan.b_kc, 128, 128);
        if (vec || fits_ragged_pipe(pp, plan.a_kc, plan.b_kc, 128, 128)) {
            double best = 0.0;
            for (const int tile : {(int)kTileMedium, (int)kTileWide, (int)kTileSmall}) {   // on a tie the larger tile
                const int64_t bm = tile == kTileMedium ? 128 : 64, bn = tile == kTileSmall ? 64 : 128;
                if (d.M <= bm / 2 || d.N <= bn / 2) continue;   // more than half of a lone tile would be padding
                for (int64_t sp = 1; sp <= kSplitMax; sp++) {
                    int64_t k_len = d.K;
                    bool equal = true;
                    if (sp > 1) {
                        if (d.K < kSplitFromK || sp * d.M * d.N * (int64_t)sizeof(float) > scratch_cap) break;
                        equal = d.K % (16 * sp) == 0;
                        k_len = equal ? d.K / sp : ((d.K + sp - 1) / sp + 15) / 16 * 16;
                        // parts of at least 256 steps, 512 for the larger tiles (their first tile takes longer to arrive)
                        if (k_len < (tile == kTileSmall ? 256 : 512)) break;
                        if ((d.K + k_len - 1) / k_len != sp) continue;   // this part length needs fewer parts
                    }
                    const bool whole = vec && equal && d.M % bm == 0 && d.N % bn == 0 && k_len % 32 == 0;
                    if (!whole && !fits_ragged_pipe(pp, plan.a_kc, plan.b_kc, (int)bm, (int)bn)) continue;
                    const double c = tiled_cost(tile, both_kc, whole, d.M, d.N, k_len, sp, cus);
                    if (!modelled || c < 0.98 * best) {
                        modelled = true;
                        best = tiles_cost = c;
                        plan.tile = tile;
                        plan.split = sp;
                        plan.k_part = sp > 1 ? k_len : 0;
                        plan.ragged_parts = !equal;
                    }
                }
            }
        }
    }

    // 129..160 rows: five rows of 32 x 128 tiles compute 160 rows where three rows of 64-row tiles compute 192.
    // A workgroup takes 0.44 us per 32 steps (0.47 alone on its compute unit), launch and parts as above: within
    // 4 % of the measured times at 130..160 rows against 2048..8192 columns wherever the workgroups fill their
    // rounds (see below), 10 % low at 8192 x 8192, where the five row blocks re-read the other operand from
    // beyond L2.  Taken where that is 7 % below the other tiles' estimate: over 57 shapes in the three operand
    // forms 1.05 x on average (144 x 4096 x 4096 53.4 -> 49.5 us, 144 x 3072 x 4096 44.8 -> 39, 144 x 6144 x 4096
    // 85 -> 70, 144 x 8192 x 4096 96 -> 88, 160 x 4096 x 11008 130 -> 123; ties at 2560 x 2560 and 1024 x 4096).
    // Reductions of 1024 steps lost (4096 x 1024: 19.3 -> 21; 2047 steps measure like 2048: 144 x 2048 x 2047 23.3 -> 20.9
    // in the audit of these rules, bench.py --plan-audit, so the bound sits a little below 2048) and 11008 columns measured between 9 % slower
    // and 8 % faster: both stay with the other tiles.  193..224 rows likewise, seven rows of tiles against four
    // (200 x 3072 x 4096 56 -> 50 us, 224 x 4608 x 4608 91 -> 77, 200 x 3072 x 3072 42 -> 39; 50 shapes x 3 forms
    // 1.04-1.05 x on average, nothing slower than measurement noise).
    if (modelled && ((d.M > 128 && d.M <= 160) || (d.M > 192 && d.M <= 224)) && d.N >= 1024 && d.N <= 8192 && d.K >= 2000 && d.N * d.K <= (1ll << 26)) {
        const GemmParams pp = make_params(dn, plan.a_kc, plan.b_kc);
        if (fits_ragged_pipe(pp, plan.a_kc, plan.b_kc, 32, 128)) {
            const int64_t tiles = ((d.M + 31) / 32) * ((d.N + 127) / 128);
            double flat_best = 0.0;
            int64_t flat_split = 0, flat_len = 0;
            for (int64_t sp = 1; sp <= kSplitMax; sp++) {
                int64_t k_len = d.K;
                if (sp > 1) {
                    if (d.K < kSplitFromK || sp * d.M * d.N * (int64_t)sizeof(float) > scratch_cap) break;
                    k_len = d.K % (16 * sp) == 0 ? d.K / sp : ((d.K + sp - 1) / sp + 15) / 16 * 16;
                    if (k_len < 256) break;
                    if ((d.K + k_len - 1) / k_len != sp) continue;
                }
                const int64_t per_cu = (tiles * sp + cus - 1) / cus;
                // measured against the other tiles: one workgroup per compute unit +15..22 %, two 0..+13 %, where
                // they cover at least 85 % of the units (200 of 256: -3 %, 390 and 420 of 512: -7 %); whole rounds
                // beyond (1280 workgroups: five per unit) +5..10 %, partly filled ones -16..+10 %, fourteen rounds
                // of 16 parts -8 %
                const int64_t wgs = tiles * sp;
                // (seven row tiles against four of 64 rows save an eighth, not a sixth: 448 workgroups of 512 lost
                // 3..7 % there, 504 and 252 gained 6..20 %)
                const int64_t min_fill = d.M <= 160 ? 85 : 95;
                if (wgs > 2 * cus ? wgs % cus != 0 || wgs > 6 * cus : 100 * wgs < min_fill * per_cu * cus) continue;
                // three workgroups fit a compute unit (45 KB of LDS each); a last round of one per unit lands
                // three to a unit on a third of the chip and costs a round of two (980 workgroups of 16 steps:
                // 37.6 us in the loop where 4 x 16 x 0.44 = 28 were expected; 1280: 35, as expected)
                const int64_t rounds = per_cu + (per_cu > 3 && per_cu % 3 == 1 ? 1 : 0);
                double c = (double)rounds * ((double)k_len / 32.0) * (per_cu == 1 ? 0.47 : 0.44) *
                           (plan.a_kc && plan.b_kc ? 1.0 : 1.02);
                if (k_len % 32 != 0) c += 1.5 * (double)per_cu;
                c += 3.5 + (sp > 1 ? 3.5 + 0.1 * (double)sp + (double)(2 * sp + 1) * (double)(d.M * d.N) * 4.0 / 6.0e6 : 0.0);
                if (flat_split == 0 || c < 0.98 * flat_best) {
                    flat_best = c;
                    flat_split = sp;
                    flat_len = k_len;
                }
            }
            if (flat_split > 0 && flat_best < 0.93 * tiles_cost) {
                tiles_cost = flat_best;
                plan.tile = kTileFlat;
                plan.split = flat_split;
                plan.k_part = flat_split > 1 ? flat_len : 0;
                plan.ragged_parts = flat_split > 1 && d.K % (16 * flat_split) != 0;
            }
        }
    }

    // (over 840 shapes x forms the choice between the two estimates is within a tenth of the faster kernel in all
    // but eleven cases, 1.45 x at worst)
    if (ws_edge && !(modelled && tiles_cost < 0.95 * ws_cost)) {
        plan.wavesplit_edge = ws_edge;
        modelled = false;
        plan.split = 1;
        plan.k_part = 0;
        plan.ragged_parts = false;
    }

    // Split-K: a single product whose output tiles leave most compute units idle is cut along K
    // into `split` equal parts that run as the batch dimension of the same kernel and write raw
    // partial products to the library's scratch; a second launch sums them in a fixed order and
    // applies the epilogue.
    if (!modelled && !plan.skinny && d.nbatch == 1 && d.K >= kSplitFromK) {
        const int64_t edge = plan.tile == kTileLarge ? 256 : plan.tile == kTileMedium ? 128 : 64;
        const int64_t tiles = plan.tile == kTileFlat ? ((d.M + 31) / 32) * ((d.N + 127) / 128) : tiles_of(d.M, d.N, 1, edge);
        int64_t split = compute_units() / tiles;
        // one row of 32 x 128 tiles is bound by the stream of the other operand from HBM: one workgroup per compute
        // unit, as split = units / tiles says, measured best or within 8 % of it at 4096 ... 16384 columns and steps
        // (32 x 8192 x 8192: 94 us with the model's 8 parts, 68 with 4); the model below is for the products that
        // the matrix cores bound
        // (the same for the 64 x 64 tile where it stands in for that row because the row's column tiles are too few)
        const bool one_flat_row = d.M <= 32 && (plan.tile == kTileFlat || (plan.tile == kTileSmall && d.N >= 256));
        if ((plan.tile == kTileSmall || plan.tile == kTileFlat) && d.K >= 1024 && !one_flat_row)
            split = small_tile_split(tiles, d.K, cus);
        while (split > 1 && split * d.M * d.N * (int64_t)sizeof(float) > scratch_cap) split /= 2;
        if (split > d.K / kSplitMinK) split = d.K / kSplitMinK;
        if (split > kSplitMax) split = kSplitMax;
        // equal parts of whole 16-step tiles if some part count allows it; else parts of whole tiles with a
        // shorter last one, which the general kernel variant handles
        int64_t whole = split;
        while (whole >= 2 && d.K % (whole * 16) != 0) whole--;
        if (whole >= 2) {
            plan.split = whole;
            plan.k_part = d.K / whole;
            plan.ragged_parts = false;
        } else if (split >= 2) {
            const int64_t per = ((d.K + split - 1) / split + 15) / 16 * 16;
            plan.split = (d.K + per - 1) / per;
            plan.k_part = per;
            plan.ragged_parts = true;
            if (plan.split < 2) plan.split = 1;
        }
    }
    if (g_forced.active && d.nbatch == 1 && d.rowsum == nullptr) {
        if (g_forced.wavesplit) {
            if (wavesplit_applies(dn) && wavesplit_estimate(dn, g_forced.wavesplit) > 0) {
                plan.forced = true;
                plan.skinny = false;
                plan.wavesplit_edge = g_forced.wavesplit;
                plan.split = 1; plan.k_part = 0; plan.ragged_parts = false;
            }
        } else {
            plan.forced = true;
            plan.skinny = false;
            plan.wavesplit_edge = 0;
            if (g_forced.tile >= 0) plan.tile = g_forced.tile;
            if (g_forced.split >= 1) {
                // the parts as the model above cuts them: equal where 16-step tiles allow it, else whole tiles with a
                // shorter last part; a part count that the length does not give, or whose sums exceed the scratch,
                // leaves one part
                const int64_t sp = g_forced.split;
                plan.split = 1; plan.k_part = 0; plan.ragged_parts = false;
                if (sp >= 2 && sp <= kSplitMax && d.K >= 32 * sp && sp * d.M * d.N * (int64_t)sizeof(float) <= scratch_cap) {
                    const bool equal = d.K % (16 * sp) == 0;
                    const int64_t k_len = equal ? d.K / sp : ((d.K + sp - 1) / sp + 15) / 16 * 16;
                    if ((d.K + k_len - 1) / k_len == sp) {
                        plan.split = sp;
                        plan.k_part = k_len;
                        plan.ragged_parts = !equal;
                    }
                }
            }
        }
    }
    return plan;
}

bool valid_dims(const GemmDesc& d) {
    return d.M >= 0 && d.N >= 0 && d.K >= 0 && d.nbatch >= 0 && d.M <= kMaxDim && d.N <= kMaxDim && d.K <= kMaxDim;
}

}  // namespace

// "auto" (or empty) clears the override; otherwise words: a tile name (large, medium, small, flat, wide), and / or
// "split N" (1 .. 16), or "wavesplit 16" / "wavesplit 32"; "stream 16" / "stream 32" / "stream 48" only sets the rows
// of W per workgroup of the skinny streaming kernel for the products that kernel takes anyway.
int set_forced_gemm_plan(const char* text) {
    ForcedPlan f;
    std::string t = text ? text : "";
    size_t pos = 0;
    auto next = [&]() -> std::string {
        while (pos < t.size() && t[pos] == ' ') pos++;
        const size_t b = pos;
        while (pos < t.size() && t[pos] != ' ') pos++;
        return t.substr(b, pos - b);
    };
    static const char* const tiles[] = {"large", "medium", "small", "flat", "wide"};
    for (std::string w = next(); !w.empty(); w = next()) {
        if (w == "auto") continue;
        bool known = false;
        for (int i = 0; i < 5; i++)
            if (w == tiles[i]) { f.tile = i; f.active = known = true; }
        if (w == "split" || w == "wavesplit" || w == "stream") {
            const std::string n = next();
            const long v = n.empty() ? -1 : strtol(n.c_str(), nullptr, 10);
            if (w == "split" && v >= 1 && v <= kSplitMax) { f.split = v; f.active = known = true; }
            if (w == "wavesplit" && (v == 16 || v == 32)) { f.wavesplit = (int)v; f.active = known = true; }
            if (w == "stream" && (v == 16 || v == 32 || v == 48)) { f.stream_rows = (int)v; known = true; }
        }
        if (!known) return fail(KAI_ERR_INVALID_ARGUMENT, "gemm plan override: cannot read \"" + w + "\"");
    }
    g_forced = f;
    set_skinny_stream_rows_override(f.stream_rows);
    return KAI_OK;
}

bool gemm_fuses_rowsum(const GemmDesc& d) {
    if (!valid_dims(d) || d.M == 0 || d.N == 0 || d.K == 0 || d.nbatch != 1) return false;
    // The row sums ride along where the product is short: they save a launch of 3 us.  A long product pays for them
    // in every tile of its first tile column and loses more than that (gw of 11008 x 4096 at a batch of 1024: 1445 us
    // with the sums riding along against 1289 with colsum_kernel on its own; 4096 x 1024 at 512: 92.2 against 85.2;
    // at a batch of 64: 29.1 against 29.6).
    if (d.K >= 64 && d.M * d.N * d.K > (1ll << 28)) return false;
    const GemmPlan plan = plan_gemm(d);
    return !plan.skinny && !plan.wavesplit_edge && !skinny_rows_applies(plan.dn) && !plan.a_kc && !plan.b_kc && plan.tile != kTileLarge &&
           plan.tile != kTileFlat && plan.tile != kTileWide && plan.split == 1;
}

// What launch_gemm would do with this product, as text: the kernel family and, for the tiled kernel, tile,
// variant and the number of parts K is cut into.  Host arithmetic only, nothing is launched or allocated.
std::string describe_gemm(const GemmDesc& d) {
    if (!valid_dims(d)) return "invalid";
    if (d.M == 0 || d.N == 0 || d.nbatch == 0) return "nothing";
    const GemmPlan plan = plan_gemm(d);
    if (plan.wavesplit_edge) return "wavesplit " + std::to_string(plan.wavesplit_edge);
    if (!plan.forced) {
        if (skinny_rows_applies(plan.dn)) return "skinny rows";
        if (plan.skinny) {
            // the streaming kernel with workgroups of 32 or 48 rows of W says so
            SkinnyParams sp{};
            sp.W = d.B; sp.X = d.A; sp.ldw = d.b_rs; sp.ldx = d.a_rs; sp.N = d.N; sp.M = (int)d.M; sp.K = (int)d.K;
            const int wide = skinny_stream_wide_rows(sp);
            return wide ? "skinny stream " + std::to_string(wide) : "skinny";
        }
        if (shortk_nt_applies(plan.dn)) return "shortk_nt";
        if (shortk_heads_applies(plan.dn)) return "shortk_heads";
        if (heads_pv_applies(d)) return "heads_pv";
    }
    const bool a_kc = plan.a_kc, b_kc = plan.b_kc;
    GemmDesc dt = plan.dn;
    if (plan.split >= 2) {
        if (plan.ragged_parts) dt.k_part = plan.k_part;
        else dt.K = plan.k_part;
        dt.nbatch = plan.split; dt.bdiv = 1;
        dt.a_bs0 = plan.k_part * d.a_ks; dt.b_bs0 = plan.k_part * d.b_ks; dt.c_bs0 = d.M * d.N;
        dt.a_bs1 = dt.b_bs1 = dt.c_bs1 = 0;
        dt.c_rs = d.N; dt.c_cs = 1;
    }
    const GemmParams p = make_params(dt, a_kc, b_kc);
    const GemmVariant v = pick_gemm_variant(p, a_kc, b_kc, dt.nbatch > 0 ? dt.nbatch : 1, plan.tile);
    static const char* const tiles[] = {"large", "medium", "small", "flat", "wide"};
    static const char* const kinds[] = {"general", "whole", "whole pipelined", "ragged pipelined"};
    std::string text = std::string("mfma ") + tiles[v.tile] + " " + kinds[v.kind];
    if ((v.kind == kKindWholePipelined || v.kind == kKindRaggedPipelined) && v.depth > 1)
        text += " staged " + std::to_string(v.depth);
    return text + " split " + std::to_string(plan.split);
}

int launch_gemm(const GemmDesc& d, hipStream_t stream) {
    if (d.M < 0 || d.N < 0 || d.K < 0 || d.nbatch < 0)
        return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: negative dimension");
    if (d.M > kMaxDim || d.N > kMaxDim || d.K > kMaxDim)
        return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: dimension does not fit 31 bits");
    if (d.M == 0 || d.N == 0 || d.nbatch == 0) return KAI_OK;
    if (!d.C || (d.K > 0 && (!d.A || !d.B))) return fail(KAI_ERR_INVALID_POINTER, "gemm: null operand");

    const GemmPlan plan = plan_gemm(d);
    if (d.rowsum && !gemm_fuses_rowsum(d))
        return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: this product cannot carry the fused row sum");

    if (plan.wavesplit_edge) return launch_gemm_wavesplit(plan.dn, plan.wavesplit_edge, stream);
    if (!plan.forced && skinny_rows_applies(plan.dn)) return launch_skinny_rows(plan.dn, stream);
    if (plan.skinny) {
        SkinnyParams s{};
        s.W = d.B; s.X = d.A; s.Y = d.C; s.Y2 = d.C2; s.bias = d.bias; s.leaky = d.leaky;
        s.ldw = d.b_rs; s.ldx = d.a_rs; s.ldy = d.c_rs;
        s.N = d.N; s.M = (int)d.M; s.K = (int)d.K;
        s.act = d.act; s.accflag = d.acc;
        return launch_skinny_nt(s, stream);
    }

    const bool a_kc = plan.a_kc, b_kc = plan.b_kc;
    if (!plan.forced) {
        if (shortk_nt_applies(plan.dn)) return launch_gemm_shortk_nt(make_params(plan.dn, true, true), d.nbatch, stream);
        if (shortk_heads_applies(plan.dn))
            return launch_gemm_shortk_heads(make_params(plan.dn, true, true), d.nbatch, stream);
        if (heads_pv_applies(d)) return launch_heads_pv(d, stream);
    }
    if (plan.split >= 2) {
        const int64_t split = plan.split;
        float* part = d.scratch;
        const int64_t part_bytes = split * d.M * d.N * (int64_t)sizeof(float);
        if (part == nullptr) KAI_TRY(workspace(part_bytes, &part));
        else if (part_bytes > d.scratch_bytes)
            return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: this product cuts its reduction into " + std::to_string(split) +
                        " parts and needs " + std::to_string(part_bytes) + " bytes for their sums; the caller's scratch holds " +
                        std::to_string(d.scratch_bytes));
        GemmDesc ds = plan.dn;
        ds.scratch = nullptr; ds.scratch_bytes = 0;
        if (plan.ragged_parts) ds.k_part = plan.k_part;   // K stays the whole length
        else ds.K = plan.k_part;
        ds.nbatch = split; ds.bdiv = 1;
        ds.a_bs0 = plan.k_part * d.a_ks; ds.b_bs0 = plan.k_part * d.b_ks; ds.c_bs0 = d.M * d.N;
        ds.a_bs1 = ds.b_bs1 = ds.c_bs1 = 0;
        ds.C = part; ds.c_rs = d.N; ds.c_cs = 1;
        ds.C2 = nullptr; ds.bias = nullptr; ds.alpha = nullptr; ds.leaky = nullptr;
        ds.act = 0; ds.acc = 0; ds.has_alpha = 0;
        KAI_TRY(launch_layout(make_params(ds, a_kc, b_kc), a_kc, b_kc, split, plan.tile, stream));
        SplitReduceParams r{};
        r.part = part; r.C = d.C; r.C2 = d.C2; r.bias = d.bias; r.alpha = d.alpha; r.leaky = d.leaky;
        r.M = d.M; r.N = d.N; r.c_rs = d.c_rs; r.c_cs = d.c_cs;
        r.nsplit = (int)split; r.act = d.act; r.accflag = d.acc; r.has_alpha = d.has_alpha;
        return launch_splitk_reduce(r, stream);
    }
    return launch_layout(make_params(plan.dn, a_kc, b_kc), a_kc, b_kc, d.nbatch, plan.tile, stream);
}

}  // namespace kai
