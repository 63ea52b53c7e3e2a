// Backward of a dense layer in one launch (plus the sum of the parts of a reduction that was cut):
//     ga = gy * f'(pre)            f = none / relu / leaky relu, applied while the tiles are loaded
//     gx[ndat,xvec] = ga . w       (VMath::matmul_backward_x, vmath.cu:3007-3047 of the reference)
//     gw[yvec,xvec] = ga^T . x     (VMath::matmul_backward_w, vmath.cu:3051-3093)
//     gb[yvec]      = colsum(ga)   (VMath::add_bias_backward_b, vmath.cu:901-932)
// i.e. the calls VTensor::activate_backprop, add_backprop and matmul_backprop issue one after the other
// (api_objects/vtensor.cpp:5697-5718, 3470-3479, 1337-1375).
//
// At the sizes of a layer's mini-batch step (a few hundred rows, widths around a thousand) each of the two
// products is a few hundred 64 x 64 tiles with a short reduction: alone, neither fills the compute units, and
// most of a launch is latency.  Here ONE grid holds the workgroups of both products and of the bias gradient:
// the first blocks_x workgroups compute gx (its reduction over yvec cut into parts so that a part is about as
// long as the reduction of gw), the next compute gw, the last few sum the columns of ga (one thread per column,
// rows ascending: the order of a sequential loop).  Workgroups are dealt out in id order, so the compute units
// hold workgroups of both products side by side.  Both products run the pipelined tile loop of gemm_mfma.h (64 rows
// x 64 or 128 columns, four waves, 32 reduction steps per tile) with the masked A operand; they share one LDS
// allocation.
#include <algorithm>
#include <string>

#include "elementwise.h"
#include "gemm_host.h"

namespace kai {

namespace {

constexpr int kPairTile = 64, kPairBK = 32;
// The tiles are 64 rows x BN columns of gx or gw (BN = 128 where xvec allows: a third less to load per flop).
template <int BN>
struct PairTiles {
    using Ax = TileShape<true, kPairTile, kPairBK>;    // gx: A = gy, reduction index contiguous
    using Bx = TileShape<false, BN, kPairBK>;          //     B = w, output index contiguous
    using Aw = TileShape<false, kPairTile, kPairBK>;   // gw: A = gy^T, B = x, both output index contiguous
    using Bw = TileShape<false, BN, kPairBK>;
    static constexpr int kLdsX = 2 * (Ax::kFloats + Bx::kFloats), kLdsW = 2 * (Aw::kFloats + Bw::kFloats);
    static constexpr int kLds = kLdsX > kLdsW ? kLdsX : kLdsW;
};

// The bias gradient of 64 columns: gb[c] (=|+=) sum over the rows of gy[m,c] * f'(pre[m,c]), rows ascending (the
// order of the reference's sequential loop, so the sum is bit-identical to it).  All 256 threads fetch blocks of
// 128 rows (one coalesced 256-byte row per wave and load, the next block requested before this one is summed)
// and put the masked values into LDS; the first wave adds them up, one thread per column.  Products and sums are
// rounded separately.
constexpr int kColsumRows = 128;
__device__ __forceinline__ void masked_colsum_64(const GemmParams& pw, int col0, float* lds) {
#pragma clang fp contract(off)
    const int tid = threadIdx.x;
    const int c = tid & 63, r0 = tid >> 6;           // this thread loads rows r0, r0 + 4, ... of a block
    const int ndat = pw.K, yvec = pw.M;              // the gw product reduces over the rows of gy
    const bool masked = pw.a_mask != 0;
    const float* gy = pw.A + col0 + c;
    const float* pre = (masked ? pw.A2 : pw.A) + col0 + c;
    const float slope = (pw.a_mask == 2 && pw.leaky) ? *pw.leaky : 0.f;
    constexpr int PER = kColsumRows / 4;
    float g[PER], x[PER];
    auto fetch = [&](int m0) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int m = min(m0 + r0 + 4 * i, ndat - 1);   // rows past the end repeat the last one and are not summed
            g[i] = gy[(int64_t)m * yvec];
            x[i] = pre[(int64_t)m * yvec];
        }
    };
    float s = 0.f;
    fetch(0);
    for (int m0 = 0; m0 < ndat; m0 += kColsumRows) {
#pragma unroll
        for (int i = 0; i < PER; i++)
            lds[(r0 + 4 * i) * 64 + c] = masked ? ((x[i] > 0) ? 1.0f : slope) * g[i] : g[i];
        __syncthreads();
        if (m0 + kColsumRows < ndat) fetch(m0 + kColsumRows);
        if (tid < 64) {
            const int rows = min(kColsumRows, ndat - m0);
            for (int m = 0; m < rows; m++) s = s + lds[m * 64 + c];
        }
        __syncthreads();
    }
    if (tid < 64) {
        float* out = pw.rowsum + col0 + c;
        *out = pw.rowsum_acc ? *out + s : s;
    }
}

// blockIdx.x < blocks_b: 64 columns of the bias gradient (first, so that these light workgroups run beside the
// others from the start); then blocks_x tiles of the parts of gx; then the tiles of gw.
template <int BN, int DEPTH>
__global__ void __launch_bounds__(256, 2)
    dense_backward_pair_kernel(const GemmParams px, const GemmParams pw, const int blocks_b, const int blocks_x,
                               const int tiles_x) {
    using T = PairTiles<BN>;
    static_assert(kColsumRows * 64 <= T::kLds, "the column-sum block must fit the shared LDS allocation");
    constexpr int NBN = BN / 64;
    __shared__ __attribute__((aligned(16))) float lds[T::kLds];
    const int bid = (int)blockIdx.x - blocks_b;
    if (bid < 0) {
        masked_colsum_64(pw, (int)blockIdx.x * 64, lds);
    } else if (bid < blocks_x) {
        gemm_tile_body<2, 2, 1, NBN, kPairBK, true, false, false, 1, DEPTH, false, true>(
            px, bid % tiles_x, bid / tiles_x, reinterpret_cast<float(*)[T::Ax::kFloats]>(lds),
            reinterpret_cast<float(*)[T::Bx::kFloats]>(lds + 2 * T::Ax::kFloats));
    } else {
        gemm_tile_body<2, 2, 1, NBN, kPairBK, false, false, false, 1, DEPTH, false, true>(
            pw, bid - blocks_x, 0, reinterpret_cast<float(*)[T::Aw::kFloats]>(lds),
            reinterpret_cast<float(*)[T::Bw::kFloats]>(lds + 2 * T::Aw::kFloats));
    }
}

GemmParams pair_params(const GemmDesc& d, bool a_kc, bool b_kc, int bn) {
    GemmParams p = make_params(d, a_kc, b_kc);
    p.tiles_m = (p.M + kPairTile - 1) / kPairTile;
    p.tiles_n = (p.N + bn - 1) / bn;
    p.group_m = 4;
    p.edge_buf = 1;
    return p;
}

}  // namespace

// Number of parts the reduction of gx is cut into for the paired launch, or 0 when the shape is not one for it:
// whole 64 x 64 tiles and whole 32-step tiles of both products, operands that allow aligned 128-bit loads, an
// activation whose derivative is a select (none, relu, leaky relu), and few enough workgroups that the launch is
// bound by latency rather than by the matrix cores (beyond that each product fills the chip on its own).
int dense_backward_pair_split(const float* pgx, const float* pgw, const float* pgy, const float* pw, const float* px,
                              const float* ppre, int64_t yvec, int64_t ndat, int64_t xvec, int act) {
    if (!pgx || !pgw) return 0;
    if (act != kActNone && act != kActRelu && act != kActLeaky) return 0;
    if (ndat % kPairTile || xvec % kPairTile || yvec % kPairTile || ndat < kPairTile || xvec < kPairTile || yvec < kPairTile)
        return 0;
    if (!aligned16(pgx) || !aligned16(pgw) || !aligned16(pgy) || !aligned16(pw) || !aligned16(px) ||
        (ppre && !aligned16(ppre)))
        return 0;
    if (ndat * yvec >= (1ll << 29) || yvec * xvec >= (1ll << 29) || ndat * xvec >= (1ll << 29)) return 0;   // 32-bit byte offsets
    const int64_t cus = compute_units();
    const int64_t tiles_x = (ndat / kPairTile) * (xvec / kPairTile), tiles_w = (yvec / kPairTile) * (xvec / kPairTile);
    // parts of gx's reduction (over yvec): as long as gw's reduction (over ndat), at least 128 steps, whole tiles
    int split = 1;
    for (int s = 2; s <= 16; s *= 2) {
        if (yvec % (s * kPairBK) != 0 || yvec / s < 128 || yvec / s < ndat) break;
        if (tiles_x * s > 2 * cus) break;
        split = s;
    }
    // (up to three workgroups per compute unit: 1024 x 1024 at a batch of 1024, 512 workgroups, 49.5 us against 50.4 with
    // the separate calls; at 2048, 768 workgroups, 95.9 against 84.3 on the larger tiles of the separate products)
    if (tiles_x * split + tiles_w >= 3 * cus) return 0;
    if (split > 1 && split * ndat * xvec * (int64_t)sizeof(float) > (64ll << 20)) return 0;
    return split;
}

int launch_dense_backward_pair(float* pgx, float* pgw, float* pgb, const float* pgy, const float* pw, const float* px,
                               const float* ppre, int64_t yvec, int64_t ndat, int64_t xvec, int act,
                               const float* leaky, bool acc, int split, hipStream_t stream) {
    const int a_mask = (ppre && act == kActRelu) ? 1 : (ppre && act == kActLeaky) ? 2 : 0;
    float* part = nullptr;
    if (split > 1) KAI_TRY(workspace(split * ndat * xvec * (int64_t)sizeof(float), &part));
    // gx[ndat,xvec] = ga[ndat,yvec] . w[yvec,xvec]: A = gy (rows ndat, reduction contiguous), B(n,k) = w[k*xvec + n]
    GemmDesc dx;
    dx.A = pgy; dx.B = pw; dx.C = split > 1 ? part : pgx;
    dx.M = ndat; dx.N = xvec; dx.K = yvec / split;
    dx.a_rs = yvec; dx.a_ks = 1; dx.b_rs = 1; dx.b_ks = xvec; dx.c_rs = xvec; dx.c_cs = 1;
    dx.acc = split > 1 ? 0 : acc;
    if (split > 1) {
        dx.nbatch = split; dx.bdiv = 1;
        dx.a_bs0 = dx.K * dx.a_ks; dx.b_bs0 = dx.K * dx.b_ks; dx.c_bs0 = ndat * xvec;
    }
    // gw[yvec,xvec] = ga^T . x: A(m,k) = gy[k*yvec + m], B(n,k) = x[k*xvec + n], reduction over ndat
    GemmDesc dw;
    dw.A = pgy; dw.B = px; dw.C = pgw;
    dw.M = yvec; dw.N = xvec; dw.K = ndat;
    dw.a_rs = 1; dw.a_ks = yvec; dw.b_rs = 1; dw.b_ks = xvec; dw.c_rs = xvec; dw.c_cs = 1;
    dw.acc = acc;
    // 128 columns per tile where that still gives every compute unit a workgroup (batch 256, 1024 -> 1024: 19.8 ->
    // 18.5 us; 512^3 with its 64 wide tiles: 16.1 -> 21.4); more than one tile on its way in registers from eight
    // tiles per workgroup on (batch 128, 1024 -> 1024 with four: 13.4 -> 13.7 us)
    const int64_t wide_blocks = (ndat / kPairTile) * (xvec / 128) * split + (yvec / kPairTile) * (xvec / 128);
    const int bn = xvec % 128 == 0 && wide_blocks >= compute_units() ? 128 : kPairTile;
    const bool deep = yvec / split / kPairBK >= 8 && ndat / kPairBK >= 8;
    GemmParams gx = pair_params(dx, true, false, bn), gw = pair_params(dw, false, false, bn);
    if (!fits_without_edges(gx, true, false, kPairTile, bn, kPairBK) || !fits_buffer_offsets(gx, true, false, kPairTile, bn) ||
        !fits_without_edges(gw, false, false, kPairTile, bn, kPairBK) || !fits_buffer_offsets(gw, false, false, kPairTile, bn))
        return fail(KAI_ERR_INVALID_ARGUMENT, "dense backward: shape does not fit the paired launch");
    gx.A2 = ppre; gx.a_mask = a_mask; gx.leaky = leaky;
    gw.A2 = ppre; gw.a_mask = a_mask; gw.leaky = leaky;
    gw.rowsum = pgb; gw.rowsum_acc = acc;   // read by the column-sum workgroups only
    const int tiles_x = gx.tiles_m * gx.tiles_n, tiles_w = gw.tiles_m * gw.tiles_n;
    const int blocks_x = tiles_x * split;
    const int blocks_b = pgb ? (int)(yvec / 64) : 0;
    const dim3 grid((unsigned)(blocks_b + blocks_x + tiles_w));
    if (bn == 128 && deep) dense_backward_pair_kernel<128, 2><<<grid, dim3(256), 0, stream>>>(gx, gw, blocks_b, blocks_x, tiles_x);
    else if (bn == 128) dense_backward_pair_kernel<128, 1><<<grid, dim3(256), 0, stream>>>(gx, gw, blocks_b, blocks_x, tiles_x);
    else if (deep) dense_backward_pair_kernel<64, 4><<<grid, dim3(256), 0, stream>>>(gx, gw, blocks_b, blocks_x, tiles_x);
    else dense_backward_pair_kernel<64, 1><<<grid, dim3(256), 0, stream>>>(gx, gw, blocks_b, blocks_x, tiles_x);
    KAI_TRY(check_launch("dense_backward_pair_kernel"));
    if (split > 1) {
        SplitReduceParams r{};
        r.part = part; r.C = pgx;
        r.M = ndat; r.N = xvec; r.c_rs = xvec; r.c_cs = 1;
        r.nsplit = split; r.accflag = acc;
        return launch_splitk_reduce(r, stream);
    }
    return KAI_OK;
}

}  // namespace kai
