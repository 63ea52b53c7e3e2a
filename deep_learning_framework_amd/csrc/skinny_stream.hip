// Skinny products (at most 16 rows of X, in one variant 32) whose operands allow aligned 128-bit loads:
//
//   y[m,n] (=|+=) act( sum_k x[m,k] * w[n,k] + bias[n] ),   m < M <= 16 (32)
//
// A workgroup of eight waves owns 16 rows of W and all of K; wave w owns a contiguous eighth of the tiles of
// 32 reduction steps.  Everything up to the final sum is private to a wave, so there is no
// barrier in the stream: a wave loads its slice tile by tile (16 x 32 of W and of X, one 128-byte
// line per row and load; rows of X beyond M are not loaded), two tiles ahead of the tile it is
// working on, and passes both through its own LDS tiles into the operand layout of
// v_mfma_f32_16x16x4_f32 (row = lane % 16, k group = lane / 16).  Loading in operand layout directly
// would touch 64 bytes per row and load, which costs a third of the bandwidth.  The matrix core only
// removes the per-row wave reductions and the X broadcasts a vector-ALU version would need; the
// kernel is bound by HBM.  The eight partial 16 x 16 results meet in LDS once, in wave order.
#include "gemv_skinny.h"

#include <type_traits>

#include "act_funcs.h"

namespace kai {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSsWaves = 8;
constexpr int kSsThreads = 64 * kSsWaves;
constexpr int kSsTileK = 32;                  // k per staged tile: one 128-byte line per row
constexpr int kSsRing = 3;                    // tiles of a wave in registers: one at work, the others on their way
constexpr int kSsLanesPerRow = kSsTileK / 4;
constexpr int kSsRowsPerLoad = 64 / kSsLanesPerRow;
// Row stride of the LDS tiles, 40 floats: a 128-bit LDS read is served eight lanes per cycle, lanes 4i .. 4i + 3
// together with lanes 4i + 16 .. 4i + 19, and the operand read (row = lane % 16, k = 4 * (lane / 16)) puts four
// consecutive rows and two k groups into such a group: their 16-byte pieces fall on eight different bank groups
// when the row stride is 8 or 24 floats modulo 32.  Measured with SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE on this
// read alone: stride 32 60 % conflict cycles, 36 (the padding this kernel had) 33 %, 40 none; the 128-bit stores
// of the tiles are conflict-free with any of them.
constexpr int kSsTileStride = kSsTileK + 8;
constexpr int kSsLoadsPerTile = 16 * kSsTileK / 4 / 64;   // 128-bit loads per lane and tile

template <int B, int E, typename F>
__device__ __forceinline__ void ss_static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        ss_static_for<B + 1, E>(f);
    }
}

__device__ __forceinline__ f32x4 keep_if(f32x4 v, bool keep) {
    const int m = keep ? -1 : 0;
    f32x4 o;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float e = v[j];
        o[j] = __int_as_float(__float_as_int(e) & m);   // bitwise: the load feeding v stays unconditional
    }
    return o;
}

// What the first loads need comes as scalars (14 dwords): this file is compiled with kernel-argument preload, so
// a wave finds them in SGPRs at its start instead of fetching the argument buffer first.
//
// WHOLE: K is a multiple of 32 (every tile of W lies inside its rows; N need not be a multiple of the workgroup's rows:
// the rows past N lie behind the end of the last workgroup's resource and read as zero).  The tiles then come through
// buffer loads: a resource over this workgroup's 16 rows of W and one over the M rows of X, a constant byte
// offset per lane and a scalar offset per tile.  Nothing is clamped or masked (a row of X past M lies behind the
// end of its resource and reads as zero), so a tile costs no vector instruction besides its LDS accesses and
// MFMAs: in the general variant the clamps, 64-bit addresses and masks of a tile were more issue cycles than its
// eight MFMAs.
//
// SLICES: K is a multiple of 8 x 512, so every wave owns the same number of slices of 512 steps and the tile loop
// of a slice is written out (16 tiles, every wait counted exactly by the compiler): 12.2 us at M = 4 against
// 12.9 us for the rolled loop that other lengths use.
//
// KT (rolled loop, whole-tile loads): K is a multiple of 4 but not of 32; the last tile's lanes past K load zeros.
//
// XL (whole tiles): 1 = at most 8 rows of X (one load per tile), 2 = more (two); 0 = decided per tile from M.  With
// the number of X loads a compile-time constant and every tile inside K, the written-out slice has no branch left,
// and the rolled loop only its own.
//
// XB: blocks of 16 rows of X.  2 (17..32 rows; whole tiles only, XL = 3 or 4): a tile of W meets
// two tiles of X and a wave keeps two accumulators -- W still streams once, where a tiled product of 17..32 rows
// cuts K over workgroups and sums the parts in a second launch.  3 and 4 (33..64 rows, XL = 5..8) with workgroups of
// 32 or 48 rows of W only: 6 to 12 accumulators per wave, and the matrix cores set the time.
//
// WR: rows of W per workgroup, 16, or 8 (whole tiles only) where workgroups of 16 rows would not cover the compute
// units: the second half of the W tile then stays zero and only eight columns of the result are stored.  32 and 48
// (whole tiles, written-out slices) where N / WR workgroups still cover the compute units: every workgroup loads
// all of X whatever it owns of W, and through the same load paths, so at 16 rows of W the tiles of X are as many
// bytes as those of W (twice as many with two blocks of X rows) and the compute unit's load path, not HBM, sets
// the time; with two or three blocks of W rows a tile of X meets two or three tiles of W.  The last workgroup may
// own fewer blocks (N a multiple of 16): the rows behind N lie behind the end of its resource and read as zero.
template <bool WHOLE, bool SLICES, int XL = 0, int XB = 1, int WR = 16, bool KT = false>
__global__ void __launch_bounds__(kSsThreads)
skinny_stream_kernel(const float* __restrict__ W, const float* __restrict__ X, const int64_t ldw, const int64_t ldx,
                     const int64_t N, const int M, const int K, float* __restrict__ Y, const SkinnyTail t) {
    const SkinnyParams p = skinny_params(W, X, ldw, ldx, N, M, K, Y, t);
    constexpr int WB = WR <= 16 ? 1 : WR / 16;      // blocks of 16 rows of W
    constexpr int kWTileRows = 16 * WB;
    __shared__ __attribute__((aligned(16))) float lds_w[kSsWaves][kWTileRows * kSsTileStride];
    static_assert(XB == 1 || (XB >= 2 && XB <= 4 && WHOLE && (SLICES || XB == 2) && XL > kSsLoadsPerTile * (XB - 1) && XL <= kSsLoadsPerTile * XB),
                  "several blocks of X rows exist for whole tiles (three and four: in written-out slices)");
    static_assert(XL == 0 || WHOLE, "a compile-time number of X loads: whole tiles");
    static_assert(!KT || (WHOLE && !SLICES && XL > 0 && WR == 16), "a last tile that K does not fill: the rolled loop over whole-tile loads");
    static_assert(XB <= 2 || WR >= 32, "three and four blocks of X rows: with two or three blocks of W rows only");
    // tiles of a wave in registers (written-out slices): with three and four blocks of X rows a tile is 10 to 14 loads
    // per lane, and two tiles are what the registers hold
    constexpr int kRing = XB >= 3 ? 2 : kSsRing;
    static_assert(WR == 16 || (WR == 8 && WHOLE && XB == 1 && kSsRowsPerLoad == 8) ||
                      ((WR == 32 || WR == 48) && WHOLE && SLICES && XL > 0),
                  "eight rows of W: one load per tile; 32 and 48: whole tiles in written-out slices");
    constexpr int kWLoads = WR / kSsRowsPerLoad;    // 128-bit loads per lane that cover the workgroup's rows of a W tile
    constexpr int kWRegs = kWLoads > kSsLoadsPerTile ? kWLoads : kSsLoadsPerTile;
    constexpr int kXLoads = kSsLoadsPerTile * XB;   // 128-bit loads per lane that cover a tile of X
    __shared__ __attribute__((aligned(16))) float lds_x[kSsWaves][16 * XB * kSsTileStride];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15;    // row of W inside the block's 16 / row of X
    const int g = lane >> 4;    // k group of the MFMA operand
    const int64_t n0 = (int64_t)blockIdx.x * WR;
    const int lrow = lane / kSsLanesPerRow;          // a load covers kSsRowsPerLoad rows x kSsTileK k
    const int lk = (lane % kSsLanesPerRow) * 4;
    float* tw = lds_w[wave];
    float* tx = lds_x[wave];

    // rows of W beyond the workgroup's WR and rows of X that are never loaded stay zero in the tiles
#pragma unroll
    for (int j = kWLoads; j < kSsLoadsPerTile; j++)
        *reinterpret_cast<f32x4*>(tw + (kSsRowsPerLoad * j + lrow) * kSsTileStride + lk) = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kXLoads; j++)
        *reinterpret_cast<f32x4*>(tx + (kSsRowsPerLoad * j + lrow) * kSsTileStride + lk) = f32x4{0.f, 0.f, 0.f, 0.f};

    f32x4 acc[WB][XB];
#pragma unroll
    for (int a = 0; a < WB; a++)
#pragma unroll
        for (int b = 0; b < XB; b++) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    // One tile = 16 rows x kSsTileK k of W and of X, kSsLoadsPerTile 128-bit loads per lane each.  Addresses past
    // K are clamped into the row (every load is unconditional); what they return is zeroed on the way to LDS.
    // WHOLE: resources and per-lane offsets (bytes)
    auto uniform_ptr = [](const float* q) -> float* {
        const uint64_t a = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
    };
    const int w_rows = WR >= 16 ? (int)min((int64_t)WR, p.N - n0) : WR;   // rows of W this workgroup has (uniform; the last workgroup may have fewer)
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        uniform_ptr(p.W + n0 * p.ldw), 0, (int)(((int64_t)(w_rows - 1) * p.ldw + p.K) * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
        uniform_ptr(p.X), 0, (int)(((int64_t)(p.M - 1) * p.ldx + p.K) * 4), 0x00020000);
    int woff[kWRegs], xoff[kXLoads];
#pragma unroll
    for (int j = 0; j < kWRegs; j++) {
        // a row past the workgroup's last must land behind the end of the resource whatever ldw is
        const int row = kSsRowsPerLoad * j + lrow;
        woff[j] = WR >= 16 && row >= w_rows ? 0x7FFFFFF0 : (int)(((int64_t)row * p.ldw + lk) * 4);
    }
#pragma unroll
    for (int j = 0; j < kXLoads; j++) {
        // a row past M must land behind the end of the resource whatever ldx is: the last row's end is the limit
        const int m = kSsRowsPerLoad * j + lrow;
        xoff[j] = m < p.M ? (int)(((int64_t)m * p.ldx + lk) * 4) : 0x7FFFFFF0;
    }
    auto load_w = [&](f32x4(&dst)[kWRegs], int kt) {
        if constexpr (WHOLE) {
            // a tile past the end of K (a wave's last slice may be short) re-reads the last whole tile instead of
            // counting on the range check for the scalar part of the address; it is never consumed
            // KT: the tile is addressed as it lies, and a lane whose four steps are past K (K is a multiple of 4) is
            // steered behind the end of the resource: zeros, in W and in X alike
            const int kc = KT ? kt * 4 : min(kt, p.K - kSsTileK) * 4;
            const bool past = KT && kt + lk >= p.K;
#pragma unroll
            for (int j = 0; j < kWLoads; j++)   // aux 2: non-temporal, as the general variant's loads
                dst[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, past ? 0x7FFFFFF0 : woff[j], kc, 2));
            return;
        }
#pragma unroll
        for (int j = 0; j < kSsLoadsPerTile; j++) {
            const int64_t n = n0 + kSsRowsPerLoad * j + lrow;
            const float* src = p.W + (n < p.N ? n : p.N - 1) * p.ldw + min(kt + lk, p.K - 4);
            dst[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src));
        }
    };
    auto load_x = [&](f32x4(&dst)[kXLoads], int kt) {
        if constexpr (WHOLE) {
            const int kc = KT ? kt * 4 : min(kt, p.K - kSsTileK) * 4;
            const bool past = KT && kt + lk >= p.K;
#pragma unroll
            for (int j = 0; j < kXLoads; j++)
                if (XL ? j < XL : kSsRowsPerLoad * j < p.M)   // uniform
                    dst[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, past ? 0x7FFFFFF0 : xoff[j], kc, 0));
            return;
        }
#pragma unroll
        for (int j = 0; j < kSsLoadsPerTile; j++) {
            if (kSsRowsPerLoad * j < p.M) {   // uniform: these rows hold a row of X
                const int m = kSsRowsPerLoad * j + lrow;
                dst[j] = *reinterpret_cast<const f32x4*>(p.X + (int64_t)min(m, p.M - 1) * p.ldx + min(kt + lk, p.K - 4));
            }
        }
    };
    auto consume = [&](const f32x4(&w)[kWRegs], const f32x4(&x)[kXLoads], int kt) {
        if ((WHOLE && XL) || kt < p.K) {   // uniform (whole tiles with a fixed number of X loads: the callers pass tiles inside K only)
#pragma unroll
            for (int j = 0; j < kWLoads; j++) {
                const int row = kSsRowsPerLoad * j + lrow;
                *reinterpret_cast<f32x4*>(tw + row * kSsTileStride + lk) =
                    WHOLE ? w[j] : keep_if(w[j], n0 + row < p.N && kt + lk < p.K);
            }
#pragma unroll
            for (int j = 0; j < kXLoads; j++) {
                const int row = kSsRowsPerLoad * j + lrow;
                if (XL ? j < XL : kSsRowsPerLoad * j < p.M)
                    *reinterpret_cast<f32x4*>(tx + row * kSsTileStride + lk) =
                        WHOLE ? x[j] : keep_if(x[j], row < p.M && kt + lk < p.K);
            }
            __builtin_amdgcn_wave_barrier();   // LDS serves a wave's accesses in order; the compiler must too
#pragma unroll
            for (int s = 0; s < kSsTileK / 16; s++) {
                if constexpr (WB == 1) {
                    const f32x4 wv = *reinterpret_cast<const f32x4*>(tw + r * kSsTileStride + 16 * s + 4 * g);
#pragma unroll
                    for (int b = 0; b < XB; b++) {
                        const f32x4 xv = *reinterpret_cast<const f32x4*>(tx + (16 * b + r) * kSsTileStride + 16 * s + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            acc[0][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[e], wv[e], acc[0][b], 0, 0, 0);
                    }
                } else {
                    // all operands of the 16 steps first, then the products with the accumulators taking turns
                    f32x4 wv[WB], xv[XB];
#pragma unroll
                    for (int a = 0; a < WB; a++)
                        wv[a] = *reinterpret_cast<const f32x4*>(tw + (16 * a + r) * kSsTileStride + 16 * s + 4 * g);
#pragma unroll
                    for (int b = 0; b < XB; b++)
                        xv[b] = *reinterpret_cast<const f32x4*>(tx + (16 * b + r) * kSsTileStride + 16 * s + 4 * g);
#pragma unroll
                    for (int e = 0; e < 4; e++)
#pragma unroll
                        for (int a = 0; a < WB; a++)
#pragma unroll
                            for (int b = 0; b < XB; b++)
                                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[b][e], wv[a][e], acc[a][b], 0, 0, 0);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    };
    if constexpr (SLICES) {
        // wave w owns the slices of 512 steps number w, w + 8, ...; per slice a ring of kRing tiles, the loads of
        // tile t + kRing issued as soon as tile t has left its registers
        constexpr int kSlice = 512, kTiles = kSlice / kSsTileK;
        // Rows of 32 KiB and more that are a power of two apart: with every wave walking its slice from the slice's
        // first tile the requests of a moment crowd onto few memory channels; wave w starts 2 w tiles into its slice
        // instead and wraps (4096 x 8192: 27.3 -> 24.3 us at M = 4, 4096 x 16384: 61.4 -> 47.9; 12288 and other
        // lengths unchanged).  At 4096 steps the plain order is the faster one (12.1 against 12.4 us).
        const int stag = p.K >= 8192 ? 2 * wave : 0;
        for (int k0 = wave * kSlice; k0 < p.K; k0 += kSsWaves * kSlice) {
            f32x4 w[kRing][kWRegs], x[kRing][kXLoads];
            ss_static_for<0, kRing>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                load_w(w[t], k0 + ((t + stag) & (kTiles - 1)) * kSsTileK);
                load_x(x[t], k0 + ((t + stag) & (kTiles - 1)) * kSsTileK);
            });
            ss_static_for<0, kTiles>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                constexpr int slot = t % kRing;
                __builtin_amdgcn_sched_barrier(0);
                consume(w[slot], x[slot], k0 + ((t + stag) & (kTiles - 1)) * kSsTileK);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (t + kRing < kTiles) {
                    load_w(w[slot], k0 + ((t + kRing + stag) & (kTiles - 1)) * kSsTileK);
                    load_x(x[slot], k0 + ((t + kRing + stag) & (kTiles - 1)) * kSsTileK);
                }
            });
        }
    } else {
        // Software pipeline over a wave's tiles: the tiles of K are dealt out evenly, wave w takes a contiguous run
        // (one or two tiles' difference between waves whatever K is; fixed slices of 512 left some waves with three
        // slices and others with two at K = 11008).  A ring of kSsRing tiles per wave, the loads of tile t + kSsRing
        // issued as soon as tile t has left its registers, so the stream of a wave goes on while the wave passes a
        // tile through LDS and the matrix core.  A deeper ring does not help: a wave that asks for more than the
        // compute unit's memory pipeline takes at once stalls at the issue of its loads, in front of the tile that
        // has long arrived.
        const int tiles_total = (p.K + kSsTileK - 1) / kSsTileK;
        const int tiles_base = tiles_total / kSsWaves, tiles_rem = tiles_total % kSsWaves;
        const int t_count = tiles_base + (wave < tiles_rem ? 1 : 0);
        const int k_begin = (wave * tiles_base + min(wave, tiles_rem)) * kSsTileK;
        f32x4 w[kSsRing][kWRegs], x[kSsRing][kXLoads];
        ss_static_for<0, kSsRing>([&](auto tc) {
            constexpr int t = decltype(tc)::value;
            load_w(w[t], k_begin + t * kSsTileK);
            load_x(x[t], k_begin + t * kSsTileK);
        });
        // Whole rounds of the ring that every wave of the workgroup has: no condition inside the loop, so the
        // compiler counts the loads in flight exactly across the back edge (with a condition around a tile it
        // waited for every load once per round: 12.2 -> 14.4 us at M = 4).  At most kSsRing tiles follow.
        const int rounds = tiles_base / kSsRing;
        for (int r = 0; r < rounds; r++) {
            ss_static_for<0, kSsRing>([&](auto sc) {
                constexpr int slot = decltype(sc)::value;
                const int kt = k_begin + (r * kSsRing + slot) * kSsTileK;
                __builtin_amdgcn_sched_barrier(0);
                consume(w[slot], x[slot], kt);
                __builtin_amdgcn_sched_barrier(0);
                load_w(w[slot], kt + kSsRing * kSsTileK);   // past the wave's run: surplus, clamped, never consumed
                load_x(x[slot], kt + kSsRing * kSsTileK);
            });
        }
        ss_static_for<0, kSsRing>([&](auto sc) {
            constexpr int slot = decltype(sc)::value;
            const int t = rounds * kSsRing + slot;
            if (t < t_count) consume(w[slot], x[slot], k_begin + t * kSsTileK);   // uniform
        });
    }

    // acc[a][b][v] = D[m = 16 * b + 4 * g + v][n = n0 + 16 * a + r]; the tiles are free now: wave w parks its
    // results in its W tile, a 16 x 16 block per (a, b), kXbPass blocks of X rows at a time
    constexpr int kParkFloats = kWTileRows * kSsTileStride;
    constexpr int kXbPass = 256 * XB * WB <= kParkFloats ? XB : (XB % 2 == 0 && 512 * WB <= kParkFloats) ? 2 : 1;
    static_assert(256 * kXbPass * WB <= kWTileRows * kSsTileStride && XB % kXbPass == 0, "a pass of a wave's results fits its W tile");
#pragma unroll
    for (int b0 = 0; b0 < XB; b0 += kXbPass) {
        __syncthreads();
#pragma unroll
        for (int a = 0; a < WB; a++)
#pragma unroll
            for (int b = 0; b < kXbPass; b++)
#pragma unroll
                for (int v = 0; v < 4; v++) tw[((a * kXbPass + b) * 16 + 4 * g + v) * 16 + r] = acc[a][b0 + b][v];
        __syncthreads();
#pragma unroll
        for (int i0 = 0; i0 < 256 * kXbPass * WB; i0 += kSsThreads) {
            const int e = i0 + tid;
            const int blk = e >> 8, a = blk / kXbPass, b = b0 + blk % kXbPass;
            const int m = 16 * b + ((e >> 4) & 15), j = e & 15;
            const int64_t n = n0 + 16 * a + j;
            if (e < 256 * kXbPass * WB && m < p.M && n < p.N && j < WR) {
                float v = 0.f;
#pragma unroll
                for (int i = 0; i < kSsWaves; i++) v += lds_w[i][e];
                const float leaky = p.leaky ? *p.leaky : 0.f;
                const int64_t idx = (int64_t)m * p.ldy + n;
                if (p.accflag) v += p.Y[idx];
                if (p.bias) v += p.bias[n];
                if (p.Y2) p.Y2[idx] = v;
                p.Y[idx] = apply_act(v, p.act, leaky);
            }
        }
    }
}

}  // namespace

// 17..32 rows: whole tiles, written-out slices, workgroups that cover the compute units.
// Measured against a row of 32 x 128 tiles with K in parts, us per call at 17 / 32 rows with 16-row workgroups, the
// matrix streamed from HBM (rotating buffers) | still in the last-level cache: 4096 x 4096 21.2 -> 15.0 / 21.3 -> 17.9 |
// 16.7 -> 14.4 / 20.2 -> 17.2; 11008 x 4096 45.4 -> 38.3 / 49.7 -> 45.8 | 39.0 -> 36.1 / 47.3 -> 44.2; 4096 x 8192
// 37.4 -> 28.9 / 38.7 -> 34.0 | 25.8 -> 27.9 / 29.6 -> 33.0.
// Which matrices 17 and more rows stream.  Up to 192 MB a matrix may still lie in the 256 MB last-level cache when a
// serving loop multiplies it again and again, and there the tiled kernels win for rows longer than 4096 steps
// (4096 x 8192, 128 MB, 17 / 32 rows, us per call from HBM | from the cache: tiles 37.7 / 38.9 | 26.2 / 31.2, this
// kernel 30.9 / 35.2 | 30.0 / 34.3), so such matrices stream only up to 96 MB.  Beyond 192 MB a matrix comes from
// HBM on every call and streams whatever its shape (8192 x 8192 at 24 / 32 / 48 rows: tiles 64.9 / 66.9 / 78.8, this
// kernel 53.8 / 55.4 / 66.7; 11008 x 8192: 87.3 / 96.3 / 105.9 against 68.4 / 72.1 / 87.3; 28672 x 4096 at 32 / 48 rows
// 110.4 / 135.8 against 98.7 / 126.6).
static bool stream_size_rule(int64_t n, int64_t k) {
    const int64_t bytes = n * k * 4;
    return bytes > (192ll << 20) || k <= 4096 || bytes <= (96ll << 20);
}

// 33..64 rows (three and four blocks of X rows) run here only where workgroups of 32 or 48 rows of W apply: with
// 16 rows of W a workgroup would load four times as many bytes of X as of W.
static bool stream_many_rows_base(const SkinnyParams& p) {
    // Which K and N, by the row count.  Rows in written-out slices (K a multiple of 4096): from 16 rows of W per
    // compute unit on, K = 4096 from 9 on (17 / 24 / 32 rows, us with W from HBM | from the last-level cache, fastest
    // tiled plan -> here: 3072 x 4096 20.1 / 20.3 / 19.5 -> 13.8 / 15.1 / 16.7 | 15.5 / 15.8 / 18.4 -> 13.4 / 14.5 / 16.0;
    // 2304 x 4096 19.2 / 19.6 / 18.4 -> 13.5 / 14.7 / 16.4 | 15.2 / 15.5 / 18.2 -> 13.1 / 14.1 / 15.8; at 8192 steps
    // 3072 columns 23.5 -> 25.0 from the cache; 2048 columns and fewer: no gain at any K).  Other K in whole tiles,
    // 17..32 rows only, through the rolled loop: 1024..2048 steps from 9 rows of W per compute unit on (4096 x 2048
    // 14.7 / 14.8 / 15.1 -> 9.9 / 10.3 / 11.5 | 11.7 / 12.1 / 14.3 -> 9.3 / 9.8 / 10.6; 3072 x 1024 10.9 / 12.2 / 13.8 ->
    // 6.9 / 7.3 / 7.8; 8192 x 2048 20.9 / 21.2 / 21.5 -> 16.6 / 17.9 / 19.5 | 15.9 / 16.2 / 19.5 -> 15.6 / 16.6 / 18.1),
    // up to 4096 steps for 12..16 rows of W per compute unit (4096 x 3072 18.7 / 18.8 / 18.7 -> 14.5 / 15.7 / 17.6 |
    // 14.6 / 14.8 / 17.5 -> 13.7 / 14.8 / 16.5; 5120 x 3072 and wider lose, 21.4 -> 24.1, and so does 2304 x 3072 from
    // the cache); longer rows (5120, 6144, 11008 steps) gain with W from HBM but lose 8..30 % from the cache.
    const int64_t cus = compute_units();
    bool k_ok;
    if (p.K % (kSsWaves * 512) == 0) k_ok = p.N >= (p.K == kSsWaves * 512 && p.M <= 2 * kSkinnyMaxRows ? 9 : 16) * cus;
    else if (p.M > 2 * kSkinnyMaxRows || p.K % 4 != 0) k_ok = false;
    else if (p.K >= 1024 && p.K <= 2048) k_ok = p.N >= 9 * cus && p.N <= 48 * cus;   // (measured up to 11008 columns; 32000 x 1024 at 17 rows: 36 us here, 22 on the tiles)
    else k_ok = p.K > 2048 && p.K < 4096 && p.N >= 12 * cus && p.N <= 16 * cus;
    return p.M > kSkinnyMaxRows && p.M <= 4 * kSkinnyMaxRows && k_ok &&
           stream_size_rule(p.N, p.K) && p.ldw % 4 == 0 && p.ldx % 4 == 0 && aligned16(p.W) && aligned16(p.X) &&
           (15 * p.ldw + p.K) * 4 < (1ll << 31) && ((int64_t)(p.M - 1) * p.ldx + p.K) * 4 < 0x7FFFFFF0ll;
}

bool skinny_stream32_applies(const SkinnyParams& p) {
    return stream_many_rows_base(p) && (p.M <= 2 * kSkinnyMaxRows || skinny_stream_wide_rows(p) != 0);
}

bool skinny_stream_applies(const SkinnyParams& p) {
    return p.M >= 1 && p.M <= kSkinnyMaxRows && p.K >= 64 && p.K % 4 == 0 && p.ldw % 4 == 0 && p.ldx % 4 == 0 &&
           aligned16(p.W) && aligned16(p.X);
}

// Eight rows of W per workgroup: whole tiles in written-out slices, N / 8 workgroups that cover at least half of the
// compute units and at most all of them (one round).  Measured against 16-row workgroups (5..16 rows) and the
// slice kernels (2..4 rows), us per call with W from HBM: 2048 x 4096 M = 4 / 8 / 16 11.8 / 9.9 / 11.9 -> 8.0 / 8.2 /
// 9.9, 1024 x 4096 11.2 / 9.2 / 11.3 -> 7.5 / 7.6 / 9.2, 2048 x 8192 M = 8 / 16 18.3 / 21.9 -> 14.7 / 17.6.  With more
// than 4096 steps the slice kernels keep 2..4 rows (1024 x 8192 M = 2: 8.5 against 12.7); N = 2560 and 3072 (a
// second, partly filled round) lost 15..40 % at 8 and 16 rows, and so did the rolled loop for other K at most row counts.
bool skinny_stream8_applies(const SkinnyParams& p) {
    const int64_t cus = compute_units();
    return skinny_stream_applies(p) && p.M >= 2 && (p.K == 4096 || p.M >= 5) && p.N % 8 == 0 && p.K % (kSsWaves * 512) == 0 &&
           p.N <= 8 * cus && p.N >= 4 * cus && (7 * p.ldw + p.K) * 4 < (1ll << 31) &&
           ((int64_t)(p.M - 1) * p.ldx + p.K) * 4 < 0x7FFFFFF0ll;
}

int launch_skinny_stream8(const SkinnyParams& p, hipStream_t stream) {
    if (!skinny_stream8_applies(p)) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: shape not served with 8-row workgroups");
    const SkinnyTail t = skinny_tail(p);
    const dim3 grid((unsigned)(p.N / 8)), block(kSsThreads);
    if (p.M <= 8) skinny_stream_kernel<true, true, 1, 1, 8><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else skinny_stream_kernel<true, true, 2, 1, 8><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    return check_launch("skinny_stream_kernel");
}

namespace {
int g_stream_rows_override = 0;

template <int WR>
int launch_wide(const SkinnyParams& p, const SkinnyTail& t, hipStream_t stream) {
    const dim3 grid((unsigned)((p.N + WR - 1) / WR)), block(kSsThreads);
    if (p.M <= 8) skinny_stream_kernel<true, true, 1, 1, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (p.M <= 16) skinny_stream_kernel<true, true, 2, 1, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (p.M <= 24) skinny_stream_kernel<true, true, 3, 2, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (p.M <= 32) skinny_stream_kernel<true, true, 4, 2, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (p.M <= 40) skinny_stream_kernel<true, true, 5, 3, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (p.M <= 48) skinny_stream_kernel<true, true, 6, 3, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (p.M <= 56) skinny_stream_kernel<true, true, 7, 4, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else skinny_stream_kernel<true, true, 8, 4, WR><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    return check_launch("skinny_stream_kernel");
}
}  // namespace

void set_skinny_stream_rows_override(int rows) { g_stream_rows_override = rows; }

// Rows of W per workgroup where workgroups of 32 or 48 rows take the product, 0 where those of 16 rows keep it.
// Fewer, larger workgroups load fewer bytes of X but leave a compute unit with one workgroup's eight waves, which
// pull less through its load path than the sixteen of two resident 16-row workgroups; so they pay only from 9 rows
// of X on, and only where their number fills the compute units.  Measured, us per call with W from HBM, 16-row
// workgroups -> these (K = 4096): 11008 columns (230 workgroups of 48) 8 / 16 / 24 / 32 rows 29.6 / 33.9 / 40.8 / 45.4 ->
// 29.5 / 29.9 / 34.8 / 36.4; 12288 (256 of 48) 31.0 / 34.7 / 41.9 / 47.2 -> 32.9 / 32.9 / 38.5 / 39.3; 32000 (667 of 48)
// 16 rows 90.2 -> 84.8; 8192 (256 of 32) 16 / 24 / 32 rows 23.9 / 28.5 / 32.0 -> 28.2 / 28.9 / 29.8; 7168 (224 of 32)
// 23.8 / 27.7 / 30.7 -> 25.1 / 26.5 / 27.8; 6144 (192 of 32) 22.9 / 26.5 / 29.9 -> 22.5 / 24.8 / 26.1; 16384 (342 of 48,
// 512 of 32) 16 rows 45.6 -> 51.4 / 51.8.  Hence: 48 rows from 9 rows of X on where the workgroups fill their rounds
// over the compute units to 85 %, or are one round that is four fifths full (10240 columns, 214 workgroups: 12 / 16
// rows 31.1 / 33.0 -> 27.8 / 28.4, 33 / 48 rows 50.6 / 51.9 on the tiled kernel -> 43.6 / 45.5), from 17 rows on in one
// round only; 32 rows from 17 rows of X on where the workgroups are one round, at least three quarters full.
// 17..24 rows on 32-row workgroups only while these are at most nine tenths of the compute units (8192 columns, 256
// workgroups, 17 / 24 rows: 25.4 / 28.9 with 16-row workgroups, 29.5 / 30.4 with these; 6144 columns 26.0 / 27.0 -> 24.5 / 25.3).
// Rows of 8192 steps (us, W from HBM, 16-row -> 32-row workgroups): 8192 columns 16 / 24 / 32 rows 55.1 / 59.5 / 66.3 ->
// 50.4 / 53.8 / 55.4; 6144 columns 45.4 / 53.8 / 59.6 -> 38.6 / 46.6 / 49.6 (hence 32-row workgroups from 9 rows on there);
// several rounds of 32-row workgroups at K = 4096: 14336 columns (448) 24 / 32 rows 54.2 / 58.9 -> 50.4 / 52.4, 16384
// (512) 57.5 / 63.0 -> 53.9 / 54.6, 28672 (896) 96.4 / 109.5 -> 95.0 / 98.7, while 48-row workgroups in a partly filled
// second or third round lose (16384: 65.7 / 69.4; 28672: 102.0 / 104.5).
// 33..64 rows run on these workgroups only; fastest tiled plan (tile and part count forced) -> here, W from HBM |
// W in the last-level cache: 11008 columns 33 / 48 / 64 rows 58.5 / 60.1 / 63.1 -> 43.1 / 45.1 / 55.7 | 53.3 / 53.8 / 54.9 ->
// 41.7 / 42.6 / 55.5; 12288 58.5 / 60.7 / 63.9 -> 44.7 / 46.2 / 58.7; 10240 33 / 48 rows 50.7 / 50.8 -> 42.5 / 44.4; 8192
// (32-row workgroups) 39.9 / 40.3 -> 34.9 / 35.3 | 37.8 / 38.3 -> 31.9 / 34.7; 6144 33.7 / 35.3 -> 30.2 / 32.7.  With four
// blocks of X rows (49..64 rows) the 32-row workgroups lose to the tiles (8192 columns 43.5 against 41.7 | 43.3 against
// 39.4; 6144 39.6 against 37.3 | 38.7 against 33.3), so those rows stream on 48-row workgroups only.  (A ring of three
// tiles with three blocks of X rows: 46.0 -> 48.8 at 11008 x 48 rows, no gain elsewhere.)
int skinny_stream_wide_rows(const SkinnyParams& p) {
    if (g_stream_rows_override == 16 && p.M <= 2 * kSkinnyMaxRows) return 0;
    const bool base = p.M > kSkinnyMaxRows ? stream_many_rows_base(p) : (p.M >= 2 && skinny_stream_applies(p));
    if (!base || p.K % (kSsWaves * 512) != 0 || (47 * p.ldw + p.K) * 4 >= (1ll << 31) ||
        ((int64_t)(p.M - 1) * p.ldx + p.K) * 4 >= 0x7FFFFFF0ll)
        return 0;
    if (g_stream_rows_override == 32 || g_stream_rows_override == 48) return g_stream_rows_override;
    const int64_t cus = compute_units();
    const int64_t groups48 = (p.N + 47) / 48, rounds48 = (groups48 + cus - 1) / cus;
    const int64_t groups32 = (p.N + 31) / 32, rounds32 = (groups32 + cus - 1) / cus;
    // A last round of 16-row workgroups that is mostly empty costs a whole round: 5..32 rows then run on one round of
    // wider workgroups although that round is only half to three quarters full.  Measured, us with W from HBM, 16-row
    // workgroups -> these (K = 4096 | 8192): 4352 columns (272 of 16, 136 of 32) 5 / 16 / 32 rows 18.0 / 21.9 / 29.3 ->
    // 16.2 / 18.3 / 24.7 | 5 / 16 rows 36.0 / 43.4 -> 29.4 / 34.3; 5120 (320, 160) 18.2 / 22.1 / 29.6 -> 17.6 / 19.2 / 24.8 |
    // 36.7 / 44.8 -> 30.9 / 35.9; 5632 (352, 176) 18.4 / 22.0 / 29.6 -> 18.5 / 20.1 / 25.3; 6144 (384 = 1.5 rounds, 192) at
    // K = 4096 5 rows 19.0 -> 20.0, 16 rows 22.6 -> 21.4, so not there, but at K = 8192 5 / 8 rows 38.6 / 40.5 -> 32.5 /
    // 33.5; 8704 (544 of 16 in three rounds, 182 of 48) 5 / 16 / 32 rows 27.1 / 31.8 / 43.1 -> 24.2 / 25.9 / 33.5 | 57.9 /
    // 66.8 / 87.8 -> 51.2 / 54.7 / 66.0; 9216 (576, 192) 27.2 / 32.3 / 43.7 -> 25.3 / 26.5 / 33.8.
    // Further: 8448 (528 of 16, 176 of 48) 5 / 16 / 32 rows 26.7 / 31.5 / 42.8 -> 23.7 / 25.4 / 33.4; 9728 (608, 203) 27.6 /
    // 32.4 / 44.0 -> 26.4 / 27.2 / 34.4; 4 rows at 4352 columns 17.7 -> 15.9 | 34.8 -> 28.6, at 8448 26.4 -> 23.6; two rounds
    // of 32-row workgroups instead of four of 16 (12800 columns, 78 % full either way) 24 / 32 rows 51.5 / 56.8 -> 47.3 /
    // 49.6 | 12 / 16 / 32 rows 88.0 / 92.2 / 117.5 -> 80.2 / 81.1 / 94.2.
    if (p.M <= 2 * kSkinnyMaxRows) {
        const int64_t groups16 = (p.N + 15) / 16, rounds16 = (groups16 + cus - 1) / cus;
        if (rounds16 >= 2 && groups16 * 100 < 82 * rounds16 * cus) {
            if (rounds48 == 1 && groups48 * 100 >= 65 * cus) return 48;
            if (groups16 * 100 < (p.K >= 8192 ? 82 : 72) * rounds16 * cus && rounds32 == 1 && groups32 * 2 >= cus) return 32;
            if (rounds32 >= 2 && 2 * rounds32 <= rounds16 && groups32 * 100 >= 75 * rounds32 * cus &&
                (p.M > kSkinnyMaxRows || (p.M > 8 && p.K >= 8192)))
                return 32;
        }
    }
    if (p.M <= 8) return 0;
    const bool many = p.M > 3 * kSkinnyMaxRows;      // 49..64 rows: four blocks of X rows
    if (rounds48 == 1 ? groups48 * 100 >= (many ? 85 : 80) * cus : (p.M <= kSkinnyMaxRows && groups48 * 100 >= 85 * rounds48 * cus))
        return 48;
    if (many || groups32 * 4 < 3 * cus) return 0;
    // 9..16 rows: only with rows of 8192 steps and more, one round
    if (p.M <= kSkinnyMaxRows) return p.K >= 8192 && rounds32 == 1 ? 32 : 0;
    // 17..48 rows: one round, or several that are filled to 85 %; 17..24 rows with rows of up to 4096 steps only
    // while the workgroups number at most nine tenths of the compute units
    if (rounds32 > 1 && groups32 * 100 < 85 * rounds32 * cus) return 0;
    if (p.M <= 24 && p.K <= 4096 && rounds32 == 1 && groups32 * 10 > 9 * cus) return 0;
    return 32;
}

int launch_skinny_stream(const SkinnyParams& p, hipStream_t stream) {
    const int64_t blocks = (p.N + 15) / 16;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: too many output columns");
    const SkinnyTail t = skinny_tail(p);
    const int wide = skinny_stream_wide_rows(p);
    if (wide == 48) return launch_wide<48>(p, t, stream);
    if (wide == 32) return launch_wide<32>(p, t, stream);
    // whole tiles, and byte offsets inside a workgroup's 16 rows of W and inside X that fit 31 bits
    const bool whole = p.K % kSsTileK == 0 && (15 * p.ldw + p.K) * 4 < (1ll << 31) &&
                       ((int64_t)(p.M - 1) * p.ldx + p.K) * 4 < 0x7FFFFFF0ll;
    const bool slices = p.K % (kSsWaves * 512) == 0;
    // whole-tile loads with a last tile that K does not fill
    const bool ktail = !whole && p.K % 4 == 0 && p.K > kSsTileK && (15 * p.ldw + p.K) * 4 < (1ll << 31) &&
                       ((int64_t)(p.M - 1) * p.ldx + p.K) * 4 < 0x7FFFFFF0ll;
    const dim3 grid((unsigned)blocks), block(kSsThreads);
    if (p.M > kSkinnyMaxRows) {
        if (!skinny_stream32_applies(p) || p.M > 2 * kSkinnyMaxRows)
            return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: more than 16 rows");
        if (ktail && p.M <= 24) skinny_stream_kernel<true, false, 3, 2, 16, true><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        else if (ktail) skinny_stream_kernel<true, false, 4, 2, 16, true><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        else if (!slices && p.M <= 24) skinny_stream_kernel<true, false, 3, 2><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        else if (!slices) skinny_stream_kernel<true, false, 4, 2><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        else if (p.M <= 24) skinny_stream_kernel<true, true, 3, 2><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        else skinny_stream_kernel<true, true, 4, 2><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        return check_launch("skinny_stream_kernel");
    }
    // (the rolled loop with one load of X per tile as a compile-time fact: 4096 x 2048 at 4 rows 8.1 -> 7.6 us, 3072 x
    // 3072 10.0 -> 9.6, 1..3 % elsewhere; with two, 9..16 rows, -2..+2 %: those keep the count read from M)
    if (whole && !slices && p.M <= 8) {
        skinny_stream_kernel<true, false, 1><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        return check_launch("skinny_stream_kernel");
    }
    if (ktail) {
        if (p.M <= 8) skinny_stream_kernel<true, false, 1, 1, 16, true><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        else skinny_stream_kernel<true, false, 2, 1, 16, true><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
        return check_launch("skinny_stream_kernel");
    }
    if (whole && slices && p.M <= 8) skinny_stream_kernel<true, true, 1><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (whole && slices) skinny_stream_kernel<true, true, 2><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else if (whole) skinny_stream_kernel<true, false><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    else skinny_stream_kernel<false, false><<<grid, block, 0, stream>>>(p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, t);
    return check_launch("skinny_stream_kernel");
}

}  // namespace kai
