// Skinny products (at most 16 rows of X) whose operands allow aligned 128-bit loads:
//
//   y[m,n] (=|+=) act( sum_k x[m,k] * w[n,k] + bias[n] ),   m < M <= 16
//
// A workgroup of eight waves owns 16 rows of W and all of K; wave w owns the slices of 512 reduction
// steps number w, w+8, ...  Everything up to the final sum is private to a wave, so there is no
// barrier in the stream: a wave loads its slice tile by tile (16 x 128 of W and of X, 512 contiguous
// bytes per row and load; rows of X beyond M are not loaded), W three tiles and X two tiles ahead of
// the tile it is working on, and passes both through its own LDS tiles into the operand layout of
// v_mfma_f32_16x16x4_f32 (row = lane % 16, k group = lane / 16).  Loading in operand layout directly
// would touch 64 bytes per row and load, which costs a third of the bandwidth.  The matrix core only
// removes the per-row wave reductions and the X broadcasts a vector-ALU version would need; the
// kernel is bound by HBM.  The eight partial 16 x 16 results meet in LDS once, in wave order.
#include "gemv_skinny.h"

#include "act_funcs.h"

namespace kai {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSsWaves = 8;
constexpr int kSsThreads = 64 * kSsWaves;
constexpr int kSsSlice = 512;                 // reduction steps per wave and pass of the pipeline: four tiles
constexpr int kSsTileK = 128;                 // k per staged tile: 512 contiguous bytes per row
constexpr int kSsTileStride = kSsTileK + 4;
constexpr int kSsLoadsPerTile = 16 * kSsTileK / 4 / 64;   // 128-bit loads per lane and tile: 8

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

__global__ void __launch_bounds__(kSsThreads) skinny_stream_kernel(const SkinnyParams p) {
    __shared__ __attribute__((aligned(16))) float lds_w[kSsWaves][16 * kSsTileStride];
    __shared__ __attribute__((aligned(16))) float lds_x[kSsWaves][16 * kSsTileStride];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15;    // row of W inside the block's 16 / row of X
    const int g = lane >> 4;    // k group of the MFMA operand
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int lrow = lane >> 5;          // a load covers 2 rows x 128 k
    const int lk = (lane & 31) * 4;
    float* tw = lds_w[wave];
    float* tx = lds_x[wave];

    // rows of X that are never loaded stay zero in the tile
#pragma unroll
    for (int j = 0; j < kSsLoadsPerTile; j++)
        *reinterpret_cast<f32x4*>(tx + (2 * j + lrow) * kSsTileStride + lk) = f32x4{0.f, 0.f, 0.f, 0.f};

    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    // One tile = 16 rows x 128 k of W and of X, eight 128-bit loads per lane each.  Addresses past K are
    // clamped into the row (every load is unconditional); what they return is zeroed on the way to LDS.
    auto load_w = [&](f32x4(&dst)[kSsLoadsPerTile], int kt) {
#pragma unroll
        for (int j = 0; j < kSsLoadsPerTile; j++) {
            const int64_t n = n0 + 2 * j + lrow;
            const float* src = p.W + (n < p.N ? n : p.N - 1) * p.ldw + min(kt + lk, p.K - 4);
            dst[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src));
        }
    };
    auto load_x = [&](f32x4(&dst)[kSsLoadsPerTile], int kt) {
#pragma unroll
        for (int j = 0; j < kSsLoadsPerTile; j++) {
            if (2 * j < p.M) {   // uniform: this pair of rows holds a row of X
                const int m = 2 * j + lrow;
                dst[j] = *reinterpret_cast<const f32x4*>(p.X + (int64_t)min(m, p.M - 1) * p.ldx + min(kt + lk, p.K - 4));
            }
        }
    };
    auto consume = [&](const f32x4(&w)[kSsLoadsPerTile], const f32x4(&x)[kSsLoadsPerTile], int kt) {
        if (kt < p.K) {   // uniform
#pragma unroll
            for (int j = 0; j < kSsLoadsPerTile; j++) {
                const int64_t n = n0 + 2 * j + lrow;
                *reinterpret_cast<f32x4*>(tw + (2 * j + lrow) * kSsTileStride + lk) = keep_if(w[j], n < p.N && kt + lk < p.K);
                if (2 * j < p.M)
                    *reinterpret_cast<f32x4*>(tx + (2 * j + lrow) * kSsTileStride + lk) =
                        keep_if(x[j], 2 * j + lrow < p.M && kt + lk < p.K);
            }
            __builtin_amdgcn_wave_barrier();   // LDS serves a wave's accesses in order; the compiler must too
#pragma unroll
            for (int s = 0; s < kSsTileK / 16; s++) {
                const f32x4 wv = *reinterpret_cast<const f32x4*>(tw + r * kSsTileStride + 16 * s + 4 * g);
                const f32x4 xv = *reinterpret_cast<const f32x4*>(tx + r * kSsTileStride + 16 * s + 4 * g);
#pragma unroll
                for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[e], wv[e], acc, 0, 0, 0);
            }
            __builtin_amdgcn_wave_barrier();
        }
    };
    // Software pipeline over the four tiles of a slice: W runs three tiles ahead (it comes from HBM), X two
    // (it comes from L2), so the stream of a wave goes on while the wave passes a tile through LDS and the
    // matrix core.  Loads return in order, which is why the X tile is issued before the W tile that follows it.
    for (int k0 = wave * kSsSlice; k0 < p.K; k0 += kSsWaves * kSsSlice) {
        f32x4 w0[kSsLoadsPerTile], w1[kSsLoadsPerTile], w2[kSsLoadsPerTile];
        f32x4 x0[kSsLoadsPerTile], x1[kSsLoadsPerTile];
        load_w(w0, k0);
        load_x(x0, k0);
        load_w(w1, k0 + kSsTileK);
        load_x(x1, k0 + kSsTileK);
        load_w(w2, k0 + 2 * kSsTileK);
        __builtin_amdgcn_sched_barrier(0);
        consume(w0, x0, k0);
        __builtin_amdgcn_sched_barrier(0);
        load_x(x0, k0 + 2 * kSsTileK);
        load_w(w0, k0 + 3 * kSsTileK);
        __builtin_amdgcn_sched_barrier(0);
        consume(w1, x1, k0 + kSsTileK);
        __builtin_amdgcn_sched_barrier(0);
        load_x(x1, k0 + 3 * kSsTileK);
        __builtin_amdgcn_sched_barrier(0);
        consume(w2, x0, k0 + 2 * kSsTileK);
        __builtin_amdgcn_sched_barrier(0);
        consume(w0, x1, k0 + 3 * kSsTileK);
    }

    // acc[v] = D[m = 4 * g + v][n = n0 + r]; the tiles are free now: wave w parks its result in its W tile
    __syncthreads();
#pragma unroll
    for (int v = 0; v < 4; v++) tw[(4 * g + v) * 16 + r] = acc[v];
    __syncthreads();
    if (tid < 256) {
        const int m = tid >> 4, j = tid & 15;
        const int64_t n = n0 + j;
        if (m < p.M && n < p.N) {
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < kSsWaves; i++) v += lds_w[i][tid];
            const float leaky = p.leaky ? *p.leaky : 0.f;
            const int64_t idx = (int64_t)m * p.ldy + n;
            if (p.accflag) v += p.Y[idx];
            if (p.bias) v += p.bias[n];
            if (p.Y2) p.Y2[idx] = v;
            p.Y[idx] = apply_act(v, p.act, leaky);
        }
    }
}

}  // namespace

bool skinny_stream_applies(const SkinnyParams& p) {
    return p.M >= 1 && p.M <= kSkinnyMaxRows && p.K >= 64 && p.K % 4 == 0 && p.ldw % 4 == 0 && p.ldx % 4 == 0 &&
           aligned16(p.W) && aligned16(p.X);
}

int launch_skinny_stream(const SkinnyParams& p, hipStream_t stream) {
    const int64_t blocks = (p.N + 15) / 16;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: too many output columns");
    skinny_stream_kernel<<<dim3((unsigned)blocks), dim3(kSsThreads), 0, stream>>>(p);
    return check_launch("skinny_stream_kernel");
}

}  // namespace kai
