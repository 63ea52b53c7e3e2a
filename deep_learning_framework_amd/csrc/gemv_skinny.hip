// Skinny products (at most 16 rows of X): bandwidth-bound streams over the weight matrix.
//
//   y[m,n] (=|+=) act( sum_k x[m,k] * w[n,k] + bias[n] ),   m < M <= 16
//
// This is VMath::matmul (vmath.cu:2961-3003 of the reference) at batch sizes where the weight
// matrix is read once and everything else is noise.  Three plans, all without a tile in LDS:
//   M == 1      gemv_rows_kernel: a wave owns whole rows, x lives in registers, 1 KiB contiguous
//               per wave load, wave-wide fold at the end (the classic wavefront-reduction GEMV)
//   M == 2..4   skinny_slice_kernel: a wave owns a 1024-wide K slice of a few rows, its slice of X
//               in registers, partial sums of the waves meet in LDS once
//   otherwise   skinny_mfma_kernel: the same stream with the multiply on the matrix core; at 5..16
//               rows the vector ALU would need 8 LDS bytes of X per byte of W and become LDS-bound.
//               It is also the plan for unaligned or ragged skinny operands (scalar loads).
#include "gemv_skinny.h"

#include "act_funcs.h"

namespace kai {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSkinnyThreads = 256;

// Sum over the 64 lanes of a wave, returned to every lane.  Cross-lane moves go through the DPP
// data path (a few cycles each) instead of LDS permutes: the fold sits on the critical path at the
// end of a kernel whose whole run time is ~10 us.
//   quad_perm [1,0,3,2] and [2,3,0,1]   -> every lane of a quad holds the quad sum
//   row_half_mirror, row_mirror        -> every lane of a row of 16 holds the row sum
//   row_bcast:15 (rows 1,3), row_bcast:31 (rows 2,3) -> lane 63 holds the wave sum
__device__ __forceinline__ float wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// ---- batch 1: the weight matrix streamed once, x in registers ------------------------------------
//
// One wave owns R whole rows of W.  K is walked in chunks of 4096: a lane issues the 16 128-bit
// loads of each of its rows for the chunk (R*16 KiB in flight per wave) and its 16 float4 of x (they
// hit in L2), then multiplies as the loads arrive.  W is read with the non-temporal hint: it is used
// once and should not displace x from the caches.  No LDS, no barrier.  K == 4096 is a kernel of its
// own (K4096), so that the common inference width is straight-line code from the entry point.

// amdgpu_waves_per_eu(1, 2): two waves per SIMD are all the grid ever gives a CU, so the register
// allocator is told not to trade loads in flight for an occupancy it cannot use.
// THREADS: 256, or 128 / 64 where 256-thread workgroups would not cover the compute units (1024 x 4096: 128
// workgroups 5.06 us, 256 of 128 threads 4.5)
template <int R, bool K4096, int THREADS>
__global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 2)))
gemv_rows_kernel(const float* __restrict__ W, const float* __restrict__ X, const int64_t ldw, const int64_t N,
                 const int K, const int act_acc, float* __restrict__ Y, const float* __restrict__ bias,
                 float* __restrict__ Y2, const float* __restrict__ leaky_ptr) {
    // The arguments are scalars in the order of their first use, not a struct: this file is compiled with
    // kernel-argument preload, so the first 14 dwords (W .. bias) are in SGPRs when a wave starts and the
    // first loads of W go out without a round trip to the argument buffer.
    const struct { const float *W, *X; int64_t ldw, N; int K, act, accflag; float *Y, *Y2; const float *bias, *leaky; }
        p = {W, X, ldw, N, K, act_acc & 0xff, act_acc >> 8, Y, Y2, bias, leaky_ptr};
    constexpr int CH = 16;   // float4 per lane per chunk of 4096 k
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t n0 = ((int64_t)blockIdx.x * (THREADS / 64) + wave) * R;
    // rows past the end are clamped to the last row (loaded, never stored): no early exit, so the
    // kernel arguments are fetched in one round trip and the first loads go out at once
    const float* __restrict__ wrow[R];
#pragma unroll
    for (int r = 0; r < R; r++) wrow[r] = p.W + ((n0 + r < p.N) ? (n0 + r) : (p.N - 1)) * p.ldw;

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    // One whole chunk of 4096 k.  The order of issue is pinned, because it decides the run time at 4096 x 4096
    // (us per call, cold): the loads of row 0 paired with those of x, then row 1, every load of the chunk out
    // before the first wait, the multiplies following the arrivals 10.9 - 11.0; the rows' loads first and x last
    // (the compiler then holds back the last 12 loads until the first ones return) 11.25; rows then x with all
    // loads out first 11.50; x first 12.0; the two rows interleaved 11.7; all loads and one wait 12.2.
    auto full_chunk = [&](int kc) {
        const int kbase = kc + 4 * lane;
        f32x4 w[R][CH];
        f32x4 x[CH];
#pragma unroll
        for (int j = 0; j < CH; j++) {
            w[0][j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wrow[0] + kbase + 256 * j));
            x[j] = *reinterpret_cast<const f32x4*>(p.X + kbase + 256 * j);
        }
#pragma unroll
        for (int r = 1; r < R; r++)
#pragma unroll
            for (int j = 0; j < CH; j++)
                w[r][j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wrow[r] + kbase + 256 * j));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < CH; j++)
                acc[r] += w[r][j][0] * x[j][0] + w[r][j][1] * x[j][1] + w[r][j][2] * x[j][2] + w[r][j][3] * x[j][3];
    };

    // The same chunk as 16 segments of 256 steps that start at segment seg0 of the row's nseg whole ones and wrap
    // round (rows a multiple of 32 KiB apart, below)
    auto wrapped_chunk = [&](int seg0, int nseg) {
        f32x4 w[R][CH];
        f32x4 x[CH];
        int koff[CH];
#pragma unroll
        for (int j = 0; j < CH; j++) {
            int sg = seg0 + j;
            if (sg >= nseg) sg -= nseg;
            koff[j] = 256 * sg + 4 * lane;
        }
#pragma unroll
        for (int j = 0; j < CH; j++) {
            w[0][j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wrow[0] + koff[j]));
            x[j] = *reinterpret_cast<const f32x4*>(p.X + koff[j]);
        }
#pragma unroll
        for (int r = 1; r < R; r++)
#pragma unroll
            for (int j = 0; j < CH; j++)
                w[r][j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wrow[r] + koff[j]));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < CH; j++)
                acc[r] += w[r][j][0] * x[j][0] + w[r][j][1] * x[j][1] + w[r][j][2] * x[j][2] + w[r][j][3] * x[j][3];
    };

    if constexpr (K4096) {
        full_chunk(0);
    } else {
        // whole chunks, each wave starting at a place of its own and wrapping round: with rows a large power of
        // two apart, waves that all walk their rows from k = 0 keep meeting in the same HBM channels.  Rows a
        // multiple of 32 KiB apart: the start moves in steps of 4 KiB (8192 x 8192: 50 us from k = 0, 44.5 with a
        // chunk of 4096 steps as the unit, 41.3 with 4 KiB; 4096 x 8192: 24.1 -> 22.6, 4096 x 16384: 43.9 -> 41.4).
        // Other lengths keep whole chunks as the unit (5120 x 5120: 20.4 us against 21.2 with the finer one).
        const int nfull = p.K / (256 * CH);
        const int wave_id = (int)(blockIdx.x * (THREADS / 64) + wave);
        if (nfull > 1 && p.ldw % 8192 == 0) {
            const int nseg = nfull * CH;
            int seg = (wave_id * 4) % nseg;
            for (int i = 0; i < nfull; i++) {
                wrapped_chunk(seg, nseg);
                seg += CH;
                if (seg >= nseg) seg -= nseg;
            }
        } else {
            const int first = nfull > 1 ? wave_id % nfull : 0;
            for (int i = 0; i < nfull; i++) {
                int c = first + i;
                if (c >= nfull) c -= nfull;
                full_chunk(c * 256 * CH);
            }
        }
        const int kc = nfull * 256 * CH;
        if (kc < p.K) {
            // last, partial chunk: K % 4 == 0, so a float4 is entirely inside or outside
            const int kbase = kc + 4 * lane;
#pragma unroll
            for (int j = 0; j < CH; j++) {
                const int k = kbase + 256 * j;
                if (k < p.K) {
                    const f32x4 x = *reinterpret_cast<const f32x4*>(p.X + k);
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const f32x4 wv = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wrow[r] + k));
                        acc[r] += wv[0] * x[0] + wv[1] * x[1] + wv[2] * x[2] + wv[3] * x[3];
                    }
                }
            }
        }
    }

    const float leaky = p.leaky ? *p.leaky : 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        float v = wave_sum(acc[r]);
        if (lane == r && n0 + r < p.N) {
            const int64_t n = n0 + r;
            if (p.accflag) v += p.Y[n];
            if (p.bias) v += p.bias[n];
            if (p.Y2) p.Y2[n] = v;
            p.Y[n] = apply_act(v, p.act, leaky);
        }
    }
}

template <int THREADS>
static void launch_gemv_rows_threads(const SkinnyParams& p, int64_t blocks, int act_acc, hipStream_t stream) {
    constexpr int R = 2;
    if (p.K == 4096)
        gemv_rows_kernel<R, true, THREADS><<<dim3((unsigned)blocks), dim3(THREADS), 0, stream>>>(
            p.W, p.X, p.ldw, p.N, p.K, act_acc, p.Y, p.bias, p.Y2, p.leaky);
    else
        gemv_rows_kernel<R, false, THREADS><<<dim3((unsigned)blocks), dim3(THREADS), 0, stream>>>(
            p.W, p.X, p.ldw, p.N, p.K, act_acc, p.Y, p.bias, p.Y2, p.leaky);
}

static int launch_gemv_rows(const SkinnyParams& p, hipStream_t stream) {
    constexpr int R = 2;
    int threads = kSkinnyThreads;
    while (threads > 64 && (p.N + (threads / 64) * R - 1) / ((threads / 64) * R) < compute_units()) threads /= 2;
    const int64_t rows_per_block = (threads / 64) * R;
    const int64_t blocks = (p.N + rows_per_block - 1) / rows_per_block;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: too many output columns");
    const int act_acc = (p.act & 0xff) | (p.accflag ? 0x100 : 0);
    if (threads == 256) launch_gemv_rows_threads<256>(p, blocks, act_acc, stream);
    else if (threads == 128) launch_gemv_rows_threads<128>(p, blocks, act_acc, stream);
    else launch_gemv_rows_threads<64>(p, blocks, act_acc, stream);
    return check_launch("gemv_rows_kernel");
}

// ---- 2 to 4 rows of X: a workgroup owns RB rows of W, each wave one 1024-wide slice of K ----------
//
// The slice of X a wave needs (MT x 1024 floats) stays in its registers for all RB rows; the RB*4
// loads of W per lane are issued back to back; the per-wave partial sums meet in LDS once, at the
// end.  K beyond waves*1024 is covered by further passes of the same wave.

constexpr int kSliceK = 1024;
constexpr int kSliceMaxWaves = 4;   // 256 threads: leaves each wave 256 registers

template <int MT, int RB>
__global__ void __launch_bounds__(64 * kSliceMaxWaves) skinny_slice_kernel(
        const float* __restrict__ W, const float* __restrict__ X, const int64_t ldw, const int64_t ldx,
        const int64_t N, const int M, const int K, float* __restrict__ Y, const SkinnyTail tail, int waves) {
    const SkinnyParams p = skinny_params(W, X, ldw, ldx, N, M, K, Y, tail);
    __shared__ float part[MT * RB][kSliceMaxWaves];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t n0 = (int64_t)blockIdx.x * RB;
    const float* __restrict__ wrow[RB];
#pragma unroll
    for (int r = 0; r < RB; r++) wrow[r] = p.W + ((n0 + r < p.N) ? (n0 + r) : n0) * p.ldw;

    float acc[MT][RB];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int r = 0; r < RB; r++) acc[m][r] = 0.f;

    for (int ks = wave * kSliceK; ks < p.K; ks += waves * kSliceK) {
        f32x4 w[RB][4];
        f32x4 x[MT][4];
        // addresses are clamped into the row and the values masked afterwards (bitwise), so that no
        // branch separates the loads
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int k = min(ks + 4 * lane + 256 * j, p.K - 4);
#pragma unroll
            for (int r = 0; r < RB; r++) w[r][j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wrow[r] + k));
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int k = min(ks + 4 * lane + 256 * j, p.K - 4);
#pragma unroll
            for (int m = 0; m < MT; m++)
                x[m][j] = *reinterpret_cast<const f32x4*>(p.X + (int64_t)min(m, p.M - 1) * p.ldx + k);
        }
        __builtin_amdgcn_sched_barrier(0);   // all loads of the pass are in flight before the first multiply
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int keep_k = (ks + 4 * lane + 256 * j < p.K) ? -1 : 0;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const int keep = (m < p.M) ? keep_k : 0;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float v = x[m][j][e];
                    x[m][j][e] = __int_as_float(__float_as_int(v) & keep);
                }
            }
            // W beyond K meets the zeros of X, but may hold anything: inf * 0 must not reach the sum
#pragma unroll
            for (int r = 0; r < RB; r++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float v = w[r][j][e];
                    w[r][j][e] = __int_as_float(__float_as_int(v) & keep_k);
                }
        }
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int r = 0; r < RB; r++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[m][r] += w[r][j][0] * x[m][j][0] + w[r][j][1] * x[m][j][1] + w[r][j][2] * x[m][j][2] +
                                 w[r][j][3] * x[m][j][3];
    }

#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const float v = wave_sum(acc[m][r]);
            if (lane == 0) part[m * RB + r][wave] = v;
        }
    __syncthreads();
    const int t = threadIdx.x;
    if (t < MT * RB) {
        const int m = t / RB, r = t % RB;
        if (m < p.M && n0 + r < p.N) {
            float v = 0.f;
            for (int i = 0; i < waves; i++) v += part[t][i];
            const float leaky = p.leaky ? *p.leaky : 0.f;
            const int64_t n = n0 + r;
            const int64_t idx = (int64_t)m * p.ldy + n;
            if (p.accflag) v += p.Y[idx];
            if (p.bias) v += p.bias[n];
            if (p.Y2) p.Y2[idx] = v;
            p.Y[idx] = apply_act(v, p.act, leaky);
        }
    }
}

// The same plan with X shared through LDS: sixteen waves = four row groups x four K slices, so the workgroup
// owns 16 rows of W and fetches X (MT x K floats, at most 64 KiB) once instead of once per four rows (with four
// rows per workgroup the slices of X re-read from L2 are as many bytes as W itself).  K <= 4096: one slice per wave.
// Measured at 4 x 4096 x 4096: 16.4 -> 15.6 us.  A wall-clock trace of the phases shows why it is not more: the
// X loads of the later waves queue behind the HBM misses of the earlier ones in the CU's memory pipeline, so the
// barrier after the LDS copy opens only when most of the stream has arrived (8.3 us) and the arithmetic (3 us of
// vector ALU work at 4 rows) follows it.  Copying X first and starting the stream after the barrier measured
// 16.2 us; a wave per whole row with X in LDS does not fit the registers of a 16-wave workgroup.
constexpr int kSliceLdsK = 4096;
constexpr int kSliceLdsGroups = 4;

template <int MT>
__global__ void __launch_bounds__(64 * kSliceMaxWaves * kSliceLdsGroups) skinny_slice_lds_kernel(
        const float* __restrict__ W, const float* __restrict__ X, const int64_t ldw, const int64_t ldx,
        const int64_t N, const int M, const int K, float* __restrict__ Y, const SkinnyTail tail) {
    const SkinnyParams p = skinny_params(W, X, ldw, ldx, N, M, K, Y, tail);
    constexpr int RB = 4;
    __shared__ __attribute__((aligned(16))) float xs[MT * kSliceLdsK];
    __shared__ float part[kSliceLdsGroups][MT * RB][kSliceMaxWaves];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int rg = wave >> 2, sl = wave & 3;
    const int64_t n0 = (int64_t)blockIdx.x * (RB * kSliceLdsGroups) + rg * RB;
    const int ks = sl * kSliceK;

    // this wave's slice of its four rows of W (HBM), then the workgroup's copy of X (L2)
    f32x4 w[RB][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int k = min(ks + 4 * lane + 256 * j, p.K - 4);
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const int64_t row = (n0 + r < p.N) ? (n0 + r) : (p.N - 1);
            w[r][j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p.W + row * p.ldw + k));
        }
    }
    {
        // two rows of X at a time: with four in flight next to the sixteen chunks of W a wave of this 16-wave
        // workgroup ran out of its 128 registers
        constexpr int XB = MT < 2 ? MT : 2;
        const int k = min(4 * tid, p.K - 4);
#pragma unroll
        for (int m0 = 0; m0 < MT; m0 += XB) {
            f32x4 xv[XB];
#pragma unroll
            for (int m = 0; m < XB; m++)
                xv[m] = *reinterpret_cast<const f32x4*>(p.X + (int64_t)min(m0 + m, p.M - 1) * p.ldx + k);
#pragma unroll
            for (int m = 0; m < XB; m++) {
                const int keep = (m0 + m < p.M && 4 * tid < p.K) ? -1 : 0;   // rows beyond M and steps beyond K read as zero
                f32x4 z;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float v = xv[m][e];
                    z[e] = __int_as_float(__float_as_int(v) & keep);
                }
                *reinterpret_cast<f32x4*>(&xs[(m0 + m) * kSliceLdsK + 4 * tid]) = z;
            }
        }
    }
    __syncthreads();

    // W beyond K meets the zeros of X, but may hold anything: inf * 0 must not reach the sum
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int keep_k = (ks + 4 * lane + 256 * j < p.K) ? -1 : 0;
#pragma unroll
        for (int r = 0; r < RB; r++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float v = w[r][j][e];
                w[r][j][e] = __int_as_float(__float_as_int(v) & keep_k);
            }
    }
    // one row of X at a time, fenced: with the rows interleaved the sixteen chunks of W, the chunks of X of several
    // rows and sixteen sums did not fit the 128 registers a wave of this 16-wave workgroup has
#pragma unroll
    for (int m = 0; m < MT; m++) {
        float acc[RB];
#pragma unroll
        for (int r = 0; r < RB; r++) acc[r] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int kk = ks + 4 * lane + 256 * j;           // < 4096: inside xs (zeros beyond K)
            const f32x4 x = *reinterpret_cast<const f32x4*>(&xs[m * kSliceLdsK + kk]);
#pragma unroll
            for (int r = 0; r < RB; r++)
                acc[r] += w[r][j][0] * x[0] + w[r][j][1] * x[1] + w[r][j][2] * x[2] + w[r][j][3] * x[3];
        }
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const float v = wave_sum(acc[r]);
            if (lane == 0) part[rg][m * RB + r][sl] = v;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    if (tid < kSliceLdsGroups * MT * RB) {
        const int g = tid / (MT * RB), t = tid % (MT * RB);
        const int m = t / RB, r = t % RB;
        const int64_t n = (int64_t)blockIdx.x * (RB * kSliceLdsGroups) + g * RB + r;
        if (m < p.M && n < p.N) {
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < kSliceMaxWaves; i++) v += part[g][t][i];
            const float leaky = p.leaky ? *p.leaky : 0.f;
            const int64_t idx = (int64_t)m * p.ldy + n;
            if (p.accflag) v += p.Y[idx];
            if (p.bias) v += p.bias[n];
            if (p.Y2) p.Y2[idx] = v;
            p.Y[idx] = apply_act(v, p.act, leaky);
        }
    }
}

template <int MT>
static int launch_slice(const SkinnyParams& p, hipStream_t stream) {
    constexpr int RB = 4;
    if (p.K <= kSliceLdsK && p.K > 3 * kSliceK && p.N >= 16 * 64) {
        // every wave has a slice, and there are workgroups for a good part of the chip
        const int64_t blocks = (p.N + RB * kSliceLdsGroups - 1) / (RB * kSliceLdsGroups);
        if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: too many output columns");
        skinny_slice_lds_kernel<MT><<<dim3((unsigned)blocks), dim3(64 * kSliceMaxWaves * kSliceLdsGroups), 0, stream>>>(
            p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, skinny_tail(p));
        return check_launch("skinny_slice_lds_kernel");
    }
    int waves = (p.K + kSliceK - 1) / kSliceK;
    if (waves < 1) waves = 1;
    if (waves > kSliceMaxWaves) waves = kSliceMaxWaves;
    const int64_t blocks = (p.N + RB - 1) / RB;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: too many output columns");
    skinny_slice_kernel<MT, RB><<<dim3((unsigned)blocks), dim3(64 * waves), 0, stream>>>(
        p.W, p.X, p.ldw, p.ldx, p.N, p.M, p.K, p.Y, skinny_tail(p), waves);
    return check_launch("skinny_slice_kernel");
}

// ---- up to 16 rows of X through the matrix core, still as a stream over W ---------------------------
//
// A workgroup of 8 waves owns 16 rows of W; wave w owns the w-th eighth of K.  Per step of 16 k a lane
// loads one float4 of W (row lane%16, k offset 4*(lane/16)) and the float4 of X at the same (row, k):
// exactly the operand layout of v_mfma_f32_16x16x4_f32 when element t of both float4 feeds step t,
// so four MFMAs consume the step with no shuffles, no LDS and no per-row scalar work.  X rows beyond
// M read as zeros.  The eight partial 16x16 results meet in LDS once, at the end.  The multiply
// itself is 3 % of what the matrix core could do at this byte rate: the kernel is bound by HBM like
// the other skinny kernels; with the vector ALU the same product needs 8 LDS bytes per byte of W at
// 16 rows and is LDS-bound at a quarter of the bandwidth.

typedef float f32x4v __attribute__((ext_vector_type(4)));
constexpr int kMmWaves = 8;
constexpr int kMmUnroll = 16;  // steps of 16 k (1 KiB of W and of X each) per chunk

// LOADS: 1 = 128-bit loads of operands whose rows start on 16-byte lines (K, ldw, ldx multiples of 4); 2 = 128-bit
// BUFFER loads, which need 4-byte alignment only, for every other operand (K = 4095, rows of 769 floats: element by
// element these took 26.5 us for 4096 x 4095 where 4096 x 4096 takes 12); what such a load reads past the end of a
// row is masked like before, past the end of the matrix the buffer returns zeros; 0 = element by element (rows too
// long for a buffer's 32-bit offsets).
// CHUNK: steps of 16 k whose loads a wave issues together (0: 16 with 128-bit loads, 8 element by element); a wave's
// share of a short row is a few steps, and a chunk is loaded whole (50257 x 769: 7 steps per wave).
template <int LOADS, int CHUNK = 0>
__global__ void __launch_bounds__(64 * kMmWaves) skinny_mfma_kernel(const SkinnyParams p) {
    constexpr bool VEC = LOADS != 0;
    __shared__ float part[kMmWaves][256];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15;    // row of W inside the block's 16 / row of X
    const int g = lane >> 4;    // k group
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const bool wvalid = n0 + r < p.N;
    const bool xvalid = r < p.M;
    const float* __restrict__ wp = p.W + (wvalid ? (n0 + r) : 0) * p.ldw;
    const float* __restrict__ xp = p.X + (int64_t)(xvalid ? r : 0) * p.ldx;

    // K split into 8 contiguous slices of whole 16-k steps
    const int steps = (p.K + 15) / 16;
    const int per = (steps + kMmWaves - 1) / kMmWaves;
    const int s_begin = wave * per;
    const int s_end = min(steps, s_begin + per);

    f32x4v acc = {0.f, 0.f, 0.f, 0.f};
    // Loads are raw: the address is clamped into the row, so that no branch sits between the loads
    // of a chunk and all of them are in flight together.  What lies beyond the row, the slice or the
    // matrix is zeroed when the value is consumed (bitwise, so that the load stays unconditional).
    // (the buffers start at the workgroup's first row of W and at X; offsets fit 32 bits, the host has checked)
    const int64_t w_bytes = ((p.N - 1 - min(n0, p.N - 1)) * p.ldw + p.K) * 4, x_bytes = ((int64_t)(p.M - 1) * p.ldx + p.K) * 4;
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(p.W + n0 * p.ldw), 0, (int)min(w_bytes, (int64_t)0x7FFFFFFF), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(p.X), 0, (int)min(x_bytes, (int64_t)0x7FFFFFFF), 0x00020000);
    const int w_row_off = (int)(r * p.ldw) * 4, x_row_off = (int)(r * p.ldx) * 4;
    auto load4 = [&](auto of_w, int k) -> f32x4v {
        constexpr bool kOfW = decltype(of_w)::value;
        const float* base = kOfW ? wp : xp;
        f32x4v v;
        if (LOADS == 2) {
            v = __builtin_bit_cast(f32x4v, __builtin_amdgcn_raw_buffer_load_b128(kOfW ? rsrc_w : rsrc_x,
                                                                                  (kOfW ? w_row_off : x_row_off) + k * 4, 0, 0));
        } else if (VEC) {
            // K % 4 == 0: the float4 at k is entirely inside or outside
            v = *reinterpret_cast<const f32x4v*>(base + min(k, p.K - 4));
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = base[min(k + j, p.K - 1)];
        }
        return v;
    };
    auto masked = [&](f32x4v v, int k, bool valid) -> f32x4v {
        f32x4v o;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int keep = (valid && k + j < p.K) ? -1 : 0;
            const float e = v[j];
            o[j] = __int_as_float(__float_as_int(e) & keep);
        }
        return o;
    };

    // chunks of kMmUnroll steps: all loads of W and of X of a chunk are issued back to back (32 KiB in
    // flight per wave), then its MFMAs; the second wave of the SIMD computes meanwhile
    // (element-wise loads, 128 of them per chunk of 16 steps with an address each, do not fit the registers:
    // chunks of 8 steps there)
    constexpr int UN = CHUNK ? CHUNK : VEC ? kMmUnroll : kMmUnroll / 2;   // (VEC: both kinds of 128-bit loads)
    for (int base = s_begin; base < s_end; base += UN) {
        f32x4v w[UN], x[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) w[u] = load4(std::true_type{}, (base + u) * 16 + 4 * g);
#pragma unroll
        for (int u = 0; u < UN; u++) x[u] = load4(std::false_type{}, (base + u) * 16 + 4 * g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int k = (base + u) * 16 + 4 * g;
            const bool in = base + u < s_end;   // steps past the end of the slice add nothing
            const f32x4v wv = masked(w[u], k, wvalid && in);
            const f32x4v xv = masked(x[u], k, xvalid && in);
#pragma unroll
            for (int t = 0; t < 4; t++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[t], wv[t], acc, 0, 0, 0);
        }
    }

    // acc[v] = D[m = 4*(lane/16) + v][n = lane%16]
#pragma unroll
    for (int v = 0; v < 4; v++) part[wave][(4 * g + v) * 16 + r] = acc[v];
    __syncthreads();
    const int t = threadIdx.x;
    if (t < 256) {
        const int m = t >> 4, j = t & 15;
        if (m < p.M && n0 + j < p.N) {
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < kMmWaves; i++) v += part[i][t];
            const float leaky = p.leaky ? *p.leaky : 0.f;
            const int64_t n = n0 + j;
            const int64_t idx = (int64_t)m * p.ldy + n;
            if (p.accflag) v += p.Y[idx];
            if (p.bias) v += p.bias[n];
            if (p.Y2) p.Y2[idx] = v;
            p.Y[idx] = apply_act(v, p.act, leaky);
        }
    }
}

static int launch_skinny_mfma(const SkinnyParams& p, bool vec, hipStream_t stream) {
    const int64_t blocks = (p.N + 15) / 16;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: too many output columns");
    // 16 rows of W (and of X) and the chunks loaded past a row's end within a buffer's 31-bit offsets
    const bool buffers = (16 * p.ldw + p.K + 1024) * 4 < (1ll << 31) && (16 * p.ldx + p.K + 1024) * 4 < (1ll << 31);
    if (vec)
        skinny_mfma_kernel<1><<<dim3((unsigned)blocks), dim3(64 * kMmWaves), 0, stream>>>(p);
    else if (buffers && p.K <= 4 * 16 * kMmWaves)
        skinny_mfma_kernel<2, 4><<<dim3((unsigned)blocks), dim3(64 * kMmWaves), 0, stream>>>(p);
    else if (buffers && p.K <= 8 * 16 * kMmWaves)
        skinny_mfma_kernel<2, 8><<<dim3((unsigned)blocks), dim3(64 * kMmWaves), 0, stream>>>(p);
    else if (buffers)
        skinny_mfma_kernel<2><<<dim3((unsigned)blocks), dim3(64 * kMmWaves), 0, stream>>>(p);
    else
        skinny_mfma_kernel<0><<<dim3((unsigned)blocks), dim3(64 * kMmWaves), 0, stream>>>(p);
    return check_launch("skinny_mfma_kernel");
}

int launch_skinny_nt(const SkinnyParams& p, hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0) return KAI_OK;
    if (p.M > kSkinnyMaxRows) {
        if (skinny_stream32_applies(p)) return launch_skinny_stream(p, stream);
        return fail(KAI_ERR_INVALID_ARGUMENT, "skinny matmul: more than 16 rows");
    }
    const bool vec = p.K % 4 == 0 && p.ldw % 4 == 0 && p.ldx % 4 == 0 && aligned16(p.W) && aligned16(p.X);
    if (vec && p.K >= 256) {
        if (p.M == 1) {
            // The batch-1 kernel walks K in chunks of 4096 with all of a chunk's loads in flight; a chunk that K does
            // not fill is loaded all the same (clamped), so it is the kernel for K in whole chunks only.  Other K:
            // the slice kernel with one row of X (slices of 1024), us per call with W from HBM, 5120 x 2048
            // 14.8 -> 8.7, 8192 x 2048 17.4 -> 11.8, 5120 x 3072 18.2 -> 11.3, 4096 x 11008 31.7 -> 29.3, 1024 x 11008
            // 14.2 -> 9.9, 11008 x 5120 37.3 -> 33.1 (K = 1024 .. 11008: 7..69 %); rows shorter than a slice, and
            // K = 1024 up to 8 rows of W per compute unit, through the streaming kernel (2048 x 512 5.5 -> 4.1,
            // 1024 x 1024 5.4 -> 4.5; matrices of up to 24 MB only: 50257 x 768 takes 35 us there and 24 in slices).
            // K in whole chunks: 4096 x 4096 11.3 against 11.7 / 12.2, 5120 x 4096 14.4
            // against 17.0 / 17.5.
            if (p.K % 4096 == 0) return launch_gemv_rows(p, stream);
            if ((p.K < kSliceK || (p.K == kSliceK && p.N <= 8 * (int64_t)compute_units())) && p.N * p.K <= (6ll << 20) &&
                skinny_stream_applies(p))
                return launch_skinny_stream(p, stream);
            return launch_slice<1>(p, stream);
        }
        if (skinny_stream8_applies(p)) return launch_skinny_stream8(p, stream);
        // 2..4 rows: the streaming kernel (16 rows of W per workgroup) or the slice kernels (8 rows per workgroup,
        // a second round of workgroups beyond 8 rows per compute unit).  Measured, us per call with W from HBM,
        // slice kernel -> streaming kernel:
        //   * N >= 16 per compute unit: 3 and 4 rows 4096 x 4096 16.0 -> 12.6, 11008 x 4096 40 -> 30; 2 rows where
        //     the streaming kernel's slices are written out (K a multiple of 4096) 12.45 -> 12.3, 30.5 -> 29.0, else
        //     the slice kernel (4096 x 11008: 30.7 against 33.3);
        //   * more than 8 and fewer than 16 per compute unit, 3 and 4 rows: 3072 x 4096 12.4 -> 10.0, 2304 x 4096
        //     11.3 -> 9.2, 3072 x 5120 18.2 -> 13.2, 3072 x 8192 21.3 -> 19.2, 3840 x 12288 35.5 -> 30.8, 2304 x 1024
        //     6.0 -> 5.3 (every K from 1024 to 12288 by 10..38 %), except the rolled loop over long rows
        //     (K > 8192 that is not a multiple of 4096: 3072 x 11008 27.2 -> 29.3), which loses at every width, most
        //     where the last round of workgroups is partly filled (5120 x 11008 at 3 rows: slices 40.0, stream 50.3;
        //     8704 x 11008 65.2 / 78.4; 8192 x 11008 60.2 / 63.4; K = 2048, 4096 and 5120 stream 0..25 % faster at the
        //     same widths); 2 rows with K = 4096 / 8192 by 2..5 %;
        //   * 8 per compute unit and fewer: the slice kernels (2048 x 8192, 128 workgroups: 15.3 against 19.8;
        //     2048 x 3072 8.4 against 8.8) unless K <= 2048 (2048 x 2048 6.9 -> 6.4, 2048 x 1024 5.8 -> 5.3).
        const int64_t cus = compute_units();
        const bool long_rolled = p.K > 8192 && p.K % 4096 != 0;
        bool streamed = p.N >= 16 * cus && (p.M >= 3 ? !long_rolled : p.K % 4096 == 0);
        if (!streamed && p.N > 8 * cus) streamed = p.M >= 3 ? !long_rolled : (p.K % 4096 == 0 && p.K <= 8192);
        if (!streamed && p.M >= 3 && p.N == 8 * cus && p.K <= 2048) streamed = true;
        // rows of W that do not start on a 128-byte line: each of the streaming kernel's 128-byte pieces of a row
        // straddles two lines, the slice kernel's 1 KiB runs one in eight (4100 x 4100 at 4 rows: 21.8 us streamed,
        // 14.3 at 2 rows in slices)
        if (p.ldw % 32 != 0) streamed = false;
        // many short rows (a vocabulary of 50257 against 768 steps): 3142 workgroups of 48 KB each are all prologue
        // and epilogue, 38 us at 4 rows against 24 at 2 rows in slices
        if (p.K <= 1024 && p.N >= 64 * cus) streamed = false;
        if (streamed && skinny_stream_applies(p)) return launch_skinny_stream(p, stream);
        if (p.M == 2) return launch_slice<2>(p, stream);
        if (p.M <= 4) return launch_slice<4>(p, stream);
    }
    if (skinny_stream_applies(p)) return launch_skinny_stream(p, stream);
    return launch_skinny_mfma(p, vec, stream);
}

}  // namespace kai
