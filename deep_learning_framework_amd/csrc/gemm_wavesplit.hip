// Small products with a long reduction: C[M,N] (=|+=) act(alpha * sum_k A(m,k) B(n,k) + bias) for the engine's
// dense layer (VMath::matmul / matmul_backward_x / matmul_backward_w, vmath.cu:2961-3093 of the reference), when
// the output has too few tiles to fill the chip and the tiled kernel would cut K over workgroups and sum the
// parts in a second launch.  Each operand is either K-contiguous ("KC": one 128-bit load gives a lane its four k;
// rows may start at any float address) or contiguous along its output index ("MC": four 32-bit loads, the lanes
// of a row group side by side).
//
// Here the reduction is cut over the WAVES of one workgroup instead.  A workgroup owns one T x T block of C
// (T = 32 on v_mfma_f32_32x32x2_f32, T = 16 on v_mfma_f32_16x16x4_f32).  K is dealt out in rounds of
// WAVES x kWsFlight k-groups (a group = one 128-bit load per lane and operand, 8 or 16 consecutive k); in every
// round a wave takes kWsFlight of them -- consecutive ones for T = 16, every WAVES-th for T = 32, each the faster
// choice where the dispatcher uses that block size -- straight from global memory into the MFMA operands: a
// lane's four consecutive k feed four successive MFMAs, and both operands use the same lane -> k mapping, so
// products pair equal k.  No LDS staging, no barrier in the loop.  The partial blocks meet in LDS, one thread
// per output element adds them in wave order (a fixed order: results do not depend on timing) and runs the
// epilogue.  One launch, and its critical path is one wave's share of K.
#include "act_funcs.h"
#include "gemm_host.h"

namespace kai {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// four consecutive floats at any float address: global memory takes 128-bit loads at 4-byte alignment
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kWsWaves = 16;
constexpr int kWsFlight = 4;   // k-groups per wave in flight

struct WaveSplitParams {
    const float* A;       // A(m,k) = A[m*a_rs + k*a_ks]
    const float* B;       // B(n,k) = B[n*b_rs + k*b_ks]
    float* C;             // [M, N], row stride ldc
    float* C2;            // optional: value before the activation
    const float* bias;
    const float* alpha;
    const float* leaky;
    int M, N, K;
    int64_t a_rs, a_ks, b_rs, b_ks, ldc;
    int tiles_fast;       // blocks along the output dimension that consecutive workgroups walk
    int m_fast;           // ... which is M (else N)
    int act, accflag, has_alpha;
};

__device__ __forceinline__ f32x4 keep_if(f32x4 v, bool keep) {
    const int m = keep ? -1 : 0;   // bitwise: a select would put the load that produced v under the condition
    f32x4 r;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float e = v[j];
        r[j] = __int_as_float(__float_as_int(e) & m);
    }
    return r;
}

// U: k-groups per wave and round: for a reduction of up to eight groups per wave (T = 32: K <= 1024, T = 16:
// K <= 2048) exactly as many as it needs, in ONE round with every load of a wave in flight at once; else four, in
// as many rounds as K needs.
template <int T, bool A_KC, bool B_KC, int U = kWsFlight>
__global__ void __launch_bounds__(64 * kWsWaves) gemm_wavesplit_kernel(const WaveSplitParams p) {
    static_assert(T == 32 || T == 16, "block edge");
    constexpr int KG = T == 32 ? 8 : 16;        // k per group
    constexpr int NR = T == 32 ? 16 : 4;        // accumulator registers per lane
    constexpr int GS = T == 32 ? kWsWaves : 1;  // distance between a wave's groups of one round
    __shared__ float red[kWsWaves * NR * 64];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r = T == 32 ? (lane & 31) : (lane & 15);   // row of the block this lane feeds, for both operands
    const int kq = T == 32 ? (lane >> 5) : (lane >> 4);  // which 4 k of the group
    // Consecutive workgroups go round the eight XCDs: they walk along the output dimension with more blocks, so that
    // an XCD's workgroups share the whole of the smaller operand and an eighth of the larger one behind its L2 (with
    // 4 column blocks and 64 row blocks numbered column-fastest, every XCD fetched half of A: 1024 x 64 x 2048 took
    // 13.4 us against 8.7 for 64 x 1024 x 2048)
    const int slow = blockIdx.x / p.tiles_fast, fast = blockIdx.x % p.tiles_fast;
    const int tm = p.m_fast ? fast : slow, tn = p.m_fast ? slow : fast;
    const int m0 = tm * T, n0 = tn * T;
    // rows past the end are read from the last row and never stored
    const float* __restrict__ arow = p.A + (int64_t)min(m0 + r, p.M - 1) * p.a_rs;
    const float* __restrict__ brow = p.B + (int64_t)min(n0 + r, p.N - 1) * p.b_rs;

    typedef typename std::conditional<T == 32, f32x16, f32x4>::type acc_t;
    acc_t acc[2];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int i = 0; i < NR; i++) acc[h][i] = 0.f;

    // The rounds cover K4 = K rounded down to a multiple of 4, so that a KC operand's chunk is inside the row as a
    // whole or not at all; wave 0 adds the last one to three k afterwards.  What lies past the end is loaded
    // from k = 0 (every load is unconditional) and zeroed.
    const int K4 = (A_KC || B_KC) ? (p.K & ~3) : p.K;
    const int ngroups = (K4 + KG - 1) / KG;
    f32x4 a[U], b[U];
    auto load_operand = [&](f32x4& dst, const float* __restrict__ row, int64_t ks, int k, auto kc_tag) {
        if constexpr (decltype(kc_tag)::value) {
            dst = *reinterpret_cast<const f32x4u*>(row + (k < K4 ? k : 0));
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) dst[j] = row[(int64_t)(k + j < K4 ? k + j : 0) * ks];
        }
    };
    auto mask_operand = [&](f32x4 v, int k, auto kc_tag) -> f32x4 {
        if constexpr (decltype(kc_tag)::value) {
            return keep_if(v, k < K4);
        } else {
            f32x4 o;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float e = v[j];
                o[j] = __int_as_float(__float_as_int(e) & (k + j < K4 ? -1 : 0));
            }
            return o;
        }
    };
    auto load = [&](int g0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = (g0 + u * GS) * KG + 4 * kq;
            load_operand(a[u], arow, p.a_ks, k, std::integral_constant<bool, A_KC>{});
            load_operand(b[u], brow, p.b_ks, k, std::integral_constant<bool, B_KC>{});
        }
    };
    // Rounds of U groups per wave; the next round's loads are issued before this round's MFMAs.  No load sits
    // under a condition inside the loop (it would be waited for at the join before anything else issues); the
    // last round runs after the loop, without a prefetch.
    auto multiply = [&](const f32x4(&av)[U], const f32x4(&bv)[U], int g0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = (g0 + u * GS) * KG + 4 * kq;
            const f32x4 am = mask_operand(av[u], k, std::integral_constant<bool, A_KC>{});
            const f32x4 bm = mask_operand(bv[u], k, std::integral_constant<bool, B_KC>{});
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (T == 32)
                    acc[u & 1] = __builtin_amdgcn_mfma_f32_32x32x2f32(am[j], bm[j], acc[u & 1], 0, 0, 0);
                else
                    acc[u & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(am[j], bm[j], acc[u & 1], 0, 0, 0);
            }
            // one round of eight: the products of a group start when its two loads have landed, not when all have
            if (U != kWsFlight) __builtin_amdgcn_sched_barrier(0);
        }
    };
    int g0 = wave * (T == 32 ? 1 : U);
    if (g0 < ngroups) {   // uniform per wave
        load(g0);
        // every load of the round is issued before the first product (left alone, the scheduler sinks the loads
        // to their uses to save registers: two in flight instead of sixteen)
        __builtin_amdgcn_sched_barrier(0);
        // (32 x 32 blocks with two operands that are not K-contiguous: eight element loads per group with a 64-bit
        // address each; a second set of operands in flight did not fit the 128 registers of a wave and spilled, so
        // this form loads a round after it has multiplied the one before -- four waves per SIMD cover the wait)
        constexpr bool kOverlap = !(T == 32 && !A_KC && !B_KC);
        for (int next = g0 + U * kWsWaves; U == kWsFlight && next < ngroups; next += U * kWsWaves) {
            if constexpr (kOverlap) {
                f32x4 a_now[U], b_now[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    a_now[u] = a[u];
                    b_now[u] = b[u];
                }
                load(next);
                multiply(a_now, b_now, g0);
            } else {
                multiply(a, b, g0);
                __builtin_amdgcn_sched_barrier(0);
                load(next);
                __builtin_amdgcn_sched_barrier(0);
            }
            g0 = next;
        }
        multiply(a, b, g0);
    }
    if ((A_KC || B_KC) && wave == 0 && K4 < p.K) {   // uniform: the one to three k past K4, in the lanes of k group 0
        f32x4 at = {0.f, 0.f, 0.f, 0.f}, bt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 3; j++) {
            if (kq == 0 && K4 + j < p.K) {
                at[j] = arow[(int64_t)(K4 + j) * p.a_ks];
                bt[j] = brow[(int64_t)(K4 + j) * p.b_ks];
            }
        }
#pragma unroll
        for (int j = 0; j < 3; j++) {
            if constexpr (T == 32)
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(at[j], bt[j], acc[0], 0, 0, 0);
            else
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(at[j], bt[j], acc[0], 0, 0, 0);
        }
    }

#pragma unroll
    for (int i = 0; i < NR; i++) red[(wave * NR + i) * 64 + lane] = acc[0][i] + acc[1][i];
    __syncthreads();

    if (tid < NR * 64) {
        const int i = tid >> 6, l = tid & 63;
        float v = red[i * 64 + l];
#pragma unroll
        for (int w = 1; w < kWsWaves; w++) v += red[(w * NR + i) * 64 + l];
        // element (register i, lane l) of an MFMA result block
        const int row = T == 32 ? 8 * (i >> 2) + 4 * (l >> 5) + (i & 3) : 4 * (l >> 4) + i;
        const int col = T == 32 ? (l & 31) : (l & 15);
        const int m = m0 + row, n = n0 + col;
        if (m < p.M && n < p.N) {
            const float alpha = p.has_alpha ? (p.alpha ? *p.alpha : 0.f) : 1.f;
            const float leaky = p.leaky ? *p.leaky : 0.f;
            const int64_t idx = (int64_t)m * p.ldc + n;
            if (p.has_alpha) v *= alpha;
            if (p.accflag) v += p.C[idx];
            if (p.bias) v += p.bias[n];
            if (p.C2) p.C2[idx] = v;
            p.C[idx] = apply_act(v, p.act, leaky);
        }
    }
}

}  // namespace

// Each operand K-contiguous or contiguous along its output index; a contiguous output row, one product.  Whether the product is small enough for this kernel to win is the dispatcher's decision.
bool wavesplit_applies(const GemmDesc& d) {
    const bool a_ok = d.a_ks == 1 || d.a_rs == 1, b_ok = d.b_ks == 1 || d.b_rs == 1;
    return d.nbatch == 1 && a_ok && b_ok && d.c_cs == 1 && d.rowsum == nullptr && d.k_part == 0 && d.K >= 1 &&
           d.K <= (1 << 24) && d.act >= kActNone && d.act <= kActSwish;
}

template <int T, int U>
static void launch_wavesplit_forms(const WaveSplitParams& p, bool a_kc, bool b_kc, dim3 grid, hipStream_t stream) {
    const dim3 block(64 * kWsWaves);
    if (a_kc && b_kc) gemm_wavesplit_kernel<T, true, true, U><<<grid, block, 0, stream>>>(p);
    else if (a_kc) gemm_wavesplit_kernel<T, true, false, U><<<grid, block, 0, stream>>>(p);
    else if (b_kc) gemm_wavesplit_kernel<T, false, true, U><<<grid, block, 0, stream>>>(p);
    else gemm_wavesplit_kernel<T, false, false, U><<<grid, block, 0, stream>>>(p);
}

int launch_gemm_wavesplit(const GemmDesc& d, int block_edge, hipStream_t stream) {
    WaveSplitParams p{};
    p.A = d.A; p.B = d.B; p.C = d.C; p.C2 = d.C2; p.bias = d.bias; p.alpha = d.alpha; p.leaky = d.leaky;
    p.M = (int)d.M; p.N = (int)d.N; p.K = (int)d.K;
    p.a_rs = d.a_rs; p.a_ks = d.a_ks; p.b_rs = d.b_rs; p.b_ks = d.b_ks; p.ldc = d.c_rs;
    p.act = d.act; p.accflag = d.acc; p.has_alpha = d.has_alpha;
    const int64_t T = block_edge;
    const int64_t tiles_m = (d.M + T - 1) / T, tiles_n = (d.N + T - 1) / T;
    if (tiles_m * tiles_n > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: grid too large");
    p.m_fast = tiles_m > tiles_n;
    p.tiles_fast = (int)(p.m_fast ? tiles_m : tiles_n);
    const dim3 grid((unsigned)(tiles_m * tiles_n));
    const bool a_kc = d.a_ks == 1, b_kc = d.b_ks == 1;
    // Up to eight groups per wave (groups of 8 k for T = 32, of 16 k for T = 16, over 16 waves): ONE round of exactly
    // as many groups as K needs, every load of a wave in flight at once (256 x 1024 x 1024: 11.0 -> 10.6 us, the
    // [K, N] form 10.3 -> 9.7; 64 x 512 x 2048 on 16-blocks 8.4 -> 7.4).  Exactly: a group past the end of K is
    // loaded and multiplied all the same, and the four waves of a SIMD share its matrix core (256 x 1024 x 640 with
    // a round of eight: 10.6 us, of five: 7.6; K <= 384 on 32-blocks took 6 us whatever K was).  Longer
    // reductions: rounds of four.
    const int64_t kg = block_edge == 32 ? 8 : 16;
    const int64_t per_wave = ((d.K + kg - 1) / kg + kWsWaves - 1) / kWsWaves;
    auto forms = [&](auto tc, auto uc) {
        launch_wavesplit_forms<decltype(tc)::value, decltype(uc)::value>(p, a_kc, b_kc, grid, stream);
    };
    auto rounds = [&](auto tc) {
        switch (per_wave) {
        case 1: forms(tc, std::integral_constant<int, 1>{}); break;
        case 2: forms(tc, std::integral_constant<int, 2>{}); break;
        case 3: forms(tc, std::integral_constant<int, 3>{}); break;
        case 5: forms(tc, std::integral_constant<int, 5>{}); break;
        case 6: forms(tc, std::integral_constant<int, 6>{}); break;
        case 7: forms(tc, std::integral_constant<int, 7>{}); break;
        case 8: forms(tc, std::integral_constant<int, 8>{}); break;
        default: forms(tc, std::integral_constant<int, kWsFlight>{}); break;
        }
    };
    if (block_edge == 32) rounds(std::integral_constant<int, 32>{});
    else rounds(std::integral_constant<int, 16>{});
    return check_launch("gemm_wavesplit_kernel");
}

}  // namespace kai
