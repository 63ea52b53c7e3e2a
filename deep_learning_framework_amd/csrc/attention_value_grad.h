// Device code of the value gradient of the attention block (the kernel of attention_value_grad.hip, and the second
// kind of workgroup in the one-launch backward of attention_backward.hip),
//   gV[b, k, h, :] = sum_q P[b, q, k, h] * gY[b, q, h, :]       VMath::mix_values_backward_value (vmath.cu:7081-7129
// of the reference; the fourth call of VTensor::multihead_attention_backprop, vtensor.cpp:3145-3154),
// per (batch entry, head) a product P^T . gY with the reduction over the rows q.
//
// Neither operand passes through LDS.  v_mfma_f32_16x16x4_f32 takes its A operand as lane (m = l % 16, k = l / 16):
// with k = the row q, a 128-bit load of P by lane (m, k) at row q0 + k brings four values that lie next to each
// other in memory, and register i of every lane together is a complete A operand:
//   * one head (HV = 1): the lane's values are the keys 4m + i, so product i yields the keys i, i + 4, ... of a block
//     of 64; lanes 0..15 read 256 contiguous bytes of a row of P;
//   * four heads (HV = 4, head counts in whole fours): the lane's values are the heads h0 + i of the key m, so
//     product i is head h0 + i's product for a block of 16 keys, and a workgroup owns four heads.
// The B operand (lane (n = l % 16, k = l / 16)) is a column block of gY[q0 + k, :]; gY is small and stays in L2.  Head
// sizes in whole 64s load it 128 bits per lane as well, columns 4n .. 4n + 3 of a group of 64: register j of every
// lane is the B operand of the columns j, j + 4, ..., so the block's columns come out permuted, which the way to LDS
// at the end undoes (one load per step and group instead of four).  Other head sizes load the columns 16 nb + n,
// 32 bits per lane.  A wave keeps the whole block of the output (64 keys x D, or 16 keys x 4 heads x D) in
// 4 x D / 16 accumulators and walks over every eighth step of four rows, its loads a few steps ahead; the eight
// waves' sums meet in LDS at the end, in a fixed order, and leave as 128-bit stores.
//
// TR (four heads only): the same with the roles of P's two middle indices exchanged,
//   Y[b, t, h, :] = sum_k P[b, t, k, h] * B[b, k, h, :]
// which is VMath::mix_values (vmath.cu:6977-7025, B = V) and VMath::mult_on_heads_backward (vmath.cu:6783-6829, P = the
// gradient of the scores, B = Q or K): the lane's row of P is the output row t = m, the step runs over the keys.
// The four heads of a (t, k) pair are still one 128-bit word, so the loads are the same.  Here a key past the end
// would read the next row's value into a row that IS stored, so those operand values are set to zero.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace kai {
namespace vgrad {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int B, int E, typename F>
__device__ __forceinline__ void vg_static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        vg_static_for<B + 1, E>(f);
    }
}

constexpr int kVgWaves = 8;
constexpr int kVgThreads = 64 * kVgWaves;

struct ValueGradParams {
    const float* P;      // [nbat, ntimes, ntimes, nhead]
    const float* gY;     // the other operand: rows of gy_rs floats, head h at column h * npiece
    float* gV;           // the output: rows of gv_rs floats, head h at column h * npiece
    int64_t p_batch_stride;
    int64_t gy_rs, gv_rs;
    int ntimes, nhead, npiece;
};

// DB = head size / 16; HV = heads per workgroup (1 or 4)
template <int DB, int HV>
constexpr int value_grad_lds_floats() {
    return 4 * (HV == 1 ? 64 : 16) * (HV * 16 * DB + 4);
}

// bid of `total` workgroups; lds: value_grad_lds_floats<DB, HV>() floats, 16-byte aligned
template <int DB, int HV, bool TR = false>
__device__ __forceinline__ void attention_value_grad_body(const ValueGradParams& p, const int bid, const int total, float* lds) {
    constexpr int D = 16 * DB;
    constexpr int kVgDepth = 4;                   // steps of a wave whose loads are in flight
    constexpr bool YV = DB % 4 == 0;              // 128-bit loads of gY
    constexpr int kKeys = HV == 1 ? 64 : 16;      // keys per workgroup = rows of its block of the output
    constexpr int kCols = HV * D;                 // columns of the block: contiguous in memory
    constexpr int kRowStride = kCols + 4;
    constexpr int kRegion = kKeys * kRowStride;   // floats; also holds a wave's 16 * DB registers x 64 lanes
    static_assert(kRegion >= 16 * DB * 64, "a region holds a wave's accumulators");
    static_assert(4 * kRegion == value_grad_lds_floats<DB, HV>(), "the size the callers reserve");
    static_assert(!TR || HV == 4, "the exchanged roles exist for four heads per workgroup");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int T = p.ntimes;
    const int H = p.nhead;
    const int ktiles = (T + kKeys - 1) / kKeys;
    const int hgroups = H / HV;
    // workgroup id -> (batch entry, key tile, head group): ids congruent modulo 8 share an L2, so each of the
    // eight gets a contiguous run of that order (the head groups of a key tile read the same lines of P)
    int id = bid;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    const int hg = id % hgroups;
    const int rest = id / hgroups;
    const int ktile = rest % ktiles;
    const int b = rest / ktiles;
    const int key0 = ktile * kKeys;
    const int h0 = hg * HV;

    auto uniform_ptr = [](const float* q) -> float* {
        const uint64_t a = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
    };
    // This batch entry's P from head h0 on and its gY from head h0's first column on.  A row q past the end lies
    // behind the end of both resources and reads as zero; a key past the end reads a value of the next row, which
    // only reaches rows of the block that are never stored.
    const int extent_p = (int)(((int64_t)T * T * H - h0) * 4);
    const int extent_y = (int)((((int64_t)(T - 1) * p.gy_rs) + (int64_t)(H - h0) * D) * 4);
    const __amdgpu_buffer_rsrc_t rsrc_p =
        __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.P + (int64_t)b * p.p_batch_stride + h0), 0, extent_p, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_y = __builtin_amdgcn_make_buffer_rsrc(
        uniform_ptr(p.gY + (int64_t)b * T * p.gy_rs + (int64_t)h0 * D), 0, extent_y, 0x00020000);
    // byte offsets of this lane at row g of step `wave`; a step later for this wave is 32 rows further on
    // (TR: key0 is the block's first output row t, the lane's row of P is t, the step runs over the keys)
    const int key_l = key0 + (HV == 1 ? 4 * r16 : r16);
    int red = 4 * wave + g;      // this lane's index along the reduction in the current step
    int poff = TR ? (int)((((int64_t)min(key_l, T) * T + red) * H) * 4) : (int)((((int64_t)red * T + key_l) * H) * 4);
    int yoff = (int)(((int64_t)red * p.gy_rs + (YV ? 4 * r16 : r16)) * 4);
    const int pstep = TR ? 4 * kVgWaves * H * 4 : (int)((int64_t)4 * kVgWaves * T * H * 4);
    const int ystep = (int)((int64_t)4 * kVgWaves * p.gy_rs * 4);

    f32x4 acc[4][DB];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int nb = 0; nb < DB; nb++) acc[i][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    f32x4 pa[kVgDepth];
    float gb[kVgDepth][HV][DB];
    auto load_step = [&](auto sc) {
        constexpr int s = decltype(sc)::value;
        // (TR: a key past the end is steered behind the end of the resource, where the load returns zero)
        const int po = (!TR || red < T) ? poff : 0x7FFFFFF0;
        pa[s] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_p, po, 0, 0));
        if constexpr (TR) red += 4 * kVgWaves;
#pragma unroll
        for (int i = 0; i < HV; i++) {
            if constexpr (YV) {
#pragma unroll
                for (int u = 0; u < DB / 4; u++) {
                    const f32x4 y = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_y, yoff + (i * D + 64 * u) * 4, 0, 0));
#pragma unroll
                    for (int j = 0; j < 4; j++) gb[s][i][4 * u + j] = y[j];
                }
            } else {
#pragma unroll
                for (int nb = 0; nb < DB; nb++)
                    gb[s][i][nb] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_y, yoff + (i * D + 16 * nb) * 4, 0, 0));
            }
        }
        poff += pstep;
        yoff += ystep;
    };
    // steps of four rows: wave w takes the steps w, w + 8, ...; rounded up to whole rings, the surplus steps lie
    // behind the last row and add zeros
    const int nsteps = (T + 3) / 4;
    const int mine = (nsteps - wave + kVgWaves - 1) / kVgWaves;
    const int rounds = (mine + kVgDepth - 1) / kVgDepth;
    vg_static_for<0, kVgDepth>([&](auto sc) {
        load_step(sc);
        __builtin_amdgcn_sched_barrier(0);   // in this order: the loop waits for the oldest step only
    });
    for (int r = 0; r < rounds; r++) {
        vg_static_for<0, kVgDepth>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int nb = 0; nb < DB; nb++)
                    acc[i][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[s][i], gb[s][HV == 1 ? 0 : i][nb], acc[i][nb], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            load_step(sc);      // the step a ring further on (past the wave's last round: zeros, never used)
        });
    }

    // ---- the eight waves' sums: 4..7 hand theirs to 0..3, which lay theirs out as the block; all threads add and store
    f32x4* ex = reinterpret_cast<f32x4*>(lds);
    if (wave >= 4) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int nb = 0; nb < DB; nb++) ex[(wave - 4) * (kRegion / 4) + (i * DB + nb) * 64 + lane] = acc[i][nb];
    }
    __syncthreads();
    if (wave < 4) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int nb = 0; nb < DB; nb++) acc[i][nb] += ex[wave * (kRegion / 4) + (i * DB + nb) * 64 + lane];
    }
    __syncthreads();
    if (wave < 4) {
        // acc[i][nb][v]: one head: key 16g + 4v + i; four heads: key 4g + v, head i.  Column of the head: 16nb + r16,
        // or, with the 128-bit loads of gY, 64 (nb / 4) + 4 r16 + nb % 4: four registers are four neighbours
        float* reg = lds + wave * kRegion;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = HV == 1 ? 16 * g + 4 * v + i : 4 * g + v;
                float* dst = reg + row * kRowStride + (HV == 1 ? 0 : i * D);
                if constexpr (YV) {
#pragma unroll
                    for (int u = 0; u < DB / 4; u++)
                        *reinterpret_cast<f32x4*>(dst + 64 * u + 4 * r16) =
                            f32x4{acc[i][4 * u][v], acc[i][4 * u + 1][v], acc[i][4 * u + 2][v], acc[i][4 * u + 3][v]};
                } else {
#pragma unroll
                    for (int nb = 0; nb < DB; nb++) dst[16 * nb + r16] = acc[i][nb][v];
                }
            }
    }
    __syncthreads();
    constexpr int kChunksPerRow = kCols / 4;
    constexpr int kChunks = kKeys * kChunksPerRow;
#pragma unroll
    for (int c0 = 0; c0 < kChunks; c0 += kVgThreads) {
        const int c = c0 + tid;
        const int row = c / kChunksPerRow, c4 = c % kChunksPerRow;
        if (c < kChunks && key0 + row < T) {
            const float* src = lds + row * kRowStride + 4 * c4;
            f32x4 v = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
            for (int w = 1; w < 4; w++) v += *reinterpret_cast<const f32x4*>(src + w * kRegion);
            *reinterpret_cast<f32x4*>(p.gV + ((int64_t)b * T + key0 + row) * p.gv_rs + (int64_t)h0 * D + 4 * c4) = v;
        }
    }
}

}  // namespace vgrad

// host side (attention_value_grad.hip): the kernel's parameters and its number of workgroups for `hv` heads per workgroup
vgrad::ValueGradParams value_grad_params(float* gv, const float* gy, const float* pp, int64_t ntimes, int64_t nvec,
                                         int64_t nhead, int64_t npiece);
int64_t value_grad_blocks(int hv, int64_t nbat, int64_t ntimes, int64_t nhead);

}  // namespace kai
