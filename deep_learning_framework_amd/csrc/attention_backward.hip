// The backward middle of the attention block in one kernel per output kind:
//   gP = gM.V^T                     VMath::mix_values_backward_prop        (vmath.cu:7029-7077 of the reference)
//   gS = coef * P * (gP - sum P*gP) VMath::softmax_direct_on_axis_backward (vmath.cu:6920-6973)
//   gS[k > q] = 0 when masked       VMath::set_mh_attention_mask, backward (vmath.cu:6833-6860)
//   gK[t] = sum_k gS[t,k] * Q[k]    VMath::mult_on_heads_backward          (vmath.cu:6783-6829)
//   gQ[t] = sum_k gS[t,k] * K[k]    VMath::mult_on_heads_backward, second call
// as VTensor::multihead_attention_backprop issues them (vtensor.cpp:3145-3154).  The reference indexes gp by the
// OUTPUT row t for the key gradient and the query gradient alike (vmath.cu:6790-6797), so gP -> gS -> gK, gQ are all
// local to a row t: a workgroup that owns 64 rows of one (batch entry, head) forms the row's gP tile by tile, turns
// it into gS in registers and multiplies it into both outputs.  Neither gP nor gS is ever stored.  The value
// gradient gV = P^T.gM is a reduction over rows and keeps its own launch (mix_values_backward_value).
//
// The sum over k of P*gP that the softmax derivative needs equals sum_d gM[t,d] * M[t,d] with M = P.V, the mixed
// output of the forward pass, which the engine keeps for the output projection's weight gradient (vtensor.cpp:3050):
// given M the row constant costs one dot product of length D; without it a first pass over the keys forms it from
// P and gP as the reference writes it.
//
// Layout of the computation: as in attention_fused.hip, transposed with the rows t along the lanes.
// v_mfma_f32_16x16x4_f32, lane = (l % 16, l / 16):  gP^T[key, t] = V[key, :] . gM[t, :] puts the gradient of
// (t, key 4g + v) into register v of lane (t, g), where the matching P values are loaded to (128-bit loads with one
// head, strided 32-bit loads otherwise), and the registers that hold gS^T are, as they are, the B operand of
// gQ^T += K^T.gS^T and gK^T += Q^T.gS^T.  Eight waves = 4 groups of 16 rows x 2 halves of every key tile; the halves
// meet in LDS at the end, in a fixed order.
#include <float.h>

#include <type_traits>

#include "attention_value_grad.h"
#include "elementwise.h"

namespace kai {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// loop with compile-time indices (register arrays must never be indexed by a run-time value)
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// Workgroup id -> (batch entry, head, row tile).  Hardware deals consecutive workgroup ids round-robin over the 8
// XCDs, so ids congruent mod 8 share an L2.  They are renumbered so that each XCD gets a contiguous run of the
// order (batch entry, row tile, head): the workgroups that read the same K, V and Q rows (all row tiles of a batch
// entry and head) and, with several heads, the same lines of the head-interleaved probabilities (all heads of a
// batch entry and row tile) then sit behind one L2 instead of fetching them into all eight.
__device__ __forceinline__ void attention_block_of(int bid, int total, int ntiles, int nhead, int& b, int& h, int& tile) {
    int id = bid;
    if ((total & 7) == 0) id = (bid & 7) * (total >> 3) + (bid >> 3);
    h = id % nhead;
    const int r = id / nhead;
    tile = r % ntiles;
    b = r / ntiles;
}

constexpr int kAbQGroups = 4;          // waves along the rows t, 16 rows each
constexpr int kAbKGroups = 2;          // waves along the keys of a tile
constexpr int kAbWaves = kAbQGroups * kAbKGroups;
constexpr int kAbThreads = 64 * kAbWaves;
constexpr int kAbRows = 16 * kAbQGroups;   // rows t per workgroup

struct AttnBwdParams {
    const float* gM;     // gradient of the mixed output, [nbat, ntimes, nvec]
    const float* M;      // the mixed output, or null
    const float* P;      // probabilities, [nbat, ntimes, ntimes, nhead]
    const float* Q;
    const float* K;
    const float* V;
    float* gQ;
    float* gK;
    const float* coef;   // device scalar, null reads as 0
    int64_t nvec;            // row stride of Q, K, V, gM, M, gQ, gK
    int64_t batch_stride;    // ntimes * nvec
    int64_t p_batch_stride;  // ntimes * ntimes * nhead
    int ntimes, nhead, npiece;
    int masked;
};

// DB = head size / 16; KB = blocks of 16 keys per wave and tile (a tile holds 32 * KB keys); PVEC: one head and
// rows of P that allow 128-bit loads.
template <int DB, int KB>
constexpr int rows_lds_floats() {
    return 2 * 3 * (16 * KB * kAbKGroups) * (16 * DB + 4);
}

// Workgroup `bid` of `nblocks`; smem: rows_lds_floats<DB, KB>() floats, 16-byte aligned.
template <int DB, int KB, bool PVEC>
__device__ __forceinline__ void attention_backward_rows_body(const AttnBwdParams& p, const int bid, const int nblocks, float* smem) {
    constexpr int D = 16 * DB;
    constexpr int kKeys = 16 * KB * kAbKGroups;
    constexpr int kStride = D + 4;           // tiles [keys][D] lie in LDS as in memory
    constexpr int kTile = kKeys * kStride;
    constexpr int kChunksPerKey = D / 4;
    constexpr int kTileChunks = kKeys * kChunksPerKey;
    constexpr int NCH = (kTileChunks + kAbThreads - 1) / kAbThreads;   // 128-bit chunks per thread, operand and tile
    constexpr bool kPartial = kTileChunks % kAbThreads != 0;
    constexpr int NP = PVEC ? KB : 4 * KB;   // loads of P per lane and tile
    // [buffer][operand V, K, Q][tile]
    static_assert(6 * kTile == rows_lds_floats<DB, KB>(), "the size the callers reserve");
    float (*lds)[3][kTile] = reinterpret_cast<float (*)[3][kTile]>(smem);
    static_assert(8 * DB * 64 * kAbQGroups + 64 * kAbQGroups <= 6 * kTile, "the merge buffer must fit the tiles");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qg = wave % kAbQGroups;
    const int kgp = wave / kAbQGroups;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int T = p.ntimes;
    const int H = p.nhead;
    int b, h, ttile;
    attention_block_of(bid, nblocks, (T + kAbRows - 1) / kAbRows, H, b, h, ttile);
    const int t0 = ttile * kAbRows;
    const int64_t base = (int64_t)b * p.batch_stride + (int64_t)h * p.npiece;
    const float coef = p.coef ? *p.coef : 0.f;

    // this lane's row and its fragments of gM, scaled by coef once: gS = P * (coef*gP - coef*sum)
    const int t = t0 + 16 * qg + r16;
    const int tc = min(t, T - 1);            // rows past the end are clamped, never stored
    f32x4 gf[DB];
#pragma unroll
    for (int s = 0; s < DB; s++)
        gf[s] = coef * *reinterpret_cast<const f32x4*>(p.gM + base + (int64_t)tc * p.nvec + 16 * s + 4 * g);

    auto uniform_ptr = [](const float* q) -> float* {
        const uint64_t a = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
    };
    // Buffer resources: the rows of V, K, Q of this (batch entry, head) up to the last key, and this batch
    // entry's block of P from this head's first element on.  Keys past the end read as zeros.
    const int extent = (int)(((int64_t)(T - 1) * p.nvec + D) * 4);   // bytes; the host keeps these below 2 GiB
    const int extent_p = (int)((((int64_t)T * T - 1) * H + 1) * 4);
    const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.V + base), 0, extent, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.K + base), 0, extent, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.Q + base), 0, extent, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_p =
        __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.P + (int64_t)b * p.p_batch_stride + h), 0, extent_p, 0x00020000);
    const int tile_bytes = kKeys * (int)p.nvec * 4;
    const int p_tile_bytes = kKeys * H * 4;
    int choff[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * kAbThreads;
        choff[i] = ((c / kChunksPerKey) * (int)p.nvec + (c % kChunksPerKey) * 4) * 4;
    }
    // P[t, key, h] with key = tile * kKeys + 16 * KB * kgp + 16 * kb + 4 * g + v
    int poff[NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int key = 16 * KB * kgp + 4 * g + (PVEC ? 16 * i : 16 * (i / 4) + (i % 4));
        poff[i] = (int)((((int64_t)tc * T + key) * H) * 4);
    }

    f32x4 rv[NCH], rk[NCH], rq[NCH];
    auto load_v = [&](int kt) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * kAbThreads;
            if (!kPartial || c < kTileChunks)
                rv[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_v, choff[i], kt * tile_bytes, 0));
        }
    };
    auto load_kq = [&](int kt) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * kAbThreads;
            if (!kPartial || c < kTileChunks) {
                rk[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_k, choff[i], kt * tile_bytes, 0));
                rq[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_q, choff[i], kt * tile_bytes, 0));
            }
        }
    };
    auto store_v = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * kAbThreads;
            if (!kPartial || c < kTileChunks)
                *reinterpret_cast<f32x4*>(&lds[buf][0][(c / kChunksPerKey) * kStride + (c % kChunksPerKey) * 4]) = rv[i];
        }
    };
    auto store_kq = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * kAbThreads;
            if (!kPartial || c < kTileChunks) {
                *reinterpret_cast<f32x4*>(&lds[buf][1][(c / kChunksPerKey) * kStride + (c % kChunksPerKey) * 4]) = rk[i];
                *reinterpret_cast<f32x4*>(&lds[buf][2][(c / kChunksPerKey) * kStride + (c % kChunksPerKey) * 4]) = rq[i];
            }
        }
    };
    // this wave's P values of one tile: pr[kb][v] = P[t, key0 + 16*kb + 4*g + v, h]
    auto load_p = [&](f32x4 (&pr)[KB], int kt) {
        if (PVEC) {
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
                pr[kb] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_p, poff[kb], kt * p_tile_bytes, 0));
        } else {
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int v = 0; v < 4; v++)
                    pr[kb][v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_p, poff[4 * kb + v], kt * p_tile_bytes, 0));
        }
    };
    // gP^T of this wave's keys: KB blocks of 16 keys x 16 rows, scaled by coef through gf.  All fragments of V are
    // requested before the first product (vf), and every block is summed in NCHAIN independent chains over the head
    // dimension, so that no product waits for the one issued just before it.
    constexpr int NCHAIN = (KB == 2 ? 2 : 4) < DB ? (KB == 2 ? 2 : 4) : DB;
    // (head sizes from 96 on: the fragments of V are read chain group by chain group instead, for want of registers)
    constexpr int NVF = DB <= 5 ? DB : NCHAIN;
    auto read_v = [&](f32x4 (&vf)[NVF][KB], const float* lv, int s0) {
#pragma unroll
        for (int s = 0; s < NVF; s++)
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
                vf[s][kb] = *reinterpret_cast<const f32x4*>(lv + (16 * kb + r16) * kStride + 16 * (s0 + s) + 4 * g);
    };
    auto grad_p = [&](f32x4 (&gp)[KB], f32x4 (&vf)[NVF][KB], const float* lv) {
        f32x4 part[KB][NCHAIN];
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int c = 0; c < NCHAIN; c++) part[kb][c] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s0 = 0; s0 < DB; s0 += NCHAIN) {
            if (NVF < DB && s0 > 0) read_v(vf, lv, s0);
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int c = 0; c < NCHAIN; c++)
#pragma unroll
                    for (int kb = 0; kb < KB; kb++)
                        if (s0 + c < DB)
                            part[kb][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[NVF < DB ? c : s0 + c][kb][e], gf[s0 + c][e],
                                                                              part[kb][c], 0, 0, 0);
        }
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            gp[kb] = part[kb][0];
#pragma unroll
            for (int c = 1; c < NCHAIN; c++) gp[kb] += part[kb][c];
        }
    };

    const int nkt_all = (T + kKeys - 1) / kKeys;
    const int t_last = min(t0 + kAbRows, T) - 1;
    // key tiles that hold a key at or below the diagonal of some row of this workgroup
    const int nkt = p.masked ? min(t_last / kKeys + 1, nkt_all) : nkt_all;

    // ---- the row constant coef * sum_k P[t,k] * gP[t,k] ---------------------------------------------------------
    float delta = 0.f;
    if (p.M != nullptr) {
        const float* mrow = p.M + base + (int64_t)tc * p.nvec;
#pragma unroll
        for (int s = 0; s < DB; s++) {
            const f32x4 mv = *reinterpret_cast<const f32x4*>(mrow + 16 * s + 4 * g);
            delta += gf[s][0] * mv[0] + gf[s][1] * mv[1] + gf[s][2] * mv[2] + gf[s][3] * mv[3];
        }
        delta += __shfl_xor(delta, 16);
        delta += __shfl_xor(delta, 32);
    } else {
        // a pass of its own over ALL keys (the reference's sum does not look at the mask): V tiles only
        f32x4 pr[KB];
        load_v(0);
        store_v(0);
        __syncthreads();
        for (int kt = 0; kt < nkt_all; kt++) {
            const int buf = kt & 1;
            load_v(min(kt + 1, nkt_all - 1));
            load_p(pr, kt);
            const int key0 = kt * kKeys + 16 * KB * kgp;
            if (key0 < T) {
                f32x4 gp[KB], vf[NVF][KB];
                const float* lv = &lds[buf][0][16 * KB * kgp * kStride];
                read_v(vf, lv, 0);
                grad_p(gp, vf, lv);
#pragma unroll
                for (int kb = 0; kb < KB; kb++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const int key = key0 + 16 * kb + 4 * g + v;
                        delta += key < T ? pr[kb][v] * gp[kb][v] : 0.f;
                    }
            }
            if (kt + 1 < nkt_all) store_v(buf ^ 1);
            __syncthreads();
        }
        delta += __shfl_xor(delta, 16);
        delta += __shfl_xor(delta, 32);
        // the two key halves add their parts
        float* ex = &lds[0][0][0];
        if (kgp == 1) ex[qg * 64 + lane] = delta;
        __syncthreads();
        if (kgp == 0) {
            delta += ex[qg * 64 + lane];
            ex[qg * 64 + lane] = delta;
        }
        __syncthreads();
        delta = ex[qg * 64 + lane];
        __syncthreads();
    }

    // ---- gS tile by tile, multiplied into both outputs ----------------------------------------------------------
    //
    // The products of a tile are dealt with in NG groups of 2 * KB * 4 (gP, one 16-wide slice s of the head dimension)
    // or 2 * DB (gQ and gK, one key column e of one block kb) matrix instructions.  The schedule is written out,
    // with fences between the groups so that the compiler keeps it:
    //   * the LDS reads of group i + 1 are issued BEFORE the products of group i (operands double buffered), so no
    //     product waits for LDS, and the eight waves do not all hit LDS in one burst at the start of a tile;
    //   * the global loads of the next tile are dealt out one per group over the first groups (issued together
    //     they fill the address unit's queue and every wave waits at its next load), its LDS stores two per group
    //     over the last groups;
    //   * the barrier sits before the LAST group, whose operands are in registers by then and whose products cover
    //     the first reads of the next tile.
    // Measured on the first version of this loop (all reads, then all products; cfg4, one head, 36.8 us): without the
    // LDS reads and the tile traffic it took 26.1 us, the time of its matrix instructions plus launch and first
    // loads; the reads added 5.5 us and the tile traffic 5.2 us on top instead of running under them.
    f32x4 acc_q[DB], acc_k[DB];
#pragma unroll
    for (int db = 0; db < DB; db++) {
        acc_q[db] = f32x4{0.f, 0.f, 0.f, 0.f};
        acc_k[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    constexpr int NA = DB;            // groups of gP products: one per slice s
    constexpr int NC = 4 * KB;        // groups of gQ / gK products: one per (kb, e)
    constexpr int NG = NA + NC;
    constexpr int NLOAD = 3 * NCH;    // global loads of a tile per thread (V, K, Q chunks), then the loads of P
    constexpr int kLoadsPerGroup = (NLOAD + 1 + (NG - 3) - 1) / (NG - 3);     // all issued by group NG - 3
    constexpr int kStoresPerGroup = 2;
    constexpr int kStoreGroups = (NLOAD + kStoresPerGroup - 1) / kStoresPerGroup;
    constexpr int kFirstStoreGroup = NG - 1 - kStoreGroups;                   // the last store is in group NG - 2
    static_assert(kFirstStoreGroup >= 1, "too many chunks for this schedule");

    f32x4 p_next[KB];
    load_v(0);
    load_kq(0);
    load_p(p_next, 0);
    store_v(0);
    store_kq(0);
    __syncthreads();

    // operand registers of the groups, double buffered by group parity
    f32x4 vf[2][KB];
    float kf[2][DB], qf2[2][DB];
    // the LDS reads of group i of the tile in buffer `buf`
    auto stage = [&](auto ic, int buf) {
        constexpr int i = decltype(ic)::value;
        constexpr int par = i & 1;
        const float* lv = &lds[buf][0][16 * KB * kgp * kStride];
        if constexpr (i < NA) {
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
                vf[par][kb] = *reinterpret_cast<const f32x4*>(lv + (16 * kb + r16) * kStride + 16 * i + 4 * g);
        } else {
            constexpr int kb = (i - NA) / 4, e = (i - NA) % 4;
            const float* lk = &lds[buf][1][16 * KB * kgp * kStride] + (16 * kb + 4 * g + e) * kStride + r16;
            const float* lq = &lds[buf][2][16 * KB * kgp * kStride] + (16 * kb + 4 * g + e) * kStride + r16;
#pragma unroll
            for (int db = 0; db < DB; db++) {
                kf[par][db] = lk[16 * db];
                qf2[par][db] = lq[16 * db];
            }
        }
    };
    // one chunk of the next tile's global loads / of its LDS stores, by number: V chunks, K chunks, Q chunks
    auto load_one = [&](auto jc, int kt) {
        constexpr int j = decltype(jc)::value;
        constexpr int i = j % NCH;
        const int c = tid + i * kAbThreads;
        if (!kPartial || c < kTileChunks) {
            if constexpr (j / NCH == 0) rv[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_v, choff[i], kt * tile_bytes, 0));
            else if constexpr (j / NCH == 1) rk[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_k, choff[i], kt * tile_bytes, 0));
            else rq[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_q, choff[i], kt * tile_bytes, 0));
        }
    };
    auto store_one = [&](auto jc, int buf) {
        constexpr int j = decltype(jc)::value;
        constexpr int i = j % NCH;
        const int c = tid + i * kAbThreads;
        if (!kPartial || c < kTileChunks) {
            float* dst = &lds[buf][j / NCH][(c / kChunksPerKey) * kStride + (c % kChunksPerKey) * 4];
            *reinterpret_cast<f32x4*>(dst) = j / NCH == 0 ? rv[i] : j / NCH == 1 ? rk[i] : rq[i];
        }
    };

    stage(std::integral_constant<int, 0>{}, 0);
    for (int kt = 0; kt < nkt; kt++) {
        const int buf = kt & 1;
        const int nxt = min(kt + 1, nkt - 1);      // the surplus loads and stores of the last tile are never used
        const int key0 = kt * kKeys + 16 * KB * kgp;    // first key of this wave's part of the tile
        f32x4 pr[KB];
#pragma unroll
        for (int kb = 0; kb < KB; kb++) pr[kb] = p_next[kb];
        f32x4 part[KB][NCHAIN];
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int c = 0; c < NCHAIN; c++) part[kb][c] = f32x4{0.f, 0.f, 0.f, 0.f};
        f32x4 gs[KB];
        static_for<0, NG>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            constexpr int par = i & 1;
            // -- the next group's operands
            if constexpr (i + 1 < NG) {
                stage(std::integral_constant<int, i + 1>{}, buf);
            } else {
                __syncthreads();     // the next tile is in LDS, and every wave has read this one
                if (kt + 1 < nkt) stage(std::integral_constant<int, 0>{}, buf ^ 1);
            }
            // -- this group's share of the next tile's traffic
            static_for<0, kLoadsPerGroup>([&](auto lc) {
                constexpr int j = i * kLoadsPerGroup + decltype(lc)::value;
                if constexpr (j < NLOAD) load_one(std::integral_constant<int, j>{}, nxt);
                else if constexpr (j == NLOAD) load_p(p_next, nxt);
            });
            if constexpr (i >= kFirstStoreGroup && i < NG - 1) {
                static_for<0, kStoresPerGroup>([&](auto sc) {
                    constexpr int j = (i - kFirstStoreGroup) * kStoresPerGroup + decltype(sc)::value;
                    if constexpr (j < NLOAD) store_one(std::integral_constant<int, j>{}, buf ^ 1);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
            // -- this group's products
            if constexpr (i < NA) {
                constexpr int c = i % NCHAIN;
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int kb = 0; kb < KB; kb++)
                        part[kb][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[par][kb][e], gf[i][e], part[kb][c], 0, 0, 0);
                if constexpr (i == NA - 1) {
                    // gS = P * (coef * gP - coef * row sum); keys past the end or above the diagonal give nothing
#pragma unroll
                    for (int kb = 0; kb < KB; kb++) {
                        gs[kb] = part[kb][0];
#pragma unroll
                        for (int cc = 1; cc < NCHAIN; cc++) gs[kb] += part[kb][cc];
                        gs[kb] = pr[kb] * (gs[kb] - delta);
                    }
                    const bool edge_tile = key0 + 16 * KB > T || (p.masked && key0 + 16 * KB - 1 > t0 + 16 * qg);   // wave-uniform
                    if (edge_tile) {
#pragma unroll
                        for (int kb = 0; kb < KB; kb++)
#pragma unroll
                            for (int v = 0; v < 4; v++) {
                                const int key = key0 + 16 * kb + 4 * g + v;
                                if (key >= T || (p.masked && key > t)) gs[kb][v] = 0.f;
                            }
                    }
                }
            } else {
                // gQ^T[d, t] += K[key, d] * gS[t, key];  gK^T[d, t] += Q[key, d] * gS[t, key]  for key = 16*kb + 4*g + e
                constexpr int kb = (i - NA) / 4, e = (i - NA) % 4;
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    acc_q[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[par][db], gs[kb][e], acc_q[db], 0, 0, 0);
                    acc_k[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf2[par][db], gs[kb][e], acc_k[db], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    // the second key half hands its sums over through LDS; the first adds them and stores
    float* mg = &lds[0][0][0] + (qg * 64 + lane);
    constexpr int kMergeStride = 64 * kAbQGroups;
    if (kgp == 1) {
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                mg[(4 * db + v) * kMergeStride] = acc_q[db][v];
                mg[(4 * DB + 4 * db + v) * kMergeStride] = acc_k[db][v];
            }
    }
    __syncthreads();
    if (kgp == 1) return;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            acc_q[db][v] += mg[(4 * db + v) * kMergeStride];
            acc_k[db][v] += mg[(4 * DB + 4 * db + v) * kMergeStride];
        }
    // acc[db][v] = gradient of (row t, d = 16*db + 4*g + v)
    if (t < T) {
        float* oq = p.gQ + base + (int64_t)t * p.nvec;
        float* ok = p.gK + base + (int64_t)t * p.nvec;
#pragma unroll
        for (int db = 0; db < DB; db++) {
            *reinterpret_cast<f32x4*>(oq + 16 * db + 4 * g) = acc_q[db];
            *reinterpret_cast<f32x4*>(ok + 16 * db + 4 * g) = acc_k[db];
        }
    }
}

template <int DB, int KB, bool PVEC>
__global__ void __launch_bounds__(kAbThreads) attention_backward_rows_kernel(const AttnBwdParams p) {
    __shared__ __attribute__((aligned(16))) float smem[rows_lds_floats<DB, KB>()];
    attention_backward_rows_body<DB, KB, PVEC>(p, blockIdx.x, gridDim.x, smem);
}

// The whole backward middle in one launch: the first `nrows` workgroups are those of the rows kernel, the others
// compute the value gradient (attention_value_grad.h; one head per workgroup where P allows 128-bit loads along the
// keys, else four).  The two kinds share nothing; one launch saves the second launch's start-up, and the value
// gradient's workgroups start as the first rows workgroups leave their compute units.
template <int DB, int KB, bool PVEC>
__global__ void __launch_bounds__(kAbThreads) attention_backward_all_kernel(const AttnBwdParams p, const vgrad::ValueGradParams v,
                                                                            const int nrows) {
    constexpr int HV = PVEC ? 1 : 4;
    constexpr int kFloats = rows_lds_floats<DB, KB>() > vgrad::value_grad_lds_floats<DB, HV>() ? rows_lds_floats<DB, KB>()
                                                                                             : vgrad::value_grad_lds_floats<DB, HV>();
    static_assert(vgrad::kVgThreads == kAbThreads, "one block size for both kinds of workgroup");
    __shared__ __attribute__((aligned(16))) float smem[kFloats];
    const int bid = blockIdx.x;
    if (bid < nrows) attention_backward_rows_body<DB, KB, PVEC>(p, bid, nrows, smem);
    else vgrad::attention_value_grad_body<DB, HV>(v, bid - nrows, (int)gridDim.x - nrows, smem);
}

}  // namespace

bool attention_backward_applies(const float* gq, const float* gk, const float* gm, const float* m, const float* pp,
                                const float* q, const float* k, const float* v, int64_t ntimes, int64_t nvec,
                                int64_t nhead, int64_t npiece) {
    // the gradients and the mixed output are [nbat, ntimes, nhead, npiece] like the output of mix_values, the
    // projections [nbat, ntimes, nvec]: the same thing only when the heads fill the vector
    return nhead * npiece == nvec && npiece % 16 == 0 && npiece >= 16 && npiece <= 128 && nvec % 4 == 0 && ntimes >= 1 &&
           ntimes <= kMaxDim && ntimes * nvec * 4 < (1ll << 31) && ntimes * ntimes * nhead * 4 < (1ll << 31) &&
           nhead >= 1 && aligned16(gq) && aligned16(gk) && aligned16(gm) && (m == nullptr || aligned16(m)) &&
           aligned16(q) && aligned16(k) && aligned16(v) && (reinterpret_cast<uintptr_t>(pp) & 3u) == 0;
}

// gv null: the rows kernel alone; else the one-launch kernel, whose value gradient workgroups follow the rows workgroups
template <int DB, int KB, bool MERGE_NOVEC = (DB <= 4)>
static int launch_rows(const AttnBwdParams& p, const vgrad::ValueGradParams* v, int64_t vblocks, bool pvec, dim3 grid,
                       hipStream_t stream) {
    const dim3 block(kAbThreads);
    if (v == nullptr) {
        if (pvec) attention_backward_rows_kernel<DB, KB, true><<<grid, block, 0, stream>>>(p);
        else attention_backward_rows_kernel<DB, KB, false><<<grid, block, 0, stream>>>(p);
        return KAI_OK;
    }
    const dim3 all(grid.x + (unsigned)vblocks);
    if (pvec) {
        attention_backward_all_kernel<DB, KB, true><<<all, block, 0, stream>>>(p, *v, (int)grid.x);
        return KAI_OK;
    }
    if constexpr (MERGE_NOVEC) {
        attention_backward_all_kernel<DB, KB, false><<<all, block, 0, stream>>>(p, *v, (int)grid.x);
        return KAI_OK;
    }
    // four heads per workgroup exist for head sizes up to 64 only; attention_backward_one_launch never sends others here
    return fail(KAI_ERR_INVALID_ARGUMENT, "attention backward: no one-launch kernel for this head size with several heads");
}

// Whether kai_attention_backward runs this geometry as ONE launch: the rows kernel applies (the caller has checked)
// and the value gradient's kernel takes the geometry with the heads per workgroup that go with the rows kernel's
// way of loading P (one head with 128-bit loads along the keys, four heads otherwise).
bool attention_backward_one_launch(const float* gv, const float* gm, const float* pp, int64_t nbat, int64_t ntimes,
                                   int64_t nvec, int64_t nhead, int64_t npiece) {
    const int hv = attention_value_grad_heads(gv, gm, pp, ntimes, nvec, nhead, npiece);
    const bool pvec = nhead == 1 && ntimes % 4 == 0 && aligned16(pp);
    if (!(pvec ? hv == 1 : hv == 4)) return false;
    const int64_t ttiles = (ntimes + kAbRows - 1) / kAbRows;
    return ttiles * nbat * nhead + value_grad_blocks(hv, nbat, ntimes, nhead) <= kMaxDim;
}

// gv null: gQ and gK only (the caller computes the value gradient); else all three in one launch, which
// attention_backward_one_launch must have allowed
int launch_attention_backward_rows(float* gq, float* gk, float* gv, const float* gm, const float* m, const float* pp,
                                   const float* q, const float* k, const float* v, int64_t nbat, int64_t ntimes,
                                   int64_t nvec, int64_t nhead, int64_t npiece, const float* hcoef, int masked,
                                   hipStream_t stream) {
    AttnBwdParams p{};
    p.gM = gm; p.M = m; p.P = pp; p.Q = q; p.K = k; p.V = v; p.gQ = gq; p.gK = gk; p.coef = hcoef;
    p.nvec = nvec; p.batch_stride = ntimes * nvec; p.p_batch_stride = ntimes * ntimes * nhead;
    p.ntimes = (int)ntimes; p.nhead = (int)nhead; p.npiece = (int)npiece;
    p.masked = masked;
    const int64_t ttiles = (ntimes + kAbRows - 1) / kAbRows;
    if (ttiles * nbat * nhead > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "attention backward: grid too large");
    const dim3 grid((unsigned)(ttiles * nbat * nhead));
    const bool pvec = nhead == 1 && ntimes % 4 == 0 && aligned16(pp);
    vgrad::ValueGradParams vp{};
    int64_t vblocks = 0;
    if (gv != nullptr) {
        if (!attention_backward_one_launch(gv, gm, pp, nbat, ntimes, nvec, nhead, npiece))
            return fail(KAI_ERR_INVALID_ARGUMENT, "attention backward: the value gradient does not fit the one-launch kernel");
        vp = value_grad_params(gv, gm, pp, ntimes, nvec, nhead, npiece);
        vblocks = value_grad_blocks(pvec ? 1 : 4, nbat, ntimes, nhead);
    }
    const vgrad::ValueGradParams* vptr = gv != nullptr ? &vp : nullptr;
    switch (npiece / 16) {
    case 1: KAI_TRY((launch_rows<1, 2>(p, vptr, vblocks, pvec, grid, stream))); break;
    case 2: KAI_TRY((launch_rows<2, 2>(p, vptr, vblocks, pvec, grid, stream))); break;
    case 3: KAI_TRY((launch_rows<3, 2>(p, vptr, vblocks, pvec, grid, stream))); break;
    case 4: KAI_TRY((launch_rows<4, 2>(p, vptr, vblocks, pvec, grid, stream))); break;
    case 5: KAI_TRY((launch_rows<5, 2>(p, vptr, vblocks, pvec, grid, stream))); break;
    case 6: KAI_TRY((launch_rows<6, 1>(p, vptr, vblocks, pvec, grid, stream))); break;
    case 7: KAI_TRY((launch_rows<7, 1>(p, vptr, vblocks, pvec, grid, stream))); break;
    default: KAI_TRY((launch_rows<8, 1>(p, vptr, vblocks, pvec, grid, stream))); break;
    }
    return check_launch(gv != nullptr ? "attention_backward_all_kernel" : "attention_backward_rows_kernel");
}

}  // namespace kai
