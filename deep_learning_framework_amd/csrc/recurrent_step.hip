// One time step of an LSTM or GRU layer in a single launch: the recurrent gate product
// r_prev[ndat, nrec] . Wr[NG*nrec, nrec]^T, both bias adds and the cell (vtensor.cpp:2468-2487 of the
// reference issues them as matmul, add_bias, add_bias, lstm_process / gru_process: three to four launches
// in a chain, each a few microseconds of work).
//
// A workgroup owns 16 rows x 16 units and ALL gates of those units, so that the cell can run on the
// gate sums without leaving the workgroup.  Wave w computes gate w % NG over the reduction steps of split
// w / NG (two splits; one and four measured slower): its 16 x 16 block with v_mfma_f32_16x16x4_f32, operands loaded straight from
// global memory in operand layout (row = lane % 16, k group = lane / 16, 16 B per lane: a step is at
// most a few hundred KB, all of it in L2 after the first workgroups).  The 2 x NG partial blocks meet in
// LDS once; 256 threads then finish one (row, unit) each: sum of the splits in fixed order, the input
// product, the biases, the cell.
#include "elementwise.h"

#include "act_funcs.h"

namespace kai {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kRsTile = 16;     // rows and units per workgroup
constexpr int kRsSplits = 2;    // waves along the reduction, per gate
// chunks of 16 reduction steps a wave keeps in flight: 4 or 8 (kRsFlight template parameter), the smaller one where it
// covers a wave's share in one round (a chunk past the end is loaded and multiplied all the same)

struct RecStepParams {
    float* r;              // [ndat, nrec] output of the step
    float* s;              // lstm: new state
    const float* s1;       // lstm: previous state or null (0)
    float* ai;             // [ndat, NG*nrec]: in: input products, out: what the cell saw (lstm: all sums)
    float* ar;             // gru: [ndat, 3*nrec] out: recurrent products + bias
    const float* wr;       // [NG*nrec, nrec]
    const float* r_prev;   // [ndat, nrec] operand of the recurrent product, null: no product (first step)
    const float* h_prev;   // gru: the output the update gate blends with, null: 0
    const float* bi;
    const float* br;
    int64_t ndat, nrec;
};

__device__ __forceinline__ float keep_bits(float x, int keep) { return __int_as_float(__float_as_int(x) & keep); }

template <int NG, int kRsFlight>
__global__ void __launch_bounds__(64 * NG * kRsSplits) recurrent_step_kernel(RecStepParams p) {
    __shared__ float part[kRsSplits][NG][kRsTile * kRsTile];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gate = wave % NG, split = wave / NG;
    const int r = lane & 15, g = lane >> 4;
    const int64_t tiles_u = (p.nrec + kRsTile - 1) / kRsTile;
    const int64_t row0 = (blockIdx.x / tiles_u) * kRsTile, u0 = (blockIdx.x % tiles_u) * kRsTile;
    const bool has_rec = p.r_prev != nullptr;   // the same for every thread
    // the threads that finish the cell fetch what it needs now, so that the product hides the latency
    const int64_t erow = row0 + (tid >> 4), eu = u0 + (tid & 15);
    const bool finishes = tid < kRsTile * kRsTile && erow < p.ndat && eu < p.nrec;
    const int64_t i = finishes ? erow * p.nrec + eu : 0;
    const int64_t gpos = finishes ? erow * NG * p.nrec + eu : 0;
    const int64_t eub = finishes ? eu : 0;
    float in_a[NG], in_bi[NG], in_br[NG];
    // (every thread loads, the ones that do not finish from position 0: loads under a per-thread condition
    // would be waited for one by one)
#pragma unroll
    for (int q = 0; q < NG; q++) {
        in_a[q] = p.ai[gpos + q * p.nrec];
        in_bi[q] = p.bi ? p.bi[q * p.nrec + eub] : 0.f;
        in_br[q] = p.br ? p.br[q * p.nrec + eub] : 0.f;
    }
    const float* prev = NG == 4 ? p.s1 : p.h_prev;
    const float in_prev = prev ? prev[i] : 0.f;
    if (has_rec) {
        const int64_t chunks = (p.nrec + 15) / 16, per = (chunks + kRsSplits - 1) / kRsSplits;
        const int64_t c0 = split * per, c1 = c0 + per < chunks ? c0 + per : chunks;
        // rows and units beyond the edge repeat the last valid one; their results are never stored
        const int64_t arow = row0 + r < p.ndat ? row0 + r : p.ndat - 1;
        const int64_t unit = u0 + r < p.nrec ? u0 + r : p.nrec - 1;
        const float* ap = p.r_prev + arow * p.nrec;
        const float* bp = p.wr + (gate * p.nrec + unit) * p.nrec;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int64_t c = c0; c < c1; c += kRsFlight) {
            f32x4 av[kRsFlight], bv[kRsFlight];
            int keep[kRsFlight];
            // every load is issued, at a clamped address; what lies beyond the reduction is masked afterwards
#pragma unroll
            for (int j = 0; j < kRsFlight; j++) {
                const int64_t k = (c + j) * 16 + 4 * g;          // nrec is a multiple of 4: k + 3 < nrec as well
                const bool valid = c + j < c1 && k < p.nrec;
                keep[j] = valid ? -1 : 0;
                const int64_t kc = valid ? k : 0;
                av[j] = *reinterpret_cast<const f32x4*>(ap + kc);
                bv[j] = *reinterpret_cast<const f32x4*>(bp + kc);
            }
            // every load of the round before the first product (the scheduler would sink them to their uses)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < kRsFlight; j++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float a = av[j][e], b = bv[j][e];
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(keep_bits(a, keep[j]), keep_bits(b, keep[j]), acc, 0, 0, 0);
                }
            }
        }
        // acc[v] = D[row 4 * g + v][unit r]
#pragma unroll
        for (int v = 0; v < 4; v++) part[split][gate][(4 * g + v) * kRsTile + r] = acc[v];
    }
    __syncthreads();
    if (!finishes) return;
    float dot[NG];
#pragma unroll
    for (int q = 0; q < NG; q++) {
        float d = 0.f;
        if (has_rec) {
#pragma unroll
            for (int sp = 0; sp < kRsSplits; sp++) d += part[sp][q][tid];
        }
        dot[q] = d;
    }
    if (NG == 4) {
        // lstm (vmath.cu:4807-4826): one buffer takes the input product, the recurrent product and both biases
        float pre[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            float v = in_a[q];
            if (has_rec) v += dot[q];
            if (p.br) v += in_br[q];
            if (p.bi) v += in_bi[q];
            p.ai[gpos + q * p.nrec] = v;
            pre[q] = v;
        }
        const float input_gate = act_sigmoid(pre[0]);
        const float forget_gate = act_sigmoid(pre[1]);
        const float input_block = act_tanh(pre[2]);
        const float output_gate = act_sigmoid(pre[3]);
        const float new_state = in_prev * forget_gate + input_block * input_gate;
        p.s[i] = new_state;
        p.r[i] = act_tanh(new_state) * output_gate;
    } else {
        // gru (vmath.cu:4946-4965): input and recurrent sums stay apart, the reset gate scales the recurrent candidate
        float vi[3], vr[3];
#pragma unroll
        for (int q = 0; q < 3; q++) {
            float a = in_a[q];
            if (p.bi) a += in_bi[q];
            float b = dot[q];
            if (p.br) b += in_br[q];
            p.ai[gpos + q * p.nrec] = a;
            p.ar[gpos + q * p.nrec] = b;
            vi[q] = a;
            vr[q] = b;
        }
        const float Rt = act_sigmoid(vi[0] + vr[0]);
        const float Zt = act_sigmoid(vi[1] + vr[1]);
        const float Nt = act_tanh(vi[2] + Rt * vr[2]);
        p.r[i] = (1.0f - Zt) * Nt + Zt * in_prev;
    }
}

template <int NG>
int launch_step(const RecStepParams& p, hipStream_t stream) {
    const int64_t blocks = ((p.ndat + kRsTile - 1) / kRsTile) * ((p.nrec + kRsTile - 1) / kRsTile);
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "recurrent step: too many tiles");
    const int64_t chunks = (p.nrec + 15) / 16, per = (chunks + kRsSplits - 1) / kRsSplits;
    if (per <= 4) recurrent_step_kernel<NG, 4><<<dim3((unsigned)blocks), dim3(64 * NG * kRsSplits), 0, stream>>>(p);
    else recurrent_step_kernel<NG, 8><<<dim3((unsigned)blocks), dim3(64 * NG * kRsSplits), 0, stream>>>(p);
    return check_launch("recurrent_step_kernel");
}

}  // namespace

bool recurrent_step_applies(const float* wr, const float* r_prev, int64_t ndat, int64_t nrec) {
    // operands are read 16 bytes at a time; beyond these sizes the tiled product of the separate calls
    // re-reads less of Wr than 16-row workgroups do
    return ndat >= 1 && nrec >= 4 && nrec % 4 == 0 && aligned16(wr) && (r_prev == nullptr || aligned16(r_prev)) &&
           ndat <= kRecStepMaxRows && nrec <= kRecStepMaxUnits;
}

int launch_lstm_step(float* r, float* s, const float* s1, float* a, const float* wr, const float* r_prev,
                     const float* bi, const float* br, int64_t ndat, int64_t nrec, hipStream_t stream) {
    RecStepParams p{r, s, s1, a, nullptr, wr, r_prev, nullptr, bi, br, ndat, nrec};
    return launch_step<4>(p, stream);
}

int launch_gru_step(float* r, float* ai, float* ar, const float* wr, const float* r_prev, const float* h_prev,
                    const float* bi, const float* br, int64_t ndat, int64_t nrec, hipStream_t stream) {
    RecStepParams p{r, nullptr, nullptr, ai, ar, wr, r_prev, h_prev, bi, br, ndat, nrec};
    return launch_step<3>(p, stream);
}

}  // namespace kai
