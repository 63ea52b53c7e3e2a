// Bandwidth-bound companions of the dense layer: bias add, bias gradient (column sum),
// activations and their derivatives, fills.  Reference: VMath::add_bias /
// add_bias_backward_b (vmath.cu:875-932), activate / activate_backward /
// activate_backward_with_y (vmath.cu:3097-3486), fill_int / fill_float (vmath.cu:494-530).
//
// All kernels are grid-stride streams with 128-bit accesses when the buffers allow it.
#include "elementwise.h"

#include <float.h>

#include "act_funcs.h"

namespace kai {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kEwThreads = 256;
constexpr int kMaxBlocks = 256 * 16;   // 16 workgroups per CU keep every CU's queues full

static unsigned blocks_for(int64_t work_items) {
    int64_t b = (work_items + kEwThreads - 1) / kEwThreads;
    if (b < 1) b = 1;
    if (b > kMaxBlocks) b = kMaxBlocks;
    return (unsigned)b;
}

// ---- add_bias ---------------------------------------------------------------------------------

template <bool VEC>
__global__ void __launch_bounds__(kEwThreads) add_bias_kernel(float* y, const float* a,
                                                              const float* __restrict__ b, int64_t total,
                                                              int64_t ncol) {
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (VEC) {
        const int64_t nvec = total / 4;   // ncol % 4 == 0, so a chunk never crosses a row
        for (; i < nvec; i += stride) {
            const int64_t e = i * 4;
            const int64_t c = e % ncol;
            const f32x4 va = *reinterpret_cast<const f32x4*>(a + e);
            const f32x4 vb = *reinterpret_cast<const f32x4*>(b + c);
            *reinterpret_cast<f32x4*>(y + e) = va + vb;
        }
    } else {
        for (; i < total; i += stride) y[i] = a[i] + b[i % ncol];
    }
}

int launch_add_bias(float* y, const float* a, const float* b, int64_t nrow, int64_t ncol, hipStream_t stream) {
    const int64_t total = nrow * ncol;
    if (total <= 0) return KAI_OK;
    const bool vec = ncol % 4 == 0 && aligned16(y) && aligned16(a) && aligned16(b);
    if (vec)
        add_bias_kernel<true><<<blocks_for(total / 4), kEwThreads, 0, stream>>>(y, a, b, total, ncol);
    else
        add_bias_kernel<false><<<blocks_for(total), kEwThreads, 0, stream>>>(y, a, b, total, ncol);
    return check_launch("add_bias_kernel");
}

// ---- add_bias_backward_b: gb[c] (=|+=) sum_r gy[r,c] -------------------------------------------
//
// One workgroup owns a panel of 32 columns (one 128-byte line per row) and all rows: thread
// (ty, tx) sums rows ty, ty+32, ... of column tx, then the 32 partial sums of a column are
// folded through LDS in a fixed order, so the result does not depend on scheduling.

constexpr int kColsumCols = 32;
constexpr int kColsumRows = 32;

__global__ void __launch_bounds__(kColsumCols* kColsumRows)
    colsum_kernel(float* __restrict__ gb, const float* __restrict__ gy, int64_t nrow_all, int64_t ncol, int acc,
                  int64_t rows_per_part) {
    __shared__ float part[kColsumRows][kColsumCols + 1];
    const int tx = threadIdx.x % kColsumCols;
    const int ty = threadIdx.x / kColsumCols;
    const int64_t c = (int64_t)blockIdx.x * kColsumCols + tx;
    // blockIdx.y: a run of rows_per_part rows whose sums go to row blockIdx.y of gb (one run: gb itself)
    const int64_t r_first = (int64_t)blockIdx.y * rows_per_part;
    const int64_t nrow = min(nrow_all, r_first + rows_per_part);
    gb += (int64_t)blockIdx.y * ncol;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (c < ncol) {
        const float* __restrict__ p = gy + c;
        int64_t r = r_first + ty;
        for (; r + 3 * kColsumRows < nrow; r += 4 * kColsumRows) {
            s0 += p[r * ncol];
            s1 += p[(r + kColsumRows) * ncol];
            s2 += p[(r + 2 * kColsumRows) * ncol];
            s3 += p[(r + 3 * kColsumRows) * ncol];
        }
        for (; r < nrow; r += kColsumRows) s0 += p[r * ncol];
    }
    part[ty][tx] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (ty == 0 && c < ncol) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < kColsumRows; i++) s += part[i][tx];
        if (acc) s += gb[c];
        gb[c] = s;
    }
}

// Few columns and many rows (the bias gradient of a narrow output layer over a long batch): one workgroup per 32
// columns walks all the rows alone, [100000, 12] took 249 us.  The rows are then cut into runs, one workgroup per run
// and column block, and a second launch adds the runs' sums.
int colsum_row_parts(int64_t nrow, int64_t ncol) {
    const int64_t blocks = (ncol + kColsumCols - 1) / kColsumCols;
    const int64_t cus = compute_units();
    if (blocks * 2 > cus || nrow < 6144) return 1;   // shorter: the second launch costs what the runs save
    int64_t parts = 4 * cus / blocks;
    if (parts > nrow / 256) parts = nrow / 256;
    if (parts > 512) parts = 512;
    return parts < 2 ? 1 : (int)parts;
}

int launch_colsum(float* gb, const float* gy, int64_t nrow, int64_t ncol, int acc, hipStream_t stream, float* parts_buf,
                  int parts) {
    if (ncol <= 0) return KAI_OK;
    const int64_t blocks = (ncol + kColsumCols - 1) / kColsumCols;
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "add_bias_backward_b: too many columns");
    if (parts < 2 || parts_buf == nullptr) {
        colsum_kernel<<<dim3((unsigned)blocks), dim3(kColsumCols * kColsumRows), 0, stream>>>(gb, gy, nrow, ncol, acc, nrow);
        return check_launch("colsum_kernel");
    }
    const int64_t rows_per_part = ((nrow + parts - 1) / parts + kColsumRows - 1) / kColsumRows * kColsumRows;
    const int nparts = (int)((nrow + rows_per_part - 1) / rows_per_part);
    colsum_kernel<<<dim3((unsigned)blocks, (unsigned)nparts), dim3(kColsumCols * kColsumRows), 0, stream>>>(
        parts_buf, gy, nrow, ncol, 0, rows_per_part);
    KAI_TRY(check_launch("colsum_kernel"));
    // the runs' sums are a matrix of nparts rows: the same kernel adds them up, in its fixed order
    colsum_kernel<<<dim3((unsigned)blocks), dim3(kColsumCols * kColsumRows), 0, stream>>>(gb, parts_buf, nparts, ncol, acc, nparts);
    return check_launch("colsum_kernel");
}

// ---- element-wise activations -------------------------------------------------------------------

// MODE 0: y = f(x);  MODE 1: gx = f'(x) * gy;  MODE 2: gx = f'(y) * gy (derivative from the output)
template <int MODE, bool VEC>
__global__ void __launch_bounds__(kEwThreads) act_kernel(float* out, const float* g,
                                                         const float* in, int64_t total, int act,
                                                         const float* __restrict__ hleaky) {
    const float leaky = hleaky ? *hleaky : 0.f;
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    auto f = [&](float x, float gy) -> float {
        if (MODE == 0) return apply_act(x, act, leaky);
        if (MODE == 1) return act_derivative(x, act, leaky) * gy;
        return act_derivative_from_y(x, act, leaky) * gy;
    };
    if (VEC) {
        const int64_t nvec = total / 4;
        for (; i < nvec; i += stride) {
            const f32x4 x = *reinterpret_cast<const f32x4*>(in + i * 4);
            f32x4 gy = {0.f, 0.f, 0.f, 0.f};
            if (MODE != 0) gy = *reinterpret_cast<const f32x4*>(g + i * 4);
            f32x4 o;
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = f(x[j], gy[j]);
            *reinterpret_cast<f32x4*>(out + i * 4) = o;
        }
        // tail (total % 4 elements)
        const int64_t t = nvec * 4 + (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
        if (t < total) out[t] = f(in[t], MODE != 0 ? g[t] : 0.f);
    } else {
        for (; i < total; i += stride) out[i] = f(in[i], MODE != 0 ? g[i] : 0.f);
    }
}

template <int MODE>
static int launch_act_mode(float* out, const float* g, const float* in, int64_t total, int act, const float* hleaky,
                           hipStream_t stream) {
    if (total <= 0) return KAI_OK;
    const bool vec = aligned16(out) && aligned16(in) && (MODE == 0 || aligned16(g)) && total >= 4;
    if (vec)
        act_kernel<MODE, true><<<blocks_for(total / 4), kEwThreads, 0, stream>>>(out, g, in, total, act, hleaky);
    else
        act_kernel<MODE, false><<<blocks_for(total), kEwThreads, 0, stream>>>(out, g, in, total, act, hleaky);
    return check_launch("act_kernel");
}

int launch_activate(float* y, const float* x, int64_t total, int act, const float* hleaky, hipStream_t stream) {
    return launch_act_mode<0>(y, nullptr, x, total, act, hleaky, stream);
}
int launch_activate_backward(float* gx, const float* gy, const float* x, int64_t total, int act, const float* hleaky,
                             hipStream_t stream) {
    return launch_act_mode<1>(gx, gy, x, total, act, hleaky, stream);
}
int launch_activate_backward_with_y(float* gx, const float* gy, const float* y, int64_t total, int act,
                                    const float* hleaky, hipStream_t stream) {
    return launch_act_mode<2>(gx, gy, y, total, act, hleaky, stream);
}

// ---- softmax as an activation (row of ncol contiguous elements) ---------------------------------
//
// One wave per row.  Forward: y = exp(x - max) / sum.  Backward (device twin of the reference,
// vmath.cu:3363-3394): gx_i = y_i * (gy_i - sum_j y_j gy_j), written there as
// sum_j (delta_ij y_i - y_i y_j) gy_j.

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_add(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <bool BACKWARD>
__global__ void __launch_bounds__(kEwThreads) softmax_rows_kernel(float* __restrict__ out,
                                                                  const float* __restrict__ gy,
                                                                  const float* __restrict__ x, int64_t nrow,
                                                                  int64_t ncol) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kEwThreads / 64) + (threadIdx.x >> 6);
    if (row >= nrow) return;
    const float* __restrict__ xr = x + row * ncol;
    float mx = -FLT_MAX;
    for (int64_t c = lane; c < ncol; c += 64) mx = fmaxf(mx, xr[c]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int64_t c = lane; c < ncol; c += 64) sum += expf(xr[c] - mx);
    sum = wave_add(sum);
    if (!BACKWARD) {
        for (int64_t c = lane; c < ncol; c += 64) out[row * ncol + c] = expf(xr[c] - mx) / sum;
    } else {
        const float* __restrict__ gr = gy + row * ncol;
        float dot = 0.f;
        for (int64_t c = lane; c < ncol; c += 64) dot += (expf(xr[c] - mx) / sum) * gr[c];
        dot = wave_add(dot);
        for (int64_t c = lane; c < ncol; c += 64) {
            const float yi = expf(xr[c] - mx) / sum;
            out[row * ncol + c] = yi * gr[c] - yi * dot;
        }
    }
}

// The same with the row in a wave's registers (ncol <= 64 * E): one read of x, one expf per element, the three
// loops of the kernel above become one load, one store; up to 4096 columns (E = 64).
template <bool BACKWARD, int E>
__global__ void __launch_bounds__(kEwThreads) softmax_rows_reg_kernel(float* __restrict__ out,
                                                                      const float* __restrict__ gy,
                                                                      const float* __restrict__ x, int64_t nrow,
                                                                      int64_t ncol) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kEwThreads / 64) + (threadIdx.x >> 6);
    if (row >= nrow) return;
    const float* __restrict__ xr = x + row * ncol;
    float v[E], gr[E];
    float mx = -FLT_MAX;
#pragma unroll
    for (int i = 0; i < E; i++) {
        const int64_t c = lane + 64 * i;
        v[i] = c < ncol ? xr[c] : -INFINITY;
        if (BACKWARD) gr[i] = c < ncol ? gy[row * ncol + c] : 0.f;
        mx = fmaxf(mx, v[i]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < E; i++) {
        v[i] = lane + 64 * i < ncol ? expf(v[i] - mx) : 0.f;
        sum += v[i];
    }
    sum = wave_add(sum);
    if (!BACKWARD) {
#pragma unroll
        for (int i = 0; i < E; i++)
            if (lane + 64 * i < ncol) out[row * ncol + lane + 64 * i] = v[i] / sum;
    } else {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < E; i++) {
            v[i] = v[i] / sum;
            dot += v[i] * gr[i];
        }
        dot = wave_add(dot);
#pragma unroll
        for (int i = 0; i < E; i++)
            if (lane + 64 * i < ncol) out[row * ncol + lane + 64 * i] = v[i] * gr[i] - v[i] * dot;
    }
}

// Short rows (ncol <= G = 2 ... 32): 64 / G rows per wave, the folds stay inside a row's G lanes.  A wave per row
// leaves 52 of 64 lanes idle on the 12 classes of an output layer ([100000, 12] 16 us).
template <bool BACKWARD, int G>
__global__ void __launch_bounds__(kEwThreads) softmax_rows_short_kernel(float* __restrict__ out,
                                                                        const float* __restrict__ gy,
                                                                        const float* __restrict__ x, int64_t nrow,
                                                                        int64_t ncol) {
    const int lane = threadIdx.x & 63, col = lane % G;
    const int64_t wave = (int64_t)blockIdx.x * (kEwThreads / 64) + (threadIdx.x >> 6);
    const int64_t row = wave * (64 / G) + lane / G;
    const bool live = row < nrow && col < ncol;      // no early exit: every lane takes part in the shuffles
    const int64_t at = live ? row * ncol + col : 0;
    const float v = live ? x[at] : -INFINITY;
    float mx = fmaxf(v, -FLT_MAX);
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    const float e = live ? expf(v - mx) : 0.f;
    float sum = e;
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (!BACKWARD) {
        if (live) out[at] = e / sum;
    } else {
        const float yi = live ? e / sum : 0.f;
        const float g = live ? gy[at] : 0.f;
        float dot = yi * g;
#pragma unroll
        for (int off = G / 2; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
        if (live) out[at] = yi * g - yi * dot;
    }
}

template <bool BACKWARD, int G>
static int launch_softmax_rows_short(float* out, const float* gy, const float* x, int64_t nrow, int64_t ncol,
                                     hipStream_t stream) {
    const int64_t rows_per_block = (kEwThreads / 64) * (64 / G);
    const int64_t blocks = (nrow + rows_per_block - 1) / rows_per_block;
    softmax_rows_short_kernel<BACKWARD, G><<<dim3((unsigned)blocks), kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    return check_launch("softmax_rows_short_kernel");
}

// Long rows, or few of them: a workgroup of 1024 threads per row, the three passes of the first kernel with
// block-wide reductions (a row of 50257 floats is 200 KB: it comes from L2 on the second and third pass).  One wave
// per row left [64, 50257] on 64 waves: 368 us.
constexpr int kSmxThreads = 1024;
template <bool BACKWARD>
__global__ void __launch_bounds__(kSmxThreads) softmax_rows_block_kernel(float* __restrict__ out,
                                                                         const float* __restrict__ gy,
                                                                         const float* __restrict__ x, int64_t ncol) {
    __shared__ float red[3][kSmxThreads / 64];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int64_t row = blockIdx.x;
    const float* __restrict__ xr = x + row * ncol;
    auto block_fold = [&](float mine, bool is_max, int which) -> float {
        mine = is_max ? wave_max(mine) : wave_add(mine);
        if (lane == 0) red[which][wave] = mine;
        __syncthreads();
        float a = red[which][0];
        for (int w = 1; w < kSmxThreads / 64; w++) a = is_max ? fmaxf(a, red[which][w]) : a + red[which][w];
        return a;
    };
    float mx = -FLT_MAX;
    for (int64_t c = t; c < ncol; c += kSmxThreads) mx = fmaxf(mx, xr[c]);
    mx = block_fold(mx, true, 0);
    float sum = 0.f;
    for (int64_t c = t; c < ncol; c += kSmxThreads) sum += expf(xr[c] - mx);
    sum = block_fold(sum, false, 1);
    if (!BACKWARD) {
        for (int64_t c = t; c < ncol; c += kSmxThreads) out[row * ncol + c] = expf(xr[c] - mx) / sum;
    } else {
        const float* __restrict__ gr = gy + row * ncol;
        float dot = 0.f;
        for (int64_t c = t; c < ncol; c += kSmxThreads) dot += (expf(xr[c] - mx) / sum) * gr[c];
        dot = block_fold(dot, false, 2);
        for (int64_t c = t; c < ncol; c += kSmxThreads) {
            const float yi = expf(xr[c] - mx) / sum;
            out[row * ncol + c] = yi * gr[c] - yi * dot;
        }
    }
}

// A workgroup per row with the row in its registers (ncol <= 1024 * E, up to 16384 columns): one read of x and one
// expf per element where the kernel above has three and two ([8192, 8192] 215 us there).
// KEEP_G (the derivative only): the incoming gradient waits in registers next to the row; without it the gradient is
// read a second time for the last pass (from L2: a row of 65536 floats is 256 KB), which leaves room for rows twice
// as long.
template <bool BACKWARD, int E, bool KEEP_G = true>
__global__ void __launch_bounds__(kSmxThreads) softmax_rows_block_reg_kernel(float* __restrict__ out,
                                                                             const float* __restrict__ gy,
                                                                             const float* __restrict__ x, int64_t ncol) {
    __shared__ float red[3][kSmxThreads / 64];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int64_t row = blockIdx.x;
    const float* __restrict__ xr = x + row * ncol;
    auto block_fold = [&](float mine, bool is_max, int which) -> float {
        mine = is_max ? wave_max(mine) : wave_add(mine);
        if (lane == 0) red[which][wave] = mine;
        __syncthreads();
        float a = red[which][0];
        for (int w = 1; w < kSmxThreads / 64; w++) a = is_max ? fmaxf(a, red[which][w]) : a + red[which][w];
        return a;
    };
    float v[E], gr[KEEP_G ? E : 1];
    float mx = -FLT_MAX;
#pragma unroll
    for (int i = 0; i < E; i++) {
        const int64_t c = t + kSmxThreads * i;
        v[i] = c < ncol ? xr[c] : -INFINITY;
        if (BACKWARD && KEEP_G) gr[i] = c < ncol ? gy[row * ncol + c] : 0.f;
        mx = fmaxf(mx, v[i]);
    }
    mx = block_fold(mx, true, 0);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < E; i++) {
        v[i] = t + kSmxThreads * i < ncol ? expf(v[i] - mx) : 0.f;
        sum += v[i];
    }
    sum = block_fold(sum, false, 1);
    if (!BACKWARD) {
#pragma unroll
        for (int i = 0; i < E; i++)
            if (t + kSmxThreads * i < ncol) out[row * ncol + t + kSmxThreads * i] = v[i] / sum;
    } else {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < E; i++) {
            v[i] = v[i] / sum;
            if (KEEP_G) dot += v[i] * gr[i];
            else if (t + kSmxThreads * i < ncol) dot += v[i] * gy[row * ncol + t + kSmxThreads * i];
        }
        dot = block_fold(dot, false, 2);
#pragma unroll
        for (int i = 0; i < E; i++)
            if (t + kSmxThreads * i < ncol) {
                const float g = KEEP_G ? gr[i] : gy[row * ncol + t + kSmxThreads * i];
                out[row * ncol + t + kSmxThreads * i] = v[i] * g - v[i] * dot;
            }
    }
}

// which of the four: rows of up to 4096 columns in registers, one wave each; longer rows, and rows of 1024 columns
// and more when there are fewer rows than waves that the compute units hold, a workgroup each (in its registers up
// to 16384 columns); else the first kernel
template <bool BACKWARD>
static int launch_softmax_rows_impl(float* out, const float* gy, const float* x, int64_t nrow, int64_t ncol,
                                    hipStream_t stream) {
    const int64_t blocks = (nrow + kEwThreads / 64 - 1) / (kEwThreads / 64);
    if (blocks > kMaxDim || nrow > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "activate(softmax): too many rows");
    const bool few_rows = nrow < 8 * (int64_t)compute_units();
    // (a vocabulary of 50257 columns: 50 registers per thread forward; the derivative holds two rows and stays within
    // a thread's 128 registers up to 32 per row: beyond, it keeps the row and reads the gradient twice)
    constexpr int kRegCols = 64 * kSmxThreads;
    if ((ncol > 4096 || (few_rows && ncol >= 1024)) && ncol <= kRegCols) {
        const dim3 g((unsigned)nrow);
        if (ncol <= 4096) softmax_rows_block_reg_kernel<BACKWARD, 4><<<g, kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        else if (ncol <= 8192) softmax_rows_block_reg_kernel<BACKWARD, 8><<<g, kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        else if (ncol <= 12288) softmax_rows_block_reg_kernel<BACKWARD, 12><<<g, kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        else if (ncol <= 16384) softmax_rows_block_reg_kernel<BACKWARD, 16><<<g, kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        else if (ncol <= 32768) softmax_rows_block_reg_kernel<BACKWARD, 32><<<g, kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        else if (ncol <= 53248) softmax_rows_block_reg_kernel<BACKWARD, 52, !BACKWARD><<<g, kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        else softmax_rows_block_reg_kernel<BACKWARD, 64, !BACKWARD><<<g, kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        return check_launch("softmax_rows_block_reg_kernel");
    }
    if (ncol > 4096 || (few_rows && ncol >= 1024)) {
        softmax_rows_block_kernel<BACKWARD><<<dim3((unsigned)nrow), kSmxThreads, 0, stream>>>(out, gy, x, ncol);
        return check_launch("softmax_rows_block_kernel");
    }
    if (ncol <= 2) return launch_softmax_rows_short<BACKWARD, 2>(out, gy, x, nrow, ncol, stream);
    if (ncol <= 4) return launch_softmax_rows_short<BACKWARD, 4>(out, gy, x, nrow, ncol, stream);
    if (ncol <= 8) return launch_softmax_rows_short<BACKWARD, 8>(out, gy, x, nrow, ncol, stream);
    if (ncol <= 16) return launch_softmax_rows_short<BACKWARD, 16>(out, gy, x, nrow, ncol, stream);
    if (ncol <= 32) return launch_softmax_rows_short<BACKWARD, 32>(out, gy, x, nrow, ncol, stream);
    const dim3 g((unsigned)blocks);
    if (ncol <= 64) softmax_rows_reg_kernel<BACKWARD, 1><<<g, kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    else if (ncol <= 128) softmax_rows_reg_kernel<BACKWARD, 2><<<g, kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    else if (ncol <= 256) softmax_rows_reg_kernel<BACKWARD, 4><<<g, kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    else if (ncol <= 512) softmax_rows_reg_kernel<BACKWARD, 8><<<g, kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    else if (ncol <= 1024) softmax_rows_reg_kernel<BACKWARD, 16><<<g, kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    else if (ncol <= 2048) softmax_rows_reg_kernel<BACKWARD, 32><<<g, kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    else softmax_rows_reg_kernel<BACKWARD, 64><<<g, kEwThreads, 0, stream>>>(out, gy, x, nrow, ncol);
    return check_launch("softmax_rows_reg_kernel");
}

int launch_softmax_rows(float* y, const float* x, int64_t nrow, int64_t ncol, hipStream_t stream) {
    if (nrow <= 0 || ncol <= 0) return KAI_OK;
    if (y != x) return launch_softmax_rows_impl<false>(y, nullptr, x, nrow, ncol, stream);
    const int64_t blocks = (nrow + kEwThreads / 64 - 1) / (kEwThreads / 64);
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "activate(softmax): too many rows");
    softmax_rows_kernel<false><<<dim3((unsigned)blocks), kEwThreads, 0, stream>>>(y, nullptr, x, nrow, ncol);
    return check_launch("softmax_rows_kernel");
}

int launch_softmax_rows_backward(float* gx, const float* gy, const float* x, int64_t nrow, int64_t ncol,
                                 hipStream_t stream) {
    if (nrow <= 0 || ncol <= 0) return KAI_OK;
    if (gx != x && gx != gy) return launch_softmax_rows_impl<true>(gx, gy, x, nrow, ncol, stream);
    const int64_t blocks = (nrow + kEwThreads / 64 - 1) / (kEwThreads / 64);
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "activate_backward(softmax): too many rows");
    softmax_rows_kernel<true><<<dim3((unsigned)blocks), kEwThreads, 0, stream>>>(gx, gy, x, nrow, ncol);
    return check_launch("softmax_rows_kernel");
}

// ---- fills ----------------------------------------------------------------------------------------

template <typename T>
__global__ void __launch_bounds__(kEwThreads) fill_kernel(T* __restrict__ p, int64_t n, T value) {
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) p[i] = value;
}

int launch_fill_float(float* p, int64_t n, float value, hipStream_t stream) {
    if (n <= 0) return KAI_OK;
    fill_kernel<float><<<blocks_for(n), kEwThreads, 0, stream>>>(p, n, value);
    return check_launch("fill_kernel");
}

int launch_fill_int(int* p, int64_t n, int value, hipStream_t stream) {
    if (n <= 0) return KAI_OK;
    fill_kernel<int><<<blocks_for(n), kEwThreads, 0, stream>>>(p, n, value);
    return check_launch("fill_kernel");
}

// ---- transposes -------------------------------------------------------------------------------------
//
// transpose_bin: y[nrow, ncol] = x[ncol, nrow]^T through a 32 x 33 LDS tile, so that both the reads and
// the writes are 128-byte rows.  transpose / transpose_backward: the engine's general axis permutation,
// driven by its device table (per output axis: source axis, output elements per step, and per SOURCE
// axis: source elements per step); a thread owns one output element, writes (forward) or reads
// (backward) are contiguous, the other side is a gather or scatter.

constexpr int kTrTile = 32;
constexpr int kTrMaxAxes = 8;

__global__ void __launch_bounds__(kTrTile * 8) transpose_bin_kernel(float* __restrict__ y, const float* __restrict__ x,
                                                                    int64_t nrow, int64_t ncol, int64_t tiles_c) {
    __shared__ float tile[kTrTile][kTrTile + 1];
    const int64_t tr = blockIdx.x / tiles_c, tc = blockIdx.x % tiles_c;   // tile of y: rows tr*32.., columns tc*32..
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;              // 32 x 8 threads
    // x is [ncol, nrow]: read rows c of x (contiguous along r)
#pragma unroll
    for (int i = 0; i < kTrTile; i += 8) {
        const int64_t c = tc * kTrTile + ty + i, r = tr * kTrTile + tx;
        if (c < ncol && r < nrow) tile[ty + i][tx] = x[c * nrow + r];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kTrTile; i += 8) {
        const int64_t r = tr * kTrTile + ty + i, c = tc * kTrTile + tx;
        if (r < nrow && c < ncol) __builtin_nontemporal_store(tile[tx][ty + i], y + r * ncol + c);
    }
}

int launch_transpose_bin(float* y, const float* x, int64_t nrow, int64_t ncol, hipStream_t stream) {
    if (nrow <= 0 || ncol <= 0) return KAI_OK;
    const int64_t tiles_r = (nrow + kTrTile - 1) / kTrTile, tiles_c = (ncol + kTrTile - 1) / kTrTile;
    if (tiles_r * tiles_c > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "transpose_bin: matrix too large");
    transpose_bin_kernel<<<dim3((unsigned)(tiles_r * tiles_c)), kTrTile * 8, 0, stream>>>(y, x, nrow, ncol, tiles_c);
    return check_launch("transpose_bin_kernel");
}

// The index arithmetic of one element (or one group of four): output position -> source position through the
// table, with 32-bit integers where the tensor allows it (a 64-bit division costs several times a 32-bit one, and
// there is one per axis and element).
template <typename I, bool BACKWARD, bool VEC>
__device__ __forceinline__ void transpose_axes_body(float* __restrict__ out, const float* __restrict__ in,
                                                    const int64_t* yblk64, const int64_t* xblk64, int axis_size, int64_t n) {
    I yblk[kTrMaxAxes], xblk[kTrMaxAxes];
#pragma unroll
    for (int m = 0; m < kTrMaxAxes; m++) {
        yblk[m] = m < axis_size ? (I)yblk64[m] : (I)1;
        xblk[m] = m < axis_size ? (I)xblk64[m] : (I)0;
    }
    const I count = (I)(VEC ? n / 4 : n);
    const I stride = (I)gridDim.x * kEwThreads;
    for (I i = (I)blockIdx.x * kEwThreads + threadIdx.x; i < count; i += stride) {
        I xpos = 0, ypos = VEC ? i * 4 : i;
#pragma unroll
        for (int m = 0; m < kTrMaxAxes; m++) {      // written out: the table stays in registers
            if (m < axis_size) {
                const I c = ypos / yblk[m];
                ypos -= c * yblk[m];
                xpos += c * xblk[m];
            }
        }
        if (VEC) {
            // four consecutive elements of the innermost axis, which is the innermost axis on both sides
            const I o = i * 4;
            if (BACKWARD) *reinterpret_cast<f32x4*>(out + xpos) = *reinterpret_cast<const f32x4*>(in + o);
            else *reinterpret_cast<f32x4*>(out + o) = *reinterpret_cast<const f32x4*>(in + xpos);
        } else {
            if (BACKWARD) out[xpos] = in[i];
            else out[i] = in[xpos];
        }
    }
}

// The innermost output axis is NOT the innermost source axis (a matrix transposed through the general entry point,
// channels first <-> channels last, [B, T, H, D] -> [B, H, D, T]): element by element one side is a gather or scatter
// with a stride of whole rows (4096 x 4096: 67 us, 2.0 TB/s; [64, 512, 12, 64] -> [64, 12, 64, 512] backward 301 us).
// Here a workgroup moves tiles of TI positions of the innermost output axis (source step s_i) x TJ positions of the
// innermost source axis (output axis mj, output step y_j) through LDS, so that it reads runs along one and writes
// runs along the other; TI x TJ = 1024, the side of a short axis (3 channels) shrinks to 4 / 8 / 16 and the other
// grows.  The remaining axes are counted through per tile.
constexpr int kTrTileFloats = 1024 + 256;
// (tensors below 2^31 elements: everything counts in 32 bits; the table stays in LDS -- osz = positions per output
// axis -- and is read once per tile, so that this path adds no registers to the kernel it shares with the loops above)
template <bool BACKWARD>
__device__ __forceinline__ void transpose_axes_tiled(float* __restrict__ out, const float* __restrict__ in,
                                                     const int64_t* yblk, const int64_t* xblk, const int* osz,
                                                     int axis_size, int mj, float* tile) {
    auto uniform = [](int64_t v) -> int { return __builtin_amdgcn_readfirstlane((int)v); };
    const int last = axis_size - 1;
    mj = __builtin_amdgcn_readfirstlane(mj);
    const int len_i = uniform(osz[last]), len_j = uniform(osz[mj]);
    const int s_i = uniform(xblk[last]), y_j = uniform(yblk[mj]);
    int log_ti = len_i <= 4 ? 2 : len_i <= 8 ? 3 : len_i <= 16 ? 4 : 5;
    if (len_j <= 16 && len_i > 16) log_ti = len_j <= 4 ? 8 : len_j <= 8 ? 7 : 6;
    const int log_tj = 10 - log_ti;
    const int ti_size = 1 << log_ti, tj_size = 1 << log_tj, pitch = tj_size + 1;
    const int tiles_i = (len_i + ti_size - 1) >> log_ti, tiles_j = (len_j + tj_size - 1) >> log_tj;
    int outer = 1;
    for (int m = 0; m < last; m++)
        if (m != mj) outer *= uniform(osz[m]);
    const int tiles = outer * tiles_i * tiles_j;   // at most n / 4: a tile side is 4 at least
    const int tid = threadIdx.x;
    for (int t = blockIdx.x; t < tiles; t += gridDim.x) {
        const int ti = t % tiles_i, rest = t / tiles_i;
        const int tj = rest % tiles_j;
        int o = rest / tiles_j, ybase = 0, xbase = 0;
        for (int m = last - 1; m >= 0; m--) {
            if (m != mj) {
                const int sz = uniform(osz[m]);
                const int c = o % sz;
                o /= sz;
                ybase += c * uniform(yblk[m]);
                xbase += c * uniform(xblk[m]);
            }
        }
        const int i0 = ti << log_ti, j0 = tj << log_tj;
        const int ni = min(ti_size, len_i - i0), nj = min(tj_size, len_j - j0);
        const float* __restrict__ src_x = in + (xbase + i0 * s_i + j0);      // forward: in is the source tensor
        float* __restrict__ dst_y = out + (ybase + j0 * y_j + i0);
        const float* __restrict__ src_y = in + (ybase + j0 * y_j + i0);      // backward: in is laid out like the output
        float* __restrict__ dst_x = out + (xbase + i0 * s_i + j0);
        // runs along j (the source's rows)
        auto along_j = [&](auto body) {
#pragma unroll
            for (int idx = tid; idx < 1024; idx += kEwThreads) {
                const int ii = idx >> log_tj, jj = idx & (tj_size - 1);
                if (ii < ni && jj < nj) body(ii, jj);
            }
        };
        // runs along i (the output's rows)
        auto along_i = [&](auto body) {
#pragma unroll
            for (int idx = tid; idx < 1024; idx += kEwThreads) {
                const int jj = idx >> log_ti, ii = idx & (ti_size - 1);
                if (ii < ni && jj < nj) body(ii, jj);
            }
        };
        if (!BACKWARD) {
            along_j([&](int ii, int jj) { tile[ii * pitch + jj] = src_x[ii * s_i + jj]; });
            __syncthreads();
            along_i([&](int ii, int jj) { __builtin_nontemporal_store(tile[ii * pitch + jj], dst_y + (jj * y_j + ii)); });
        } else {
            along_i([&](int ii, int jj) { tile[ii * pitch + jj] = src_y[jj * y_j + ii]; });
            __syncthreads();
            along_j([&](int ii, int jj) { __builtin_nontemporal_store(tile[ii * pitch + jj], dst_x + (ii * s_i + jj)); });
        }
        __syncthreads();   // the tile is free for the next one
    }
}

// The table lives in device memory (the engine builds it there), so the kernel itself looks whether the innermost
// output axis is the innermost source axis (the head split / merge [B, T, H, D] <-> [B, H, T, D] of the attention
// layers and every permutation of outer axes): then whole 128-bit words move, the innermost 4 * k floats being
// contiguous on both sides.  `aligned16` is the host's check of the two base pointers.
template <bool BACKWARD>
__global__ void __launch_bounds__(kEwThreads) transpose_axes_kernel(float* __restrict__ out,
                                                                    const float* __restrict__ in,
                                                                    const int* __restrict__ pn, int axis_size,
                                                                    int64_t n, int aligned16) {
    // the table is tiny and the same for every thread; thread m reads the row of output axis m and leaves what the
    // choice among the loops needs as bits, so that no thread walks the table again:
    //   bit 1: the axis allows 128-bit moves (steps in whole fours; the last axis: innermost on both sides)
    //   bit 2: the axis allows the tiles (only the last one can forbid them: it must be innermost in the output only)
    //   bit 0, with m in the bits above: the axis walks the source's innermost axis and has more than one position
    __shared__ int64_t yblk[kTrMaxAxes], xblk[kTrMaxAxes];
    __shared__ int osz[kTrMaxAxes];   // positions per output axis (where the tensor counts in 32 bits)
    __shared__ __attribute__((aligned(16))) int flags[kTrMaxAxes];
    const bool small = n < (1ll << 31);
    const int last = axis_size - 1;
    if (threadIdx.x < kTrMaxAxes) {
        const int m = threadIdx.x;
        int f = 2 | 4;
        if (m < axis_size) {
            const int64_t yb = pn[m * 3 + 1], xb = pn[pn[m * 3] * 3 + 2];
            const int64_t span = m == 0 ? n : pn[(m - 1) * 3 + 1];   // output elements per step of the axis before
            yblk[m] = yb;
            xblk[m] = xb;
            osz[m] = small ? (int)((uint32_t)span / (uint32_t)max((int)yb, 1)) : 0;
            if (m == last) f = (yb == 1 && xb == 1 ? 2 : 0) | (yb == 1 && xb > 1 && span > 1 ? 4 : 0);
            else f = (xb % 4 == 0 && yb % 4 == 0 ? 2 : 0) | 4;
            if (xb == 1 && span >= 2 * yb) f |= 1 | (m << 4);
        }
        flags[m] = f;
    }
    __syncthreads();
    const int4 fa = *reinterpret_cast<const int4*>(&flags[0]), fb = *reinterpret_cast<const int4*>(&flags[4]);
    const int fl[kTrMaxAxes] = {fa.x, fa.y, fa.z, fa.w, fb.x, fb.y, fb.z, fb.w};
    int all = 6, mj = -1;
#pragma unroll
    for (int m = 0; m < kTrMaxAxes; m++) {
        all &= fl[m];
        mj = max(mj, (fl[m] & 1) ? (fl[m] >> 4) : -1);
    }
    // length of the innermost output axis = output elements per step of the axis before it
    const int64_t inner = last > 0 ? yblk[last - 1] : n;
    const bool vec = aligned16 && (all & 2) && inner % 4 == 0 && n % 4 == 0;
    // the tiles: the source's innermost axis is not the output's (tensors of 2^31 elements and more stay with the
    // element-wise loop: the tiles count in 32 bits)
    if (small && mj >= 0 && mj != last && (all & 4)) {
        __shared__ float tile[kTrTileFloats];
        transpose_axes_tiled<BACKWARD>(out, in, yblk, xblk, osz, axis_size, mj, tile);
        return;
    }
    if (vec) {
        if (small) transpose_axes_body<int32_t, BACKWARD, true>(out, in, yblk, xblk, axis_size, n);
        else transpose_axes_body<int64_t, BACKWARD, true>(out, in, yblk, xblk, axis_size, n);
    } else {
        if (small) transpose_axes_body<int32_t, BACKWARD, false>(out, in, yblk, xblk, axis_size, n);
        else transpose_axes_body<int64_t, BACKWARD, false>(out, in, yblk, xblk, axis_size, n);
    }
}

int launch_transpose(float* y, const float* x, const int* pn, int64_t axis_size, int64_t n, bool backward,
                     hipStream_t stream) {
    if (n <= 0) return KAI_OK;
    if (axis_size < 1 || axis_size > kTrMaxAxes) return fail(KAI_ERR_INVALID_ARGUMENT, "transpose: 1 to 8 axes");
    const int al = aligned16(y) && aligned16(x);
    // a thread moves up to four elements: a quarter of the workgroups cover the tensor when it does (grid-stride)
    const dim3 grid = blocks_for(al ? (n + 3) / 4 : n);
    if (backward) transpose_axes_kernel<true><<<grid, kEwThreads, 0, stream>>>(y, x, pn, (int)axis_size, n, al);
    else transpose_axes_kernel<false><<<grid, kEwThreads, 0, stream>>>(y, x, pn, (int)axis_size, n, al);
    return check_launch("transpose_axes_kernel");
}

// ---- parameter update ------------------------------------------------------------------------------
//
// Elementwise streams over the parameter, gradient and optimizer-state tensors.  The arithmetic keeps
// the reference's rounding: its host build forbids contraction (-ffp-contract=off,
// source/engine/CMakeLists.txt:196), so products and sums are rounded separately here too
// (contraction is switched off below for the rest of this file; it must be this pragma around plain
// operators: HIP's __fmul_rn / __fadd_rn are inline functions of a header outside its reach and get
// fused after inlining) and the first three kernels are bit-identical to the host loops.
// MODE selects the function; VEC = four elements per thread with 128-bit accesses.
#pragma clang fp contract(off)

enum UpdateMode { kUpdAccumulate = 0, kUpdSubtract = 1, kUpdDecay = 2 };

struct UpdateParams {
    float* out;         // accumulate: y (in place); subtract: p (in place); decay: d
    const float* a;     // accumulate: x; subtract: g; decay: p
    const float* b;     // decay: g
    const float* h1;    // subtract: learning rate; decay: l1
    const float* h2;    // decay: l2
    int64_t n;
};

template <int MODE>
__device__ __forceinline__ float update_one(float out, float a, float b, float h1, float h2) {
    if (MODE == kUpdAccumulate) return out + a;
    if (MODE == kUpdSubtract) return out - a * h1;
    float delta = b;   // decay: a = p, b = g, h1 = l1, h2 = l2
    if (h2 > 0) delta += h2 * a;
    if (h1 > 0) delta += h1 * ((a > 0) ? 1.f : ((a < 0) ? -1.f : 0.f));
    return delta;
}

template <int MODE, bool VEC>
__global__ void __launch_bounds__(kEwThreads) update_kernel(UpdateParams p) {
    const float h1 = p.h1 ? *p.h1 : 0.f;
    const float h2 = p.h2 ? *p.h2 : 0.f;
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    const int64_t n = VEC ? p.n / 4 : p.n;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
        if (VEC) {
            f32x4 o = MODE == kUpdDecay ? f32x4{0.f, 0.f, 0.f, 0.f} : *reinterpret_cast<const f32x4*>(p.out + i * 4);
            const f32x4 a = *reinterpret_cast<const f32x4*>(p.a + i * 4);
            const f32x4 b = MODE == kUpdDecay ? *reinterpret_cast<const f32x4*>(p.b + i * 4) : a;
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = update_one<MODE>(o[j], a[j], b[j], h1, h2);
            *reinterpret_cast<f32x4*>(p.out + i * 4) = o;
        } else {
            const float o = MODE == kUpdDecay ? 0.f : p.out[i];
            p.out[i] = update_one<MODE>(o, p.a[i], MODE == kUpdDecay ? p.b[i] : 0.f, h1, h2);
        }
    }
}

template <int MODE>
static int launch_update(const UpdateParams& p, const char* name, hipStream_t stream) {
    if (p.n <= 0) return KAI_OK;
    const bool vec = p.n % 4 == 0 && aligned16(p.out) && aligned16(p.a) && (p.b == nullptr || aligned16(p.b));
    if (vec) update_kernel<MODE, true><<<blocks_for(p.n / 4), kEwThreads, 0, stream>>>(p);
    else update_kernel<MODE, false><<<blocks_for(p.n), kEwThreads, 0, stream>>>(p);
    return check_launch(name);
}

int launch_accumulate_grad(float* y, const float* x, int64_t n, hipStream_t stream) {
    UpdateParams p{y, x, nullptr, nullptr, nullptr, n};
    return launch_update<kUpdAccumulate>(p, "accumulate_grad", stream);
}

int launch_subtract_param_grad(float* pp, const float* g, int64_t n, const float* hlr, hipStream_t stream) {
    UpdateParams p{pp, g, nullptr, hlr, nullptr, n};
    return launch_update<kUpdSubtract>(p, "subtract_param_grad", stream);
}

int launch_apply_decay(float* d, const float* pp, const float* g, int64_t n, const float* hl1, const float* hl2,
                       hipStream_t stream) {
    UpdateParams p{d, pp, g, hl1, hl2, n};
    return launch_update<kUpdDecay>(p, "apply_decay", stream);
}

// One Adam step (vmath.cu:449-468): s and t are the moment tensors, nstep the per-element step count
// (a float tensor in the engine), all updated in place; a receives the update direction.
__global__ void __launch_bounds__(kEwThreads)
    adam_delta_kernel(float* __restrict__ a, const float* __restrict__ g, float* __restrict__ s, float* __restrict__ t,
                      float* __restrict__ nstep, int64_t n, const float* __restrict__ hro1,
                      const float* __restrict__ hro2, const float* __restrict__ heps) {
    const float ro1 = hro1 ? *hro1 : 0.f;
    const float ro2 = hro2 ? *hro2 : 0.f;
    const float eps = heps ? *heps : 0.f;
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
        const float delta = g[i];
        const float ns = nstep[i] + 1.f;
        const float si = ro1 * s[i] + (1.f - ro1) * delta;
        const float ti = ro2 * t[i] + (1.f - ro2) * delta * delta;
        const float sterm = si / (1.f - powf(ro1, ns));
        const float tterm = ti / (1.f - powf(ro2, ns));
        s[i] = si;
        t[i] = ti;
        a[i] = sterm / (sqrtf(tterm) + eps);
        nstep[i] = ns;
    }
}

// Four elements per thread.  The two powers are most of the arithmetic of a step; the four step counts of a thread
// are equal wherever a tensor has been updated as a whole, and then one pair of powers serves all four (the same
// function on the same arguments: the same bits).
__global__ void __launch_bounds__(kEwThreads)
    adam_delta_vec_kernel(float4* __restrict__ a, const float4* __restrict__ g, float4* __restrict__ s,
                          float4* __restrict__ t, float4* __restrict__ nstep, int64_t n4,
                          const float* __restrict__ hro1, const float* __restrict__ hro2,
                          const float* __restrict__ heps) {
    const float ro1 = hro1 ? *hro1 : 0.f;
    const float ro2 = hro2 ? *hro2 : 0.f;
    const float eps = heps ? *heps : 0.f;
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n4; i += stride) {
        const float4 gv = g[i], nv = nstep[i], sv = s[i], tv = t[i];
        const float gi[4] = {gv.x, gv.y, gv.z, gv.w};
        const float so[4] = {sv.x, sv.y, sv.z, sv.w};
        const float to[4] = {tv.x, tv.y, tv.z, tv.w};
        const float ns[4] = {nv.x + 1.f, nv.y + 1.f, nv.z + 1.f, nv.w + 1.f};
        float p1[4], p2[4];
        if (ns[0] == ns[1] && ns[0] == ns[2] && ns[0] == ns[3]) {
            p1[0] = p1[1] = p1[2] = p1[3] = powf(ro1, ns[0]);
            p2[0] = p2[1] = p2[2] = p2[3] = powf(ro2, ns[0]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                p1[j] = powf(ro1, ns[j]);
                p2[j] = powf(ro2, ns[j]);
            }
        }
        float si[4], ti[4], ai[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            si[j] = ro1 * so[j] + (1.f - ro1) * gi[j];
            ti[j] = ro2 * to[j] + (1.f - ro2) * gi[j] * gi[j];
            const float sterm = si[j] / (1.f - p1[j]);
            const float tterm = ti[j] / (1.f - p2[j]);
            ai[j] = sterm / (sqrtf(tterm) + eps);
        }
        s[i] = make_float4(si[0], si[1], si[2], si[3]);
        t[i] = make_float4(ti[0], ti[1], ti[2], ti[3]);
        a[i] = make_float4(ai[0], ai[1], ai[2], ai[3]);
        nstep[i] = make_float4(ns[0], ns[1], ns[2], ns[3]);
    }
}

int launch_eval_adam_delta(float* a, const float* g, float* s, float* t, float* nstep, int64_t n, const float* hro1,
                           const float* hro2, const float* heps, hipStream_t stream) {
    if (n <= 0) return KAI_OK;
    if (n % 4 == 0 && aligned16(a) && aligned16(g) && aligned16(s) && aligned16(t) && aligned16(nstep)) {
        adam_delta_vec_kernel<<<blocks_for(n / 4), kEwThreads, 0, stream>>>(
            reinterpret_cast<float4*>(a), reinterpret_cast<const float4*>(g), reinterpret_cast<float4*>(s),
            reinterpret_cast<float4*>(t), reinterpret_cast<float4*>(nstep), n / 4, hro1, hro2, heps);
        return check_launch("adam_delta_vec_kernel");
    }
    adam_delta_kernel<<<blocks_for(n), kEwThreads, 0, stream>>>(a, g, s, t, nstep, n, hro1, hro2, heps);
    return check_launch("adam_delta_kernel");
}

// ---- recurrent cells: what runs between the gate products of an RNN / LSTM / GRU step -------------------
//
// One thread per (row, unit); the gate pre-activations of a row lie nrec apart, so neighbouring threads
// read neighbouring floats of every gate.

__global__ void __launch_bounds__(kEwThreads) add_kernel(float* y, const float* a, const float* b, int64_t n) {
    // y may alias a or b (the engine adds in place)
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) y[i] = a[i] + b[i];
}

int launch_add(float* y, const float* a, const float* b, int64_t n, hipStream_t stream) {
    if (n <= 0) return KAI_OK;
    add_kernel<<<blocks_for(n), kEwThreads, 0, stream>>>(y, a, b, n);
    return check_launch("add_kernel");
}

__global__ void __launch_bounds__(kEwThreads)
    lstm_process_kernel(float* __restrict__ r, float* s, const float* s1, const float* __restrict__ a, int64_t n,
                        int64_t nrec) {
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
        const int64_t nd = i / nrec, nr = i - nd * nrec;
        const float* g = a + nd * 4 * nrec + nr;
        const float state = s1 ? s1[i] : 0.f;
        const float input_gate = act_sigmoid(g[0]);
        const float forget_gate = act_sigmoid(g[nrec]);
        const float input_block = act_tanh(g[2 * nrec]);
        const float output_gate = act_sigmoid(g[3 * nrec]);
        const float new_state = state * forget_gate + input_block * input_gate;
        s[i] = new_state;
        r[i] = act_tanh(new_state) * output_gate;
    }
}

int launch_lstm_process(float* r, float* s, const float* s1, const float* a, int64_t ndat, int64_t nrec,
                        hipStream_t stream) {
    const int64_t n = ndat * nrec;
    if (n <= 0) return KAI_OK;
    lstm_process_kernel<<<blocks_for(n), kEwThreads, 0, stream>>>(r, s, s1, a, n, nrec);
    return check_launch("lstm_process_kernel");
}

// VMath::lstm_process_backward after the reference's device kernel (vmath.cu:4899-4937): one thread per
// (row, unit) recomputes the four gates from this step's gate sums, writes the four gate-sum gradients
// nrec apart in ga[ndat, 4*nrec] and replaces gs (gradient of this step's state) by the gradient of the
// state the step started from.  gr is only read.
__global__ void __launch_bounds__(kEwThreads)
    lstm_process_backward_kernel(const float* __restrict__ gr, float* gs, float* __restrict__ ga, const float* s_prev,
                                 const float* __restrict__ a, int64_t n, int64_t nrec) {
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
        const int64_t nd = i / nrec, nr = i - nd * nrec;
        const int64_t apos = nd * 4 * nrec + nr;
        const float old_state = s_prev ? s_prev[i] : 0.f;
        const float input_gate = act_sigmoid(a[apos]);
        const float forget_gate = act_sigmoid(a[apos + nrec]);
        const float input_block = act_tanh(a[apos + 2 * nrec]);
        const float output_gate = act_sigmoid(a[apos + 3 * nrec]);
        const float new_state = old_state * forget_gate + input_block * input_gate;
        const float g_new_recur = gr[i];
        const float th = act_tanh(new_state);
        const float g_output_gate = th * g_new_recur;
        const float g_tanh_state = output_gate * g_new_recur;
        const float g_new_state = (1.0f - th * th) * g_tanh_state + gs[i];
        const float g_forget_gate = old_state * g_new_state;
        const float g_input_block = input_gate * g_new_state;
        const float g_input_gate = input_block * g_new_state;
        ga[apos] = input_gate * (1.0f - input_gate) * g_input_gate;
        ga[apos + nrec] = forget_gate * (1.0f - forget_gate) * g_forget_gate;
        ga[apos + 2 * nrec] = (1.0f - input_block * input_block) * g_input_block;
        ga[apos + 3 * nrec] = output_gate * (1.0f - output_gate) * g_output_gate;
        gs[i] = forget_gate * g_new_state;
    }
}

int launch_lstm_process_backward(const float* gr, float* gs, float* ga, const float* s_prev, const float* a,
                                 int64_t ndat, int64_t nrec, hipStream_t stream) {
    const int64_t n = ndat * nrec;
    if (n <= 0) return KAI_OK;
    lstm_process_backward_kernel<<<blocks_for(n), kEwThreads, 0, stream>>>(gr, gs, ga, s_prev, a, n, nrec);
    return check_launch("lstm_process_backward_kernel");
}

struct GruGates {
    float Rt, Zt, Nt, Ht_1, par_n;
};

__device__ __forceinline__ GruGates gru_gates(const float* h_prev, const float* ai, const float* ar, int64_t i,
                                              int64_t nrec, int64_t& gpos) {
    const int64_t nd = i / nrec, ny = i - nd * nrec;
    gpos = nd * 3 * nrec + ny;
    GruGates g;
    g.Rt = act_sigmoid(ai[gpos] + ar[gpos]);
    g.Zt = act_sigmoid(ai[gpos + nrec] + ar[gpos + nrec]);
    g.par_n = ar[gpos + 2 * nrec];
    g.Nt = act_tanh(ai[gpos + 2 * nrec] + g.Rt * g.par_n);
    g.Ht_1 = h_prev ? h_prev[i] : 0.f;
    return g;
}

__global__ void __launch_bounds__(kEwThreads)
    gru_process_kernel(float* r, const float* h_prev, const float* __restrict__ ai, const float* __restrict__ ar,
                       int64_t n, int64_t nrec) {
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
        int64_t gpos;
        const GruGates g = gru_gates(h_prev, ai, ar, i, nrec, gpos);
        r[i] = (1.0f - g.Zt) * g.Nt + g.Zt * g.Ht_1;
    }
}

__global__ void __launch_bounds__(kEwThreads)
    gru_process_backward_kernel(float* gr, float* __restrict__ gai, float* __restrict__ gar, const float* h_prev,
                                const float* __restrict__ ai, const float* __restrict__ ar, int64_t n, int64_t nrec) {
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
        int64_t gpos;
        const GruGates g = gru_gates(h_prev, ai, ar, i, nrec, gpos);
        const float gHt = gr[i];
        const float gNt = (1 - g.Zt) * gHt;
        const float gZt = (g.Ht_1 - g.Nt) * gHt;
        const float gNt_seed = (1 + g.Nt) * (1 - g.Nt) * gNt;
        const float gRt = g.par_n * gNt_seed;
        const float dr = g.Rt * (1 - g.Rt) * gRt, dz = g.Zt * (1 - g.Zt) * gZt;
        gai[gpos] = dr;
        gar[gpos] = dr;
        gai[gpos + nrec] = dz;
        gar[gpos + nrec] = dz;
        gai[gpos + 2 * nrec] = gNt_seed;
        gar[gpos + 2 * nrec] = g.Rt * gNt_seed;
        gr[i] = g.Zt * gHt;
    }
}

int launch_gru_process(float* r, const float* ai, const float* ar, int64_t nt, int64_t ndat, int64_t nrec,
                       hipStream_t stream) {
    const int64_t n = ndat * nrec;
    if (n <= 0) return KAI_OK;
    // the previous time step lies one [ndat, nrec] block before r (vmath.cu:4961)
    gru_process_kernel<<<blocks_for(n), kEwThreads, 0, stream>>>(r, nt > 0 ? r - n : nullptr, ai, ar, n, nrec);
    return check_launch("gru_process_kernel");
}

int launch_gru_process_from(float* r, const float* h_prev, const float* ai, const float* ar, int64_t ndat, int64_t nrec,
                            hipStream_t stream) {
    const int64_t n = ndat * nrec;
    if (n <= 0) return KAI_OK;
    gru_process_kernel<<<blocks_for(n), kEwThreads, 0, stream>>>(r, h_prev, ai, ar, n, nrec);
    return check_launch("gru_process_kernel");
}

int launch_gru_process_backward(float* gr, float* gai, float* gar, const float* r, const float* ai, const float* ar,
                                int64_t nt, int64_t ndat, int64_t nrec, hipStream_t stream) {
    const int64_t n = ndat * nrec;
    if (n <= 0) return KAI_OK;
    gru_process_backward_kernel<<<blocks_for(n), kEwThreads, 0, stream>>>(gr, gai, gar, nt > 0 ? r - n : nullptr, ai, ar, n,
                                                                          nrec);
    return check_launch("gru_process_backward_kernel");
}

// ---- cosine similarity: the two passes around the row-pair product ---------------------------------------
//
// y[i,j] = <a_i, b_j> / (|a_i| |b_j| + 1e-20).  The products come from the GEMM; row_norm_kernel writes
// |row| for the rows of both operands (a wave per row), cosine_scale_kernel divides.

// VEC: ncol a multiple of 4 and both operands on 16-byte lines: 128-bit loads
template <bool VEC>
__global__ void __launch_bounds__(256) row_norm_kernel(float* __restrict__ out, const float* __restrict__ x1,
                                                       int64_t nrow1, const float* __restrict__ x2, int64_t nrow2,
                                                       int64_t ncol) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= nrow1 + nrow2) return;
    const float* xr = row < nrow1 ? x1 + row * ncol : x2 + (row - nrow1) * ncol;
    float s = 0.f;
    if (VEC) {
        const f32x4* __restrict__ x4 = reinterpret_cast<const f32x4*>(xr);
        for (int64_t c = lane; c < ncol / 4; c += 64) {
            const f32x4 v = x4[c];
            s += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        }
    } else {
        for (int64_t c = lane; c < ncol; c += 64) s += xr[c] * xr[c];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (lane == 0) out[row] = sqrtf(s);
}

__global__ void __launch_bounds__(kEwThreads) cosine_scale_kernel(float* __restrict__ y, const float* __restrict__ norms,
                                                                  int64_t nrow1, int64_t nrow2) {
    const int64_t n = nrow1 * nrow2;
    const int64_t stride = (int64_t)gridDim.x * kEwThreads;
    for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
        const int64_t r1 = i / nrow2, r2 = i - r1 * nrow2;
        y[i] = y[i] / (norms[r1] * norms[nrow1 + r2] + 1e-20f);
    }
}

int launch_cosine_norms_and_scale(float* y, float* norms, const float* x1, const float* x2, int64_t nrow1,
                                  int64_t nrow2, int64_t ncol, hipStream_t stream) {
    const int64_t rows = nrow1 + nrow2;
    if (rows <= 0 || nrow1 * nrow2 <= 0) return KAI_OK;
    if ((rows + 3) / 4 > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "cosinesim: too many rows");
    if (ncol % 4 == 0 && aligned16(x1) && aligned16(x2))
        row_norm_kernel<true><<<dim3((unsigned)((rows + 3) / 4)), 256, 0, stream>>>(norms, x1, nrow1, x2, nrow2, ncol);
    else
        row_norm_kernel<false><<<dim3((unsigned)((rows + 3) / 4)), 256, 0, stream>>>(norms, x1, nrow1, x2, nrow2, ncol);
    KAI_TRY(check_launch("row_norm_kernel"));
    cosine_scale_kernel<<<blocks_for(nrow1 * nrow2), kEwThreads, 0, stream>>>(y, norms, nrow1, nrow2);
    return check_launch("cosine_scale_kernel");
}

// Up to four rows on one side against many on the other (a query against a table): one pass over the table.  The
// few rows wait in LDS with their norms; a wave takes four rows of the table at a time, forms their norms and their
// products with the few rows from one read, and lane 0 writes the quotients.  The three launches above read the
// table twice ([1, 100000, 256]: 55 us for 100 MB).
constexpr int kCosFewFloats = 8192;   // the few rows in LDS: nrow1 * ncol floats at most
constexpr int kCosFewUnroll = 4;
template <int R>
__global__ void __launch_bounds__(256) cosine_few_rows_kernel(float* __restrict__ y, const float* __restrict__ x1,
                                                              const float* __restrict__ x2, int64_t nrow2, int ncol) {
    __shared__ __attribute__((aligned(16))) float a[kCosFewFloats];
    __shared__ float na[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nc4 = ncol / 4;
    f32x4* a4 = reinterpret_cast<f32x4*>(a);
    for (int i = tid; i < R * nc4; i += 256) a4[i] = reinterpret_cast<const f32x4*>(x1)[i];
    __syncthreads();
    if (wave < R) {
        float s = 0.f;
        for (int c = lane; c < nc4; c += 64) {
            const f32x4 v = a4[wave * nc4 + c];
            s += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        }
        s = wave_add(s);
        if (lane == 0) na[wave] = sqrtf(s);
    }
    __syncthreads();
    const f32x4* __restrict__ b4 = reinterpret_cast<const f32x4*>(x2);
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    for (int64_t j0 = ((int64_t)blockIdx.x * 4 + wave) * kCosFewUnroll; j0 < nrow2; j0 += nwaves * kCosFewUnroll) {
        float nb[kCosFewUnroll], dot[kCosFewUnroll][R];
#pragma unroll
        for (int u = 0; u < kCosFewUnroll; u++) {
            nb[u] = 0.f;
#pragma unroll
            for (int r = 0; r < R; r++) dot[u][r] = 0.f;
        }
        for (int c = lane; c < nc4; c += 64) {
            f32x4 v[kCosFewUnroll];
#pragma unroll
            for (int u = 0; u < kCosFewUnroll; u++) v[u] = b4[min(j0 + u, nrow2 - 1) * nc4 + c];   // past the end: the last row again
#pragma unroll
            for (int r = 0; r < R; r++) {
                const f32x4 av = a4[r * nc4 + c];
#pragma unroll
                for (int u = 0; u < kCosFewUnroll; u++)
                    dot[u][r] += v[u][0] * av[0] + v[u][1] * av[1] + v[u][2] * av[2] + v[u][3] * av[3];
            }
#pragma unroll
            for (int u = 0; u < kCosFewUnroll; u++)
                nb[u] += v[u][0] * v[u][0] + v[u][1] * v[u][1] + v[u][2] * v[u][2] + v[u][3] * v[u][3];
        }
#pragma unroll
        for (int u = 0; u < kCosFewUnroll; u++) {
            nb[u] = wave_add(nb[u]);
#pragma unroll
            for (int r = 0; r < R; r++) dot[u][r] = wave_add(dot[u][r]);
        }
        if (lane == 0) {
#pragma unroll
            for (int u = 0; u < kCosFewUnroll; u++)
                if (j0 + u < nrow2) {
                    const float nbu = sqrtf(nb[u]);
#pragma unroll
                    for (int r = 0; r < R; r++) y[(int64_t)r * nrow2 + j0 + u] = dot[u][r] / (na[r] * nbu + 1e-20f);
                }
        }
    }
}

bool cosine_few_rows_applies(const float* x1, const float* x2, int64_t nrow1, int64_t nrow2, int64_t ncol) {
    return nrow1 >= 1 && nrow1 <= 4 && nrow2 >= 512 && ncol >= 4 && ncol % 4 == 0 && nrow1 * ncol <= kCosFewFloats &&
           aligned16(x1) && aligned16(x2);
}

int launch_cosine_few_rows(float* y, const float* x1, const float* x2, int64_t nrow1, int64_t nrow2, int64_t ncol,
                           hipStream_t stream) {
    const int64_t want = (nrow2 + 4 * kCosFewUnroll - 1) / (4 * kCosFewUnroll);
    const int64_t cap = 4 * (int64_t)compute_units();
    const dim3 grid((unsigned)(want < cap ? want : cap));
    switch (nrow1) {
    case 1: cosine_few_rows_kernel<1><<<grid, 256, 0, stream>>>(y, x1, x2, nrow2, (int)ncol); break;
    case 2: cosine_few_rows_kernel<2><<<grid, 256, 0, stream>>>(y, x1, x2, nrow2, (int)ncol); break;
    case 3: cosine_few_rows_kernel<3><<<grid, 256, 0, stream>>>(y, x1, x2, nrow2, (int)ncol); break;
    default: cosine_few_rows_kernel<4><<<grid, 256, 0, stream>>>(y, x1, x2, nrow2, (int)ncol); break;
    }
    return check_launch("cosine_few_rows_kernel");
}

// ---- split-K final pass ---------------------------------------------------------------------
//
// Sums the partial products in split order (fixed, so the result does not depend on scheduling)
// and applies the GEMM epilogue.  VEC: four consecutive columns per thread with 128-bit accesses.

template <bool VEC, int NMAX>
__global__ void __launch_bounds__(kEwThreads) splitk_reduce_kernel(SplitReduceParams p) {
    constexpr int W = VEC ? 4 : 1;
    const int64_t total = p.M * p.N;
    const int64_t e = ((int64_t)blockIdx.x * kEwThreads + threadIdx.x) * W;
    if (e >= total) return;
    const float alpha = p.has_alpha ? (p.alpha ? *p.alpha : 0.0f) : 1.0f;
    const float leaky = p.leaky ? *p.leaky : 0.0f;
    const int64_t m = e / p.N, n = e - m * p.N;
    const int64_t idx = m * p.c_rs + n * p.c_cs;
    // all NMAX >= nsplit partial sums are requested before the first one is used (parts beyond nsplit repeat
    // the last one and are masked out of the sum), so the loads overlap instead of queueing behind the adds
    float v[W];
    if (VEC) {
        f32x4 part[NMAX];
#pragma unroll
        for (int k = 0; k < NMAX; k++)
            part[k] = *reinterpret_cast<const f32x4*>(p.part + (k < p.nsplit ? k : p.nsplit - 1) * total + e);
        f32x4 s = part[0];
#pragma unroll
        for (int k = 1; k < NMAX; k++) {
            const int keep = k < p.nsplit ? -1 : 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float x = part[k][j];
                s[j] += __int_as_float(__float_as_int(x) & keep);
            }
        }
        for (int j = 0; j < W; j++) v[j] = s[j];
    } else {
        float part[NMAX];
#pragma unroll
        for (int k = 0; k < NMAX; k++) part[k] = p.part[(k < p.nsplit ? k : p.nsplit - 1) * total + e];
        float s = part[0];
#pragma unroll
        for (int k = 1; k < NMAX; k++) s += __int_as_float(__float_as_int(part[k]) & (k < p.nsplit ? -1 : 0));
        v[0] = s;
    }
    for (int j = 0; j < W; j++) {
        float o = p.has_alpha ? v[j] * alpha : v[j];
        if (p.accflag) o += p.C[idx + j * p.c_cs];
        if (p.bias) o += p.bias[n + j];
        v[j] = o;
    }
    if (VEC) {
        f32x4 o = {v[0], v[1], v[2], v[3]};
        if (p.C2) *reinterpret_cast<f32x4*>(p.C2 + idx) = o;
        for (int j = 0; j < W; j++) o[j] = apply_act(o[j], p.act, leaky);
        *reinterpret_cast<f32x4*>(p.C + idx) = o;
    } else {
        if (p.C2) p.C2[idx] = v[0];
        p.C[idx] = apply_act(v[0], p.act, leaky);
    }
}

// one thread per output element (or four of them): the grid covers the output, it is not capped like the
// grids of the kernels above, which loop
template <int NMAX>
static int launch_splitk_reduce_n(const SplitReduceParams& p, bool vec, int64_t total, hipStream_t stream) {
    const int64_t items = vec ? total / 4 : total;
    const int64_t blocks = (items + kEwThreads - 1) / kEwThreads;
    if (blocks > 0x7fffffffll) return fail(KAI_ERR_INVALID_ARGUMENT, "split-K: output too large for one grid");
    if (vec) splitk_reduce_kernel<true, NMAX><<<(unsigned)blocks, kEwThreads, 0, stream>>>(p);
    else splitk_reduce_kernel<false, NMAX><<<(unsigned)blocks, kEwThreads, 0, stream>>>(p);
    return check_launch("splitk_reduce_kernel");
}

int launch_splitk_reduce(const SplitReduceParams& p, hipStream_t stream) {
    const int64_t total = p.M * p.N;
    if (total <= 0) return KAI_OK;
    if (p.nsplit < 1 || p.nsplit > 16) return fail(KAI_ERR_INVALID_ARGUMENT, "split-K: 1 to 16 parts");
    const bool vec = p.c_cs == 1 && p.N % 4 == 0 && p.c_rs % 4 == 0 && aligned16(p.part) && aligned16(p.C) &&
                     (!p.C2 || aligned16(p.C2)) && (!p.bias || aligned16(p.bias));
    if (p.nsplit <= 4) return launch_splitk_reduce_n<4>(p, vec, total, stream);
    if (p.nsplit <= 8) return launch_splitk_reduce_n<8>(p, vec, total, stream);
    return launch_splitk_reduce_n<16>(p, vec, total, stream);
}

}  // namespace kai
