// Skinny products against a matrix whose rows run along the OUTPUT index:
//
//   c[m,n] (=|+=) act( alpha * sum_k a[m,k] * b[k,n] + bias[n] ),   m < M <= 16, b stored [K, N]
//
// the engine's VMath::matmul_backward_x at small batches (gx = gy . w with w[yvec, xvec], vmath.cu:3007-3047 of
// the reference) and a forward product against a transposed weight layout.  Every element of b is used M
// times and read once, so the product is bound by the stream of b from HBM; its rows are contiguous along n,
// which makes this the axpy form: c[m, :] += a[m,k] * b[k, :].
//
// A workgroup owns a slice of 256 columns and one part of K; wave w takes a run of consecutive rows of that
// part.  A lane owns four consecutive columns: a row of b arrives as one fully coalesced 1 KiB load per wave,
// non-temporal, four rows per round and the next round's loads issued before this round's arithmetic.  The
// a values of a part sit in LDS (M x part floats, copied once per workgroup) and are read as broadcasts, four
// consecutive k at a time.  The waves' partial sums meet in LDS in a fixed tree (4+4, 2+2, 1+1), wave 0 writes
// the part; the parts of K are summed, in part order, by the reduce pass that also runs the epilogue.
#include "elementwise.h"
#include "gemm_host.h"

namespace kai {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));   // 128-bit load at 4-byte alignment

constexpr int kSrWaves = 8;
constexpr int kSrThreads = 64 * kSrWaves;
constexpr int kSrCols = 256;          // columns per workgroup: four per lane
constexpr int kSrRound = 4;           // rows of b per wave and round
constexpr int kSrMaxPart = 512;       // steps of K whose a values sit in LDS at a time (16 x 512 floats)

struct SkinnyRowsParams {
    const float* A;      // [M, K], row stride lda
    const float* B;      // [K, N], row stride ldb
    float* part;         // [splits][M][N]
    int64_t lda, ldb;
    int64_t N;
    int M, K;
    int k_part;          // reduction steps per part: a multiple of kSrWaves * kSrRound
    int slices;          // column slices
};

template <int MT>
__global__ void __launch_bounds__(kSrThreads)
skinny_rows_kernel(const float* __restrict__ A, const float* __restrict__ B, const int64_t lda, const int64_t ldb,
                   const int64_t N, const int M, const int K, const int k_part, const int slices,
                   float* __restrict__ part) {
    // scalars, what the loads need first: this file is compiled with kernel-argument preload, so the first 14
    // dwords are in SGPRs when a wave starts and the stream begins without a fetch of the argument buffer
    const SkinnyRowsParams p{A, B, part, lda, ldb, N, M, K, k_part, slices};
    __shared__ __attribute__((aligned(16))) float a_lds[MT * kSrMaxPart];
    __shared__ __attribute__((aligned(16))) float red[(kSrWaves / 2) * MT * kSrCols];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slice = blockIdx.x % p.slices, split = blockIdx.x / p.slices;
    const int k0 = split * p.k_part;
    const int klen = min(p.k_part, p.K - k0);             // >= 1: the host launches no empty part
    const int64_t n = (int64_t)slice * kSrCols + 4 * lane;
    const bool col_ok = n < p.N;                           // N % 4 == 0: four columns are inside or outside together
    const float* __restrict__ bcol = p.B + (col_ok ? n : 0);

    auto load_rows = [&](f32x4(&dst)[kSrRound], int kk) {
#pragma unroll
        for (int j = 0; j < kSrRound; j++) {
            const int k = min(kk + j, klen - 1);           // clamped: what lies past the part is multiplied by zeros
            dst[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4u*>(bcol + (int64_t)(k0 + k) * p.ldb));
        }
    };

    f32x4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};

    // The part is walked in chunks of at most kSrMaxPart steps (what fits LDS); within a chunk wave w takes a
    // run of consecutive rows, whole rounds of kSrRound.
    for (int c0 = 0; c0 < p.k_part; c0 += kSrMaxPart) {
        const int chunk = min(kSrMaxPart, p.k_part - c0);  // a multiple of kSrWaves * kSrRound
        const int per_wave = chunk / kSrWaves;
        const int kw0 = c0 + wave * per_wave;
        f32x4 cur[kSrRound], nxt[kSrRound];
        load_rows(cur, kw0);                               // on their way while the a values are copied
        __syncthreads();                                   // the previous chunk's a values are no longer read
        // a_lds[m][k - c0], zeros past M and past the part (so clamped rows add nothing)
        for (int i = tid; i < MT * chunk; i += kSrThreads) {
            const int m = i / chunk, k = i - m * chunk;
            a_lds[m * kSrMaxPart + k] = (m < p.M && c0 + k < klen) ? p.A[(int64_t)m * p.lda + k0 + c0 + k] : 0.f;
        }
        __syncthreads();
        for (int kk = kw0; kk < kw0 + per_wave; kk += kSrRound) {
            load_rows(nxt, kk + kSrRound);                 // past the run: clamped, never used
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const f32x4 av = *reinterpret_cast<const f32x4*>(a_lds + m * kSrMaxPart + (kk - c0));   // broadcast
#pragma unroll
                for (int j = 0; j < kSrRound; j++) acc[m] += av[j] * cur[j];
            }
#pragma unroll
            for (int j = 0; j < kSrRound; j++) cur[j] = nxt[j];
        }
    }

    // fixed tree over the waves: (0+4, 1+5, 2+6, 3+7), then (0+2, 1+3), then (0+1)
#pragma unroll
    for (int step = kSrWaves / 2; step >= 1; step /= 2) {
        if (wave >= step && wave < 2 * step) {
#pragma unroll
            for (int m = 0; m < MT; m++)
                *reinterpret_cast<f32x4*>(red + ((wave - step) * MT + m) * kSrCols + 4 * lane) = acc[m];
        }
        __syncthreads();
        if (wave < step) {
#pragma unroll
            for (int m = 0; m < MT; m++) acc[m] += *reinterpret_cast<const f32x4*>(red + (wave * MT + m) * kSrCols + 4 * lane);
        }
        __syncthreads();
    }
    if (wave == 0 && col_ok) {
        float* out = p.part + (int64_t)split * p.M * p.N + n;
#pragma unroll
        for (int m = 0; m < MT; m++)
            if (m < p.M) *reinterpret_cast<f32x4*>(out + (int64_t)m * p.N) = acc[m];
    }
}

}  // namespace

// a K-contiguous, b contiguous along its output index with whole groups of four columns, at most 16 rows, a
// contiguous output row, and enough of b for the stream to matter
// Which products: up to 8 rows, and 9..16 rows (where the vector FMAs of this kernel begin to show) only in the
// window in which a sweep of 1..65 rows over 5 reduction lengths x 7 widths, the matrix streamed from HBM, found it
// faster than the tiled kernels at 17 rows: widths of 3072..5120 with up to 2048 steps, about 4096 columns with up
// to 8192 steps, and short reductions up to 4096 columns (us at 9 rows against the tiles at 17: 2048 x 4096 13.6 /
// 14.5, 8192 x 4096 31.4 / 33.1, 1024 x 4096 8.7 / 12.4; outside the window 4096 x 1024 18.7 / 13.7, 8192 x 1024 28.5 /
// 17.1, 11008 x 2048 38.4 / 27.1, 4096 x 8192 43.9 / 30.0, 11008 x 11008 105.5 / 94.2).  Reductions of up to 1024 steps
// against more than 4096 columns go to the tiles at every row count (1024 x 5120: 14.0 .. 16.2 against 10.4).
bool skinny_rows_applies(const GemmDesc& d) {
    if (!(d.nbatch == 1 && d.M >= 1 && d.M <= 16 && d.a_ks == 1 && d.b_rs == 1 && d.b_ks >= d.N && d.c_cs == 1 &&
          d.N % 4 == 0 && d.N >= 1024 && d.K >= 256 && d.K * d.N >= (1ll << 21) && d.rowsum == nullptr && d.k_part == 0))
        return false;
    if (d.K <= 1024 && d.N > 4096) return false;
    if (d.N < 2048 && d.K > 4096) return false;   // 4..7 column slices x 16 parts leave compute units idle: 8192 x 1024 18.7 against 16.6, 11008 x 1024 24.2 / 20.2
    if (d.M <= 8) return true;
    return d.N <= 5120 && ((d.K <= 1024 && d.N <= 4096) || (d.N >= 3072 && d.K <= 2048) || (d.N >= 3584 && d.N <= 4608 && d.K <= 8192));
}

int launch_skinny_rows(const GemmDesc& d, hipStream_t stream) {
    const int64_t slices = (d.N + kSrCols - 1) / kSrCols;
    // parts of K: about one workgroup per compute unit, at most 16 parts (the reduce pass), each a multiple
    // of a round of all waves
    constexpr int64_t unit = kSrWaves * kSrRound;
    int64_t splits = compute_units() / slices;
    if (splits < 1) splits = 1;
    if (splits > 16) splits = 16;
    const int64_t k_first = ((d.K + splits - 1) / splits + unit - 1) / unit * unit;
    splits = (d.K + k_first - 1) / k_first;
    // a caller's fixed buffer: fewer, longer parts until their sums fit it
    int64_t k_len = k_first;
    while (d.scratch && splits > 1 && splits * d.M * d.N * (int64_t)sizeof(float) > d.scratch_bytes) {
        k_len += unit;
        splits = (d.K + k_len - 1) / k_len;
    }
    const int64_t k_part = k_len;
    float* part = d.scratch;
    const int64_t part_bytes = splits * d.M * d.N * (int64_t)sizeof(float);
    if (part == nullptr) KAI_TRY(workspace(part_bytes, &part));
    else if (part_bytes > d.scratch_bytes)
        return fail(KAI_ERR_INVALID_ARGUMENT, "skinny rows: the partial sums need " + std::to_string(part_bytes) +
                    " bytes; the caller's scratch holds " + std::to_string(d.scratch_bytes));
    SkinnyRowsParams p{};
    p.A = d.A; p.B = d.B; p.part = part;
    p.lda = d.a_rs; p.ldb = d.b_ks; p.N = d.N; p.M = (int)d.M; p.K = (int)d.K;
    p.k_part = (int)k_part; p.slices = (int)slices;
    const dim3 grid((unsigned)(slices * splits)), block(kSrThreads);
    if (d.M <= 4) skinny_rows_kernel<4><<<grid, block, 0, stream>>>(p.A, p.B, p.lda, p.ldb, p.N, p.M, p.K, p.k_part, p.slices, p.part);
    else if (d.M <= 8) skinny_rows_kernel<8><<<grid, block, 0, stream>>>(p.A, p.B, p.lda, p.ldb, p.N, p.M, p.K, p.k_part, p.slices, p.part);
    else skinny_rows_kernel<16><<<grid, block, 0, stream>>>(p.A, p.B, p.lda, p.ldb, p.N, p.M, p.K, p.k_part, p.slices, p.part);
    KAI_TRY(check_launch("skinny_rows_kernel"));
    SplitReduceParams r{};
    r.part = part; r.C = d.C; r.C2 = d.C2; r.bias = d.bias; r.alpha = d.alpha; r.leaky = d.leaky;
    r.M = d.M; r.N = d.N; r.c_rs = d.c_rs; r.c_cs = d.c_cs;
    r.nsplit = (int)splits; r.act = d.act; r.accflag = d.acc; r.has_alpha = d.has_alpha;
    return launch_splitk_reduce(r, stream);
}

}  // namespace kai
