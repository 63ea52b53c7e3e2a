// Skinny products (at most 16 rows; 17..64 on the streaming kernel where skinny_stream32_applies): parameters and
// launcher, see gemv_skinny.hip.
#pragma once

#include "kai_common.h"

namespace kai {

constexpr int kSkinnyMaxRows = 16;

struct SkinnyParams {
    const float* W;      // [N, K], row stride ldw
    const float* X;      // [M, K], row stride ldx
    float* Y;            // [M, N], row stride ldy
    float* Y2;           // optional: value before the activation
    const float* bias;   // optional [N]
    const float* leaky;  // optional device scalar
    int64_t ldw, ldx, ldy;
    int64_t N;
    int M, K;
    int act, accflag;
};

// The arguments only an epilogue reads.  Kernels that stream from HBM take what their first loads need as
// leading scalar arguments (W, X, ldw, ldx, N, M, K, Y: 14 dwords), which kernel-argument preload puts into
// SGPRs before a wave starts, and the rest as this struct.
struct SkinnyTail {
    float* Y2;
    const float* bias;
    const float* leaky;
    int64_t ldy;
    int act, accflag;
};

inline SkinnyTail skinny_tail(const SkinnyParams& p) { return SkinnyTail{p.Y2, p.bias, p.leaky, p.ldy, p.act, p.accflag}; }

__device__ __forceinline__ SkinnyParams skinny_params(const float* W, const float* X, int64_t ldw, int64_t ldx, int64_t N,
                                                      int M, int K, float* Y, const SkinnyTail& t) {
    SkinnyParams p;
    p.W = W; p.X = X; p.Y = Y; p.Y2 = t.Y2; p.bias = t.bias; p.leaky = t.leaky;
    p.ldw = ldw; p.ldx = ldx; p.ldy = t.ldy; p.N = N; p.M = M; p.K = K; p.act = t.act; p.accflag = t.accflag;
    return p;
}

int launch_skinny_nt(const SkinnyParams& p, hipStream_t stream);

// skinny_stream.hip: aligned operands, K split over workgroups (uses the library's scratch memory)
bool skinny_stream_applies(const SkinnyParams& p);
bool skinny_stream32_applies(const SkinnyParams& p);   // 17..32 rows, and 33..64 where workgroups of 32 / 48 rows of W apply
bool skinny_stream8_applies(const SkinnyParams& p);    // workgroups of 8 rows of W
int launch_skinny_stream8(const SkinnyParams& p, hipStream_t stream);
int launch_skinny_stream(const SkinnyParams& p, hipStream_t stream);
int skinny_stream_wide_rows(const SkinnyParams& p);    // 32 or 48 rows of W per workgroup, 0 = workgroups of 16 rows
void set_skinny_stream_rows_override(int rows);        // audits: 16, 32 or 48 rows of W per workgroup, 0 = the rule

}  // namespace kai
