// Skinny (at most 16 rows) products: parameters and launcher, see gemv_skinny.hip.
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

int launch_skinny_nt(const SkinnyParams& p, hipStream_t stream);

// skinny_stream.hip: aligned operands, K split over workgroups (uses the library's scratch memory)
bool skinny_stream_applies(const SkinnyParams& p);
int launch_skinny_stream(const SkinnyParams& p, hipStream_t stream);

}  // namespace kai
