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

}  // namespace kai
