// The value gradient of the attention block as a launch of its own: VMath::mix_values_backward_value
// (vmath.cu:7081-7129 of the reference).  The device code and its description are in attention_value_grad.h.
#include "attention_value_grad.h"
#include "elementwise.h"

namespace kai {

namespace {

using namespace vgrad;

template <int DB, int HV>
__global__ void __launch_bounds__(kVgThreads) attention_value_grad_kernel(const ValueGradParams p) {
    __shared__ __attribute__((aligned(16))) float lds[value_grad_lds_floats<DB, HV>()];
    attention_value_grad_body<DB, HV>(p, blockIdx.x, gridDim.x, lds);
}

template <int DB, int HV>
void launch_vg(const ValueGradParams& p, dim3 grid, hipStream_t stream) {
    attention_value_grad_kernel<DB, HV><<<grid, dim3(kVgThreads), 0, stream>>>(p);
}

// the same with the roles of P's middle indices exchanged (attention_value_grad.h, TR): four heads per workgroup
template <int DB>
__global__ void __launch_bounds__(kVgThreads) attention_heads_mix_kernel(const ValueGradParams p) {
    __shared__ __attribute__((aligned(16))) float lds[value_grad_lds_floats<DB, 4>()];
    attention_value_grad_body<DB, 4, true>(p, blockIdx.x, gridDim.x, lds);
}

}  // namespace

// 0 = the kernel does not take the geometry, else the heads per workgroup (1 or 4)
int attention_value_grad_heads(const float* gv, const float* gy, const float* pp, int64_t ntimes, int64_t nvec,
                               int64_t nhead, int64_t npiece) {
    if (npiece % 16 != 0 || npiece < 16 || npiece > 128 || nhead < 1 || ntimes < 32 || nvec % 4 != 0 ||
        nhead * npiece > nvec || !aligned16(gv) || !aligned16(pp) || (reinterpret_cast<uintptr_t>(gy) & 3u) != 0 ||
        (ntimes + 1024) * ntimes * nhead * 4 >= (1ll << 31) || (ntimes + 1024) * nhead * npiece * 4 >= (1ll << 31))
        return 0;
    if (nhead == 1 && ntimes % 4 == 0) return 1;
    if (nhead % 4 == 0 && npiece <= 64) return 4;
    return 0;
}

vgrad::ValueGradParams value_grad_params(float* gv, const float* gy, const float* pp, int64_t ntimes, int64_t nvec,
                                         int64_t nhead, int64_t npiece) {
    vgrad::ValueGradParams p{};
    p.P = pp; p.gY = gy; p.gV = gv;
    p.p_batch_stride = ntimes * ntimes * nhead;
    p.gy_rs = nhead * npiece; p.gv_rs = nvec;
    p.ntimes = (int)ntimes; p.nhead = (int)nhead; p.npiece = (int)npiece;
    return p;
}

int64_t value_grad_blocks(int hv, int64_t nbat, int64_t ntimes, int64_t nhead) {
    const int64_t keys = hv == 1 ? 64 : 16;
    return nbat * (nhead / hv) * ((ntimes + keys - 1) / keys);
}

int launch_attention_value_grad(float* gv, const float* gy, const float* pp, int64_t nbat, int64_t ntimes, int64_t nvec,
                                int64_t nhead, int64_t npiece, hipStream_t stream) {
    const int hv = attention_value_grad_heads(gv, gy, pp, ntimes, nvec, nhead, npiece);
    if (hv == 0) return fail(KAI_ERR_INVALID_ARGUMENT, "attention value gradient: geometry not served");
    const ValueGradParams p = value_grad_params(gv, gy, pp, ntimes, nvec, nhead, npiece);
    const int64_t blocks = value_grad_blocks(hv, nbat, ntimes, nhead);
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "attention value gradient: grid too large");
    const dim3 grid((unsigned)blocks);
    if (hv == 1) {
        switch (npiece / 16) {
        case 1: launch_vg<1, 1>(p, grid, stream); break;
        case 2: launch_vg<2, 1>(p, grid, stream); break;
        case 3: launch_vg<3, 1>(p, grid, stream); break;
        case 4: launch_vg<4, 1>(p, grid, stream); break;
        case 5: launch_vg<5, 1>(p, grid, stream); break;
        case 6: launch_vg<6, 1>(p, grid, stream); break;
        case 7: launch_vg<7, 1>(p, grid, stream); break;
        default: launch_vg<8, 1>(p, grid, stream); break;
        }
    } else {
        switch (npiece / 16) {
        case 1: launch_vg<1, 4>(p, grid, stream); break;
        case 2: launch_vg<2, 4>(p, grid, stream); break;
        case 3: launch_vg<3, 4>(p, grid, stream); break;
        default: launch_vg<4, 4>(p, grid, stream); break;
        }
    }
    return check_launch("attention_value_grad_kernel");
}

// Y[b, t, h, :] = sum_k P[b, t, k, h] * B[b, k, h, :] for head counts in whole fours: mix_values (B = V, rows of Y
// nhead * npiece floats) and mult_on_heads_backward (P = the gradient of the scores, B = Q or K, rows of nvec floats).
bool attention_heads_mix_applies(const float* out, int64_t out_rs, const float* pp, const float* other, int64_t other_rs,
                                 int64_t ntimes, int64_t nhead, int64_t npiece) {
    return npiece % 16 == 0 && npiece >= 16 && npiece <= 64 && nhead >= 4 && nhead % 4 == 0 && ntimes >= 32 && out_rs % 4 == 0 &&
           nhead * npiece <= out_rs && nhead * npiece <= other_rs && aligned16(out) && aligned16(pp) &&
           (reinterpret_cast<uintptr_t>(other) & 3u) == 0 && (ntimes + 1024) * ntimes * nhead * 4 < (1ll << 31) &&
           (ntimes + 1024) * other_rs * 4 < (1ll << 31);
}

int launch_attention_heads_mix(float* out, int64_t out_rs, const float* pp, const float* other, int64_t other_rs, int64_t nbat,
                               int64_t ntimes, int64_t nhead, int64_t npiece, hipStream_t stream) {
    if (!attention_heads_mix_applies(out, out_rs, pp, other, other_rs, ntimes, nhead, npiece))
        return fail(KAI_ERR_INVALID_ARGUMENT, "attention heads product: geometry not served");
    vgrad::ValueGradParams p{};
    p.P = pp; p.gY = other; p.gV = out;
    p.p_batch_stride = ntimes * ntimes * nhead;
    p.gy_rs = other_rs; p.gv_rs = out_rs;
    p.ntimes = (int)ntimes; p.nhead = (int)nhead; p.npiece = (int)npiece;
    const int64_t blocks = value_grad_blocks(4, nbat, ntimes, nhead);
    if (blocks > kMaxDim) return fail(KAI_ERR_INVALID_ARGUMENT, "attention heads product: grid too large");
    const dim3 grid((unsigned)blocks), block(kVgThreads);
    switch (npiece / 16) {
    case 1: attention_heads_mix_kernel<1><<<grid, block, 0, stream>>>(p); break;
    case 2: attention_heads_mix_kernel<2><<<grid, block, 0, stream>>>(p); break;
    case 3: attention_heads_mix_kernel<3><<<grid, block, 0, stream>>>(p); break;
    default: attention_heads_mix_kernel<4><<<grid, block, 0, stream>>>(p); break;
    }
    return check_launch("attention_heads_mix_kernel");
}

}  // namespace kai
