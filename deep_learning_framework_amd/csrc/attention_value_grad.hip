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

}  // namespace kai
