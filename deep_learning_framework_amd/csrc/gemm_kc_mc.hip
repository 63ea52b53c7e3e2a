// MFMA GEMM kernels for operand orientations A:kc B:mc (see gemm_mfma.h).
#include "gemm_layout_impl.h"

namespace kai {
int launch_gemm_kc_mc(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream) {
    return launch_gemm_layout<true, false>(p, nbatch, tile, stream);
}
}  // namespace kai
