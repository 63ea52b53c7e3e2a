// MFMA GEMM kernels for operand orientations A:mc B:kc (see gemm_mfma.h).
#include "gemm_layout_impl.h"

namespace kai {
int launch_gemm_mc_kc(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream) {
    return launch_gemm_layout<false, true>(p, nbatch, tile, stream);
}
}  // namespace kai
