// MFMA GEMM kernels for operand orientations A:mc B:mc (see gemm_mfma.h).
#include "gemm_layout_impl.h"

namespace kai {
int launch_gemm_mc_mc(const GemmParams& p, int64_t nbatch, int tile, hipStream_t stream) {
    if (p.rowsum) return launch_gemm_layout_rowsum<false, false>(p, nbatch, tile, stream);
    return launch_gemm_layout<false, false>(p, nbatch, tile, stream);
}
}  // namespace kai
