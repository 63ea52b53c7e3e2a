// Chooses the kernel for one (batched) product: the bandwidth-bound skinny kernel for at
// most 16 rows against a K-contiguous weight matrix, otherwise the MFMA kernel in the LDS
// orientation pair that matches how the operands lie in memory, with the largest tile that still
// fills the 256 compute units.
#include "gemm_host.h"
#include "gemv_skinny.h"

namespace kai {

static int64_t tiles_of(int64_t M, int64_t N, int64_t nbatch, int64_t t) {
    return ((M + t - 1) / t) * ((N + t - 1) / t) * nbatch;
}

int launch_gemm(const GemmDesc& d, hipStream_t stream) {
    if (d.M < 0 || d.N < 0 || d.K < 0 || d.nbatch < 0)
        return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: negative dimension");
    if (d.M > kMaxDim || d.N > kMaxDim || d.K > kMaxDim)
        return fail(KAI_ERR_INVALID_ARGUMENT, "gemm: dimension does not fit 31 bits");
    if (d.M == 0 || d.N == 0 || d.nbatch == 0) return KAI_OK;
    if (!d.C || (d.K > 0 && (!d.A || !d.B))) return fail(KAI_ERR_INVALID_POINTER, "gemm: null operand");

    // skinny: y = x . w^T with both operands K-contiguous, a contiguous output row, no scaling
    if (d.M <= kSkinnyMaxRows && d.nbatch == 1 && d.a_ks == 1 && d.b_ks == 1 && d.c_cs == 1 && !d.has_alpha &&
        d.K > 0 && d.N >= 256) {
        SkinnyParams s{};
        s.W = d.B; s.X = d.A; s.Y = d.C; s.Y2 = d.C2; s.bias = d.bias; s.leaky = d.leaky;
        s.ldw = d.b_rs; s.ldx = d.a_rs; s.ldy = d.c_rs;
        s.N = d.N; s.M = (int)d.M; s.K = (int)d.K;
        s.act = d.act; s.accflag = d.acc;
        return launch_skinny_nt(s, stream);
    }

    // batch strides that are never multiplied by a non-zero index must not spoil the alignment checks
    GemmDesc dn = d;
    if (dn.bdiv <= 1) { dn.bdiv = 1; dn.a_bs1 = dn.b_bs1 = dn.c_bs1 = 0; }
    if (dn.nbatch <= dn.bdiv) dn.a_bs0 = dn.b_bs0 = dn.c_bs0 = 0;
    const bool a_kc = operand_is_kc(dn.a_rs, dn.a_ks);
    const bool b_kc = operand_is_kc(dn.b_rs, dn.b_ks);
    const GemmParams p = make_params(dn, a_kc, b_kc);

    // largest tile that still yields about one workgroup per compute unit and is not mostly padding
    const int64_t short_side = d.M < d.N ? d.M : d.N;
    int tile = kTileSmall;
    if (short_side > 128 && tiles_of(d.M, d.N, d.nbatch, 256) >= 192) tile = kTileLarge;
    else if (short_side > 64 && tiles_of(d.M, d.N, d.nbatch, 128) >= 128) tile = kTileMedium;

    if (a_kc && b_kc) return launch_gemm_kc_kc(p, d.nbatch, tile, stream);
    if (a_kc && !b_kc) return launch_gemm_kc_mc(p, d.nbatch, tile, stream);
    if (!a_kc && !b_kc) return launch_gemm_mc_mc(p, d.nbatch, tile, stream);
    return launch_gemm_mc_kc(p, d.nbatch, tile, stream);
}

}  // namespace kai
