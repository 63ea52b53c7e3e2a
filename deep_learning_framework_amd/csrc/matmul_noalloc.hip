// kai_matmul_noalloc: VMath::matmul for callers that cannot allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).  Same kernels and the same choice of
// kernel as kai_matmul; the one difference is where a reduction that is cut into parts keeps its partial
// sums: in `scratch` below, a fixed array in the code object's own device memory, instead of the library's
// heap scratch that is allocated and grown on demand.
//
// Every GPU holds its own copy of the array, from the moment the code object is loaded there until the process
// ends.  All calls on one GPU share it: calls that overlap on one GPU (two streams, two threads) race on it and
// must be serialised by the caller.  Nothing in it has to start at zero: every part writes all M x N of its
// sums before the second launch reads them, so what an earlier, larger call left behind is never read.
#include <mutex>

#include "gemm_host.h"
#include "kai_common.h"

constexpr int64_t kNoAllocScratchBytes = 32ll << 20;

static __device__ __align__(256) float scratch[kNoAllocScratchBytes / sizeof(float)];

namespace {

constexpr int kNoAllocMaxDevices = 64;

// In host code the name `scratch` is only a handle for hipGetSymbolAddress: the address the kernels need is
// asked for once per device, with that device current, and kept here.
std::mutex g_noalloc_mutex;
float* g_scratch_ptr[kNoAllocMaxDevices] = {};

int noalloc_scratch(float** out) {
    int dev = 0;
    KAI_TRY(kai::check_hip(hipGetDevice(&dev), "hipGetDevice"));
    if (dev < 0 || dev >= kNoAllocMaxDevices)
        return kai::fail(KAI_ERR_INVALID_ARGUMENT, "kai_matmul_noalloc: device index out of range");
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        // The look-up may load the code object onto this device, which allocates: it must not happen while the
        // calling thread's stream is being captured.  kai_matmul_noalloc_scratch_bytes() or any earlier call on
        // the device does it ahead of time.
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(kai::current_stream(), &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
            return kai::fail(KAI_ERR_GPU, "kai_matmul_noalloc: first use on this device while its stream is being captured; "
                                          "call kai_matmul_noalloc_scratch_bytes() on the device before the capture");
        (void)hipGetLastError();
        float* ptr = nullptr;
        KAI_TRY(kai::check_hip(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)),
                               "hipGetSymbolAddress(scratch)"));
        if (ptr == nullptr) return kai::fail(KAI_ERR_INVALID_POINTER, "kai_matmul_noalloc: no address for the scratch array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return KAI_OK;
}

}  // namespace

extern "C" int kai_matmul_noalloc(int device, float* py, const float* pw, const float* px, int64_t yvec, int64_t ndat,
                                  int64_t xvec, int acc) {
    using namespace kai;
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(yvec >= 0 && yvec <= kMaxDim && ndat >= 0 && ndat <= kMaxDim && xvec >= 0 && xvec <= kMaxDim,
                KAI_ERR_INVALID_ARGUMENT, "dimension out of range");
    if (ndat == 0 || yvec == 0) return KAI_OK;
    KAI_REQUIRE(py != nullptr, KAI_ERR_INVALID_POINTER, "null pointer: py");
    if (xvec > 0) KAI_REQUIRE(pw != nullptr && px != nullptr, KAI_ERR_INVALID_POINTER, "null operand");
    float* ptr = nullptr;
    KAI_TRY(noalloc_scratch(&ptr));
    // y[ndat,yvec] (=|+=) x[ndat,xvec] . w[yvec,xvec]^T, as kai_matmul describes it
    GemmDesc d;
    d.A = px; d.B = pw; d.C = py;
    d.M = ndat; d.N = yvec; d.K = xvec;
    d.a_rs = xvec; d.a_ks = 1; d.b_rs = xvec; d.b_ks = 1; d.c_rs = yvec; d.c_cs = 1;
    d.acc = acc != 0;
    d.scratch = ptr;
    d.scratch_bytes = kNoAllocScratchBytes;
    return launch_gemm(d, current_stream());
}

// Also the set-up call: it looks up the array's address on the current device, so that a later kai_matmul_noalloc
// there has nothing left to do but launch (a failure of the look-up is reported by that later call).
extern "C" int64_t kai_matmul_noalloc_scratch_bytes(void) {
    float* ptr = nullptr;
    (void)noalloc_scratch(&ptr);
    return kNoAllocScratchBytes;
}
