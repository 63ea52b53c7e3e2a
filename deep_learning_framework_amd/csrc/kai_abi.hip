// extern "C" surface of libkai_hip.so (declared in include/kai_hip.h): argument checks, mapping
// of the engine's VMath argument lists onto GEMM descriptors, library state.
//
// The mapping of (yvec, ndat, xvec) follows the call sites in the reference:
// VTensor::matmul (api_objects/vtensor.cpp:1282-1335), matmul_backprop (:1337-1375),
// mh_attention (:2978-3052) and multihead_attention_backprop (:3054-3227).
#include <cstring>
#include <cstdlib>
#include <cstdio>
#include <mutex>
#include <vector>

#include "elementwise.h"
#include "gemm_host.h"
#include "kai_common.h"

namespace kai {

static thread_local std::string tl_error;
static thread_local hipStream_t tl_stream = nullptr;

int fail(int code, const std::string& msg) {
    tl_error = msg;
    return code;
}
void clear_error() { tl_error.clear(); }
hipStream_t current_stream() { return tl_stream; }

int check_hip(hipError_t st, const char* what) {
    if (st == hipSuccess) return KAI_OK;
    return fail(KAI_ERR_GPU, std::string("hip:") + what + ": " + hipGetErrorString(st));
}

int check_launch(const char* kernel_name) { return check_hip(hipGetLastError(), kernel_name); }

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_ws_mutex;
// Per device: one scratch buffer per STREAM that calls of the library have been enqueued on (the stream a thread
// set with kai_set_stream; the null stream counts as one), so that calls on different streams of a device never
// share partial sums, and the smaller buffers that grown ones replaced.  A replaced buffer is only retired: kernels
// already enqueued that use it stay valid, and growing needs neither a wait for the device nor a hipFree (which
// waits for the device, too).  Retired buffers are released at the library's own synchronisation points, when the
// device is idle anyway (kai_device_synchronize, kai_shutdown) -- except those that were handed out while a stream
// capture was active: a recorded graph keeps the address and may be replayed at any later time, so they stay until
// kai_shutdown.  Growth at least doubles the size, so the retired buffers of a stream together are smaller than
// its current one.
struct StreamScratch {
    hipStream_t stream = nullptr;
    void* ptr = nullptr;
    int64_t bytes = 0;
    bool in_graph = false;     // handed out during a capture
};
struct RetiredScratch {
    void* ptr;
    int64_t bytes;
    bool in_graph;
};
struct DeviceScratch {
    std::vector<StreamScratch> streams;
    std::vector<RetiredScratch> retired;
    int64_t retired_bytes = 0;
    int64_t growths = 0;
};
DeviceScratch g_ws[kMaxDevices];
int g_cu_count[kMaxDevices] = {};
// bytes at the front of the scratch that an enclosing call of this thread holds (ScratchHold)
thread_local int64_t tl_ws_held = 0;
constexpr int64_t kScratchMin = 4ll << 20;
constexpr size_t kMaxScratchStreams = 64;

bool stream_is_capturing(hipStream_t st) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    const hipError_t st_rc = hipStreamIsCapturing(st, &capturing);
    if (st_rc != hipSuccess) {
        (void)hipGetLastError();   // e.g. the query of the null stream while another stream records: not this call's error
        return false;
    }
    return capturing != hipStreamCaptureStatusNone;
}

int grow_scratch(DeviceScratch& d, StreamScratch& s, int64_t need, bool capturing) {
    // an allocation is not allowed while the stream records a graph: the caller sizes the scratch first
    if (capturing)
        return fail(KAI_ERR_GPU, "the library scratch would have to grow to " + std::to_string(need) +
                                     " bytes while the stream is being captured: run the call once before the "
                                     "capture or call kai_reserve_scratch");
    int64_t want = need;
    if (want < 2 * s.bytes) want = 2 * s.bytes;
    if (want < kScratchMin) want = kScratchMin;
    void* fresh = nullptr;
    KAI_TRY(check_hip(hipMalloc(&fresh, (size_t)want), "hipMalloc(scratch)"));
    if (s.ptr) {
        d.retired.push_back(RetiredScratch{s.ptr, s.bytes, s.in_graph});
        d.retired_bytes += s.bytes;
    }
    s.ptr = fresh;
    s.bytes = want;
    s.in_graph = false;
    d.growths++;
    return KAI_OK;
}

// the device is idle: every retired buffer that no recorded graph may still name goes back
void release_retired(DeviceScratch& d) {
    std::vector<RetiredScratch> kept;
    for (const RetiredScratch& r : d.retired) {
        if (r.in_graph || hipFree(r.ptr) != hipSuccess) kept.push_back(r);
        else d.retired_bytes -= r.bytes;
    }
    d.retired.swap(kept);
}
}  // namespace

int workspace(int64_t bytes, float** out) {
    int dev = 0;
    KAI_TRY(check_hip(hipGetDevice(&dev), "hipGetDevice"));
    if (dev < 0 || dev >= kMaxDevices) return fail(KAI_ERR_INVALID_ARGUMENT, "workspace: device index out of range");
    if (bytes < 0) return fail(KAI_ERR_INVALID_ARGUMENT, "workspace: negative size");
    const hipStream_t st = current_stream();
    const bool capturing = stream_is_capturing(st);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    DeviceScratch& d = g_ws[dev];
    StreamScratch* s = nullptr;
    for (StreamScratch& e : d.streams)
        if (e.stream == st) s = &e;
    if (s == nullptr) {
        if (d.streams.size() >= kMaxScratchStreams)
            return fail(KAI_ERR_INVALID_ARGUMENT, "workspace: more than 64 streams of one device have asked for scratch memory; "
                                                  "kai_shutdown releases the buffers of streams that are gone");
        d.streams.push_back(StreamScratch{});
        s = &d.streams.back();
        s->stream = st;
    }
    const int64_t need = tl_ws_held + bytes;
    if (s->bytes < need) KAI_TRY(grow_scratch(d, *s, need, capturing));
    if (capturing) s->in_graph = true;
    *out = reinterpret_cast<float*>(static_cast<char*>(s->ptr) + tl_ws_held);
    return KAI_OK;
}

ScratchHold::ScratchHold(int64_t bytes) : previous_(tl_ws_held) { tl_ws_held += (bytes + 255) / 256 * 256; }
ScratchHold::~ScratchHold() { tl_ws_held = previous_; }

int compute_units() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    if (g_cu_count[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        g_cu_count[dev] = n;
    }
    return g_cu_count[dev];
}

static int release_workspaces() {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    int old = 0;
    if (hipGetDevice(&old) != hipSuccess) old = 0;
    int rc = KAI_OK;
    for (int d = 0; d < kMaxDevices; d++) {
        DeviceScratch& s = g_ws[d];
        if (s.streams.empty() && s.retired.empty()) continue;
        if (hipSetDevice(d) == hipSuccess) {
            (void)hipDeviceSynchronize();
            for (const StreamScratch& e : s.streams)
                if (e.ptr && hipFree(e.ptr) != hipSuccess) rc = KAI_ERR_GPU;
            for (const RetiredScratch& r : s.retired)
                if (hipFree(r.ptr) != hipSuccess) rc = KAI_ERR_GPU;
        }
        s = DeviceScratch();
    }
    (void)hipSetDevice(old);
    return rc;
}

// after a successful wait for the current device
static void release_retired_of_current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    release_retired(g_ws[dev]);
}

static bool act_is_elementwise(int act) { return act >= KAI_ACT_NONE && act <= KAI_ACT_SWISH; }

}  // namespace kai

using namespace kai;

#define KAI_REQUIRE_PTR(p) KAI_REQUIRE((p) != nullptr, KAI_ERR_INVALID_POINTER, "null pointer: " #p)
#define KAI_REQUIRE_DIM(v) \
    KAI_REQUIRE((v) >= 0 && (v) <= kMaxDim, KAI_ERR_INVALID_ARGUMENT, "dimension out of range: " #v)

extern "C" {

// ---- library state -----------------------------------------------------------------------------

const char* kai_last_error(void) { return tl_error.c_str(); }

int kai_device_count(int* count) {
    KAI_REQUIRE_PTR(count);
    return check_hip(hipGetDeviceCount(count), "hipGetDeviceCount");
}

int kai_set_device(int device) { return check_hip(hipSetDevice(device), "hipSetDevice"); }

int kai_device_synchronize(void) {
    KAI_TRY(check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize"));
    release_retired_of_current_device();   // the device is idle: scratch buffers that grown ones replaced go back
    return KAI_OK;
}

int kai_set_stream(void* hip_stream) {
    tl_stream = reinterpret_cast<hipStream_t>(hip_stream);
    return KAI_OK;
}

int kai_shutdown(void) {
    const int rc = release_workspaces();
    if (rc != KAI_OK) return fail(rc, "kai_shutdown: hipFree failed");
    return KAI_OK;
}

int kai_reserve_scratch(int64_t bytes) {
    KAI_REQUIRE(bytes >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    float* unused = nullptr;
    return workspace(bytes, &unused);
}

int kai_scratch_info(int64_t* bytes, int64_t* growths, int64_t* retired_bytes) {
    int dev = 0;
    KAI_TRY(check_hip(hipGetDevice(&dev), "hipGetDevice"));
    KAI_REQUIRE(dev >= 0 && dev < kMaxDevices, KAI_ERR_INVALID_ARGUMENT, "device index out of range");
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (bytes) {
        *bytes = 0;
        for (const StreamScratch& e : g_ws[dev].streams)
            if (e.stream == current_stream()) *bytes = e.bytes;
    }
    if (growths) *growths = g_ws[dev].growths;
    if (retired_bytes) *retired_bytes = g_ws[dev].retired_bytes;
    return KAI_OK;
}

int kai_arch_info(char* built_for, char* device_arch, int buflen) {
    KAI_REQUIRE(buflen > 0, KAI_ERR_INVALID_ARGUMENT, "buflen <= 0");
    if (built_for) {
        std::strncpy(built_for, "gfx950", buflen - 1);
        built_for[buflen - 1] = 0;
    }
    if (device_arch) {
        int dev = 0;
        KAI_TRY(check_hip(hipGetDevice(&dev), "hipGetDevice"));
        hipDeviceProp_t prop;
        KAI_TRY(check_hip(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties"));
        std::strncpy(device_arch, prop.gcnArchName, buflen - 1);
        device_arch[buflen - 1] = 0;
    }
    return KAI_OK;
}

// ---- memory ------------------------------------------------------------------------------------

int kai_mem_alloc(int device, int64_t size, void** out_ptr) {
    KAI_REQUIRE_PTR(out_ptr);
    *out_ptr = nullptr;
    KAI_REQUIRE(size >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (device < 0) {
        void* p = std::malloc((size_t)(size > 0 ? size : 1));
        if (!p) return fail(KAI_ERR_HOSTMEM_ALLOC_FAILURE, "kai_mem_alloc: host allocation failed");
        *out_ptr = p;
        return KAI_OK;
    }
    if (size % 16 != 0) size += 16 - size % 16;
    if (size == 0) size = 16;
    int old_device = 0;
    KAI_TRY(check_hip(hipGetDevice(&old_device), "hipGetDevice"));
    KAI_TRY(check_hip(hipSetDevice(device), "hipSetDevice"));
    void* p = nullptr;
    const hipError_t st = hipMalloc(&p, (size_t)size);
    const hipError_t st2 = hipSetDevice(old_device);
    KAI_TRY(check_hip(st, "hipMalloc"));
    KAI_TRY(check_hip(st2, "hipSetDevice"));
    if (!p) return fail(KAI_ERR_INVALID_POINTER, "kai_mem_alloc: hipMalloc returned null");
    *out_ptr = p;
    return KAI_OK;
}

int kai_mem_free(int device, void* ptr) {
    if (device < 0) {
        std::free(ptr);
        return KAI_OK;
    }
    return check_hip(hipFree(ptr), "hipFree");
}

static int copy_blocking(void* d, const void* s, int64_t size, hipMemcpyKind kind, const char* what) {
    KAI_REQUIRE(size >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (size == 0) return KAI_OK;
    KAI_REQUIRE(d != nullptr && s != nullptr, KAI_ERR_INVALID_POINTER, "null pointer");
    if (kind == hipMemcpyHostToHost) {
        std::memcpy(d, s, (size_t)size);
        return KAI_OK;
    }
    // ordered after the work already enqueued on this thread's stream, then blocks, like the
    // reference's cudaMemcpy on the legacy stream
    hipStream_t st = current_stream();
    KAI_TRY(check_hip(hipMemcpyAsync(d, s, (size_t)size, kind, st), what));
    return check_hip(hipStreamSynchronize(st), what);
}

int kai_memcpy_host_to_host(void* d, const void* s, int64_t size) {
    return copy_blocking(d, s, size, hipMemcpyHostToHost, "memcpy_host_to_host");
}
int kai_memcpy_host_to_device(void* d, const void* s, int64_t size) {
    return copy_blocking(d, s, size, hipMemcpyHostToDevice, "memcpy_host_to_device");
}
int kai_memcpy_device_to_host(void* d, const void* s, int64_t size) {
    return copy_blocking(d, s, size, hipMemcpyDeviceToHost, "memcpy_device_to_host");
}
int kai_memcpy_device_to_device(void* d, const void* s, int64_t size) {
    return copy_blocking(d, s, size, hipMemcpyDeviceToDevice, "memcpy_device_to_device");
}

int kai_copy_data(int dest_device, int src_device, void* py, const void* px, int64_t nbytes) {
    if (dest_device < 0)
        return src_device < 0 ? kai_memcpy_host_to_host(py, px, nbytes) : kai_memcpy_device_to_host(py, px, nbytes);
    return src_device < 0 ? kai_memcpy_host_to_device(py, px, nbytes) : kai_memcpy_device_to_device(py, px, nbytes);
}

int kai_fill_int(int device, int* ptr, int64_t size, int value) {
    KAI_REQUIRE(size >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (size == 0) return KAI_OK;
    KAI_REQUIRE_PTR(ptr);
    if (device < 0) {
        for (int64_t i = 0; i < size; i++) ptr[i] = value;
        return KAI_OK;
    }
    return launch_fill_int(ptr, size, value, current_stream());
}

int kai_fill_float(int device, float* ptr, int64_t size, float value) {
    KAI_REQUIRE(size >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (size == 0) return KAI_OK;
    KAI_REQUIRE_PTR(ptr);
    if (device < 0) {
        for (int64_t i = 0; i < size; i++) ptr[i] = value;
        return KAI_OK;
    }
    return launch_fill_float(ptr, size, value, current_stream());
}

int kai_set_zero(int device, void* ptr, int64_t size) {
    KAI_REQUIRE(size >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (size == 0) return KAI_OK;
    KAI_REQUIRE_PTR(ptr);
    if (device < 0) {
        std::memset(ptr, 0, (size_t)size);
        return KAI_OK;
    }
    // a fill kernel rather than hipMemsetAsync, so that callers may capture the call in a graph
    if (size % 4 == 0 && (reinterpret_cast<uintptr_t>(ptr) & 3u) == 0)
        return launch_fill_int(static_cast<int*>(ptr), size / 4, 0, current_stream());
    return check_hip(hipMemsetAsync(ptr, 0, (size_t)size, current_stream()), "hipMemsetAsync");
}

int kai_memcpy_from_host(int device, void* py, const void* px, int64_t size) {
    return device < 0 ? kai_memcpy_host_to_host(py, px, size) : kai_memcpy_host_to_device(py, px, size);
}
int kai_memcpy_to_host(int device, void* py, const void* px, int64_t size) {
    return device < 0 ? kai_memcpy_host_to_host(py, px, size) : kai_memcpy_device_to_host(py, px, size);
}
int kai_memcpy_to_device(int device, void* py, const void* px, int64_t size) {
    return device < 0 ? kai_memcpy_host_to_device(py, px, size) : kai_memcpy_device_to_device(py, px, size);
}
int kai_get_slice(int device, void* py, const void* px, int64_t nbytes) {
    return device < 0 ? kai_memcpy_host_to_device(py, px, nbytes) : kai_memcpy_device_to_device(py, px, nbytes);
}

// ---- dense layer -------------------------------------------------------------------------------

int kai_gemm_f32(int device, int transA, int transB, int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                 const float* B, int64_t ldb, float* C, int64_t ldc, const float* bias, int actFunc,
                 const float* hLeakyAlpha, int acc) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE_DIM(M); KAI_REQUIRE_DIM(N); KAI_REQUIRE_DIM(K);
    KAI_REQUIRE(act_is_elementwise(actFunc), KAI_ERR_CONDITIONAL_STATEMENT, "activation code must be 0..8");
    if (M == 0 || N == 0) return KAI_OK;
    KAI_REQUIRE_PTR(C);
    if (K > 0) { KAI_REQUIRE_PTR(A); KAI_REQUIRE_PTR(B); }
    KAI_REQUIRE(lda >= (transA ? M : K) && ldb >= (transB ? K : N) && ldc >= N, KAI_ERR_INVALID_ARGUMENT,
                "leading dimension smaller than the row length");
    KAI_REQUIRE(lda <= kMaxDim && ldb <= kMaxDim && ldc <= kMaxDim, KAI_ERR_INVALID_ARGUMENT,
                "leading dimension out of range");
    GemmDesc d;
    d.A = A; d.B = B; d.C = C; d.bias = bias; d.leaky = hLeakyAlpha;
    d.M = M; d.N = N; d.K = K;
    if (transA) { d.a_rs = 1; d.a_ks = lda; } else { d.a_rs = lda; d.a_ks = 1; }
    if (transB) { d.b_rs = ldb; d.b_ks = 1; } else { d.b_rs = 1; d.b_ks = ldb; }
    d.c_rs = ldc; d.c_cs = 1;
    d.act = actFunc; d.acc = acc != 0;
    return launch_gemm(d, current_stream());
}

int kai_gemm_plan(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                  int has_bias, int actFunc, int acc, char* out, int buflen) {
    KAI_REQUIRE_PTR(out);
    KAI_REQUIRE(buflen > 0, KAI_ERR_INVALID_ARGUMENT, "buflen <= 0");
    KAI_REQUIRE_DIM(M); KAI_REQUIRE_DIM(N); KAI_REQUIRE_DIM(K);
    KAI_REQUIRE(act_is_elementwise(actFunc), KAI_ERR_CONDITIONAL_STATEMENT, "activation code must be 0..8");
    KAI_REQUIRE(lda >= (transA ? M : K) && ldb >= (transB ? K : N) && ldc >= N, KAI_ERR_INVALID_ARGUMENT,
                "leading dimension smaller than the row length");
    // stand-ins for 16-byte aligned operands; nothing dereferences them
    static float dummy[16] __attribute__((aligned(64)));
    GemmDesc d;
    d.A = dummy; d.B = dummy; d.C = dummy; d.bias = has_bias ? dummy : nullptr;
    d.M = M; d.N = N; d.K = K;
    if (transA) { d.a_rs = 1; d.a_ks = lda; } else { d.a_rs = lda; d.a_ks = 1; }
    if (transB) { d.b_rs = ldb; d.b_ks = 1; } else { d.b_rs = 1; d.b_ks = ldb; }
    d.c_rs = ldc; d.c_cs = 1;
    d.act = actFunc; d.acc = acc != 0;
    const std::string text = describe_gemm(d);
    std::strncpy(out, text.c_str(), (size_t)buflen - 1);
    out[buflen - 1] = 0;
    return KAI_OK;
}

int kai_matmul(int device, float* py, const float* pw, const float* px, int64_t yvec, int64_t ndat, int64_t xvec,
               int acc) {
    // y[ndat,yvec] = x[ndat,xvec] . w[yvec,xvec]^T : A = x (K-contiguous), B = w stored [N,K]
    return kai_gemm_f32(device, 0, 1, ndat, yvec, xvec, px, xvec, pw, xvec, py, yvec, nullptr, KAI_ACT_NONE, nullptr,
                        acc);
}

int kai_matmul_backward_x(int device, float* pgx, const float* pgy, const float* pw, int64_t yvec, int64_t ndat,
                          int64_t xvec, int acc) {
    // gx[ndat,xvec] = gy[ndat,yvec] . w[yvec,xvec] : reduction over yvec, B = w stored [K,N]
    return kai_gemm_f32(device, 0, 0, ndat, xvec, yvec, pgy, yvec, pw, xvec, pgx, xvec, nullptr, KAI_ACT_NONE,
                        nullptr, acc);
}

int kai_matmul_backward_w(int device, float* pgw, const float* pgy, const float* px, int64_t yvec, int64_t ndat,
                          int64_t xvec, int acc) {
    // gw[yvec,xvec] = gy[ndat,yvec]^T . x[ndat,xvec] : reduction over ndat, A stored [K,M], B stored [K,N]
    return kai_gemm_f32(device, 1, 0, yvec, xvec, ndat, pgy, yvec, px, xvec, pgw, xvec, nullptr, KAI_ACT_NONE,
                        nullptr, acc);
}

int kai_add_bias(int device, float* py, const float* pa, const float* pb, int64_t nrow, int64_t ncol) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (nrow == 0 || ncol == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(pa); KAI_REQUIRE_PTR(pb);
    return launch_add_bias(py, pa, pb, nrow, ncol, current_stream());
}

int kai_add_bias_backward_b(int device, float* pgb, const float* pgy, int64_t nrow, int64_t ncol, int acc) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (ncol == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgb);
    if (nrow > 0) KAI_REQUIRE_PTR(pgy);
    int parts = colsum_row_parts(nrow, ncol);
    float* parts_buf = nullptr;
    // no scratch to be had (the stream is being captured and the buffer would have to grow, or the allocation
    // failed): the single launch needs none
    if (parts >= 2 && workspace(parts * ncol * (int64_t)sizeof(float), &parts_buf) != KAI_OK) {
        parts = 1;
        parts_buf = nullptr;
    }
    return launch_colsum(pgb, pgy, nrow, ncol, acc != 0, current_stream(), parts_buf, parts);
}

int kai_activate(int device, float* py, const float* px, int64_t nrow, int64_t ncol, int actFunc,
                 const float* hLeakyAlpha) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    KAI_REQUIRE(actFunc >= KAI_ACT_NONE && actFunc <= KAI_ACT_SOFTMAX, KAI_ERR_CONDITIONAL_STATEMENT,
                "unknown activation code");
    if (nrow == 0 || ncol == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(px);
    if (actFunc == KAI_ACT_SOFTMAX) return launch_softmax_rows(py, px, nrow, ncol, current_stream());
    return launch_activate(py, px, nrow * ncol, actFunc, hLeakyAlpha, current_stream());
}

int kai_activate_backward(int device, float* pgx, const float* pgy, const float* px, int64_t nrow, int64_t ncol,
                          int actFunc, const float* hLeakyAlpha) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    KAI_REQUIRE(actFunc >= KAI_ACT_NONE && actFunc <= KAI_ACT_SOFTMAX, KAI_ERR_CONDITIONAL_STATEMENT,
                "unknown activation code");
    if (nrow == 0 || ncol == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgx); KAI_REQUIRE_PTR(pgy); KAI_REQUIRE_PTR(px);
    if (actFunc == KAI_ACT_SOFTMAX) return launch_softmax_rows_backward(pgx, pgy, px, nrow, ncol, current_stream());
    return launch_activate_backward(pgx, pgy, px, nrow * ncol, actFunc, hLeakyAlpha, current_stream());
}

int kai_activate_backward_with_y(int device, float* pgx, const float* pgy, const float* py, int64_t nrow,
                                 int64_t ncol, int actFunc, const float* hLeakyAlpha) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    KAI_REQUIRE(actFunc >= KAI_ACT_NONE && actFunc <= KAI_ACT_TANH, KAI_ERR_CONDITIONAL_STATEMENT,
                "activation code must be 0..4");
    if (nrow == 0 || ncol == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgx); KAI_REQUIRE_PTR(pgy); KAI_REQUIRE_PTR(py);
    return launch_activate_backward_with_y(pgx, pgy, py, nrow * ncol, actFunc, hLeakyAlpha, current_stream());
}

// ---- attention ---------------------------------------------------------------------------------

static int check_heads(const char* fn, int64_t nbat, int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece) {
    if (nbat < 0 || ntimes < 0 || nvec < 0 || nhead < 0 || npiece < 0)
        return fail(KAI_ERR_INVALID_ARGUMENT, std::string(fn) + ": negative dimension");
    if (nhead * npiece > nvec) return fail(KAI_ERR_INVALID_ARGUMENT, std::string(fn) + ": nhead*npiece > nvec");
    if (ntimes > kMaxDim || nvec > kMaxDim || nbat * nhead > 65535)
        return fail(KAI_ERR_INVALID_ARGUMENT, std::string(fn) + ": dimension out of range");
    return KAI_OK;
}

int kai_mult_on_heads(int device, float* pp, const float* pK, const float* pQ, int64_t nbat, int64_t ntimes,
                      int64_t nvec, int64_t nhead, int64_t npiece, const float* hCoef) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pp); KAI_REQUIRE_PTR(pK); KAI_REQUIRE_PTR(pQ);
    // per (b,h): S[q,k] = coef * Q_h[q,:] . K_h[k,:] ; both K-contiguous; S element stride nhead
    GemmDesc d;
    d.A = pQ; d.B = pK; d.C = pp; d.alpha = hCoef; d.has_alpha = 1;
    d.M = ntimes; d.N = ntimes; d.K = npiece;
    d.a_rs = nvec; d.a_ks = 1; d.b_rs = nvec; d.b_ks = 1;
    d.c_rs = ntimes * nhead; d.c_cs = nhead;
    d.nbatch = nbat * nhead; d.bdiv = nhead;
    d.a_bs0 = ntimes * nvec; d.a_bs1 = npiece;
    d.b_bs0 = ntimes * nvec; d.b_bs1 = npiece;
    d.c_bs0 = ntimes * ntimes * nhead; d.c_bs1 = 1;
    return launch_gemm(d, current_stream());
}

int kai_mult_on_heads_backward(int device, float* pgQKV, const float* pgp, const float* pQKV, int64_t nbat,
                               int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0 || npiece == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgQKV); KAI_REQUIRE_PTR(pgp); KAI_REQUIRE_PTR(pQKV);
    if (attention_heads_mix_applies(pgQKV, nvec, pgp, pQKV, nvec, ntimes, nhead, npiece))
        return launch_attention_heads_mix(pgQKV, nvec, pgp, pQKV, nvec, nbat, ntimes, nhead, npiece, current_stream());
    // per (b,h): G[t,p] = sum_k gp[b,t,k,h] * KQ[b,k,h*npiece+p]
    GemmDesc d;
    d.A = pgp; d.B = pQKV; d.C = pgQKV;
    d.M = ntimes; d.N = npiece; d.K = ntimes;
    d.a_rs = ntimes * nhead; d.a_ks = nhead;
    d.b_rs = 1; d.b_ks = nvec;
    d.c_rs = nvec; d.c_cs = 1;
    d.nbatch = nbat * nhead; d.bdiv = nhead;
    d.a_bs0 = ntimes * ntimes * nhead; d.a_bs1 = 1;
    d.b_bs0 = ntimes * nvec; d.b_bs1 = npiece;
    d.c_bs0 = ntimes * nvec; d.c_bs1 = npiece;
    return launch_gemm(d, current_stream());
}

int kai_set_mh_attention_mask(int device, float* pp, int64_t ndat, int64_t ntimes, int64_t nhead, int forward) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0 && ntimes >= 0 && nhead >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (ndat == 0 || ntimes == 0 || nhead == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pp);
    return launch_attention_mask(pp, ndat, ntimes, nhead, forward != 0, current_stream());
}

int kai_softmax_direct_on_axis(int device, float* pp, int64_t nrow, int64_t nvec, int64_t ncol) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0 && nvec >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (nrow == 0 || nvec == 0 || ncol == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pp);
    return launch_softmax_axis(pp, nrow, nvec, ncol, current_stream());
}

int kai_softmax_direct_on_axis_backward(int device, float* pgp, const float* pp, int64_t nbat, int64_t ntimes,
                                        int64_t nhead, const float* hCoef) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nbat >= 0 && ntimes >= 0 && nhead >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (nbat == 0 || ntimes == 0 || nhead == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgp); KAI_REQUIRE_PTR(pp);
    return launch_softmax_axis_backward(pgp, pp, nbat * ntimes, ntimes, nhead, hCoef, current_stream());
}

int kai_mix_values(int device, float* py, const float* pp, const float* pV, int64_t nbat, int64_t ntimes,
                   int64_t nvec, int64_t nhead, int64_t npiece) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0 || npiece == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(pp); KAI_REQUIRE_PTR(pV);
    if (attention_heads_mix_applies(py, nhead * npiece, pp, pV, nvec, ntimes, nhead, npiece))
        return launch_attention_heads_mix(py, nhead * npiece, pp, pV, nvec, nbat, ntimes, nhead, npiece, current_stream());
    // per (b,h): Y[q,p] = sum_k P[b,q,k,h] * V[b,k,h*npiece+p]; Y is [nbat, ntimes, nhead, npiece]
    GemmDesc d;
    d.A = pp; d.B = pV; d.C = py;
    d.M = ntimes; d.N = npiece; d.K = ntimes;
    d.a_rs = ntimes * nhead; d.a_ks = nhead;
    d.b_rs = 1; d.b_ks = nvec;
    d.c_rs = nhead * npiece; d.c_cs = 1;
    d.nbatch = nbat * nhead; d.bdiv = nhead;
    d.a_bs0 = ntimes * ntimes * nhead; d.a_bs1 = 1;
    d.b_bs0 = ntimes * nvec; d.b_bs1 = npiece;
    d.c_bs0 = ntimes * nhead * npiece; d.c_bs1 = npiece;
    return launch_gemm(d, current_stream());
}

int kai_mix_values_backward_prop(int device, float* pgp, const float* pgy, const float* pV, int64_t nbat,
                                 int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgp); KAI_REQUIRE_PTR(pgy); KAI_REQUIRE_PTR(pV);
    // per (b,h): gP[q,k] = sum_p gY[b,q,h,p] * V[b,k,h*npiece+p]
    GemmDesc d;
    d.A = pgy; d.B = pV; d.C = pgp;
    d.M = ntimes; d.N = ntimes; d.K = npiece;
    d.a_rs = nhead * npiece; d.a_ks = 1;
    d.b_rs = nvec; d.b_ks = 1;
    d.c_rs = ntimes * nhead; d.c_cs = nhead;
    d.nbatch = nbat * nhead; d.bdiv = nhead;
    d.a_bs0 = ntimes * nhead * npiece; d.a_bs1 = npiece;
    d.b_bs0 = ntimes * nvec; d.b_bs1 = npiece;
    d.c_bs0 = ntimes * ntimes * nhead; d.c_bs1 = 1;
    return launch_gemm(d, current_stream());
}

int kai_mix_values_backward_value(int device, float* pgV, const float* pgy, const float* pp, int64_t nbat,
                                  int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0 || npiece == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgV); KAI_REQUIRE_PTR(pgy); KAI_REQUIRE_PTR(pp);
    if (attention_value_grad_heads(pgV, pgy, pp, ntimes, nvec, nhead, npiece))
        return launch_attention_value_grad(pgV, pgy, pp, nbat, ntimes, nvec, nhead, npiece, current_stream());
    // per (b,h): gV[k,p] = sum_q P[b,q,k,h] * gY[b,q,h,p] : rows of the product are k, reduction over q
    GemmDesc d;
    d.A = pp; d.B = pgy; d.C = pgV;
    d.M = ntimes; d.N = npiece; d.K = ntimes;
    d.a_rs = nhead; d.a_ks = ntimes * nhead;
    d.b_rs = 1; d.b_ks = nhead * npiece;
    d.c_rs = nvec; d.c_cs = 1;
    d.nbatch = nbat * nhead; d.bdiv = nhead;
    d.a_bs0 = ntimes * ntimes * nhead; d.a_bs1 = 1;
    d.b_bs0 = ntimes * nhead * npiece; d.b_bs1 = npiece;
    d.c_bs0 = ntimes * nvec; d.c_bs1 = npiece;
    return launch_gemm(d, current_stream());
}

// ---- fused dense layer -------------------------------------------------------------------------

int kai_dense_forward(int device, float* py, float* ppre, const float* pw, const float* pb, const float* px,
                      int64_t yvec, int64_t ndat, int64_t xvec, int actFunc, const float* hLeakyAlpha) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE_DIM(yvec); KAI_REQUIRE_DIM(ndat); KAI_REQUIRE_DIM(xvec);
    KAI_REQUIRE(act_is_elementwise(actFunc), KAI_ERR_CONDITIONAL_STATEMENT, "activation code must be 0..8");
    if (ndat == 0 || yvec == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py);
    if (xvec > 0) { KAI_REQUIRE_PTR(pw); KAI_REQUIRE_PTR(px); }
    GemmDesc d;
    d.A = px; d.B = pw; d.C = py; d.C2 = ppre; d.bias = pb; d.leaky = hLeakyAlpha;
    d.M = ndat; d.N = yvec; d.K = xvec;
    d.a_rs = xvec; d.a_ks = 1; d.b_rs = xvec; d.b_ks = 1; d.c_rs = yvec; d.c_cs = 1;
    d.act = actFunc;
    return launch_gemm(d, current_stream());
}

int kai_dense_backward(int device, float* pgx, float* pgw, float* pgb, float* pga_work, const float* pgy,
                       const float* pw, const float* px, const float* ppre, int64_t yvec, int64_t ndat,
                       int64_t xvec, int actFunc, const float* hLeakyAlpha, int acc) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE_DIM(yvec); KAI_REQUIRE_DIM(ndat); KAI_REQUIRE_DIM(xvec);
    KAI_REQUIRE(act_is_elementwise(actFunc), KAI_ERR_CONDITIONAL_STATEMENT, "activation code must be 0..8");
    KAI_REQUIRE_PTR(pgy);
    if (pgx) KAI_REQUIRE_PTR(pw);
    if (pgw && yvec > 0 && xvec > 0) KAI_REQUIRE_PTR(px);
    const bool has_act = actFunc != KAI_ACT_NONE && ppre != nullptr;
    // a mini-batch step's sizes: both products, the activation's derivative and the bias gradient in ONE
    // launch (dense_backward.hip), plus the sum of the parts when gx's reduction is cut
    const int pair_split = dense_backward_pair_split(pgx, pgw, pgy, pw, px, has_act ? ppre : nullptr, yvec, ndat, xvec,
                                                     has_act ? actFunc : KAI_ACT_NONE);
    if (pair_split > 0)
        return launch_dense_backward_pair(pgx, pgw, pgb, pgy, pw, px, has_act ? ppre : nullptr, yvec, ndat, xvec,
                                          has_act ? actFunc : KAI_ACT_NONE, hLeakyAlpha, acc != 0, pair_split,
                                          current_stream());
    // otherwise the separate calls.  ga = gy * f'(pre) goes to the caller's work buffer, or, without one, to
    // the library scratch (the products below may ask for scratch of their own: it is placed behind ga)
    const float* ga = pgy;
    int64_t held_bytes = 0;
    if (has_act && ndat > 0 && yvec > 0) {
        float* work = pga_work;
        if (work == nullptr) {
            held_bytes = ndat * yvec * (int64_t)sizeof(float);
            KAI_TRY(workspace(held_bytes, &work));
        }
        KAI_TRY(launch_activate_backward(work, pgy, ppre, ndat * yvec, actFunc, hLeakyAlpha, current_stream()));
        ga = work;
    }
    ScratchHold held(held_bytes);
    // gw[yvec,xvec] = ga^T . x reads every element of ga; where that product runs on the medium or small
    // tile its first tile column also produces gb = column sums of ga, in the order of a sequential loop
    GemmDesc dw;
    bool fused_gb = false;
    if (pgw && yvec > 0 && xvec > 0) {
        dw.A = ga; dw.B = px; dw.C = pgw;
        dw.M = yvec; dw.N = xvec; dw.K = ndat;
        dw.a_rs = 1; dw.a_ks = yvec; dw.b_rs = 1; dw.b_ks = xvec; dw.c_rs = xvec; dw.c_cs = 1;
        dw.acc = acc != 0;
        if (pgb && ndat > 0 && gemm_fuses_rowsum(dw)) {
            dw.rowsum = pgb;
            dw.rowsum_acc = acc != 0;
            fused_gb = true;
        }
    }
    if (pgb && !fused_gb) KAI_TRY(kai_add_bias_backward_b(device, pgb, ga, ndat, yvec, acc));
    if (pgx) KAI_TRY(kai_matmul_backward_x(device, pgx, ga, pw, yvec, ndat, xvec, acc));
    if (pgw && yvec > 0 && xvec > 0) KAI_TRY(launch_gemm(dw, current_stream()));
    return KAI_OK;
}

// ---- cosine similarity ------------------------------------------------------------------------------

int kai_cosinesim(int device, float* py, const float* px1, const float* px2, int64_t nrow1, int64_t nrow2,
                  int64_t ncol) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow1 >= 0 && nrow2 >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (nrow1 == 0 || nrow2 == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py);
    if (ncol == 0) return launch_fill_float(py, nrow1 * nrow2, 0.0f, current_stream());   // 0 / 1e-20
    KAI_REQUIRE_PTR(px1); KAI_REQUIRE_PTR(px2);
    if (cosine_few_rows_applies(px1, px2, nrow1, nrow2, ncol))
        return launch_cosine_few_rows(py, px1, px2, nrow1, nrow2, ncol, current_stream());
    // the products are y = x1 . x2^T, the same NT product as matmul with x2 in the weight's place
    KAI_TRY(kai_matmul(device, py, px2, px1, nrow2, nrow1, ncol, 0));
    // the product may have used the scratch for its own partial sums; in stream order it is free again here
    float* norms = nullptr;
    KAI_TRY(workspace((nrow1 + nrow2) * (int64_t)sizeof(float), &norms));
    return launch_cosine_norms_and_scale(py, norms, px1, px2, nrow1, nrow2, ncol, current_stream());
}

// ---- recurrent cells: the element-wise steps between the gate products -----------------------------

int kai_copy(int device, float* py, const float* pa, int64_t ndat) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (ndat == 0 || py == pa) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(pa);
    // in stream order, like the reference's copy kernel
    const hipError_t e = hipMemcpyAsync(py, pa, (size_t)ndat * sizeof(float), hipMemcpyDeviceToDevice, current_stream());
    if (e != hipSuccess) return fail(KAI_ERR_GPU, std::string("copy: ") + hipGetErrorString(e));
    return KAI_OK;
}

int kai_add(int device, float* py, const float* pa, const float* pb, int64_t ndat) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (ndat == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(pa); KAI_REQUIRE_PTR(pb);
    return launch_add(py, pa, pb, ndat, current_stream());
}

int kai_lstm_process(int device, float* pr, float* ps, const float* ps1, const float* pa, int64_t ndat, int64_t nrec,
                     int64_t ninp) {
    (void)ninp;   // carried by the reference's signature, not used by its loops either
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0 && nrec >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (ndat == 0 || nrec == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pr); KAI_REQUIRE_PTR(ps); KAI_REQUIRE_PTR(pa);
    return launch_lstm_process(pr, ps, ps1, pa, ndat, nrec, current_stream());
}

int kai_lstm_process_backward(int device, const float* pgr, float* pgs, float* pga, const float* ps, const float* pa,
                              int64_t ndat, int64_t nrec, int64_t ninp) {
    (void)ninp;
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0 && nrec >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (ndat == 0 || nrec == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgr); KAI_REQUIRE_PTR(pgs); KAI_REQUIRE_PTR(pga); KAI_REQUIRE_PTR(pa);
    return launch_lstm_process_backward(pgr, pgs, pga, ps, pa, ndat, nrec, current_stream());
}

int kai_gru_process(int device, float* pr, const float* pai, const float* par, int64_t nt, int64_t ntimes, int64_t ndat,
                    int64_t nrec) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0 && nrec >= 0 && nt >= 0 && nt < ntimes, KAI_ERR_INVALID_ARGUMENT, "bad time step or dimension");
    if (ndat == 0 || nrec == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pr); KAI_REQUIRE_PTR(pai); KAI_REQUIRE_PTR(par);
    return launch_gru_process(pr, pai, par, nt, ndat, nrec, current_stream());
}

int kai_gru_process_backward(int device, float* pgr, float* pgai, float* pgar, const float* pr, const float* pai,
                             const float* par, int64_t nt, int64_t ntimes, int64_t ndat, int64_t nrec) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0 && nrec >= 0 && nt >= 0 && nt < ntimes, KAI_ERR_INVALID_ARGUMENT, "bad time step or dimension");
    if (ndat == 0 || nrec == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgr); KAI_REQUIRE_PTR(pgai); KAI_REQUIRE_PTR(pgar);
    KAI_REQUIRE_PTR(pr); KAI_REQUIRE_PTR(pai); KAI_REQUIRE_PTR(par);
    KAI_REQUIRE(pgai != pgar, KAI_ERR_INVALID_ARGUMENT, "gru_process_backward needs separate gate gradient buffers");
    return launch_gru_process_backward(pgr, pgai, pgar, pr, pai, par, nt, ndat, nrec, current_stream());
}

// ---- one recurrent time step per launch (additive) ----------------------------------------------------

int kai_lstm_step(int device, float* pr, float* ps, const float* ps_prev, float* pa, const float* pwr,
                  const float* pr_prev, const float* pbi, const float* pbr, int64_t ndat, int64_t nrec) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0 && nrec >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (ndat == 0 || nrec == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pr); KAI_REQUIRE_PTR(ps); KAI_REQUIRE_PTR(pa);
    if (pr_prev) KAI_REQUIRE_PTR(pwr);
    if (recurrent_step_applies(pwr, pr_prev, ndat, nrec))
        return launch_lstm_step(pr, ps, ps_prev, pa, pwr, pr_prev, pbi, pbr, ndat, nrec, current_stream());
    // the separate calls, in the engine's order (vtensor.cpp:2468-2483)
    if (pr_prev) KAI_TRY(kai_matmul(device, pa, pwr, pr_prev, 4 * nrec, ndat, nrec, 1));
    if (pbr) KAI_TRY(kai_add_bias(device, pa, pa, pbr, ndat, 4 * nrec));
    if (pbi) KAI_TRY(kai_add_bias(device, pa, pa, pbi, ndat, 4 * nrec));
    return kai_lstm_process(device, pr, ps, ps_prev, pa, ndat, nrec, 0);
}

int kai_gru_step(int device, float* pr, float* pai, float* par, const float* pwr, const float* pr_prev,
                 const float* ph_prev, const float* pbi, const float* pbr, int64_t ndat, int64_t nrec) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(ndat >= 0 && nrec >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (ndat == 0 || nrec == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pr); KAI_REQUIRE_PTR(pai); KAI_REQUIRE_PTR(par);
    KAI_REQUIRE(pai != par, KAI_ERR_INVALID_ARGUMENT, "the gru keeps input and recurrent sums in separate buffers");
    if (pr_prev) KAI_REQUIRE_PTR(pwr);
    if (recurrent_step_applies(pwr, pr_prev, ndat, nrec))
        return launch_gru_step(pr, pai, par, pwr, pr_prev, ph_prev, pbi, pbr, ndat, nrec, current_stream());
    if (pr_prev) KAI_TRY(kai_matmul(device, par, pwr, pr_prev, 3 * nrec, ndat, nrec, 0));
    else KAI_TRY(kai_set_zero(device, par, ndat * 3 * nrec * (int64_t)sizeof(float)));
    if (pbr) KAI_TRY(kai_add_bias(device, par, par, pbr, ndat, 3 * nrec));
    if (pbi) KAI_TRY(kai_add_bias(device, pai, pai, pbi, ndat, 3 * nrec));
    return launch_gru_process_from(pr, ph_prev, pai, par, ndat, nrec, current_stream());
}

// ---- transposes ----------------------------------------------------------------------------------

int kai_transpose(int device, float* py, const float* px, const int* pn, int64_t axis_size, int64_t data_size) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(data_size >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (data_size == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(px); KAI_REQUIRE_PTR(pn);
    return launch_transpose(py, px, pn, axis_size, data_size, false, current_stream());
}

int kai_transpose_backward(int device, float* pgx, const float* pgy, const int* pn, int64_t axis_size,
                           int64_t data_size) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(data_size >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (data_size == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgx); KAI_REQUIRE_PTR(pgy); KAI_REQUIRE_PTR(pn);
    return launch_transpose(pgx, pgy, pn, axis_size, data_size, true, current_stream());
}

int kai_transpose_bin(int device, float* py, const float* px, int64_t nrow, int64_t ncol) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0 && ncol >= 0, KAI_ERR_INVALID_ARGUMENT, "negative dimension");
    if (nrow == 0 || ncol == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(px);
    KAI_REQUIRE(py != px, KAI_ERR_INVALID_ARGUMENT, "transpose_bin cannot run in place");
    return launch_transpose_bin(py, px, nrow, ncol, current_stream());
}

// ---- parameter update: what consumes dW and db ---------------------------------------------------

int kai_accumulate_grad(int device, float* py, const float* px, int64_t nrow) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (nrow == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(px);
    return launch_accumulate_grad(py, px, nrow, current_stream());
}

int kai_subtract_param_grad(int device, float* pp, const float* pg, int64_t nrow, const float* hLearningRate) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (nrow == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pp); KAI_REQUIRE_PTR(pg);
    return launch_subtract_param_grad(pp, pg, nrow, hLearningRate, current_stream());
}

int kai_apply_decay(int device, float* pd, const float* pp, const float* pg, int64_t nrow, const float* hL1Decay,
                    const float* hL2Decay) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (nrow == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pd); KAI_REQUIRE_PTR(pp); KAI_REQUIRE_PTR(pg);
    return launch_apply_decay(pd, pp, pg, nrow, hL1Decay, hL2Decay, current_stream());
}

int kai_eval_adam_delta(int device, float* pa, const float* pg, float* ps, float* pt, float* pn, int64_t nrow,
                        const float* hRo1, const float* hRo2, const float* hEpsilon) {
    KAI_REQUIRE_DEVICE(device);
    KAI_REQUIRE(nrow >= 0, KAI_ERR_INVALID_ARGUMENT, "negative size");
    if (nrow == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pa); KAI_REQUIRE_PTR(pg); KAI_REQUIRE_PTR(ps); KAI_REQUIRE_PTR(pt); KAI_REQUIRE_PTR(pn);
    return launch_eval_adam_delta(pa, pg, ps, pt, pn, nrow, hRo1, hRo2, hEpsilon, current_stream());
}

int kai_attention_forward(int device, float* py, const float* pQ, const float* pK, const float* pV, int64_t nbat,
                          int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, const float* hCoef,
                          int masked) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0 || npiece == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(pQ); KAI_REQUIRE_PTR(pK); KAI_REQUIRE_PTR(pV);
    if (attention_fused_applies(pQ, pK, pV, py, ntimes, nvec, nhead, npiece))
        return launch_attention_fused(py, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef, masked != 0,
                                      current_stream());
    // any other shape: the separate kernels, probabilities in the library's scratch memory
    // (the products below may ask for scratch of their own, for partial sums of a reduction cut into parts:
    // while `held` lives, such requests are placed behind the probabilities)
    const int64_t pbytes = nbat * ntimes * ntimes * nhead * (int64_t)sizeof(float);
    float* pp = nullptr;
    KAI_TRY(workspace(pbytes, &pp));
    ScratchHold held(pbytes);
    KAI_TRY(kai_mult_on_heads(device, pp, pK, pQ, nbat, ntimes, nvec, nhead, npiece, hCoef));
    if (masked) KAI_TRY(kai_set_mh_attention_mask(device, pp, nbat, ntimes, nhead, 1));
    KAI_TRY(kai_softmax_direct_on_axis(device, pp, nbat * ntimes, ntimes, nhead));
    return kai_mix_values(device, py, pp, pV, nbat, ntimes, nvec, nhead, npiece);
}

int kai_gemm_force_plan(const char* text) { return set_forced_gemm_plan(text); }

int kai_attention_plan(int which, int64_t nbat, int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, char* out,
                       int buflen) {
    KAI_REQUIRE(out != nullptr && buflen > 0, KAI_ERR_INVALID_POINTER, "null output buffer");
    KAI_REQUIRE(which >= 0 && which <= 4, KAI_ERR_INVALID_ARGUMENT,
                "which must be 0 (forward), 1 (forward, training), 2 (backward), 3 (value gradient) or 4 (mix_values)");
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    // 16-byte aligned operands are assumed: a pointer value that satisfies every alignment test
    const float* a = reinterpret_cast<const float*>(uintptr_t(256));
    std::string text = "separate";
    if (nbat == 0 || ntimes == 0 || nhead == 0 || npiece == 0) text = "nothing";
    else if (which == 0 && attention_fused_applies(a, a, a, a, ntimes, nvec, nhead, npiece)) text = "fused";
    else if (which == 1 && attention_probs_applies(a, a, a, a, a, ntimes, nvec, nhead, npiece) &&
             attention_probs_pays(a, nbat, ntimes, nhead, npiece))
        text = attention_probs_four_heads(a, ntimes, nhead, npiece) ? "fused, four heads per workgroup" : "fused";
    else if (which == 2 && attention_backward_applies(a, a, a, a, a, a, a, a, ntimes, nvec, nhead, npiece))
        text = attention_backward_one_launch(a, a, a, nbat, ntimes, nvec, nhead, npiece) ? "fused rows and value gradient in one launch"
                                                                                        : "fused rows + value gradient";
    else if (which == 3) {
        const int hv = attention_value_grad_heads(a, a, a, ntimes, nvec, nhead, npiece);
        text = hv == 1 ? "streamed, one head per workgroup" : hv == 4 ? "streamed, four heads per workgroup" : "tiled";
    } else if (which == 4) {
        text = attention_heads_mix_applies(a, nhead * npiece, a, a, nvec, ntimes, nhead, npiece) ? "streamed, four heads per workgroup"
                                                                                               : "tiled";
    }
    snprintf(out, (size_t)buflen, "%s", text.c_str());
    return KAI_OK;
}

int kai_attention_forward_train(int device, float* py, float* pp, const float* pQ, const float* pK, const float* pV,
                                int64_t nbat, int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece,
                                const float* hCoef, int masked) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0) return KAI_OK;
    KAI_REQUIRE_PTR(py); KAI_REQUIRE_PTR(pp); KAI_REQUIRE_PTR(pQ); KAI_REQUIRE_PTR(pK); KAI_REQUIRE_PTR(pV);
    if (npiece > 0 && attention_probs_applies(pQ, pK, pV, py, pp, ntimes, nvec, nhead, npiece) &&
        attention_probs_pays(pp, nbat, ntimes, nhead, npiece))
        return launch_attention_probs(py, pp, pQ, pK, pV, nbat, ntimes, nvec, nhead, npiece, hCoef, masked != 0,
                                      current_stream());
    // any other shape: the reference's calls one by one
    KAI_TRY(kai_mult_on_heads(device, pp, pK, pQ, nbat, ntimes, nvec, nhead, npiece, hCoef));
    if (masked) KAI_TRY(kai_set_mh_attention_mask(device, pp, nbat, ntimes, nhead, 1));
    KAI_TRY(kai_softmax_direct_on_axis(device, pp, nbat * ntimes, ntimes, nhead));
    return kai_mix_values(device, py, pp, pV, nbat, ntimes, nvec, nhead, npiece);
}

int kai_attention_backward(int device, float* pgQ, float* pgK, float* pgV, const float* pgm, const float* pp,
                           const float* pm, const float* pQ, const float* pK, const float* pV, int64_t nbat,
                           int64_t ntimes, int64_t nvec, int64_t nhead, int64_t npiece, const float* hCoef,
                           int masked) {
    KAI_REQUIRE_DEVICE(device);
    KAI_TRY(check_heads(__func__, nbat, ntimes, nvec, nhead, npiece));
    if (nbat == 0 || ntimes == 0 || nhead == 0 || npiece == 0) return KAI_OK;
    KAI_REQUIRE_PTR(pgQ); KAI_REQUIRE_PTR(pgK); KAI_REQUIRE_PTR(pgV); KAI_REQUIRE_PTR(pgm); KAI_REQUIRE_PTR(pp);
    KAI_REQUIRE_PTR(pQ); KAI_REQUIRE_PTR(pK); KAI_REQUIRE_PTR(pV);
    // The value gradient is a reduction over the rows, workgroups of its own: behind the rows workgroups in the
    // same launch where its streaming kernel takes the geometry, else a launch of its own.
    if (attention_backward_applies(pgQ, pgK, pgm, pm, pp, pQ, pK, pV, ntimes, nvec, nhead, npiece)) {
        const bool one = attention_backward_one_launch(pgV, pgm, pp, nbat, ntimes, nvec, nhead, npiece);
        if (!one) KAI_TRY(kai_mix_values_backward_value(device, pgV, pgm, pp, nbat, ntimes, nvec, nhead, npiece));
        return launch_attention_backward_rows(pgQ, pgK, one ? pgV : nullptr, pgm, pm, pp, pQ, pK, pV, nbat, ntimes, nvec,
                                              nhead, npiece, hCoef, masked != 0, current_stream());
    }
    KAI_TRY(kai_mix_values_backward_value(device, pgV, pgm, pp, nbat, ntimes, nvec, nhead, npiece));
    // any other shape: the reference's calls one by one, the gradient of the probabilities in the library's scratch
    const int64_t pbytes = nbat * ntimes * ntimes * nhead * (int64_t)sizeof(float);
    float* pgp = nullptr;
    KAI_TRY(workspace(pbytes, &pgp));
    ScratchHold held(pbytes);
    KAI_TRY(kai_mix_values_backward_prop(device, pgp, pgm, pV, nbat, ntimes, nvec, nhead, npiece));
    KAI_TRY(kai_softmax_direct_on_axis_backward(device, pgp, pp, nbat, ntimes, nhead, hCoef));
    if (masked) KAI_TRY(kai_set_mh_attention_mask(device, pgp, nbat, ntimes, nhead, 0));
    KAI_TRY(kai_mult_on_heads_backward(device, pgK, pgp, pQ, nbat, ntimes, nvec, nhead, npiece));
    return kai_mult_on_heads_backward(device, pgQ, pgp, pK, nbat, ntimes, nvec, nhead, npiece);
}

}  // extern "C"
