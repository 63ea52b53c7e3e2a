// Internal helpers shared by the host-side translation units of libkai_hip.so:
// error reporting (numeric codes of the reference, thread-local message), the
// calling thread's stream, and argument checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "../../include/kai_hip.h"

namespace kai {

// thread-local last error text; returns `code` so that callers can `return fail(...)`
int fail(int code, const std::string& msg);
void clear_error();
// stream of the calling thread (null stream unless kai_set_stream was called on this thread)
hipStream_t current_stream();

// turns a HIP status into KAI_ERR_GPU with the runtime's message
int check_hip(hipError_t st, const char* what);
// status of the launch that was just enqueued
int check_launch(const char* kernel_name);

// Library-owned scratch memory on the CURRENT device (partial sums of a reduction cut into parts, row norms,
// the probabilities of an attention call that runs as separate kernels), one buffer per stream that calls are
// enqueued on (the calling thread's stream, kai_set_stream): calls on different streams of a device never share
// it.  Allocated on first use and released by kai_shutdown.  When a call needs more than there is, a larger
// buffer is allocated and the old one is retired -- kept, so that growth never waits for the device and
// pointers handed out earlier (to kernels in flight, to recorded graphs) stay valid -- until the device is
// idle at one of the library's own synchronisation points (kai_device_synchronize, kai_shutdown); buffers
// handed out during a stream capture stay until kai_shutdown.  While a stream capture is active, growth is
// refused with an error.  Every call on a stream returns the front of that stream's buffer.
int workspace(int64_t bytes, float** out);
// While an object of this type lives, workspace() calls of the same thread return memory BEHIND the first
// `bytes` bytes of the scratch: for a call that keeps data in the scratch across inner calls which may ask
// for scratch themselves.
class ScratchHold {
public:
    explicit ScratchHold(int64_t bytes);
    ~ScratchHold();
    ScratchHold(const ScratchHold&) = delete;
    ScratchHold& operator=(const ScratchHold&) = delete;

private:
    int64_t previous_;
};
// number of compute units of the current device (cached)
int compute_units();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int64_t kMaxDim = (1ll << 31) - 1;

}  // namespace kai

#define KAI_REQUIRE(cond, code, msg)                                   \
    do {                                                               \
        if (!(cond)) return ::kai::fail((code), std::string(__func__) + ": " + (msg)); \
    } while (0)

#define KAI_REQUIRE_DEVICE(device) \
    KAI_REQUIRE((device) >= 0, KAI_ERR_INVALID_ARGUMENT, "device < 0 selects the engine's host loop, which this GPU library does not contain")

#define KAI_TRY(expr)               \
    do {                            \
        int kai_rc_ = (expr);       \
        if (kai_rc_ != KAI_OK) return kai_rc_; \
    } while (0)
