// Test driver for the C++ mirror of the engine's operator interface (include/vmath_hip.h): engine-style
// code that calls VMath:: methods exactly as the reference's call sites do
// (CALL_MATH(matmul, device(), py, pw, px, yvec, ndat, xvec, false), api_objects/vtensor.cpp:1332,
//  CALL_MATH(mult_on_heads, ...), vtensor.cpp:3034) and catches the exception a failing call raises.
// Built with the host compiler against libkai_hip.so (tests/Makefile), started by tests/test_vmath_mirror.py.
//
//   vmath_mirror_driver cpu
//       the checks that need no GPU: error codes of refused calls, host-side memory helpers
//   vmath_mirror_driver gpu <dir> <ndat> <xvec> <yvec> <nbat> <ntimes> <nhead> <npiece>
//       reads x.bin w.bin b.bin q.bin k.bin (inputs) and y_ref.bin act_ref.bin p_ref.bin (expected results,
//       written by the Python side from the CPU oracle) in <dir>, runs the calls on GPU 0 and compares
//       (relative Frobenius error <= 1e-5).
// Exit status 0 = every check passed; each check prints one line.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "vmath_hip.h"

static int g_failed = 0;

static void report(bool ok, const std::string& what) {
    std::printf("%s %s\n", ok ? "ok  " : "FAIL", what.c_str());
    std::fflush(stdout);
    if (!ok) g_failed++;
}

// runs `call`, expects KaiMathError with `code` and a message
template <class F>
static void expect_error(int code, const std::string& what, F call) {
    try {
        call();
        report(false, what + ": no exception");
    } catch (const KaiMathError& e) {
        const bool ok = e.code() == code && std::strlen(e.what()) > 0;
        report(ok, what + ": KaiMathError " + std::to_string(e.code()) + " \"" + e.what() + "\"");
    } catch (...) {
        report(false, what + ": another exception type");
    }
}

static std::vector<float> read_floats(const std::string& path, size_t n) {
    std::vector<float> v(n);
    FILE* f = std::fopen(path.c_str(), "rb");
    if (!f || std::fread(v.data(), sizeof(float), n, f) != n) {
        std::fprintf(stderr, "cannot read %zu floats from %s\n", n, path.c_str());
        std::exit(2);
    }
    std::fclose(f);
    return v;
}

static double rel_fro(const std::vector<float>& got, const std::vector<float>& ref, double scale = 1.0) {
    double num = 0, den = 0;
    for (size_t i = 0; i < ref.size(); i++) {
        const double r = scale * ref[i], d = got[i] - r;
        num += d * d;
        den += r * r;
    }
    return den > 0 ? std::sqrt(num / den) : std::sqrt(num);
}

// a device tensor the way VTensorData holds one: VMath::mem_alloc in the constructor, mem_free in the destructor
struct DeviceTensor {
    float* ptr;
    int64 count;
    explicit DeviceTensor(int64 n) : ptr((float*)VMath::mem_alloc(0, n * (int64)sizeof(float))), count(n) {}
    explicit DeviceTensor(const std::vector<float>& host) : DeviceTensor((int64)host.size()) {
        VMath::memcpy_from_host(0, ptr, (void*)host.data(), count * (int64)sizeof(float));
    }
    ~DeviceTensor() { VMath::mem_free(0, ptr); }
    std::vector<float> to_host() const {
        std::vector<float> v((size_t)count);
        VMath::memcpy_to_host(0, v.data(), ptr, count * (int64)sizeof(float));
        return v;
    }
};

static void checks_without_gpu() {
    float* one = reinterpret_cast<float*>(16);   // non-null, never dereferenced on these paths
    // device < 0 is the engine's host loop, which the GPU library does not contain
    expect_error(510, "matmul on device -1", [&] { VMath::matmul(-1, one, one, one, 4, 4, 4, false); });
    expect_error(510, "mult_on_heads on device -1",
                 [&] { VMath::mult_on_heads(-1, one, one, one, 1, 4, 8, 2, 4, nullptr); });
    // unknown activation code: VERR_CONDITIONAL_STATEMENT, as the reference's switch throws (vmath.cu:3159-3161)
    expect_error(8, "activate with code 10", [&] { VMath::activate(0, one, one, 1, 1, 10, nullptr); });
    expect_error(8, "dense_forward with the softmax code",
                 [&] { VMath::dense_forward(0, one, nullptr, one, nullptr, one, 4, 4, 4, 9, nullptr); });
    expect_error(523, "matmul with a null output", [&] { VMath::matmul(0, nullptr, one, one, 4, 4, 4, false); });
    expect_error(510, "matmul with a negative size", [&] { VMath::matmul(0, one, one, one, -1, 4, 4, false); });
    // an empty product returns without touching anything
    try {
        VMath::matmul(0, one, one, one, 0, 4, 4, false);
        report(true, "empty matmul returns");
    } catch (...) {
        report(false, "empty matmul returns");
    }
    // host-side memory helpers (VTensorData uses them for host tensors)
    float* h = (float*)VMath::mem_alloc(-1, 64);
    float src[16], dst[16];
    for (int i = 0; i < 16; i++) src[i] = (float)i;
    VMath::memcpy_from_host(-1, h, src, 64);
    VMath::fill_float(-1, h, 4, 9.0f);
    VMath::copy_data(-1, -1, dst, h, 64);
    bool ok = true;
    for (int i = 0; i < 16; i++) ok = ok && dst[i] == (i < 4 ? 9.0f : (float)i);
    VMath::set_zero(-1, h, 64);
    VMath::memcpy_to_host(-1, dst, h, 64);
    for (int i = 0; i < 16; i++) ok = ok && dst[i] == 0.0f;
    VMath::mem_free(-1, h);
    report(ok, "host memory helpers");
}

static void checks_on_gpu(const std::string& dir, int64 ndat, int64 xvec, int64 yvec, int64 nbat, int64 ntimes,
                          int64 nhead, int64 npiece) {
    const double tol = 1e-5;
    const int64 nvec = nhead * npiece;
    const auto x = read_floats(dir + "/x.bin", ndat * xvec), w = read_floats(dir + "/w.bin", yvec * xvec);
    const auto b = read_floats(dir + "/b.bin", yvec);
    const auto y_ref = read_floats(dir + "/y_ref.bin", ndat * yvec), act_ref = read_floats(dir + "/act_ref.bin", ndat * yvec);
    const auto q = read_floats(dir + "/q.bin", nbat * ntimes * nvec), k = read_floats(dir + "/k.bin", nbat * ntimes * nvec);
    const auto p_ref = read_floats(dir + "/p_ref.bin", nbat * ntimes * ntimes * nhead);

    DeviceTensor dx(x), dw(w), db(b), dy(ndat * yvec);
    // the dense layer's three calls, as VTensor::matmul / add / activate issue them
    VMath::matmul(0, dy.ptr, dw.ptr, dx.ptr, yvec, ndat, xvec, false);
    double e = rel_fro(dy.to_host(), y_ref);
    report(e <= tol, "VMath::matmul vs oracle, rel error " + std::to_string(e));
    VMath::matmul(0, dy.ptr, dw.ptr, dx.ptr, yvec, ndat, xvec, true);
    e = rel_fro(dy.to_host(), y_ref, 2.0);
    report(e <= tol, "VMath::matmul with acc doubles the result, rel error " + std::to_string(e));
    VMath::matmul(0, dy.ptr, dw.ptr, dx.ptr, yvec, ndat, xvec, false);
    VMath::add_bias(0, dy.ptr, dy.ptr, db.ptr, ndat, yvec);
    VMath::activate(0, dy.ptr, dy.ptr, ndat, yvec, 1 /* ActFunc::relu */, nullptr);
    e = rel_fro(dy.to_host(), act_ref);
    report(e <= tol, "matmul + add_bias + activate(relu) vs oracle, rel error " + std::to_string(e));
    // the same layer in one launch
    DeviceTensor dy2(ndat * yvec);
    VMath::dense_forward(0, dy2.ptr, nullptr, dw.ptr, db.ptr, dx.ptr, yvec, ndat, xvec, 1, nullptr);
    e = rel_fro(dy2.to_host(), act_ref);
    report(e <= tol, "VMath::dense_forward vs oracle, rel error " + std::to_string(e));

    // attention scores; the coefficient is a device-resident hyper-parameter (HYPER = float*)
    DeviceTensor dq(q), dk(k), dp(nbat * ntimes * ntimes * nhead), dcoef(1);
    VMath::fill_float(0, dcoef.ptr, 1, 1.0f / std::sqrt((float)npiece));
    VMath::mult_on_heads(0, dp.ptr, dk.ptr, dq.ptr, nbat, ntimes, nvec, nhead, npiece, dcoef.ptr);
    e = rel_fro(dp.to_host(), p_ref);
    report(e <= tol, "VMath::mult_on_heads vs oracle, rel error " + std::to_string(e));

    // failing calls raise, and the library keeps working afterwards
    expect_error(8, "activate with code 11 on the GPU", [&] { VMath::activate(0, dy.ptr, dy.ptr, ndat, yvec, 11, nullptr); });
    expect_error(510, "mult_on_heads with nhead * npiece > nvec",
                 [&] { VMath::mult_on_heads(0, dp.ptr, dk.ptr, dq.ptr, nbat, ntimes, nvec, nhead + 1, npiece, dcoef.ptr); });
    expect_error(523, "matmul with a null weight", [&] { VMath::matmul(0, dy.ptr, nullptr, dx.ptr, yvec, ndat, xvec, false); });
    VMath::matmul(0, dy.ptr, dw.ptr, dx.ptr, yvec, ndat, xvec, false);
    e = rel_fro(dy.to_host(), y_ref);
    report(e <= tol, "matmul after the refused calls, rel error " + std::to_string(e));
}

int main(int argc, char** argv) {
    try {
        if (argc == 2 && std::string(argv[1]) == "cpu") {
            checks_without_gpu();
        } else if (argc == 10 && std::string(argv[1]) == "gpu") {
            int64 d[7];
            for (int i = 0; i < 7; i++) d[i] = std::atoll(argv[3 + i]);
            checks_on_gpu(argv[2], d[0], d[1], d[2], d[3], d[4], d[5], d[6]);
        } else {
            std::fprintf(stderr, "usage: %s cpu | gpu <dir> ndat xvec yvec nbat ntimes nhead npiece\n", argv[0]);
            return 2;
        }
    } catch (const KaiMathError& e) {
        std::printf("FAIL unexpected KaiMathError %d: %s\n", e.code(), e.what());
        return 1;
    }
    std::printf("%s\n", g_failed ? "FAILED" : "all checks passed");
    return g_failed ? 1 : 0;
}
