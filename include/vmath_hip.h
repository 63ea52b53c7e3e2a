/*
 * vmath_hip.h -- C++ mirror of the engine's operator interface for the matmul path:
 * a class VMath whose static methods have the names, argument order and argument meaning of
 * the reference's (source/engine/support/vmath.h:18-56, 65-66, 137-143, 234-241) and forward
 * to the C-ABI of libkai_hip.so (kai_hip.h).  Engine code written against the reference's VMath
 * (the CALL_MATH sites of api_objects/vtensor.cpp and the replay switch of
 * local_objects/vexectracer.cpp:586-1190) compiles against this header unchanged.
 *
 * Error behaviour: the reference throws VException from VMath::cudaCheck
 * (VP_THROW1(VERR_CUDA_ERROR, "cuda:"+msg), vmath.cu:64-87) and VERR_CONDITIONAL_STATEMENT for an
 * unknown activation code (vmath.cu:3159-3161).  Here a non-zero C-ABI status is thrown as
 * KaiMathError carrying the same numeric code and the library's message.
 *
 * device < 0 selects the engine's own host loops in the reference; they are not part of this
 * GPU library, so compute methods throw KaiMathError(510) for device < 0.  The memory helpers
 * keep their host behaviour (malloc / memcpy) because VTensorData uses them for host tensors.
 */
#ifndef VMATH_HIP_H
#define VMATH_HIP_H

#include <stdint.h>

#include <stdexcept>
#include <string>

typedef int64_t int64;
typedef float* HYPER;   /* source/engine/local_objects/vhypermanager.h:6 */

class KaiMathError : public std::runtime_error {
public:
    KaiMathError(int code, const std::string& msg) : std::runtime_error(msg), m_code(code) {}
    int code() const { return m_code; }

private:
    int m_code;
};

class VMath {
public:
    static void* mem_alloc(int device, int64 size);
    static void mem_free(int device, void* ptr);

    static void memcpy_host_to_host(void* dptr, void* sptr, int64 size);
    static void memcpy_host_to_device(void* dptr, void* sptr, int64 size);
    static void memcpy_device_to_host(void* dptr, void* sptr, int64 size);
    static void memcpy_device_to_device(void* dptr, void* sptr, int64 size);

    static void copy_data(int dest_device, int src_device, void* py, void* px, int64 nbytes);

    static void fill_int(int device, int* ptr, int64 size, int value);
    static void fill_float(int device, float* ptr, int64 size, float value);
    static void set_zero(int device, void* ptr, int64 size);

    static void memcpy_from_host(int device, void* py, void* px, int64 size);
    static void memcpy_to_host(int device, void* py, void* px, int64 size);
    static void memcpy_to_device(int device, void* py, void* px, int64 size);

    static void get_slice(int device, void* py, void* px, int64 nbytes);

    static void add_bias(int device, float* py, float* pa, float* pb, int64 nrow, int64 ncol);
    static void add_bias_backward_b(int device, float* pgb, float* pgy, int64 nrow, int64 ncol, bool acc);

    static void matmul(int device, float* py, float* pw, float* px, int64 yvec, int64 ndat, int64 xvec, bool acc);
    static void matmul_backward_x(int device, float* pgx, float* pgy, float* pw, int64 yvec, int64 ndat, int64 xvec, bool acc);
    static void matmul_backward_w(int device, float* pgw, float* pgy, float* px, int64 yvec, int64 ndat, int64 xvec, bool acc);

    static void activate(int device, float* py, float* px, int64 nrow, int64 ncol, int actFunc, HYPER hLeakyAlpha);
    static void activate_backward(int device, float* pgx, float* pgy, float* px, int64 nrow, int64 ncol, int actFunc, HYPER hLeakyAlpha);
    static void activate_backward_with_y(int device, float* pgx, float* pgy, float* py, int64 nrow, int64 ncol, int actFunc, HYPER hLeakyAlpha);

    static void mult_on_heads(int device, float* pp, float* pK, float* pQ, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef);
    static void mult_on_heads_backward(int device, float* pgQKV, float* pgp, float* pQKV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece);
    static void set_mh_attention_mask(int device, float* pp, int64 ndat, int64 ntimes, int64 nhead, bool forward);
    static void softmax_direct_on_axis(int device, float* pp, int64 nrow, int64 nvec, int64 ncol);
    static void softmax_direct_on_axis_backward(int device, float* pgp, float* pp, int64 nbat, int64 ntimes, int64 nhead, HYPER hCoef);
    static void mix_values(int device, float* py, float* pp, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece);
    static void mix_values_backward_prop(int device, float* pgp, float* pgy, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece);
    static void mix_values_backward_value(int device, float* pV, float* pgy, float* pp, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece);

    /* additive: the `dense` layer formula activate(add(matmul(x,w),b)) (api/vconst.cpp:11) in one launch */
    static void cosinesim(int device, float* py, float* px1, float* px2, int64 nrow1, int64 nrow2, int64 ncol);
    static void copy(int device, float* py, float* pa, int64 ndat);
    static void add(int device, float* py, float* pa, float* pb, int64 ndat);
    static void lstm_process(int device, float* pr, float* ps, float* ps1, float* pa, int64 ndat, int64 nrec, int64 ninp);
    static void lstm_process_backward(int device, float* pgr, float* pgs, float* pga, float* ps, float* pa, int64 ndat,
                                      int64 nrec, int64 ninp);
    static void gru_process(int device, float* pr, float* pai, float* par, int64 nt, int64 ntimes, int64 ndat, int64 nrec);
    static void gru_process_backward(int device, float* pgr, float* pgai, float* pgar, float* pr, float* pai, float* par,
                                     int64 nt, int64 ntimes, int64 ndat, int64 nrec);
    // additive: one recurrent time step per launch (see kai_lstm_step / kai_gru_step)
    static void lstm_step(int device, float* pr, float* ps, float* ps_prev, float* pa, float* pwr, float* pr_prev,
                          float* pbi, float* pbr, int64 ndat, int64 nrec);
    static void gru_step(int device, float* pr, float* pai, float* par, float* pwr, float* pr_prev, float* ph_prev,
                         float* pbi, float* pbr, int64 ndat, int64 nrec);
    static void transpose(int device, float* py, float* px, int* pn, int64 axis_size, int64 data_size);
    static void transpose_backward(int device, float* pgx, float* pgy, int* pn, int64 axis_size, int64 data_size);
    static void transpose_bin(int device, float* py, float* px, int64 nrow, int64 ncol);
    static void accumulate_grad(int device, float* py, float* px, int64 nrow);
    static void subtract_param_grad(int device, float* pp, float* pg, int64 nrow, HYPER hLearningRate);
    static void apply_decay(int device, float* pd, float* pp, float* pg, int64 nrow, HYPER hL1Decay, HYPER hL2Decay);
    static void eval_adam_delta(int device, float* pa, float* pg, float* ps, float* pt, float* pn, int64 nrow, HYPER hRo1, HYPER hRo2, HYPER hEpsilon);
    static void attention_forward(int device, float* py, float* pQ, float* pK, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef, bool masked);
    static void attention_forward_train(int device, float* py, float* pp, float* pQ, float* pK, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef, bool masked);
    static void attention_backward(int device, float* pgQ, float* pgK, float* pgV, float* pgm, float* pp, float* pm, float* pQ, float* pK, float* pV, int64 nbat, int64 ntimes, int64 nvec, int64 nhead, int64 npiece, HYPER hCoef, bool masked);
    static void dense_forward(int device, float* py, float* ppre, float* pw, float* pb, float* px, int64 yvec, int64 ndat, int64 xvec, int actFunc, HYPER hLeakyAlpha);
    static void dense_backward(int device, float* pgx, float* pgw, float* pgb, float* pga_work, float* pgy, float* pw, float* px, float* ppre, int64 yvec, int64 ndat, int64 xvec, int actFunc, HYPER hLeakyAlpha, bool acc);
};

#endif
