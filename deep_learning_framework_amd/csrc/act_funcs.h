// Element-wise activation functions of the engine (enum class ActFunc,
// source/engine/include/vtypes.h:37-39 of the reference) as device functions, shared by the
// stand-alone activate kernels and by the GEMM epilogue.  Formulas follow
// VMath::activate / activate_backward / activate_backward_with_y
// (source/engine/support/vmath.cu:3097-3167, 3247-3308, 3411-3444), in fp32 with
// the same operation order.
#pragma once

#include <hip/hip_runtime.h>

namespace kai {

enum : int {
    kActNone = 0, kActRelu = 1, kActLeaky = 2, kActSigmoid = 3, kActTanh = 4,
    kActGelu = 5, kActSelu = 6, kActMish = 7, kActSwish = 8, kActSoftmax = 9
};

__device__ __forceinline__ float act_sigmoid(float x) {
    // vmath.cu:301-303
    return (x > 0) ? (1.0f / (1.0f + expf(-x))) : (expf(x) / (expf(x) + 1.0f));
}

__device__ __forceinline__ float act_tanh(float x) {
    // vmath.cu:309-311
    return 2 * act_sigmoid(2 * x) - 1;
}

// tanh of a value t expressed through exp, as the mish formulas write it
__device__ __forceinline__ float act_tanh_by_exp(float t) {
    return (t > 0) ? ((1.0f - expf(-t)) / (1.0f + expf(-t))) : ((expf(t) - 1.0f) / (expf(t) + 1.0f));
}

// y = f(x) for the element-wise codes 0..8 (softmax is a row operation and has its own kernel)
__device__ __forceinline__ float apply_act(float x, int act, float leaky_alpha) {
    switch (act) {
    case kActNone:
        return x;
    case kActRelu:
        return (x > 0) ? x : 0.0f;
    case kActLeaky:
        return (x > 0) ? x : x * leaky_alpha;
    case kActSigmoid:
        return act_sigmoid(x);
    case kActTanh:
        return act_tanh(x);
    case kActGelu:
        return x * 0.5f * (1.0f + erff(x / sqrtf(2.0f)));
    case kActSelu: {
        const float lambda = 1.0507009f;
        const float alpha = 1.6732632f;
        return (x > 0) ? lambda * x : lambda * alpha * (expf(x) - 1);
    }
    case kActMish: {
        const float t = logf(1.0f + expf(x)) * 2;
        return x * act_tanh_by_exp(t);
    }
    case kActSwish:
        return x * act_sigmoid(x);
    default:
        return x;
    }
}

// d f(x) / dx from the pre-activation x, codes 0..8
__device__ __forceinline__ float act_derivative(float x, int act, float leaky_alpha) {
    switch (act) {
    case kActNone:
        return 1.0f;
    case kActRelu:
        return (x > 0) ? 1.0f : 0.0f;
    case kActLeaky:
        return (x > 0) ? 1.0f : leaky_alpha;
    case kActSigmoid: {
        const float y = act_sigmoid(x);
        return y * (1.0f - y);
    }
    case kActTanh: {
        const float y = act_tanh(x);
        return 1.0f - y * y;
    }
    case kActGelu: {
        const float s = 0.5f * (1.0f + erff(x / sqrtf(2.0f)));
        const float t = 0.5f * x * sqrtf(2.0f / 3.14159265358979323846f) * expf(-x * x / 2.0f);
        return s + t;
    }
    case kActSelu: {
        const float lambda = 1.0507009f;
        const float alpha = 1.6732632f;
        return (x > 0) ? lambda : lambda * alpha * expf(x);
    }
    case kActMish: {
        float s = logf(1.0f + expf(x));
        const float t = (x > 0) ? (1.0f / (1.0f + expf(-x))) : (expf(x) / (1.0f + expf(x)));
        s = s * 2.0f;
        const float u = act_tanh_by_exp(s);
        const float v = 1.0f - u * u;
        return u + x * v * t;
    }
    case kActSwish: {
        const float s = act_sigmoid(x);
        const float t = s * (1.0f - s);
        return s + x * t;
    }
    default:
        return 1.0f;
    }
}

// d f / dx from the OUTPUT y, codes 0..4
__device__ __forceinline__ float act_derivative_from_y(float y, int act, float leaky_alpha) {
    switch (act) {
    case kActNone:
        return 1.0f;
    case kActRelu:
        return (y > 0) ? 1.0f : 0.0f;
    case kActLeaky:
        return (y > 0) ? 1.0f : leaky_alpha;
    case kActSigmoid:
        return y * (1 - y);
    case kActTanh:
        return 1 - y * y;
    default:
        return 1.0f;
    }
}

}  // namespace kai
