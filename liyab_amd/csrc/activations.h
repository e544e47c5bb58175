// Activation functions of feed-forward parts, in 32-bit.
#pragma once

#include "common.h"

namespace liyab {

enum Epilogue : int {
    kEpiNone = 0,      // out = acc + bias
    kEpiGeluTanh = 1,  // out = gelu_tanh(acc + bias)
    kEpiGeluErf = 2,   // out = gelu_erf(acc + bias)
    kEpiResidual = 3,  // residual += acc + bias   (32-bit residual stream)
};

// 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))), the reference's gelu_tanh
// (src/core/transformer.cpp:123-130), float throughout.
__device__ __forceinline__ float gelu_tanh(float x) {
    constexpr float kSqrt2OverPi = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(kSqrt2OverPi * (x + 0.044715f * x * x * x)));
}

// The same function for the bfloat16 path, as x / (1 + exp(-2u)) with u the tanh's argument
// (0.5 (1 + tanh u) = 1 / (1 + exp(-2u))): one hardware exponential and one reciprocal, no
// cancellation at either end (exp overflows to infinity and the quotient to 0 for very negative x).
__device__ __forceinline__ float gelu_tanh_fast(float x) {
    constexpr float kMinus2Sqrt2OverPiLog2e = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
    const float t = __builtin_amdgcn_exp2f(kMinus2Sqrt2OverPiLog2e * (x + 0.044715f * x * x * x));
    return x * __builtin_amdgcn_rcpf(1.0f + t);
}

// 0.5 x (1 + erf(x / sqrt 2)); the reference evaluates it in double and
// rounds once (src/core/transformer.cpp:134-142): kept for the 32-bit path.
__device__ __forceinline__ float gelu_erf_exact(float x) {
    const double xd = x;
    return static_cast<float>(0.5 * xd * (1.0 + erf(xd * 0.70710678118654752440)));
}
__device__ __forceinline__ float gelu_erf_fast(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }

}  // namespace liyab
