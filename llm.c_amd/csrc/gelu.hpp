// tanh-GELU and its derivative as device functions, shared by the standalone kernels and the
// GEMM epilogues. Same formulas as train_gpt2.c:407-433 / llmc/gelu.cuh:13-47.
#pragma once
#include "common.hpp"

#if defined(LLMK_FP32)
// fp32 build: library tanhf, to stay within 1e-5 of the CPU oracle
__device__ __forceinline__ float llmk_tanh(float u) { return tanhf(u); }

__device__ __forceinline__ float gelu_f(float x) {
    const float k = 0.7978845608028654f;  // sqrt(2/pi)
    float u = k * (x + 0.044715f * x * x * x);
    return 0.5f * x * (1.0f + llmk_tanh(u));
}
// d/dx gelu(x), with sech^2 = 1 - tanh^2 (the reference's 1/cosh^2 overflows to 0 the same way)
__device__ __forceinline__ float gelu_grad_f(float x) {
    const float k = 0.7978845608028654f;
    float u = k * (x + 0.044715f * x * x * x);
    float th = llmk_tanh(u);
    float sech2 = 1.0f - th * th;
    return 0.5f * (1.0f + th) + x * 0.5f * sech2 * k * (1.0f + 3.0f * 0.044715f * x * x);
}
#else
// bf16 build. With u = sqrt(2/pi) (x + 0.044715 x^3), 0.5 (1 + tanh u) is the logistic function s = 1 / (1 + exp(-2u)),
// so gelu(x) = x s and gelu'(x) = s + x s (1 - s) 2u'. That is one hardware exp2 and one reciprocal (1 ulp each, far
// below bf16 resolution) plus five / eleven full-rate operations per element, which matters in the GEMM epilogue,
// where the matrix cores wait for them. Saturation is exact: exp2 -> inf gives s = 0, exp2 -> 0 gives s = 1.
__device__ __forceinline__ float gelu_sigmoid(float x, float x2) {
    const float a0 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;    // -2 sqrt(2/pi) log2(e)
    const float a1 = a0 * 0.044715f;
    const float e = __builtin_amdgcn_exp2f(x * fmaf(x2, a1, a0));           // exp(-2u)
    return __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float gelu_f(float x) { return x * gelu_sigmoid(x, x * x); }
__device__ __forceinline__ float gelu_grad_f(float x) {
    const float k2 = 2.0f * 0.7978845608028654f;
    const float x2 = x * x;
    const float s = gelu_sigmoid(x, x2);
    const float du2 = fmaf(x2, k2 * 3.0f * 0.044715f, k2);                  // 2 u'
    return fmaf(x * s, (1.0f - s) * du2, s);
}
#endif
// gelu(x) and gelu'(x) together, each the same bits as the function of its own: for a forward pass that leaves the
// derivative behind for the backward pass (gelu_fusion 3) instead of the pre-activation.
#if defined(LLMK_FP32)
__device__ __forceinline__ float gelu_with_grad_f(float x, float& grad) { grad = gelu_grad_f(x); return gelu_f(x); }
#else
__device__ __forceinline__ float gelu_with_grad_f(float x, float& grad) {
    const float k2 = 2.0f * 0.7978845608028654f;
    const float x2 = x * x;
    const float s = gelu_sigmoid(x, x2);                                    // shared: the one exp2 and the one reciprocal
    const float xs = x * s;
    const float du2 = fmaf(x2, k2 * 3.0f * 0.044715f, k2);
    grad = fmaf(xs, (1.0f - s) * du2, s);
    return xs;
}
#endif
