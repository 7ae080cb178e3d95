// tanh-GELU and its derivative as device functions, shared by the standalone kernels and the
// GEMM epilogues. Same formulas as train_gpt2.c:407-433 / llmc/gelu.cuh:13-47.
#pragma once
#include "common.hpp"

#if defined(LLMK_FP32)
// fp32 build: library tanhf, to stay within 1e-5 of the CPU oracle
__device__ __forceinline__ float llmk_tanh(float u) { return tanhf(u); }
#else
// bf16 build: tanh(u) = 1 - 2/(exp(2u)+1) on the hardware exp2 and reciprocal (1 ulp each); the error is
// far below bf16 resolution and the two transcendental ops are all the epilogues of the GEMMs can afford
__device__ __forceinline__ float llmk_tanh(float u) {
    float e = __builtin_amdgcn_exp2f(u * 2.8853900817779268f);   // exp(2u) = 2^(2u*log2(e))
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}
#endif

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
