// tanh-GELU forward and in-place backward (reference: llmc/gelu.cuh:50-66, train_gpt2.c:407-433).
// Pure streaming kernels: one 16-byte vector per lane, HBM-bound.
#include "common.hpp"
#include "gelu.hpp"
#include "../../include/llmk.h"

namespace {
constexpr int VN = vecX::N;

__global__ void __launch_bounds__(256)
gelu_forward_kernel(floatX* __restrict__ out, const floatX* __restrict__ inp, size_t nvec) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec) return;
    vecX x = ld_vec_nt(inp + i * VN), o;
#pragma unroll
    for (int k = 0; k < VN; k++) o[k] = from_f32<floatX>(gelu_f(to_f32(x[k])));
    st_vec(out + i * VN, o);
}

__global__ void __launch_bounds__(256)
gelu_backward_kernel(floatX* __restrict__ d_in_out, const floatX* __restrict__ inp, size_t nvec) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec) return;
    vecX x = ld_vec_nt(inp + i * VN), d = ld_vec(d_in_out + i * VN), o;
#pragma unroll
    for (int k = 0; k < VN; k++) o[k] = from_f32<floatX>(gelu_grad_f(to_f32(x[k])) * to_f32(d[k]));
    st_vec(d_in_out + i * VN, o);
}
// out = gelu(x), and x is replaced by gelu'(x): what the backward pass needs of it
__global__ void __launch_bounds__(256)
gelu_forward_keep_grad_kernel(floatX* __restrict__ out, floatX* __restrict__ inp_to_grad, size_t nvec) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec) return;
    vecX x = ld_vec_nt(inp_to_grad + i * VN), o, d;
#pragma unroll
    for (int k = 0; k < VN; k++) {
        float gr;
        o[k] = from_f32<floatX>(gelu_with_grad_f(to_f32(x[k]), gr));
        d[k] = from_f32<floatX>(gr);
    }
    st_vec(out + i * VN, o);
    st_vec(inp_to_grad + i * VN, d);
}
// d_in_out *= grad (the stored gelu'), rounded once
__global__ void __launch_bounds__(256)
gelu_backward_from_grad_kernel(floatX* __restrict__ d_in_out, const floatX* __restrict__ grad, size_t nvec) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec) return;
    vecX g = ld_vec_nt(grad + i * VN), d = ld_vec(d_in_out + i * VN), o;
#pragma unroll
    for (int k = 0; k < VN; k++) o[k] = from_f32<floatX>(to_f32(g[k]) * to_f32(d[k]));
    st_vec(d_in_out + i * VN, o);
}
}  // namespace

extern "C" {
void llmk_gelu_forward(void* out, const void* inp, int N, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(N % VN == 0, "gelu_forward: N=%d must be a multiple of %d", N, VN);
    if (N == 0) return;
    size_t nvec = (size_t)N / VN;
    llmk::ProfScope prof("gelu_forward", 0, 2.0 * N * sizeof(floatX), (hipStream_t)stream);
    gelu_forward_kernel<<<(unsigned)CEIL_DIV(nvec, (size_t)256), 256, 0, (hipStream_t)stream>>>((floatX*)out, (const floatX*)inp, nvec);
    LAUNCH_CHECK();
}
void llmk_gelu_backward_inplace(void* d_in_out, const void* inp, int N, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(N % VN == 0, "gelu_backward_inplace: N=%d must be a multiple of %d", N, VN);
    if (N == 0) return;
    size_t nvec = (size_t)N / VN;
    llmk::ProfScope prof("gelu_backward_inplace", 0, 3.0 * N * sizeof(floatX), (hipStream_t)stream);
    gelu_backward_kernel<<<(unsigned)CEIL_DIV(nvec, (size_t)256), 256, 0, (hipStream_t)stream>>>((floatX*)d_in_out, (const floatX*)inp, nvec);
    LAUNCH_CHECK();
}
void llmk_gelu_forward_keep_grad(void* out, void* inp_to_grad, int N, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(N % VN == 0, "gelu_forward_keep_grad: N=%d must be a multiple of %d", N, VN);
    if (N == 0) return;
    size_t nvec = (size_t)N / VN;
    llmk::ProfScope prof("gelu_forward_keep_grad", 0, 3.0 * N * sizeof(floatX), (hipStream_t)stream);
    gelu_forward_keep_grad_kernel<<<(unsigned)CEIL_DIV(nvec, (size_t)256), 256, 0, (hipStream_t)stream>>>((floatX*)out, (floatX*)inp_to_grad, nvec);
    LAUNCH_CHECK();
}
void llmk_gelu_backward_from_grad(void* d_in_out, const void* grad, int N, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(N % VN == 0, "gelu_backward_from_grad: N=%d must be a multiple of %d", N, VN);
    if (N == 0) return;
    size_t nvec = (size_t)N / VN;
    llmk::ProfScope prof("gelu_backward_from_grad", 0, 3.0 * N * sizeof(floatX), (hipStream_t)stream);
    gelu_backward_from_grad_kernel<<<(unsigned)CEIL_DIV(nvec, (size_t)256), 256, 0, (hipStream_t)stream>>>((floatX*)d_in_out, (const floatX*)grad, nvec);
    LAUNCH_CHECK();
}
}
