// Fused softmax + cross-entropy + dlogits over (B*T, P) logits, in place.
// Reference: llmc/fused_classifier.cuh:139 (kernel :68), CPU definition train_gpt2.c:449-521.
//
// The largest HBM consumer of the step (6.1 GiB of bf16 logits at B=64,T=1024). One workgroup of
// 1024 lanes owns one row and keeps the whole row in registers (7 x 16-byte vectors per lane
// for P=50304 in bf16), so the row is read from HBM once and written once; max and sum are
// workgroup reductions. Rows are visited last-to-first, the order in which the LM-head GEMM's
// output is most likely still in cache (same trick as the reference, fused_classifier.cuh:76).
#include "common.hpp"
#include "../../include/llmk.h"

namespace {
constexpr int VN = vecX::N;
constexpr int CLS_BLOCK = 1024;

#if defined(LLMK_FP32)
__device__ __forceinline__ float cls_exp(float x) { return expf(x); }
#else
__device__ __forceinline__ float cls_exp(float x) { return __expf(x); }
#endif

// NVT: 16-byte vectors held per lane; requires P/VN <= NVT*CLS_BLOCK.
template <int NVT, bool WRITE>
__global__ void __launch_bounds__(CLS_BLOCK)
fused_classifier_kernel(floatX* __restrict__ logits, float* __restrict__ losses, float dloss,
                        const int* __restrict__ targets, int V, int P) {
    __shared__ float red[2][16];
    const int64_t row = (int64_t)gridDim.x - 1 - blockIdx.x;
    floatX* x = logits + row * (int64_t)P;
    const int nvec = P / VN;               // vectors that hold at least one of the V real columns:
    const int nvalid = CEIL_DIV(V, VN);    // [0, nvalid); the rest is padding and is never touched
    const int tid = threadIdx.x;
    const int target = targets[row];

    vecX r[NVT];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NVT; i++) {
        int v = tid + i * CLS_BLOCK;
        if (v < nvalid) {
            r[i] = ld_vec(x + (size_t)v * VN);
#pragma unroll
            for (int k = 0; k < VN; k++)
                if (v * VN + k < V) mx = fmaxf(mx, to_f32(r[i][k]));
        }
    }
    (void)nvec;
    mx = block_reduce<true>(mx, red[0]);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NVT; i++) {
        int v = tid + i * CLS_BLOCK;
        if (v < nvalid) {
#pragma unroll
            for (int k = 0; k < VN; k++)
                if (v * VN + k < V) sum += cls_exp(to_f32(r[i][k]) - mx);
        }
    }
    sum = block_reduce<false>(sum, red[1]);
    const float inv = 1.0f / sum;

#pragma unroll
    for (int i = 0; i < NVT; i++) {
        int v = tid + i * CLS_BLOCK;
        if (v < nvalid) {
            bool has_target = (target / VN) == v;
            if (has_target) {
                // -log softmax[target] = (max - logit) + log(sum); accumulates like the reference (:81).
                // Compare-select instead of r[i][target % VN]: a run-time index would push the row out of registers.
                float lt = 0.f;
#pragma unroll
                for (int k = 0; k < VN; k++)
                    if (k == target % VN) lt = to_f32(r[i][k]);
                losses[row] += (mx - lt) + logf(sum);
            }
            if (WRITE) {
#pragma unroll
                for (int k = 0; k < VN; k++) {
                    int e = v * VN + k;
                    if (e < V) {
                        float p = cls_exp(to_f32(r[i][k]) - mx) * inv;
                        r[i][k] = from_f32<floatX>((p - (e == target ? 1.0f : 0.0f)) * dloss);
                    }
                }
                st_vec_nt(x + (size_t)v * VN, r[i]);
            }
        }
    }
}

// rows too long for registers: three passes over global memory (the row stays in L2)
template <bool WRITE>
__global__ void __launch_bounds__(CLS_BLOCK)
fused_classifier_generic_kernel(floatX* __restrict__ logits, float* __restrict__ losses, float dloss,
                                const int* __restrict__ targets, int V, int P) {
    __shared__ float red[2][16];
    const int64_t row = (int64_t)gridDim.x - 1 - blockIdx.x;
    floatX* x = logits + row * (int64_t)P;
    const int target = targets[row];
    float mx = -INFINITY;
    for (int e = threadIdx.x; e < V; e += CLS_BLOCK) mx = fmaxf(mx, to_f32(x[e]));
    mx = block_reduce<true>(mx, red[0]);
    float sum = 0.f;
    for (int e = threadIdx.x; e < V; e += CLS_BLOCK) sum += cls_exp(to_f32(x[e]) - mx);
    sum = block_reduce<false>(sum, red[1]);
    const float inv = 1.0f / sum;
    float lt = to_f32(x[target]);
    __syncthreads();   // every lane has read the target logit before anyone overwrites it
    if (threadIdx.x == 0) losses[row] += (mx - lt) + logf(sum);
    if (WRITE) {
        for (int e = threadIdx.x; e < V; e += CLS_BLOCK) {
            float p = cls_exp(to_f32(x[e]) - mx) * inv;
            x[e] = from_f32<floatX>((p - (e == target ? 1.0f : 0.0f)) * dloss);
        }
    }
}
}  // namespace

extern "C" void llmk_fused_classifier(void* logits, float* losses, float dloss, const int* targets, int B, int T,
                                      int V, int P, int write_dlogits, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(V > 0 && V <= P, "fused_classifier: need 0 < V=%d <= P=%d", V, P);
    const int N = B * T;
    if (N == 0) return;
    hipStream_t st = (hipStream_t)stream;
    floatX* lg = (floatX*)logits;
    const bool vec_ok = (P % VN == 0) && ((uintptr_t)logits % 16 == 0);
    const int nvalid = CEIL_DIV(V, VN);
    llmk::ProfScope prof("fused_classifier", 0, (write_dlogits ? 2.0 : 1.0) * N * (double)P * sizeof(floatX), st);
#define CLS_LAUNCH(NVT)                                                                                     \
    do {                                                                                                    \
        if (write_dlogits) fused_classifier_kernel<NVT, true><<<N, CLS_BLOCK, 0, st>>>(lg, losses, dloss, targets, V, P); \
        else fused_classifier_kernel<NVT, false><<<N, CLS_BLOCK, 0, st>>>(lg, losses, dloss, targets, V, P);            \
    } while (0)
    if (vec_ok && nvalid <= 2 * CLS_BLOCK) CLS_LAUNCH(2);
    else if (vec_ok && nvalid <= 4 * CLS_BLOCK) CLS_LAUNCH(4);
    else if (vec_ok && nvalid <= 7 * CLS_BLOCK) CLS_LAUNCH(7);
    else if (vec_ok && nvalid <= 13 * CLS_BLOCK) CLS_LAUNCH(13);
    else {
        if (write_dlogits) fused_classifier_generic_kernel<true><<<N, CLS_BLOCK, 0, st>>>(lg, losses, dloss, targets, V, P);
        else fused_classifier_generic_kernel<false><<<N, CLS_BLOCK, 0, st>>>(lg, losses, dloss, targets, V, P);
    }
#undef CLS_LAUNCH
    LAUNCH_CHECK();
}
