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

// exp(x - mx) as the two passes below evaluate it. bf16 build: one fma and one hardware exp2 with the 1/ln2
// folded into both operands (mxl = mx * log2(e)); fp32 build: the library expf of the difference.
#if defined(LLMK_FP32)
__device__ __forceinline__ float cls_exp_rel(float x, float mx, float) { return expf(x - mx); }
__device__ __forceinline__ float cls_scaled(float e, float inv, float dloss, float) { return e * inv * dloss; }
#else
__device__ __forceinline__ float cls_exp_rel(float x, float, float mxl) { return __builtin_amdgcn_exp2f(fmaf(x, 1.4426950408889634f, -mxl)); }
__device__ __forceinline__ float cls_scaled(float e, float, float, float inv_dloss) { return e * inv_dloss; }
#endif

// The row's vectors are addressed through a buffer descriptor: one per-lane byte offset (16 * lane) plus a scalar
// offset per vector slot. With plain pointers the compiler keeps one per-lane offset per slot alive from the loads to
// the stores; seven of them do not fit beside the row in 64 registers and went to scratch memory and back, a quarter
// more traffic than the logits themselves.
typedef int cls_i4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t cls_row_rsrc(floatX* row, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(row, 0, bytes, 0x00020000);   // raw buffer, 32-bit data format
}
__device__ __forceinline__ vecX cls_ld(__amdgpu_buffer_rsrc_t rs, int lane_bytes, int slot_bytes) {
    const cls_i4 q = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_bytes, slot_bytes, 0);
    vecX out;
    *reinterpret_cast<cls_i4*>(&out) = q;
    return out;
}
__device__ __forceinline__ void cls_st_nt(__amdgpu_buffer_rsrc_t rs, int lane_bytes, int slot_bytes, const vecX& w) {
    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const cls_i4*>(&w), rs, lane_bytes, slot_bytes, 2 /* nt */);
}

// NVT: 16-byte vectors held per lane of a BLK-lane workgroup; requires V/VN <= NVT*BLK. A CU holds 2048 lanes: two
// rows with 1024-lane workgroups, three with 512-lane ones when the row fits their registers (13 vectors, 70 registers,
// six waves per SIMD), which measured 4 % faster on GPT-2's vocabulary.
// The vectors whose VN columns are all real ([0, V/VN)) take loops without any per-element test; the one vector
// that straddles V (when V is not a multiple of VN) is held by a single lane and handled on the side, and the
// target column is patched in the one vector that holds it. Per element that leaves: max; fma, exp2, add; and
// fma, exp2, multiply, convert.
template <int NVT, bool WRITE, int BLK = CLS_BLOCK>
__global__ void __launch_bounds__(BLK, BLK == 512 ? 6 : NVT <= 7 ? 8 : 4)
fused_classifier_kernel(floatX* __restrict__ logits, float* __restrict__ losses, float dloss,
                        const int* __restrict__ targets, int V, int P) {
    __shared__ float red[2][16];
    const int64_t row = (int64_t)gridDim.x - 1 - blockIdx.x;
    floatX* x = logits + row * (int64_t)P;
    const int nfull = V / VN, rem = V - nfull * VN;     // padding columns [V, P) are never touched
    const int tid = threadIdx.x;
    const int target = targets[row];
    const int tvec = target / VN, tk = target - tvec * VN;
    const bool edge = rem != 0 && tid == nfull % BLK;   // this lane holds the straddling vector

    const __amdgpu_buffer_rsrc_t rs = cls_row_rsrc(x, P * (int)sizeof(floatX));
    const int lane_bytes = tid * 16;

    vecX r[NVT], re;
    float mx = -INFINITY;
    // The row stays in registers as loaded. Without this the compiler carries converted or unpacked columns from one
    // pass into the next, which takes more registers than there are and ends in scratch memory.
    auto keep_packed = [&]() {
#pragma unroll
        for (int i = 0; i < NVT; i++) {
            unsigned* w32 = reinterpret_cast<unsigned*>(&r[i]);
#pragma unroll
            for (int q = 0; q < 4; q++) asm volatile("" : "+v"(w32[q]));
        }
    };
#pragma unroll
    for (int i = 0; i < NVT; i++) {
        const int v = tid + i * BLK;
        if (v < nfull) {
            r[i] = cls_ld(rs, lane_bytes, i * BLK * 16);
            if (WRITE) {
#pragma unroll
                for (int k = 0; k < VN; k++) mx = fmaxf(mx, to_f32(r[i][k]));
            }
        }
    }
    if (!WRITE) {   // no store needs the vectors whole, so they are pinned as loaded before their first use too
        keep_packed();
#pragma unroll
        for (int i = 0; i < NVT; i++) {
            if (tid + i * BLK < nfull) {
#pragma unroll
                for (int k = 0; k < VN; k++) mx = fmaxf(mx, to_f32(r[i][k]));
            }
        }
    }
    if (edge) {
        re = ld_vec(x + (size_t)nfull * VN);
#pragma unroll
        for (int k = 0; k < VN; k++)
            if (k < rem) mx = fmaxf(mx, to_f32(re[k]));
    }
    mx = block_reduce<true>(mx, red[0]);
    const float mxl = mx * 1.4426950408889634f;
    keep_packed();
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NVT; i++) {
        const int v = tid + i * BLK;
        if (v < nfull) {
#pragma unroll
            for (int k = 0; k < VN; k++) sum += cls_exp_rel(to_f32(r[i][k]), mx, mxl);
        }
    }
    if (edge) {
#pragma unroll
        for (int k = 0; k < VN; k++)
            if (k < rem) sum += cls_exp_rel(to_f32(re[k]), mx, mxl);
    }
    sum = block_reduce<false>(sum, red[1]);
    const float inv = 1.0f / sum, inv_dloss = inv * dloss;
    keep_packed();

    // The vector `w` holds the target column: the loss term. The column is picked as a 32-bit word by compare-select
    // (a run-time index would push the row out of registers) and, in bf16, as one half of that word: converting all
    // columns here made the compiler carry the converted values into the exponent loop, through scratch memory.
    constexpr int PER_WORD = VN / 4;                       // 2 bf16 or 1 fp32 per 32-bit word
    const int tq = tk / PER_WORD, th = tk - tq * PER_WORD;
    auto target_logit = [&](const vecX& w) {
        const unsigned* w32 = reinterpret_cast<const unsigned*>(&w);
        unsigned word = 0;
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (q == tq) word = w32[q];
        const float lt = __uint_as_float(PER_WORD == 1 ? word : th ? word & 0xffff0000u : word << 16);
        // -log softmax[target] = (max - logit) + log(sum); accumulates like the reference (fused_classifier.cuh:81)
        losses[row] += (mx - lt) + logf(sum);
        return lt;
    };
    auto patch_target = [&](vecX& w, float lt) {          // ... and, after the vector's other columns, its gradient
        const float gf = (cls_exp_rel(lt, mx, mxl) * inv - 1.0f) * dloss;
        unsigned* w32 = reinterpret_cast<unsigned*>(&w);
        unsigned bits;
        if constexpr (PER_WORD == 1) {
            bits = __float_as_uint(gf);
        } else {
            const __bf16 g = from_f32<__bf16>(gf);
            bits = (unsigned)__builtin_bit_cast(unsigned short, g);
        }
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (q == tq) w32[q] = PER_WORD == 1 ? bits : th ? (w32[q] & 0x0000ffffu) | (bits << 16) : (w32[q] & 0xffff0000u) | bits;
    };
#pragma unroll
    for (int i = 0; i < NVT; i++) {
        const int v = tid + i * BLK;
        if (v < nfull) {
            float lt = 0.f;
            const bool has_target = tvec == v;
            if (has_target) lt = target_logit(r[i]);
            if (WRITE) {
#pragma unroll
                for (int k = 0; k < VN; k++)
                    r[i][k] = from_f32<floatX>(cls_scaled(cls_exp_rel(to_f32(r[i][k]), mx, mxl), inv, dloss, inv_dloss));
                if (has_target) patch_target(r[i], lt);
                cls_st_nt(rs, lane_bytes, i * BLK * 16, r[i]);
            }
        }
    }
    if (edge) {
        float lt = 0.f;
        const bool has_target = tvec == nfull;
        if (has_target) lt = target_logit(re);
        if (WRITE) {
#pragma unroll
            for (int k = 0; k < VN; k++)
                if (k < rem) re[k] = from_f32<floatX>(cls_scaled(cls_exp_rel(to_f32(re[k]), mx, mxl), inv, dloss, inv_dloss));
            if (has_target) patch_target(re, lt);
            st_vec_nt(x + (size_t)nfull * VN, re);       // its padding columns go back as they came
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
    const int nvalid = V / VN;                            // full vectors; the straddling one sits beside them
    llmk::ProfScope prof("fused_classifier", 0, (write_dlogits ? 2.0 : 1.0) * N * (double)P * sizeof(floatX), st);
#define CLS_LAUNCH(NVT, BLK)                                                                                \
    do {                                                                                                    \
        if (write_dlogits) fused_classifier_kernel<NVT, true, BLK><<<N, BLK, 0, st>>>(lg, losses, dloss, targets, V, P); \
        else fused_classifier_kernel<NVT, false, BLK><<<N, BLK, 0, st>>>(lg, losses, dloss, targets, V, P);            \
    } while (0)
    if (vec_ok && nvalid <= 2 * CLS_BLOCK) CLS_LAUNCH(2, CLS_BLOCK);
    else if (vec_ok && nvalid <= 4 * CLS_BLOCK) CLS_LAUNCH(4, CLS_BLOCK);
    else if (vec_ok && nvalid <= 13 * 512 && write_dlogits)       // GPT-2's vocabulary in bf16: three rows per CU at 70 registers
        fused_classifier_kernel<13, true, 512><<<N, 512, 0, st>>>(lg, losses, dloss, targets, V, P);
    else if (vec_ok && nvalid <= 7 * CLS_BLOCK) CLS_LAUNCH(7, CLS_BLOCK);
    else if (vec_ok && nvalid <= 13 * CLS_BLOCK) CLS_LAUNCH(13, CLS_BLOCK);
    else {
        if (write_dlogits) fused_classifier_generic_kernel<true><<<N, CLS_BLOCK, 0, st>>>(lg, losses, dloss, targets, V, P);
        else fused_classifier_generic_kernel<false><<<N, CLS_BLOCK, 0, st>>>(lg, losses, dloss, targets, V, P);
    }
#undef CLS_LAUNCH
    LAUNCH_CHECK();
}
