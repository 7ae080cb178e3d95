// Shared device/host utilities for the gfx950 kernels: storage type, 16-byte vectors,
// wave64 / workgroup reductions, counter-based noise for stochastic rounding, error handling.
// Plays the role of the reference's llmc/cuda_common.h + llmc/cuda_utils.cuh, written for
// 64-wide wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>
#include <hip/hip_bf16.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstddef>

// ------------------------------------------------------------------------------------------
// Storage precision of activations/params/grads: a build-time property of the library,
// like the reference's PRECISION=FP32|BF16 switch (reference Makefile:232-244,
// llmc/cuda_common.h:82-92). Accumulation is always fp32.
#if defined(LLMK_FP32)
typedef float floatX;
#define LLMK_PRECISION_NAME "fp32"
#else
typedef __bf16 floatX;
#define LLMK_PRECISION_NAME "bf16"
#endif

#define WAVE 64
#define CEIL_DIV(a, b) (((a) + (b) - 1) / (b))

// ------------------------------------------------------------------------------------------
// Errors. Default: print and exit, as the reference does (llmc/cuda_common.h:52-58).
// Tests switch to "record" mode and read the message back.
namespace llmk {
void fail(const char* file, int line, const char* fmt, ...) __attribute__((format(printf, 3, 4)));
bool failed();   // true once a failure was recorded in record mode (launchers then return early)
struct DeviceInfo {
    int device = -1;
    int num_cu = 0;
    int max_threads_per_cu = 0;
    size_t lds_per_block = 0;
    char name[256] = {0};
    bool ready = false;
};
const DeviceInfo& device_info();
// persistent library workspace (grown on demand, never per call once large enough)
void* workspace(size_t bytes);

// Optional per-kernel timing with HIP events on the launch stream (off by default). The reference
// marks the same spots with NVTX ranges and post-processes an ncu run (llmc/cuda_common.h:115-124,
// profile_gpt2cu.py); here the library can time its own launches and report time, algorithmic
// flops and algorithmic bytes per kernel family.
bool profiling(const char* name);
void prof_begin(const char* name, double flops, double bytes, hipStream_t st);
void prof_end(hipStream_t st);
struct ProfScope {
    hipStream_t st;
    bool on;
    ProfScope(const char* name, double flops, double bytes, hipStream_t s) : st(s), on(profiling(name)) {
        if (on) prof_begin(name, flops, bytes, st);
    }
    // never_time: for callers that must not create events (entry points that allocate nothing)
    ProfScope(bool never_time, const char* name, double flops, double bytes, hipStream_t s) : st(s), on(!never_time && profiling(name)) {
        if (on) prof_begin(name, flops, bytes, st);
    }
    ~ProfScope() { if (on) prof_end(st); }
};
}  // namespace llmk

#define HIP_CHECK(expr)                                                                       \
    do {                                                                                      \
        hipError_t err__ = (expr);                                                            \
        if (err__ != hipSuccess) {                                                            \
            llmk::fail(__FILE__, __LINE__, "[HIP ERROR] %s: %s", #expr, hipGetErrorString(err__)); \
        }                                                                                     \
    } while (0)

#define LLMK_REQUIRE(cond, ...)                                           \
    do {                                                                  \
        if (!(cond)) { llmk::fail(__FILE__, __LINE__, __VA_ARGS__); return; } \
    } while (0)

#define LAUNCH_CHECK() HIP_CHECK(hipGetLastError())

// ------------------------------------------------------------------------------------------
// conversions
__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(__bf16 x) { return (float)x; }
template <class T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ __bf16 from_f32<__bf16>(float x) { return (__bf16)x; }  // RNE

// ------------------------------------------------------------------------------------------
// 16-byte vector of T (8 bf16 or 4 fp32): the unit of every global load/store in the
// bandwidth-bound kernels, so each lane moves a full dwordx4.
template <class T>
struct alignas(16) Vec {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
    __device__ __forceinline__ T& operator[](int i) { return v[i]; }
    __device__ __forceinline__ const T& operator[](int i) const { return v[i]; }
};
typedef Vec<floatX> vecX;
typedef Vec<float> vecF;

template <class T>
__device__ __forceinline__ Vec<T> ld_vec(const T* p) {
    return *reinterpret_cast<const Vec<T>*>(p);
}
template <class T>
__device__ __forceinline__ void st_vec(T* p, const Vec<T>& v) {
    *reinterpret_cast<Vec<T>*>(p) = v;
}
// streaming variants: data that will not be read again soon
template <class T>
__device__ __forceinline__ Vec<T> ld_vec_nt(const T* p) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    f4 r = __builtin_nontemporal_load(reinterpret_cast<const f4*>(p));
    Vec<T> out;
    *reinterpret_cast<f4*>(&out) = r;
    return out;
}
template <class T>
__device__ __forceinline__ void st_vec_nt(T* p, const Vec<T>& v) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(*reinterpret_cast<const f4*>(&v), reinterpret_cast<f4*>(p));
}

// ------------------------------------------------------------------------------------------
// wave64 reductions (butterfly over all 64 lanes) and workgroup reductions through LDS
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
// The same sum through the data-parallel-primitive lane moves of the vector ALU instead of six trips through the LDS
// crossbar: prefix sums inside each row of 16 lanes, row totals passed on to the later rows, lane 63's total read
// back as a wave-uniform value. A different (fixed) summation order than wave_sum's butterfly.
__device__ __forceinline__ float wave_sum_dpp(float v) {
    auto shifted = [](float x, auto ctrl, auto row_mask) -> float {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                                                     decltype(row_mask)::value, 0xf, true));
    };
    using std::integral_constant;
    v += shifted(v, integral_constant<int, 0x111>{}, integral_constant<int, 0xf>{});     // row_shr:1
    v += shifted(v, integral_constant<int, 0x112>{}, integral_constant<int, 0xf>{});     // row_shr:2
    v += shifted(v, integral_constant<int, 0x114>{}, integral_constant<int, 0xf>{});     // row_shr:4
    v += shifted(v, integral_constant<int, 0x118>{}, integral_constant<int, 0xf>{});     // row_shr:8: lane 15 of a row has the row's sum
    v += shifted(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xa>{});     // row_bcast:15 into rows 1 and 3
    v += shifted(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xc>{});     // row_bcast:31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
// all threads of the block must call; blockDim.x a multiple of 64, at most 1024.
// `slot` selects one of a few LDS arrays so consecutive reductions need no extra barrier.
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* smem /* >= 16 floats */) {
    v = IS_MAX ? wave_max(v) : wave_sum(v);
    const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    if (lane == 0) smem[wid] = v;
    __syncthreads();
    float r = lane < nw ? smem[lane] : (IS_MAX ? -INFINITY : 0.f);
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) r = IS_MAX ? fmaxf(r, __shfl_xor(r, o, WAVE)) : r + __shfl_xor(r, o, WAVE);
    return __shfl(r, 0, WAVE);
}

// ------------------------------------------------------------------------------------------
// Counter-based noise for stochastic rounding: SquirrelNoise5, the generator the reference
// uses (llmc/cuda_utils.cuh:238-264).
__host__ __device__ __forceinline__ uint32_t squirrel_noise5(uint32_t pos, uint32_t seed) {
    uint32_t x = pos;
    x *= 0xd2a80a3fu; x += seed; x ^= x >> 9;
    x += 0xa884f197u; x ^= x >> 11;
    x *= 0x6C736F4Bu; x ^= x >> 13;
    x += 0xB79F3ABBu; x ^= x >> 15;
    x *= 0x1b56c4f5u; x ^= x >> 17;
    return x;
}
__host__ __device__ __forceinline__ uint32_t noise_2d(uint32_t x, uint32_t y, uint32_t seed) {
    return squirrel_noise5(x + 198491317u * y, seed);
}
// fp32 -> storage type with stochastic rounding driven by the 16 low bits of `rnd`
// (llmc/cuda_utils.cuh:267-278). Identity for fp32 storage.
__device__ __forceinline__ void stochastic_store(float in, __bf16* out, uint32_t rnd) {
    uint32_t thr = rnd & 0xffffu;
    uint32_t bits = __float_as_uint(in);
    uint32_t low = bits & 0xffffu;
    bits = (low > thr) ? (bits | 0xffffu) : (bits & ~0xffffu);
    *out = (__bf16)__uint_as_float(bits);
}
__device__ __forceinline__ void stochastic_store(float in, float* out, uint32_t) { *out = in; }
__device__ __forceinline__ __bf16 stochastic_round(float in, __bf16, uint32_t rnd) {
    __bf16 r; stochastic_store(in, &r, rnd); return r;
}
__device__ __forceinline__ float stochastic_round(float in, float, uint32_t) { return in; }
