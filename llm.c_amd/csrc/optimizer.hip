// AdamW with fp32 master weights and stochastic rounding, the squared gradient norm, the
// deterministic single-workgroup sum, and the fp32 cast used to seed the master copy.
// Reference: llmc/adamw.cuh:74-98, llmc/global_norm.cuh:52-89, llmc/cuda_utils.cuh:134-212.
// All HBM-bound streaming kernels over 16-byte vectors.
#include "common.hpp"
#include "../../include/llmk.h"

namespace {
constexpr int VN = vecX::N;

// two-instruction lerp, as the reference (llmc/adamw.cuh:14-16)
__device__ __forceinline__ float lerp2(float start, float end, float w) { return fmaf(w, end, fmaf(-w, start, start)); }

// noise word of element i of slice s: what the reference's (block 512, grid (n/512, slices))
// launch computes from threadIdx/blockIdx (llmc/cuda_utils.cuh:272), as a function of (i, s)
__device__ __forceinline__ uint32_t adamw_noise(size_t i, int slice, uint32_t seed) {
    return noise_2d((uint32_t)(i & 511), (uint32_t)((i >> 9) << 9) + (uint32_t)slice, seed);
}

struct AdamArgs {
    float lr, b1, b2, c1, c2, eps, wd, gscale;
    uint32_t seed;
};

__device__ __forceinline__ float adam_one(float g, float& m, float& v, float old, const AdamArgs& a) {
    g *= a.gscale;
    m = lerp2(g, m, a.b1);
    v = lerp2(g * g, v, a.b2);
    float mh = m / a.c1, vh = v / a.c2;
    return old - a.lr * (mh / (sqrtf(vh) + a.eps) + a.wd * old);
}

// vector path: n, strides multiples of VN and all pointers 16-byte aligned
__global__ void __launch_bounds__(256)
adamw_vec_kernel(floatX* __restrict__ params, float* __restrict__ master, const floatX* __restrict__ grads,
                 float* __restrict__ m, float* __restrict__ v, size_t n, ptrdiff_t w_stride, ptrdiff_t g_stride,
                 ptrdiff_t s_stride, AdamArgs a) {
    const int slice = blockIdx.y;
    size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VN;
    if (i >= n) return;
    params += slice * w_stride; grads += slice * g_stride; m += slice * s_stride; v += slice * s_stride;
    if (master) master += slice * s_stride;
    vecX g = ld_vec_nt(grads + i);
    vecX p;
    if (!master) p = ld_vec(params + i);
    float mm[VN], vv[VN], ms[VN];
#pragma unroll
    for (int q = 0; q < VN / 4; q++) {
        vecF t = ld_vec(m + i + q * 4), u = ld_vec(v + i + q * 4);
#pragma unroll
        for (int k = 0; k < 4; k++) { mm[q * 4 + k] = t[k]; vv[q * 4 + k] = u[k]; }
        if (master) {
            vecF w = ld_vec(master + i + q * 4);
#pragma unroll
            for (int k = 0; k < 4; k++) ms[q * 4 + k] = w[k];
        }
    }
#pragma unroll
    for (int k = 0; k < VN; k++) {
        float old = master ? ms[k] : to_f32(p[k]);
        float np = adam_one(to_f32(g[k]), mm[k], vv[k], old, a);
        ms[k] = np;
        stochastic_store(np, &p[k], adamw_noise(i + k, slice, a.seed));
    }
    st_vec(params + i, p);
#pragma unroll
    for (int q = 0; q < VN / 4; q++) {
        vecF t, u, w;
#pragma unroll
        for (int k = 0; k < 4; k++) { t[k] = mm[q * 4 + k]; u[k] = vv[q * 4 + k]; w[k] = ms[q * 4 + k]; }
        st_vec(m + i + q * 4, t);
        st_vec(v + i + q * 4, u);
        if (master) st_vec(master + i + q * 4, w);
    }
}

// All tensors of a model in one launch: block b belongs to the tensor whose range of blocks contains it, then to a slice
// and a 2048-element piece of that slice. Same arithmetic, same noise words as one adamw_vec_kernel launch per tensor.
struct AdamTensorTable {
    static constexpr int MAX = 16;
    int count;
    unsigned first_block[MAX + 1];        // first_block[count] = grid size
    unsigned blocks_per_slice[MAX];
    unsigned long long offset[MAX];       // elements from the start of every arena
    unsigned long long n[MAX];            // elements per slice (slices are contiguous: stride n)
    float wd[MAX];
    unsigned seed[MAX];
};
__global__ void __launch_bounds__(256)
adamw_multi_kernel(floatX* __restrict__ params, float* __restrict__ master, const floatX* __restrict__ grads,
                   float* __restrict__ m, float* __restrict__ v, AdamTensorTable tab, AdamArgs a,
                   const float* __restrict__ grad_norm_squared, float grad_clip) {
    int ti = 0;
    while (ti + 1 < tab.count && blockIdx.x >= tab.first_block[ti + 1]) ti++;      // wave-uniform, at most 15 steps
    const unsigned local = blockIdx.x - tab.first_block[ti];
    const int slice = (int)(local / tab.blocks_per_slice[ti]);
    const size_t n = tab.n[ti];
    const size_t i = ((size_t)(local % tab.blocks_per_slice[ti]) * 256 + threadIdx.x) * VN;
    if (i >= n) return;
    const size_t base = tab.offset[ti] + (size_t)slice * n + i;
    a.wd = tab.wd[ti];
    a.seed = tab.seed[ti];
    if (grad_norm_squared) {              // clipping decided here: the host's two statements (train_gpt2.cu:1841-1851), correctly rounded alike
        const float norm = sqrtf(*grad_norm_squared);
        a.gscale = norm > grad_clip ? grad_clip / norm : 1.0f;
    }
    vecX g = ld_vec_nt(grads + base);
    vecX p;
    if (!master) p = ld_vec(params + base);
    float mm[VN], vv[VN], ms[VN];
#pragma unroll
    for (int q = 0; q < VN / 4; q++) {
        vecF t = ld_vec(m + base + q * 4), u = ld_vec(v + base + q * 4);
#pragma unroll
        for (int k = 0; k < 4; k++) { mm[q * 4 + k] = t[k]; vv[q * 4 + k] = u[k]; }
        if (master) {
            vecF w = ld_vec(master + base + q * 4);
#pragma unroll
            for (int k = 0; k < 4; k++) ms[q * 4 + k] = w[k];
        }
    }
#pragma unroll
    for (int k = 0; k < VN; k++) {
        float old = master ? ms[k] : to_f32(p[k]);
        float np = adam_one(to_f32(g[k]), mm[k], vv[k], old, a);
        ms[k] = np;
        stochastic_store(np, &p[k], adamw_noise(i + k, slice, a.seed));
    }
    st_vec(params + base, p);
#pragma unroll
    for (int q = 0; q < VN / 4; q++) {
        vecF t, u, w;
#pragma unroll
        for (int k = 0; k < 4; k++) { t[k] = mm[q * 4 + k]; u[k] = vv[q * 4 + k]; w[k] = ms[q * 4 + k]; }
        st_vec(m + base + q * 4, t);
        st_vec(v + base + q * 4, u);
        if (master) st_vec(master + base + q * 4, w);
    }
}

__global__ void __launch_bounds__(256)
adamw_scalar_kernel(floatX* __restrict__ params, float* __restrict__ master, const floatX* __restrict__ grads,
                    float* __restrict__ m, float* __restrict__ v, size_t n, ptrdiff_t w_stride, ptrdiff_t g_stride,
                    ptrdiff_t s_stride, AdamArgs a) {
    const int slice = blockIdx.y;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    params += slice * w_stride; grads += slice * g_stride; m += slice * s_stride; v += slice * s_stride;
    if (master) master += slice * s_stride;
    float mi = m[i], vi = v[i];
    float old = master ? master[i] : to_f32(params[i]);
    float np = adam_one(to_f32(grads[i]), mi, vi, old, a);
    m[i] = mi; v[i] = vi;
    stochastic_store(np, &params[i], adamw_noise(i, slice, a.seed));
    if (master) master[i] = np;
}

__global__ void __launch_bounds__(256)
init_from_master_kernel(floatX* __restrict__ params, const float* __restrict__ master, size_t n, ptrdiff_t w_stride,
                        ptrdiff_t s_stride, uint32_t seed) {
    const int slice = blockIdx.y;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    stochastic_store(master[i + slice * s_stride], &params[i + slice * w_stride], adamw_noise(i, slice, seed));
}

__global__ void __launch_bounds__(256)
copy_cast_kernel(float* __restrict__ dst, const floatX* __restrict__ src, size_t n, ptrdiff_t stride_dst,
                 ptrdiff_t stride_src) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    dst[i + stride_dst * blockIdx.y] = to_f32(src[i + stride_src * blockIdx.y]);
}

// ---- squared norm ---------------------------------------------------------------------------
constexpr int NORM_BLOCK = 512;
__global__ void __launch_bounds__(NORM_BLOCK)
norm_squared_kernel(float* __restrict__ out, const floatX* __restrict__ data, size_t count, ptrdiff_t stride) {
    __shared__ float red[16];
    const floatX* x = data + blockIdx.y * stride;
    float acc = 0.f;
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nth = (size_t)gridDim.x * blockDim.x;
    const bool aligned = ((uintptr_t)x % 16) == 0;
    if (aligned) {
        const size_t nvec = count / VN;
        for (size_t i = tid; i < nvec; i += nth) {
            vecX d = ld_vec_nt(x + i * VN);
#pragma unroll
            for (int k = 0; k < VN; k++) { float f = to_f32(d[k]); acc += f * f; }
        }
        for (size_t i = nvec * VN + tid; i < count; i += nth) { float f = to_f32(x[i]); acc += f * f; }
    } else {
        for (size_t i = tid; i < count; i += nth) { float f = to_f32(x[i]); acc += f * f; }
    }
    float s = block_reduce<false>(acc, red);
    if (threadIdx.x == 0) {
        size_t o = (size_t)blockIdx.y * gridDim.x + blockIdx.x;
        out[o] = out[o] + s;      // accumulates across calls, as the reference (global_norm.cuh:36-39)
    }
}

__global__ void __launch_bounds__(1024)
sum_single_block_kernel(float* __restrict__ result, const float* __restrict__ values, size_t count) {
    __shared__ float red[16];
    float acc = 0.f;
    for (size_t i = threadIdx.x; i < count; i += blockDim.x) acc += values[i];
    float s = block_reduce<false>(acc, red);
    if (threadIdx.x == 0) *result = s;
}

__global__ void fill_zero_kernel(float* p, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

int norm_grid() { return llmk::device_info().num_cu * 2; }
}  // namespace

extern "C" {

void llmk_adamw_update(void* params_memory, float* master, const void* grads_memory, float* m, float* v,
                       size_t n, ptrdiff_t w_stride, ptrdiff_t g_stride, ptrdiff_t s_stride, int num_slices,
                       float lr, float beta1, float beta2, int t, float eps, float weight_decay, float grad_scale,
                       unsigned int seed, void* stream) {
    if (llmk::failed()) return;
    if (n == 0 || num_slices <= 0) return;
    AdamArgs a{lr, beta1, beta2, 1.0f - powf(beta1, (float)t), 1.0f - powf(beta2, (float)t), eps, weight_decay, grad_scale, seed};
    hipStream_t st = (hipStream_t)stream;
    auto al = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    llmk::ProfScope prof("adamw_update", 0, (double)n * num_slices * (master ? 2.0 * sizeof(floatX) + 24.0 : 3.0 * sizeof(floatX) + 16.0), st);
    bool vec = (n % VN == 0) && (w_stride % VN == 0) && (g_stride % VN == 0) && (s_stride % VN == 0) &&
               al(params_memory) && al(grads_memory) && al(m) && al(v) && (!master || al(master));
    if (vec) {
        dim3 grid((unsigned)CEIL_DIV(n / VN, (size_t)256), num_slices);
        adamw_vec_kernel<<<grid, 256, 0, st>>>((floatX*)params_memory, master, (const floatX*)grads_memory, m, v, n,
                                               w_stride, g_stride, s_stride, a);
    } else {
        dim3 grid((unsigned)CEIL_DIV(n, (size_t)256), num_slices);
        adamw_scalar_kernel<<<grid, 256, 0, st>>>((floatX*)params_memory, master, (const floatX*)grads_memory, m, v, n,
                                                  w_stride, g_stride, s_stride, a);
    }
    LAUNCH_CHECK();
}

static int adamw_multi(void* params_memory, float* master, const void* grads_memory, float* m, float* v, int count,
                       const size_t* offsets, const size_t* sizes, const int* num_slices, const float* weight_decays,
                       const unsigned int* seeds, float lr, float beta1, float beta2, int t, float eps, float grad_scale,
                       const float* grad_norm_squared, float grad_clip, void* stream) {
    if (llmk::failed()) return 0;
    if (count <= 0 || count > AdamTensorTable::MAX) return 0;
    auto al = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    if (!(al(params_memory) && al(grads_memory) && al(m) && al(v) && (!master || al(master)))) return 0;
    AdamTensorTable tab{};
    tab.count = count;
    unsigned long long blocks = 0;
    double elems = 0;
    for (int i = 0; i < count; i++) {
        if (sizes[i] == 0 || num_slices[i] <= 0 || sizes[i] % VN != 0 || offsets[i] % VN != 0) return 0;
        tab.first_block[i] = (unsigned)blocks;
        tab.blocks_per_slice[i] = (unsigned)CEIL_DIV(sizes[i] / VN, (size_t)256);
        tab.offset[i] = offsets[i]; tab.n[i] = sizes[i]; tab.wd[i] = weight_decays[i]; tab.seed[i] = seeds[i];
        blocks += (unsigned long long)tab.blocks_per_slice[i] * num_slices[i];
        elems += (double)sizes[i] * num_slices[i];
        if (blocks > 0x7fffffffull) return 0;
    }
    tab.first_block[count] = (unsigned)blocks;
    AdamArgs a{lr, beta1, beta2, 1.0f - powf(beta1, (float)t), 1.0f - powf(beta2, (float)t), eps, 0.f, grad_scale, 0u};
    hipStream_t st = (hipStream_t)stream;
    llmk::ProfScope prof("adamw_update", 0, elems * (master ? 2.0 * sizeof(floatX) + 24.0 : 3.0 * sizeof(floatX) + 16.0), st);
    adamw_multi_kernel<<<(unsigned)blocks, 256, 0, st>>>((floatX*)params_memory, master, (const floatX*)grads_memory, m, v, tab, a,
                                                         grad_norm_squared, grad_clip);
    LAUNCH_CHECK();
    return 1;
}

int llmk_adamw_update_multi(void* params_memory, float* master, const void* grads_memory, float* m, float* v, int count,
                            const size_t* offsets, const size_t* sizes, const int* num_slices, const float* weight_decays,
                            const unsigned int* seeds, float lr, float beta1, float beta2, int t, float eps, float grad_scale,
                            void* stream) {
    return adamw_multi(params_memory, master, grads_memory, m, v, count, offsets, sizes, num_slices, weight_decays, seeds, lr, beta1,
                       beta2, t, eps, grad_scale, nullptr, 0.f, stream);
}

int llmk_adamw_update_multi_clip(void* params_memory, float* master, const void* grads_memory, float* m, float* v, int count,
                                 const size_t* offsets, const size_t* sizes, const int* num_slices, const float* weight_decays,
                                 const unsigned int* seeds, float lr, float beta1, float beta2, int t, float eps,
                                 const float* grad_norm_squared, float grad_clip, void* stream) {
    if (grad_norm_squared == nullptr) return 0;
    return adamw_multi(params_memory, master, grads_memory, m, v, count, offsets, sizes, num_slices, weight_decays, seeds, lr, beta1,
                       beta2, t, eps, 1.0f, grad_norm_squared, grad_clip, stream);
}

void llmk_init_from_master(void* params_memory, const float* master, size_t n, ptrdiff_t w_stride,
                           ptrdiff_t s_stride, int num_slices, unsigned int seed, void* stream) {
    if (llmk::failed()) return;
    if (n == 0 || num_slices <= 0) return;
    dim3 grid((unsigned)CEIL_DIV(n, (size_t)256), num_slices);
    init_from_master_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((floatX*)params_memory, master, n, w_stride, s_stride, seed);
    LAUNCH_CHECK();
}

void llmk_copy_and_cast_to_f32(float* dst, const void* src, size_t n, ptrdiff_t stride_dst, ptrdiff_t stride_src,
                               int num_slices, void* stream) {
    if (llmk::failed()) return;
    if (n == 0 || num_slices <= 0) return;
    dim3 grid((unsigned)CEIL_DIV(n, (size_t)256), num_slices);
    copy_cast_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(dst, (const floatX*)src, n, stride_dst, stride_src);
    LAUNCH_CHECK();
}

int llmk_get_max_num_block_sums(const int* num_slices_all, int numel) {
    const int grid = norm_grid();
    int mx = 0;
    for (int i = 0; i < numel; i++) {
        int s = num_slices_all[i];
        mx = max(mx, CEIL_DIV(grid, s) * s);
    }
    return mx;
}

void llmk_global_norm_squared(float* out, const void* values, size_t count, ptrdiff_t stride, int num_slices,
                              int max_num_block_sums, int reset, void* stream) {
    if (llmk::failed()) return;
    hipStream_t st = (hipStream_t)stream;
    const int gx = CEIL_DIV(norm_grid(), num_slices), gy = num_slices;
    LLMK_REQUIRE(gx * gy <= max_num_block_sums, "global_norm_squared: %d block sums exceed max_num_block_sums=%d",
                 gx * gy, max_num_block_sums);
    if (reset) {
        fill_zero_kernel<<<CEIL_DIV(max_num_block_sums, 256), 256, 0, st>>>(out, max_num_block_sums);
        LAUNCH_CHECK();
    }
    llmk::ProfScope prof("global_norm_squared", 0, (double)count * num_slices * sizeof(floatX), st);
    norm_squared_kernel<<<dim3(gx, gy), NORM_BLOCK, 0, st>>>(out, (const floatX*)values, count, stride);
    LAUNCH_CHECK();
}

void llmk_global_sum_deterministic(float* result, const float* values, int count, void* stream) {
    if (llmk::failed()) return;
    sum_single_block_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(result, values, (size_t)count);
    LAUNCH_CHECK();
}
}
