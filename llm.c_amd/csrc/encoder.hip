// Token + position embedding: forward gather-add, backward scatter without atomics.
// Reference: llmc/encoder.cuh (forward :157, backward :169), CPU definition train_gpt2.c:35-76.
//
// Backward design for MI355X. dwpe[t,:] is a sum over the batch of rows B apart: one lane per
// 16-byte column vector walks the B rows. dwte needs, per distinct token, the sum of all rows
// that used it. The host groups positions by token with a counting sort (O(B*T), stable, so
// every bucket lists its positions in ascending order), sorts buckets by size so long ones
// start first, and the device gives each (token, 512-channel group) one workgroup whose four
// wavefronts stride over the bucket's positions and are then added in wave order. Nothing
// depends on scheduling, so the result is bit-reproducible.
#include "common.hpp"
#include "../../include/llmk.h"
#include <algorithm>
#include <vector>

namespace {
constexpr int VN = vecX::N;

__global__ void __launch_bounds__(256)
encoder_forward_kernel(floatX* __restrict__ out, const int* __restrict__ inp, const floatX* __restrict__ wte,
                       const floatX* __restrict__ wpe, int N, int T, int C) {
    const int vec_per_row = C / VN;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)N * vec_per_row) return;
    int bt = (int)(i / vec_per_row), c = (int)(i % vec_per_row) * VN;
    int t = bt % T;
    int tok = inp[bt];
    vecX a = ld_vec(wte + (size_t)tok * C + c), p = ld_vec(wpe + (size_t)t * C + c), o;
#pragma unroll
    for (int k = 0; k < VN; k++) o[k] = from_f32<floatX>(to_f32(a[k]) + to_f32(p[k]));
    st_vec_nt(out + (size_t)bt * C + c, o);
}

__global__ void __launch_bounds__(256)
wpe_backward_kernel(floatX* __restrict__ dwpe, const floatX* __restrict__ dout, int B, int T, int C, uint32_t seed) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;   // vector index into (T, C)
    size_t nvec = (size_t)T * C / VN;
    if (i >= nvec) return;
    size_t e = i * VN;
    float acc[VN];
#pragma unroll
    for (int k = 0; k < VN; k++) acc[k] = 0.f;
    for (int b = 0; b < B; b++) {
        vecX d = ld_vec(dout + (size_t)b * T * C + e);
#pragma unroll
        for (int k = 0; k < VN; k++) acc[k] += to_f32(d[k]);
    }
    vecX cur = ld_vec(dwpe + e);
#pragma unroll
    for (int k = 0; k < VN; k++)
        stochastic_store(acc[k] + to_f32(cur[k]), &cur[k], squirrel_noise5((uint32_t)(e + k), seed));
    st_vec(dwpe + e, cur);
}

struct Bucket { int start, size, token, cgroup; };   // the reference's int4 bucket_info record

// one workgroup (4 waves) per bucket; lane = one 16-byte column vector of the 64*VN-channel group
__global__ void __launch_bounds__(256)
wte_backward_kernel(floatX* __restrict__ dwte, const Bucket* __restrict__ buckets, const int* __restrict__ positions,
                    const floatX* __restrict__ dout, int C, uint32_t seed) {
    __shared__ float part[3][64][VN];
    const Bucket bk = buckets[blockIdx.x];
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int c = bk.cgroup * 64 * VN + lane * VN;
    const bool active = c < C;
    float acc[VN];
#pragma unroll
    for (int k = 0; k < VN; k++) acc[k] = 0.f;
    if (active) {
        for (int it = wid; it < bk.size; it += 4) {
            int bt = positions[bk.start + it];
            vecX d = ld_vec(dout + (size_t)bt * C + c);
#pragma unroll
            for (int k = 0; k < VN; k++) acc[k] += to_f32(d[k]);
        }
    }
    if (wid > 0) {
#pragma unroll
        for (int k = 0; k < VN; k++) part[wid - 1][lane][k] = acc[k];
    }
    __syncthreads();
    if (wid == 0 && active) {
        const size_t e = (size_t)bk.token * C + c;
        vecX cur = ld_vec(dwte + e);
#pragma unroll
        for (int k = 0; k < VN; k++) {
            float s = acc[k] + part[0][lane][k] + part[1][lane][k] + part[2][lane][k];
            stochastic_store(s + to_f32(cur[k]), &cur[k], squirrel_noise5((uint32_t)(e + k), seed ^ 0x9E3779B9u));
        }
        st_vec(dwte + e, cur);
    }
}
}  // namespace

extern "C" {

void llmk_encoder_forward(void* out, const int* inp, const void* wte, const void* wpe, int B, int T, int C,
                          void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(C > 0 && C % VN == 0, "encoder_forward: C=%d must be a multiple of %d", C, VN);
    size_t n = (size_t)B * T * (C / VN);
    if (n == 0) return;
    llmk::ProfScope prof("encoder_forward", 0, 3.0 * B * T * C * sizeof(floatX) + 4.0 * B * T, (hipStream_t)stream);
    encoder_forward_kernel<<<(unsigned)CEIL_DIV(n, (size_t)256), 256, 0, (hipStream_t)stream>>>(
        (floatX*)out, inp, (const floatX*)wte, (const floatX*)wpe, B * T, T, C);
    LAUNCH_CHECK();
}

void llmk_encoder_backward(void* dwte, void* dwpe, void* scratch, int* workload_indices, int* bucket_info,
                           const void* dout, const int* inp, const int* inputs_cpu, int B, int T, int C,
                           unsigned int seed, void* stream) {
    if (llmk::failed()) return;
    (void)inp;
    LLMK_REQUIRE(C > 0 && C % VN == 0, "encoder_backward: C=%d must be a multiple of %d", C, VN);
    const int N = B * T;
    if (N == 0) return;
    hipStream_t st = (hipStream_t)stream;
    // dwpe first: it runs on the GPU while the host builds the buckets
    size_t nvec = (size_t)T * C / VN;
    {
    llmk::ProfScope prof("wpe_backward", 0, ((double)B * T * C + 2.0 * T * C) * sizeof(floatX), st);
    wpe_backward_kernel<<<(unsigned)CEIL_DIV(nvec, (size_t)256), 256, 0, st>>>((floatX*)dwpe, (const floatX*)dout, B, T, C, seed);
    LAUNCH_CHECK();
    }

    // counting sort of positions by token (stable)
    int maxtok = 0;
    for (int i = 0; i < N; i++) {
        LLMK_REQUIRE(inputs_cpu[i] >= 0, "encoder_backward: negative token at %d", i);
        maxtok = std::max(maxtok, inputs_cpu[i]);
    }
    std::vector<int> count((size_t)maxtok + 2, 0);
    for (int i = 0; i < N; i++) count[(size_t)inputs_cpu[i] + 1]++;
    for (int v = 0; v <= maxtok; v++) count[v + 1] += count[v];          // count[v] = start of token v
    {
        std::vector<int> cursor(count.begin(), count.end() - 1);
        for (int i = 0; i < N; i++) workload_indices[cursor[inputs_cpu[i]]++] = i;
    }
    const int ncg = CEIL_DIV(C, 64 * VN);
    Bucket* bk = reinterpret_cast<Bucket*>(bucket_info);
    int nb = 0;
    for (int v = 0; v <= maxtok; v++) {
        int sz = count[v + 1] - count[v];
        if (sz == 0) continue;
        for (int g = 0; g < ncg; g++) bk[nb++] = Bucket{count[v], sz, v, g};
    }
    // largest buckets first; ties by (token, group) so the order is a pure function of the input
    std::sort(bk, bk + nb, [](const Bucket& a, const Bucket& b) {
        if (a.size != b.size) return a.size > b.size;
        if (a.token != b.token) return a.token < b.token;
        return a.cgroup < b.cgroup;
    });
    Bucket* d_bk = reinterpret_cast<Bucket*>(scratch);
    int* d_pos = reinterpret_cast<int*>(reinterpret_cast<char*>(scratch) + (size_t)N * ncg * sizeof(Bucket));
    HIP_CHECK(hipMemcpyAsync(d_bk, bk, (size_t)nb * sizeof(Bucket), hipMemcpyHostToDevice, st));
    HIP_CHECK(hipMemcpyAsync(d_pos, workload_indices, (size_t)N * sizeof(int), hipMemcpyHostToDevice, st));
    llmk::ProfScope prof("wte_backward", 0, 3.0 * N * C * sizeof(floatX), st);
    wte_backward_kernel<<<nb, 256, 0, st>>>((floatX*)dwte, d_bk, d_pos, (const floatX*)dout, C, seed);
    LAUNCH_CHECK();
}
}
