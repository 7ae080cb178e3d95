// LayerNorm forward / fused residual+LayerNorm / residual add / LayerNorm backward for gfx950.
//
// All four are HBM-bound. Layout: one 64-lane wavefront owns one row at a time and keeps it in
// registers (16-byte vectors, lane-interleaved so every load instruction of the wave covers a
// contiguous 1 KiB), so each activation byte crosses HBM exactly once; weight/bias vectors of
// the lane's columns stay in registers while the wave walks over its rows.
//
// Arithmetic follows the reference's CPU definitions: two-pass mean / biased variance with
// eps 1e-5 (train_gpt2.c:78-118), backward per train_gpt2.c:120-161, statistics in fp32,
// and — in the fused kernel — statistics of the residual AFTER rounding it to the storage
// type (llmc/layernorm.cuh:178-184).
#include "common.hpp"
#include "../../include/llmk.h"

namespace {

constexpr int LN_BLOCK = 256;                 // 4 wavefronts per workgroup
constexpr int LN_WAVES = LN_BLOCK / WAVE;
constexpr int VN = vecX::N;

// ---- forward ------------------------------------------------------------------------------
// NV = vectors per lane (ceil(C / (VN*64))). RES: out-of-place residual add first.
template <int NV, bool RES>
__global__ void __launch_bounds__(LN_BLOCK)
ln_forward_kernel(floatX* __restrict__ normed, floatX* __restrict__ residual, float* __restrict__ mean,
                  float* __restrict__ rstd, const floatX* __restrict__ inp1, const floatX* __restrict__ inp2,
                  const floatX* __restrict__ weight, const floatX* __restrict__ bias, int N, int C) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * LN_WAVES + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * LN_WAVES;
    const int nvec = C / VN;

    vecX w[NV], b[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int v = lane + i * 64;
        if (v < nvec) { w[i] = ld_vec(weight + (size_t)v * VN); b[i] = ld_vec(bias + (size_t)v * VN); }
    }
    const float invC = 1.0f / (float)C;

    // Wide rows (NV >= 3) keep row, weight and bias in registers in their packed form: `pin` names a vector in an
    // empty asm, so that the compiler converts its columns where they are used instead of keeping fp32 copies alive
    // across the row loop and the reductions, which gives those rows another wave per SIMD. Up to NV = 2 (C = 768,
    // 1024) the fp32 copies are the better trade: with them the kernel measured 10 % faster there.
    auto pin = [](vecX& v) {
        if constexpr (NV >= 3) {
            unsigned* p = reinterpret_cast<unsigned*>(&v);
#pragma unroll
            for (int q = 0; q < 4; q++) asm volatile("" : "+v"(p[q]));
        }
    };
    for (int row = wave; row < N; row += nwaves) {
        const size_t base = (size_t)row * C;
        vecX x[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) { pin(w[i]); pin(b[i]); }
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int v = lane + i * 64;
            if (v < nvec) {
                x[i] = ld_vec_nt(inp1 + base + (size_t)v * VN);
                if (RES) {
                    vecX y = ld_vec_nt(inp2 + base + (size_t)v * VN);
#pragma unroll
                    for (int k = 0; k < VN; k++) x[i][k] = from_f32<floatX>(to_f32(x[i][k]) + to_f32(y[k]));
                    st_vec(residual + base + (size_t)v * VN, x[i]);
                }
            }
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NV; i++)
            if (lane + i * 64 < nvec) {
#pragma unroll
                for (int k = 0; k < VN; k++) s += to_f32(x[i][k]);
            }
        const float m = wave_sum(s) * invC;
#pragma unroll
        for (int i = 0; i < NV; i++) pin(x[i]);
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < NV; i++)
            if (lane + i * 64 < nvec) {
#pragma unroll
                for (int k = 0; k < VN; k++) { float d = to_f32(x[i][k]) - m; q += d * d; }
            }
        const float var = wave_sum(q) * invC;
        const float r = 1.0f / sqrtf(var + 1e-5f);
#pragma unroll
        for (int i = 0; i < NV; i++) pin(x[i]);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int v = lane + i * 64;
            if (v < nvec) {
                vecX o;
#pragma unroll
                for (int k = 0; k < VN; k++)
                    o[k] = from_f32<floatX>(r * (to_f32(x[i][k]) - m) * to_f32(w[i][k]) + to_f32(b[i][k]));
                st_vec(normed + base + (size_t)v * VN, o);
            }
        }
        if (lane == 0) {
            if (mean) mean[row] = m;
            if (rstd) rstd[row] = r;
        }
    }
}

// Any C (multiple of VN) beyond what fits in registers: re-reads the row (it sits in L2).
template <bool RES>
__global__ void __launch_bounds__(LN_BLOCK)
ln_forward_generic_kernel(floatX* __restrict__ normed, floatX* __restrict__ residual, float* __restrict__ mean,
                          float* __restrict__ rstd, const floatX* __restrict__ inp1,
                          const floatX* __restrict__ inp2, const floatX* __restrict__ weight,
                          const floatX* __restrict__ bias, int N, int C) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * LN_WAVES + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * LN_WAVES;
    const int nvec = C / VN;
    const float invC = 1.0f / (float)C;
    for (int row = wave; row < N; row += nwaves) {
        const size_t base = (size_t)row * C;
        const floatX* src = inp1 + base;
        if (RES) {
            for (int v = lane; v < nvec; v += 64) {
                vecX a = ld_vec(inp1 + base + (size_t)v * VN), y = ld_vec(inp2 + base + (size_t)v * VN);
#pragma unroll
                for (int k = 0; k < VN; k++) a[k] = from_f32<floatX>(to_f32(a[k]) + to_f32(y[k]));
                st_vec(residual + base + (size_t)v * VN, a);
            }
            __threadfence_block();
            src = residual + base;
        }
        float s = 0.f;
        for (int v = lane; v < nvec; v += 64) {
            vecX a = ld_vec(src + (size_t)v * VN);
#pragma unroll
            for (int k = 0; k < VN; k++) s += to_f32(a[k]);
        }
        const float m = wave_sum(s) * invC;
        float q = 0.f;
        for (int v = lane; v < nvec; v += 64) {
            vecX a = ld_vec(src + (size_t)v * VN);
#pragma unroll
            for (int k = 0; k < VN; k++) { float d = to_f32(a[k]) - m; q += d * d; }
        }
        const float r = 1.0f / sqrtf(wave_sum(q) * invC + 1e-5f);
        for (int v = lane; v < nvec; v += 64) {
            vecX a = ld_vec(src + (size_t)v * VN), w = ld_vec(weight + (size_t)v * VN), b = ld_vec(bias + (size_t)v * VN), o;
#pragma unroll
            for (int k = 0; k < VN; k++) o[k] = from_f32<floatX>(r * (to_f32(a[k]) - m) * to_f32(w[k]) + to_f32(b[k]));
            st_vec(normed + base + (size_t)v * VN, o);
        }
        if (lane == 0) {
            if (mean) mean[row] = m;
            if (rstd) rstd[row] = r;
        }
    }
}

template <bool RES>
void launch_ln_forward(floatX* normed, floatX* residual, float* mean, float* rstd, const floatX* inp1,
                       const floatX* inp2, const floatX* weight, const floatX* bias, int N, int C, hipStream_t st) {
    const int nvec = C / VN;
    const int nv = CEIL_DIV(nvec, 64);
    const llmk::DeviceInfo& d = llmk::device_info();
    const double bytes = (RES ? 4.0 : 2.0) * N * C * sizeof(floatX) + 2.0 * N * sizeof(float);
    llmk::ProfScope prof(RES ? "fused_residual_forward" : "layernorm_forward", 0, bytes, st);
    // Exactly as many workgroups as are resident at once (the kernel's registers decide how many per CU), each wave
    // walking its share of the rows: with more, the workgroups of the second round start when the first ones end and
    // the CUs finish unevenly (8 per CU where 5 fit measured 2 % slower than 5, 6 where 5 fit 15 % slower).
    auto grid_for = [&](const void* kernel, int& per_cu) -> int {
        if (per_cu == 0) {            // asked once per kernel
            HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, LN_BLOCK, 0));
            if (per_cu < 1) per_cu = 1;
        }
        const int blocks = min(d.num_cu * per_cu, CEIL_DIV(N, LN_WAVES));
        return blocks < 1 ? 1 : blocks;
    };
#define LN_CASE(K)                                                                                            \
    case K: {                                                                                                 \
        static int per_cu = 0;                                                                                \
        const int blocks = grid_for((const void*)ln_forward_kernel<K, RES>, per_cu);                          \
        ln_forward_kernel<K, RES><<<blocks, LN_BLOCK, 0, st>>>(normed, residual, mean, rstd, inp1, inp2,      \
                                                               weight, bias, N, C);                           \
        break; }
    switch (nv) {
        LN_CASE(1) LN_CASE(2) LN_CASE(3) LN_CASE(4) LN_CASE(5) LN_CASE(6) LN_CASE(7) LN_CASE(8)
        default: {
            static int per_cu = 0;
            const int blocks = grid_for((const void*)ln_forward_generic_kernel<RES>, per_cu);
            ln_forward_generic_kernel<RES><<<blocks, LN_BLOCK, 0, st>>>(normed, residual, mean, rstd, inp1, inp2,
                                                                        weight, bias, N, C);
        }
    }
#undef LN_CASE
    LAUNCH_CHECK();
}

// ---- residual add --------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
residual_kernel(floatX* __restrict__ out, const floatX* __restrict__ a, const floatX* __restrict__ b, size_t nvec) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec) return;
    vecX x = ld_vec_nt(a + i * VN), y = ld_vec_nt(b + i * VN), o;
#pragma unroll
    for (int k = 0; k < VN; k++) o[k] = from_f32<floatX>(to_f32(x[k]) + to_f32(y[k]));
    st_vec(out + i * VN, o);
}

// ---- backward ------------------------------------------------------------------------------
// Each wave walks rows; per-lane fp32 accumulators hold dweight/dbias of the lane's columns.
// At the end the 4 waves of a workgroup are added in wave order through LDS and the workgroup's
// partial goes to scratch[block][2][C]; a second kernel adds the partials in block order, so
// the result does not depend on scheduling (no atomics).
// One workgroup per CU, as many waves as the accumulators leave room for: 12 (three per SIMD) up to NV = 2, where the
// kernel needs 170 registers, two more than three waves per SIMD allow, hence the occupancy request; 8 at NV = 3 and,
// with one row in flight per wave instead of two, at NV = 4 and 5 (C = 1600 .. 2560); 4 beyond, also with one row in
// flight (two rows of 7 or 8 vectors beside the accumulators do not fit 256 registers). At NV = 2, 16 waves with one
// row each measured the same as 12 with two.
constexpr int lnb_waves(int nv) { return nv <= 2 ? 12 : nv <= 5 ? 8 : 4; }
template <int NV>
__global__ void __launch_bounds__(lnb_waves(NV) * 64, NV <= 2 ? 3 : NV <= 5 ? 2 : 1)
ln_backward_kernel(floatX* __restrict__ dinp, float* __restrict__ partial, const floatX* __restrict__ dout,
                   const floatX* __restrict__ inp, const floatX* __restrict__ weight,
                   const float* __restrict__ mean, const float* __restrict__ rstd, int N, int C) {
    constexpr int LNB_WAVES = lnb_waves(NV);
    extern __shared__ float lds[];   // [LNB_WAVES-1][2][C]
    const int lane = threadIdx.x & 63;
    const int wid = threadIdx.x >> 6;
    const int wave = blockIdx.x * LNB_WAVES + wid;
    const int nwaves = gridDim.x * LNB_WAVES;
    const int nvec = C / VN;
    const float invC = 1.0f / (float)C;

    vecX w[NV];                          // packed: the fp32 copy would cost 8 more registers per vector
    float dw[NV][VN], db[NV][VN];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int v = lane + i * 64;
        if (v < nvec) w[i] = ld_vec(weight + (size_t)v * VN);
#pragma unroll
        for (int k = 0; k < VN; k++) { dw[i][k] = 0.f; db[i][k] = 0.f; }
    }

    // Two rows are in flight per wave: the loads of the next row are issued before the current row is reduced,
    // which doubles the bytes each CU keeps in flight at the occupancy the accumulators allow.
    auto load_row = [&](int row, vecX (&g)[NV], vecX (&x)[NV], vecX (&di)[NV]) {
        const size_t base = (size_t)row * C;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            // Every lane loads, the lanes past the row's end a copy of its last vector (NV = ceil(nvec / 64), so only the
            // last slot has such lanes; what they hold is never added to a sum nor stored). With the loads under a
            // per-lane test each sits behind a branch that may skip it, the compiler's count of loads certainly younger
            // than the ones it waits for drops to zero, and the wait for the current row also waits for the row
            // requested ahead: one row in flight instead of two.
            const int v = i == NV - 1 ? min(lane + i * 64, nvec - 1) : lane + i * 64;
            g[i] = ld_vec_nt(dout + base + (size_t)v * VN);
            x[i] = ld_vec_nt(inp + base + (size_t)v * VN);
            di[i] = ld_vec_nt(dinp + base + (size_t)v * VN);
        }
    };
    auto process_row = [&](int row, float m, float r, vecX (&g)[NV], vecX (&x)[NV], vecX (&di)[NV]) {
        const size_t base = (size_t)row * C;
        float a = 0.f, bsum = 0.f;
#pragma unroll
        for (int i = 0; i < NV; i++)
            if (lane + i * 64 < nvec) {
#pragma unroll
                for (int k = 0; k < VN; k++) {
                    float nh = (to_f32(x[i][k]) - m) * r, dn = to_f32(w[i][k]) * to_f32(g[i][k]);
                    a += dn;
                    bsum += dn * nh;
                }
            }
        a = wave_sum_dpp(a) * invC;             // lane moves inside the vector ALU: 2-4 % off the kernel against the LDS butterfly
        bsum = wave_sum_dpp(bsum) * invC;
        // the row stays packed as loaded: converted columns carried over the reductions cost up to 50 registers
#pragma unroll
        for (int i = 0; i < NV; i++) {
            unsigned* g32 = reinterpret_cast<unsigned*>(&g[i]);
            unsigned* x32 = reinterpret_cast<unsigned*>(&x[i]);
#pragma unroll
            for (int q = 0; q < 4; q++) { asm volatile("" : "+v"(g32[q])); asm volatile("" : "+v"(x32[q])); }
        }
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int v = lane + i * 64;
            if (v < nvec) {
                vecX o;
#pragma unroll
                for (int k = 0; k < VN; k++) {
                    float gk = to_f32(g[i][k]);
                    float nh = (to_f32(x[i][k]) - m) * r, dn = to_f32(w[i][k]) * gk;
                    db[i][k] += gk;
                    dw[i][k] += nh * gk;
                    o[k] = from_f32<floatX>(to_f32(di[i][k]) + (dn - a - nh * bsum) * r);
                }
                st_vec(dinp + base + (size_t)v * VN, o);
            }
        }
    };
    if constexpr (NV >= 4) {
        // wide rows: one row in flight per wave leaves room for twice the waves
        vecX g0[NV], x0[NV], d0[NV];
        for (int row = wave; row < N; row += nwaves) {
            load_row(row, g0, x0, d0);
            process_row(row, mean[row], rstd[row], g0, x0, d0);
        }
    } else {
        // The row index is kept wave-uniform and the row requested ahead is requested unconditionally (past the end: the
        // last row again, never processed): loop control is scalar branches around straight-line loads, which is what
        // the compiler needs to count the loads behind the ones it waits for. With the request under a per-lane test of
        // the row index, every wait for the current row was a wait for everything in flight.
        vecX g0[NV], x0[NV], d0[NV], g1[NV], x1[NV], d1[NV];
        int row = __builtin_amdgcn_readfirstlane(wave);
        float m0 = 0.f, r0 = 0.f, m1 = 0.f, r1 = 0.f;
        if (row < N) {
            load_row(row, g0, x0, d0); m0 = mean[row]; r0 = rstd[row];
            while (true) {
                const int row1 = row + nwaves, row1c = min(row1, N - 1);
                load_row(row1c, g1, x1, d1); m1 = mean[row1c]; r1 = rstd[row1c];
                process_row(row, m0, r0, g0, x0, d0);
                if (row1 >= N) break;
                const int row2 = row1 + nwaves, row2c = min(row2, N - 1);
                load_row(row2c, g0, x0, d0); m0 = mean[row2c]; r0 = rstd[row2c];
                process_row(row1, m1, r1, g1, x1, d1);
                if (row2 >= N) break;
                row = row2;
            }
        }
    }

    // workgroup reduction in fixed wave order
    if (wid > 0) {
        float* dst = lds + (size_t)(wid - 1) * 2 * C;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int v = lane + i * 64;
            if (v < nvec) {
#pragma unroll
                for (int k = 0; k < VN; k++) { dst[v * VN + k] = dw[i][k]; dst[C + v * VN + k] = db[i][k]; }
            }
        }
    }
    __syncthreads();
    if (wid == 0) {
        float* out = partial + (size_t)blockIdx.x * 2 * C;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int v = lane + i * 64;
            if (v < nvec) {
#pragma unroll
                for (int k = 0; k < VN; k++) {
                    float sw = dw[i][k], sb = db[i][k];
                    for (int o = 0; o < LNB_WAVES - 1; o++) {
                        sw += lds[(size_t)o * 2 * C + v * VN + k];
                        sb += lds[(size_t)o * 2 * C + C + v * VN + k];
                    }
                    out[v * VN + k] = sw;
                    out[C + v * VN + k] = sb;
                }
            }
        }
    }
}

// Rows too wide for the register-resident kernel above (more than 8 vectors per lane: C > 4096 in bf16, > 2048 in fp32,
// the GPT-3 descriptors of train_gpt2.cu:511-560 go to 12288): one 256-thread workgroup per row at a time, thread t owning
// the vectors t, t + 256, ...; the row is read twice (sums, then the update; the second read comes from cache) and the
// workgroup's dweight / dbias partials live in LDS (2 C floats) across all its rows. Same outputs and the same partial
// layout as ln_backward_kernel, so the reduce kernel below serves both. Not tuned: no benchmarked model is this wide.
__global__ void __launch_bounds__(256)
ln_backward_wide_kernel(floatX* __restrict__ dinp, float* __restrict__ partial, const floatX* __restrict__ dout,
                        const floatX* __restrict__ inp, const floatX* __restrict__ weight,
                        const float* __restrict__ mean, const float* __restrict__ rstd, int N, int C) {
    extern __shared__ float lds[];       // [2][C] partials, then 2 x 16 floats for the workgroup reductions
    float* sdw = lds;
    float* sdb = lds + C;
    float* red = lds + 2 * (size_t)C;
    const int nvec = C / VN;
    const float invC = 1.0f / (float)C;
    for (int c = threadIdx.x; c < 2 * C; c += 256) lds[c] = 0.f;
    __syncthreads();
    for (int row = blockIdx.x; row < N; row += gridDim.x) {
        const size_t base = (size_t)row * C;
        const float m = mean[row], r = rstd[row];
        float a = 0.f, bsum = 0.f;
        for (int v = threadIdx.x; v < nvec; v += 256) {
            const vecX g = ld_vec(dout + base + (size_t)v * VN), x = ld_vec(inp + base + (size_t)v * VN), w = ld_vec(weight + (size_t)v * VN);
#pragma unroll
            for (int k = 0; k < VN; k++) {
                const float nh = (to_f32(x[k]) - m) * r, dn = to_f32(w[k]) * to_f32(g[k]);
                a += dn;
                bsum += dn * nh;
            }
        }
        a = block_reduce<false>(a, red) * invC;
        bsum = block_reduce<false>(bsum, red + 16) * invC;
        for (int v = threadIdx.x; v < nvec; v += 256) {
            const vecX g = ld_vec(dout + base + (size_t)v * VN), x = ld_vec(inp + base + (size_t)v * VN), w = ld_vec(weight + (size_t)v * VN);
            const vecX di = ld_vec(dinp + base + (size_t)v * VN);
            vecX o;
#pragma unroll
            for (int k = 0; k < VN; k++) {
                const float gk = to_f32(g[k]);
                const float nh = (to_f32(x[k]) - m) * r, dn = to_f32(w[k]) * gk;
                sdb[v * VN + k] += gk;                        // column v * VN + k belongs to this thread alone
                sdw[v * VN + k] += nh * gk;
                o[k] = from_f32<floatX>(to_f32(di[k]) + (dn - a - nh * bsum) * r);
            }
            st_vec(dinp + base + (size_t)v * VN, o);
        }
        __syncthreads();                                      // the reduction slots are reused by the next row
    }
    float* out = partial + (size_t)blockIdx.x * 2 * C;
    for (int c = threadIdx.x; c < 2 * C; c += 256) out[c] = lds[c];
}

// dweight[c] += sum_blocks partial[b][0][c]; dbias likewise. A workgroup owns 32 columns; its 32 row
// groups each add every 32nd partial in ascending order, then the 32 sub-sums are added in group order:
// a fixed summation tree, so the result is reproducible, with 32x the memory parallelism of one thread
// per column.
constexpr int LNR_COLS = 32, LNR_GROUPS = 32;
__global__ void __launch_bounds__(LNR_COLS * LNR_GROUPS)
ln_backward_reduce_kernel(floatX* __restrict__ dweight, floatX* __restrict__ dbias, const float* __restrict__ partial,
                          int nblocks, int C) {
    __shared__ float sub[LNR_GROUPS][LNR_COLS];
    const int cl = threadIdx.x % LNR_COLS, grp = threadIdx.x / LNR_COLS;
    const int c = blockIdx.x * LNR_COLS + cl;
    float s = 0.f;
    if (c < 2 * C)
        for (int b = grp; b < nblocks; b += LNR_GROUPS) s += partial[(size_t)b * 2 * C + c];
    sub[grp][cl] = s;
    __syncthreads();
    if (grp == 0 && c < 2 * C) {
        float t = 0.f;
#pragma unroll
        for (int g2 = 0; g2 < LNR_GROUPS; g2++) t += sub[g2][cl];
        floatX* dst = c < C ? dweight + c : dbias + (c - C);
        *dst = from_f32<floatX>(to_f32(*dst) + t);
    }
}

int ln_backward_blocks() { return llmk::device_info().num_cu; }

}  // namespace

extern "C" {

void llmk_layernorm_forward(void* out, float* mean, float* rstd, const void* inp, const void* weight,
                            const void* bias, int B, int T, int C, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(C > 0 && C % VN == 0, "layernorm_forward: C=%d must be a multiple of %d", C, VN);
    if ((size_t)B * T == 0) return;
    launch_ln_forward<false>((floatX*)out, nullptr, mean, rstd, (const floatX*)inp, nullptr, (const floatX*)weight,
                             (const floatX*)bias, B * T, C, (hipStream_t)stream);
}

void llmk_fused_residual_forward5(void* residual, void* normed, float* mean, float* rstd, const void* inp1,
                                  const void* inp2, const void* weight, const void* bias, int N, int C,
                                  void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(C > 0 && C % VN == 0, "fused_residual_forward5: C=%d must be a multiple of %d", C, VN);
    if (N == 0) return;
    launch_ln_forward<true>((floatX*)normed, (floatX*)residual, mean, rstd, (const floatX*)inp1, (const floatX*)inp2,
                            (const floatX*)weight, (const floatX*)bias, N, C, (hipStream_t)stream);
}

void llmk_residual_forward(void* out, const void* inp1, const void* inp2, int N, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(N % VN == 0, "residual_forward: N=%d must be a multiple of %d", N, VN);
    if (N == 0) return;
    size_t nvec = (size_t)N / VN;
    llmk::ProfScope prof("residual_forward", 0, 3.0 * N * sizeof(floatX), (hipStream_t)stream);
    residual_kernel<<<(unsigned)CEIL_DIV(nvec, (size_t)256), 256, 0, (hipStream_t)stream>>>(
        (floatX*)out, (const floatX*)inp1, (const floatX*)inp2, nvec);
    LAUNCH_CHECK();
}

size_t llmk_layernorm_backward_scratch_floats(int C) { return (size_t)ln_backward_blocks() * 2 * C; }

void llmk_layernorm_backward(void* dinp, void* dweight, void* dbias, float* scratch, const void* dout,
                             const void* inp, const void* weight, const float* mean, const float* rstd, int B,
                             int T, int C, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(C > 0 && C % VN == 0, "layernorm_backward: C=%d must be a multiple of %d", C, VN);
    const int nv = CEIL_DIV(C / VN, 64);
    const int N = B * T;
    if (N == 0) return;
    hipStream_t st = (hipStream_t)stream;
    if (nv > 8) {                                             // wider than the register-resident kernel takes
        const size_t smem = (2 * (size_t)C + 32) * sizeof(float);
        LLMK_REQUIRE(smem <= 160 * 1024, "layernorm_backward: C=%d too large (max %d)", C, (160 * 1024 / 4 - 32) / 2);
        const int blocks = min(ln_backward_blocks(), N);
        {
            llmk::ProfScope prof("layernorm_backward", 0, 4.0 * N * C * sizeof(floatX) + 2.0 * N * sizeof(float), st);
            static bool attr_set = false;
            if (!attr_set) {
                HIP_CHECK(hipFuncSetAttribute((const void*)ln_backward_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
                attr_set = true;
            }
            ln_backward_wide_kernel<<<blocks, 256, smem, st>>>((floatX*)dinp, scratch, (const floatX*)dout, (const floatX*)inp,
                                                             (const floatX*)weight, mean, rstd, N, C);
            LAUNCH_CHECK();
        }
        llmk::ProfScope prof2("layernorm_backward_reduce", 0, (double)blocks * 2 * C * sizeof(float), st);
        ln_backward_reduce_kernel<<<CEIL_DIV(2 * C, LNR_COLS), LNR_COLS * LNR_GROUPS, 0, st>>>((floatX*)dweight, (floatX*)dbias, scratch, blocks, C);
        LAUNCH_CHECK();
        return;
    }
    const int waves = lnb_waves(nv);
    const int blocks = min(ln_backward_blocks(), CEIL_DIV(N, waves));
    const size_t smem = (size_t)(waves - 1) * 2 * C * sizeof(float);
    {
    llmk::ProfScope prof("layernorm_backward", 0, 4.0 * N * C * sizeof(floatX) + 2.0 * N * sizeof(float), st);
#define LNB_CASE(K)                                                                                          \
    case K: {                                                                                                \
        static bool attr_set = false;                                                                        \
        if (!attr_set) {                                                                                     \
            HIP_CHECK(hipFuncSetAttribute((const void*)ln_backward_kernel<K>,                                \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));          \
            attr_set = true;                                                                                 \
        }                                                                                                    \
        ln_backward_kernel<K><<<blocks, lnb_waves(K) * 64, smem, st>>>((floatX*)dinp, scratch, (const floatX*)dout, \
                                                              (const floatX*)inp, (const floatX*)weight,    \
                                                              mean, rstd, N, C);                             \
        break; }
    switch (nv) { LNB_CASE(1) LNB_CASE(2) LNB_CASE(3) LNB_CASE(4) LNB_CASE(5) LNB_CASE(6) LNB_CASE(7) LNB_CASE(8) }
#undef LNB_CASE
    LAUNCH_CHECK();
    }
    llmk::ProfScope prof2("layernorm_backward_reduce", 0, (double)blocks * 2 * C * sizeof(float), st);
    ln_backward_reduce_kernel<<<CEIL_DIV(2 * C, LNR_COLS), LNR_COLS * LNR_GROUPS, 0, st>>>((floatX*)dweight, (floatX*)dbias, scratch, blocks, C);
    LAUNCH_CHECK();
}

}  // extern "C"
