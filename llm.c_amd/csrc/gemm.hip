// Dense contractions of the GPT-2 step on gfx950 matrix cores: matmul_forward / matmul_backward
// (reference launchers llmc/matmul.cuh:231 and :244, which hand the work to cuBLASLt; CPU
// definition train_gpt2.c:163-269).
//
//   forward   out[M,OC]  = inp[M,C] . W[OC,C]^T (+bias) (+GELU)      "NT": both operands K-contiguous
//   dinp      dinp[M,C]  = dout[M,OC] . W[OC,C]      (* gelu')        "NN": B stored K-major
//   dweight   dW[OC,C]  += dout[M,OC]^T . inp[M,C]                    "TN": both stored K-major, K = M = B*T
//
// bf16 build: one kernel template. A workgroup owns a BM x BN tile of C and walks K in steps
// of 64: global -> registers -> LDS (double-buffered, one barrier per step), LDS -> MFMA
// operands, v_mfma_f32_32x32x16_bf16 with fp32 accumulators.
//   * K-contiguous operands sit in LDS as [row][64] with the eight 16-byte chunks of a row
//     XOR-swizzled by (row & 7): both the 16-byte writes and the ds_read_b128 operand reads
//     are bank-conflict free without padding.
//   * K-major operands (the weight in dinp, both operands in dweight) sit in LDS as they are
//     in memory, [k][row] with a padded pitch, and are turned into MFMA operand layout by the
//     gfx950 transposing LDS read (ds_read_b64_tr_b16): 16 lanes fetch a 4(k) x 16(row) patch
//     and each lane receives the 4 k-values of its row. No software transpose anywhere.
//   * Workgroup ids are remapped so that consecutive tiles land on the same XCD (ids are dealt
//     round-robin over the 8 XCDs, each with a private L2) and walk the tile grid in groups of
//     8 row-tiles, so an XCD's 32 resident tiles share operand panels through its L2.
//   * dweight has few output tiles (27 for 2304x768) but K = 65536: the contraction is split
//     over workgroups, partials go to the library workspace in fp32 and are added in split
//     order by a second kernel (deterministic; no atomics), which also does the += into dW.
// fp32 build: same structure with v_mfma_f32_32x32x2_f32 (true fp32 multiply-add), the mode
// used for 1e-5 parity against the CPU reference.
#include "common.hpp"
#include "gelu.hpp"
#include "gemm_pipelined.hpp"
#include <vector>
#include <algorithm>
#include "../../include/llmk.h"

namespace {
using namespace gemmk;

constexpr int GROUP_M = 8;

__device__ __forceinline__ void tile_coords(int tiles_m, int tiles_n, int& tm, int& tn) {
    int pid = blockIdx.x;
    const int nblk = gridDim.x;
    if ((nblk & 7) == 0) pid = (pid & 7) * (nblk >> 3) + (pid >> 3);   // same-XCD ids become consecutive
    const int per_group = GROUP_M * tiles_n;
    const int group = pid / per_group;
    const int first_m = group * GROUP_M;
    const int gsz = min(tiles_m - first_m, GROUP_M);
    const int in_group = pid - group * per_group;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

template <int EPI>
__device__ __forceinline__ void epilogue_store(const GemmArgs& g, int m, int n, float v, float bias_n) {
    const size_t idx = (size_t)m * g.ldc + n;
    if (EPI == EPI_BIAS) {
        g.C[idx] = from_f32<floatX>(v + bias_n);
    } else if (EPI == EPI_BIAS_GELU) {
        floatX pre = from_f32<floatX>(v + bias_n);
        g.aux[idx] = pre;
        g.C[idx] = from_f32<floatX>(gelu_f(to_f32(pre)));   // GELU of the rounded pre-activation, as a separate kernel would see it
    } else if (EPI == EPI_STORE) {
        g.C[idx] = from_f32<floatX>(v);
    } else if (EPI == EPI_DGELU) {
        g.C[idx] = from_f32<floatX>(gelu_grad_f(to_f32(g.aux[idx])) * to_f32(from_f32<floatX>(v)));
    } else if (EPI == EPI_ACCUM) {
        g.C[idx] = from_f32<floatX>(to_f32(g.C[idx]) + v);
    } else {
        g.partial[((size_t)blockIdx.y * g.M + m) * g.N + n] = v;
    }
}

#if !defined(LLMK_FP32)
// =============================================================================================
// bf16 MFMA kernel
// =============================================================================================
constexpr int BK = 64;

template <int R, bool TRANS> struct TileLayout;
template <int R> struct TileLayout<R, false> {           // [R][64] bf16, chunk-swizzled
    static constexpr int BYTES = R * 128;
};
template <int R> struct TileLayout<R, true> {            // [64][R] bf16, padded pitch
    static constexpr int PITCH = R * 2 + 64;
    static constexpr int BYTES = 64 * PITCH;
};

// Per-thread description of the 16-byte chunks it moves for one operand tile.
template <int R, bool TRANS, int NT>
struct Loader {
    static constexpr int NCH = R * 8 / NT;               // chunks per thread
    const floatX* gptr[NCH];                             // address at k0 = 0 (or nullptr-equivalent when masked)
    int lds_off[NCH];
    bool ok[NCH];
    int kidx[NCH];                                       // k offset of the chunk inside the tile (for the K tail)
    size_t kstride;                                      // elements to advance per K step

    __device__ __forceinline__ void init(const floatX* base, int ld, int r0, int rmax, int tid) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int q = tid + i * NT;
            if (!TRANS) {
                const int row = q >> 3, c = q & 7;
                ok[i] = (r0 + row) < rmax;
                gptr[i] = base + (size_t)(r0 + row) * ld + c * 8;
                lds_off[i] = row * 128 + ((c ^ (row & 7)) << 4);
                kidx[i] = c * 8;
            } else {
                constexpr int CPR = R / 8;               // chunks per k-row
                const int krow = q / CPR, cc = q % CPR;
                ok[i] = (r0 + cc * 8) < rmax;
                gptr[i] = base + (size_t)krow * ld + r0 + cc * 8;
                lds_off[i] = krow * TileLayout<R, true>::PITCH + cc * 16;
                kidx[i] = krow;
            }
        }
        kstride = TRANS ? (size_t)BK * ld : (size_t)BK;
    }
    __device__ __forceinline__ void load(u32x4 (&reg)[NCH], int kt, int k0, int kend) const {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const bool p = ok[i] && (k0 + kidx[i] < kend);
            u32x4 z = {0, 0, 0, 0};
            reg[i] = p ? *reinterpret_cast<const u32x4*>(gptr[i] + (size_t)kt * kstride) : z;
        }
    }
    __device__ __forceinline__ void store(char* lds, const u32x4 (&reg)[NCH]) const {
#pragma unroll
        for (int i = 0; i < NCH; i++) *reinterpret_cast<u32x4*>(lds + lds_off[i]) = reg[i];
    }
};

// MFMA operand (32 rows x 16 k) for k-step s of the tile, rows [row0, row0+32)
template <int R, bool TRANS>
__device__ __forceinline__ bf16x8 read_frag(const char* lds, int row0, int s, int lane) {
    if (!TRANS) {
        const int row = row0 + (lane & 31);
        const int c = 2 * s + (lane >> 5);
        return *reinterpret_cast<const bf16x8*>(lds + row * 128 + ((c ^ (row & 7)) << 4));
    } else {
        constexpr int PITCH = TileLayout<R, true>::PITCH;
        const int s16 = lane & 15, grp = lane >> 4;
        const int krow = 16 * s + 8 * (grp >> 1) + (s16 >> 2);
        const int col = row0 + (grp & 1) * 16 + 4 * (s16 & 3);
        const char* p = lds + krow * PITCH + col * 2;
        typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * PITCH));
        union { struct { s16x4 a, b; } s; bf16x8 v; } u;
        u.s.a = lo; u.s.b = hi;
        return u.v;
    }
}

template <int BM, int BN, int WGM, int WGN, bool A_T, bool B_T, int EPI>
__global__ void __launch_bounds__(WGM * WGN * 64)
gemm_bf16_kernel(GemmArgs g) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_BYTES = TileLayout<BM, A_T>::BYTES, B_BYTES = TileLayout<BN, B_T>::BYTES;
    constexpr int STAGE = A_BYTES + B_BYTES;
    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    int tile_m, tile_n;
    tile_coords(CEIL_DIV(g.M, BM), CEIL_DIV(g.N, BN), tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int kbeg = blockIdx.y * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);
    const int KT = CEIL_DIV(kend - kbeg, BK);

    Loader<BM, A_T, NT> la;
    Loader<BN, B_T, NT> lb;
    la.init(g.A + (A_T ? (size_t)kbeg * g.lda : (size_t)kbeg), g.lda, m0, g.M, tid);
    lb.init(g.B + (B_T ? (size_t)kbeg * g.ldb : (size_t)kbeg), g.ldb, n0, g.N, tid);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    u32x4 ra[Loader<BM, A_T, NT>::NCH], rb[Loader<BN, B_T, NT>::NCH];
    if (KT > 0) {
        la.load(ra, 0, kbeg, kend);
        lb.load(rb, 0, kbeg, kend);
        la.store(lds, ra);
        lb.store(lds + A_BYTES, rb);
    }
    __syncthreads();

    for (int kt = 0; kt < KT; kt++) {
        const char* cur = lds + (kt & 1) * STAGE;
        char* nxt = lds + ((kt + 1) & 1) * STAGE;
        const bool more = kt + 1 < KT;
        if (more) {
            la.load(ra, kt + 1, kbeg + (kt + 1) * BK, kend);
            lb.load(rb, kt + 1, kbeg + (kt + 1) * BK, kend);
        }
#pragma unroll
        for (int s = 0; s < BK / 16; s++) {
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) fa[i] = read_frag<BM, A_T>(cur, wm * WTM + i * 32, s, lane);
#pragma unroll
            for (int j = 0; j < TN; j++) fb[j] = read_frag<BN, B_T>(cur + A_BYTES, wn * WTN + j * 32, s, lane);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            la.store(nxt, ra);
            lb.store(nxt + A_BYTES, rb);
        }
        __syncthreads();
    }

    // epilogue: lane holds column (lane & 31) and rows (r/4)*8 + (lane>>5)*4 + r%4 of each 32x32 tile
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + wn * WTN + j * 32 + (lane & 31);
        if (n >= g.N) continue;
        float bias_n = 0.f;
        if ((EPI == EPI_BIAS || EPI == EPI_BIAS_GELU) && g.bias) bias_n = to_f32(g.bias[n]);
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int mb = m0 + wm * WTM + i * 32 + (lane >> 5) * 4;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = mb + (r >> 2) * 8 + (r & 3);
                if (m < g.M) epilogue_store<EPI>(g, m, n, acc[i][j][r], bias_n);
            }
        }
    }
}

template <int BM, int BN, int WGM, int WGN, bool A_T, bool B_T, int EPI>
void launch_bf16(const GemmArgs& g, int splits, hipStream_t st) {
    constexpr int SMEM = 2 * (TileLayout<BM, A_T>::BYTES + TileLayout<BN, B_T>::BYTES);
    auto kern = gemm_bf16_kernel<BM, BN, WGM, WGN, A_T, B_T, EPI>;
    static bool attr_set = false;
    if (!attr_set) {
        HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM));
        attr_set = true;
    }
    dim3 grid(CEIL_DIV(g.M, BM) * CEIL_DIV(g.N, BN), splits);
    kern<<<grid, WGM * WGN * 64, SMEM, st>>>(g);
    LAUNCH_CHECK();
}

template <bool A_T, bool B_T, int EPI>
void launch_gemm(const GemmArgs& g, int splits, bool big, hipStream_t st) {
    if (big) launch_bf16<256, 256, 2, 4, A_T, B_T, EPI>(g, splits, st);
    else launch_bf16<128, 128, 2, 2, A_T, B_T, EPI>(g, splits, st);
}
constexpr int K_ALIGN = 8;       // K-contiguous rows are read in 16-byte chunks
constexpr int BIG_TILE = 256, SMALL_TILE = 128, K_STEP = 64;

// Persistent direct-to-LDS kernel (gemm_pipelined.hpp). Preconditions: K and the per-split K multiples of 32,
// leading dimensions and N multiples of 8, 16-byte aligned operands, 8-byte aligned bias.
bool pipelined_ok(const GemmArgs& g) {
    auto al = [](const void* p, uintptr_t a) { return ((uintptr_t)p % a) == 0; };
    return g.K % KGRAN == 0 && g.k_per_split % KGRAN == 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 && g.ldc % 8 == 0 &&
           g.N % 8 == 0 && al(g.A, 16) && al(g.B, 16) && al(g.C, 16) && (!g.bias || al(g.bias, 8)) && (!g.aux || al(g.aux, 16));
}
// The pipelined kernel's += epilogue spills registers (it holds the old values of a whole tile); with it available,
// a single "split" written as fp32 partials and folded in by the reduce pass is 30 % faster than accumulating in place.
bool tn_partial_always(const GemmArgs& g) { return pipelined_ok(g); }
template <int BM, int BN, int WGM, int WGN, bool A_T, bool B_T, int EPI>
void launch_pipelined_cfg(GemmArgs g, int splits, hipStream_t st) {
    constexpr int NW = WGM * WGN;
    constexpr int SMEM = gemmk::smem_bytes(BM, BN, NW);
    auto kern = gemm_pipelined_kernel<BM, BN, WGM, WGN, A_T, B_T, EPI>;
    static bool attr_set = false;
    if (!attr_set) {
        HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM));
        attr_set = true;
    }
    g.splits = splits;
    const int work = CEIL_DIV(g.M, BM) * CEIL_DIV(g.N, BN) * splits;
    const int grid = min((work + 7) & ~7, llmk::device_info().num_cu & ~7);   // a multiple of 8: one share per XCD
    kern<<<grid, NW * 64, SMEM, st>>>(g);
    LAUNCH_CHECK();
}
template <bool A_T, bool B_T, int EPI>
void launch_pipelined(const GemmArgs& g, int splits, bool big, hipStream_t st) {
    if constexpr (A_T && B_T) {                          // the weight gradient's kernels: compiled in gemm_tn.hip
        launch_pipelined_tn(g, splits, big, EPI, 0, st);
    } else {
        if (big) launch_pipelined_cfg<256, 256, 2, 4, A_T, B_T, EPI>(g, splits, st);
        else launch_pipelined_cfg<128, 128, 2, 2, A_T, B_T, EPI>(g, splits, st);
    }
}
// pipelined kernel when its preconditions hold, generic kernel otherwise
template <bool A_T, bool B_T, int EPI>
void launch_best(const GemmArgs& g, int splits, bool big, hipStream_t st) {
    if (pipelined_ok(g)) launch_pipelined<A_T, B_T, EPI>(g, splits, big, st);
    else launch_gemm<A_T, B_T, EPI>(g, splits, big, st);
}

#else
// =============================================================================================
// fp32 MFMA kernel (parity mode): 128x128 tile, K step 16, 4 waves of 64x64
// =============================================================================================
constexpr int FBM = 128, FBN = 128, FBK = 16;
constexpr int F_PITCH_K = FBK + 4;       // [row][k] tiles, 16-byte aligned rows
constexpr int F_PITCH_T = 128 + 4;       // [k][row] tiles

template <bool A_T, bool B_T, int EPI>
__global__ void __launch_bounds__(256)
gemm_f32_kernel(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) float sA[2][A_T ? FBK * F_PITCH_T : FBM * F_PITCH_K];
    __shared__ __attribute__((aligned(16))) float sB[2][B_T ? FBK * F_PITCH_T : FBN * F_PITCH_K];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tile_m, tile_n;
    tile_coords(CEIL_DIV(g.M, FBM), CEIL_DIV(g.N, FBN), tile_m, tile_n);
    const int m0 = tile_m * FBM, n0 = tile_n * FBN;
    const int kbeg = blockIdx.y * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);
    const int KT = CEIL_DIV(kend - kbeg, FBK);

    // each thread moves 2 float4 per operand tile (128*16/4 = 512 float4)
    auto load_tile = [&](const float* base, int ld, bool trans, int r0, int rmax, int k0, vecF (&reg)[2]) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int q = tid + i * 256;
            vecF z; z[0] = z[1] = z[2] = z[3] = 0.f;
            if (!trans) {
                const int row = q >> 2, c = (q & 3) * 4;
                const bool p = (r0 + row < rmax) && (k0 + c < kend);
                reg[i] = p ? ld_vec(base + (size_t)(r0 + row) * ld + k0 + c) : z;
            } else {
                const int krow = q >> 5, c = (q & 31) * 4;
                const bool p = (k0 + krow < kend) && (r0 + c < rmax);
                reg[i] = p ? ld_vec(base + (size_t)(k0 + krow) * ld + r0 + c) : z;
            }
        }
    };
    auto store_tile = [&](float* s, bool trans, const vecF (&reg)[2]) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int q = tid + i * 256;
            if (!trans) st_vec(s + (q >> 2) * F_PITCH_K + (q & 3) * 4, reg[i]);
            else st_vec(s + (q >> 5) * F_PITCH_T + (q & 31) * 4, reg[i]);
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    vecF ra[2], rb[2];
    if (KT > 0) {
        load_tile(g.A, g.lda, A_T, m0, g.M, kbeg, ra);
        load_tile(g.B, g.ldb, B_T, n0, g.N, kbeg, rb);
        store_tile(sA[0], A_T, ra);
        store_tile(sB[0], B_T, rb);
    }
    __syncthreads();
    for (int kt = 0; kt < KT; kt++) {
        const int cur = kt & 1;
        const bool more = kt + 1 < KT;
        if (more) {
            load_tile(g.A, g.lda, A_T, m0, g.M, kbeg + (kt + 1) * FBK, ra);
            load_tile(g.B, g.ldb, B_T, n0, g.N, kbeg + (kt + 1) * FBK, rb);
        }
#pragma unroll
        for (int s = 0; s < FBK / 2; s++) {
            const int k = 2 * s + (lane >> 5);
            float fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int row = wm * 64 + i * 32 + (lane & 31);
                fa[i] = A_T ? sA[cur][k * F_PITCH_T + row] : sA[cur][row * F_PITCH_K + k];
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int row = wn * 64 + j * 32 + (lane & 31);
                fb[j] = B_T ? sB[cur][k * F_PITCH_T + row] : sB[cur][row * F_PITCH_K + k];
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            store_tile(sA[cur ^ 1], A_T, ra);
            store_tile(sB[cur ^ 1], B_T, rb);
        }
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int n = n0 + wn * 64 + j * 32 + (lane & 31);
        if (n >= g.N) continue;
        float bias_n = 0.f;
        if ((EPI == EPI_BIAS || EPI == EPI_BIAS_GELU) && g.bias) bias_n = g.bias[n];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int mb = m0 + wm * 64 + i * 32 + (lane >> 5) * 4;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = mb + (r >> 2) * 8 + (r & 3);
                if (m < g.M) epilogue_store<EPI>(g, m, n, acc[i][j][r], bias_n);
            }
        }
    }
}

template <bool A_T, bool B_T, int EPI>
void launch_gemm(const GemmArgs& g, int splits, bool /*big*/, hipStream_t st) {
    dim3 grid(CEIL_DIV(g.M, FBM) * CEIL_DIV(g.N, FBN), splits);
    gemm_f32_kernel<A_T, B_T, EPI><<<grid, 256, 0, st>>>(g);
    LAUNCH_CHECK();
}
constexpr int K_ALIGN = 4;
constexpr int BIG_TILE = 128, SMALL_TILE = 128, K_STEP = 16;
template <bool A_T, bool B_T, int EPI>
void launch_best(const GemmArgs& g, int splits, bool big, hipStream_t st) { launch_gemm<A_T, B_T, EPI>(g, splits, big, st); }
bool tn_partial_always(const GemmArgs&) { return false; }
#endif

// C[m][n] (+)= sum over splits of partial[s][m][n], in split order. Workgroups past the ones that cover C add up the
// row sums of EPI_PARTIAL_ROWSUM: rowvec[m] += sum over parts of rowsum[p][m], 32 rows per workgroup, 8 groups of lanes
// each adding every 8th part, then the 8 sub-sums in group order (a fixed tree, like bias_grad_reduce_kernel).
constexpr int SKR_ROWS = 32, SKR_GROUPS = 8;
template <bool ACCUM>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(floatX* __restrict__ C, const float* __restrict__ partial, size_t mn, int splits,
                     floatX* __restrict__ rowvec, const float* __restrict__ rowsum, int rows, int parts, unsigned main_blocks) {
    if (blockIdx.x >= main_blocks) {                      // workgroup-uniform
        __shared__ float sub[SKR_GROUPS][SKR_ROWS];
        const int rl = threadIdx.x % SKR_ROWS, grp = threadIdx.x / SKR_ROWS;
        const int m = (int)(blockIdx.x - main_blocks) * SKR_ROWS + rl;
        float t = 0.f;
        if (m < rows)
            for (int p = grp; p < parts; p += SKR_GROUPS) t += rowsum[(size_t)p * rows + m];
        sub[grp][rl] = t;
        __syncthreads();
        if (grp == 0 && m < rows) {
            float u = 0.f;
#pragma unroll
            for (int g2 = 0; g2 < SKR_GROUPS; g2++) u += sub[g2][rl];
            rowvec[m] = from_f32<floatX>(to_f32(rowvec[m]) + u);
        }
        return;
    }
    size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= mn) return;
    vecF s = ld_vec(partial + i);
    for (int k = 1; k < splits; k++) {
        vecF p = ld_vec(partial + (size_t)k * mn + i);
#pragma unroll
        for (int e = 0; e < 4; e++) s[e] += p[e];
    }
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float base = ACCUM ? to_f32(C[i + e]) : 0.f;
        C[i + e] = from_f32<floatX>(base + s[e]);
    }
}

#if !defined(LLMK_FP32)
// Cutting the weight gradient's contraction when its T tiles are a sizable part of the G workgroups (GPT-2 1558M at B*T =
// 16384: 133-175 tiles of 256 x 256 for 256 CUs). Equal splits fill the launch only at 4-5 per tile, and each split costs a
// pass of fp32 partials over the output. Here every tile is cut at the SAME K positions into one long piece and s - 1
// short ones: T workgroups take a long piece each, the other G - T take p short pieces each, and the cut is placed where
// both finish together (long = p x short). The pieces that run side by side still cover the same K range, so the 32 CUs
// of an XCD go on sharing operand panels through their L2 (handing out contiguous (tile, K) ranges of equal length
// instead, each workgroup at its own K offset, left every panel to be streamed once per tile: slower than the equal
// splits). Partial slot = rank of the piece along K, so the sum order is fixed.
constexpr int SK_MIN_BLOCKS = 4;
int g_sk_mode = -1;                  // llmk_matmul_backward_split_mode
struct SkPlan {
    int slots = 0;                   // pieces per tile
    int long_blocks = 0;             // K blocks of the long piece
    int each = 0;                    // short pieces per workgroup
    double cost = 1e30;              // launch time in units of the perfectly balanced GEMM, partial passes included
    bool valid = false;
};
// Pure arithmetic on the shape: nothing is allocated or copied, the kernel derives each workgroup's pieces from
// (tiles, long_blocks, each, slots) by the same enumeration (gemm_pipelined.hpp, work_item).
SkPlan sk_build(int tiles_m, int tiles_n, int kblocks, int G, double pass) {
    SkPlan p;
    const int T = tiles_m * tiles_n, S = kblocks;
    if (T >= G || T * 8 < G) return p;
    for (int s = 2; s <= 6; s++) {
        const int ny = T * (s - 1), p_each = CEIL_DIV(ny, G - T);
        if (p_each > SK_MAX_ITEMS) continue;
        int x = (int)((long long)p_each * S / (s - 1 + p_each));           // long piece = p short ones
        const int y_max = CEIL_DIV(S - x, s - 1), y_min = (S - x) / (s - 1);
        if (x < SK_MIN_BLOCKS || y_min < SK_MIN_BLOCKS) continue;
        const int makespan = std::max(x, p_each * y_max);
        const double cost = (double)makespan * G / ((double)T * S) + pass * s;
        if (cost < p.cost) { p.cost = cost; p.slots = s; p.long_blocks = x; p.each = p_each; p.valid = true; }
    }
    return p;
}
#endif

// Equal splits of the weight gradient's K = B*T so that the work items fill whole rounds of the persistent launch (27
// tiles -> 9 splits = 243 items on 256 CUs; 591 tiles -> 3 splits, 1773 items = 6.9 rounds instead of 3 rounds at 77 %;
// 175 tiles -> 4 splits). Each split costs one fp32 pass over the output (8 bytes per element written and read back,
// against 2*M flop per element in the GEMM): 800/M of the GEMM's time at the rates measured, 1.2 % at M = 65536.
int tn_equal_splits(int M, size_t tiles, int num_cu, double* cost_out) {
    int splits = 1;
    double best = 1e30;
    const double pass = 800.0 / (double)M;
    for (int s = 1; s <= 32; s++) {
        const size_t work = tiles * s, rounds = CEIL_DIV(work, (size_t)num_cu);
        const double cost = (double)(rounds * num_cu) / (double)work + pass * s;
        if (cost < best) { best = cost; splits = s; }
    }
    if (cost_out) *cost_out = best;
    const int ksteps = CEIL_DIV(M, K_STEP);
    splits = min(splits, max(1, ksteps / 8));                     // at least 8 K steps per split
    return CEIL_DIV(ksteps, CEIL_DIV(ksteps, splits));
}

// what the last weight-gradient GEMM did with K: 0 = not cut, 1 = equal splits, 2 = one long + short pieces
int g_last_split_kind = 0, g_last_split_pieces = 0;

// ---- bias gradient: column sums of dout[N][OC] -----------------------------------------------
// HBM-bound streaming reduction. Workgroup = 32 column-vectors (512 B of a row) x 8 row lanes; each lane keeps
// four row loads in flight. grid.y splits the rows so that ~2 workgroups per CU are resident; their partial sums
// go to the caller's fp32 scratch and are added in a fixed order by a second, tiny kernel (no atomics).
constexpr int VN = vecX::N;
// DGELU: dout is first multiplied in place by gelu'(pre) (rounded to the storage type, and it is the rounded value
// that is summed, so the result equals gelu_backward_inplace followed by the plain reduction).
constexpr int BG_COLV = 32, BG_ROWL = 8, BG_UNROLL = 4;
template <bool DGELU>
__global__ void __launch_bounds__(256)
bias_grad_kernel(float* __restrict__ partial, floatX* __restrict__ dout, const floatX* __restrict__ pre, int N, int OC) {
    __shared__ float red[BG_ROWL][BG_COLV * VN + 1];
    const int cv = threadIdx.x % BG_COLV, rl = threadIdx.x / BG_COLV;
    const int col = (blockIdx.x * BG_COLV + cv) * VN;
    float acc[VN];
#pragma unroll
    for (int k = 0; k < VN; k++) acc[k] = 0.f;
    if (col < OC) {
        const int rstep = gridDim.y * BG_ROWL;
        int r = blockIdx.y * BG_ROWL + rl;
        for (; r + (BG_UNROLL - 1) * rstep < N; r += BG_UNROLL * rstep) {
            vecX d[BG_UNROLL], x[BG_UNROLL];
#pragma unroll
            for (int u = 0; u < BG_UNROLL; u++) {
                d[u] = ld_vec_nt(dout + (size_t)(r + u * rstep) * OC + col);
                if (DGELU) x[u] = ld_vec_nt(pre + (size_t)(r + u * rstep) * OC + col);
            }
#pragma unroll
            for (int u = 0; u < BG_UNROLL; u++) {
                if (DGELU) {
#pragma unroll
                    for (int k = 0; k < VN; k++) d[u][k] = from_f32<floatX>(gelu_grad_f(to_f32(x[u][k])) * to_f32(d[u][k]));
                    st_vec(dout + (size_t)(r + u * rstep) * OC + col, d[u]);
                }
#pragma unroll
                for (int k = 0; k < VN; k++) acc[k] += to_f32(d[u][k]);
            }
        }
        for (; r < N; r += rstep) {
            vecX d = ld_vec_nt(dout + (size_t)r * OC + col);
            if (DGELU) {
                vecX x = ld_vec_nt(pre + (size_t)r * OC + col);
#pragma unroll
                for (int k = 0; k < VN; k++) d[k] = from_f32<floatX>(gelu_grad_f(to_f32(x[k])) * to_f32(d[k]));
                st_vec(dout + (size_t)r * OC + col, d);
            }
#pragma unroll
            for (int k = 0; k < VN; k++) acc[k] += to_f32(d[k]);
        }
    }
#pragma unroll
    for (int k = 0; k < VN; k++) red[rl][cv * VN + k] = acc[k];
    __syncthreads();
    for (int c = threadIdx.x; c < BG_COLV * VN; c += 256) {
        const int oc = blockIdx.x * BG_COLV * VN + c;
        if (oc < OC) {
            float s = 0.f;
#pragma unroll
            for (int r = 0; r < BG_ROWL; r++) s += red[r][c];
            partial[(size_t)blockIdx.y * OC + oc] = s;
        }
    }
}
// dbias[oc] += sum_y partial[y][oc]: 32 columns per workgroup, 8 groups each adding every 8th partial, then the
// 8 sub-sums in group order
constexpr int BGR_COLS = 32, BGR_GROUPS = 8;
__global__ void __launch_bounds__(BGR_COLS * BGR_GROUPS)
bias_grad_reduce_kernel(floatX* __restrict__ dbias, const float* __restrict__ partial, int OC, int ny) {
    __shared__ float sub[BGR_GROUPS][BGR_COLS];
    const int cl = threadIdx.x % BGR_COLS, grp = threadIdx.x / BGR_COLS;
    const int oc = blockIdx.x * BGR_COLS + cl;
    float s = 0.f;
    if (oc < OC)
        for (int y = grp; y < ny; y += BGR_GROUPS) s += partial[(size_t)y * OC + oc];
    sub[grp][cl] = s;
    __syncthreads();
    if (grp == 0 && oc < OC) {
        float t = 0.f;
#pragma unroll
        for (int g2 = 0; g2 < BGR_GROUPS; g2++) t += sub[g2][cl];
        dbias[oc] = from_f32<floatX>(to_f32(dbias[oc]) + t);
    }
}
int bias_grad_ny(int OC) {
    int gx = CEIL_DIV(OC, BG_COLV * VN);
    return max(1, llmk::device_info().num_cu * 2 / gx);
}

bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

#if !defined(LLMK_FP32)
// What the matrix cores deliver when nothing else is in the way: every wave issues independent chains of
// v_mfma_f32_32x32x16_bf16 on operands it holds in registers (non-trivial values: the clock the chip sustains depends on
// the data), two waves per SIMD.
__global__ void __launch_bounds__(512)
mfma_peak_kernel(float* __restrict__ sink, int iters) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int lane = threadIdx.x & 63;
    bf16x8 a, b;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        a[e] = (__bf16)(0.03125f * (float)(((lane * 8 + e) * 37 + blockIdx.x) % 61 - 30));
        b[e] = (__bf16)(0.0625f * (float)(((lane * 8 + e) * 53 + threadIdx.x) % 59 - 29));
    }
    f32x16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[c][r] = 0.f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) s += acc[c][r];
    if (s == 12345.678f) sink[0] = s;                                   // keeps the chains alive
#endif
}
#endif

}  // namespace

extern "C" {

void llmk_probe_mfma_peak(double* tflops, float* scratch, void* stream) {
    if (tflops) *tflops = 0.0;
#if !defined(LLMK_FP32)
    if (llmk::failed()) return;
    LLMK_REQUIRE(scratch != nullptr, "probe_mfma_peak: one float of device scratch is required");
    hipStream_t st = (hipStream_t)stream;
    const int num_cu = llmk::device_info().num_cu, iters = 16384;       // 16 MFMAs per iteration and wave
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    mfma_peak_kernel<<<num_cu, 512, 0, st>>>(scratch, 1024);            // warm-up: the clock settles under matrix load
    HIP_CHECK(hipEventRecord(e0, st));
    mfma_peak_kernel<<<num_cu, 512, 0, st>>>(scratch, iters);
    HIP_CHECK(hipEventRecord(e1, st));
    HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    HIP_CHECK(hipEventDestroy(e0));
    HIP_CHECK(hipEventDestroy(e1));
    const double flops = (double)num_cu * 8.0 * iters * 16.0 * 32768.0;    // 8 waves per workgroup, 2*32*32*16 flop per MFMA
    if (ms > 0.f && tflops) *tflops = flops / (ms * 1e-3) / 1e12;
#endif
}

void llmk_matmul_forward(void* out, const void* inp, const void* weight, const void* bias, int B, int T, int C,
                         int OC, void* stream, void* pre_gelu, int gelu_fusion) {
    if (llmk::failed()) return;
    const int M = B * T;
    LLMK_REQUIRE(C % K_ALIGN == 0, "matmul_forward: C=%d must be a multiple of %d", C, K_ALIGN);
    LLMK_REQUIRE(aligned16(inp) && aligned16(weight), "matmul_forward: operands must be 16-byte aligned");
    if (M == 0 || OC == 0) return;
    hipStream_t st = (hipStream_t)stream;
    GemmArgs g{};
    g.A = (const floatX*)inp; g.B = (const floatX*)weight; g.M = M; g.N = OC; g.K = C;
    g.lda = C; g.ldb = C; g.ldc = OC; g.bias = (const floatX*)bias; g.k_per_split = CEIL_DIV(C, K_STEP) * K_STEP;
    const int num_cu = llmk::device_info().num_cu;
    const bool big = (size_t)CEIL_DIV(M, BIG_TILE) * CEIL_DIV(OC, BIG_TILE) >= (size_t)num_cu;
    const bool gelu_in_gemm = pre_gelu && gelu_fusion >= 1;            // then the kernel writes two (M, OC) tensors
    llmk::ProfScope prof(gelu_in_gemm ? "gemm_nt_gelu" : "gemm_nt", 2.0 * M * (double)OC * C,
                         ((double)M * C + (double)OC * C + (gelu_in_gemm ? 2.0 : 1.0) * M * OC) * sizeof(floatX), st);
    if (pre_gelu && gelu_fusion >= 3) {
        // pre_gelu receives gelu'(pre-activation): in the direct-to-LDS kernel's epilogue, else by a pass of its own
        g.C = (floatX*)out; g.aux = (floatX*)pre_gelu;
#if !defined(LLMK_FP32)
        if (big && pipelined_ok(g)) {
            launch_pipelined_cfg<256, 256, 2, 4, false, false, EPI_BIAS_GELU_D>(g, 1, st);
            return;
        }
#endif
        g.C = (floatX*)pre_gelu; g.aux = nullptr;
        launch_best<false, false, EPI_BIAS>(g, 1, big, st);
        if (prof.on) { llmk::prof_end(st); prof.on = false; }
        llmk_gelu_forward_keep_grad(out, pre_gelu, M * OC, stream);
    } else if (pre_gelu && gelu_fusion >= 1) {
        g.C = (floatX*)out; g.aux = (floatX*)pre_gelu;
        launch_best<false, false, EPI_BIAS_GELU>(g, 1, big, st);
    } else if (pre_gelu) {
        g.C = (floatX*)pre_gelu;
        launch_best<false, false, EPI_BIAS>(g, 1, big, st);
        if (prof.on) { llmk::prof_end(st); prof.on = false; }
        llmk_gelu_forward(out, pre_gelu, M * OC, stream);
    } else {
        g.C = (floatX*)out;
        if (bias) launch_best<false, false, EPI_BIAS>(g, 1, big, st);
        else launch_best<false, false, EPI_STORE>(g, 1, big, st);     // the LM head: no bias to fetch, no window to keep for it
    }
}

void llmk_gelu_backward_bias(void* d_in_out, const void* inp, void* dbias, float* dbias_buffer, int B, int T, int OC,
                             void* stream) {
    if (llmk::failed()) return;
    const int M = B * T;
    LLMK_REQUIRE(OC > 0 && OC % VN == 0, "gelu_backward_bias: OC=%d must be a multiple of %d", OC, VN);
    LLMK_REQUIRE(aligned16(d_in_out) && aligned16(inp), "gelu_backward_bias: pointers must be 16-byte aligned");
    if (M == 0) return;
    hipStream_t st = (hipStream_t)stream;
    const int ny = bias_grad_ny(OC);
    llmk::ProfScope prof("gelu_backward_bias", 0, 3.0 * M * OC * sizeof(floatX), st);
    bias_grad_kernel<true><<<dim3(CEIL_DIV(OC, BG_COLV * VN), ny), 256, 0, st>>>(dbias_buffer, (floatX*)d_in_out, (const floatX*)inp, M, OC);
    LAUNCH_CHECK();
    bias_grad_reduce_kernel<<<CEIL_DIV(OC, BGR_COLS), BGR_COLS * BGR_GROUPS, 0, st>>>((floatX*)dbias, dbias_buffer, OC, ny);
    LAUNCH_CHECK();
}

size_t llmk_matmul_backward_bias_scratch_floats(int OC) { return (size_t)bias_grad_ny(OC) * OC; }

void llmk_matmul_backward_split_mode(int mode) {
#if !defined(LLMK_FP32)
    g_sk_mode = mode < 0 ? -1 : mode > 0 ? 1 : 0;
#else
    (void)mode;                          // the fp32 library has one weight-gradient path
#endif
}

void llmk_matmul_backward_last_split(int* kind, int* pieces) {
    if (kind) *kind = g_last_split_kind;
    if (pieces) *pieces = g_last_split_pieces;
}

size_t llmk_matmul_backward_workspace_bytes(int B, int T, int C, int OC) {
    const int M = B * T, num_cu = llmk::device_info().num_cu;
    if (M <= 0 || C <= 0 || OC <= 0) return 0;
    const size_t tiles_big = (size_t)CEIL_DIV(OC, BIG_TILE) * CEIL_DIV(C, BIG_TILE);
    const size_t tiles_small = (size_t)CEIL_DIV(OC, SMALL_TILE) * CEIL_DIV(C, SMALL_TILE);
    int pieces = tn_equal_splits(M, tiles_big >= 8 ? tiles_big : tiles_small, num_cu, nullptr);
#if !defined(LLMK_FP32)
    if (tiles_big >= 8 && M % K_STEP == 0) {
        const SkPlan plan = sk_build(CEIL_DIV(OC, BIG_TILE), CEIL_DIV(C, BIG_TILE), M / K_STEP, num_cu & ~7, 800.0 / (double)M);
        if (plan.valid) pieces = max(pieces, plan.slots);
    }
#endif
    return ((size_t)OC * C + (size_t)OC * 4) * pieces * sizeof(float);     // partial products + the bias gradient's row sums
}

// out = bf16(bf16(inp . weight^T + bias) + residual): the projection and the residual stream's add in one launch, with
// both roundings of the two-kernel form (llmk_matmul_forward, then llmk_residual_forward or llmk_fused_residual_forward5's
// add), so the bits are the same. out may be the residual buffer's successor or any other buffer; not inp.
void llmk_matmul_forward_residual(void* out, const void* inp, const void* weight, const void* bias, const void* residual,
                                  int B, int T, int C, int OC, void* stream) {
    if (llmk::failed()) return;
    const int M = B * T;
    LLMK_REQUIRE(C % K_ALIGN == 0, "matmul_forward_residual: C=%d must be a multiple of %d", C, K_ALIGN);
    LLMK_REQUIRE(aligned16(inp) && aligned16(weight), "matmul_forward_residual: operands must be 16-byte aligned");
    if (M == 0 || OC == 0) return;
    hipStream_t st = (hipStream_t)stream;
#if !defined(LLMK_FP32)
    GemmArgs g{};
    g.A = (const floatX*)inp; g.B = (const floatX*)weight; g.M = M; g.N = OC; g.K = C;
    g.lda = C; g.ldb = C; g.ldc = OC; g.bias = (const floatX*)bias; g.k_per_split = CEIL_DIV(C, K_STEP) * K_STEP;
    g.C = (floatX*)out; g.aux = (floatX*)residual;
    const bool big = (size_t)CEIL_DIV(M, BIG_TILE) * CEIL_DIV(OC, BIG_TILE) >= (size_t)llmk::device_info().num_cu;
    if (big && out != residual && aligned16(residual) && aligned16(out) && pipelined_ok(g)) {
        llmk::ProfScope prof("gemm_nt_res", 2.0 * M * (double)OC * C, ((double)M * C + (double)OC * C + 2.0 * M * OC) * sizeof(floatX), st);
        launch_pipelined_cfg<256, 256, 2, 4, false, false, EPI_BIAS_RES>(g, 1, st);
        return;
    }
#endif
    // shapes the fused epilogue does not take: the two kernels (out first holds the projection, then the sum; the add reads
    // and writes element by element, so in place is fine)
    LLMK_REQUIRE(out != residual, "matmul_forward_residual: out must not be the residual buffer");
    llmk_matmul_forward(out, inp, weight, bias, B, T, C, OC, stream, nullptr, 1);
    llmk_residual_forward(out, residual, out, M * OC, stream);
}

void llmk_matmul_backward(void* dinp, void* dweight, void* dbias, const void* dout, const void* inp,
                          const void* weight, float* dbias_buffer, int B, int T, int C, int OC, void* stream,
                          const void* pre_gelu, int gelu_fusion) {
    if (llmk::failed()) return;
    const int M = B * T;
    LLMK_REQUIRE(C % 8 == 0 && OC % 8 == 0, "matmul_backward: C=%d and OC=%d must be multiples of 8", C, OC);
    LLMK_REQUIRE(aligned16(dout) && aligned16(inp) && aligned16(weight), "matmul_backward: operands must be 16-byte aligned");
    if (M == 0 || OC == 0 || C == 0) return;
    hipStream_t st = (hipStream_t)stream;
    const int num_cu = llmk::device_info().num_cu;

    // The weight-gradient GEMM below reads dout as its K-major A operand; when it is the direct-to-LDS split-K kernel
    // it adds up the rows of that operand on the side (EPI_PARTIAL_ROWSUM), which is the bias gradient without another
    // pass over dout. Same preconditions as that kernel; otherwise the streaming reduction in (1).
    bool dbias_in_gemm = false;
#if !defined(LLMK_FP32)
    if (dbias) {
        GemmArgs t{};
        t.A = (const floatX*)dout; t.B = (const floatX*)inp; t.C = (floatX*)dweight;
        t.M = OC; t.N = C; t.K = M; t.lda = OC; t.ldb = C; t.ldc = C; t.k_per_split = KGRAN;
        dbias_in_gemm = pipelined_ok(t) && M % K_STEP == 0;
    }
#endif

    // (1) dbias += column sums of dout
    if (dbias && !dbias_in_gemm) {
        LLMK_REQUIRE(dbias_buffer != nullptr, "matmul_backward: dbias_buffer is required when dbias is given");
        const int ny = bias_grad_ny(OC);
        llmk::ProfScope prof("bias_grad", 0, (double)M * OC * sizeof(floatX), st);
        bias_grad_kernel<false><<<dim3(CEIL_DIV(OC, BG_COLV * VN), ny), 256, 0, st>>>(dbias_buffer, (floatX*)dout, nullptr, M, OC);
        LAUNCH_CHECK();
        bias_grad_reduce_kernel<<<CEIL_DIV(OC, BGR_COLS), BGR_COLS * BGR_GROUPS, 0, st>>>((floatX*)dbias, dbias_buffer, OC, ny);
        LAUNCH_CHECK();
    }

    // (2) dinp[M,C] = dout[M,OC] . W[OC,C]   (A = dout K-contiguous, B(n=c,k=oc) stored [k][n])
    {
        GemmArgs g{};
        g.A = (const floatX*)dout; g.B = (const floatX*)weight; g.C = (floatX*)dinp;
        g.M = M; g.N = C; g.K = OC; g.lda = OC; g.ldb = C; g.ldc = C;
        g.k_per_split = CEIL_DIV(OC, K_STEP) * K_STEP;
        const bool big = (size_t)CEIL_DIV(M, BIG_TILE) * CEIL_DIV(C, BIG_TILE) >= (size_t)num_cu;
        const bool stored_grad = pre_gelu && gelu_fusion >= 3;   // pre_gelu holds gelu'(pre-activation), see llmk_matmul_forward
#if defined(LLMK_FP32)
        const bool fused = pre_gelu && gelu_fusion >= 2 && !stored_grad;
#else
        // bf16: gelu' goes into the epilogue of the direct-to-LDS kernel (big tiles only); the bias gradient of the layer
        // below then comes out of its weight-gradient GEMM, and no elementwise pass over (B,T,4C) is left
        const bool fused = pre_gelu && gelu_fusion >= 2 && big && aligned16(pre_gelu) && pipelined_ok(g);
#endif
        {
            // with GELU backward in the epilogue the kernel also reads the (M, C) pre-activations
            llmk::ProfScope prof(fused ? "gemm_nn_dgelu" : "gemm_nn", 2.0 * M * (double)OC * C,
                                 ((double)M * OC + (double)OC * C + (fused ? 2.0 : 1.0) * M * C) * sizeof(floatX), st);
            if (fused) {
                g.aux = (floatX*)pre_gelu;
#if defined(LLMK_FP32)
                launch_best<false, true, EPI_DGELU>(g, 1, big, st);
#else
                if (stored_grad) launch_pipelined_cfg<256, 256, 2, 4, false, true, EPI_DGELU_D>(g, 1, st);
                else launch_pipelined_cfg<256, 256, 2, 4, false, true, EPI_DGELU>(g, 1, st);
#endif
            } else {
                launch_best<false, true, EPI_STORE>(g, 1, big, st);
            }
        }
        if (pre_gelu && !fused) {
            if (stored_grad) llmk_gelu_backward_from_grad(dinp, pre_gelu, M * C, stream);
            else llmk_gelu_backward_inplace(dinp, pre_gelu, M * C, stream);
        }
    }

    // (3) dW[OC,C] += dout^T . inp   (A(m=oc,k=row) stored [k][m], B(n=c,k=row) stored [k][n])
    {
        GemmArgs g{};
        g.A = (const floatX*)dout; g.B = (const floatX*)inp; g.C = (floatX*)dweight;
        g.M = OC; g.N = C; g.K = M; g.lda = OC; g.ldb = C; g.ldc = C;
        const size_t tiles_big = (size_t)CEIL_DIV(OC, BIG_TILE) * CEIL_DIV(C, BIG_TILE);
        const size_t tiles_small = (size_t)CEIL_DIV(OC, SMALL_TILE) * CEIL_DIV(C, SMALL_TILE);
        const bool big = tiles_big >= 8;                          // split-K fills the machine when there are few big tiles
        const size_t tiles = big ? tiles_big : tiles_small;
        double best_uniform = 1e30;
        const int splits = tn_equal_splits(M, tiles, num_cu, &best_uniform);
        g.k_per_split = CEIL_DIV(CEIL_DIV(M, K_STEP), splits) * K_STEP;
        const double tn_bytes = ((double)M * OC + (double)M * C + 2.0 * OC * C) * sizeof(floatX);
        if (splits == 1 && !tn_partial_always(g)) {
            LLMK_REQUIRE(!dbias_in_gemm, "matmul_backward: bias gradient was left to a kernel that is not being run");
            llmk::ProfScope prof("gemm_tn", 2.0 * M * (double)OC * C, tn_bytes, st);
            launch_best<true, true, EPI_ACCUM>(g, 1, big, st);
            g_last_split_kind = 0; g_last_split_pieces = 1;
#if !defined(LLMK_FP32)
        } else if (const SkPlan plan = (big && M % K_STEP == 0 && pipelined_ok(g) && (!dbias || dbias_in_gemm) && g_sk_mode != 0)
                                           ? sk_build(CEIL_DIV(OC, BIG_TILE), CEIL_DIV(C, BIG_TILE), M / K_STEP, num_cu & ~7, 800.0 / (double)M)
                                           : SkPlan();
                   plan.valid && (g_sk_mode == 1 || plan.cost < 0.98 * best_uniform)) {
            // one long and s - 1 short pieces per tile (see sk_build)
            const size_t mn = (size_t)OC * C;
            const int parts = 4, slots = plan.slots, G = num_cu & ~7;
            g.partial = (float*)llmk::workspace((mn + (dbias_in_gemm ? (size_t)OC * parts : 0)) * slots * sizeof(float));
            g.k_per_split = M;
            g.sk_tiles = CEIL_DIV(OC, BIG_TILE) * CEIL_DIV(C, BIG_TILE); g.sk_long = plan.long_blocks; g.sk_each = plan.each;
            g.splits = slots;
            g_last_split_kind = 2; g_last_split_pieces = slots;
            {
                llmk::ProfScope prof("gemm_tn_splitk", 2.0 * M * (double)OC * C, tn_bytes, st);
                if (dbias_in_gemm) g.rowsum = g.partial + mn * slots;            // [slots * parts][OC]
                launch_pipelined_tn(g, slots, true, dbias_in_gemm ? EPI_PARTIAL_ROWSUM : EPI_PARTIAL, G, st);
            }
            llmk::ProfScope prof("splitk_reduce", 0, (double)mn * slots * sizeof(float) + 2.0 * mn * sizeof(floatX), st);
            const unsigned main_blocks = (unsigned)CEIL_DIV(mn / 4, (size_t)256);
            const unsigned bias_blocks = dbias_in_gemm ? (unsigned)CEIL_DIV(OC, SKR_ROWS) : 0u;
            splitk_reduce_kernel<true><<<main_blocks + bias_blocks, 256, 0, st>>>((floatX*)dweight, g.partial, mn, slots,
                                                                               (floatX*)dbias, g.rowsum, OC, slots * parts, main_blocks);
            LAUNCH_CHECK();
#endif
        } else {
            const size_t mn = (size_t)OC * C;
            const int parts = big ? 4 : 2;                        // column waves of the tile configuration: each leaves a partial
            g_last_split_kind = 1; g_last_split_pieces = splits;
            g.partial = (float*)llmk::workspace((mn + (dbias_in_gemm ? (size_t)OC * parts : 0)) * splits * sizeof(float));
            {
                llmk::ProfScope prof("gemm_tn_splitk", 2.0 * M * (double)OC * C, tn_bytes, st);
#if !defined(LLMK_FP32)
                if (dbias_in_gemm) {
                    LLMK_REQUIRE(pipelined_ok(g), "matmul_backward: split of K (%d) does not suit the direct-to-LDS kernel", g.k_per_split);
                    g.rowsum = g.partial + mn * splits;           // [splits * parts][OC]
                    launch_pipelined<true, true, EPI_PARTIAL_ROWSUM>(g, splits, big, st);
                } else
#endif
                launch_best<true, true, EPI_PARTIAL>(g, splits, big, st);
            }
            // dweight += the splits' partial products and, in the same launch, dbias += the row sums (in split order)
            llmk::ProfScope prof("splitk_reduce", 0, (double)mn * splits * sizeof(float) + 2.0 * mn * sizeof(floatX), st);
            const unsigned main_blocks = (unsigned)CEIL_DIV(mn / 4, (size_t)256);
            const unsigned bias_blocks = dbias_in_gemm ? (unsigned)CEIL_DIV(OC, SKR_ROWS) : 0u;
            splitk_reduce_kernel<true><<<main_blocks + bias_blocks, 256, 0, st>>>((floatX*)dweight, g.partial, mn, splits,
                                                                               (floatX*)dbias, g.rowsum, OC, splits * parts, main_blocks);
            LAUNCH_CHECK();
        }
    }
}

}  // extern "C"
