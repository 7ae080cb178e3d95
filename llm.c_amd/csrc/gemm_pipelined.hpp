// Persistent, software-pipelined bf16 MFMA GEMM for gfx950 (MI355X).
//
//   C[M][N] (op)= sum_k A(m,k) * B(n,k)        A, B: bf16, K-contiguous or K-major storage
//
// Why it looks the way it does (all measured on MI355X, 256 CUs):
//   * A 256x256 output tile per workgroup is the largest that fits the register file
//     (256 KiB of fp32 accumulators per CU); it needs 64 KiB of operands per 64 of K.
//   * LDS write bandwidth (~64 B/clk/CU) did not double with the matrix rate of this chip, so the
//     classic "global -> registers -> ds_write" staging leaves the matrix cores idle while every
//     wave writes LDS. Here operands go global -> LDS directly (global_load_lds_dwordx4): no
//     staging registers, no ds_write instructions, and the LDS writes trickle in while MFMAs run.
//   * K advances in blocks of 32 through a ring of five 32 KiB LDS slots (all 160 KiB of the CU); loads run
//     four blocks (128 KiB per CU) ahead of the math, which is what it takes to cover HBM/L2 latency at
//     this consumption rate. One s_barrier per block, without a memory fence (a fence would drain the ring).
//   * A direct-to-LDS load deposits each wave's 64 x 16 B linearly, so the anti-bank-conflict
//     swizzle is applied on the global side: lane p of a row fetches chunk p ^ f(row), and the
//     MFMA operand reads undo it. K-contiguous tiles: [row][32] with f = (row>>2)&3 (ds_read_b128
//     conflict-free). K-major tiles: [k][row] as in memory, f = 4*(k&3), read with the transposing
//     ds_read_b64_tr_b16 so no software transpose is needed for dinp/dweight.
//   * The kernel is persistent (one workgroup per CU walks a list of tiles). When a tile's K loop
//     ends, the first four K-blocks of the NEXT tile are requested into four ring slots while the
//     epilogue stages its output through the fifth.
//   * The MFMA is issued with swapped operands (D^T = B.A^T): each lane then owns 4 consecutive
//     output columns of one row, which it writes as 8 bytes into a per-wave LDS staging strip; the
//     strip is read back row-contiguously so that global stores (and the loads of pre_gelu / the
//     old dW for the fused epilogues) are full 128-byte lines.
//   * Tile ids are dealt so that the 32 CUs of an XCD (which share an L2) work on an 8x4 patch of
//     neighbouring tiles.
#pragma once
#include "common.hpp"
#include "gelu.hpp"

namespace gemmk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

enum Epi { EPI_BIAS = 0, EPI_BIAS_GELU = 1, EPI_STORE = 2, EPI_DGELU = 3, EPI_ACCUM = 4, EPI_PARTIAL = 5 };

struct GemmArgs {
    const floatX* A;
    const floatX* B;
    floatX* C;
    int M, N, K;          // C[M][N] = sum_k A(m,k) * B(n,k)
    int lda, ldb, ldc;    // leading dimensions of the stored matrices, in elements
    const floatX* bias;   // [N] or nullptr                         (EPI_BIAS*)
    floatX* aux;          // pre-GELU output (EPI_BIAS_GELU) / pre-GELU input (EPI_DGELU)
    float* partial;       // [splits][M][N] fp32                    (EPI_PARTIAL)
    int k_per_split;      // multiple of the K block
    int splits;
};

#if !defined(LLMK_FP32)

constexpr int PBK = 32;                 // K per pipeline block
constexpr int STAGES = 5;                // ring slots; loads run STAGES-1 K blocks ahead of the math
constexpr int LDS_TOTAL = 160 * 1024;
constexpr int EPI_PITCH = 144;          // bytes per staged output row: 128 + 16

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// wait until at most N of this wave's vector-memory operations are outstanding (gfx9 encoding, other counters untouched)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// Workgroup barrier WITHOUT the memory fence of __syncthreads(): the fence would wait for every outstanding
// direct-to-LDS load (vmcnt(0)) and serialize the pipeline. Visibility of the K block that is about to be
// read is established by the explicit vmcnt wait each wave does before arriving here.
__device__ __forceinline__ void barrier_no_fence() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// tile id -> tile coordinates; consecutive ids walk an 8-row group of tiles column by column
__device__ __forceinline__ void tile_of(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int per_group = 8 * tiles_n;
    const int group = t / per_group;
    const int first_m = group * 8;
    const int gsz = min(tiles_m - first_m, 8);
    const int in_group = t - group * per_group;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

template <int BM, int BN, int WGM, int WGN, bool A_T, bool B_T, int EPI, int DBG = 0>   // DBG: measurement ablations (1: no loads, 2: no math)
__global__ void __launch_bounds__(WGM * WGN * 64)
gemm_pipelined_kernel(GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only builtins below; the host pass only needs the launch stub
    constexpr int NW = WGM * WGN, NT = NW * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN, TM = WTM / 32, TN = WTN / 32;
    constexpr int A_STAGE = BM * PBK * 2, B_STAGE = BN * PBK * 2, STAGE = A_STAGE + B_STAGE;
    constexpr int A_CHUNKS = A_STAGE / 1024, B_CHUNKS = B_STAGE / 1024;
    constexpr int CPW = (A_CHUNKS + B_CHUNKS) / NW;            // 1 KiB chunks each wave requests per K block
    static_assert((A_CHUNKS + B_CHUNKS) % NW == 0, "chunks must divide evenly over the waves");
    static_assert(STAGES * STAGE <= LDS_TOTAL, "LDS budget");
    static_assert(TN % 2 == 0, "epilogue strips are 64 columns wide");
    static_assert(A_CHUNKS % NW == 0, "each load slot of a wave must be all-A or all-B");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // scalar: LDS-DMA destinations must be wave-uniform
    const int wm = wave / WGN, wn = wave % WGN;
    const int idx = lane & 31, half = lane >> 5;
    const int tiles_m = CEIL_DIV(g.M, BM), tiles_n = CEIL_DIV(g.N, BN);
    const int num_tiles = tiles_m * tiles_n;
    const int num_work = num_tiles * g.splits;

    // --- this workgroup's share of the work list ---------------------------------------------
    // Workgroups are dispatched round-robin over the 8 XCDs; give XCD x the ids [32x, 32x+32) of
    // every round of 256 so that its CUs share operand panels in its L2.
    const int G = gridDim.x;
    auto work_id = [&](int it) -> int {
        int w = it * G + blockIdx.x;
        if ((G & 7) == 0) {
            const int per = G >> 3;
            w = it * G + (blockIdx.x & 7) * per + (blockIdx.x >> 3);
        }
        return w;
    };

    // --- per-thread load descriptors -----------------------------------------------------------
    const floatX* gp[CPW];       // global address of this lane's 16 bytes for K block 0 of the current work item
    int lds_dst[CPW];            // wave-uniform byte offset of the chunk inside a stage
    size_t kstep[CPW];           // elements to advance per K block
    auto setup_loads = [&](int m0, int n0, int kbeg) {
#pragma unroll
        for (int i = 0; i < CPW; i++) {
            const int ci = wave + i * NW;
            const bool isA = i * NW < A_CHUNKS;                   // compile-time after unrolling
            const int cc = isA ? ci : ci - A_CHUNKS;
            const floatX* base = isA ? g.A : g.B;
            const int ld = isA ? g.lda : g.ldb;
            const int r0 = isA ? m0 : n0, rmax = isA ? g.M : g.N;
            const bool trans = isA ? A_T : B_T;
            constexpr int RA = BM, RB = BN;
            const int R = isA ? RA : RB;
            lds_dst[i] = (isA ? 0 : A_STAGE) + cc * 1024;
            if (!trans) {
                const int row = cc * 16 + (lane >> 2), p = lane & 3;
                const int c = p ^ ((row >> 2) & 3);
                const int grow = min(r0 + row, rmax - 1);
                gp[i] = base + (size_t)grow * ld + kbeg + c * 8;
                kstep[i] = PBK;
            } else {
                const int byte = cc * 1024 + lane * 16;
                const int krow = byte / (R * 2), p = (byte % (R * 2)) >> 4;
                const int cn = p ^ (4 * (krow & 3));
                int col = r0 + cn * 8;
                if (col >= rmax) col = r0;
                gp[i] = base + (size_t)(kbeg + krow) * ld + col;
                kstep[i] = (size_t)PBK * ld;
            }
        }
    };
    auto issue = [&](int kb, int slot) {
        char* stage = lds + slot * STAGE;
        if (DBG & 1) return;
#pragma unroll
        for (int i = 0; i < CPW; i++)
            __builtin_amdgcn_global_load_lds(gp[i] + (size_t)kb * kstep[i], (lds_void_ptr)(stage + lds_dst[i]), 16, 0, 0);
    };

    // --- MFMA operand reads ----------------------------------------------------------------------
    auto frag_k = [&](const char* tile, int row0, int s) -> bf16x8 {        // K-contiguous tile [row][32]
        const int row = row0 + idx, c = 2 * s + half;
        return *reinterpret_cast<const bf16x8*>(tile + row * 64 + ((c ^ ((row >> 2) & 3)) << 4));
    };
    // The transposing reads are issued as inline asm on purpose: for the builtin, the compiler cannot tell that the
    // read does not alias the in-flight direct-to-LDS loads and would wait for ALL of them (vmcnt(0)) first, which
    // serialises loading and math. The price is that their completion has to be awaited by hand (lds_wait below).
    auto frag_t = [&](const char* tile, int pitch, int row0, int s) -> bf16x8 {   // K-major tile [k][row], transposing read
        const int s16 = lane & 15, grp = lane >> 4;
        const int krow = 16 * s + 8 * (grp >> 1) + (s16 >> 2);             // (krow & 3) is the same for krow + 4
        const int col = row0 + (grp & 1) * 16 + 4 * (s16 & 3);
        const int cn = (col >> 3) ^ (4 * (krow & 3));
        const char* p = tile + krow * pitch + cn * 16 + (col & 7) * 2;
        const unsigned a0 = (unsigned)(size_t)(__attribute__((address_space(3))) const char*)p;
        const unsigned a1 = a0 + 4 * pitch;
        s16x4 lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(a0));
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(hi) : "v"(a1));
        union { struct { s16x4 a, b; } s; bf16x8 v; } u;
        u.s.a = lo; u.s.b = hi;
        return u.v;
    };

    f32x16 acc[TM][TN];
    int ring = 0;                       // ring slot that holds K block 0 of the current work item
    int it = 0;
    int w = work_id(0);
    if (w >= num_work) return;
    int tile_m, tile_n;
    tile_of(w % num_tiles, tiles_m, tiles_n, tile_m, tile_n);
    int split = w / num_tiles;
    int kbeg = split * g.k_per_split;
    int nkb = (min(g.K, kbeg + g.k_per_split) - kbeg) / PBK;
    setup_loads(tile_m * BM, tile_n * BN, kbeg);
#pragma unroll
    for (int j = 0; j < STAGES - 1; j++)
        if (j < nkb) issue(j, (ring + j) % STAGES);

    while (true) {
        const int m0 = tile_m * BM, n0 = tile_n * BN;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

        // ---- K loop -----------------------------------------------------------------------------
        for (int kb = 0; kb < nkb; kb++) {
            const int ahead = min(STAGES - 2, nkb - 1 - kb);      // younger blocks that may stay in flight
            if (ahead >= 3) wait_vmcnt<3 * CPW>();
            else if (ahead == 2) wait_vmcnt<2 * CPW>();
            else if (ahead == 1) wait_vmcnt<CPW>();
            else wait_vmcnt<0>();
            barrier_no_fence();                                   // block kb landed for everyone; slot of kb-1 is free
            if (kb + STAGES - 1 < nkb) issue(kb + STAGES - 1, (ring + kb + STAGES - 1) % STAGES);
            const char* sa = lds + ((ring + kb) % STAGES) * STAGE;
            const char* sb = sa + A_STAGE;
#pragma unroll
            for (int s = 0; s < ((DBG & 2) ? 0 : PBK / 16); s++) {
                bf16x8 fa[TM], fb[TN];
#pragma unroll
                for (int i = 0; i < TM; i++) fa[i] = A_T ? frag_t(sa, BM * 2, wm * WTM + i * 32, s) : frag_k(sa, wm * WTM + i * 32, s);
#pragma unroll
                for (int j = 0; j < TN; j++) fb[j] = B_T ? frag_t(sb, BN * 2, wn * WTN + j * 32, s) : frag_k(sb, wn * WTN + j * 32, s);
                if (A_T || B_T) {      // hand-issued reads: wait for LDS, with the operands tied to the wait so nothing moves above it
                    if (A_T) {
#pragma unroll
                        for (int i = 0; i < TM; i++) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[i]));
                    }
                    if (B_T) {
#pragma unroll
                        for (int j = 0; j < TN; j++) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fb[j]));
                    }
                }
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)   // swapped operands: acc[i][j] = D^T block, rows = n, cols = m
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
            }
        }

        // ---- request the next work item's first K blocks, then run the epilogue under them --------
        barrier_no_fence();                                       // every wave is done reading the ring
        const int ring_free = (ring + nkb) % STAGES;              // slot the epilogue may use
        const int cur_m0 = m0, cur_n0 = n0, cur_split = split;
        it++;
        w = work_id(it);
        const bool have_next = w < num_work;
        int next_nkb = 0;
        if (have_next) {
            tile_of(w % num_tiles, tiles_m, tiles_n, tile_m, tile_n);
            split = w / num_tiles;
            kbeg = split * g.k_per_split;
            next_nkb = (min(g.K, kbeg + g.k_per_split) - kbeg) / PBK;
            setup_loads(tile_m * BM, tile_n * BN, kbeg);
            ring = (ring_free + 1) % STAGES;
#pragma unroll
            for (int j = 0; j < STAGES - 1; j++)
                if (j < next_nkb) issue(j, (ring + j) % STAGES);
        }

        // ---- epilogue ---------------------------------------------------------------------------------
        // wave-private staging strip inside the free ring slot: 16 rows x (128 B + 16 B pad)
        {
            constexpr int STRIP_ROWS = 16;
            constexpr int STRIP = STRIP_ROWS * EPI_PITCH;
            static_assert(NW * STRIP <= STAGE, "all strips must fit in one ring slot");
            char* strip = lds + ring_free * STAGE + wave * STRIP;
            const int wm0 = cur_m0 + wm * WTM, wn0 = cur_n0 + wn * WTN;
            constexpr bool F32OUT = (EPI == EPI_PARTIAL || EPI == EPI_ACCUM);   // staged in fp32 so that C += acc rounds once
            constexpr int PASSES = F32OUT ? TN : TN / 2;          // a strip row is 128 B: 64 bf16 columns or 32 fp32 columns
            constexpr int JP = F32OUT ? 1 : 2;                    // 32-column blocks per pass
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int pass = 0; pass < PASSES; pass++) {
#pragma unroll
                    for (int hsel = 0; hsel < 2; hsel++) {        // rows 0..15 / 16..31 of the 32-row block
                        // phase 1: lane (m = idx, half) owns n = 8q + 4*half + 0..3 of each 32-column block
                        if ((idx >> 4) == hsel) {
#pragma unroll
                            for (int j = pass * JP; j < (pass + 1) * JP; j++) {
#pragma unroll
                                for (int q = 0; q < 4; q++) {
                                    const int nl = j * 32 + 8 * q + 4 * half;                 // column inside the wave tile
                                    const int sl = (j - pass * JP) * 32 + 8 * q + 4 * half;   // column inside the strip
                                    float v[4];
#pragma unroll
                                    for (int e = 0; e < 4; e++) v[e] = acc[i][j][4 * q + e];
                                    if (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU) {
                                        if (g.bias) {
                                            const int n = wn0 + nl;
                                            if (n < g.N) {
                                                bf16x4 b4 = *reinterpret_cast<const bf16x4*>(g.bias + n);
#pragma unroll
                                                for (int e = 0; e < 4; e++) v[e] += (float)b4[e];
                                            }
                                        }
                                    }
                                    char* dst = strip + (idx & 15) * EPI_PITCH;
                                    if (F32OUT) {
                                        f32x4 o = {v[0], v[1], v[2], v[3]};
                                        *reinterpret_cast<f32x4*>(dst + (8 * q + 4 * half) * 4) = o;
                                    } else {
                                        bf16x4 o;
#pragma unroll
                                        for (int e = 0; e < 4; e++) o[e] = (__bf16)v[e];
                                        *reinterpret_cast<bf16x4*>(dst + sl * 2) = o;
                                    }
                                }
                            }
                        }
                        __builtin_amdgcn_s_waitcnt(0xC07F);          // lgkmcnt(0): the strip is written
                        __builtin_amdgcn_wave_barrier();
                        // phase 2: 16 rows x 128 B, 8 lanes per row
#pragma unroll
                        for (int t = 0; t < 2; t++) {
                            const int row = t * 8 + (lane >> 3), ch = lane & 7;
                            const int m = wm0 + i * 32 + hsel * 16 + row;
                            u32x4 raw = *reinterpret_cast<const u32x4*>(strip + row * EPI_PITCH + ch * 16);
                            if (F32OUT) {
                                const int n = wn0 + pass * 32 + ch * 4;
                                if (m < g.M && n < g.N) {
                                    if (EPI == EPI_PARTIAL) {
                                        *reinterpret_cast<u32x4*>(g.partial + ((size_t)cur_split * g.M + m) * g.N + n) = raw;
                                    } else {
                                        union { u32x4 u; f32x4 f; } x;
                                        x.u = raw;
                                        floatX* cp = g.C + (size_t)m * g.ldc + n;
                                        bf16x4 old = *reinterpret_cast<const bf16x4*>(cp), o4;
#pragma unroll
                                        for (int e = 0; e < 4; e++) o4[e] = (__bf16)((float)old[e] + x.f[e]);
                                        *reinterpret_cast<bf16x4*>(cp) = o4;
                                    }
                                }
                            } else {
                                const int n = wn0 + pass * 64 + ch * 8;
                                if (m < g.M && n < g.N) {
                                    const size_t o = (size_t)m * g.ldc + n;
                                    union { u32x4 u; bf16x8 h; } x, y, z;
                                    x.u = raw;
                                    if (EPI == EPI_BIAS_GELU) {
                                        *reinterpret_cast<u32x4*>(g.aux + o) = x.u;
#pragma unroll
                                        for (int e = 0; e < 8; e++) y.h[e] = (__bf16)gelu_f((float)x.h[e]);
                                        *reinterpret_cast<u32x4*>(g.C + o) = y.u;
                                    } else if (EPI == EPI_DGELU) {
                                        z.u = *reinterpret_cast<const u32x4*>(g.aux + o);
#pragma unroll
                                        for (int e = 0; e < 8; e++) y.h[e] = (__bf16)(gelu_grad_f((float)z.h[e]) * (float)x.h[e]);
                                        *reinterpret_cast<u32x4*>(g.C + o) = y.u;
                                    } else {
                                        *reinterpret_cast<u32x4*>(g.C + o) = x.u;
                                    }
                                }
                            }
                        }
                        __builtin_amdgcn_s_waitcnt(0xC07F);          // strip reads done before it is overwritten
                        __builtin_amdgcn_wave_barrier();
                    }
                }
            }
        }
        if (!have_next) break;
        nkb = next_nkb;
    }
#endif  // __HIP_DEVICE_COMPILE__
}

#endif  // !LLMK_FP32

}  // namespace gemmk
