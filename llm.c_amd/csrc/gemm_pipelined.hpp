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
#include <type_traits>

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
constexpr int STAGES = 5;               // ring slots of one K block: two pairs of blocks and a spare for the epilogue
constexpr int KGRAN = 2 * PBK;          // K (and the K range of a split) must be a multiple of this
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
template <int DBG = 0>
__device__ __forceinline__ void barrier_no_fence() {
    if (DBG & 8) return;
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Output stores are non-temporal: a tile's output is not read again by this kernel, and a store that allocates in
// L2 is acknowledged late enough (the waves count stores and loads with one counter) to hold up the next tile's loads.
template <int DBG = 0, typename T>
__device__ __forceinline__ void st_out(T* p, T v) {
    if (DBG & 4096) *p = v; else __builtin_nontemporal_store(v, p);
}
// ... except where the next kernel reads a small result straight back (split-K partial sums, weight gradients)
template <typename T>
__device__ __forceinline__ void st_cached(T* p, T v) {
    *p = v;
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

template <int BM, int BN, int WGM, int WGN, bool A_T, bool B_T, int EPI, int DBG = 0>   // DBG: measurement ablations (1: no loads, 2: no math, 4: no stores)
__global__ void __launch_bounds__(WGM * WGN * 64)
gemm_pipelined_kernel(GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only builtins below; the host pass only needs the launch stub
    constexpr int NW = WGM * WGN, NT = NW * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN, TM = WTM / 32, TN = WTN / 32;
    constexpr int A_STAGE = BM * PBK * 2, B_STAGE = BN * PBK * 2, STAGE = A_STAGE + B_STAGE;
    constexpr int A_CHUNKS = A_STAGE / 1024, B_CHUNKS = B_STAGE / 1024;
    constexpr int PASSES_OF_EPI = (EPI == EPI_PARTIAL || EPI == EPI_ACCUM) ? TN : TN / 2;   // epilogue passes over a 32-row block
    constexpr int CPW = (A_CHUNKS + B_CHUNKS) / NW;            // 1 KiB chunks each wave requests per K block
    static_assert((A_CHUNKS + B_CHUNKS) % NW == 0, "chunks must divide evenly over the waves");
    static_assert(STAGES * STAGE <= LDS_TOTAL, "LDS budget");
    static_assert(TN % 2 == 0, "epilogue strips are 64 columns wide");
    static_assert(A_CHUNKS % NW == 0, "each load slot of a wave must be all-A or all-B");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    if (DBG & 64) {  // experiment: stagger the workgroups of an XCD over one tile period
        const int phase = (blockIdx.x >> 3) & 7;
        for (int i = 0; i < phase; i++) __builtin_amdgcn_s_sleep(100);
    }
    if (DBG & 1) {   // ablation without loads: define the LDS contents (32: pseudo-random bits, else zeros)
        for (int i = tid * 4; i < STAGES * STAGE; i += NT * 4) {
            unsigned v = (DBG & 32) ? ((squirrel_noise5((uint32_t)i, 17u) & 0x3fff3fffu) | 0x30003000u) : 0u;
            *reinterpret_cast<unsigned*>(lds + i) = v;
        }
        __syncthreads();
    }
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // scalar: LDS-DMA destinations must be wave-uniform
    const int wm = wave / WGN, wn = wave % WGN;
    // The two waves that share a SIMD (w and w + NW/2) request their share of a K block at different points of
    // the block's math, so that a wave held up at the memory pipeline's entrance always has a partner issuing MFMAs.
    const bool late = (DBG & 2048) ? false : wave >= NW / 2;
    const int idx = lane & 31, half = lane >> 5;
    const int tiles_m = CEIL_DIV(g.M, BM), tiles_n = CEIL_DIV(g.N, BN);
    const int num_tiles = tiles_m * tiles_n;
    const int num_work = num_tiles * g.splits;

    // --- this workgroup's share of the work list ---------------------------------------------
    // Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2 (the host launches a multiple
    // of 8). Without split-K and with enough row panels, XCD x owns the row panels [tiles_m*x/8, tiles_m*(x+1)/8)
    // outright and its CUs walk them together, 8 panels by all columns at a time: the streamed operand (A) then
    // crosses HBM once. Otherwise XCD x takes the ids [x*G/8, (x+1)*G/8) of every round, so that a split's tiles
    // (which share their K range of both operands) sit on one XCD.
    const int G = gridDim.x;
    auto work_item = [&](int it, int& tm, int& tn, int& sp) -> bool {
        const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3, per_x = G >> 3;
        if (!(DBG & 65536) && g.splits == 1 && tiles_m >= 64) {
            const int r0 = (tiles_m * xcd) >> 3, rows = ((tiles_m * (xcd + 1)) >> 3) - r0;
            const int q = it * per_x + local;
            if (q >= rows * tiles_n) return false;
            tile_of(q, rows, tiles_n, tm, tn);
            tm += r0;
            sp = 0;
            return true;
        }
        const int w = it * G + xcd * per_x + local;
        if (w >= num_work) return false;
        tile_of(w % num_tiles, tiles_m, tiles_n, tm, tn);
        sp = w / num_tiles;
        return true;
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
            if (!trans && (DBG & 256)) {   // experiment (loads only): full 128-byte lines per row
                const int row = cc * 8 + (lane >> 3), p = lane & 7;
                gp[i] = base + (size_t)min(r0 + row, rmax - 1) * ld + kbeg + p * 8;
                kstep[i] = (size_t)128 * ld;
            } else if (!trans) {
                const int row = cc * 16 + (lane >> 2), p = lane & 3;
                const int c = p ^ ((row >> 2) & 3);
                const int grow = min(r0 + row, rmax - 1);
                gp[i] = base + (size_t)grow * ld + kbeg + c * 8;
                kstep[i] = PBK;
            } else {
                const int byte = cc * 1024 + lane * 16;
                const int krow = byte / (R * 2), p = (byte % (R * 2)) >> 4;
                const int cn = (DBG & 16384) ? p : p ^ (4 * (krow & 3));
                int col = r0 + cn * 8;
                if (col >= rmax) col = r0;
                gp[i] = base + (size_t)(kbeg + krow) * ld + col;
                kstep[i] = (size_t)PBK * ld;
            }
        }
    };
    // two consecutive K blocks at once, the two 64-byte halves of every 128-byte line requested back to back
    auto issue2 = [&](int kb, int slot0, int slot1) {
        char* stage0 = lds + slot0 * STAGE;
        char* stage1 = lds + slot1 * STAGE;
        if (DBG & 1) return;
#pragma unroll
        for (int i = 0; i < CPW; i++) {
            __builtin_amdgcn_global_load_lds(gp[i] + (size_t)kb * kstep[i], (lds_void_ptr)(stage0 + lds_dst[i]), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(gp[i] + (size_t)(kb + 1) * kstep[i], (lds_void_ptr)(stage1 + lds_dst[i]), 16, 0, 0);
        }
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

    // fragments of one 16-wide K step
    auto read_frags = [&](const char* sa, int s, bf16x8 (&fa)[TM], bf16x8 (&fb)[TN]) {
        if (DBG & 16) {
#pragma unroll
            for (int i = 0; i < TM; i++) asm volatile("" : "+v"(fa[i]));
#pragma unroll
            for (int j = 0; j < TN; j++) asm volatile("" : "+v"(fb[j]));
            return;
        }
        const char* sb = sa + A_STAGE;
#pragma unroll
        for (int i = 0; i < TM; i++) fa[i] = A_T ? frag_t(sa, BM * 2, wm * WTM + i * 32, s) : frag_k(sa, wm * WTM + i * 32, s);
        if (DBG & 512) {
#pragma unroll
            for (int j = 0; j < TN; j++) asm volatile("" : "+v"(fb[j]));
            return;
        }
#pragma unroll
        for (int j = 0; j < TN; j++) fb[j] = B_T ? frag_t(sb, BN * 2, wn * WTN + j * 32, s) : frag_k(sb, wn * WTN + j * 32, s);
    };
    // Hand-issued (transposing) reads have to be awaited by hand. LDS operations return in order, so "at most
    // YOUNGER operations outstanding" means these operands have arrived when YOUNGER hand-issued reads were
    // requested after them (compiler-issued reads in between only make the wait longer). The operands are tied
    // to the wait so that nothing that uses them moves above it.
    constexpr int TR_READS = (A_T ? 2 * TM : 0) + (B_T ? 2 * TN : 0);       // hand-issued reads per 16-wide step
    auto await_frags = [&](bf16x8 (&fa)[TM], bf16x8 (&fb)[TN], auto younger) {
        constexpr int Y = decltype(younger)::value;
        if (A_T) {
#pragma unroll
            for (int i = 0; i < TM; i++) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(fa[i]) : "n"(Y));
        }
        if (B_T) {
#pragma unroll
            for (int j = 0; j < TN; j++) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(fb[j]) : "n"(Y));
        }
    };
    using Younger = std::integral_constant<int, TR_READS>;
    using NoneYounger = std::integral_constant<int, 0>;
    f32x16 acc[TM][TN];
    auto mma = [&](const bf16x8 (&fa)[TM], const bf16x8 (&fb)[TN]) {
        if (DBG & 2) return;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)   // swapped operands: acc[i][j] = D^T block, rows = n, cols = m
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    };
    // Waiting for loads: vector-memory operations retire in issue order, so "at most N outstanding" means that
    // everything but the N youngest has landed. The pairs of a tile are requested one at a time, so the only
    // younger operations a wait ever has to allow are the second pair of the tile's prologue and the previous
    // tile's output stores (NS_EPI per wave when every lane stored, which holds for interior tiles).
    constexpr int NS_EPI = TM * PASSES_OF_EPI * 4 * (EPI == EPI_BIAS_GELU ? 2 : 1);
    static_assert(2 * CPW + NS_EPI <= 63, "vmcnt is a 6-bit counter");

    int ring = 0;                       // ring slot that holds K block 0 of the current work item
    int it = 0;
    int tile_m, tile_n, split;
    if (!work_item(0, tile_m, tile_n, split)) return;
    int kbeg = split * g.k_per_split;
    int nkb = (min(g.K, kbeg + g.k_per_split) - kbeg) / PBK;
    setup_loads(tile_m * BM, tile_n * BN, kbeg);
    issue2(0, ring % STAGES, (ring + 1) % STAGES);
    if (nkb > 2) issue2(2, (ring + 2) % STAGES, (ring + 3) % STAGES);
    bool st_young = false;              // the previous epilogue's stores are all issued and counted

    // Epilogues that read global memory (the pre-GELU activations, the old weight gradient) request it while the
    // last K blocks of the tile are still being multiplied: the addresses are the ones the epilogue will store to.
    constexpr bool F32OUT = (EPI == EPI_PARTIAL || EPI == EPI_ACCUM);   // staged in fp32 so that C += acc rounds once
    constexpr int PASSES = F32OUT ? TN : TN / 2;          // a strip row is 128 B: 64 bf16 columns or 32 fp32 columns
    constexpr bool EPI_READS = (EPI == EPI_DGELU || EPI == EPI_ACCUM);
    u32x4 pre_aux[EPI == EPI_DGELU ? TM : 1][2][2];
    bf16x4 pre_old[EPI == EPI_ACCUM ? TM : 1][EPI == EPI_ACCUM ? PASSES : 1][2][2];
    auto prefetch_epilogue = [&](int tm0, int tn0) {
        if (!EPI_READS || (DBG & 4)) return;
        const int wm0 = tm0 + wm * WTM, wn0 = tn0 + wn * WTN;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int pass = 0; pass < PASSES; pass++)
#pragma unroll
                for (int hsel = 0; hsel < 2; hsel++)
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        const int row = t * 8 + (lane >> 3), ch = lane & 7;
                        const int m = wm0 + i * 32 + hsel * 16 + row;
                        if (EPI == EPI_DGELU) {
                            const int n = wn0 + pass * 64 + ch * 8;
                            if (m < g.M && n < g.N) pre_aux[i][hsel][t] = *reinterpret_cast<const u32x4*>(g.aux + (size_t)m * g.ldc + n);
                        } else {
                            const int n = wn0 + pass * 32 + ch * 4;
                            if (m < g.M && n < g.N) pre_old[i][pass][hsel][t] = *reinterpret_cast<const bf16x4*>(g.C + (size_t)m * g.ldc + n);
                        }
                    }
    };

    long long tc[8] = {0, 0, 0, 0, 0, 0, 0, 0};        // DBG & 128: cycle counts by phase (wave 0)
    auto now = [&]() -> long long { return (DBG & 128) ? (long long)__builtin_readcyclecounter() : 0; };
    const long long t_kernel = now();

    while (true) {
        const int m0 = tile_m * BM, n0 = tile_n * BN;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

        // ---- K loop over pairs of K blocks (one barrier per 64 of K), software-pipelined: the operands of the
        // next 16-wide step (and the barrier that publishes the next pair) are requested while the matrix cores
        // work on the current step. Pair p lives in ring slots 2p and 2p+1 (mod STAGES); while pair p is
        // multiplied, pair p+1 is in flight and the fifth slot is spare (the epilogue's).
        bf16x8 fa0[TM], fb0[TN], fa1[TM], fb1[TN];
        const int npairs = nkb >> 1;                              // the host guarantees an even number of K blocks
        auto slot_of = [&](int kb) -> const char* { return lds + ((ring + kb) % STAGES) * STAGE; };
        auto issue_pair = [&](int q) { issue2(2 * q, (ring + 2 * q) % STAGES, (ring + 2 * q + 1) % STAGES); };
        long long ta = now();
        if (npairs >= 2) { if (st_young) wait_vmcnt<2 * CPW + NS_EPI>(); else wait_vmcnt<2 * CPW>(); }
        else wait_vmcnt<0>();
        barrier_no_fence<DBG>();                                  // pair 0 landed for everyone
        long long tb = now();
        tc[0] += tb - ta;
        const long long t_loop = tb;
        read_frags(slot_of(0), 0, fa0, fb0);
        for (int p = 0; p < npairs - 1; p++) {
            read_frags(slot_of(2 * p), 1, fa1, fb1);
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0);
            if (late && p >= 1) issue_pair(p + 1);
            read_frags(slot_of(2 * p + 1), 0, fa0, fb0);
            await_frags(fa1, fb1, Younger{});
            mma(fa1, fb1);
            read_frags(slot_of(2 * p + 1), 1, fa1, fb1);
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0);
            __builtin_amdgcn_s_waitcnt(0xC07F);                   // lgkmcnt(0): this wave is done reading pair p
            ta = now();
            if (p == 0 && st_young) wait_vmcnt<NS_EPI>(); else wait_vmcnt<0>();     // pair p+1 has landed (for this wave's share)
            if (DBG & 128) { tb = now(); tc[6] += tb - ta; }
            barrier_no_fence<DBG>();                              // ... and for everyone; the slots of pair p are free
            if (DBG & 128) { tb = now(); tc[2] += tb - ta; }
            if (!late && p + 2 < npairs) issue_pair(p + 2);
            read_frags(slot_of(2 * p + 2), 0, fa0, fb0);
            await_frags(fa1, fb1, Younger{});
            mma(fa1, fb1);
        }
        {
            const int p = npairs - 1;
            prefetch_epilogue(m0, n0);
            read_frags(slot_of(2 * p), 1, fa1, fb1);
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0);
            read_frags(slot_of(2 * p + 1), 0, fa0, fb0);
            await_frags(fa1, fb1, Younger{});
            mma(fa1, fb1);
            read_frags(slot_of(2 * p + 1), 1, fa1, fb1);
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0);
            await_frags(fa1, fb1, NoneYounger{});
            mma(fa1, fb1);
        }
        if (DBG & 128) { ta = now(); tc[3] += ta - t_loop; }

        // ---- request the next work item's first K blocks, then run the epilogue under them --------
        barrier_no_fence<DBG>();                                       // every wave is done reading the ring
        const int ring_free = (ring + nkb) % STAGES;              // slot the epilogue may use
        const int cur_m0 = m0, cur_n0 = n0, cur_split = split;
        it++;
        const bool have_next = work_item(it, tile_m, tile_n, split);
        int next_nkb = 0;
        if (have_next) {
            kbeg = split * g.k_per_split;
            next_nkb = (min(g.K, kbeg + g.k_per_split) - kbeg) / PBK;
            setup_loads(tile_m * BM, tile_n * BN, kbeg);
            ring = (ring_free + 1) % STAGES;
            issue2(0, ring % STAGES, (ring + 1) % STAGES);
            if (!(DBG & 8192) && next_nkb > 2) issue2(2, (ring + 2) % STAGES, (ring + 3) % STAGES);
        }

        // ---- epilogue ---------------------------------------------------------------------------------
        // wave-private staging strip inside the free ring slot: 16 rows x (128 B + 16 B pad)
        {
            constexpr int STRIP_ROWS = 16;
            constexpr int STRIP = STRIP_ROWS * EPI_PITCH;
            static_assert(NW * STRIP <= STAGE, "all strips must fit in one ring slot");
            char* strip = lds + ring_free * STAGE + wave * STRIP;
            const int wm0 = cur_m0 + wm * WTM, wn0 = cur_n0 + wn * WTN;
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
                                if (m < g.M && n < g.N && !(DBG & 4)) {
                                    if (EPI == EPI_PARTIAL) {
                                        st_cached(reinterpret_cast<u32x4*>(g.partial + ((size_t)cur_split * g.M + m) * g.N + n), raw);
                                    } else {
                                        union { u32x4 u; f32x4 f; } x;
                                        x.u = raw;
                                        floatX* cp = g.C + (size_t)m * g.ldc + n;
                                        bf16x4 old = pre_old[EPI == EPI_ACCUM ? i : 0][EPI == EPI_ACCUM ? pass : 0][hsel][t], o4;
#pragma unroll
                                        for (int e = 0; e < 4; e++) o4[e] = (__bf16)((float)old[e] + x.f[e]);
                                        st_cached(reinterpret_cast<bf16x4*>(cp), o4);
                                    }
                                }
                            } else {
                                const int n = wn0 + pass * 64 + ch * 8;
                                if (m < g.M && n < g.N && !(DBG & 4)) {
                                    const size_t o = (size_t)m * g.ldc + n;
                                    union { u32x4 u; bf16x8 h; } x, y, z;
                                    x.u = raw;
                                    if (EPI == EPI_BIAS_GELU) {
                                        st_out<DBG>(reinterpret_cast<u32x4*>(g.aux + o), x.u);
#pragma unroll
                                        for (int e = 0; e < 8; e++) y.h[e] = (__bf16)gelu_f((float)x.h[e]);
                                        st_out<DBG>(reinterpret_cast<u32x4*>(g.C + o), y.u);
                                    } else if (EPI == EPI_DGELU) {
                                        z.u = pre_aux[EPI == EPI_DGELU ? i : 0][hsel][t];
#pragma unroll
                                        for (int e = 0; e < 8; e++) y.h[e] = (__bf16)(gelu_grad_f((float)z.h[e]) * (float)x.h[e]);
                                        st_out<DBG>(reinterpret_cast<u32x4*>(g.C + o), y.u);
                                    } else {
                                        st_out<DBG>(reinterpret_cast<u32x4*>(g.C + o), x.u);
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
        if ((DBG & 8192) && have_next && next_nkb > 2) issue2(2, (ring + 2) % STAGES, (ring + 3) % STAGES);
        if (DBG & 128) { tb = now(); tc[4] += tb - ta; }
        if (!have_next) break;
        st_young = (DBG & 8192) ? false : cur_m0 + BM <= g.M && cur_n0 + BN <= g.N;    // interior tile: every lane stored, NS_EPI stores per wave
        nkb = next_nkb;
    }
    if ((DBG & 128) && lane == 0) {
        tc[5] = now() - t_kernel;
        long long* o = reinterpret_cast<long long*>(g.partial) + (blockIdx.x * NW + wave) * 8;
        for (int i = 0; i < 8; i++) o[i] = tc[i];
    }
#endif  // __HIP_DEVICE_COMPILE__
}

#endif  // !LLMK_FP32

}  // namespace gemmk
