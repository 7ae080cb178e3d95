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
//   * K advances in stages of 64 through two 64 KiB LDS buffers: one is multiplied while the other fills. One
//     stage ahead is enough to cover the latency (deeper rings of smaller blocks measured no faster), a stage of
//     64 means every row of a K-contiguous operand is fetched as one full 128-byte line, and there is one
//     s_barrier per 64 of K - without a memory fence, which would drain the loads in flight.
//   * A direct-to-LDS load deposits each wave's 64 x 16 B linearly, so the anti-bank-conflict
//     swizzle is applied on the global side: lane p of a row fetches chunk p ^ f(row), and the
//     MFMA operand reads undo it. K-contiguous tiles: [row][64] with f = (row>>1)&7 (ds_read_b128
//     conflict-free). K-major tiles: [k][row] as in memory, f = 4*(k&3), read with the transposing
//     ds_read_b64_tr_b16 so no software transpose is needed for dinp/dweight.
//   * Operand reads are software-pipelined one 16-wide step ahead of the MFMAs, across the barrier.
//   * The two waves that share a SIMD request their part of a stage at different points of the math.
//   * The kernel is persistent (one workgroup per CU walks a list of tiles). When a tile's K loop
//     ends, the first two stages of the NEXT tile are requested while the epilogue stages its output
//     through a third LDS region.
//   * The MFMA is issued with swapped operands (D^T = B.A^T): each lane then owns 4 consecutive
//     output columns of one row, which it writes as 8 bytes into a per-wave LDS staging strip; the
//     strip is read back row-contiguously so that global stores (and the loads of pre_gelu / the
//     old dW for the fused epilogues) are full 128-byte lines.
#pragma once
#include "common.hpp"
#include "gelu.hpp"
#include <type_traits>
#include <utility>

namespace gemmk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

// EPI_PARTIAL_ROWSUM: EPI_PARTIAL plus, per row m of the output, the sum over the split's K range of A(m, k): with
// A = dout^T that is the bias gradient, taken from the operand fragments the matrix cores are being fed anyway.
// EPI_BIAS_GELU_D / EPI_DGELU_D (gelu_fusion 3): the forward epilogue leaves gelu'(pre-activation) in the second output
// instead of the pre-activation, and the backward epilogue multiplies by that stored value: the exponential, the
// reciprocal and nine of the thirteen vector operations per element move out of the backward epilogue, four into the forward one.
// EPI_BIAS_RES: C = bf16(bf16(acc + bias) + aux), the residual stream's add taken into the projection that feeds it
// (both roundings of the two-kernel form: the GEMM's output rounded to bf16, then the sum).
enum Epi { EPI_BIAS = 0, EPI_BIAS_GELU = 1, EPI_STORE = 2, EPI_DGELU = 3, EPI_ACCUM = 4, EPI_PARTIAL = 5, EPI_PARTIAL_ROWSUM = 6,
           EPI_BIAS_GELU_D = 7, EPI_DGELU_D = 8, EPI_BIAS_RES = 9 };
constexpr bool epi_gelu_fwd(int e) { return e == EPI_BIAS_GELU || e == EPI_BIAS_GELU_D; }
constexpr bool epi_gelu_bwd(int e) { return e == EPI_DGELU || e == EPI_DGELU_D; }
// epilogues that read a tensor of the output's shape (g.aux) with the lanes' store pattern
constexpr bool epi_reads_aux(int e) { return epi_gelu_bwd(e) || e == EPI_BIAS_RES; }

struct GemmArgs {
    const floatX* A;
    const floatX* B;
    floatX* C;
    int M, N, K;          // C[M][N] = sum_k A(m,k) * B(n,k)
    int lda, ldb, ldc;    // leading dimensions of the stored matrices, in elements
    const floatX* bias;   // [N] or nullptr                         (EPI_BIAS*)
    floatX* aux;          // pre-GELU output (EPI_BIAS_GELU) / pre-GELU input (EPI_DGELU); gelu' of it for the _D pair
    float* partial;       // [splits][M][N] fp32                    (EPI_PARTIAL*)
    float* rowsum;        // [splits * WGN][M] fp32 (WGN: column waves of the tile configuration)  (EPI_PARTIAL_ROWSUM)
    int k_per_split;      // multiple of the K block
    int splits;
    // Uneven cut of K (EPI_PARTIAL*), or sk_tiles = 0: every one of the sk_tiles output tiles is cut at the same K blocks
    // into one long piece of sk_long blocks (partial slot 0) and splits - 1 short ones that share the rest evenly (slot =
    // rank along K). Workgroup list c = xcd * (grid / 8) + index within the XCD takes the long piece of tile c when
    // c < sk_tiles; the others take sk_each consecutive short pieces, numbered (slot - 1) * sk_tiles + tile.
    int sk_tiles, sk_long, sk_each;
};
constexpr int SK_MAX_ITEMS = 8;         // most short pieces one workgroup takes

#if !defined(LLMK_FP32)

#ifndef LLMK_TR_ASM_BOTH
#define LLMK_TR_ASM_BOTH 1
#endif
#ifndef LLMK_TR_ASM_MIXED
#define LLMK_TR_ASM_MIXED 0
#endif
// Timing-only ablations of the kernel's parts, for llm.c_amd/microbench.py --variant (python llm.c_amd/build.py --variant
// NAME -DLLMK_GEMM_ABL=bits builds a library beside the product one; results of such a build are wrong by design):
//   1  no global -> LDS stage loads after a workgroup's first two stages     2  no matrix instructions
//   4  no fragment reads from LDS                                             8  no epilogue (strip passes and stores)
#ifndef LLMK_GEMM_ABL
#define LLMK_GEMM_ABL 0
#endif
// Switch for a measured alternative, off in the product: the last K stage of a tile taken one 32-row block at a time, each
// finished block's epilogue (strip pass and stores) placed behind the matrix instructions of the next block, the barrier and
// the tile change before the last block. Bit-exact; it needs 20 more registers (253-255) and, timed against the product on
// one machine, both libraries loaded in one process and called in turn: NT bias kernels +2 to +7 % (fc 0.299 -> 0.315 ms,
// fcproj 0.266 -> 0.285, qkv 0.206 -> 0.217), NT GELU +3 to +5 %, NN store within +-1 %, NN GELU backward +20 %. python llm.c_amd/build.py --variant rowwise -DLLMK_ROWWISE_LAST=1 builds it for
// llm.c_amd/microbench.py --variant rowwise (2: also the GELU-backward kernels).
#ifndef LLMK_DGELU_ASM
#define LLMK_DGELU_ASM 1
#endif
#ifndef LLMK_BIAS_ASM
#define LLMK_BIAS_ASM 1
#endif
#ifndef LLMK_ROWWISE_LAST
#define LLMK_ROWWISE_LAST 0
#endif
constexpr int PBK = 64;                 // K per stage
constexpr int STAGES = 2;               // operand buffers: one being multiplied, one being filled
constexpr int KGRAN = PBK;              // K (and the K range of a split) must be a multiple of this
constexpr int LDS_TOTAL = 160 * 1024;

// dynamic LDS of a launch: the operand buffers plus the epilogue's staging strips (32 rows of 128 B per wave)
constexpr int smem_bytes(int bm, int bn, int nw) { return STAGES * (bm + bn) * PBK * 2 + nw * 32 * 128; }

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): loops whose index has to be a constant expression
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F& f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }

// wait until at most N of this wave's vector-memory operations are outstanding (gfx9 encoding, other counters untouched)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}
// Registers loaded by inline asm, whose completion the compiler does not track: after the wait for them they pass through
// here, so that nothing that reads them can move above it
template <typename V>
__device__ __forceinline__ void tie4(V& a, V& b, V& c, V& d) { asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d)); }

// Workgroup barrier WITHOUT the memory fence of __syncthreads(): the fence would wait for every outstanding
// direct-to-LDS load (vmcnt(0)) and serialize the pipeline. Visibility of the K block that is about to be
// read is established by the explicit vmcnt wait each wave does before arriving here.
__device__ __forceinline__ void barrier_no_fence() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Output stores are non-temporal: a tile's output is not read again by this kernel, and a store that allocates in
// L2 is acknowledged late enough (the waves count stores and loads with one counter) to hold up the next tile's loads.
template <typename T>
__device__ __forceinline__ void st_out(T* p, T v) {
    __builtin_nontemporal_store(v, p);
}
// ... except where the next kernel reads a small result straight back (split-K partial sums, weight gradients)
template <typename T>
__device__ __forceinline__ void st_cached(T* p, T v) {
    *p = v;
}

// transposing 8-byte LDS read at addr + OFF (see the kernel for why it is not the builtin)
template <int OFF>
__device__ __forceinline__ s16x4 ds_read_tr16(unsigned addr) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS instruction offsets are 16 bits");
    s16x4 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}

// tile id -> tile coordinates; consecutive ids walk a group of TILE_GROUP rows of tiles column by column. The 32 CUs
// of an XCD then hold 4 row panels and 8 column panels at a time; groups of 8 and 16 measured 0.3 % and 1.5 % slower
// on the whole training step, groups of 2 the same, single rows 0.6 % slower.
#ifndef LLMK_TILE_GROUP
#define LLMK_TILE_GROUP 4
#endif
constexpr int TILE_GROUP = LLMK_TILE_GROUP;
__device__ __forceinline__ void tile_of(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int per_group = TILE_GROUP * tiles_n;
    const int group = t / per_group;
    const int first_m = group * TILE_GROUP;
    const int gsz = min(tiles_m - first_m, TILE_GROUP);
    const int in_group = t - group * per_group;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

template <int BM, int BN, int WGM, int WGN, bool A_T, bool B_T, int EPI>
__global__ void __launch_bounds__(WGM * WGN * 64)
gemm_pipelined_kernel(GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only builtins below; the host pass only needs the launch stub
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN, TM = WTM / 32, TN = WTN / 32;
    constexpr int A_STAGE = BM * PBK * 2, B_STAGE = BN * PBK * 2, STAGE = A_STAGE + B_STAGE;
    constexpr int A_CHUNKS = A_STAGE / 1024, B_CHUNKS = B_STAGE / 1024;
    constexpr bool IS_PARTIAL = (EPI == EPI_PARTIAL || EPI == EPI_PARTIAL_ROWSUM);
    constexpr bool ROWSUM = (EPI == EPI_PARTIAL_ROWSUM);
    static_assert(!ROWSUM || A_T, "row sums are taken from K-major A fragments");
    constexpr int PASSES_OF_EPI = (IS_PARTIAL || EPI == EPI_ACCUM) ? TN : TN / 2;   // epilogue passes over a 32-row block
    constexpr int CPW = (A_CHUNKS + B_CHUNKS) / NW;            // 1 KiB chunks each wave requests per K block
    static_assert((A_CHUNKS + B_CHUNKS) % NW == 0, "chunks must divide evenly over the waves");
    constexpr bool TR_ASM = (A_T && B_T) ? LLMK_TR_ASM_BOTH : LLMK_TR_ASM_MIXED;   // hand-issued or compiler-issued transposing reads
    constexpr int STRIP = 32 * 128;                            // epilogue staging per wave: 32 rows x 128 B
    constexpr int SPARE = (NW * STRIP + 1023) & ~1023;
    static_assert(STAGES * STAGE + SPARE <= LDS_TOTAL, "LDS budget");
    static_assert(TN % 2 == 0, "epilogue strips are 64 columns wide");
    static_assert(A_CHUNKS % NW == 0, "each load slot of a wave must be all-A or all-B");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // scalar: LDS-DMA destinations must be wave-uniform
    const int wm = wave / WGN, wn = wave % WGN;
    // The two waves that share a SIMD (w and w + NW/2) request their share of a K block at different points of
    // the block's math, so that a wave held up at the memory pipeline's entrance always has a partner issuing MFMAs.
    const bool late = wave >= NW / 2;
    const int idx = lane & 31, half = lane >> 5;
    const int tiles_m = CEIL_DIV(g.M, BM), tiles_n = CEIL_DIV(g.N, BN);
    const int num_tiles = tiles_m * tiles_n;
    const int num_work = num_tiles * g.splits;

    // --- this workgroup's share of the work list ---------------------------------------------
    // Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2 (the host launches a multiple
    // of 8). Without split-K and with enough row panels, XCD x owns the row panels [tiles_m*x/8, tiles_m*(x+1)/8)
    // outright and its CUs walk them together, TILE_GROUP panels by all columns at a time: the streamed operand (A) then
    // crosses HBM once. Otherwise XCD x takes the ids [x*G/8, (x+1)*G/8) of every round, so that a split's tiles
    // (which share their K range of both operands) sit on one XCD.
    const int G = gridDim.x;
    auto work_item = [&](int it, int& tm, int& tn, int& sp, int& kb, int& nk) -> bool {
        if constexpr (IS_PARTIAL) {
            if (g.sk_tiles) {                                     // uneven cut: see GemmArgs
                const int c = (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3);
                const int S = g.K / PBK;
                int t;
                if (c < g.sk_tiles) {
                    if (it > 0) return false;
                    t = c; sp = 0; kb = 0; nk = g.sk_long;
                } else {
                    const int q = (c - g.sk_tiles) * g.sk_each + it;
                    if (it >= g.sk_each || q >= g.sk_tiles * (g.splits - 1)) return false;
                    const int j = q / g.sk_tiles, rest = S - g.sk_long;
                    t = q - j * g.sk_tiles; sp = j + 1;
                    const int k0 = g.sk_long + (int)((long long)rest * j / (g.splits - 1));
                    const int k1 = g.sk_long + (int)((long long)rest * (j + 1) / (g.splits - 1));
                    kb = k0 * PBK; nk = k1 - k0;
                }
                tm = t / tiles_n; tn = t - tm * tiles_n;
                return true;
            }
        }
        auto k_range = [&](int split) { kb = split * g.k_per_split; nk = (min(g.K, kb + g.k_per_split) - kb) / PBK; };
        const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3, per_x = G >> 3;
        if (g.splits == 1 && tiles_m >= 64) {
            const int r0 = (tiles_m * xcd) >> 3, rows = ((tiles_m * (xcd + 1)) >> 3) - r0;
            const int q = it * per_x + local;
            if (q >= rows * tiles_n) return false;
            tile_of(q, rows, tiles_n, tm, tn);
            tm += r0;
            sp = 0;
            k_range(0);
            return true;
        }
        const int w = it * G + xcd * per_x + local;
        if (w >= num_work) return false;
        tile_of(w % num_tiles, tiles_m, tiles_n, tm, tn);
        sp = w / num_tiles;
        k_range(sp);
        return true;
    };

    // --- per-thread load descriptors -----------------------------------------------------------
    typedef __attribute__((address_space(3))) const char* lds_cptr;
    const unsigned lds0 = (unsigned)(size_t)(lds_cptr)lds;                 // 1 KiB aligned
    // Each lane's 16 bytes of chunk i sit at (tile base of the operand) + voff[i]; the tile bases and the advance
    // per stage are wave-uniform, so a load costs one 32-bit VGPR of address.
    unsigned voff[CPW];          // byte offset of this lane's 16 bytes inside the operand's tile panel
    int lds_dst[CPW];            // wave-uniform byte offset of the chunk inside a stage
    const char* tile_base[2];    // A and B panels of the current work item at its first K
    const char* tile_base_n[2];  // ... of the next work item, when its first stage is requested before the current one ends
    size_t stage_step[2];        // bytes to advance per stage
    auto bases_into = [&](const char* (&tb)[2], int m0, int n0, int kbeg) {
        tb[0] = reinterpret_cast<const char*>(A_T ? g.A + (size_t)kbeg * g.lda + m0 : g.A + (size_t)m0 * g.lda + kbeg);
        tb[1] = reinterpret_cast<const char*>(B_T ? g.B + (size_t)kbeg * g.ldb + n0 : g.B + (size_t)n0 * g.ldb + kbeg);
    };
    auto setup_bases = [&](int m0, int n0, int kbeg) {
        bases_into(tile_base, m0, n0, kbeg);
        stage_step[0] = (A_T ? (size_t)PBK * g.lda : (size_t)PBK) * sizeof(floatX);
        stage_step[1] = (B_T ? (size_t)PBK * g.ldb : (size_t)PBK) * sizeof(floatX);
    };
    // the lane offsets depend on the tile only through the clamping at the matrix edges: interior tiles share them
    auto setup_voff = [&](int m0, int n0) {
#pragma unroll
        for (int i = 0; i < CPW; i++) {
            const int ci = wave + i * NW;
            const bool isA = i * NW < A_CHUNKS;                   // compile-time after unrolling
            const int cc = isA ? ci : ci - A_CHUNKS;
            const int ld = isA ? g.lda : g.ldb;
            const int r0 = isA ? m0 : n0, rmax = isA ? g.M : g.N;
            const bool trans = isA ? A_T : B_T;
            const int R = isA ? BM : BN;
            lds_dst[i] = (isA ? 0 : A_STAGE) + cc * 1024;
            if (!trans) {
                const int row = cc * 8 + (lane >> 3), p = lane & 7;
                const int c = p ^ ((row >> 1) & 7);
                const int lrow = min(row, rmax - 1 - r0);         // rows past the edge re-read the last valid row
                voff[i] = ((unsigned)lrow * (unsigned)ld + c * 8) * (unsigned)sizeof(floatX);
            } else {
                const int byte = cc * 1024 + lane * 16;
                const int krow = byte / (R * 2), p = (byte % (R * 2)) >> 4;
                const int cn = p ^ (4 * (krow & 3));
                const int lcol = (r0 + cn * 8 < rmax) ? cn * 8 : 0;
                voff[i] = ((unsigned)krow * (unsigned)ld + lcol) * (unsigned)sizeof(floatX);
            }
        }
    };
    // The loads are issued from inline asm, M0 (the LDS destination) included: when the compiler knows of a
    // direct-to-LDS load in flight it makes every later LDS read it can see wait for ALL loads, e.g. the epilogue's
    // strip reads for the next tile's first stages. All waiting for these loads is explicit (wait_vmcnt).
    bool abl_loads_on = true;          // (LLMK_GEMM_ABL & 1: switched off after the first two stage requests)
    auto issue_from = [&](const char* const (&tb)[2], int st, int buf) {
        if ((LLMK_GEMM_ABL & 1) && !abl_loads_on) return;
        const unsigned stage = lds0 + buf * STAGE;
        const unsigned long long pa = (unsigned long long)(size_t)(tb[0] + (size_t)st * stage_step[0]);
        const unsigned long long pb = (unsigned long long)(size_t)(tb[1] + (size_t)st * stage_step[1]);
        unsigned saved;
        asm volatile("s_mov_b32 %0, m0" : "=s"(saved));
#pragma unroll
        for (int i = 0; i < CPW; i++)
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :: "s"(stage + lds_dst[i]), "v"(voff[i]), "s"(i * NW < A_CHUNKS ? pa : pb) : "memory");
        asm volatile("s_mov_b32 m0, %0" :: "s"(saved));
    };
    auto issue = [&](int st, int buf) { issue_from(tile_base, st, buf); };

    // --- MFMA operand reads ----------------------------------------------------------------------
    // One LDS address per 32-row fragment and lane, for K step 0 of buffer 0; the other steps and the other buffer
    // are reached by an XOR with the step (K-contiguous tiles: the swizzle is an XOR, so stepping the chunk index
    // commutes with it) or an immediate offset (K-major tiles), so the loop keeps TM + TN address registers.
    auto frag_base = [&](bool trans, int region, int rows, int row0) -> unsigned {
        if (!trans) {
            const int row = row0 + idx, f = (row >> 1) & 7;
            return lds0 + region + row * 128 + ((f ^ half) << 4);
        }
        const int s16 = lane & 15, grp = lane >> 4;
        const int krow = 8 * (grp >> 1) + (s16 >> 2);                      // (krow & 3) is the same for krow + 4 and + 16 s
        const int col = row0 + (grp & 1) * 16 + 4 * (s16 & 3);
        const int cn = (col >> 3) ^ (4 * (krow & 3));
        return lds0 + region + krow * (rows * 2) + cn * 16 + (col & 7) * 2;
    };
    unsigned abase[TM], bbase[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) abase[i] = frag_base(A_T, 0, BM, wm * WTM + i * 32);
#pragma unroll
    for (int j = 0; j < TN; j++) bbase[j] = frag_base(B_T, A_STAGE, BN, wn * WTN + j * 32);
    // K-contiguous tile [row][64]: one 16-byte read
    auto frag_k = [&](unsigned base, int s) -> bf16x8 {
        return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>((size_t)(base ^ (unsigned)(s << 5)));
    };
    // K-major tile [k][row]: two transposing 8-byte reads. They are issued as inline asm on purpose: for the builtin,
    // the compiler cannot tell that the read does not alias the in-flight direct-to-LDS loads and would wait for ALL
    // of them (vmcnt(0)) first, which serialises loading and math. The price is that their completion has to be
    // awaited by hand (await_frags below).
    auto frag_t = [&](unsigned base, auto off_lo, auto off_hi) -> bf16x8 {
        union { struct { s16x4 a, b; } s; bf16x8 v; } u;
        if (TR_ASM) {
            u.s.a = ds_read_tr16<decltype(off_lo)::value>(base);
            u.s.b = ds_read_tr16<decltype(off_hi)::value>(base);
        } else {
            typedef s16x4 __attribute__((address_space(3))) * lp;
            u.s.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lp)(size_t)(base + decltype(off_lo)::value));
            u.s.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lp)(size_t)(base + decltype(off_hi)::value));
        }
        return u.v;
    };

    // fragments of the 16-wide K step S of the buffer at byte offset bufoff
    auto read_frags = [&](unsigned bufoff, auto sc, bf16x8 (&fa)[TM], bf16x8 (&fb)[TN]) {
        constexpr int S = decltype(sc)::value;
        if (LLMK_GEMM_ABL & 4) {                                  // the registers count as rewritten, nothing is read
#pragma unroll
            for (int i = 0; i < TM; i++) asm volatile("" : "+v"(fa[i]));
#pragma unroll
            for (int j = 0; j < TN; j++) asm volatile("" : "+v"(fb[j]));
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; i++) {
            if constexpr (A_T) fa[i] = frag_t(abase[i] + bufoff, std::integral_constant<int, S * 16 * BM * 2>{}, std::integral_constant<int, (S * 16 + 4) * BM * 2>{});
            else fa[i] = frag_k(abase[i] + bufoff, S);
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if constexpr (B_T) fb[j] = frag_t(bbase[j] + bufoff, std::integral_constant<int, S * 16 * BN * 2>{}, std::integral_constant<int, (S * 16 + 4) * BN * 2>{});
            else fb[j] = frag_k(bbase[j] + bufoff, S);
        }
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;
    // Hand-issued (transposing) reads have to be awaited by hand. LDS operations return in order, so "at most
    // YOUNGER operations outstanding" means these operands have arrived when YOUNGER hand-issued reads were
    // requested after them (compiler-issued reads in between only make the wait longer). The operands are tied
    // to the wait so that nothing that uses them moves above it.
    constexpr int TR_READS = (A_T ? 2 * TM : 0) + (B_T ? 2 * TN : 0);       // hand-issued reads per 16-wide step
    auto await_frags = [&](bf16x8 (&fa)[TM], bf16x8 (&fb)[TN], auto younger) {
        if (!TR_ASM) return;
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
    // Row sums of A (EPI_PARTIAL_ROWSUM): in the swapped MFMA the A fragment is the second operand, so lane l of
    // fa[i] holds eight consecutive k of row i*32 + l%32 (k half l/32): a dot product with ones per pair adds them up.
    // The WGN column waves of a row of waves hold the same fragments: they share the work by K, wave wn taking the
    // 16-wide steps s of every stage with s % WGN == wn (one wave-uniform test per step), and only in the first tile
    // column. Each wave writes its own partial, so there are splits * WGN of them per row, added up by the caller.
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    float rsum[ROWSUM ? TM : 1];
    int rowsum_step = -1;                  // the step of a stage this wave sums in the current tile, or none
    auto mma = [&](const bf16x8 (&fa)[TM], const bf16x8 (&fb)[TN], auto step) {
        if (LLMK_GEMM_ABL & 2) {                                  // the fragments count as used, nothing is multiplied
#pragma unroll
            for (int i = 0; i < TM; i++) asm volatile("" :: "v"(fa[i]));
#pragma unroll
            for (int j = 0; j < TN; j++) asm volatile("" :: "v"(fb[j]));
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)   // swapped operands: acc[i][j] = D^T block, rows = n, cols = m
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        if constexpr (ROWSUM) {
            if (rowsum_step == decltype(step)::value % WGN) {     // wave-uniform
                const bf16x2 ones2 = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const bf16x2 pr = {fa[i][2 * e], fa[i][2 * e + 1]};
                        rsum[i] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones2, rsum[i], false);
                    }
            }
        }
    };
    // Waiting for loads: vector-memory operations retire in issue order, so "at most N outstanding" means that
    // everything but the N youngest has landed. The stages of a tile are requested one at a time, so the only
    // younger operations a wait ever has to allow are the second stage of the tile's prologue and the previous
    // tile's output stores (NS_EPI per wave when every lane stored, which holds for interior tiles).
    constexpr int NS_EPI = TM * PASSES_OF_EPI * 4 * (epi_gelu_fwd(EPI) ? 2 : 1);
    static_assert(CPW + NS_EPI <= 63, "vmcnt is a 6-bit counter");

    int it = 0;
    int tile_m, tile_n, split, kbeg, nkb;
    if (!work_item(0, tile_m, tile_n, split, kbeg, nkb)) return;
    auto is_edge = [&](int tm, int tn) -> bool { return tm * BM + BM > g.M || tn * BN + BN > g.N; };
    bool voff_edge = is_edge(tile_m, tile_n);
    setup_bases(tile_m * BM, tile_n * BN, kbeg);
    setup_voff(tile_m * BM, tile_n * BN);
    int par = 0;                        // stage s of the current work item lives in buffer (s + par) & 1
    issue(0, 0);
    if (nkb > 1) issue(1, 1);
    abl_loads_on = false;
    bool st_young = false;              // the previous epilogue's stores are all issued and counted

    // Epilogues that read global memory (the pre-GELU activations, the old weight gradient) request it while the
    // last K blocks of the tile are still being multiplied: the addresses are the ones the epilogue will store to.
    constexpr bool F32OUT = (IS_PARTIAL || EPI == EPI_ACCUM);   // staged in fp32 so that C += acc rounds once
    constexpr int PASSES = F32OUT ? TN : TN / 2;          // a strip row is 128 B: 64 bf16 columns or 32 fp32 columns
    constexpr bool EPI_READS = (EPI == EPI_ACCUM || epi_reads_aux(EPI));
    bf16x4 pre_old[EPI == EPI_ACCUM ? TM : 1][EPI == EPI_ACCUM ? PASSES : 1][2][2];
    // GELU backward: the pre-activation values of the 16 bytes each lane stores per (block, pass, quarter), as it stores them
    u32x4 pre_act[epi_reads_aux(EPI) ? TM : 1][epi_reads_aux(EPI) ? PASSES : 1][4];
    // Row groups of a tile that lies wholly inside the output (no lane tests its row or column): 8 rows x 128 B, lane
    // (row = lane / 8, chunk = lane % 8) at a wave-uniform base (scalar registers) plus one per-lane byte offset that is the
    // same for every group of every tile. The general form costs each load and store a 64-bit address of its own.
    const unsigned row_lane_off = (unsigned)(((lane >> 3) * g.ldc + (lane & 7) * 8) * (int)sizeof(floatX));
    auto group_ptr = [&](const floatX* buf, int row0, int col0) -> char* {
        const size_t off = ((size_t)row0 * g.ldc + col0) * sizeof(floatX);
        const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)off);
        const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(off >> 32));
        return const_cast<char*>(reinterpret_cast<const char*>(buf)) + (((size_t)hi << 32) | lo) + row_lane_off;
    };
    // (measured: 4 % off the kernel whose epilogue only multiplies by a stored derivative, which is short of registers and
    // of little else; 1-2 % slower for the forward epilogues with activation math. The two backward GELU epilogues take
    // this form: it is also what their hand-issued loads below address by)
    constexpr bool UNIFORM_GROUPS = epi_reads_aux(EPI);
    // the wave's part of the tile whose epilogue is running (or about to) lies wholly inside the output: all rows of the tile
    // and the wave's own WTN columns (a tile on the ragged right edge still has waves like that when N is a multiple of WTN)
    bool tile_inside = false;
    auto group_base = [&](const floatX* buf, int row0, int col0) -> const char* {      // the wave-uniform part of group_ptr
        const size_t off = ((size_t)row0 * g.ldc + col0) * sizeof(floatX);
        const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)off);
        const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(off >> 32));
        return reinterpret_cast<const char*>(buf) + (((size_t)hi << 32) | lo);
    };
    // The loads of the backward GELU epilogues (stored derivatives or pre-activations), interior tiles: issued from inline
    // asm and awaited by count, like the stage loads. Left to the compiler, every wait for them is a wait for (nearly) everything in flight: the compiler cannot see
    // the hand-issued stage requests between them, and the epilogue's per-lane edge tests put each of its loads and stores
    // behind a branch, which makes its own count of younger operations collapse to 0-2 - each 32-row block then waits for
    // the previous block's stores to be acknowledged and for the next block's derivatives to arrive, four memory round
    // trips per tile with the matrix cores idle. pre_young[b]: stage requests (units of CPW loads) issued behind the loads
    // of block b (b = 0, 1; the later blocks' loads are issued inside the epilogue, where no stage is requested).
    constexpr bool PRE_ASM = LLMK_DGELU_ASM && UNIFORM_GROUPS && LLMK_ROWWISE_LAST < 2 && LLMK_GEMM_ABL == 0;
    constexpr int PRE_PB = PASSES * 4;   // derivative loads, and output stores, per 32-row block and wave
    int pre_young[2] = {0, 0};
    auto prefetch_epilogue = [&](int tm0, int tn0, int i) {      // the 32-row block i of this wave's tile
        if (!EPI_READS || i >= TM) return;
        const int wm0 = tm0 + wm * WTM, wn0 = tn0 + wn * WTN;
        if constexpr (epi_reads_aux(EPI)) {
            if (tile_inside) {
#pragma unroll
                for (int pass = 0; pass < PASSES; pass++)
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        if constexpr (PRE_ASM) {
                            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(pre_act[i][pass][t])
                                         : "v"(row_lane_off), "s"(group_base(g.aux, wm0 + i * 32 + t * 8, wn0 + pass * 64)));
                        } else {
                            pre_act[i][pass][t] = *reinterpret_cast<const u32x4*>(group_ptr(g.aux, wm0 + i * 32 + t * 8, wn0 + pass * 64));
                        }
                    }
                return;
            }
            int eln = lane;       // (PRE_ASM: the lane's row and chunk are formed here, not kept - and spilled - as loop invariants)
            if constexpr (PRE_ASM) asm volatile("" : "+v"(eln));
#pragma unroll
            for (int pass = 0; pass < PASSES; pass++)
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const int row = t * 8 + (eln >> 3), ch = eln & 7;
                    const int m = wm0 + i * 32 + row;
                    const int n = wn0 + pass * 64 + ch * 8;
                    if (m < g.M && n < g.N) {
                        if constexpr (PRE_ASM) {   // (no load of this kernel is left to the compiler's counting: it would await them all before each hand-issued one)
                            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(pre_act[i][pass][t]) : "v"(g.aux + (size_t)m * g.ldc + n));
                        } else {
                            pre_act[i][pass][t] = *reinterpret_cast<const u32x4*>(g.aux + (size_t)m * g.ldc + n);
                        }
                    }
                }
            return;
        }
#pragma unroll
        for (int pass = 0; pass < PASSES; pass++)
#pragma unroll
            for (int hsel = 0; hsel < 2; hsel++)
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const int row = t * 8 + (lane >> 3), ch = lane & 7;
                    const int m = wm0 + i * 32 + hsel * 16 + row;
                    const int n = wn0 + pass * 32 + ch * 4;
                    if (m < g.M && n < g.N) pre_old[i][pass][hsel][t] = *reinterpret_cast<const bf16x4*>(g.C + (size_t)m * g.ldc + n);
                }
    };


    // Bias of the wave's columns (EPI_BIAS, EPI_BIAS_GELU*). The matrix cores add it, after the tile's last K stage: one more
    // K step whose column-side operand holds bias[n] at k = 0 (lane n of the lower half-wave, element 0; zeros elsewhere)
    // and whose row-side operand holds 1 at k = 0. bf16 x 1 is exact, so every accumulator gets its column's bias in one
    // fp32 addition, as the epilogue's vector add gave it; that is TM x TN matrix instructions per tile while the matrix
    // cores would idle anyway, in place of an unpack and an add per element of the epilogue (64 vector instructions per
    // 32-row block), and two 2-byte loads per lane in place of eight 8-byte ones. Lanes past N, or a null bias, add zero:
    // the epilogue has no bias code at all. The loads are requested at the start of the tile's last stage and claimed
    // (bias_ready) half-way through it. As ordinary loads the compiler awaits them with vmcnt(0), which also waits for
    // every hand-issued tile load in flight, so a kernel with such loads cannot request the next tile's first stage
    // before it has claimed its bias (BIAS_LATE below); the product kernels issue and count them by hand (BIAS_ASM).
    constexpr bool HAS_BIAS = (EPI == EPI_BIAS || EPI == EPI_BIAS_RES || epi_gelu_fwd(EPI));
    unsigned biasw[HAS_BIAS ? TN : 1];   // bias of column j*32 + idx of the wave tile in the low 16 bits (lanes 0-31; 0 in lanes 32-63)
    bool bias_lane[HAS_BIAS ? TN : 1];
    // BIAS_ASM: the two bias loads are issued from inline asm and awaited by count, so the next tile's first stage can be
    // requested as early as in the kernels without a bias (the early waves a whole stage before this tile's last one);
    // bias_young: a stage request of this wave sits behind them. BIAS_LATE (the row-wise variant and the ablation builds):
    // ordinary loads, awaited by the compiler with vmcnt(0), and no stage request until they are claimed.
    constexpr bool BIAS_ASM = HAS_BIAS && LLMK_BIAS_ASM && LLMK_ROWWISE_LAST == 0 && LLMK_GEMM_ABL == 0;
    constexpr bool BIAS_LATE = HAS_BIAS && !BIAS_ASM;
    bool bias_young = false;
    auto request_bias = [&](int n0) {
        if constexpr (HAS_BIAS) {
            int bln = lane;       // (as above: with epilogue loads in flight a reload of a spilled lane value would wait for them)
            if constexpr (PRE_ASM) asm volatile("" : "+v"(bln));
            const int idx = bln & 31, half = bln >> 5;
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int n = n0 + wn * WTN + j * 32 + idx;
                bias_lane[j] = g.bias != nullptr && half == 0 && n < g.N;
                // unconditional, so that the value stays in the register it arrives in: lanes without a bias read the first
                // bytes of A, which are there, and drop what they got when they claim it
                const floatX* bp = bias_lane[j] ? g.bias + n : g.A;
                if constexpr (BIAS_ASM) asm volatile("global_load_ushort %0, %1, off" : "=v"(biasw[j]) : "v"(bp));
                else biasw[j] = *reinterpret_cast<const unsigned short*>(bp);
            }
            bias_young = false;
            asm volatile("" ::: "memory");                        // the loads stay here: nothing below may pull them down to their use
        }
    };
    auto bias_ready = [&]() {
        if constexpr (HAS_BIAS) {
            if constexpr (BIAS_ASM) {
                // behind the bias loads: the first block's loads of an epilogue that reads (interior tile: all of them
                // issued; an edge tile waits for everything) and the late waves' request of the next tile's first stage
                constexpr int PB = PRE_ASM ? PRE_PB : 0;
                if (PRE_ASM && !tile_inside) wait_vmcnt<0>();
                else if (bias_young) wait_vmcnt<PB + CPW>();
                else wait_vmcnt<PB>();
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                asm volatile("" : "+v"(biasw[j]));
                biasw[j] = bias_lane[j] ? biasw[j] : 0u;
            }
        }
    };
    // acc[i][*] += bias: the one-hot K step for the 32-row block i (after bias_ready)
    auto add_bias = [&](auto ic) {
        if constexpr (HAS_BIAS && !(LLMK_GEMM_ABL & 2)) {
            constexpr int i = decltype(ic)::value;
            union { unsigned u[4]; bf16x8 v; } one, bj;
            one.u[0] = half == 0 ? 0x3F80u : 0u;                  // bf16 1.0 at k = 0
            one.u[1] = one.u[2] = one.u[3] = 0u;
            bj.u[1] = bj.u[2] = bj.u[3] = 0u;
#pragma unroll
            for (int j = 0; j < TN; j++) {
                bj.u[0] = biasw[j];
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bj.v, one.v, acc[i][j], 0, 0, 0);
            }
        }
    };

    // ---- epilogue of one 32-row block of this wave's tile ---------------------------------------------
    // Wave-private staging strip behind the operand buffers: 32 rows x 128 B, the 16-byte chunk c of row r stored
    // at chunk c ^ ((r >> 1) & 7). One 32-row block of the wave's tile goes through it at a time: every lane
    // writes the 4-column pieces it owns, then the wave reads the rows back 8 lanes to a row and stores
    // full 128-byte lines. e_m0, e_n0, e_split: the tile (they outlive the tile change, which renames the current one).
    int e_m0 = 0, e_n0 = 0, e_split = 0;
    // the derivatives of block i have arrived (PRE_ASM, interior tile). Younger operations of the wave, in issue order: the
    // stage requests counted in pre_young (blocks 0 and 1), the loads of the blocks requested after this one and the stores
    // of the blocks that ran since. The registers are tied to the wait so that nothing that reads them moves above it.
    auto await_pre = [&](auto ic) {
        if constexpr (PRE_ASM) {
            constexpr int i = decltype(ic)::value;
            static_assert(PASSES == 1, "one pass per block");
            constexpr int NEXT = i + 1 < TM ? PRE_PB : 0;         // the next block's loads: behind this block's, ahead of its wait
            constexpr int BASE = i == 0 ? NEXT : PRE_PB + NEXT;   // ... and the previous block's stores
            if (!tile_inside) wait_vmcnt<0>();                    // an edge tile: lanes outside load and store nothing, no count holds
            else if (i >= 2 || pre_young[i < 2 ? i : 0] == 0) wait_vmcnt<BASE>();
            else if (pre_young[i < 2 ? i : 0] == 1) wait_vmcnt<BASE + CPW>();
            else wait_vmcnt<BASE + 2 * CPW>();
            tie4(pre_act[i][0][0], pre_act[i][0][1], pre_act[i][0][2], pre_act[i][0][3]);
        }
    };
    auto epi_block = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const int cur_m0 = e_m0, cur_n0 = e_n0, cur_split = e_split;
        char* strip = lds + STAGES * STAGE + wave * STRIP;
        const int wm0 = cur_m0 + wm * WTM, wn0 = cur_n0 + wn * WTN;
        constexpr int JP = F32OUT ? 1 : 2;                    // 32-column blocks per pass
        (void)cur_split;
        // (PRE_ASM: the lane's strip addresses are formed anew in every block. As loop invariants they were spilled, and a
        // reload is a load the compiler awaits with vmcnt(0): the stage requests and derivative loads in flight with it)
        int e_lane = lane;
        if constexpr (PRE_ASM) asm volatile("" : "+v"(e_lane));
        {
                const int lane = e_lane, idx = lane & 31, half = lane >> 5;
                const int wswz = (idx >> 1) & 7;
#pragma unroll
                for (int pass = 0; pass < PASSES; pass++) {
                    // phase 1: lane (row = idx, half) owns columns 8q + 4*half + 0..3 of each 32-column block
#pragma unroll
                    for (int j = pass * JP; j < (pass + 1) * JP; j++) {
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            const int nl = j * 32 + 8 * q + 4 * half;                 // column inside the wave tile
                            float v[4];
#pragma unroll
                            for (int e = 0; e < 4; e++) v[e] = acc[i][j][4 * q + e];
                            char* dst = strip + idx * 128;
                            if (F32OUT) {                         // 16 bytes: chunk 2q + half
                                f32x4 o = {v[0], v[1], v[2], v[3]};
                                *reinterpret_cast<f32x4*>(dst + (((2 * q + half) ^ wswz) << 4)) = o;
                            } else {                              // 8 bytes: half of chunk 4(j - pass*JP) + q
                                bf16x4 o;
#pragma unroll
                                for (int e = 0; e < 4; e++) o[e] = (__bf16)v[e];
                                *reinterpret_cast<bf16x4*>(dst + ((((j - pass * JP) * 4 + q) ^ wswz) << 4) + half * 8) = o;
                            }
                        }
                    }
                    __builtin_amdgcn_s_waitcnt(0xC07F);          // lgkmcnt(0): the strip is written
                    __builtin_amdgcn_wave_barrier();
                    await_pre(ic);
                    // phase 2: 32 rows x 128 B, 8 lanes per row
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const int row = t * 8 + (lane >> 3), ch = lane & 7;
                        const int m = wm0 + i * 32 + row;
                        u32x4 raw = *reinterpret_cast<const u32x4*>(strip + row * 128 + ((ch ^ ((row >> 1) & 7)) << 4));
                        if (F32OUT) {
                            const int n = wn0 + pass * 32 + ch * 4;
                            if (m < g.M && n < g.N) {
                                if (IS_PARTIAL) {
                                    st_cached(reinterpret_cast<u32x4*>(g.partial + ((size_t)cur_split * g.M + m) * g.N + n), raw);
                                } else {
                                    union { u32x4 u; f32x4 f; } x;
                                    x.u = raw;
                                    floatX* cp = g.C + (size_t)m * g.ldc + n;
                                    bf16x4 old = pre_old[EPI == EPI_ACCUM ? i : 0][EPI == EPI_ACCUM ? pass : 0][t >> 1][t & 1], o4;
#pragma unroll
                                    for (int e = 0; e < 4; e++) o4[e] = (__bf16)((float)old[e] + x.f[e]);
                                    st_cached(reinterpret_cast<bf16x4*>(cp), o4);
                                }
                            }
                        } else {
                            const int n = wn0 + pass * 64 + ch * 8;
                            if (tile_inside || (m < g.M && n < g.N)) {
                                u32x4 *cptr, *auxptr = nullptr;
                                if (tile_inside) {
                                    cptr = reinterpret_cast<u32x4*>(group_ptr(g.C, wm0 + i * 32 + t * 8, wn0 + pass * 64));
                                    if (epi_gelu_fwd(EPI)) auxptr = reinterpret_cast<u32x4*>(group_ptr(g.aux, wm0 + i * 32 + t * 8, wn0 + pass * 64));
                                } else {
                                    const size_t o = (size_t)m * g.ldc + n;
                                    cptr = reinterpret_cast<u32x4*>(g.C + o);
                                    if (epi_gelu_fwd(EPI)) auxptr = reinterpret_cast<u32x4*>(g.aux + o);
                                }
                                union { u32x4 u; bf16x8 h; } x, y;
                                x.u = raw;
                                if (EPI == EPI_BIAS_GELU) {
                                    st_out(auxptr, x.u);
#pragma unroll
                                    for (int e = 0; e < 8; e++) y.h[e] = (__bf16)gelu_f((float)x.h[e]);
                                    st_out(cptr, y.u);
                                } else if (EPI == EPI_BIAS_GELU_D) {
                                    union { u32x4 u; bf16x8 h; } d;
#pragma unroll
                                    for (int e = 0; e < 8; e++) {
                                        float gr;
                                        y.h[e] = (__bf16)gelu_with_grad_f((float)x.h[e], gr);
                                        d.h[e] = (__bf16)gr;
                                    }
                                    st_out(auxptr, d.u);
                                    st_out(cptr, y.u);
                                } else if (EPI == EPI_BIAS_RES) {
                                    union { u32x4 u; bf16x8 h; } pa;
                                    pa.u = pre_act[epi_reads_aux(EPI) ? i : 0][epi_reads_aux(EPI) ? pass : 0][t];
#pragma unroll
                                    for (int e = 0; e < 8; e++) y.h[e] = (__bf16)((float)x.h[e] + (float)pa.h[e]);
                                    st_out(cptr, y.u);
                                } else if (epi_gelu_bwd(EPI)) {
                                    // the product of the rounded gradient and gelu'(pre), as gelu_backward_inplace forms it
                                    // (EPI_DGELU_D: gelu'(pre) is what was stored)
                                    union { u32x4 u; bf16x8 h; } pa;
                                    pa.u = pre_act[epi_reads_aux(EPI) ? i : 0][epi_reads_aux(EPI) ? pass : 0][t];
#pragma unroll
                                    for (int e = 0; e < 8; e++)
                                        y.h[e] = (__bf16)((EPI == EPI_DGELU_D ? (float)pa.h[e] : gelu_grad_f((float)pa.h[e])) * (float)x.h[e]);
                                    st_out(cptr, y.u);
                                } else {
                                    st_out(cptr, x.u);
                                }
                            }
                        }
                    }
                    __builtin_amdgcn_s_waitcnt(0xC07F);          // strip reads done before it is overwritten
                    __builtin_amdgcn_wave_barrier();
                }
                prefetch_epilogue(cur_m0, cur_n0, i + 2);
        }
    };

    while (true) {
        const int m0 = tile_m * BM, n0 = tile_n * BN;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
        if constexpr (ROWSUM) {
            rowsum_step = tile_n == 0 ? wn : -1;
#pragma unroll
            for (int i = 0; i < TM; i++) rsum[i] = 0.f;
        }

        // ---- K loop over stages of 64, software-pipelined: the operands of the next 16-wide step (and the
        // barrier that publishes the next stage) are requested while the matrix cores work on the current step.
        // Stage s lives in buffer (s + par) & 1; while it is multiplied, stage s+1 is in flight.
        bf16x8 fa0[TM], fb0[TN], fa1[TM], fb1[TN];
        const int nst = nkb;
        // the next work item's coordinates are worked out here (integer divisions), under the K loop's MFMAs
        int next_m, next_n, next_split, next_kbeg = 0, next_nkb = 0;
        const bool have_next = work_item(it + 1, next_m, next_n, next_split, next_kbeg, next_nkb);
        auto buf_idx = [&](int st) -> int { return (st + par) & 1; };
        auto buf_of = [&](int st) -> unsigned { return (unsigned)buf_idx(st) * STAGE; };
        // The last-but-one stage frees a buffer a whole stage before the tile ends: the next work item's first stage
        // is requested into it there and then instead of at the tile change, and the next item's stages alternate
        // from that buffer on (interior tiles only: they share the lane offsets; not with the += epilogue, whose reads of the old
        // values must stay ahead of these loads, nor for split-K partials, whose tiles are long and whose kernel is
        // short of scalar registers).
        constexpr bool EARLY0 = EPI != EPI_ACCUM && !IS_PARTIAL;
        constexpr bool ROWWISE = LLMK_ROWWISE_LAST && EARLY0 && !TR_ASM && (!epi_reads_aux(EPI) || LLMK_ROWWISE_LAST >= 2);
        bool early0 = false;
        if (have_next) {
            if constexpr (EARLY0) {
                early0 = nst >= 2 && !voff_edge && !is_edge(next_m, next_n);
                if (early0) bases_into(tile_base_n, next_m * BM, next_n * BN, next_kbeg);
            }
        }
        // (with the row-wise last stage a tile's stores are only counted as younger when its successor's first stage was
        // requested ahead of them, half of them ahead of its second stage)
        if (nst >= 2) { if (st_young) wait_vmcnt<CPW + NS_EPI>(); else wait_vmcnt<CPW>(); }
        else wait_vmcnt<0>();
        barrier_no_fence();                                       // stage 0 landed for everyone
        read_frags(buf_of(0), S0{}, fa0, fb0);
        for (int st = 0; st < nst - 1; st++) {
            const unsigned cur = buf_of(st);
            read_frags(cur, S1{}, fa1, fb1);
            // where the late waves request the next stage: behind the step's first matrix instructions, or - the kernels
            // with both operands K-major - ahead of them (measured per kernel family: the other choice costs either 1-4 %;
            // a step or two later costs 9-25 %)
            constexpr bool LATE_AHEAD = A_T && B_T;
            if (LATE_AHEAD && late && st >= 1) issue(st + 1, buf_idx(st + 1));
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0, S0{});
            if (!LATE_AHEAD && late && st >= 1) issue(st + 1, buf_idx(st + 1));
            read_frags(cur, S2{}, fa0, fb0);
            await_frags(fa1, fb1, Younger{});
            mma(fa1, fb1, S1{});
            read_frags(cur, S3{}, fa1, fb1);
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0, S2{});
            __builtin_amdgcn_s_waitcnt(0xC07F);                   // lgkmcnt(0): this wave is done reading stage st
            if (st == 0 && st_young) wait_vmcnt<ROWWISE ? NS_EPI / 2 : NS_EPI>(); else wait_vmcnt<0>();     // stage st+1 has landed (this wave's share)
            barrier_no_fence();                              // ... and for everyone; the buffer of stage st is free
            if (!late) {
                if (st + 2 < nst) issue(st + 2, buf_idx(st));
                else if (EARLY0 && !BIAS_LATE && early0) issue_from(tile_base_n, 0, buf_idx(st));
            }
            read_frags(buf_of(st + 1), S0{}, fa0, fb0);
            await_frags(fa1, fb1, Younger{});
            mma(fa1, fb1, S3{});
        }
        // what happens between the last read of this tile's operands and the epilogue's end: the next work item becomes the
        // current one and its first stages are requested
        auto tile_change = [&]() {
            it++;
            if (!have_next) return;
            tile_m = next_m; tile_n = next_n; split = next_split;
            kbeg = next_kbeg;
            if (EARLY0 && early0) {                               // its first stage is already on the way, in the buffer of stage nst-2
                tile_base[0] = tile_base_n[0]; tile_base[1] = tile_base_n[1];
                par = (nst - 2 + par) & 1;
            } else {
                setup_bases(tile_m * BM, tile_n * BN, kbeg);
                const bool edge = is_edge(tile_m, tile_n);
                if (edge || voff_edge) setup_voff(tile_m * BM, tile_n * BN);
                voff_edge = edge;
                par = 0;
                issue(0, 0);
                pre_young[0]++; pre_young[1]++;
            }
            if (next_nkb > 1) { issue(1, (1 + par) & 1); pre_young[0]++; pre_young[1]++; }
        };
        e_m0 = m0; e_n0 = n0; e_split = split;
        if constexpr (ROWWISE) {
            // The last stage by 32-row blocks: the B fragments of all four steps are held, block i takes its A fragments and
            // its 4 x TN matrix instructions, and the finished block i - 1 goes through the strip and out behind them. The
            // operands are read for the last time before the final block's matrix instructions: the barrier and the tile
            // change sit there, two blocks of output stores ahead of the next tile's second stage and two behind it.
            const unsigned cur = buf_of(nst - 1);
            request_bias(n0);
            tile_inside = UNIFORM_GROUPS && m0 + BM <= g.M && n0 + wn * WTN + WTN <= g.N;
            prefetch_epilogue(m0, n0, 0);
            prefetch_epilogue(m0, n0, 1);
            bf16x8 fbs[3][TN], far[2][3];
            auto read_b = [&](auto sc, bf16x8 (&fb)[TN]) {
                constexpr int S = decltype(sc)::value;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    if (LLMK_GEMM_ABL & 4) asm volatile("" : "+v"(fb[j]));
                    else if constexpr (B_T) fb[j] = frag_t(bbase[j] + cur, std::integral_constant<int, S * 16 * BN * 2>{}, std::integral_constant<int, (S * 16 + 4) * BN * 2>{});
                    else fb[j] = frag_k(bbase[j] + cur, S);
                }
            };
            auto read_a = [&](auto ic, bf16x8 (&fa)[3]) {
                constexpr int i = decltype(ic)::value;
                static_for<3>([&](auto sc) {
                    constexpr int S = decltype(sc)::value + 1;
                    if (LLMK_GEMM_ABL & 4) asm volatile("" : "+v"(fa[S - 1]));
                    else fa[S - 1] = frag_k(abase[i] + cur, S);
                });
            };
            static_assert(!A_T, "row-wise last stage: A fragments are K-contiguous");
            auto mfma1 = [&](f32x16& c, const bf16x8& b, const bf16x8& a) {
                if (LLMK_GEMM_ABL & 2) asm volatile("" :: "v"(a), "v"(b));
                else c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, c, 0, 0, 0);
            };
            read_b(S1{}, fbs[0]);
            read_a(std::integral_constant<int, 0>{}, far[0]);
            read_b(S2{}, fbs[1]);
            read_b(S3{}, fbs[2]);
            static_for<TM>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                if constexpr (i + 1 < TM) read_a(std::integral_constant<int, i + 1>{}, far[(i + 1) & 1]);
                if constexpr (i == TM - 1) {
                    __builtin_amdgcn_s_waitcnt(0xC07F);           // lgkmcnt(0): this wave is done reading the operand buffers
                    barrier_no_fence();                           // ... and so is everyone
                    tile_change();
                }
#pragma unroll
                for (int j = 0; j < TN; j++) mfma1(acc[i][j], fb0[j], fa0[i]);
#pragma unroll
                for (int sidx = 0; sidx < 3; sidx++)
#pragma unroll
                    for (int j = 0; j < TN; j++) mfma1(acc[i][j], fbs[sidx][j], far[i & 1][sidx]);
                if constexpr (i == 0) {
                    bias_ready();
                    if (early0 && (HAS_BIAS || late)) issue_from(tile_base_n, 0, buf_idx(nst - 2));   // (the early waves of a kernel without bias: one stage ago)
                }
                add_bias(ic);
                if constexpr (i >= 1) {
                    if (!(LLMK_GEMM_ABL & 8)) epi_block(std::integral_constant<int, i - 1>{});
                }
            });
        } else {
            const unsigned cur = buf_of(nst - 1);
            request_bias(n0);                                     // nothing of this wave is in flight here (kernels with a bias)
            tile_inside = UNIFORM_GROUPS && m0 + BM <= g.M && n0 + wn * WTN + WTN <= g.N;
            prefetch_epilogue(m0, n0, 0);
            read_frags(cur, S1{}, fa1, fb1);
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0, S0{});
            pre_young[0] = pre_young[1] = 0;
            if (EARLY0 && !BIAS_LATE && late && early0) { issue_from(tile_base_n, 0, buf_idx(nst - 2)); pre_young[0]++; bias_young = true; }
            read_frags(cur, S2{}, fa0, fb0);
            await_frags(fa1, fb1, Younger{});
            mma(fa1, fb1, S1{});
            bias_ready();                                         // two 16-wide steps after the request
            if (EARLY0 && BIAS_LATE && early0) { issue_from(tile_base_n, 0, buf_idx(nst - 2)); pre_young[0]++; }
            read_frags(cur, S3{}, fa1, fb1);
            await_frags(fa0, fb0, Younger{});
            mma(fa0, fb0, S2{});
            await_frags(fa1, fb1, NoneYounger{});
            mma(fa1, fb1, S3{});
            static_for<TM>([&](auto ic) { add_bias(ic); });

            // ---- request the next work item's first K blocks, then run the epilogue under them --------
            barrier_no_fence();                                  // every wave is done reading both buffers
            if constexpr (ROWSUM) {
                if (rowsum_step >= 0) {                               // the two k halves of a row sit 32 lanes apart
#pragma unroll
                    for (int i = 0; i < TM; i++) {
                        const float s = rsum[i] + __shfl_xor(rsum[i], 32, 64);
                        const int m = e_m0 + wm * WTM + i * 32 + idx;
                        if (half == 0 && m < g.M) g.rowsum[((size_t)e_split * WGN + wn) * g.M + m] = s;
                    }
                }
            }
            prefetch_epilogue(e_m0, e_n0, 1);                     // before the next tile's loads: it is needed before them
            tile_change();
        }
        const int cur_m0 = e_m0, cur_n0 = e_n0;

        // ---- epilogue (what the last stage did not already take) ---------------------------------------
        if (LLMK_GEMM_ABL & 8) {                                  // the accumulators count as used, nothing is stored
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) asm volatile("" :: "v"(acc[i][j]));
        } else {
            if constexpr (ROWWISE) {
                epi_block(std::integral_constant<int, TM - 1>{});
            } else {
                static_for<TM>([&](auto ic) { epi_block(ic); });
            }
        }
        if (!have_next) break;
        st_young = !(LLMK_GEMM_ABL & 8) && cur_m0 + BM <= g.M && cur_n0 + BN <= g.N     // interior tile: every lane stored, NS_EPI stores per wave
                   && (!ROWWISE || early0);
        nkb = next_nkb;
    }
#endif  // __HIP_DEVICE_COMPILE__
}

// The kernels with both operands K-major (the weight gradient: EPI_ACCUM, EPI_PARTIAL, EPI_PARTIAL_ROWSUM) live in a
// translation unit of their own, gemm_tn.hip, because they are compiled with another instruction-scheduling strategy
// than the rest of the library (see llm.c_amd/build.py). grid = 0: the usual grid (one workgroup per CU, at most one per
// work item); otherwise that many workgroups (the uneven split of K, whose schedule is derived from the grid size).
void launch_pipelined_tn(GemmArgs g, int splits, bool big, int epi, int grid, hipStream_t st);

#endif  // !LLMK_FP32

}  // namespace gemmk
