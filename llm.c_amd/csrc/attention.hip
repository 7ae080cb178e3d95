// Causal self-attention, forward and backward, as fused flash-style kernels for gfx950.
// Replaces the reference's cuDNN path (llmc/cudnn_att.cpp:222 forward, :256 backward):
// QKV is read in place as (B,T,3,NH,hs), the output is (B,T,NH,hs), and the only thing kept for
// backward is one fp32 log-sum-exp per (b,h,t). CPU definition: train_gpt2.c:271-405.
//
// bf16 build (head size 64). Everything is computed "transposed" so that no softmax statistic
// ever has to cross lanes. A 32x32 MFMA accumulator gives each lane ONE column and 16 rows;
// by computing S^T = K.Q^T the lane's column is a query, so the running max / sum / rescale
// of the online softmax are per-lane scalars (one cross-half exchange per tile for the max).
// The probabilities never leave registers: an accumulator, converted to bf16, already has the
// MFMA B-operand layout (lane = non-contracted index, 8 contracted values), provided the other
// operand is fetched in the same key order — which the transposing LDS read
// (ds_read_b64_tr_b16) does for free. The same identity drives backward:
//   dK/dV kernel: S = Q.K^T (lane = key), P and dS feed dV^T = dO^T.P and dK^T = Q^T.dS
//   dQ kernel:    S^T = K.Q^T (lane = query), dS^T feeds dQ^T = K^T.dS^T
// Two kernels instead of one with atomics: every output element has exactly one owner, so the
// result is deterministic, as the reference requests from cuDNN (cudnn_att.cpp:187-189).
//
// fp32 build: straightforward one-wave-per-row kernels (lanes = head dimensions), used only for
// parity runs against the CPU reference at small sizes.
#include "common.hpp"
#include <type_traits>
#include <utility>
#include "../../include/llmk.h"

namespace {

#if !defined(LLMK_FP32)
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int HS = 64;
constexpr int KP = 144;               // LDS pitch (bytes) of a [row][64 x bf16] tile: 128 + 16, conflict-free for
                                      // both ds_read_b128 down a column of rows and the transposing 8-byte reads
constexpr int TILE_BYTES = 64 * KP;   // 64 rows
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// rows [row0,row0+32) x k in [16s, 16s+16): MFMA operand read along K-contiguous rows
__device__ __forceinline__ bf16x8 frag_rows(const char* tile, int row0, int s, int lane) {
    return *reinterpret_cast<const bf16x8*>(tile + (row0 + (lane & 31)) * KP + (2 * s + (lane >> 5)) * 16);
}
// Transposed operand: lane (idx = lane&31, half = lane>>5) receives, for e = 0..7,
//   tile[kbase + 8*(e/4) + 4*half + e%4][col0 + idx]
// i.e. the contracted index runs over tile ROWS, in exactly the order in which a 32x32
// accumulator's registers r = 8*s2 .. 8*s2+7 enumerate its rows.
__device__ __forceinline__ bf16x8 frag_cols_accorder(const char* tile, int kbase, int col0, int lane) {
    const int s16 = lane & 15, grp = lane >> 4;
    const int row = kbase + 4 * (grp >> 1) + (s16 >> 2);
    const int col = col0 + (grp & 1) * 16 + 4 * (s16 & 3);
    const char* p = tile + row * KP + col * 2;
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 8 * KP));
    union { struct { s16x4 a, b; } s; bf16x8 v; } u;
    u.s.a = lo; u.s.b = hi;
    return u.v;
}
// accumulator registers r = 8*s2 .. 8*s2+7 as a bf16 operand
__device__ __forceinline__ bf16x8 pack_acc(const f32x16& a, int s2) {
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = (__bf16)a[8 * s2 + e];
    return o;
}
// The lane id as a value the compiler cannot trace back: what is derived from it (row offsets, per-lane pointers) is then
// formed where it is used and dies there, instead of being carried in registers through the tile loops of kernels that
// have none to spare.
__device__ __forceinline__ int fresh_lane(int lane) {
    asm volatile("" : "+v"(lane));
    return lane;
}
// max of a value with the one held by the lane 32 away (the other 16 keys of each 32-key block): one lane swap inside
// the vector ALU instead of a trip through the LDS crossbar, which sits in every step's dependent chain
__device__ __forceinline__ float fa_max_with_other_half(float v) {
    // As an instruction, not through __builtin_amdgcn_permlane32_swap: this compiler hands back the first result for both
    // elements of the builtin's pair, which silently drops the maximum (and overflows the exponentials as soon as scores
    // are large). The two wait states are the ones the compiler puts between a vector write and this instruction.
    unsigned a = __builtin_bit_cast(unsigned, v), b = a;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
// row index (within a 32-row block) of accumulator register r for this lane
__device__ __forceinline__ int acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

// The causal mask of a 32 x 32 block on the diagonal (its first row and its first column are the same position; the
// direct-to-LDS kernels meet no other kind, all their blocks start at multiples of 32). Register r of lane l is row
// acc_row(r, l) against column l % 32, so WHICH LANES are masked in register r is a constant of r: a 64-bit lane mask
// that lives in scalar registers, and one select per element - where the per-lane form took an add, a compare and a
// select each, with wait states between them, a tenth of the forward loop's vector instructions at T = 1024.
// ROW_GT: rows past the column are masked (rows are keys: forward, dQ); else rows before it (rows are queries: dK/dV).
template <int R, bool ROW_GT>
constexpr unsigned long long fa_diag_lanes() {
    unsigned long long m = 0;
    for (int l = 0; l < 64; l++) {
        const int row = (R >> 2) * 8 + (l >> 5) * 4 + (R & 3), col = l & 31;
        if (ROW_GT ? row > col : row < col) m |= 1ull << l;
    }
    return m;
}
template <int R, bool ROW_GT>
__device__ __forceinline__ float fa_mask_one(float x, float fill) {
    // (the builtin, not the instruction in asm: x comes straight out of an MFMA, and the wait states between a matrix
    // instruction and a vector instruction that reads its result are the compiler's to insert - it does not look into asm)
    return __builtin_amdgcn_inverse_ballot_w64(fa_diag_lanes<R, ROW_GT>()) ? fill : x;
}
template <bool ROW_GT, int... R>
__device__ __forceinline__ void fa_mask_diag_seq(f32x16& a, float fill, std::integer_sequence<int, R...>) {
    ((a[R] = fa_mask_one<R, ROW_GT>(a[R], fill)), ...);
}
template <bool ROW_GT>
__device__ __forceinline__ void fa_mask_diag(f32x16& a, float fill) {
    fa_mask_diag_seq<ROW_GT>(a, fill, std::make_integer_sequence<int, 16>{});
}

// cooperative 64x64 bf16 tile copy global -> registers (2 x 16 B per thread, 256 threads)
struct TileRegs { u32x4 v[2]; };
// `tile` points at the first row of the tile (wave-uniform); thread (row = tid/8, chunk = tid%8) copies rows row and
// row+32. The per-thread part of the address never changes from tile to tile, so it is 32-bit and loop-invariant.
__device__ __forceinline__ void tile_load(TileRegs& t, const floatX* tile, size_t row_stride, int rows_left, int tid) {
    const char* p = reinterpret_cast<const char*>(tile);
    const int row = tid >> 3;
    const unsigned off0 = (unsigned)((size_t)row * row_stride + (tid & 7) * 8) * (unsigned)sizeof(floatX);
    const unsigned off1 = off0 + (unsigned)(32 * row_stride * sizeof(floatX));
    if (rows_left >= 64) {                                // whole tile inside the sequence (wave-uniform)
        t.v[0] = *reinterpret_cast<const u32x4*>(p + off0);
        t.v[1] = *reinterpret_cast<const u32x4*>(p + off1);
    } else {
        const u32x4 z = {0, 0, 0, 0};
        t.v[0] = row < rows_left ? *reinterpret_cast<const u32x4*>(p + off0) : z;
        t.v[1] = row + 32 < rows_left ? *reinterpret_cast<const u32x4*>(p + off1) : z;
    }
}
__device__ __forceinline__ void tile_store(char* tile, const TileRegs& t, int tid) {
    const int off = (tid >> 3) * KP + (tid & 7) * 16;
    *reinterpret_cast<u32x4*>(tile + off) = t.v[0];
    *reinterpret_cast<u32x4*>(tile + off + 32 * KP) = t.v[1];
}
// 4 consecutive head-dim values of one row -> 8-byte store
__device__ __forceinline__ void store4(floatX* p, float a, float b, float c, float d) {
    bf16x4 o;
    o[0] = (__bf16)a; o[1] = (__bf16)b; o[2] = (__bf16)c; o[3] = (__bf16)d;
    *reinterpret_cast<bf16x4*>(p) = o;
}

// ---- tiles filled by direct-to-LDS loads ---------------------------------------------------------
// A 64-row x 64-column bf16 tile stored without padding (128 B per row); the 16-byte chunk c of row r sits at chunk
// c ^ swz(r). A direct-to-LDS load deposits a wave's 64 x 16 B linearly, so the swizzle is applied on the global
// side (lane p of a row fetches chunk p ^ swz(row)). swz is chosen so that 16 consecutive rows read at one chunk
// (MFMA operand along rows) and 4 rows x 32 B (transposing reads) both spread over all banks.
constexpr int SW_TILE = 64 * 128;
// swz = the three bits of row >> 1 in reverse order: rows 2 apart (the ones a transposing read takes from the same half
// of the banks in one cycle) land 64 bytes apart, and the 8 even (odd) rows of a 16-row column read get 8 different chunks.
__device__ __forceinline__ int fa_swz(int row) { return (((row >> 1) & 1) << 2) | (((row >> 2) & 1) << 1) | ((row >> 3) & 1); }
typedef __attribute__((address_space(3))) void* fa_lds_ptr;
struct FaLane {
    unsigned rowb;          // frag along rows: byte offset of (row = lane%32, K step 0); step s is rowb ^ (s << 5)
    unsigned colb0, colb1;  // transposing reads: byte offsets of this lane's two 8-byte pieces for (kbase 0, col0 0)
    unsigned ld_off[2];     // staging: byte offset inside the global tile of this lane's 16 bytes of chunk i (row stride given at init)
    __device__ __forceinline__ void init(int lane, int wave, size_t row_stride) {
        const int idx = lane & 31, half = lane >> 5;
        rowb = idx * 128 + ((half ^ fa_swz(idx)) << 4);
        const int s16 = lane & 15, grp = lane >> 4;
        const int r = 4 * (grp >> 1) + (s16 >> 2), col = (grp & 1) * 16 + 4 * (s16 & 3);
        colb0 = r * 128 + (((col >> 3) ^ fa_swz(r)) << 4) + (col & 7) * 2;
        colb1 = (r + 8) * 128 + (((col >> 3) ^ fa_swz(r + 8)) << 4) + (col & 7) * 2;
#pragma unroll
        for (int i = 0; i < 2; i++) {                     // a 4-wave workgroup: wave w deposits the 1 KiB chunks w and w + 4
            const int row = (wave + 4 * i) * 8 + (lane >> 3), p = lane & 7;
            ld_off[i] = (unsigned)((size_t)row * row_stride + ((p ^ fa_swz(row)) * 8)) * (unsigned)sizeof(floatX);
        }
    }
};
// A wave-uniform pointer, stated as such: pointer arithmetic that follows stays in scalar registers, which is where
// fa_tile_request needs the tile address. (The builtin returns int: the halves are widened as unsigned.)
template <typename T>
__device__ __forceinline__ const T* fa_uniform(const T* p) {
    const unsigned long long v = (unsigned long long)(size_t)p;
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(v >> 32));
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)v);
    return reinterpret_cast<const T*>((size_t)(((unsigned long long)hi << 32) | (unsigned long long)lo));
}
// Request this wave's two chunks of the tile whose first row is at `gtile` (all 64 rows must exist). The loads are
// issued from inline asm, M0 (the LDS destination) included: when the compiler knows of a direct-to-LDS load in
// flight it makes every later LDS read wait for it, whatever the read's address, which would turn the prefetch into
// a synchronous copy. The kernel waits for its loads explicitly (fa_tiles_landed) before the barrier that publishes them.
__device__ __forceinline__ void fa_tile_request(const FaLane& a, const floatX* gtile, unsigned lds_tile, int wave) {
    const unsigned long long g = (unsigned long long)(size_t)gtile;
    const unsigned dst = lds_tile + wave * 1024;
    unsigned saved;
    asm volatile("s_mov_b32 %0, m0\n\t"
                 "s_mov_b32 m0, %1\n\t"
                 "global_load_lds_dwordx4 %3, %2\n\t"
                 "s_add_u32 m0, m0, 0x1000\n\t"
                 "global_load_lds_dwordx4 %4, %2\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(saved) : "s"(dst), "s"(g), "v"(a.ld_off[0]), "v"(a.ld_off[1]) : "memory", "scc");
}
__device__ __forceinline__ void fa_tiles_landed() {
    __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0), other counters untouched; as a builtin, so that the compiler also knows its own loads are done
    asm volatile("" ::: "memory");
}
// LDS reads of these tiles go through integer addresses: a read the compiler can trace to the array that a
// direct-to-LDS load is filling is preceded by a wait for every load in flight, which would undo the prefetch.
__device__ __forceinline__ unsigned fa_lds_addr(const void* p) {
    return (unsigned)(size_t)(__attribute__((address_space(3))) const char*)p;
}
__device__ __forceinline__ bf16x8 fa_frag_rows(unsigned tile, const FaLane& a, int row0, int s) {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>((size_t)(tile + row0 * 128 + (a.rowb ^ (unsigned)(s << 5))));
}
// The same reads for a kernel short of registers: the swizzled address of each step is formed at the read (one
// xor-add) rather than held for the life of the kernel.
// (lane ^ X) + tile as ONE vector instruction issued where it is written: stated in asm, the compiler neither hoists the
// four (eight) variants of an address into registers of their own nor copies the lane part first to protect it. X has to
// be an inline constant (0, 32, 64); 96 takes a xor and an add. `tile` is wave-uniform (a scalar register).
template <int X>
__device__ __forceinline__ unsigned fa_xad(unsigned lane_part, unsigned tile) {
    unsigned r;
    if constexpr (X == 0) asm volatile("v_add_u32 %0, %2, %1" : "=v"(r) : "v"(lane_part), "s"(tile));
    else if constexpr (X <= 64) asm volatile("v_xad_u32 %0, %1, %2, %3" : "=v"(r) : "v"(lane_part), "n"(X), "s"(tile));
    else asm volatile("v_xor_b32 %0, %2, %1\n\tv_add_u32 %0, %3, %0" : "=&v"(r) : "v"(lane_part), "n"(X), "s"(tile));
    return r;
}
template <int S>
__device__ __forceinline__ bf16x8 fa_frag_rows_lean(unsigned tile, const FaLane& a, int row0) {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>((size_t)(fa_xad<(S << 5)>(a.rowb, tile) + (unsigned)(row0 * 128)));
}
__device__ __forceinline__ f32x4 fa_lds_f32x4(unsigned addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>((size_t)addr);
}
// transposed operand of a swizzled tile (the order of frag_cols_accorder): two transposing 8-byte reads
__device__ __forceinline__ bf16x8 fa_frag_cols(unsigned tile, const FaLane& a, int kbase, int col0) {
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
    const unsigned x = col0 ? 64u : 0u, t = tile + kbase * 128;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(size_t)(t + (a.colb0 ^ x)));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(size_t)(t + (a.colb1 ^ x)));
    union { struct { s16x4 a, b; } s; bf16x8 v; } u;
    u.s.a = lo; u.s.b = hi;
    return u.v;
}

template <int COL0>
__device__ __forceinline__ bf16x8 fa_frag_cols_lean(unsigned tile, const FaLane& a, int kbase) {
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
    constexpr int X = COL0 ? 64 : 0;
    const unsigned off = (unsigned)(kbase * 128);
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(size_t)(fa_xad<X>(a.colb0, tile) + off));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(size_t)(fa_xad<X>(a.colb1, tile) + off));
    union { struct { s16x4 a, b; } s; bf16x8 v; } u;
    u.s.a = lo; u.s.b = hi;
    return u.v;
}

// Which (tile along T, batch*head) a workgroup works on. The grid is (tiles, B*NH) with x fastest, and workgroups
// are dealt round-robin over the 8 XCDs, each with its own L2: taken literally, the tiles of one head would land
// on 8 different XCDs and each would pull that head's K and V through its own L2. Instead XCD x takes the heads
// x, x+8, ... and walks all tiles of a head with consecutive workgroups, so a head's K/V cross HBM once.
__device__ __forceinline__ void fa_block_coords(int& tile, int& bh) {
    const int nt = gridDim.x, nbh = gridDim.y;
    tile = blockIdx.x; bh = blockIdx.y;
    if ((nbh & 7) == 0) {
        const int lin = blockIdx.y * nt + blockIdx.x;
        const int xcd = lin & 7, slot = lin >> 3;
        bh = (slot / nt) * 8 + xcd;
        tile = slot % nt;
    }
}

// The running reference point m of a row (log2 units) only has to stay near the row's maximum, not at it: the
// probabilities are exp2(s - m) and the final division by their sum takes m out again. Moving m costs 48 multiplies
// per lane (output and row-sum accumulators), a fifth of the loop's vector work, and with m at the exact maximum some
// row of the 32 moves in most steps. So a row's m follows its maximum only once a score exceeds m by FA_MAX_SLACK;
// until then probabilities may reach 2^FA_MAX_SLACK instead of 1, which neither bf16 nor the fp32 sums mind.
constexpr float FA_MAX_SLACK = 8.0f;

// ---- forward ----------------------------------------------------------------------------------
// grid (ceil(T/128), B*NH), 256 threads: wave w owns queries [128*qt + 32w, +32) and walks the key tiles up to
// its diagonal, 32 keys at a time. The loop is bound by the vector ALU (one exp2 per score costs as much as the
// two MFMAs that score takes part in), so everything else per score is kept to a minimum: the first MFMA of a
// block starts from a constant zero instead of a cleared accumulator, maxima are taken three at a time, and the
// K/V staging loads use a wave-uniform base with per-thread offsets that never change.
template <int NWAVES = 4>
__global__ void __launch_bounds__(NWAVES * 64)
fa_forward_kernel(floatX* __restrict__ out, float* __restrict__ stats, const floatX* __restrict__ qkv, int T, int NH) {
    __shared__ __attribute__((aligned(16))) char sK[2][TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char sV[2][TILE_BYTES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, idx = lane & 31, half = lane >> 5;
    int tile_x, bh;
    fa_block_coords(tile_x, bh);
    const int qt = gridDim.x - 1 - tile_x;              // longest rows first
    const int b = bh / NH, h = bh % NH;
    const int C = NH * HS;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * HS;
    constexpr int GQ = 32 * NWAVES, NT = 64 * NWAVES, NLD = 512 / NT;   // queries per workgroup, threads, 16-byte loads per thread and tile
    const int qw0 = qt * GQ + wave * 32, my_q = qw0 + idx;
    const float c = 0.125f * LOG2E;                       // 1/sqrt(64) folded into the exp2 argument

    bf16x8 qf[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        if (my_q < T) qf[s] = *reinterpret_cast<const bf16x8*>(base + (size_t)my_q * C3 + 16 * s + 8 * half);
        else
#pragma unroll
            for (int e = 0; e < 8; e++) qf[s][e] = (__bf16)0.f;
    }
    f32x16 o[2];
#pragma unroll
    for (int d = 0; d < 2; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[d][r] = 0.f;
    float m = -INFINITY;
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // The softmax denominator is accumulated by the matrix cores, which have cycles to spare here: a ones operand
    // in place of V makes every row of this accumulator the sum over keys of the (bf16-rounded) probabilities of
    // the lane's query - the same rounded values that multiply V.
    f32x16 lacc = zero;
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; e++) ones[e] = (__bf16)1.0f;

    const int last_q = min(qt * GQ + GQ - 1, T - 1);
    const int n_kt = last_q / 64 + 1;
    // staging: thread (row = tid/8, chunk = tid%8) copies NLD rows, NT/8 apart, of the K and of the V tile
    const int srow = tid >> 3, schunk = tid & 7;
    const unsigned g_off = (unsigned)((size_t)srow * C3 + schunk * 8) * (unsigned)sizeof(floatX);
    const unsigned g_step = (unsigned)((NT / 8) * C3 * sizeof(floatX));
    const int l_off = srow * KP + schunk * 16;
    const char* kbase = reinterpret_cast<const char*>(base + C);
    const char* vbase = reinterpret_cast<const char*>(base + 2 * C);
    const size_t tile_step = 64 * C3 * sizeof(floatX);
    u32x4 rk[NLD], rv[NLD];
    auto stage_load = [&](int j) {
        const char* pk = kbase + (size_t)j * tile_step;
        const char* pv = vbase + (size_t)j * tile_step;
        const u32x4 z = {0, 0, 0, 0};
        if (64 * j + 64 <= T) {                          // whole tile inside the sequence (wave-uniform)
#pragma unroll
            for (int i = 0; i < NLD; i++) {
                rk[i] = *reinterpret_cast<const u32x4*>(pk + g_off + i * g_step);
                rv[i] = *reinterpret_cast<const u32x4*>(pv + g_off + i * g_step);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NLD; i++) {
                const bool in = 64 * j + srow + i * (NT / 8) < T;
                rk[i] = in ? *reinterpret_cast<const u32x4*>(pk + g_off + i * g_step) : z;
                rv[i] = in ? *reinterpret_cast<const u32x4*>(pv + g_off + i * g_step) : z;
            }
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            *reinterpret_cast<u32x4*>(sK[buf] + l_off + i * (NT / 8) * KP) = rk[i];
            *reinterpret_cast<u32x4*>(sV[buf] + l_off + i * (NT / 8) * KP) = rv[i];
        }
    };
    stage_load(0);
    stage_store(0);
    __syncthreads();

    for (int j = 0; j < n_kt; j++) {
        const char* tk = sK[j & 1];
        const char* tv = sV[j & 1];
        const bool more = j + 1 < n_kt;
        if (more) stage_load(j + 1);
        auto kfrag = [&](int row0, int s) -> bf16x8 { return frag_rows(tk, row0, s, lane); };
        auto vfrag = [&](int kbase, int col0) -> bf16x8 { return frag_cols_accorder(tv, kbase, col0, lane); };
        if (64 * j <= qw0 + 31) {                          // else: every key of this tile is in the future of this wave
            // S^T for both 32-key blocks, the two accumulation chains interleaved
            f32x16 sacc[2];
            sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(0, 0), qf[0], zero, 0, 0, 0);
            sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(32, 0), qf[0], zero, 0, 0, 0);
#pragma unroll
            for (int s = 1; s < 4; s++) {
                sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(0, s), qf[s], sacc[0], 0, 0, 0);
                sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(32, s), qf[s], sacc[1], 0, 0, 0);
            }
            if (64 * j + 63 > qw0) {                      // diagonal tile: some (key, query) pairs are masked (wave-uniform test)
                asm volatile("" ::: "memory");            // keep this a branch: off the diagonal the selects are pure overhead
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        if (64 * j + 32 * kb + acc_row(r, lane) > my_q) sacc[kb][r] = -INFINITY;
            }
            float mx = fmaxf(sacc[0][0], sacc[1][0]);
#pragma unroll
            for (int r = 1; r < 16; r++) mx = fmaxf(fmaxf(mx, sacc[0][r]), sacc[1][r]);     // v_max3_f32
            mx = fa_max_with_other_half(mx);
            const float m_top = fmaxf(m, mx * c);
            const bool outgrown = m_top > m + FA_MAX_SLACK;
            if (__builtin_amdgcn_ballot_w64(outgrown) != 0) {   // some row's scores outgrew its reference point: rescale
                asm volatile("" ::: "memory");
                // every row decides for itself, so that what a row computes depends on that row's scores alone
                const float m_new = outgrown ? m_top : m;
                const float alpha = fast_exp2(m - m_new);
                m = m_new;
#pragma unroll
                for (int r = 0; r < 16; r++) lacc[r] *= alpha;
#pragma unroll
                for (int d = 0; d < 2; d++)
#pragma unroll
                    for (int r = 0; r < 16; r++) o[d][r] *= alpha;
            }
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    sacc[kb][r] = fast_exp2(fmaf(sacc[kb][r], c, -m));
#pragma unroll
            for (int s2 = 0; s2 < 4; s2++) {
                const bf16x8 pf = pack_acc(sacc[s2 >> 1], s2 & 1);
                lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf, lacc, 0, 0, 0);       // every row: sum over keys of P
#pragma unroll
                for (int d = 0; d < 2; d++)
                    o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfrag(16 * s2, 32 * d), pf, o[d], 0, 0, 0);
            }
        }
        if (more) stage_store((j + 1) & 1);
        __syncthreads();
    }

    const float l = lacc[0];                              // complete: the MFMA already summed over all 32 keys of both halves
    if (my_q < T) {
        const float inv = 1.0f / l;
        floatX* dst = out + ((size_t)b * T + my_q) * C + h * HS;
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                store4(dst + 32 * d + 8 * g + 4 * half, o[d][4 * g] * inv, o[d][4 * g + 1] * inv, o[d][4 * g + 2] * inv, o[d][4 * g + 3] * inv);
        if (stats && half == 0) stats[((size_t)b * NH + h) * T + my_q] = (m + __log2f(l)) * 0.6931471805599453f;
    }
}

// The same forward pass with K and V brought in by direct-to-LDS loads (T a multiple of 128: every tile is whole and a
// query tile walks an even number of key tiles).
// Without the staging registers the kernel fits 128 VGPRs, a fourth wave per SIMD, and with the loads issued from
// inline asm the reads of the tile in use do not wait for the tile in flight. Same arithmetic in the same order as
// fa_forward_kernel: the two give identical bits.
__global__ void __launch_bounds__(256, 4)
fa_forward_dma_kernel(floatX* __restrict__ out, float* __restrict__ stats, const floatX* __restrict__ qkv, int T, int NH, int nq) {
    constexpr int NWAVES = 4;
    __shared__ __attribute__((aligned(1024))) char sK[2][SW_TILE];
    __shared__ __attribute__((aligned(1024))) char sV[2][SW_TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, idx = lane & 31, half = lane >> 5;
    int tile_x, bh;
    fa_block_coords(tile_x, bh);
    // A workgroup takes TWO tiles of 128 queries of its head, nq - 1 - x and then x (one when they coincide): together
    // they walk nq + 1 pairs of key tiles whatever x is, so every workgroup of the launch does the same work, and the
    // second tile's first keys are already on their way when the first tile is stored.
    const int qt_first = nq - 1 - tile_x, qt_second = tile_x;
    const int nphase = qt_first == qt_second ? 1 : 2;
    const int b = bh / NH, h = bh % NH;
    const int C = NH * HS;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * HS;
    // the first K and V tiles are requested before anything else: they travel while the wave fetches its own rows
    const int uwave = __builtin_amdgcn_readfirstlane(wave);
    FaLane la;
    la.init(lane, uwave, C3);
    const floatX* kbase = fa_uniform(base + C);
    const floatX* vbase = fa_uniform(base + 2 * C);
    fa_tile_request(la, kbase, fa_lds_addr(sK[0]), uwave);
    fa_tile_request(la, vbase, fa_lds_addr(sV[0]), uwave);
    constexpr int GQ = 32 * NWAVES;                       // queries per tile
    const float c = 0.125f * LOG2E;                       // 1/sqrt(64) folded into the exp2 argument
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; e++) ones[e] = (__bf16)1.0f;

    for (int phase = 0; phase < nphase; phase++) {
        const int qt = phase == 0 ? qt_first : qt_second;
        const int qw0 = qt * GQ + uwave * 32;             // wave-uniform
        bf16x8 qf[4];
        {
            const int ln = fresh_lane(lane), idx = ln & 31, half = ln >> 5, my_q = qw0 + idx;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if (my_q < T) qf[s] = *reinterpret_cast<const bf16x8*>(base + (size_t)my_q * C3 + 16 * s + 8 * half);
            else
#pragma unroll
                for (int e = 0; e < 8; e++) qf[s][e] = (__bf16)0.f;
        }
        }
        f32x16 o[2];
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[d][r] = 0.f;
        float m = -INFINITY;
        // The softmax denominator is accumulated by the matrix cores, which have cycles to spare here: a ones operand
        // in place of V makes every row of this accumulator the sum over keys of the (bf16-rounded) probabilities of
        // the lane's query - the same rounded values that multiply V.
        f32x16 lacc = zero;

        const int last_q = min(qt * GQ + GQ - 1, T - 1);
        const int n_kt = last_q / 64 + 1;
        // the wave's own rows have arrived (and, for the first tile, the first keys; the second tile's first keys were
        // awaited by the step that ended the first tile): after this the only loads in flight are tile requests
        fa_tiles_landed();
        if (phase == 0) __syncthreads();

        // One step = one tile of 64 keys. The buffer is a compile-time constant (the loop below alternates two copies of
        // the step), so a fragment's LDS address is a lane register plus an immediate: no vector add per read.
        auto step = [&](int j, auto bufc) {
            constexpr int BUF = decltype(bufc)::value;
            const unsigned tk = fa_lds_addr(sK[BUF]), tv = fa_lds_addr(sV[BUF]);
            constexpr int buf = BUF ^ 1;
            if (j + 1 < n_kt) {                          // the other buffer was last read before the barrier that ended the previous step
                fa_tile_request(la, kbase + (size_t)(64 * (j + 1)) * C3, fa_lds_addr(sK[buf]), uwave);
                fa_tile_request(la, vbase + (size_t)(64 * (j + 1)) * C3, fa_lds_addr(sV[buf]), uwave);
            } else if (phase + 1 < nphase) {             // the second tile starts over at the head's first keys
                fa_tile_request(la, kbase, fa_lds_addr(sK[buf]), uwave);
                fa_tile_request(la, vbase, fa_lds_addr(sV[buf]), uwave);
            }
            auto kfrag = [&](int row0, int s) -> bf16x8 { return fa_frag_rows(tk, la, row0, s); };
            auto vfrag = [&](int kb, int col0) -> bf16x8 { return fa_frag_cols(tv, la, kb, col0); };
            if (64 * j <= qw0 + 31) {                          // else: every key of this tile is in the future of this wave
                // S^T for both 32-key blocks, the two accumulation chains interleaved
                f32x16 sacc[2];
                sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(0, 0), qf[0], zero, 0, 0, 0);
                sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(32, 0), qf[0], zero, 0, 0, 0);
#pragma unroll
                for (int s = 1; s < 4; s++) {
                    sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(0, s), qf[s], sacc[0], 0, 0, 0);
                    sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag(32, s), qf[s], sacc[1], 0, 0, 0);
                }
                if (64 * j + 63 > qw0) {                      // diagonal tile: some (key, query) pairs are masked (wave-uniform test)
                    asm volatile("" ::: "memory");            // keep this a branch: off the diagonal the selects are pure overhead
                    // qw0 - 64 j is 0 (the first 32 keys are the wave's diagonal block, the other 32 all in the future) or 32
                    // (the first 32 all visible, the other 32 the diagonal block)
                    if (qw0 == 64 * j) {
                        fa_mask_diag<true>(sacc[0], -INFINITY);
#pragma unroll
                        for (int r = 0; r < 16; r++) sacc[1][r] = -INFINITY;
                    } else {
                        fa_mask_diag<true>(sacc[1], -INFINITY);
                    }
                }
                float mx = fmaxf(sacc[0][0], sacc[1][0]);
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(fmaxf(mx, sacc[0][r]), sacc[1][r]);     // v_max3_f32
                mx = fa_max_with_other_half(mx);
                const float m_top = fmaxf(m, mx * c);
                const bool outgrown = m_top > m + FA_MAX_SLACK;
                if (__builtin_amdgcn_ballot_w64(outgrown) != 0) {   // some row's scores outgrew its reference point: rescale
                    asm volatile("" ::: "memory");
                    // every row decides for itself, so that what a row computes depends on that row's scores alone
                    const float m_new = outgrown ? m_top : m;
                    const float alpha = fast_exp2(m - m_new);
                    m = m_new;
#pragma unroll
                    for (int r = 0; r < 16; r++) lacc[r] *= alpha;
#pragma unroll
                    for (int d = 0; d < 2; d++)
#pragma unroll
                        for (int r = 0; r < 16; r++) o[d][r] *= alpha;
                }
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        sacc[kb][r] = fast_exp2(fmaf(sacc[kb][r], c, -m));
#pragma unroll
                for (int s2 = 0; s2 < 4; s2++) {
                    const bf16x8 pf = pack_acc(sacc[s2 >> 1], s2 & 1);
                    lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf, lacc, 0, 0, 0);       // every row: sum over keys of P
#pragma unroll
                    for (int d = 0; d < 2; d++)
                        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfrag(16 * s2, 32 * d), pf, o[d], 0, 0, 0);
                }
            }
            fa_tiles_landed();
            __syncthreads();
        };
        for (int j = 0; j < n_kt; j += 2) {             // n_kt is even: a tile of 128 queries ends on a multiple of 128 keys
            step(j, std::integral_constant<int, 0>{});
            step(j + 1, std::integral_constant<int, 1>{});
        }

        const float l = lacc[0];                              // complete: the MFMA already summed over all 32 keys of both halves
        const int ln = fresh_lane(lane), idx = ln & 31, half = ln >> 5, my_q = qw0 + idx;
        if (my_q < T) {
            const float inv = 1.0f / l;
            floatX* dst = out + ((size_t)b * T + my_q) * C + h * HS;
#pragma unroll
            for (int d = 0; d < 2; d++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    store4(dst + 32 * d + 8 * g + 4 * half, o[d][4 * g] * inv, o[d][4 * g + 1] * inv, o[d][4 * g + 2] * inv, o[d][4 * g + 3] * inv);
            if (stats && half == 0) stats[((size_t)b * NH + h) * T + my_q] = (m + __log2f(l)) * 0.6931471805599453f;
        }
    }
}

// ---- backward: D[b,h,t] = sum_d dO * O ------------------------------------------------------------
__global__ void __launch_bounds__(256)
fa_dot_do_o_kernel(float* __restrict__ D, const floatX* __restrict__ dout, const floatX* __restrict__ o, int B, int T, int NH) {
    // 8 lanes per (b,t,h) row of 64 values
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t row = gid >> 3;
    const int part = (int)(gid & 7);
    const size_t nrows = (size_t)B * T * NH;
    float s = 0.f;
    if (row < nrows) {
        vecX a = ld_vec(dout + row * HS + part * 8), bb = ld_vec(o + row * HS + part * 8);
#pragma unroll
        for (int k = 0; k < 8; k++) s += to_f32(a[k]) * to_f32(bb[k]);
    }
    s += __shfl_xor(s, 1, WAVE);
    s += __shfl_xor(s, 2, WAVE);
    s += __shfl_xor(s, 4, WAVE);
    if (row < nrows && part == 0) {
        const size_t bt = row / NH;
        const int h = (int)(row % NH);
        const size_t b = bt / T, t = bt % T;
        D[(b * NH + h) * T + t] = s;
    }
}

// ---- backward: dK, dV --------------------------------------------------------------------------------
// grid (ceil(T/128), B*NH): wave w owns keys [128*kt + 32w, +32) and walks all later query tiles
__global__ void __launch_bounds__(256)
fa_backward_dkdv_kernel(floatX* __restrict__ dqkv, const floatX* __restrict__ dout, const floatX* __restrict__ qkv,
                        const float* __restrict__ stats, const float* __restrict__ Dsum, int T, int NH) {
    __shared__ __attribute__((aligned(16))) char sQ[2][TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char sdO[2][TILE_BYTES];
    __shared__ __attribute__((aligned(16))) float sL[2][64];
    __shared__ __attribute__((aligned(16))) float sD[2][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, idx = lane & 31, half = lane >> 5;
    int kt, bh;
    fa_block_coords(kt, bh);
    const int b = bh / NH, h = bh % NH;
    const int C = NH * HS;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * HS;
    const floatX* dobase = dout + (size_t)b * T * C + h * HS;
    const float* lbase = stats + ((size_t)b * NH + h) * T;
    const float* dbase = Dsum + ((size_t)b * NH + h) * T;
    const int kw0 = kt * 128 + wave * 32, my_k = kw0 + idx;
    const float c = 0.125f * LOG2E;

    bf16x8 kf[4], vf[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        if (my_k < T) {
            kf[s] = *reinterpret_cast<const bf16x8*>(base + C + (size_t)my_k * C3 + 16 * s + 8 * half);
            vf[s] = *reinterpret_cast<const bf16x8*>(base + 2 * C + (size_t)my_k * C3 + 16 * s + 8 * half);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) { kf[s][e] = (__bf16)0.f; vf[s][e] = (__bf16)0.f; }
        }
    }
    f32x16 dv[2], dk[2];
#pragma unroll
    for (int d = 0; d < 2; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) { dv[d][r] = 0.f; dk[d][r] = 0.f; }

    const int q_first = (kt * 128) / 64, q_end = CEIL_DIV(T, 64);
    TileRegs rq, rdo;
    float rstat = 0.f;
    auto load_stats = [&](int qi) {
        const int q = 64 * qi + (tid & 63);
        if (tid < 64) rstat = q < T ? lbase[q] * LOG2E : 0.f;
        else if (tid < 128) rstat = q < T ? -dbase[q] : 0.f;          // negated: it is the start value of the dP accumulator
    };
    auto store_stats = [&](int buf) {
        if (tid < 64) sL[buf][tid] = rstat;
        else if (tid < 128) sD[buf][tid - 64] = rstat;
    };
    if (q_first < q_end) {
        tile_load(rq, base + (size_t)(64 * q_first) * C3, C3, T - (64 * q_first), tid);
        tile_load(rdo, dobase + (size_t)(64 * q_first) * (size_t)C, (size_t)C, T - (64 * q_first), tid);
        load_stats(q_first);
        tile_store(sQ[0], rq, tid);
        tile_store(sdO[0], rdo, tid);
        store_stats(0);
    }
    __syncthreads();

    for (int qi = q_first; qi < q_end; qi++) {
        const int buf = (qi - q_first) & 1;
        const char* tq = sQ[buf];
        const char* tdo = sdO[buf];
        const bool more = qi + 1 < q_end;
        if (more) {
            tile_load(rq, base + (size_t)(64 * (qi + 1)) * C3, C3, T - (64 * (qi + 1)), tid);
            tile_load(rdo, dobase + (size_t)(64 * (qi + 1)) * (size_t)C, (size_t)C, T - (64 * (qi + 1)), tid);
            load_stats(qi + 1);
        }
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            const int q0 = 64 * qi + 32 * qb;
            if (q0 + 31 < kw0) continue;                 // all 32 queries precede every key of this wave
            // dP - rowsum(dO*O) comes out of the matrix cores: the accumulator of dO.V^T starts from -rowsum(dO*O) of its
            // 16 queries (an accumulator register is a query here), which takes a subtraction per score off the vector ALU
            f32x16 sacc, pacc;
#pragma unroll
            for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sD[buf][32 * qb + g * 8 + half * 4]);
#pragma unroll
                for (int e = 0; e < 4; e++) pacc[4 * g + e] = d4[e];
            }
            constexpr int LAG = 4;                               // the S chain first, then the dP chain (one loop: see fa_backward_dkdv_dma_kernel)
#pragma unroll
            for (int s = 0; s < 4 + LAG; s++) {
                if (s < 4) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rows(tq, 32 * qb, s, lane), kf[s], sacc, 0, 0, 0);
                if (s >= LAG) pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rows(tdo, 32 * qb, s - LAG, lane), vf[s - LAG], pacc, 0, 0, 0);
            }
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int rr = 32 * qb + g * 8 + half * 4;
                const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sL[buf][rr]);
#pragma unroll
                for (int e = 0; e < 4; e++) sacc[4 * g + e] = fast_exp2(fmaf(sacc[4 * g + e], c, -l4[e]));
            }
            if (q0 < kw0 + 31 || q0 + 31 >= T) {            // diagonal block or rows past the end (wave-uniform test)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int q = q0 + acc_row(r, lane);
                    if (q < my_k || q >= T) sacc[r] = 0.f;
                }
            }
#pragma unroll
            for (int r = 0; r < 16; r++) pacc[r] = sacc[r] * pacc[r];
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                const bf16x8 pf = pack_acc(sacc, s2);
#pragma unroll
                for (int d = 0; d < 2; d++)
                    dv[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_cols_accorder(tdo, 32 * qb + 16 * s2, 32 * d, lane), pf, dv[d], 0, 0, 0);
            }
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                const bf16x8 dsf = pack_acc(pacc, s2);
#pragma unroll
                for (int d = 0; d < 2; d++)
                    dk[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_cols_accorder(tq, 32 * qb + 16 * s2, 32 * d, lane), dsf, dk[d], 0, 0, 0);
            }
        }
        if (more) {
            tile_store(sQ[buf ^ 1], rq, tid);
            tile_store(sdO[buf ^ 1], rdo, tid);
            store_stats(buf ^ 1);
        }
        __syncthreads();
    }

    if (my_k < T) {
        floatX* dkp = dqkv + ((size_t)b * T + my_k) * C3 + C + h * HS;
        floatX* dvp = dqkv + ((size_t)b * T + my_k) * C3 + 2 * C + h * HS;
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int col = 32 * d + 8 * g + 4 * half;
                store4(dkp + col, dk[d][4 * g] * 0.125f, dk[d][4 * g + 1] * 0.125f, dk[d][4 * g + 2] * 0.125f, dk[d][4 * g + 3] * 0.125f);
                store4(dvp + col, dv[d][4 * g], dv[d][4 * g + 1], dv[d][4 * g + 2], dv[d][4 * g + 3]);
            }
    }
}

// Same computation with the Q / dO tiles brought in by direct-to-LDS loads (needs T % 64 == 0): no staging registers.
__global__ void __launch_bounds__(256)
fa_backward_dkdv_dma_kernel(floatX* __restrict__ dqkv, const floatX* __restrict__ dout, const floatX* __restrict__ qkv,
                        const float* __restrict__ stats, const float* __restrict__ Dsum, int T, int NH, int nk) {
    // Q tiles in sT[0..1], dO tiles in sT[2..3]. One array, aligned to twice the tile pair: the buffer in use is bit 13 of an
    // LDS address, and the dO tile of a buffer is a constant 2 * SW_TILE behind its Q tile.
    __shared__ __attribute__((aligned(4 * SW_TILE))) char sT[4][SW_TILE];
    static_assert(SW_TILE == 0x2000, "the buffer toggle below is an XOR with the tile size");
    extern __shared__ __attribute__((aligned(16))) float sStat[];   // [2][T]: log-sum-exp (in log2 units) and -rowsum(dO*O) of every query of this head
    float* sLall = sStat;
    float* sDall = sStat + T;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, idx = lane & 31, half = lane >> 5;
    int tile_x, bh;
    fa_block_coords(tile_x, bh);
    // Two tiles of 128 keys per workgroup, x (the one with more queries after it) and then nk - 1 - x (one when they
    // coincide): equal work for every workgroup of the launch, and the second tile's first queries are on their way
    // when the first tile is stored.
    const int kt_first = tile_x, kt_second = nk - 1 - tile_x;
    const int nphase = kt_first == kt_second ? 1 : 2;
    const int b = bh / NH, h = bh % NH;
    const int C = NH * HS;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * HS;      // reassigned below, stated uniform
    const floatX* dobase = dout + (size_t)b * T * C + h * HS;
    const float* lbase = stats + ((size_t)b * NH + h) * T;
    const float* dbase = Dsum + ((size_t)b * NH + h) * T;
    const float c = 0.125f * LOG2E;
    // the first Q and dO tiles are requested before anything else: they travel while the wave fetches its own rows
    const int q_end = CEIL_DIV(T, 64);
    const int uwave = __builtin_amdgcn_readfirstlane(wave);
    FaLane laq, lado;
    laq.init(lane, uwave, C3);
    lado.init(lane, uwave, (size_t)C);
    base = fa_uniform(base);
    dobase = fa_uniform(dobase);
    {
        const int q_first = (kt_first * 128) / 64;
        if (q_first < q_end) {
            fa_tile_request(laq, base + (size_t)(64 * q_first) * C3, fa_lds_addr(sT[0]), uwave);
            fa_tile_request(lado, dobase + (size_t)(64 * q_first) * C, fa_lds_addr(sT[2]), uwave);
        }
        // the per-query statistics of the head go to LDS once (the first tile's queries include the second's): no global
        // loads besides the tiles inside the loops
        for (int q = 64 * q_first + tid; q < T; q += 256) { sLall[q] = lbase[q] * LOG2E; sDall[q] = -dbase[q]; }    // negated: see below
    }
    int buf = 0;
    // LDS addresses of this lane's operand pieces in the Q tile of the buffer in use, one register each: the four K steps
    // of a fragment along rows, and the two 8-byte pieces of a transposing read for the two column halves. Everything
    // else about a read (the 32-query block, the 16-query step, the dO tile) is an immediate offset, and the change of
    // buffer is one XOR per register and iteration: no address arithmetic at the reads themselves (it was a vector add
    // per read, a quarter of the loop's vector instructions).
    unsigned ar[4], ac[4];
    {
        const unsigned t0 = fa_lds_addr(sT[0]);
#pragma unroll
        for (int s = 0; s < 4; s++) ar[s] = t0 + (laq.rowb ^ (unsigned)(s << 5));
        ac[0] = t0 + laq.colb0; ac[1] = t0 + laq.colb1; ac[2] = t0 + (laq.colb0 ^ 64u); ac[3] = t0 + (laq.colb1 ^ 64u);
    }
    typedef const __attribute__((address_space(3))) bf16x8* lds_frag_ptr;
    typedef s16x4 __attribute__((address_space(3))) * lds_tr_ptr;
    auto rows_frag = [&](bool of_do, int qb, int s) -> bf16x8 {
        return *reinterpret_cast<lds_frag_ptr>((size_t)(ar[s] + (unsigned)(32 * qb * 128 + (of_do ? 2 * SW_TILE : 0))));
    };
    auto cols_frag = [&](bool of_do, int kbase, int d) -> bf16x8 {
        const unsigned off = (unsigned)(kbase * 128 + (of_do ? 2 * SW_TILE : 0));
        union { struct { s16x4 a, b; } s; bf16x8 v; } u;
        u.s.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(size_t)(ac[2 * d] + off));
        u.s.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(size_t)(ac[2 * d + 1] + off));
        return u.v;
    };

    for (int phase = 0; phase < nphase; phase++) {
        const int kt = phase == 0 ? kt_first : kt_second;
        const int kw0 = kt * 128 + uwave * 32;           // wave-uniform
        const int q_first = (kt * 128) / 64;
        bf16x8 kf[4], vf[4];
        {
        const int ln = fresh_lane(lane), idx = ln & 31, half = ln >> 5, my_k = kw0 + idx;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if (my_k < T) {
                kf[s] = *reinterpret_cast<const bf16x8*>(base + C + (size_t)my_k * C3 + 16 * s + 8 * half);
                vf[s] = *reinterpret_cast<const bf16x8*>(base + 2 * C + (size_t)my_k * C3 + 16 * s + 8 * half);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) { kf[s][e] = (__bf16)0.f; vf[s][e] = (__bf16)0.f; }
            }
        }
        }
        f32x16 dv[2], dk[2];
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) { dv[d][r] = 0.f; dk[d][r] = 0.f; }
        fa_tiles_landed();                               // the wave's own rows (and, first time, the first tiles and the statistics)
        if (phase == 0) __syncthreads();

        // this lane's four statistics of a 16-query group: one address register per table, advanced by a tile per iteration
        unsigned stat_l = fa_lds_addr(sLall + 64 * q_first) + (unsigned)(lane >> 5) * 16u;
        unsigned stat_d = fa_lds_addr(sDall + 64 * q_first) + (unsigned)(lane >> 5) * 16u;
        for (int qi = q_first; qi < q_end; qi++) {
            buf ^= 1;
            if (qi + 1 < q_end) {
                fa_tile_request(laq, base + (size_t)(64 * (qi + 1)) * C3, fa_lds_addr(sT[buf]), uwave);
                fa_tile_request(lado, dobase + (size_t)(64 * (qi + 1)) * C, fa_lds_addr(sT[2 + buf]), uwave);
            } else if (phase + 1 < nphase) {             // the second tile's first queries
                const int qn = (kt_second * 128) / 64;
                fa_tile_request(laq, base + (size_t)(64 * qn) * C3, fa_lds_addr(sT[buf]), uwave);
                fa_tile_request(lado, dobase + (size_t)(64 * qn) * C, fa_lds_addr(sT[2 + buf]), uwave);
            }
#pragma unroll
            for (int qb = 0; qb < 2; qb++) {
                const int q0 = 64 * qi + 32 * qb;
                if (q0 + 31 < kw0) continue;                 // all 32 queries precede every key of this wave
                // the accumulator of dO.V^T starts from -rowsum(dO*O) of its 16 queries (see fa_backward_dkdv_kernel)
                f32x16 sacc, pacc;
#pragma unroll
                for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f32x4 d4 = fa_lds_f32x4(stat_d + (32 * qb + g * 8) * 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) pacc[4 * g + e] = d4[e];
                }
                // one chain after the other, S first: its exponentials then run under the dP chain's matrix instructions, and
                // the -rowsum(dO*O) values have the S chain's time to arrive from LDS (measured against the two chains
                // interleaved step by step: -9 %). Written as ONE loop on purpose: two loops of four are fused by the
                // compiler, which puts the chains back side by side.
                constexpr int LAG = 4;                           // steps by which the dP chain runs behind the S chain
#pragma unroll
                for (int s = 0; s < 4 + LAG; s++) {
                    if (s < 4) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rows_frag(false, qb, s), kf[s], sacc, 0, 0, 0);
                    if (s >= LAG) pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rows_frag(true, qb, s - LAG), vf[s - LAG], pacc, 0, 0, 0);
                }
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f32x4 l4 = fa_lds_f32x4(stat_l + (32 * qb + g * 8) * 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) sacc[4 * g + e] = fast_exp2(fmaf(sacc[4 * g + e], c, -l4[e]));
                }
                if (q0 < kw0 + 31) {                             // diagonal block (wave-uniform test; T % 64 == 0: no rows past the end)
                    asm volatile("" ::: "memory");                // keep this a branch: off the diagonal the selects are pure overhead
                    fa_mask_diag<false>(sacc, 0.f);               // q0 == kw0: query q0 + acc_row(r) against key kw0 + idx
                }
#pragma unroll
                for (int r = 0; r < 16; r++) pacc[r] = sacc[r] * pacc[r];
                // dV needs only P, dK needs dS: the dV matrix instructions go first and run under the vector work that forms dS
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) {
                    const bf16x8 pf = pack_acc(sacc, s2);
#pragma unroll
                    for (int d = 0; d < 2; d++)
                        dv[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cols_frag(true, 32 * qb + 16 * s2, d), pf, dv[d], 0, 0, 0);
                }
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) {
                    const bf16x8 dsf = pack_acc(pacc, s2);
#pragma unroll
                    for (int d = 0; d < 2; d++)
                        dk[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cols_frag(false, 32 * qb + 16 * s2, d), dsf, dk[d], 0, 0, 0);
                }
            }
#pragma unroll
            for (int s = 0; s < 4; s++) { ar[s] ^= (unsigned)SW_TILE; ac[s] ^= (unsigned)SW_TILE; }    // the other buffer
            // (in asm: as a plain addition the compiler re-bases the reads on the advanced value, with negative offsets that
            // a read cannot encode, and is back to an add per read)
            asm volatile("v_add_u32 %0, 0x100, %0\n\tv_add_u32 %1, 0x100, %1" : "+v"(stat_l), "+v"(stat_d));
            fa_tiles_landed();
            __syncthreads();
        }

        const int ln = fresh_lane(lane), idx = ln & 31, half = ln >> 5, my_k = kw0 + idx;
        if (my_k < T) {
            floatX* dkp = dqkv + ((size_t)b * T + my_k) * C3 + C + h * HS;
            floatX* dvp = dqkv + ((size_t)b * T + my_k) * C3 + 2 * C + h * HS;
#pragma unroll
            for (int d = 0; d < 2; d++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int col = 32 * d + 8 * g + 4 * half;
                    store4(dkp + col, dk[d][4 * g] * 0.125f, dk[d][4 * g + 1] * 0.125f, dk[d][4 * g + 2] * 0.125f, dk[d][4 * g + 3] * 0.125f);
                    store4(dvp + col, dv[d][4 * g], dv[d][4 * g + 1], dv[d][4 * g + 2], dv[d][4 * g + 3]);
                }
        }
    }
}

// ---- backward: dQ ---------------------------------------------------------------------------------------
// grid (ceil(T/128), B*NH): wave w owns queries [128*qt + 32w, +32) and walks the key tiles up to the diagonal
__global__ void __launch_bounds__(256)
fa_backward_dq_kernel(floatX* __restrict__ dqkv, const floatX* __restrict__ dout, const floatX* __restrict__ qkv,
                      const float* __restrict__ stats, const float* __restrict__ Dsum, int T, int NH) {
    __shared__ __attribute__((aligned(16))) char sK[2][TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char sV[2][TILE_BYTES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, idx = lane & 31, half = lane >> 5;
    int tile_x, bh;
    fa_block_coords(tile_x, bh);
    const int qt = gridDim.x - 1 - tile_x;
    const int b = bh / NH, h = bh % NH;
    const int C = NH * HS;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * HS;
    const int qw0 = qt * 128 + wave * 32, my_q = qw0 + idx;
    const float c = 0.125f * LOG2E;

    bf16x8 qf[4], dof[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        if (my_q < T) {
            qf[s] = *reinterpret_cast<const bf16x8*>(base + (size_t)my_q * C3 + 16 * s + 8 * half);
            dof[s] = *reinterpret_cast<const bf16x8*>(dout + ((size_t)b * T + my_q) * C + h * HS + 16 * s + 8 * half);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) { qf[s][e] = (__bf16)0.f; dof[s][e] = (__bf16)0.f; }
        }
    }
    const float lse2 = my_q < T ? stats[((size_t)b * NH + h) * T + my_q] * LOG2E : 0.f;
    const float dsum = my_q < T ? Dsum[((size_t)b * NH + h) * T + my_q] : 0.f;
    f32x16 dq[2];
#pragma unroll
    for (int d = 0; d < 2; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) dq[d][r] = 0.f;

    const int last_q = min(qt * 128 + 127, T - 1);
    const int n_kt = last_q / 64 + 1;
    TileRegs rk, rv;
    tile_load(rk, base + C + (size_t)(0) * C3, C3, T - (0), tid);
    tile_load(rv, base + 2 * C + (size_t)(0) * C3, C3, T - (0), tid);
    tile_store(sK[0], rk, tid);
    tile_store(sV[0], rv, tid);
    __syncthreads();

    for (int j = 0; j < n_kt; j++) {
        const char* tk = sK[j & 1];
        const char* tv = sV[j & 1];
        const bool more = j + 1 < n_kt;
        if (more) {
            tile_load(rk, base + C + (size_t)(64 * (j + 1)) * C3, C3, T - (64 * (j + 1)), tid);
            tile_load(rv, base + 2 * C + (size_t)(64 * (j + 1)) * C3, C3, T - (64 * (j + 1)), tid);
        }
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            const int k0 = 64 * j + 32 * kb;
            if (k0 > qw0 + 31) continue;
            f32x16 sacc, pacc;
#pragma unroll
            for (int r = 0; r < 16; r++) { sacc[r] = 0.f; pacc[r] = 0.f; }
#pragma unroll
            for (int s = 0; s < 4; s++) {
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rows(tk, 32 * kb, s, lane), qf[s], sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rows(tv, 32 * kb, s, lane), dof[s], pacc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 16; r++) sacc[r] = fast_exp2(fmaf(sacc[r], c, -lse2));
            if (k0 + 31 > qw0) {                              // diagonal block (wave-uniform test)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (k0 + acc_row(r, lane) > my_q) sacc[r] = 0.f;
            }
#pragma unroll
            for (int r = 0; r < 16; r++) pacc[r] = sacc[r] * (pacc[r] - dsum);
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                const bf16x8 dsf = pack_acc(pacc, s2);
#pragma unroll
                for (int d = 0; d < 2; d++)
                    dq[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_cols_accorder(tk, 32 * kb + 16 * s2, 32 * d, lane), dsf, dq[d], 0, 0, 0);
            }
        }
        if (more) {
            tile_store(sK[(j + 1) & 1], rk, tid);
            tile_store(sV[(j + 1) & 1], rv, tid);
        }
        __syncthreads();
    }
    if (my_q < T) {
        floatX* dqp = dqkv + ((size_t)b * T + my_q) * C3 + h * HS;
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                store4(dqp + 32 * d + 8 * g + 4 * half, dq[d][4 * g] * 0.125f, dq[d][4 * g + 1] * 0.125f, dq[d][4 * g + 2] * 0.125f,
                       dq[d][4 * g + 3] * 0.125f);
    }
}

// The same kernel with K and V brought in by direct-to-LDS loads (T a multiple of 64), like fa_forward_dma_kernel:
// no staging registers, a fourth wave per SIMD. It also produces D = rowsum(dO * O) itself and writes it out,
// which takes the place of fa_dot_do_o_kernel's pass over dO and O: it runs before the dK/dV kernel.
__global__ void __launch_bounds__(256, 4)
fa_backward_dq_dma_kernel(floatX* __restrict__ dqkv, const floatX* __restrict__ dout, const floatX* __restrict__ qkv,
                          const floatX* __restrict__ o, const float* __restrict__ stats, float* __restrict__ Dsum, int T, int NH,
                          int nq) {
    __shared__ __attribute__((aligned(1024))) char sK[2][SW_TILE];
    __shared__ __attribute__((aligned(1024))) char sV[2][SW_TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, idx = lane & 31, half = lane >> 5;
    int tile_x, bh;
    fa_block_coords(tile_x, bh);
    // two query tiles per workgroup, nq - 1 - x and then x, as in fa_forward_dma_kernel: equal work for every workgroup
    const int qt_first = nq - 1 - tile_x, qt_second = tile_x;
    const int nphase = qt_first == qt_second ? 1 : 2;
    const int b = bh / NH, h = bh % NH;
    const int C = NH * HS;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * HS;
    // the first K and V tiles are requested before anything else: they travel while the wave fetches its own rows
    const int uwave = __builtin_amdgcn_readfirstlane(wave);
    FaLane la;
    la.init(lane, uwave, C3);
    const floatX* kbase = fa_uniform(base + C);
    const floatX* vbase = fa_uniform(base + 2 * C);
    fa_tile_request(la, kbase, fa_lds_addr(sK[0]), uwave);
    fa_tile_request(la, vbase, fa_lds_addr(sV[0]), uwave);
    const float c = 0.125f * LOG2E;
    int buf = 0;

    for (int phase = 0; phase < nphase; phase++) {
        const int qt = phase == 0 ? qt_first : qt_second;
        const int qw0 = qt * 128 + uwave * 32;           // wave-uniform
        bf16x8 qf[4], dof[4];
        float lse2, dsum = 0.f;
        {
        const int ln = fresh_lane(lane), idx = ln & 31, half = ln >> 5, my_q = qw0 + idx;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if (my_q < T) {
                qf[s] = *reinterpret_cast<const bf16x8*>(base + (size_t)my_q * C3 + 16 * s + 8 * half);
                dof[s] = *reinterpret_cast<const bf16x8*>(dout + ((size_t)b * T + my_q) * C + h * HS + 16 * s + 8 * half);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) { qf[s][e] = (__bf16)0.f; dof[s][e] = (__bf16)0.f; }
            }
        }
        lse2 = my_q < T ? stats[((size_t)b * NH + h) * T + my_q] * LOG2E : 0.f;
        // D = rowsum(dO * O) of the lane's query from the dO values it already holds: the two halves of the wave own
        // 32 head dimensions each. The dK/dV kernel, launched after this one, reads D from memory.
        if (my_q < T) {
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const bf16x8 of = *reinterpret_cast<const bf16x8*>(o + ((size_t)b * T + my_q) * C + h * HS + 16 * s + 8 * half);
#pragma unroll
                for (int e = 0; e < 8; e++) dsum = fmaf((float)dof[s][e], (float)of[e], dsum);
            }
        }
        dsum += __shfl_xor(dsum, 32, WAVE);
        if (my_q < T && half == 0) Dsum[((size_t)b * NH + h) * T + my_q] = dsum;
        }
        f32x16 dq[2];
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) dq[d][r] = 0.f;

        const int last_q = min(qt * 128 + 127, T - 1);
        const int n_kt = last_q / 64 + 1;
        fa_tiles_landed();                               // the wave's own rows (and the first keys of the first tile)
        if (phase == 0) __syncthreads();

        for (int j = 0; j < n_kt; j++) {
            const unsigned tk = fa_lds_addr(sK[buf]), tv = fa_lds_addr(sV[buf]);
            buf ^= 1;
            if (j + 1 < n_kt) {                          // the other buffer was last read before the barrier that ended the previous step
                fa_tile_request(la, kbase + (size_t)(64 * (j + 1)) * C3, fa_lds_addr(sK[buf]), uwave);
                fa_tile_request(la, vbase + (size_t)(64 * (j + 1)) * C3, fa_lds_addr(sV[buf]), uwave);
            } else if (phase + 1 < nphase) {             // the second tile starts over at the head's first keys
                fa_tile_request(la, kbase, fa_lds_addr(sK[buf]), uwave);
                fa_tile_request(la, vbase, fa_lds_addr(sV[buf]), uwave);
            }
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                const int k0 = 64 * j + 32 * kb;
                if (k0 > qw0 + 31) continue;
                f32x16 sacc, pacc;
#pragma unroll
                for (int r = 0; r < 16; r++) { sacc[r] = 0.f; pacc[r] = 0.f; }
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<0>(tk, la, 32 * kb), qf[0], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<1>(tk, la, 32 * kb), qf[1], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<2>(tk, la, 32 * kb), qf[2], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<3>(tk, la, 32 * kb), qf[3], sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<0>(tv, la, 32 * kb), dof[0], pacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<1>(tv, la, 32 * kb), dof[1], pacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<2>(tv, la, 32 * kb), dof[2], pacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_rows_lean<3>(tv, la, 32 * kb), dof[3], pacc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) sacc[r] = fast_exp2(fmaf(sacc[r], c, -lse2));
                if (k0 + 31 > qw0) {                              // diagonal block (wave-uniform test)
                    asm volatile("" ::: "memory");                // keep this a branch: off the diagonal the selects are pure overhead
                    fa_mask_diag<true>(sacc, 0.f);                // k0 == qw0: key k0 + acc_row(r) against query qw0 + idx
                }
#pragma unroll
                for (int r = 0; r < 16; r++) pacc[r] = sacc[r] * (pacc[r] - dsum);
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) {
                    const bf16x8 dsf = pack_acc(pacc, s2);
                    dq[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_cols_lean<0>(tk, la, 32 * kb + 16 * s2), dsf, dq[0], 0, 0, 0);
                    dq[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa_frag_cols_lean<32>(tk, la, 32 * kb + 16 * s2), dsf, dq[1], 0, 0, 0);
                }
            }
            fa_tiles_landed();
            __syncthreads();
        }
        const int ln = fresh_lane(lane), idx = ln & 31, half = ln >> 5, my_q = qw0 + idx;
        if (my_q < T) {
            floatX* dqp = dqkv + ((size_t)b * T + my_q) * C3 + h * HS;
#pragma unroll
            for (int d = 0; d < 2; d++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    store4(dqp + 32 * d + 8 * g + 4 * half, dq[d][4 * g] * 0.125f, dq[d][4 * g + 1] * 0.125f, dq[d][4 * g + 2] * 0.125f,
                           dq[d][4 * g + 3] * 0.125f);
        }
    }
}

#endif  // !LLMK_FP32

// =============================================================================================
// Any head size up to 128, either storage type: one wavefront per row, lane l holds head dimensions l and l + 64
// (EPL = 2) or l alone (EPL = 1, hs <= 64). All arithmetic in fp32. The fp32 build's only path; the bf16 build takes
// it for the head sizes its MFMA kernels do not cover (80, 96 and 128 in the GPT-3 descriptors, train_gpt2.cu:538-559).
// =============================================================================================
template <int EPL>
__global__ void __launch_bounds__(256)
att_forward_rows_kernel(floatX* __restrict__ out, float* __restrict__ stats, const floatX* __restrict__ qkv, int B, int T,
                        int NH, int hs) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);       // (b, h, t)
    if (row >= (size_t)B * NH * T) return;
    const int t = (int)(row % T), h = (int)((row / T) % NH), b = (int)(row / ((size_t)T * NH));
    const int C = NH * hs;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * hs;
    const float scale = 1.0f / sqrtf((float)hs);
    bool act[EPL];
    float q[EPL], acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; e++) {
        act[e] = lane + 64 * e < hs;
        q[e] = act[e] ? to_f32(base[(size_t)t * C3 + lane + 64 * e]) : 0.f;
        acc[e] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    for (int t2 = 0; t2 <= t; t2++) {
        float qk = 0.f, v[EPL];
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            const float k = act[e] ? to_f32(base[(size_t)t2 * C3 + C + lane + 64 * e]) : 0.f;
            v[e] = act[e] ? to_f32(base[(size_t)t2 * C3 + 2 * C + lane + 64 * e]) : 0.f;
            qk = e == 0 ? q[e] * k : qk + q[e] * k;
        }
        const float s = wave_sum(qk) * scale;
        const float m_new = fmaxf(m, s);
        const float alpha = expf(m - m_new), p = expf(s - m_new);
#pragma unroll
        for (int e = 0; e < EPL; e++) acc[e] = acc[e] * alpha + p * v[e];
        l = l * alpha + p;
        m = m_new;
    }
#pragma unroll
    for (int e = 0; e < EPL; e++)
        if (act[e]) out[((size_t)b * T + t) * C + h * hs + lane + 64 * e] = from_f32<floatX>(acc[e] / l);
    if (stats && lane == 0) stats[((size_t)b * NH + h) * T + t] = m + logf(l);
}

// dQ: one wave per query row
template <int EPL>
__global__ void __launch_bounds__(256)
att_backward_dq_rows_kernel(floatX* __restrict__ dqkv, const floatX* __restrict__ dout, const floatX* __restrict__ qkv,
                            const floatX* __restrict__ o, const float* __restrict__ stats, int B, int T, int NH, int hs) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (size_t)B * NH * T) return;
    const int t = (int)(row % T), h = (int)((row / T) % NH), b = (int)(row / ((size_t)T * NH));
    const int C = NH * hs;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * hs;
    const float scale = 1.0f / sqrtf((float)hs);
    const size_t orow = ((size_t)b * T + t) * C + h * hs;
    bool act[EPL];
    float q[EPL], go[EPL], dq[EPL], go_o = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; e++) {
        const int d = lane + 64 * e;
        act[e] = d < hs;
        q[e] = act[e] ? to_f32(base[(size_t)t * C3 + d]) : 0.f;
        go[e] = act[e] ? to_f32(dout[orow + d]) : 0.f;
        const float prod = act[e] ? go[e] * to_f32(o[orow + d]) : 0.f;
        go_o = e == 0 ? prod : go_o + prod;
        dq[e] = 0.f;
    }
    const float dsum = wave_sum(go_o);
    const float lse = stats[((size_t)b * NH + h) * T + t];
    for (int t2 = 0; t2 <= t; t2++) {
        float k[EPL], qk = 0.f, gv = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            const int d = lane + 64 * e;
            k[e] = act[e] ? to_f32(base[(size_t)t2 * C3 + C + d]) : 0.f;
            const float v = act[e] ? to_f32(base[(size_t)t2 * C3 + 2 * C + d]) : 0.f;
            qk = e == 0 ? q[e] * k[e] : qk + q[e] * k[e];
            gv = e == 0 ? go[e] * v : gv + go[e] * v;
        }
        const float s = wave_sum(qk) * scale;
        const float dp = wave_sum(gv);
        const float p = expf(s - lse);
#pragma unroll
        for (int e = 0; e < EPL; e++) dq[e] += p * (dp - dsum) * scale * k[e];
    }
#pragma unroll
    for (int e = 0; e < EPL; e++)
        if (act[e]) dqkv[((size_t)b * T + t) * C3 + h * hs + lane + 64 * e] = from_f32<floatX>(dq[e]);
}

// dK, dV: one wave per key row
template <int EPL>
__global__ void __launch_bounds__(256)
att_backward_dkdv_rows_kernel(floatX* __restrict__ dqkv, const floatX* __restrict__ dout, const floatX* __restrict__ qkv,
                              const floatX* __restrict__ o, const float* __restrict__ stats, int B, int T, int NH, int hs) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (size_t)B * NH * T) return;
    const int t2 = (int)(row % T), h = (int)((row / T) % NH), b = (int)(row / ((size_t)T * NH));
    const int C = NH * hs;
    const size_t C3 = 3 * (size_t)C;
    const floatX* base = qkv + (size_t)b * T * C3 + h * hs;
    const float scale = 1.0f / sqrtf((float)hs);
    bool act[EPL];
    float k[EPL], v[EPL], dk[EPL], dv[EPL];
#pragma unroll
    for (int e = 0; e < EPL; e++) {
        const int d = lane + 64 * e;
        act[e] = d < hs;
        k[e] = act[e] ? to_f32(base[(size_t)t2 * C3 + C + d]) : 0.f;
        v[e] = act[e] ? to_f32(base[(size_t)t2 * C3 + 2 * C + d]) : 0.f;
        dk[e] = dv[e] = 0.f;
    }
    for (int t = t2; t < T; t++) {
        const size_t orow = ((size_t)b * T + t) * C + h * hs;
        float q[EPL], go[EPL], go_o = 0.f, qk = 0.f, gv = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            const int d = lane + 64 * e;
            q[e] = act[e] ? to_f32(base[(size_t)t * C3 + d]) : 0.f;
            go[e] = act[e] ? to_f32(dout[orow + d]) : 0.f;
            const float prod = act[e] ? go[e] * to_f32(o[orow + d]) : 0.f;
            go_o = e == 0 ? prod : go_o + prod;
            qk = e == 0 ? q[e] * k[e] : qk + q[e] * k[e];
            gv = e == 0 ? go[e] * v[e] : gv + go[e] * v[e];
        }
        const float dsum = wave_sum(go_o);
        const float s = wave_sum(qk) * scale;
        const float dp = wave_sum(gv);
        const float p = expf(s - stats[((size_t)b * NH + h) * T + t]);
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            dv[e] += p * go[e];
            dk[e] += p * (dp - dsum) * scale * q[e];
        }
    }
#pragma unroll
    for (int e = 0; e < EPL; e++)
        if (act[e]) {
            dqkv[((size_t)b * T + t2) * C3 + C + h * hs + lane + 64 * e] = from_f32<floatX>(dk[e]);
            dqkv[((size_t)b * T + t2) * C3 + 2 * C + h * hs + lane + 64 * e] = from_f32<floatX>(dv[e]);
        }
}

void launch_forward_rows(floatX* out, float* stats, const floatX* qkv, int B, int T, int NH, int hs, hipStream_t st) {
    const unsigned blocks = (unsigned)CEIL_DIV((size_t)B * NH * T, (size_t)4);
    if (hs <= 64) att_forward_rows_kernel<1><<<blocks, 256, 0, st>>>(out, stats, qkv, B, T, NH, hs);
    else att_forward_rows_kernel<2><<<blocks, 256, 0, st>>>(out, stats, qkv, B, T, NH, hs);
}
void launch_backward_rows(floatX* dqkv, const floatX* dout, const floatX* qkv, const floatX* o, const float* stats, int B,
                          int T, int NH, int hs, hipStream_t st) {
    const unsigned blocks = (unsigned)CEIL_DIV((size_t)B * NH * T, (size_t)4);
    if (hs <= 64) {
        att_backward_dq_rows_kernel<1><<<blocks, 256, 0, st>>>(dqkv, dout, qkv, o, stats, B, T, NH, hs);
        att_backward_dkdv_rows_kernel<1><<<blocks, 256, 0, st>>>(dqkv, dout, qkv, o, stats, B, T, NH, hs);
    } else {
        att_backward_dq_rows_kernel<2><<<blocks, 256, 0, st>>>(dqkv, dout, qkv, o, stats, B, T, NH, hs);
        att_backward_dkdv_rows_kernel<2><<<blocks, 256, 0, st>>>(dqkv, dout, qkv, o, stats, B, T, NH, hs);
    }
}


// ---- scratch that needs no allocation ------------------------------------------------------------------------------
// Device memory that exists from the moment the code object is loaded: the rowsum(dO*O) vector of
// llmk_attention_backward_static. Each GPU holds its own copy at its own address; in host code the array's name is
// only a handle for hipGetSymbolAddress, never an address to hand to a kernel.
constexpr size_t STATIC_SCRATCH_FLOATS = (size_t)1 << 20;        // 4 MiB: B*NH*T up to 1048576 (GPT-2 124M at B=64, T=1024 needs 786432)
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];
constexpr int MAX_DEVICES = 64;
float* g_static_scratch[MAX_DEVICES];                             // per device, filled by static_scratch_setup()

float* static_scratch_setup() {
    int dev = -1;
    HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) { llmk::fail(__FILE__, __LINE__, "device index %d out of range", dev); return nullptr; }
    if (!g_static_scratch[dev]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            llmk::fail(__FILE__, __LINE__, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_static_scratch[dev] = (float*)p;
    }
    return g_static_scratch[dev];
}
float* static_scratch_ptr() { return static_scratch_setup(); }    // the current device's copy (looked up once per device)

// Dsum_static: device memory for the B*NH*T floats of rowsum(dO*O), or nullptr to take them from the library workspace
// (which may allocate). With Dsum_static nothing on this path allocates: no workspace, no timing events.
void attention_backward_impl(void* dqkvr, const void* dout, const void* qkvr, const void* o, const float* stats,
                             int B, int T, int NH, int C, void* stream, float* Dsum_static) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(NH > 0 && C % NH == 0, "attention_backward: C=%d not divisible by NH=%d", C, NH);
    LLMK_REQUIRE(stats != nullptr, "attention_backward: stats from the forward pass are required");
    const int hs = C / NH;
    if ((size_t)B * T == 0) return;
    hipStream_t st = (hipStream_t)stream;
    LLMK_REQUIRE(hs <= 128, "attention_backward: head size %d unsupported (up to 128)", hs);
#if !defined(LLMK_FP32)
    if (hs == HS) {
        float* Dsum = Dsum_static ? Dsum_static : (float*)llmk::workspace((size_t)B * NH * T * sizeof(float));
        const size_t nrows = (size_t)B * T * NH;
        const double fwd_flops = 4.0 * B * NH * hs * ((double)T * (T + 1) / 2);
        const dim3 grid(CEIL_DIV(T, 128), B * NH);
        // algorithmic backward work is 2.5x forward (5 contractions vs 2); booked 1.5x on dK/dV, 1.0x on dQ
        if (T % 64 == 0) {                      // whole tiles only: direct-to-LDS kernels, dQ first (it also leaves D for dK/dV)
            {
                llmk::ProfScope prof(Dsum_static != nullptr, "attention_backward_dq", 1.0 * fwd_flops, 6.0 * B * T * C * sizeof(floatX), st);
                const int nq = CEIL_DIV(T, 128);             // a workgroup takes two query tiles
                fa_backward_dq_dma_kernel<<<dim3((nq + 1) / 2, B * NH), 256, 0, st>>>((floatX*)dqkvr, (const floatX*)dout, (const floatX*)qkvr, (const floatX*)o, stats, Dsum, T, NH, nq);
                LAUNCH_CHECK();
            }
            llmk::ProfScope prof(Dsum_static != nullptr, "attention_backward_dkdv", 1.5 * fwd_flops, 6.0 * B * T * C * sizeof(floatX), st);
            if (T <= 4096)                      // 2*T floats of statistics in LDS beside the 32 KiB of tiles
            {
                const int nk = CEIL_DIV(T, 128);             // a workgroup takes two key tiles
                fa_backward_dkdv_dma_kernel<<<dim3((nk + 1) / 2, B * NH), 256, 2 * (size_t)T * sizeof(float), st>>>((floatX*)dqkvr, (const floatX*)dout, (const floatX*)qkvr, stats, Dsum, T, NH, nk);
            }
            else
                fa_backward_dkdv_kernel<<<grid, 256, 0, st>>>((floatX*)dqkvr, (const floatX*)dout, (const floatX*)qkvr, stats, Dsum, T, NH);
            LAUNCH_CHECK();
        } else {
            {
                llmk::ProfScope prof(Dsum_static != nullptr, "attention_backward_dot", 0, 2.0 * B * T * C * sizeof(floatX), st);
                fa_dot_do_o_kernel<<<(unsigned)CEIL_DIV(nrows * 8, (size_t)256), 256, 0, st>>>(Dsum, (const floatX*)dout, (const floatX*)o, B, T, NH);
                LAUNCH_CHECK();
            }
            {
                llmk::ProfScope prof(Dsum_static != nullptr, "attention_backward_dkdv", 1.5 * fwd_flops, 6.0 * B * T * C * sizeof(floatX), st);
                fa_backward_dkdv_kernel<<<grid, 256, 0, st>>>((floatX*)dqkvr, (const floatX*)dout, (const floatX*)qkvr, stats, Dsum, T, NH);
                LAUNCH_CHECK();
            }
            llmk::ProfScope prof(Dsum_static != nullptr, "attention_backward_dq", 1.0 * fwd_flops, 5.0 * B * T * C * sizeof(floatX), st);
            fa_backward_dq_kernel<<<grid, 256, 0, st>>>((floatX*)dqkvr, (const floatX*)dout, (const floatX*)qkvr, stats, Dsum, T, NH);
            LAUNCH_CHECK();
        }
        return;
    }
#endif
    llmk::ProfScope prof(Dsum_static != nullptr, "attention_backward_rows", 2.5 * 4.0 * B * NH * hs * ((double)T * (T + 1) / 2), 6.0 * B * T * C * sizeof(floatX), st);
    launch_backward_rows((floatX*)dqkvr, (const floatX*)dout, (const floatX*)qkvr, (const floatX*)o, stats, B, T, NH, hs, st);
    LAUNCH_CHECK();
}

}  // namespace

namespace llmk {
void attention_static_scratch_init() { (void)static_scratch_setup(); }
}  // namespace llmk

extern "C" {

void llmk_attention_forward(void* out, float* stats, const void* inp, int B, int T, int NH, int C, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE(NH > 0 && C % NH == 0, "attention_forward: C=%d not divisible by NH=%d", C, NH);
    const int hs = C / NH;
    if ((size_t)B * T == 0) return;
    hipStream_t st = (hipStream_t)stream;
    const double fwd_flops = 4.0 * B * NH * hs * ((double)T * (T + 1) / 2);
    llmk::ProfScope prof("attention_forward", fwd_flops, 4.0 * B * T * C * sizeof(floatX), st);
    LLMK_REQUIRE(hs <= 128, "attention_forward: head size %d unsupported (up to 128)", hs);
#if !defined(LLMK_FP32)
    if (hs == HS) {
        LLMK_REQUIRE(((uintptr_t)inp % 16) == 0 && ((uintptr_t)out % 8) == 0, "attention_forward: misaligned buffers");
        if (T % 128 == 0)                       // whole tiles of 128 queries: an even number of key tiles per query tile
        {
            const int nq = CEIL_DIV(T, 128);                 // query tiles of a head; a workgroup takes two of them
            fa_forward_dma_kernel<<<dim3((nq + 1) / 2, B * NH), 256, 0, st>>>((floatX*)out, stats, (const floatX*)inp, T, NH, nq);
        }
        else
            fa_forward_kernel<4><<<dim3(CEIL_DIV(T, 128), B * NH), 256, 0, st>>>((floatX*)out, stats, (const floatX*)inp, T, NH);
        LAUNCH_CHECK();
        return;
    }
#endif
    launch_forward_rows((floatX*)out, stats, (const floatX*)inp, B, T, NH, hs, st);
    LAUNCH_CHECK();
}

size_t llmk_attention_backward_workspace_bytes(int B, int T, int NH) {
    return (size_t)B * NH * T * sizeof(float);                   // rowsum(dO * O), one float per (batch, head, query)
}

void llmk_attention_backward(void* dqkvr, const void* dout, const void* qkvr, const void* o, const float* stats,
                             int B, int T, int NH, int C, void* stream) {
    attention_backward_impl(dqkvr, dout, qkvr, o, stats, B, T, NH, C, stream, nullptr);
}

// The reference's launchers for builds without cuDNN (llmc/attention.cuh:195, :239) keep a permuted copy of Q, K, V and
// the (B,NH,T,T) probabilities between the passes. Here the same buffers carry what the flash kernels need instead: qkvr
// holds Q, K, V as they came (B,T,3,NH,hs), and the first B*NH*T*4 bytes of att hold the fp32 log-sum-exp of every row.
void llmk_attention_forward_fallback(void* out, void* qkvr, void* att, void* inp, int B, int T, int C, int NH, void* stream) {
    if (llmk::failed()) return;
    if ((size_t)B * T == 0) return;
    LLMK_REQUIRE((size_t)T * sizeof(floatX) >= sizeof(float), "attention_forward: T=%d too short for the statistics to fit the att buffer", T);
    LLMK_REQUIRE(((uintptr_t)att % 4) == 0, "attention_forward: att must be 4-byte aligned");
    HIP_CHECK(hipMemcpyAsync(qkvr, inp, (size_t)B * T * 3 * C * sizeof(floatX), hipMemcpyDeviceToDevice, (hipStream_t)stream));
    llmk_attention_forward(out, (float*)att, qkvr, B, T, NH, C, stream);
}

void llmk_attention_backward_fallback(void* dinp, void* dqkvr, void* datt, void* scratch, const void* dout, const void* qkvr,
                                      const void* att, int B, int T, int C, int NH, void* stream) {
    if (llmk::failed()) return;
    (void)dqkvr; (void)datt;                                     // the flash kernels need neither
    if ((size_t)B * T == 0) return;
    // the output of the forward pass is not among the arguments: it is formed again, in scratch (B*T*C elements)
    llmk_attention_forward(scratch, nullptr, qkvr, B, T, NH, C, stream);
    llmk_attention_backward(dinp, dout, qkvr, scratch, (const float*)att, B, T, NH, C, stream);
}

void llmk_attention_backward_static(void* dqkvr, const void* dout, const void* qkvr, const void* o, const float* stats,
                                    int B, int T, int NH, int C, void* stream) {
    if (llmk::failed()) return;
    LLMK_REQUIRE((size_t)B * (size_t)max(NH, 0) * (size_t)T <= STATIC_SCRATCH_FLOATS,
                 "attention_backward_static: B*NH*T = %zu exceeds the %zu floats of static scratch; use llmk_attention_backward",
                 (size_t)B * NH * T, STATIC_SCRATCH_FLOATS);
    float* ptr = static_scratch_ptr();
    if (!ptr) return;                                            // the failure is recorded
    attention_backward_impl(dqkvr, dout, qkvr, o, stats, B, T, NH, C, stream, ptr);
}

}  // extern "C"
