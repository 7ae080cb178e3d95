// The weight-gradient instances of the pipelined GEMM kernel (both operands K-major; gemm_pipelined.hpp), by themselves.
// Reference counterpart: the dweight cuBLASLt call of matmul_backward, llmc/matmul.cuh:254-261.
//
// Why a file of their own: these kernels read their operand fragments with hand-issued transposing LDS reads and
// hand-counted waits, and the compiler's "max-ilp" scheduling strategy arranges that loop 1.2-2.7 % faster than the default
// one (3072 x 768 x 65536: 0.278 -> 0.270 ms; the LM head's 50304 x 768 x 65536: 4.22 -> 4.17 ms), while the same
// strategy makes the other GEMM kernels 2-8 % slower and the attention dK/dV kernel 9 % slower. The strategy is a
// per-file compiler option (llm.c_amd/build.py, FILE_FLAGS), so the kernels that want it are compiled apart.
#include "common.hpp"
#include "gelu.hpp"
#include "gemm_pipelined.hpp"
#include "../../include/llmk.h"

#if !defined(LLMK_FP32)
namespace gemmk {
namespace {
template <int BM, int BN, int WGM, int WGN, int EPI>
void launch_tn_cfg(GemmArgs g, int splits, int grid, hipStream_t st) {
    constexpr int NW = WGM * WGN;
    constexpr int SMEM = smem_bytes(BM, BN, NW);
    auto kern = gemm_pipelined_kernel<BM, BN, WGM, WGN, true, true, EPI>;
    static bool attr_set = false;
    if (!attr_set) {
        HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM));
        attr_set = true;
    }
    g.splits = splits;
    if (grid <= 0) {
        const int work = CEIL_DIV(g.M, BM) * CEIL_DIV(g.N, BN) * splits;
        grid = min((work + 7) & ~7, llmk::device_info().num_cu & ~7);       // a multiple of 8: one share per XCD
    }
    kern<<<grid, NW * 64, SMEM, st>>>(g);
    LAUNCH_CHECK();
}
template <int EPI>
void launch_tn(const GemmArgs& g, int splits, bool big, int grid, hipStream_t st) {
    if (big) launch_tn_cfg<256, 256, 2, 4, EPI>(g, splits, grid, st);
    else launch_tn_cfg<128, 128, 2, 2, EPI>(g, splits, grid, st);
}
}  // namespace

void launch_pipelined_tn(GemmArgs g, int splits, bool big, int epi, int grid, hipStream_t st) {
    if (llmk::failed()) return;
    switch (epi) {
        case EPI_ACCUM: launch_tn<EPI_ACCUM>(g, splits, big, grid, st); break;
        case EPI_PARTIAL: launch_tn<EPI_PARTIAL>(g, splits, big, grid, st); break;
        case EPI_PARTIAL_ROWSUM: launch_tn<EPI_PARTIAL_ROWSUM>(g, splits, big, grid, st); break;
        default: LLMK_REQUIRE(false, "launch_pipelined_tn: epilogue %d is not one of the weight gradient's", epi);
    }
}
}  // namespace gemmk
#endif
