/*
 * llmk.h — C ABI of the MI355X (gfx950) kernel library behind llm.c's GPT-2 training step.
 *
 * One entry point per kernel launcher of the reference (karpathy/llm.c, llmc/ *.cuh), same
 * argument order and meaning, with
 *     floatX*       -> void*   (bf16 in libllmk_bf16.so, fp32 in libllmk_fp32.so; the
 *                               precision is a property of the shared object, as PRECISION=
 *                               is of the reference build, reference Makefile:232-244)
 *     cudaStream_t  -> void*   (a hipStream_t; NULL = the default stream)
 *     templates / std::bool_constant / default arguments -> plain int / explicit arguments.
 * Citations give the reference launcher each function replaces (paths relative to the
 * reference checkout).
 *
 * Contract (same as the reference's launchers):
 *   - the caller owns every buffer; functions enqueue work on `stream` and return without
 *     waiting (exception: llmk_encoder_backward builds its buckets on the host first);
 *   - a single host thread drives the library;
 *   - no entry point here allocates device memory per call. Two launchers take scratch from ONE
 *     library-owned workspace (the role of the reference's cublaslt_workspace,
 *     llmc/cublas_common.h:28-31): llmk_matmul_backward (fp32 partial products of the split
 *     weight gradient) and llmk_attention_backward (one float per query and head). The
 *     workspace grows to the largest request seen (a free, an allocation and a device
 *     synchronisation at that call) and is then reused; a caller that must not allocate inside
 *     a step sizes it beforehand with llmk_workspace_reserve() from the
 *     llmk_*_workspace_bytes() of its shapes, as gpt2_allocate_state does. Nothing else is
 *     allocated or copied behind the caller's back: work lists are derived in the kernels;
 *   - errors: a failed HIP call or a violated shape precondition prints a message and exits
 *     (llmc/cuda_common.h:52-58). llmk_set_error_mode(1) makes the library record the
 *     message and return instead, for tests; read it with llmk_last_error().
 *
 * Shape preconditions: C % 8 == 0 (bf16) / C % 4 == 0 (fp32) for every row length,
 * head size up to 128 for attention (the bf16 build's MFMA kernels cover 64, the size of every
 * GPT-2 model; other sizes take one-wave-per-row kernels), 16-byte aligned pointers.
 */
#ifndef LLMK_H
#define LLMK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- library / device ------------------------------------------------------------------ */

/* Selects the device and reads its properties (reference: common_start, train_gpt2.cu:1173-1200). */
void llmk_init(int device);
void llmk_shutdown(void);
/* The library workspace (see the contract above): grow it to at least `bytes` now / its present size. The reference
 * allocates its cuBLASLt workspace once at start-up (llmc/cublas_common.h:28-31, train_gpt2.cu:1190-1195). */
void llmk_workspace_reserve(size_t bytes);
size_t llmk_workspace_bytes(void);
/* "bf16" or "fp32": the floatX of this shared object (reference: PRECISION_MODE, llmc/cuda_common.h:68-92) */
const char* llmk_precision(void);
/* sizeof(floatX) */
int llmk_sizeof_floatx(void);
/* multiProcessorCount / maxThreadsPerMultiProcessor / name of cudaDeviceProp (llmc/cuda_common.h:27) */
void llmk_device_props(int* num_cu, int* max_threads_per_cu, char* name256);
void llmk_set_error_mode(int record_instead_of_exit);
const char* llmk_last_error(void); /* "" when none; cleared by llmk_clear_error */
void llmk_clear_error(void);

/* Per-kernel timing (no launcher counterpart in the reference, which marks the same places with NVTX
 * ranges, llmc/cuda_common.h:115-124, and reads times from an ncu run, profile_gpt2cu.py). When enabled,
 * every kernel launch of this library is bracketed by HIP events on its stream; the report aggregates
 * by kernel family: number of launches, total milliseconds, algorithmic flops and algorithmic bytes. */
void llmk_profile_enable(int on);
/* NULL or "": time every family; otherwise only launches of the named family are bracketed by events */
void llmk_profile_only(const char* family);
void llmk_profile_reset(void);
int llmk_profile_count(void);
void llmk_profile_get(int i, char* name64, int* calls, double* ms, double* flops, double* bytes);

/* Zero `bytes` bytes at `ptr` on `stream`: the cudaMemsetAsync calls of the training step (gradients and losses,
 * train_gpt2.cu:800-801; the residual-stream gradient, train_gpt2.cu:828) as a store kernel that runs at HBM write
 * bandwidth. Any alignment and size. */
void llmk_zero(void* ptr, size_t bytes, void* stream);

/* Measurement aid, no counterpart in the reference (its mfu.h tabulates vendor peaks, llmc/mfu.h:43-147): the
 * TFLOP/s the matrix cores of this GPU deliver to back-to-back bf16 MFMAs on register operands (non-trivial values), two
 * waves per SIMD, for about ten milliseconds - i.e. CUs x 4096 flop per CU and clock x the clock the chip holds under that
 * load. scratch: one float of device memory. Synchronises the stream. The fp32 library returns zero. */
void llmk_probe_mfma_peak(double* tflops, float* scratch, void* stream);

/* ---- encoder (llmc/encoder.cuh) ---------------------------------------------------------- */

/* encoder_forward, llmc/encoder.cuh:157. out[b,t,:] = wte[inp[b,t],:] + wpe[t,:] */
void llmk_encoder_forward(void* out, const int* inp, const void* wte, const void* wpe, int B, int T, int C,
                          void* stream);

/* encoder_backward, llmc/encoder.cuh:169. dwpe[t,:] += sum_b dout[b,t,:];
 * dwte[tok,:] += sum_{bt: inp[bt]==tok} dout[bt,:]; fp32 accumulation in ascending bt order,
 * stochastic rounding into bf16 (plain store in fp32), no atomics.
 *   scratch           device, >= B*T*G*20 bytes with G = ceil(C / (64 * 16/sizeof(floatX))): bucket records, then
 *                     the position list (same layout and bound as the reference, llmc/encoder.cuh:183-184,225-226)
 *   workload_indices  host, >= B*T ints         (reference sizes it B*T*G)
 *   bucket_info       host, >= B*T*G * 4 ints   (reference: one int4 per bucket)
 *   inp / inputs_cpu  the same tokens on device / host
 * The two host lists are copied to the device by asynchronous copies on `stream`: where the caller gives pinned memory
 * (the driver does) the call returns with the copies and the kernel queued, and the lists must not be written again
 * before the stream has passed them; with pageable memory the copies are done when the call returns. */
void llmk_encoder_backward(void* dwte, void* dwpe, void* scratch, int* workload_indices, int* bucket_info,
                           const void* dout, const int* inp, const int* inputs_cpu, int B, int T, int C,
                           unsigned int seed, void* stream);

/* ---- layernorm / residual (llmc/layernorm.cuh) ------------------------------------------- */

/* layernorm_forward, llmc/layernorm.cuh:433. mean/rstd (fp32, B*T) may be NULL. */
void llmk_layernorm_forward(void* out, float* mean, float* rstd, const void* inp, const void* weight,
                            const void* bias, int B, int T, int C, void* stream);

/* residual_forward, llmc/layernorm.cuh:458 */
void llmk_residual_forward(void* out, const void* inp1, const void* inp2, int N, void* stream);

/* fused_residual_forward5, llmc/layernorm.cuh:467. residual = inp1 + inp2 (rounded to floatX),
 * normed = LN(residual). mean/rstd may be NULL. */
void llmk_fused_residual_forward5(void* residual, void* normed, float* mean, float* rstd, const void* inp1,
                                  const void* inp2, const void* weight, const void* bias, int N, int C,
                                  void* stream);

/* layernorm_backward, llmc/layernorm.cuh:492. dinp += ..., dweight += ..., dbias += ...
 * scratch: device fp32, >= llmk_layernorm_backward_scratch_floats(C) floats. */
void llmk_layernorm_backward(void* dinp, void* dweight, void* dbias, float* scratch, const void* dout,
                             const void* inp, const void* weight, const float* mean, const float* rstd, int B,
                             int T, int C, void* stream);
size_t llmk_layernorm_backward_scratch_floats(int C);

/* ---- matmul (llmc/matmul.cuh) ------------------------------------------------------------ */

/* matmul_forward_cublaslt, llmc/matmul.cuh:231. out[B*T,OC] = inp[B*T,C] . weight[OC,C]^T + bias[OC].
 * bias may be NULL. If pre_gelu != NULL: pre_gelu receives the pre-activation and out = gelu(pre_gelu)
 * (gelu_fusion >= 1: in the GEMM epilogue; < 1: separate gelu kernel).
 * gelu_fusion 3 has no counterpart in the reference (its levels are 0-2, train_gpt2.cu:1419-1470): pre_gelu then
 * receives gelu'(pre-activation), rounded to the storage type, instead of the pre-activation, for a backward pass that
 * only multiplies by it (llmk_matmul_backward with gelu_fusion 3). For callers that keep the tensor for nothing else,
 * i.e. that do not recompute gelu from it. out is the same bits as with gelu_fusion 1 and 2. */
void llmk_matmul_forward(void* out, const void* inp, const void* weight, const void* bias, int B, int T, int C,
                         int OC, void* stream, void* pre_gelu, int gelu_fusion);

/* The projection and the residual add that follows it in one launch: out = round(round(inp . weight^T + bias) + residual),
 * both roundings to the storage type as llmk_matmul_forward followed by the add of llmk_fused_residual_forward5
 * (llmc/layernorm.cuh:467, its residual = inp1 + inp2) give them, so the bits are the same. It has no counterpart in the
 * reference (which runs matmul_forward_cublaslt and fused_residual_forward5, train_gpt2.cu:713-727); a LayerNorm of out
 * (llmk_layernorm_forward) then takes the place of the fused kernel. out must not be residual or inp. */
void llmk_matmul_forward_residual(void* out, const void* inp, const void* weight, const void* bias, const void* residual,
                                  int B, int T, int C, int OC, void* stream);

/* matmul_backward, llmc/matmul.cuh:244.
 *   dbias[OC]   += column sums of dout          (skipped when dbias == NULL)
 *   dinp[B*T,C]  = dout . weight                 (then *= gelu'(pre_gelu) when pre_gelu != NULL;
 *                                                 gelu_fusion >= 2: in the epilogue, else separate kernel)
 *   dweight[OC,C] += dout^T . inp
 * gelu_fusion 3: pre_gelu holds gelu'(pre-activation) as llmk_matmul_forward(.., gelu_fusion 3) left it, and dinp is
 * the product of the rounded dout . weight with that stored value, rounded once more.
 * dbias_buffer: device fp32 scratch, >= llmk_matmul_backward_bias_scratch_floats(OC) floats
 * (may be NULL when dbias == NULL). */
void llmk_matmul_backward(void* dinp, void* dweight, void* dbias, const void* dout, const void* inp,
                          const void* weight, float* dbias_buffer, int B, int T, int C, int OC, void* stream,
                          const void* pre_gelu, int gelu_fusion);
size_t llmk_matmul_backward_bias_scratch_floats(int OC);
/* How llmk_matmul_backward cuts the weight gradient's contraction over B*T into work items (bf16 library): -1 (default)
 * picks by a cost estimate between equal splits of every tile and, when the tiles are a sizable part of the workgroups
 * of a launch, one long and a few short pieces per tile (cut at the same K positions for every tile, scheduled so that
 * all workgroups finish together); 0 always takes equal splits, 1 takes the uneven pieces whenever the shape allows
 * them. The result is the same sum in a different (fixed) order of fp32 partials. No counterpart in the reference
 * (cuBLASLt chooses its own split there); for tests and tuning. */
void llmk_matmul_backward_split_mode(int mode);
/* What the last llmk_matmul_backward did with the weight gradient's contraction: *kind = 0 not cut, 1 equal splits,
 * 2 one long and several short pieces per tile; *pieces = fp32 partials per output element. For tests. */
void llmk_matmul_backward_last_split(int* kind, int* pieces);
/* Upper bound of the workspace llmk_matmul_backward(B, T, C, OC) asks for, whichever way it cuts K. */
size_t llmk_matmul_backward_workspace_bytes(int B, int T, int C, int OC);

/* gelu_backward_inplace (llmc/gelu.cuh:59) and the bias gradient of matmul_backward (llmc/matmul.cuh:251-266) in
 * one pass over (B*T, OC): d_in_out *= gelu'(inp), then dbias[OC] += column sums of the result. Same values as
 * llmk_gelu_backward_inplace followed by llmk_matmul_backward's bias step (bit for bit in the bf16 library, to
 * the rounding of one fused multiply-add in the fp32 library); the caller then passes dbias = NULL to
 * llmk_matmul_backward. dbias_buffer: llmk_matmul_backward_bias_scratch_floats(OC) floats. */
void llmk_gelu_backward_bias(void* d_in_out, const void* inp, void* dbias, float* dbias_buffer, int B, int T, int OC,
                             void* stream);

/* ---- attention (llmc/cudnn_att.cpp; the flash path the reference takes with ENABLE_CUDNN) -- */

/* attention_forward_cudnn, llmc/cudnn_att.cpp:222. Causal softmax(Q K^T / sqrt(hs)) V.
 * inp (B,T,3,NH,hs) read in place; out (B,T,NH,hs); stats (B,NH,T) fp32 = log-sum-exp of the
 * scaled scores of each row, NULL for inference. */
void llmk_attention_forward(void* out, float* stats, const void* inp, int B, int T, int NH, int C, void* stream);

/* attention_backward_cudnn, llmc/cudnn_att.cpp:256. dqkvr (B,T,3,NH,hs) is overwritten.
 * Deterministic (no atomics), as the reference requests from cuDNN (cudnn_att.cpp:187-189).
 * Uses B*NH*T floats of the library workspace for the rowsum(dO*O) term. */
void llmk_attention_backward(void* dqkvr, const void* dout, const void* qkvr, const void* o, const float* stats,
                             int B, int T, int NH, int C, void* stream);
size_t llmk_attention_backward_workspace_bytes(int B, int T, int NH);

/* attention_forward, llmc/attention.cuh:195: the launcher of reference builds without cuDNN, same argument order.
 * inp (B,T,3C) Q, K, V as the qkv projection wrote them; out (B,T,C). qkvr (B*T*3C elements) and att (B*NH*T*T elements)
 * are the buffers the reference keeps for its backward pass; this library keeps other things in them (qkvr: a copy of inp
 * as it came; att: the fp32 log-sum-exp of every row in its first B*NH*T*4 bytes, which needs T*sizeof(floatX) >= 4), so
 * they are only meaningful to llmk_attention_backward_fallback. inp is left intact (the reference overwrites it). */
void llmk_attention_forward_fallback(void* out, void* qkvr, void* att, void* inp, int B, int T, int C, int NH, void* stream);

/* attention_backward, llmc/attention.cuh:239, same argument order. dinp (B,T,3C) is overwritten with the gradient of
 * the un-permuted Q, K, V; qkvr and att as llmk_attention_forward_fallback left them; scratch (B*T*C elements) receives
 * the forward output again (the reference's signature does not pass it); dqkvr and datt are not touched. */
void llmk_attention_backward_fallback(void* dinp, void* dqkvr, void* datt, void* scratch, const void* dout, const void* qkvr,
                                      const void* att, int B, int T, int C, int NH, void* stream);

/* The same operation for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. The rowsum(dO*O) vector lives in a
 * 4 MiB array that is part of the library's code object on every GPU instead of the grow-only workspace, so the call
 * makes no hipMalloc/hipFree and creates no events (it is not timed by llmk_profile_*). Limit: B*NH*T <= 1048576
 * (larger sizes are rejected with an error; GPT-2 124M at B=64, T=1024 needs 786432). Results are bit-identical to
 * llmk_attention_backward. All calls on one GPU share the one array: calls that overlap on a GPU (two streams) race. */
void llmk_attention_backward_static(void* dqkvr, const void* dout, const void* qkvr, const void* o, const float* stats,
                                    int B, int T, int NH, int C, void* stream);

/* ---- gelu (llmc/gelu.cuh) ----------------------------------------------------------------- */

/* The two halves of gelu_fusion 3 as passes of their own (what llmk_matmul_forward / llmk_matmul_backward run for shapes
 * their fused epilogues do not take); no counterpart in the reference. out = gelu(inp_to_grad), then inp_to_grad =
 * gelu'(inp_to_grad) in place; d_in_out *= grad. */
void llmk_gelu_forward_keep_grad(void* out, void* inp_to_grad, int N, void* stream);
void llmk_gelu_backward_from_grad(void* d_in_out, const void* grad, int N, void* stream);

/* gelu_forward, llmc/gelu.cuh:50 */
void llmk_gelu_forward(void* out, const void* inp, int N, void* stream);
/* gelu_backward_inplace, llmc/gelu.cuh:59. d_in_out *= gelu'(inp) */
void llmk_gelu_backward_inplace(void* d_in_out, const void* inp, int N, void* stream);

/* ---- fused classifier (llmc/fused_classifier.cuh) ---------------------------------------- */

/* fused_classifier, llmc/fused_classifier.cuh:139. Per row of logits (B*T, P), over the first V
 * columns: losses[row] -= log softmax(row)[target]  (accumulates, like the reference's `-=` at :81);
 * if write_dlogits: logits[row,i] = (softmax_i - [i==target]) * dloss in place for i < V.
 * Columns [V,P) are left untouched. */
void llmk_fused_classifier(void* logits, float* losses, float dloss, const int* targets, int B, int T, int V,
                           int P, int write_dlogits, void* stream);

/* ---- global norm (llmc/global_norm.cuh, llmc/cuda_utils.cuh) ------------------------------ */

/* get_max_num_block_sums, llmc/global_norm.cuh:52 */
int llmk_get_max_num_block_sums(const int* num_slices_all, int numel);
/* global_norm_squared, llmc/global_norm.cuh:68. out[block] (+)= partial sums of values^2;
 * reset != 0 zeroes out[0..max_num_block_sums) first. */
void llmk_global_norm_squared(float* out, const void* values, size_t count, ptrdiff_t stride, int num_slices,
                              int max_num_block_sums, int reset, void* stream);
/* global_sum_deterministic<float>, llmc/cuda_utils.cuh:202. *result = sum(values[0..count)), one block. */
void llmk_global_sum_deterministic(float* result, const float* values, int count, void* stream);

/* ---- AdamW (llmc/adamw.cuh) --------------------------------------------------------------- */

/* adamw_update, llmc/adamw.cuh:74. params/grads are floatX, m/v/master fp32; master may be NULL.
 * The stochastic-rounding word of element i of slice s is
 * SquirrelNoise5(i % 512 + 198491317 * ((i / 512) * 512 + s), seed): a pure function of
 * (i, s, seed) that equals what the reference's launch geometry yields (llmc/cuda_utils.cuh:272). */
void llmk_adamw_update(void* params_memory, float* master_params_memory, const void* grads_memory, float* m_memory,
                       float* v_memory, size_t num_parameters, ptrdiff_t w_stride, ptrdiff_t g_stride,
                       ptrdiff_t s_stride, int num_slices, float learning_rate, float beta1, float beta2, int t,
                       float eps, float weight_decay, float grad_scale, unsigned int seed, void* stream);
/* Several tensors in one launch; no counterpart in the reference, whose gpt2_update launches adamw_update once per
 * tensor (train_gpt2.cu:1056-1106; ten of GPT-2's sixteen tensors are a few KB). All five arenas share one layout: tensor
 * i starts offsets[i] elements into each of them and has num_slices[i] contiguous slices of sizes[i] elements, its own
 * weight decay and seed. Same arithmetic and the same stochastic-rounding words as count calls of llmk_adamw_update with
 * strides equal to sizes[i]. Returns 1 when it ran; 0 (nothing done) when the tensors do not suit it - more than 16,
 * sizes or offsets not multiples of 16 bytes of floatX, misaligned arenas - and the caller falls back to per-tensor calls. */
int llmk_adamw_update_multi(void* params_memory, float* master, const void* grads_memory, float* m, float* v, int count,
                            const size_t* offsets, const size_t* sizes, const int* num_slices, const float* weight_decays,
                            const unsigned int* seeds, float lr, float beta1, float beta2, int t, float eps, float grad_scale,
                            void* stream);
/* The same launch with the clipping decided on the device: grad_scale = norm > grad_clip ? grad_clip / norm : 1 with
 * norm = sqrt(*grad_norm_squared) (device memory: the result of llmk_global_norm_squared + llmk_global_sum_deterministic),
 * the two statements of the reference's training loop (train_gpt2.cu:1841-1851) in the same fp32 arithmetic. No
 * counterpart in the reference: for step loops that do not want to wait for the norm on the host between the backward
 * pass and the update. Returns 0 (nothing launched) where llmk_adamw_update_multi would. */
int llmk_adamw_update_multi_clip(void* params_memory, float* master, const void* grads_memory, float* m, float* v, int count,
                                 const size_t* offsets, const size_t* sizes, const int* num_slices, const float* weight_decays,
                                 const unsigned int* seeds, float lr, float beta1, float beta2, int t, float eps,
                                 const float* grad_norm_squared, float grad_clip, void* stream);

/* init_from_master, llmc/adamw.cuh:90. params = stochastic_round(master), same noise as above. */
void llmk_init_from_master(void* params_memory, const float* master_params_memory, size_t num_parameters,
                           ptrdiff_t w_stride, ptrdiff_t s_stride, int num_slices, unsigned int seed,
                           void* stream);
/* copy_and_cast_kernel<float, floatX> launch, llmc/cuda_utils.cuh:134 / train_gpt2.cu:1089-1094:
 * dst[i + s*stride_dst] = (float)src[i + s*stride_src] */
void llmk_copy_and_cast_to_f32(float* dst, const void* src, size_t n, ptrdiff_t stride_dst, ptrdiff_t stride_src,
                               int num_slices, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMK_H */
