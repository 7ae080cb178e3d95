/*
 * llmk_gpt2.h — C ABI of the host-side GPT-2 training driver that sits on top of llmk.h.
 *
 * It is the reference's `GPT2` object and its functions (train_gpt2.cu:285-1168, save_state /
 * load_state :1209-1314), re-hosted on the HIP kernel library: same parameter / activation
 * arenas, same call order of the kernel launchers, same .bin checkpoint and state layouts. The
 * struct itself is opaque here so that tests and the benchmark can drive it through ctypes.
 * Each function cites the reference function of the same name.
 */
#ifndef LLMK_GPT2_H
#define LLMK_GPT2_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct LLMK_GPT2 LLMK_GPT2;

/* gpt2_init_common, train_gpt2.cu:324. Defaults: use_master_weights=1, recompute=1, gelu_fusion=0,
 * rng_state=13371337. */
LLMK_GPT2* gpt2_create(void);
/* options that the reference sets on the struct before gpt2_allocate_state (train_gpt2.cu:1578-1581):
 * use_master_weights 0|1, recompute 0|1|2, gelu_fusion 0|1|2; negative = leave unchanged.
 * gelu_fusion 3 (this library's own, see llmk_matmul_forward): the fch tensor keeps gelu'(pre-activation) for the backward
 * epilogue instead of the pre-activation; with recompute >= 1, which needs the pre-activation again, it runs as 2. */
void gpt2_set_options(LLMK_GPT2* m, int use_master_weights, int recompute, int gelu_fusion);

/* gpt_build_from_descriptor, train_gpt2.cu:562: "d12", "gpt2:d48", "gpt3:c768"; mt19937 seed 42 */
void gpt2_build_from_descriptor(LLMK_GPT2* m, const char* descriptor);
/* same random init for an arbitrary shape (tests): N(0,0.02), residual projections / sqrt(2L) */
void gpt2_build_from_config(LLMK_GPT2* m, int max_seq_len, int vocab_size, int padded_vocab_size, int num_layers,
                            int num_heads, int channels, unsigned int seed);
/* gpt2_build_from_checkpoint, train_gpt2.cu:454: version 3 (fp32) for the fp32 library,
 * version 5 (bf16) for the bf16 library; anything else is an error. */
void gpt2_build_from_checkpoint(LLMK_GPT2* m, const char* checkpoint_path, int weight_init);
/* gpt2_write_to_checkpoint, train_gpt2.cu:430 */
void gpt2_write_to_checkpoint(LLMK_GPT2* m, const char* checkpoint_path);
/* gpt2_allocate_state, train_gpt2.cu:367 */
void gpt2_allocate_state(LLMK_GPT2* m, int B, int T);

/* gpt2_forward, train_gpt2.cu:646. inputs: host, B*T ints. Logits end up in the output buffer. */
void gpt2_forward(LLMK_GPT2* m, const int* inputs, size_t B, size_t T);
/* gpt2_validate, train_gpt2.cu:761. Returns the mean loss; per-token losses via gpt2_cpu_losses. */
float gpt2_validate(LLMK_GPT2* m, const int* inputs, const int* targets, size_t B, size_t T);
/* The text-generation loop of the reference's main, train_gpt2.cu:1751-1796 (minus the printing). gen_tokens: host,
 * batch*seq_len ints as allocated; on return positions 1..genT-1 of the first sequence hold the sampled tokens and
 * everything else eot_token. sample_rng_state: llmc/sampler.h's xorshift state (the reference restarts it at 1337). */
void gpt2_generate(LLMK_GPT2* m, int* gen_tokens, int genT, int eot_token, unsigned long long* sample_rng_state);
/* gpt2_backward_and_reduce, train_gpt2.cu:788 (the reduce is a no-op on one GPU) */
void gpt2_backward_and_reduce(LLMK_GPT2* m, const int* inputs, const int* targets, int grad_accum_steps, int micro_step);
/* gpt2_calculate_grad_norm, train_gpt2.cu:992 */
float gpt2_calculate_grad_norm(LLMK_GPT2* m);
/* gpt2_update, train_gpt2.cu:1035 */
void gpt2_update(LLMK_GPT2* m, float learning_rate, float beta1, float beta2, float eps, float weight_decay,
                 float grad_scale, int t, int init_from_master_only);
/* One optimizer step over one micro-batch with a single wait at its end: gpt2_forward + gpt2_backward_and_reduce(.., 1, 0)
 * + gpt2_calculate_grad_norm + gpt2_update with grad_scale = norm > grad_clip ? grad_clip / norm : 1 (train_gpt2.cu:1835-1851),
 * queued back to back, the clipping factor formed on the device, the mean loss and the gradient norm read back together
 * after the update is queued. Same kernels in the same order on the same data: the parameters, the loss and the norm are
 * those of the four calls, bit for bit. No counterpart in the reference (whose loop waits for the device after the forward
 * pass, after the backward pass, for the norm and after the update). mean_loss / grad_norm may be NULL. */
void gpt2_train_step(LLMK_GPT2* m, const int* inputs, const int* targets, float learning_rate, float beta1, float beta2,
                     float eps, float weight_decay, float grad_clip, int t, float* mean_loss, float* grad_norm);
/* gpt2_estimate_mfu, train_gpt2.cu:1126, against the MI355X dense peak of the library's precision */
float gpt2_estimate_mfu(LLMK_GPT2* m, int num_tokens, float dt);
/* gpt2_free, train_gpt2.cu:1155 */
void gpt2_free(LLMK_GPT2* m);

/* save_state / load_state, train_gpt2.cu:1209 / :1250 (dataloader fields are written as zero /
 * ignored: the data loader is outside this library). load_state needs gpt2_allocate_state first. */
void gpt2_save_state(LLMK_GPT2* m, const char* filename, int step);
void gpt2_load_state(LLMK_GPT2* m, const char* filename, int* step);
/* The same two under the reference's names and argument order, with the training data loader (llmk_data.h) whose
 * position and, when it shuffles, permutations and generator go into / come out of the file (train_gpt2.cu:1228-1247,
 * :1289-1310). loader may be NULL. For load_state the loader must have been initialised on the same shards. */
void gpt2_save_state_with_loader(const char* filename, int step, LLMK_GPT2* model, struct LLMK_DataLoader* loader);
void gpt2_load_state_with_loader(int* step, LLMK_GPT2* model, struct LLMK_DataLoader* loader, const char* filename);

/* ---- accessors (the reference reads the struct fields directly) ---- */
float gpt2_mean_loss(const LLMK_GPT2* m);
size_t gpt2_num_parameters(const LLMK_GPT2* m);
void gpt2_get_config(const LLMK_GPT2* m, int* six_ints); /* max_seq_len, vocab, padded_vocab, L, NH, C */
void gpt2_param_sizes(const LLMK_GPT2* m, size_t* sixteen);
const float* gpt2_cpu_losses(const LLMK_GPT2* m);         /* host, B*T floats, filled by gpt2_validate */
/* device arenas, for tests that check individual tensors */
void* gpt2_params_memory(LLMK_GPT2* m);
void* gpt2_grads_memory(LLMK_GPT2* m);
void* gpt2_output_memory(LLMK_GPT2* m);                   /* acts.output: logits after forward */
/* whole arenas converted to / from fp32 on the host */
void gpt2_get_params_f32(LLMK_GPT2* m, float* out);
void gpt2_set_params_f32(LLMK_GPT2* m, const float* in);
void gpt2_get_grads_f32(LLMK_GPT2* m, float* out);
void gpt2_get_logits_f32(LLMK_GPT2* m, float* out, size_t B, size_t T); /* (B*T, padded_vocab) */
unsigned long long gpt2_get_rng_state(const LLMK_GPT2* m);
void gpt2_set_rng_state(LLMK_GPT2* m, unsigned long long s);
size_t gpt2_activation_bytes(const LLMK_GPT2* m);

#ifdef __cplusplus
}
#endif
#endif /* LLMK_GPT2_H */
