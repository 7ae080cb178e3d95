/*
 * llmk_data.h — C ABI of the host-side pieces that feed the training step and consume its results:
 * the token-shard loader, the multiple-choice evaluation loader, the learning-rate schedules, the
 * token decoder, the outlier detector and the run log. They are the reference's llmc/dataloader.h,
 * schedulers.h, tokenizer.h, outlier_detector.h and logger.h under their own function names, with the structs opaque (created and freed by the library) so that
 * C, C++ and ctypes callers share one layout. File formats are the reference's, byte for byte.
 * None of these functions touches the GPU.
 *
 * Error behaviour follows the reference: a missing or malformed file prints a message and exits the
 * process (llmc/utils.h:26-64, dataloader.h:74-80).
 */
#ifndef LLMK_DATA_H
#define LLMK_DATA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- training / validation shards (llmc/dataloader.h:28-248) ---------------------------------
 * A shard is 256 int32 of header {20240520, 1, ntok, 0...} followed by ntok uint16 tokens. Process p of P
 * takes the p-th B*T slice of every P*B*T-token sample; a batch is B*T+1 consecutive tokens, inputs =
 * the first B*T, targets = the same shifted by one. With should_shuffle the order of the shards and of the
 * samples inside a shard are permutations drawn from mt19937 seeded with 42 + process_rank. */
typedef struct LLMK_DataLoader LLMK_DataLoader;
LLMK_DataLoader* dataloader_create(void);
/* dataloader_init, llmc/dataloader.h:142 */
void dataloader_init(LLMK_DataLoader* loader, const char* filename_pattern, size_t B, size_t T, int process_rank,
                     int num_processes, int should_shuffle);
/* dataloader_reset, llmc/dataloader.h:110: back to the first sample of a (re-drawn, if shuffling) first shard */
void dataloader_reset(LLMK_DataLoader* loader);
/* dataloader_load_batch, llmc/dataloader.h:203: fills inputs/targets from the current sample without advancing */
void dataloader_load_batch(LLMK_DataLoader* loader);
/* dataloader_next_batch, llmc/dataloader.h:222 */
void dataloader_next_batch(LLMK_DataLoader* loader);
/* dataloader_resume, llmc/dataloader.h:232 */
void dataloader_resume(LLMK_DataLoader* loader, size_t current_shard_idx, size_t current_sample_idx);
/* dataloader_free, llmc/dataloader.h:239 (also releases the handle) */
void dataloader_free(LLMK_DataLoader* loader);
/* the struct fields the trainer reads (train_gpt2.cu:1610-1616, :1831-1834, :1228-1229) */
const int* dataloader_inputs(const LLMK_DataLoader* loader);    /* host, B*T */
const int* dataloader_targets(const LLMK_DataLoader* loader);   /* host, B*T */
size_t dataloader_num_tokens(const LLMK_DataLoader* loader);
size_t dataloader_num_shards(const LLMK_DataLoader* loader);
size_t dataloader_shard_num_samples(const LLMK_DataLoader* loader);
size_t dataloader_current_shard_idx(const LLMK_DataLoader* loader);
size_t dataloader_current_sample_idx(const LLMK_DataLoader* loader);
int dataloader_should_shuffle(const LLMK_DataLoader* loader);
/* The shuffle state as save_state appends it to the optimizer-state file (train_gpt2.cu:1241-1247): number of
 * shards (size_t), shard permutation (int each), samples in the shard (size_t), sample permutation (int each), the
 * generator (llmc/rand.h:98-104: 8 bytes that the reference leaves unset and this library writes as zero, left_,
 * next_, 624 state words, MATRIX_A). Returns the byte count; buf may be NULL to ask for it. 0 without shuffling. */
size_t dataloader_get_shuffle_state(const LLMK_DataLoader* loader, void* buf);
/* ... and as load_state reads it back (train_gpt2.cu:1289-1308); follow with dataloader_resume. Returns bytes consumed.
 * bytes == 0 is the state of a loader that does not shuffle: the loader stops shuffling (train_gpt2.cu:1289). */
size_t dataloader_set_shuffle_state(LLMK_DataLoader* loader, const void* buf, size_t bytes);

/* ---- multiple-choice evaluation file, e.g. HellaSwag (llmc/dataloader.h:250-518) ---------------
 * 256 int32 of header {20240522, 1, num_examples, longest_example_bytes, 0...}, then per example a uint16 stream:
 * 65535, example bytes, example index, label, number of completions (4), context length + tokens, and per
 * completion its length + tokens. Every example fills four rows of the (B,T) batch. */
typedef struct LLMK_EvalLoader LLMK_EvalLoader;
LLMK_EvalLoader* evalloader_create(void);
/* evalloader_init, llmc/dataloader.h:340 */
void evalloader_init(LLMK_EvalLoader* loader, const char* filename, size_t B, size_t T, int process_rank, int num_processes);
/* evalloader_reset, llmc/dataloader.h:298 */
void evalloader_reset(LLMK_EvalLoader* loader);
/* evalloader_next_batch, llmc/dataloader.h:449 */
void evalloader_next_batch(LLMK_EvalLoader* loader);
/* evalloader_stat_losses, llmc/dataloader.h:468: examples of the batch whose lowest mean masked loss is the label's row */
int evalloader_stat_losses(const LLMK_EvalLoader* loader, const float* losses);
/* evalloader_free, llmc/dataloader.h:511 (also releases the handle) */
void evalloader_free(LLMK_EvalLoader* loader);
const int* evalloader_inputs(const LLMK_EvalLoader* loader);    /* host, B*T */
const int* evalloader_targets(const LLMK_EvalLoader* loader);   /* host, B*T */
const char* evalloader_mask(const LLMK_EvalLoader* loader);     /* host, B*T: 1 where a completion token is predicted */
const int* evalloader_label(const LLMK_EvalLoader* loader);     /* host, B/4 */
int evalloader_num_examples(const LLMK_EvalLoader* loader);
int evalloader_num_batches(const LLMK_EvalLoader* loader);
int evalloader_start_example_index(const LLMK_EvalLoader* loader);
int evalloader_end_example_index(const LLMK_EvalLoader* loader);
int evalloader_current_example_index(const LLMK_EvalLoader* loader);

/* ---- learning-rate schedules (llmc/schedulers.h) ---------------------------------------------- */
typedef struct LLMK_LRScheduler LLMK_LRScheduler;
LLMK_LRScheduler* lr_scheduler_create(void);
/* lr_scheduler_init, llmc/schedulers.h:19. scheduler_type: "cosine", "linear", "constant" or "wsd" (copied) */
void lr_scheduler_init(LLMK_LRScheduler* scheduler, const char* scheduler_type, float learning_rate, int warmup_iterations,
                       int train_num_batches, float final_learning_rate_frac);
/* get_learning_rate, llmc/schedulers.h:83; an unknown type prints a message and exits, as there */
float get_learning_rate(LLMK_LRScheduler* scheduler, int step);
void lr_scheduler_free(LLMK_LRScheduler* scheduler);

/* ---- token decoder (llmc/tokenizer.h) ---------------------------------------------------------
 * File: 256 uint32 of header {20240328, version, vocab_size, eot_token (version 2)}, then per token one length byte
 * and that many bytes. */
typedef struct LLMK_Tokenizer LLMK_Tokenizer;
LLMK_Tokenizer* tokenizer_create(void);
/* tokenizer_init, llmc/tokenizer.h:41: a file that cannot be opened leaves init_ok = 0 (with a warning), as there */
void tokenizer_init(LLMK_Tokenizer* tokenizer, const char* filename);
/* tokenizer_decode, llmc/tokenizer.h:86: NULL when not initialised or for an id outside the vocabulary */
const char* tokenizer_decode(LLMK_Tokenizer* tokenizer, uint32_t token_id);
/* safe_printf, llmc/tokenizer.h:25: prints the piece unless it is a single unprintable byte */
void safe_printf(const char* piece);
void tokenizer_free(LLMK_Tokenizer* tokenizer);
int tokenizer_init_ok(const LLMK_Tokenizer* tokenizer);
int tokenizer_eot_token(const LLMK_Tokenizer* tokenizer);
uint32_t tokenizer_vocab_size(const LLMK_Tokenizer* tokenizer);

/* ---- loss / gradient-norm outlier detector (llmc/outlier_detector.h) ---------------------------
 * A window of the last 128 values with running sum and sum of squares in double. */
typedef struct LLMK_OutlierDetector LLMK_OutlierDetector;
LLMK_OutlierDetector* outlier_detector_create(void);
/* init_detector, llmc/outlier_detector.h:26 */
void init_detector(LLMK_OutlierDetector* detector);
/* update_detector, llmc/outlier_detector.h:36: NaN until the window is full, then the z-score of new_value against
 * the window that already contains it (0 when the window has no spread) */
double update_detector(LLMK_OutlierDetector* detector, double new_value);
void outlier_detector_free(LLMK_OutlierDetector* detector);

/* ---- run log (llmc/logger.h): lines appended to <log_dir>/main.log by process 0 ------------------ */
typedef struct LLMK_Logger LLMK_Logger;
LLMK_Logger* logger_create(void);
/* logger_init, llmc/logger.h:19: inactive when log_dir is NULL or process_rank != 0; resume == 0 empties the file */
void logger_init(LLMK_Logger* logger, const char* log_dir, int process_rank, int resume);
/* logger_log_eval, llmc/logger.h:34: "s:%d eval:%.4f" */
void logger_log_eval(LLMK_Logger* logger, int step, float val);
/* logger_log_val, llmc/logger.h:42: "s:%d tel:%.4f" */
void logger_log_val(LLMK_Logger* logger, int step, float val_loss);
/* logger_log_train, llmc/logger.h:50: "s:%d trl:%.4f lr:%.6f norm:%.2f" */
void logger_log_train(LLMK_Logger* logger, int step, float train_loss, float learning_rate, float grad_norm);
void logger_free(LLMK_Logger* logger);

#ifdef __cplusplus
}
#endif
#endif /* LLMK_DATA_H */
