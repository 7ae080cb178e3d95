/*
 * ref_runner.c — thin exports around the UNMODIFIED reference CPU trainer.
 *
 * TEST INFRASTRUCTURE ONLY; built only where the reference checkout exists (see Makefile,
 * target _ref). This translation unit pulls in the reference's train_gpt2.c where it lies
 * (include path given on the compiler command line), exactly the way the reference's own
 * test_gpt2.c does (test_gpt2.c:1-2), so every per-op function of the reference
 * (layernorm_forward, matmul_backward, attention_backward, ...) and llmc/rand.h's
 * mt19937/normal_ are exported from the resulting shared object as they are. The functions
 * below only add a flat, struct-free entry point for whole-model runs.
 */
#define TESTING
#include "train_gpt2.c"
/* the sampler of the reference's GPU trainer (random_u32, random_f32, sample_softmax): a plain C header. The CPU
 * trainer's own copies of the first two sit behind #ifndef TESTING (train_gpt2.c:1046-1073), so nothing clashes. */
#include "llmc/sampler.h"
/* the learning-rate schedules: also a plain C header that train_gpt2.c does not pull in (the data loaders and the
 * tokenizer it does, train_gpt2.c:25-29, so those are exported as they are) */
#include "llmc/schedulers.h"
#include "llmc/outlier_detector.h"
#include "llmc/logger.h"

/* Runs the reference's own gpt2_forward / gpt2_zero_grad / gpt2_backward / gpt2_update
 * (train_gpt2.c:1163-1169 call order) for `steps` steps on one fixed batch.
 * The checkpoint must be a version-3 fp32 file (train_gpt2.c:713-718). */
int ref_gpt2_train(const char* ckpt, int* inputs, int* targets, int B, int T, int steps, float lr, float b1,
                   float b2, float eps, float wd, float* losses_out, float* grads_out, int grad_step,
                   float* logits_out, float* step_ms_out, float* params_out) {
    GPT2 model;
    gpt2_build_from_checkpoint(&model, ckpt);
    for (int s = 0; s < steps; s++) {
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        gpt2_forward(&model, inputs, targets, (size_t)B, (size_t)T);
        gpt2_zero_grad(&model);
        gpt2_backward(&model);
        if (grads_out && s == grad_step) memcpy(grads_out, model.grads_memory, model.num_parameters * sizeof(float));
        if (logits_out && s == 0) memcpy(logits_out, model.acts.logits, (size_t)B * T * model.config.padded_vocab_size * sizeof(float));
        gpt2_update(&model, lr, b1, b2, eps, wd, s + 1);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        losses_out[s] = model.mean_loss;
        if (step_ms_out) step_ms_out[s] = (float)((t1.tv_sec - t0.tv_sec) * 1e3 + (t1.tv_nsec - t0.tv_nsec) * 1e-6);
    }
    if (params_out) memcpy(params_out, model.params_memory, model.num_parameters * sizeof(float));
    gpt2_free(&model);
    return 0;
}

/* The generation loop of train_gpt2.cu:1751-1796 put together from the reference's own parts: its CPU forward pass
 * (train_gpt2.c gpt2_forward, on one sequence of the rounded length) and llmc/sampler.h. */
int ref_gpt2_generate(const char* ckpt, int* tokens, int T, int genT, int eot_token, unsigned long long* rng_state) {
    GPT2 model;
    gpt2_build_from_checkpoint(&model, ckpt);
    const int V = model.config.vocab_size, Vp = model.config.padded_vocab_size;
    const int chunk = T < 256 ? T : 256;
    for (int i = 0; i < T; i++) tokens[i] = eot_token;
    gpt2_forward(&model, tokens, NULL, 1, (size_t)T);     /* sizes the activations for the longest sequence */
    for (int t = 1; t < genT; t++) {
        gpt2_forward(&model, tokens, NULL, 1, (size_t)((t + chunk - 1) / chunk * chunk));
        float coin = random_f32(rng_state);
        tokens[t] = sample_softmax(model.acts.logits + (size_t)(t - 1) * Vp, V, coin);
    }
    gpt2_free(&model);
    return 0;
}

/* ---- flat entry points around the reference's structs for the data path ---------------------------------- */

/* nbatches calls of dataloader_next_batch (llmc/dataloader.h:222): every batch's inputs and targets and the loader's
 * position after it. With reset_every > 0, dataloader_reset is called before every reset_every-th batch (the way the
 * trainer restarts the validation loader, train_gpt2.cu:1721). state_out (optional) receives the shuffle state in the
 * order save_state writes it (train_gpt2.cu:1241-1247); returns its byte count. */
size_t ref_dataloader_run(const char* pattern, size_t B, size_t T, int rank, int nproc, int shuffle, int nbatches,
                          int reset_every, int* inputs_out, int* targets_out, size_t* shard_idx_out, size_t* sample_idx_out,
                          size_t* num_tokens_out, void* state_out) {
    DataLoader loader;
    dataloader_init(&loader, pattern, B, T, rank, nproc, shuffle);
    *num_tokens_out = loader.num_tokens;
    for (int i = 0; i < nbatches; i++) {
        if (reset_every > 0 && i > 0 && i % reset_every == 0) dataloader_reset(&loader);
        dataloader_next_batch(&loader);
        memcpy(inputs_out + (size_t)i * B * T, loader.inputs, B * T * sizeof(int));
        memcpy(targets_out + (size_t)i * B * T, loader.targets, B * T * sizeof(int));
        shard_idx_out[i] = loader.current_shard_idx;
        sample_idx_out[i] = loader.current_sample_idx;
    }
    size_t bytes = 0;
    if (shuffle && state_out) {
        char* p = (char*)state_out;
        memcpy(p, &loader.glob_result.gl_pathc, sizeof(size_t)); p += sizeof(size_t);
        memcpy(p, loader.shard_indices, loader.glob_result.gl_pathc * sizeof(int)); p += loader.glob_result.gl_pathc * sizeof(int);
        memcpy(p, &loader.shard_num_samples, sizeof(size_t)); p += sizeof(size_t);
        memcpy(p, loader.intra_shard_indices, loader.shard_num_samples * sizeof(int)); p += loader.shard_num_samples * sizeof(int);
        memcpy(p, &loader.shuffle_rng, sizeof(mt19937_state)); p += sizeof(mt19937_state);
        bytes = (size_t)(p - (char*)state_out);
    }
    dataloader_free(&loader);
    return bytes;
}

/* nbatches calls of evalloader_next_batch (llmc/dataloader.h:449) and evalloader_stat_losses on the given losses */
int ref_evalloader_run(const char* filename, size_t B, size_t T, int rank, int nproc, int nbatches, int* inputs_out,
                       int* targets_out, char* mask_out, int* label_out, const float* losses, int* correct_out, int* info_out) {
    EvalLoader loader;
    evalloader_init(&loader, filename, B, T, rank, nproc);
    info_out[0] = loader.num_examples; info_out[1] = loader.num_batches;
    info_out[2] = loader.start_example_index; info_out[3] = loader.end_example_index;
    int can_fit = (int)(B / ASSUMED_NUM_COMPLETIONS);
    for (int i = 0; i < nbatches; i++) {
        evalloader_next_batch(&loader);
        memcpy(inputs_out + (size_t)i * B * T, loader.inputs, B * T * sizeof(int));
        memcpy(targets_out + (size_t)i * B * T, loader.targets, B * T * sizeof(int));
        memcpy(mask_out + (size_t)i * B * T, loader.mask, B * T);
        memcpy(label_out + (size_t)i * can_fit, loader.label, can_fit * sizeof(int));
        correct_out[i] = evalloader_stat_losses(&loader, (float*)losses + (size_t)i * B * T);
    }
    info_out[4] = loader.current_example_index;
    evalloader_free(&loader);
    return 0;
}

/* get_learning_rate (llmc/schedulers.h:83) for steps 0..nsteps-1 */
void ref_learning_rates(const char* type, float lr, int warmup, int num_batches, float final_frac, int nsteps, float* out) {
    LearningRateScheduler s;
    lr_scheduler_init(&s, type, lr, warmup, num_batches, final_frac);
    for (int i = 0; i < nsteps; i++) out[i] = get_learning_rate(&s, i);
}

/* tokenizer_init + tokenizer_decode (llmc/tokenizer.h:41,86): the decoded bytes of ids[0..n) back to back into out
 * (each followed by a 0 byte); returns the end-of-text id, or -1 when the file could not be opened */
int ref_tokenizer_decode(const char* filename, const unsigned int* ids, int n, char* out, size_t out_bytes, unsigned int* vocab_out) {
    Tokenizer t;
    tokenizer_init(&t, filename);
    if (!t.init_ok) return -1;
    *vocab_out = t.vocab_size;
    size_t o = 0;
    for (int i = 0; i < n; i++) {
        const char* sp = tokenizer_decode(&t, ids[i]);
        size_t len = sp ? strlen(sp) : 0;
        if (o + len + 1 > out_bytes) break;
        if (sp) memcpy(out + o, sp, len);
        out[o + len] = 0;
        o += len + 1;
    }
    int eot = t.eot_token;
    tokenizer_free(&t);
    return eot;
}

/* update_detector (llmc/outlier_detector.h:36) over a series */
void ref_detector_run(const double* values, int n, double* z_out) {
    OutlierDetector d;
    init_detector(&d);
    for (int i = 0; i < n; i++) z_out[i] = update_detector(&d, values[i]);
}

/* one line of each kind through llmc/logger.h, n times */
void ref_logger_run(const char* log_dir, int rank, int resume, int n, const float* vals) {
    Logger lg;
    logger_init(&lg, log_dir, rank, resume);
    for (int i = 0; i < n; i++) {
        logger_log_train(&lg, i, vals[4 * i], vals[4 * i + 1], vals[4 * i + 2]);
        if (i % 3 == 0) logger_log_val(&lg, i, vals[4 * i + 3]);
        if (i % 5 == 0) logger_log_eval(&lg, i, vals[4 * i + 3] * 0.01f);
    }
}

int ref_num_threads(void) {
#ifdef OMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* known-answer sequence printed in llmc/rand.h:48-80 */
void ref_mt_kat(unsigned int seed, unsigned int* ints5, float* n8, unsigned int* mid, float* n16, unsigned int* last) {
    mt19937_state st;
    manual_seed(&st, seed);
    for (int i = 0; i < 5; i++) ints5[i] = randint32(&st);
    normal_(n8, 8, 0.f, 1.f, &st);
    *mid = randint32(&st);
    normal_(n16, 16, 0.f, 1.f, &st);
    *last = randint32(&st);
}
