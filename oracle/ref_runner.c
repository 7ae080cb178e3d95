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
