// train_gpt2: the reference trainer's main loop (train_gpt2.cu:1419-1900) on one MI355X, written against the C ABI of
// this library (include/llmk_gpt2.h, include/llmk_data.h). Same command-line letters and defaults for everything that
// applies to one process; the multi-process options (-pn, -pr, -pg, -pi, -pf, -ps, -z) are accepted and must describe a
// single process. Output lines, log file, checkpoint / state / DONE file names are the reference's, so its tooling
// (dev/vislog.ipynb, resume with -y 1) reads them unchanged.
#include <hip/hip_runtime.h>

#include <cassert>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <sys/stat.h>
#include <dirent.h>

#include "../../include/llmk.h"
#include "../../include/llmk_data.h"
#include "../../include/llmk_gpt2.h"

namespace {

[[noreturn]] void usage() {
    fprintf(stderr,
            "Usage:   train_gpt2 [options]\n"
            "  -i <string> train data filename pattern (default = dev/data/tinyshakespeare/tiny_shakespeare_train.bin)\n"
            "  -j <string> val data filename pattern (default = dev/data/tinyshakespeare/tiny_shakespeare_val.bin)\n"
            "  -e <string> input .bin filename or descriptor, e.g. d12 (default = gpt2_124M_bf16.bin)\n"
            "  -o <string> output log dir (default = NULL, no logging)\n"
            "  -lg <int>   log gpu info every x steps (ignored)\n"
            "  -n <int>    write optimization checkpoints every how many steps? (default 0, don't)\n"
            "  -nk <int>   max number of checkpoints to keep in the directory, removing old ones (0 = disable, default)\n"
            "  -nm <int>   every how many step checkpoints are considered major? major checkpoints never get deleted\n"
            "  -y <int>    resume optimization found inside output log dir? (0=restart/overwrite, 1=resume/append)\n"
            "  -b <int>    (per-GPU, micro) batch size B (default = 4)\n"
            "  -t <int>    sequence length T (default = 1024)\n"
            "  -d <int>    total desired batch size (default = B * T, i.e. no grad accumulation)\n"
            "  -x <int>    max_steps of optimization to run (-1 (default) = one epoch of the training data)\n"
            "  -k <string> learning rate scheduler: cosine, linear, constant, wsd (default = cosine)\n"
            "  -l <float>  learning rate (default = 3e-4f)\n"
            "  -u <int>    learning rate warmup iterations (default = 0, no warmup)\n"
            "  -q <float>  learning rate decay: final fraction, at end of training (default = 1.0 (no decay))\n"
            "  -c <float>  weight decay (default = 0.0f)\n"
            "  -sl <float> outlier stability: skip update if loss goes above this in zscore (0.0f = off)\n"
            "  -sg <float> outlier stability: skip update if grad_norm goes above this in zscore (0.0f = off)\n"
            "  -v <int>    val_loss_every, how often we evaluate val loss (default = 20)\n"
            "  -m <int>    val_max_steps, up to how many val batches to estimate val loss? (default = 20)\n"
            "  -s <int>    sample_every, how often we inference the model (default = 20)\n"
            "  -g <int>    genT, how many steps of inference we do (default = 64)\n"
            "  -h <int>    hellaswag eval run? (default = 0)\n"
            "  -a <int>    overfit a single batch? 0/1. useful for debugging\n"
            "  -w <int>    keep f32 copy of weights for the optimizer? (default: 1)\n"
            "  -ge <int>   gelu fusion: 0=none, 1=forward, 2=forward+backward, 3=2 with gelu' kept for backward (with -r 0) (default: 2)\n"
            "  -r <int>    recompute: less memory but less speed. (default = 1), 0|1|2 = none,gelu,gelu+ln\n"
            "  -f, -z, -pn, -pr, -pg, -pi, -pf, -ps: accepted for compatibility; one process only\n");
    exit(EXIT_FAILURE);
}

bool ends_with(const std::string& s, const char* suffix) {
    const size_t n = strlen(suffix);
    return s.size() >= n && s.compare(s.size() - n, n, suffix) == 0;
}

// the largest step with a DONE_%08d file in the log dir, or -1 (find_max_step, llmc/utils.h)
int find_max_step(const char* dir) {
    DIR* d = opendir(dir);
    if (!d) return -1;
    int best = -1;
    while (dirent* e = readdir(d)) {
        int step;
        if (strncmp(e->d_name, "DONE_", 5) == 0 && sscanf(e->d_name + 5, "%d", &step) == 1 && step > best) best = step;
    }
    closedir(d);
    return best;
}

std::string step_file(const char* dir, const char* fmt, int step) {
    char name[64];
    snprintf(name, sizeof name, fmt, step);
    return std::string(dir) + "/" + name;
}

// model, state and DONE files of one step (write_checkpoint, train_gpt2.cu:1316)
void write_checkpoint(const char* dir, int step, LLMK_GPT2* model, LLMK_DataLoader* loader) {
    printf("Writing checkpoint at step %d\n", step);
    gpt2_write_to_checkpoint(model, step_file(dir, "model_%08d.bin", step).c_str());
    gpt2_save_state_with_loader(step_file(dir, "state_%08d_00000.bin", step).c_str(), step, model, loader);
    FILE* done = fopen(step_file(dir, "DONE_%08d", step).c_str(), "w");
    if (!done) { fprintf(stderr, "Error: cannot write the DONE file in %s\n", dir); exit(EXIT_FAILURE); }
    fclose(done);
}

void delete_checkpoint(const char* dir, int step) {   // train_gpt2.cu:1339
    printf("Deleting checkpoint at step %d\n", step);
    remove(step_file(dir, "model_%08d.bin", step).c_str());
    remove(step_file(dir, "state_%08d_00000.bin", step).c_str());
}

}  // namespace

int main(int argc, char** argv) {
    const char* train_data_pattern = "dev/data/tinyshakespeare/tiny_shakespeare_train.bin";
    const char* val_data_pattern = "dev/data/tinyshakespeare/tiny_shakespeare_val.bin";
    const char* load_filename = "gpt2_124M_bf16.bin";
    const char* lr_scheduler_type = "cosine";
    const char* output_log_dir = nullptr;
    int checkpoint_every = 0, checkpoints_keep = 0, major_checkpoint_every = 0, resume = 0;
    int B = 4, T = 1024, total_batch_size = -1;
    float learning_rate = 3e-4f, final_learning_rate_frac = 1.0f, weight_decay = 0.0f;
    int warmup_iterations = 0;
    float skip_update_lossz = 0.0f, skip_update_gradz = 0.0f;
    int val_loss_every = 20, val_max_steps = 20, sample_every = 20, genT = 64;
    int overfit_single_batch = 0, max_steps = -1, use_master_weights = 1, gelu_fusion = 2, recompute = 1;
    int hellaswag_eval = 0, num_processes = 1, process_rank = 0;
    for (int i = 1; i < argc; i += 2) {
        if (i + 1 >= argc || argv[i][0] != '-' || !(strlen(argv[i]) == 2 || strlen(argv[i]) == 3)) usage();
        const char a = argv[i][1], b = argv[i][2];
        const char* v = argv[i + 1];
        if (a == 'i') train_data_pattern = v;
        else if (a == 'j') val_data_pattern = v;
        else if (a == 'e') load_filename = v;
        else if (a == 'o') output_log_dir = v;
        else if (a == 'n' && b == '\0') checkpoint_every = atoi(v);
        else if (a == 'n' && b == 'k') checkpoints_keep = atoi(v);
        else if (a == 'n' && b == 'm') major_checkpoint_every = atoi(v);
        else if (a == 'y') resume = atoi(v);
        else if (a == 'b') B = atoi(v);
        else if (a == 't') T = atoi(v);
        else if (a == 'd') total_batch_size = atoi(v);
        else if (a == 'l' && b == '\0') learning_rate = (float)atof(v);
        else if (a == 'l' && b == 'g') { /* GPU utilisation printing: not available */ }
        else if (a == 'u') warmup_iterations = atoi(v);
        else if (a == 'q') final_learning_rate_frac = (float)atof(v);
        else if (a == 'c') weight_decay = (float)atof(v);
        else if (a == 'x') max_steps = atoi(v);
        else if (a == 'v') val_loss_every = atoi(v);
        else if (a == 'm') val_max_steps = atoi(v);
        else if (a == 's' && b == '\0') sample_every = atoi(v);
        else if (a == 's' && b == 'l') skip_update_lossz = (float)atof(v);
        else if (a == 's' && b == 'g') skip_update_gradz = (float)atof(v);
        else if (a == 'g' && b == 'e') gelu_fusion = atoi(v);
        else if (a == 'g') genT = atoi(v);
        else if (a == 'a') overfit_single_batch = atoi(v);
        else if (a == 'w') use_master_weights = atoi(v);
        else if (a == 'r') recompute = atoi(v);
        else if (a == 'h') hellaswag_eval = atoi(v);
        else if (a == 'k') lr_scheduler_type = v;
        else if (a == 'p' && b == 'n') num_processes = atoi(v);
        else if (a == 'p' && b == 'r') process_rank = atoi(v);
        else if (a == 'f' || a == 'z' || (a == 'p' && (b == 'g' || b == 'i' || b == 'f' || b == 's'))) { /* no effect here */ }
        else usage();
    }
    if (num_processes != 1 || process_rank != 0) {
        fprintf(stderr, "train_gpt2: this build runs one process on one GPU (-pn 1 -pr 0)\n");
        return EXIT_FAILURE;
    }
    assert(warmup_iterations >= 0);
    const int tokens_per_fwdbwd = B * T;
    if (total_batch_size == -1) total_batch_size = tokens_per_fwdbwd;
    if (total_batch_size % tokens_per_fwdbwd != 0) { fprintf(stderr, "-d must be a multiple of B*T\n"); return EXIT_FAILURE; }
    const int grad_accum_steps = total_batch_size / tokens_per_fwdbwd;

    llmk_init(0);
    if (output_log_dir) mkdir(output_log_dir, 0755);

    // ---- the model: fresh, from a file, or from the last checkpoint in the log dir ----
    int resume_max_step = -1;
    std::string resume_model, resume_state;
    if (resume == 1) {
        if (!output_log_dir) { fprintf(stderr, "-y 1 needs -o\n"); return EXIT_FAILURE; }
        resume_max_step = find_max_step(output_log_dir);
        if (resume_max_step != -1) {
            resume_model = step_file(output_log_dir, "model_%08d.bin", resume_max_step);
            resume_state = step_file(output_log_dir, "state_%08d_00000.bin", resume_max_step);
        }
    }
    const bool resuming_run = resume_max_step != -1;
    LLMK_GPT2* model = gpt2_create();
    gpt2_set_options(model, use_master_weights, recompute, gelu_fusion);
    // with master weights the parameters are re-derived from the state file; without them they are in the model file only
    // (train_gpt2.cu:1577-1578)
    if (resuming_run) gpt2_build_from_checkpoint(model, resume_model.c_str(), /*weight_init*/ use_master_weights ? 0 : 1);
    else if (ends_with(load_filename, ".bin")) gpt2_build_from_checkpoint(model, load_filename, 1);
    else gpt2_build_from_descriptor(model, load_filename);
    int cfg[6];
    gpt2_get_config(model, cfg);
    const int max_seq_len = cfg[0], vocab_size = cfg[1];
    if (T > max_seq_len) { fprintf(stderr, "T=%d exceeds the model's max_seq_len=%d\n", T, max_seq_len); return EXIT_FAILURE; }
    printf("| parameters %zu | B %d | T %d | grad accum %d | %s |\n", gpt2_num_parameters(model), B, T, grad_accum_steps,
           llmk_precision());

    // ---- loaders, schedule, log ----
    const int permute_train_loader = overfit_single_batch == 1 ? 0 : 1;
    LLMK_DataLoader* train_loader = dataloader_create();
    LLMK_DataLoader* val_loader = dataloader_create();
    dataloader_init(train_loader, train_data_pattern, B, T, 0, 1, permute_train_loader);
    dataloader_init(val_loader, val_data_pattern, B, T, 0, 1, 0);
    int train_num_batches = max_steps;
    if (train_num_batches == -1) train_num_batches = (int)(dataloader_num_tokens(train_loader) / (size_t)total_batch_size);
    int val_num_batches = (int)(dataloader_num_tokens(val_loader) / (size_t)tokens_per_fwdbwd);
    if (val_num_batches > val_max_steps) val_num_batches = val_max_steps;
    printf("| train_num_batches %d | val_num_batches %d |\n", train_num_batches, val_num_batches);
    LLMK_EvalLoader* eval_loader = nullptr;
    const char* hellaswag_path = "dev/data/hellaswag/hellaswag_val.bin";
    if (hellaswag_eval == 1) {
        struct stat st;
        if (stat(hellaswag_path, &st) == 0) {
            eval_loader = evalloader_create();
            evalloader_init(eval_loader, hellaswag_path, B, T, 0, 1);
        } else {
            printf("HellaSwag eval not found at %s, skipping its evaluation\n", hellaswag_path);
        }
    }
    LLMK_Logger* logger = logger_create();
    logger_init(logger, output_log_dir, 0, resume);
    LLMK_Tokenizer* tokenizer = tokenizer_create();
    tokenizer_init(tokenizer, "gpt2_tokenizer.bin");
    LLMK_LRScheduler* sched = lr_scheduler_create();
    lr_scheduler_init(sched, lr_scheduler_type, learning_rate, warmup_iterations, train_num_batches, final_learning_rate_frac);
    LLMK_OutlierDetector* loss_detector = outlier_detector_create();
    LLMK_OutlierDetector* norm_detector = outlier_detector_create();

    gpt2_allocate_state(model, B, T);
    int step = 0;
    if (resuming_run) gpt2_load_state_with_loader(&step, model, train_loader, resume_state.c_str());
    int* gen_tokens = (int*)malloc((size_t)B * T * sizeof(int));

    hipEvent_t start, end;
    (void)hipEventCreate(&start);
    (void)hipEventCreate(&end);
    double total_sum_iteration_time_s = 0.0;
    float ema_tokens_per_second = 0.0f;
    bool just_resumed = resuming_run;       // the checkpoint we resumed from is not written again
    for (; step <= train_num_batches; step++) {
        const bool last_step = step == train_num_batches;

        if (step % val_loss_every == 0 || last_step) {
            float val_loss = 0.0f;
            dataloader_reset(val_loader);
            for (int i = 0; i < val_num_batches; i++) {
                dataloader_next_batch(val_loader);
                val_loss += gpt2_validate(model, dataloader_inputs(val_loader), dataloader_targets(val_loader), B, T);
            }
            val_loss /= val_num_batches;
            printf("val loss %f\n", val_loss);
            logger_log_val(logger, step, val_loss);
        }

        if (eval_loader && (step % val_loss_every == 0 || last_step)) {
            float correct = 0.0f;
            evalloader_reset(eval_loader);
            for (int i = 0; i < evalloader_num_batches(eval_loader); i++) {
                evalloader_next_batch(eval_loader);
                gpt2_validate(model, evalloader_inputs(eval_loader), evalloader_targets(eval_loader), B, T);
                correct += (float)evalloader_stat_losses(eval_loader, gpt2_cpu_losses(model));
            }
            const int n = evalloader_num_examples(eval_loader);
            printf("HellaSwag: %d/%d = %f\n", (int)correct, n, correct / n);
            logger_log_eval(logger, step, correct / n);
        }

        if (sample_every > 0 && ((step > 0 && step % sample_every == 0) || last_step)) {
            unsigned long long sample_rng_state = 1337;
            const int eot = tokenizer_init_ok(tokenizer) ? tokenizer_eot_token(tokenizer) : vocab_size - 1;
            gpt2_generate(model, gen_tokens, genT < T ? genT : T, eot, &sample_rng_state);
            printf("generating:\n---\n");
            for (int t = 1; t < (genT < T ? genT : T); t++) {
                if (tokenizer_init_ok(tokenizer)) safe_printf(tokenizer_decode(tokenizer, (uint32_t)gen_tokens[t]));
                else printf("%d ", gen_tokens[t]);
            }
            printf("\n---\n");
        }

        if (checkpoint_every > 0 && output_log_dir && !just_resumed && ((step > 0 && step % checkpoint_every == 0) || last_step)) {
            write_checkpoint(output_log_dir, step, model, train_loader);
            const int step_delete = step - checkpoints_keep * checkpoint_every;
            if (checkpoints_keep > 0 && step_delete > 0 && (major_checkpoint_every == 0 || step_delete % major_checkpoint_every != 0))
                delete_checkpoint(output_log_dir, step_delete);
        }
        just_resumed = false;
        if (last_step) break;

        // ---- one optimisation step over total_batch_size tokens ----
        if (overfit_single_batch == 1) dataloader_reset(train_loader);
        (void)hipEventRecord(start, nullptr);
        float mean_loss, grad_norm, zloss, zgrad;
        const float step_learning_rate = get_learning_rate(sched, step);
        if (grad_accum_steps == 1 && skip_update_lossz == 0.0f && skip_update_gradz == 0.0f) {
            // nothing can veto the update and there is one micro-batch: the whole step is queued at once, the clipping
            // factor is formed on the device, and the host waits once (same results as the calls below, bit for bit)
            dataloader_next_batch(train_loader);
            gpt2_train_step(model, dataloader_inputs(train_loader), dataloader_targets(train_loader), step_learning_rate, 0.9f, 0.95f,
                            1e-8f, weight_decay, 1.0f, step + 1, &mean_loss, &grad_norm);
            zloss = (float)update_detector(loss_detector, (double)mean_loss);
            zgrad = (float)update_detector(norm_detector, (double)grad_norm);
        } else {
            for (int micro_step = 0; micro_step < grad_accum_steps; micro_step++) {
                dataloader_next_batch(train_loader);
                gpt2_forward(model, dataloader_inputs(train_loader), B, T);
                gpt2_backward_and_reduce(model, dataloader_inputs(train_loader), dataloader_targets(train_loader), grad_accum_steps, micro_step);
            }
            mean_loss = gpt2_mean_loss(model);
            zloss = (float)update_detector(loss_detector, (double)mean_loss);
            grad_norm = gpt2_calculate_grad_norm(model);
            zgrad = (float)update_detector(norm_detector, (double)grad_norm);
            if (std::isfinite(zloss) && skip_update_lossz != 0.0f && zloss > skip_update_lossz) {
                printf("skipping update due to loss z-score of %f\n", zloss);
            } else if (std::isfinite(zgrad) && skip_update_gradz != 0.0f && zgrad > skip_update_gradz) {
                printf("skipping update due to grad z-score of %f\n", zgrad);
            } else {
                const float grad_clip = 1.0f;
                const float grad_scale = grad_norm > grad_clip ? grad_clip / grad_norm : 1.0f;
                gpt2_update(model, step_learning_rate, 0.9f, 0.95f, 1e-8f, weight_decay, grad_scale, step + 1, 0);
            }
        }
        (void)hipEventRecord(end, nullptr);
        (void)hipEventSynchronize(end);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, start, end);
        const size_t tokens_processed = (size_t)B * T * grad_accum_steps;
        const float tokens_per_second = tokens_processed / ms * 1000.0f;
        float ema = tokens_per_second;
        if (step > 0) {                       // the first step counts as warm-up
            total_sum_iteration_time_s += ms / 1000.0f;
            ema_tokens_per_second = 0.95f * ema_tokens_per_second + 0.05f * tokens_per_second;
            ema = ema_tokens_per_second / (1.0f - powf(0.95f, (float)step));
        }
        const float mfu = gpt2_estimate_mfu(model, B * T * grad_accum_steps, ms / 1000.0f);
        printf("step %4d/%d | loss %7.6f (%+.2fz)| norm %6.4f (%+.2fz)| lr %.2e | %.2f ms | %.1f%% %s MFU | %.0f tok/s\n", step + 1,
               train_num_batches, mean_loss, zloss, grad_norm, zgrad, step_learning_rate, ms, 100 * mfu, llmk_precision(), ema);
        logger_log_train(logger, step, mean_loss, step_learning_rate, grad_norm);
    }
    if (train_num_batches > 1)
        printf("total average iteration time: %f ms\n", total_sum_iteration_time_s / (train_num_batches - 1) * 1000);

    (void)hipEventDestroy(start);
    (void)hipEventDestroy(end);
    free(gen_tokens);
    if (eval_loader) evalloader_free(eval_loader);
    dataloader_free(train_loader);
    dataloader_free(val_loader);
    tokenizer_free(tokenizer);
    lr_scheduler_free(sched);
    outlier_detector_free(loss_detector);
    outlier_detector_free(norm_detector);
    logger_free(logger);
    gpt2_free(model);
    llmk_shutdown();
    return 0;
}
