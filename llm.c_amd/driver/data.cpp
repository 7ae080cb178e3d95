// Host-side data path around the training step: token shards in, evaluation batches in, learning rate per step,
// token ids back to text, z-scores of loss and gradient norm, the run log. Re-hosts the reference's llmc/dataloader.h,
// schedulers.h, tokenizer.h, outlier_detector.h and logger.h behind
// include/llmk_data.h (same function names, same file formats, same sequence of batches for the same files and
// seed). Files are read with pread at 64-bit offsets (the reference seeks with an offset cast to int,
// dataloader.h:213, which limits a shard to 2 GiB); nothing here touches the GPU.
#include "../../include/llmk_data.h"

#include <fcntl.h>
#include <glob.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cassert>
#include <cctype>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "rand.hpp"

namespace {

constexpr int HEADER_INTS = 256;
constexpr int64_t HEADER_BYTES = HEADER_INTS * (int64_t)sizeof(int);
constexpr int COMPLETIONS = 4;                   // ASSUMED_NUM_COMPLETIONS, dataloader.h:271

[[noreturn]] void die(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    va_end(ap);
    fputc('\n', stderr);
    exit(EXIT_FAILURE);
}

int open_or_die(const char* path) {
    int fd = open(path, O_RDONLY);
    if (fd < 0) die("Error: Failed to open file '%s'", path);
    return fd;
}

void pread_or_die(int fd, void* dst, size_t bytes, int64_t offset, const char* what) {
    char* p = (char*)dst;
    while (bytes > 0) {
        ssize_t r = pread(fd, p, bytes, offset);
        if (r < 0) die("Error: File read error (%s)", what);
        if (r == 0) die("Error: Unexpected end of file (%s)", what);
        p += r; offset += r; bytes -= (size_t)r;
    }
}

int64_t file_size(int fd) {
    struct stat st;
    if (fstat(fd, &st) != 0) die("Error: cannot stat an open file");
    return (int64_t)st.st_size;
}

// Fisher-Yates from the top with randint32 % (i + 1): llmc/rand.h:229-238
void permute(std::vector<int>& v, llmk::Mt19937& rng) {
    for (int i = (int)v.size() - 1; i > 0; i--) {
        int j = (int)(rng.u32() % (uint32_t)(i + 1));
        int t = v[i]; v[i] = v[j]; v[j] = t;
    }
}

void identity(std::vector<int>& v, size_t n) {
    v.resize(n);
    for (size_t i = 0; i < n; i++) v[i] = (int)i;
}

}  // namespace

// ---------------------------------------------------------------------------------------------------------------
// training / validation shards

struct LLMK_DataLoader {
    int process_rank = 0, num_processes = 1;
    size_t B = 0, T = 0;
    size_t num_tokens = 0;               // over all shards
    size_t shard_num_samples = 0;        // samples of P*B*T tokens in the open shard
    std::vector<std::string> shards;     // in glob order
    size_t current_shard_idx = 0, current_sample_idx = 0;
    int fd = -1;
    std::vector<uint16_t> buffer;        // B*T + 1 tokens as stored
    std::vector<int> inputs, targets;
    bool should_shuffle = false;
    llmk::Mt19937 shuffle_rng{0};
    std::vector<int> shard_indices, intra_shard_indices;
    bool have_intra = false;
    size_t total_batch_size_bytes = 0, local_batch_offset_bytes = 0;
    bool initialised = false;
};

namespace {

// dataloader_load_shard_, dataloader.h:61: opens shard `shard_index` (through the permutation when shuffling),
// checks the header against the file size and returns its token count
int64_t load_shard(LLMK_DataLoader* l, int shard_index) {
    if (l->should_shuffle) shard_index = l->shard_indices[shard_index];
    const char* filename = l->shards[shard_index].c_str();
    if (l->fd >= 0) close(l->fd);
    l->fd = open_or_die(filename);
    int header[HEADER_INTS];
    pread_or_die(l->fd, header, sizeof header, 0, filename);
    if (header[0] != 20240520) {
        die("Bad magic in the data file\n---> HINT: Are you passing in a correct file?\n"
            "---> HINT: The data encoding may have changed, re-run data prepro or refer again to README.");
    }
    if (header[1] != 1) die("Bad version in data file");
    const int64_t ntok = header[2];
    if (ntok <= 0) die("Error: data file %s holds no tokens", filename);
    if (file_size(l->fd) != HEADER_BYTES + ntok * (int64_t)sizeof(uint16_t)) die("Error: file size is not as expected");
    // one token less: a batch takes B*T + 1 tokens but moves on by B*T
    l->shard_num_samples = (size_t)(ntok * sizeof(uint16_t) - sizeof(uint16_t)) / l->total_batch_size_bytes;
    return ntok;
}

void draw_intra_shard_order(LLMK_DataLoader* l) {   // prepare_intra_shard_indices_, dataloader.h:99
    identity(l->intra_shard_indices, l->shard_num_samples);
    permute(l->intra_shard_indices, l->shuffle_rng);
    l->have_intra = true;
}

void advance(LLMK_DataLoader* l) {                  // dataloader_advance_, dataloader.h:125
    if (l->current_shard_idx == l->shards.size() - 1) {   // last shard: a new epoch
        dataloader_reset(l);
        return;
    }
    l->current_shard_idx = (l->current_shard_idx + 1) % l->shards.size();
    l->current_sample_idx = 0;
    load_shard(l, (int)l->current_shard_idx);
    if (l->should_shuffle) draw_intra_shard_order(l);
}

}  // namespace

extern "C" {

LLMK_DataLoader* dataloader_create(void) { return new LLMK_DataLoader(); }

void dataloader_init(LLMK_DataLoader* l, const char* filename_pattern, size_t B, size_t T, int process_rank,
                     int num_processes, int should_shuffle) {
    l->process_rank = process_rank;
    l->num_processes = num_processes;
    l->B = B;
    l->T = T;
    l->fd = -1;
    l->should_shuffle = should_shuffle != 0;
    l->total_batch_size_bytes = (size_t)num_processes * B * T * sizeof(uint16_t);
    l->local_batch_offset_bytes = (size_t)process_rank * B * T * sizeof(uint16_t);

    glob_t g;
    if (glob(filename_pattern, 0, nullptr, &g) != 0) die("Error: failed to glob pattern: %s", filename_pattern);
    if (g.gl_pathc == 0) die("Error: no files found matching the pattern: %s", filename_pattern);
    l->shards.assign(g.gl_pathv, g.gl_pathv + g.gl_pathc);
    globfree(&g);

    if (l->should_shuffle) {
        l->shuffle_rng.reseed(42u + (uint32_t)process_rank);
        identity(l->shard_indices, l->shards.size());
        l->intra_shard_indices.clear();
        l->have_intra = false;
    }
    // every shard is opened once up front, so that a bad one is found now and not hours into a run
    int64_t total = 0;
    for (size_t s = 0; s < l->shards.size(); s++) {
        const int64_t ntok = load_shard(l, (int)s);
        if (ntok < (int64_t)((size_t)num_processes * B * T + 1))
            die("Error: shard %s holds fewer tokens than one batch over all processes", l->shards[s].c_str());
        total += ntok;
    }
    l->buffer.assign(B * T + 1, 0);
    l->inputs.assign(B * T, 0);
    l->targets.assign(B * T, 0);
    l->num_tokens = (size_t)total;
    l->initialised = true;
    dataloader_reset(l);
}

void dataloader_reset(LLMK_DataLoader* l) {
    l->current_shard_idx = 0;
    l->current_sample_idx = 0;
    if (l->should_shuffle) permute(l->shard_indices, l->shuffle_rng);   // permutes the previous epoch's order further
    load_shard(l, (int)l->current_shard_idx);
    if (l->should_shuffle) draw_intra_shard_order(l);
}

void dataloader_load_batch(LLMK_DataLoader* l) {
    assert(!l->should_shuffle || l->have_intra);
    assert(l->current_sample_idx < l->shard_num_samples);
    const size_t idx = l->should_shuffle ? (size_t)l->intra_shard_indices[l->current_sample_idx] : l->current_sample_idx;
    const int64_t offset = HEADER_BYTES + (int64_t)(idx * l->total_batch_size_bytes) + (int64_t)l->local_batch_offset_bytes;
    const size_t n = l->B * l->T;
    pread_or_die(l->fd, l->buffer.data(), (n + 1) * sizeof(uint16_t), offset, "token shard");
    for (size_t i = 0; i < n; i++) {
        l->inputs[i] = (int)l->buffer[i];
        l->targets[i] = (int)l->buffer[i + 1];
    }
}

void dataloader_next_batch(LLMK_DataLoader* l) {
    if (l->current_sample_idx >= l->shard_num_samples) advance(l);   // the shard is used up
    dataloader_load_batch(l);
    l->current_sample_idx += 1;
}

void dataloader_resume(LLMK_DataLoader* l, size_t current_shard_idx, size_t current_sample_idx) {
    l->current_shard_idx = current_shard_idx;
    l->current_sample_idx = current_sample_idx;
    load_shard(l, (int)l->current_shard_idx);
}

void dataloader_free(LLMK_DataLoader* l) {
    if (!l) return;
    if (l->fd >= 0) close(l->fd);
    delete l;
}

const int* dataloader_inputs(const LLMK_DataLoader* l) { return l->inputs.data(); }
const int* dataloader_targets(const LLMK_DataLoader* l) { return l->targets.data(); }
size_t dataloader_num_tokens(const LLMK_DataLoader* l) { return l->num_tokens; }
size_t dataloader_num_shards(const LLMK_DataLoader* l) { return l->shards.size(); }
size_t dataloader_shard_num_samples(const LLMK_DataLoader* l) { return l->shard_num_samples; }
size_t dataloader_current_shard_idx(const LLMK_DataLoader* l) { return l->current_shard_idx; }
size_t dataloader_current_sample_idx(const LLMK_DataLoader* l) { return l->current_sample_idx; }
int dataloader_should_shuffle(const LLMK_DataLoader* l) { return l->should_shuffle ? 1 : 0; }

size_t dataloader_get_shuffle_state(const LLMK_DataLoader* l, void* buf) {
    if (!l->should_shuffle) return 0;
    const size_t nshards = l->shards.size(), nsamples = l->shard_num_samples;
    const size_t rng_bytes = 8 + 4 + 4 + llmk::Mt19937::STATE_WORDS * 4 + 8;
    const size_t bytes = sizeof(size_t) + nshards * sizeof(int) + sizeof(size_t) + nsamples * sizeof(int) + rng_bytes;
    if (!buf) return bytes;
    assert(l->intra_shard_indices.size() == nsamples);
    char* p = (char*)buf;
    auto put = [&](const void* src, size_t n) { memcpy(p, src, n); p += n; };
    put(&nshards, sizeof(size_t));
    put(l->shard_indices.data(), nshards * sizeof(int));
    put(&nsamples, sizeof(size_t));
    put(l->intra_shard_indices.data(), nsamples * sizeof(int));
    const unsigned long long unused = 0;
    int32_t left; uint32_t next; uint32_t words[llmk::Mt19937::STATE_WORDS];
    l->shuffle_rng.export_state(left, next, words);
    const uint32_t matrix_a[2] = {0x0u, 0x9908b0dfu};
    put(&unused, 8); put(&left, 4); put(&next, 4); put(words, sizeof words); put(matrix_a, sizeof matrix_a);
    return bytes;
}

size_t dataloader_set_shuffle_state(LLMK_DataLoader* l, const void* buf, size_t bytes) {
    if (bytes == 0) { l->should_shuffle = false; return 0; }      // the state of a loader that does not shuffle
    const char* p = (const char*)buf;
    const char* end = p + bytes;
    auto get = [&](void* dst, size_t n) {
        if ((size_t)(end - p) < n) die("Error: dataloader state is shorter than its own counts say");
        memcpy(dst, p, n); p += n;
    };
    size_t nshards = 0, nsamples = 0;
    get(&nshards, sizeof(size_t));
    if (nshards != l->shards.size()) die("Error: dataloader state was written for %zu shards, the pattern matches %zu", nshards, l->shards.size());
    l->should_shuffle = true;
    l->shard_indices.resize(nshards);
    get(l->shard_indices.data(), nshards * sizeof(int));
    get(&nsamples, sizeof(size_t));
    l->intra_shard_indices.resize(nsamples);
    get(l->intra_shard_indices.data(), nsamples * sizeof(int));
    l->have_intra = true;
    unsigned long long unused; int32_t left; uint32_t next; uint32_t words[llmk::Mt19937::STATE_WORDS]; uint32_t matrix_a[2];
    get(&unused, 8); get(&left, 4); get(&next, 4); get(words, sizeof words); get(matrix_a, sizeof matrix_a);
    l->shuffle_rng.import_state(left, next, words);
    return (size_t)(p - (const char*)buf);
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------------------------
// multiple-choice evaluation

struct LLMK_EvalLoader {
    int process_rank = 0, num_processes = 1;
    size_t B = 0, T = 0;
    int fd = -1;
    int64_t pos = 0;                       // byte offset of the next example
    std::vector<uint16_t> buffer;
    int num_examples = 0, num_batches = 0;
    int start_example_index = 0, end_example_index = 0, current_example_index = 0;
    std::vector<int> inputs, targets, label;
    std::vector<char> mask;
    int num_completions = 0;
};

namespace {

// one example into rows 4*slot .. 4*slot+3 of the batch: evalloader_next_example_, dataloader.h:380
void next_example(LLMK_EvalLoader* l, int slot) {
    const size_t B = l->B, T = l->T;
    const int row0 = slot * COMPLETIONS;
    uint16_t head[3];                      // <START_EXAMPLE>, <EXAMPLE_BYTES>, <EXAMPLE_INDEX>
    pread_or_die(l->fd, head, sizeof head, l->pos, "evaluation file");
    if (head[0] != 65535) die("Error: evaluation example does not start with its delimiter");
    if ((int)head[2] != l->current_example_index) die("Error: evaluation example index %d where %d was expected", (int)head[2], l->current_example_index);
    const size_t body = (size_t)head[1] - sizeof head;
    if (body > l->buffer.size() * sizeof(uint16_t)) die("Error: evaluation example longer than the header's longest");
    pread_or_die(l->fd, l->buffer.data(), body, l->pos + (int64_t)sizeof head, "evaluation file");
    l->pos += head[1];
    const uint16_t* b = l->buffer.data();
    const int label = (int)b[0], ncomp = (int)b[1], ctx_len = (int)b[2];
    const int can_fit = (int)(B / COMPLETIONS);
    if (label < 0 || label >= COMPLETIONS || ncomp != COMPLETIONS) die("Error: evaluation example with label %d and %d completions", label, ncomp);
    assert(slot >= 0 && slot < can_fit);
    (void)can_fit;
    if (ctx_len <= 0 || (size_t)ctx_len >= T) die("Error: evaluation context of %d tokens does not fit T=%zu", ctx_len, T);
    l->label[slot] = label;
    l->num_completions = ncomp;
    const uint16_t* ctx = b + 3;
    for (int c = 0; c < ncomp; c++)                      // the context is shared by the four rows
        for (int i = 0; i < ctx_len; i++) l->inputs[(size_t)(row0 + c) * T + i] = (int)ctx[i];
    const uint16_t* it = ctx + ctx_len;
    for (int c = 0; c < ncomp; c++) {
        const int len = (int)it[0];
        const uint16_t* tok = it + 1;
        if (len <= 0 || (size_t)(ctx_len + len) >= T) die("Error: evaluation completion of %d tokens does not fit T=%zu", len, T);
        int* in = l->inputs.data() + (size_t)(row0 + c) * T;
        int* tg = l->targets.data() + (size_t)(row0 + c) * T;
        char* mk = l->mask.data() + (size_t)(row0 + c) * T;
        for (int i = 0; i < len; i++) {
            in[ctx_len + i] = (int)tok[i];               // the completion follows the context
            tg[ctx_len + i - 1] = (int)tok[i];           // ... and is predicted from one position earlier
            mk[ctx_len + i - 1] = 1;                     // ... which is where the loss counts
        }
        it += 1 + len;
    }
    l->current_example_index += 1;
}

}  // namespace

extern "C" {

LLMK_EvalLoader* evalloader_create(void) { return new LLMK_EvalLoader(); }

void evalloader_reset(LLMK_EvalLoader* l) {
    // process p of P owns the examples [p * ceil(N/P), (p+1) * ceil(N/P)), cropped to N
    const int per_process = (l->num_examples + l->num_processes - 1) / l->num_processes;
    const int can_fit = (int)(l->B / COMPLETIONS);
    if (can_fit == 0) {
        die("HellaSwag EvalLoader: batch size %zu is < %d\n---> HINT: Disable HellaSwag eval with -h 0, or increase batch size with -b",
            l->B, COMPLETIONS);
    }
    l->num_batches = (per_process + can_fit - 1) / can_fit;
    l->start_example_index = per_process * l->process_rank;
    l->end_example_index = per_process * (l->process_rank + 1);
    if (l->end_example_index > l->num_examples) l->end_example_index = l->num_examples;
    // skip to the first owned example by the byte counts in the example headers
    l->pos = HEADER_BYTES;
    for (int i = 0; i < l->start_example_index; i++) {
        uint16_t head[3];
        pread_or_die(l->fd, head, sizeof head, l->pos, "evaluation file");
        if (head[0] != 65535 || (int)head[2] != i || head[1] <= sizeof head) die("Error: malformed example %d in the evaluation file", i);
        l->pos += head[1];
    }
    l->current_example_index = l->start_example_index;
}

void evalloader_init(LLMK_EvalLoader* l, const char* filename, size_t B, size_t T, int process_rank, int num_processes) {
    l->process_rank = process_rank;
    l->num_processes = num_processes;
    l->B = B;
    l->T = T;
    l->fd = open_or_die(filename);
    int header[HEADER_INTS];
    pread_or_die(l->fd, header, sizeof header, 0, filename);
    if (header[0] != 20240522) die("Bad magic in eval file");
    if (header[1] != 1) die("Bad version in data file");
    l->num_examples = header[2];
    if (l->num_examples < num_processes) die("Error: %d evaluation examples for %d processes", l->num_examples, num_processes);
    const size_t longest = (size_t)header[3];
    if (longest == 0 || longest >= (size_t)(1 + COMPLETIONS) * T * 2) die("Error: longest evaluation example (%zu bytes) is not plausible for T=%zu", longest, T);
    const int can_fit = (int)(B / COMPLETIONS);
    l->buffer.assign((longest + 1) / 2, 0);
    l->inputs.assign(B * T, 0);
    l->targets.assign(B * T, 0);
    l->mask.assign(B * T, 0);
    l->label.assign(can_fit > 0 ? can_fit : 1, 0);
    evalloader_reset(l);
}

void evalloader_next_batch(LLMK_EvalLoader* l) {
    // only the mask is cleared: inputs and targets are overwritten wherever the mask is set
    memset(l->mask.data(), 0, l->mask.size());
    const int can_fit = (int)(l->B / COMPLETIONS);
    for (int i = 0; i < can_fit; i++) {
        if (l->current_example_index >= l->end_example_index) break;   // this process has no examples left
        next_example(l, i);
    }
}

int evalloader_stat_losses(const LLMK_EvalLoader* l, const float* losses) {
    int correct = 0;
    const size_t T = l->T;
    const int can_fit = (int)(l->B / COMPLETIONS);
    for (int i = 0; i < can_fit; i++) {
        float min_loss = 0.0f;
        int min_row = -1;
        bool active = false;               // a slot left empty at the end of the data has no masked positions
        for (int c = 0; c < COMPLETIONS; c++) {
            const size_t row = (size_t)(i * COMPLETIONS + c);
            float sum = 0.0f;
            int count = 0;
            for (size_t t = 0; t < T; t++) {
                if (l->mask[row * T + t] == 1) { active = true; sum += losses[row * T + t]; count++; }
            }
            if (count > 0) sum /= count;
            if (c == 0 || sum < min_loss) { min_loss = sum; min_row = c; }
        }
        if (active && min_row == l->label[i]) correct += 1;
    }
    return correct;
}

void evalloader_free(LLMK_EvalLoader* l) {
    if (!l) return;
    if (l->fd >= 0) close(l->fd);
    delete l;
}

const int* evalloader_inputs(const LLMK_EvalLoader* l) { return l->inputs.data(); }
const int* evalloader_targets(const LLMK_EvalLoader* l) { return l->targets.data(); }
const char* evalloader_mask(const LLMK_EvalLoader* l) { return l->mask.data(); }
const int* evalloader_label(const LLMK_EvalLoader* l) { return l->label.data(); }
int evalloader_num_examples(const LLMK_EvalLoader* l) { return l->num_examples; }
int evalloader_num_batches(const LLMK_EvalLoader* l) { return l->num_batches; }
int evalloader_start_example_index(const LLMK_EvalLoader* l) { return l->start_example_index; }
int evalloader_end_example_index(const LLMK_EvalLoader* l) { return l->end_example_index; }
int evalloader_current_example_index(const LLMK_EvalLoader* l) { return l->current_example_index; }

}  // extern "C"

// ---------------------------------------------------------------------------------------------------------------
// learning-rate schedules (llmc/schedulers.h:27-99). All arithmetic in float, in the reference's order.

struct LLMK_LRScheduler {
    std::string type;
    float learning_rate = 0.f;
    int warmup_iterations = 0, train_num_batches = 0;
    float final_learning_rate_frac = 0.f;
};

namespace {

float warmup_lr(const LLMK_LRScheduler* s, int step) { return s->learning_rate * ((float)(step + 1)) / s->warmup_iterations; }

float decay_ratio_from(const LLMK_LRScheduler* s, int step, int from) {
    const float r = ((float)(step - from)) / (s->train_num_batches - from);
    assert(0.0f <= r && r <= 1.0f);
    return r;
}

}  // namespace

extern "C" {

LLMK_LRScheduler* lr_scheduler_create(void) { return new LLMK_LRScheduler(); }

void lr_scheduler_init(LLMK_LRScheduler* s, const char* scheduler_type, float learning_rate, int warmup_iterations,
                       int train_num_batches, float final_learning_rate_frac) {
    s->type = scheduler_type;
    s->learning_rate = learning_rate;
    s->warmup_iterations = warmup_iterations;
    s->train_num_batches = train_num_batches;
    s->final_learning_rate_frac = final_learning_rate_frac;
}

float get_learning_rate(LLMK_LRScheduler* s, int step) {
    const float max_lr = s->learning_rate, min_lr = s->learning_rate * s->final_learning_rate_frac;
    if (s->type == "cosine") {          // linear warm-up, then half a cosine down to max_lr * final_frac
        if (step < s->warmup_iterations) return warmup_lr(s, step);
        const float coeff = 0.5f * (1.0f + cosf(M_PI * decay_ratio_from(s, step, s->warmup_iterations)));
        return min_lr + coeff * (max_lr - min_lr);
    }
    if (s->type == "linear") {          // linear warm-up, then a straight line down
        if (step < s->warmup_iterations) return warmup_lr(s, step);
        return max_lr - decay_ratio_from(s, step, s->warmup_iterations) * (max_lr - min_lr);
    }
    if (s->type == "constant") return max_lr;
    if (s->type == "wsd") {             // warm-up, constant, and over the last fifth 1 - sqrt down (arXiv 2405.18392)
        const int decay_point = (int)(0.8f * s->train_num_batches);
        if (step < s->warmup_iterations) return max_lr * (((float)(step + 1)) / s->warmup_iterations);
        if (step < decay_point) return max_lr;
        return min_lr + (1.0f - sqrtf(decay_ratio_from(s, step, decay_point))) * (max_lr - min_lr);
    }
    die("Unknown learning rate scheduler type: %s", s->type.c_str());
}

void lr_scheduler_free(LLMK_LRScheduler* s) { delete s; }

}  // extern "C"

// ---------------------------------------------------------------------------------------------------------------
// token decoder (llmc/tokenizer.h)

struct LLMK_Tokenizer {
    uint32_t vocab_size = 0;
    std::vector<std::string> table;
    int init_ok = 0;
    int eot_token = 0;
};

extern "C" {

LLMK_Tokenizer* tokenizer_create(void) { return new LLMK_Tokenizer(); }

void safe_printf(const char* piece) {
    if (piece == nullptr || piece[0] == '\0') return;
    if (piece[1] == '\0') {                // a single byte: control codes and the like are dropped
        const unsigned char byte = (unsigned char)piece[0];
        if (!(isprint(byte) || isspace(byte))) return;
    }
    printf("%s", piece);
}

void tokenizer_init(LLMK_Tokenizer* t, const char* filename) {
    t->init_ok = 0;
    FILE* f = fopen(filename, "rb");
    if (!f) {
        printf("---\nWARNING: Failed to open the tokenizer file %s\n---\n", filename);
        return;
    }
    uint32_t header[HEADER_INTS];
    if (fread(header, sizeof(uint32_t), HEADER_INTS, f) != (size_t)HEADER_INTS) die("Error: short tokenizer header in %s", filename);
    if (header[0] != 20240328) die("Bad magic in tokenizer file %s", filename);
    const int version = (int)header[1];
    t->vocab_size = header[2];
    if (version == 1) {                    // version 1 carries no end-of-text id: GPT-2's
        if (t->vocab_size != 50257) die("Tokenizer file %s: version 1 with a vocabulary of %u", filename, t->vocab_size);
        t->eot_token = 50256;
    } else if (version == 2) {
        t->eot_token = (int)header[3];
    } else {
        die("Tokenizer model file %s has bad version: %d", filename, version);
    }
    t->table.assign(t->vocab_size, std::string());
    for (uint32_t i = 0; i < t->vocab_size; i++) {
        unsigned char length;
        if (fread(&length, 1, 1, f) != 1 || length == 0) die("Error: tokenizer file %s: bad length for token %u", filename, i);
        t->table[i].resize(length);
        if (fread(&t->table[i][0], 1, length, f) != length) die("Error: tokenizer file %s ends inside token %u", filename, i);
    }
    fclose(f);
    t->init_ok = 1;
}

const char* tokenizer_decode(LLMK_Tokenizer* t, uint32_t token_id) {
    if (t->init_ok == 0) return nullptr;
    if (token_id < t->vocab_size) return t->table[token_id].c_str();
    printf("invalid token id %u!\n", token_id);
    return nullptr;
}

void tokenizer_free(LLMK_Tokenizer* t) { delete t; }
int tokenizer_init_ok(const LLMK_Tokenizer* t) { return t->init_ok; }
int tokenizer_eot_token(const LLMK_Tokenizer* t) { return t->eot_token; }
uint32_t tokenizer_vocab_size(const LLMK_Tokenizer* t) { return t->vocab_size; }

}  // extern "C"

// ---------------------------------------------------------------------------------------------------------------
// outlier detector (llmc/outlier_detector.h) and run log (llmc/logger.h)

struct LLMK_OutlierDetector {
    static constexpr int WINDOW = 128;
    double buffer[WINDOW];
    int count = 0, index = 0;
    double sum = 0.0, sum_sq = 0.0;
};

struct LLMK_Logger {
    int active = 0;
    std::string path;
};

namespace {

void append_line(const LLMK_Logger* lg, const char* fmt, ...) {
    if (lg->active != 1) return;
    FILE* f = fopen(lg->path.c_str(), "a");
    if (!f) die("Error: Failed to open file '%s'", lg->path.c_str());
    va_list ap;
    va_start(ap, fmt);
    vfprintf(f, fmt, ap);
    va_end(ap);
    fclose(f);
}

}  // namespace

extern "C" {

LLMK_OutlierDetector* outlier_detector_create(void) {
    LLMK_OutlierDetector* d = new LLMK_OutlierDetector();
    init_detector(d);
    return d;
}

void init_detector(LLMK_OutlierDetector* d) {
    for (double& x : d->buffer) x = 0.0;
    d->count = 0; d->index = 0; d->sum = 0.0; d->sum_sq = 0.0;
}

double update_detector(LLMK_OutlierDetector* d, double v) {
    constexpr int W = LLMK_OutlierDetector::WINDOW;
    if (d->count < W) {                    // still filling the window
        d->buffer[d->count++] = v;
        d->sum += v;
        d->sum_sq += v * v;
        return nan("");
    }
    const double old = d->buffer[d->index];   // the oldest value leaves, the new one takes its place
    d->sum -= old;
    d->sum_sq -= old * old;
    d->buffer[d->index] = v;
    d->sum += v;
    d->sum_sq += v * v;
    d->index = (d->index + 1) % W;
    const double mean = d->sum / W;
    const double std_dev = sqrt(d->sum_sq / W - mean * mean);
    if (std_dev == 0.0) return 0.0;
    return (v - mean) / std_dev;
}

void outlier_detector_free(LLMK_OutlierDetector* d) { delete d; }

LLMK_Logger* logger_create(void) { return new LLMK_Logger(); }

void logger_init(LLMK_Logger* lg, const char* log_dir, int process_rank, int resume) {
    lg->active = 0;
    if (log_dir == nullptr || process_rank != 0) return;   // only the first process writes
    lg->active = 1;
    lg->path = std::string(log_dir) + "/main.log";
    if (resume == 0) {                                      // a fresh run starts from an empty file
        FILE* f = fopen(lg->path.c_str(), "w");
        if (!f) die("Error: Failed to open file '%s'", lg->path.c_str());
        fclose(f);
    }
}

void logger_log_eval(LLMK_Logger* lg, int step, float val) { append_line(lg, "s:%d eval:%.4f\n", step, val); }
void logger_log_val(LLMK_Logger* lg, int step, float val_loss) { append_line(lg, "s:%d tel:%.4f\n", step, val_loss); }
void logger_log_train(LLMK_Logger* lg, int step, float train_loss, float learning_rate, float grad_norm) {
    append_line(lg, "s:%d trl:%.4f lr:%.6f norm:%.2f\n", step, train_loss, learning_rate, grad_norm);
}
void logger_free(LLMK_Logger* lg) { delete lg; }

}  // extern "C"
