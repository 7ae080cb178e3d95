// Host driver: the reference's GPT2 object (train_gpt2.cu:87-1168, :1209-1314) on top of the
// llmk.h kernel ABI. Same parameter / gradient / activation arenas, same order of launcher
// calls, same buffer aliasing, same .bin checkpoint and state layouts. Host C++ only: every
// device operation goes through llmk.h or plain HIP runtime calls (malloc / memcpy / memset).
//
// The storage type is opaque here (the kernel library says how wide it is), so the same source
// serves the bf16 and the fp32 library.
#include <hip/hip_runtime.h>
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <algorithm>

// 1: the residual adds of the forward pass run as epilogues of the projections that feed them (see the layer loop);
// 0: the reference's call sequence, projection into a scratch buffer and then the fused residual + LayerNorm kernel
#ifndef LLMK_FUSE_RESIDUAL
#define LLMK_FUSE_RESIDUAL 1
#endif

#include "../../include/llmk.h"
#include "../../include/llmk_gpt2.h"
#include "../../include/llmk_data.h"
#include "rand.hpp"

#define hipCheck(expr)                                                                            \
    do {                                                                                          \
        hipError_t e__ = (expr);                                                                  \
        if (e__ != hipSuccess) {                                                                  \
            fprintf(stderr, "[HIP ERROR] at %s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e__)); \
            exit(EXIT_FAILURE);                                                                   \
        }                                                                                         \
    } while (0)

namespace {

constexpr int NUM_PARAMETER_TENSORS = 16;
constexpr int NUM_ACTIVATION_TENSORS = 21;
constexpr size_t IO_BUF_SIZE = 32 * 1024 * 1024;
// MI355X dense matrix peaks (TFLOP/s) used as the MFU denominator; the reference's table
// (llmc/mfu.h:42-152) has no AMD entry
constexpr float MI355X_PEAK_BF16_TFLOPS = 2500.0f;
constexpr float MI355X_PEAK_FP32_TFLOPS = 157.3f;

struct GPT2Config { int max_seq_len, vocab_size, padded_vocab_size, num_layers, num_heads, channels; };

// byte pointers: the element width is a run-time property of the kernel library
typedef char* xptr;

struct ParameterTensors {   // order of train_gpt2.cu:97-116
    xptr wte, wpe, ln1w, ln1b, qkvw, qkvb, attprojw, attprojb, ln2w, ln2b, fcw, fcb, fcprojw, fcprojb, lnfw, lnfb;
};
struct ActivationTensors {  // train_gpt2.cu:171-207, cuDNN branch: att holds fp32 row statistics
    xptr encoded, ln1;
    float *ln1_mean, *ln1_rstd;
    xptr atty;
    float* att;
    xptr residual2, ln2;
    float *ln2_mean, *ln2_rstd;
    xptr fch, fch_gelu, residual3, lnf;
    float *lnf_mean, *lnf_rstd, *losses;
    xptr qkvr, output, scratch_bt4c, scratch_btc;
};
struct TensorSpec { void** ptr; size_t size; size_t elem; };

}  // namespace

struct LLMK_GPT2 {
    GPT2Config config{};
    size_t X = 2;                              // sizeof(floatX) of the kernel library
    ParameterTensors params{};
    size_t param_elements[NUM_PARAMETER_TENSORS]{};
    void* params_memory = nullptr;
    size_t num_parameters = 0, num_parameters_bytes = 0;
    ParameterTensors grads{};
    void* grads_memory = nullptr;
    float *m_memory = nullptr, *v_memory = nullptr, *master_weights = nullptr;
    ActivationTensors acts{};
    TensorSpec acts_specs[NUM_ACTIVATION_TENSORS]{};
    void* acts_memory = nullptr;
    size_t acts_bytes = 0;
    int batch_size = 0, seq_len = 0;
    int *inputs = nullptr, *targets = nullptr;
    float mean_loss = -1.0f;
    float* accumulated_mean_loss = nullptr;
    float* cpu_losses = nullptr;
    unsigned long long rng_state = 13371337ull, rng_state_last_update = 0;
    int use_master_weights = 1;
    bool init_state = true;
    int gelu_fusion = 0, recompute = 1;
    int* workload_indices = nullptr;
    int* bucket_info = nullptr;
    hipStream_t stream = nullptr;
};

namespace {

xptr off(xptr p, size_t elems, size_t X) { return p + elems * X; }

// ---- host-side conversions between fp32 and the storage type --------------------------------
uint16_t f32_to_bf16_rne(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
void to_storage(void* dst, const float* src, size_t n, size_t X) {
    if (X == 4) { memcpy(dst, src, n * 4); return; }
    uint16_t* d = (uint16_t*)dst;
    for (size_t i = 0; i < n; i++) d[i] = f32_to_bf16_rne(src[i]);
}
void from_storage(float* dst, const void* src, size_t n, size_t X) {
    if (X == 4) { memcpy(dst, src, n * 4); return; }
    const uint16_t* s = (const uint16_t*)src;
    for (size_t i = 0; i < n; i++) { uint32_t u = (uint32_t)s[i] << 16; memcpy(&dst[i], &u, 4); }
}

void fill_in_parameter_sizes(size_t* sz, const GPT2Config& c) {   // train_gpt2.cu:118-139
    size_t Vp = c.padded_vocab_size, C = c.channels, maxT = c.max_seq_len, L = c.num_layers;
    sz[0] = Vp * C; sz[1] = maxT * C; sz[2] = L * C; sz[3] = L * C; sz[4] = L * 3 * C * C; sz[5] = L * 3 * C;
    sz[6] = L * C * C; sz[7] = L * C; sz[8] = L * C; sz[9] = L * C; sz[10] = L * 4 * C * C; sz[11] = L * 4 * C;
    sz[12] = L * C * 4 * C; sz[13] = L * C; sz[14] = C; sz[15] = C;
}

void* malloc_and_point_parameters(ParameterTensors* p, const size_t* elems, size_t X) {  // train_gpt2.cu:147
    size_t bytes = 0;
    for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) bytes += elems[i] * X;
    void* mem;
    hipCheck(hipMalloc(&mem, bytes));
    xptr* ptrs[] = {&p->wte, &p->wpe, &p->ln1w, &p->ln1b, &p->qkvw, &p->qkvb, &p->attprojw, &p->attprojb,
                    &p->ln2w, &p->ln2b, &p->fcw, &p->fcb, &p->fcprojw, &p->fcprojb, &p->lnfw, &p->lnfb};
    xptr it = (xptr)mem;
    for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) { *ptrs[i] = it; it += elems[i] * X; }
    return mem;
}

// What the kernels behind this driver can run, checked before anything is allocated: channels a multiple of 8 (one
// 16-byte vector of bf16), at most 64 lanes x 8 vectors per row in LayerNorm backward (4096 channels in bf16, 2048 in
// fp32), heads of at most 128 channels.
static void check_config(const LLMK_GPT2* m) {
    const GPT2Config& c = m->config;
    const int max_channels = 8 * 64 * (16 / (int)m->X);
    const char* why = nullptr;
    if (c.channels <= 0 || c.num_heads <= 0 || c.num_layers <= 0 || c.max_seq_len <= 0) why = "sizes must be positive";
    else if (c.channels % 8 != 0) why = "channels must be a multiple of 8";
    else if (c.channels > max_channels) why = "too many channels for this precision's LayerNorm backward";
    else if (c.channels % c.num_heads != 0) why = "channels must divide into the heads";
    else if (c.channels / c.num_heads > 128) why = "head size above 128";
    else if (c.padded_vocab_size < c.vocab_size || c.padded_vocab_size % 8 != 0) why = "padded vocabulary must cover the vocabulary and be a multiple of 8";
    if (why) {
        fprintf(stderr, "Unsupported model (layers %d, heads %d, channels %d, vocabulary %d/%d) in the %s build: %s (channels <= %d)\n",
                c.num_layers, c.num_heads, c.channels, c.vocab_size, c.padded_vocab_size, m->X == 2 ? "bf16" : "fp32", why, max_channels);
        exit(EXIT_FAILURE);
    }
}

void gpt2_allocate_weights(LLMK_GPT2* m) {   // train_gpt2.cu:353
    check_config(m);
    fill_in_parameter_sizes(m->param_elements, m->config);
    m->num_parameters = 0;
    for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) m->num_parameters += m->param_elements[i];
    m->num_parameters_bytes = m->num_parameters * m->X;
    assert(m->params_memory == nullptr);
    m->params_memory = malloc_and_point_parameters(&m->params, m->param_elements, m->X);
}

size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

// train_gpt2.cu:219-254, cuDNN branch. The `output` scratchpad is additionally made large enough
// for every scratch use the backward pass puts it to (the reference relies on B*T*Vp dwarfing them).
void fill_in_activation_sizes(LLMK_GPT2* m, size_t B, size_t T) {
    const GPT2Config& c = m->config;
    size_t Vp = c.padded_vocab_size, L = c.num_layers, NH = c.num_heads, C = c.channels, X = m->X;
    int R = m->recompute;
    ActivationTensors* a = &m->acts;
    size_t out_elems = B * T * std::max(3 * C, std::max(NH * T, Vp));
    size_t scratch_bytes = std::max({llmk_layernorm_backward_scratch_floats((int)C) * sizeof(float),
                                     llmk_matmul_backward_bias_scratch_floats((int)(4 * C)) * sizeof(float),
                                     B * T * ceil_div(C, 64 * (16 / X)) * 20 + 64,
                                     (size_t)4096 * sizeof(float)});
    out_elems = std::max(out_elems, ceil_div(scratch_bytes, X));
    TensorSpec* t = m->acts_specs;
    t[0] = {(void**)&a->encoded, B * T * C, X};
    t[1] = {(void**)&a->ln1, R < 2 ? L * B * T * C : 0, X};
    t[2] = {(void**)&a->ln1_mean, L * B * T, 4};
    t[3] = {(void**)&a->ln1_rstd, L * B * T, 4};
    t[4] = {(void**)&a->atty, L * B * T * C, X};
    t[5] = {(void**)&a->att, L * B * NH * T, 4};
    t[6] = {(void**)&a->residual2, L * B * T * C, X};
    t[7] = {(void**)&a->ln2, R < 2 ? L * B * T * C : 0, X};
    t[8] = {(void**)&a->ln2_mean, L * B * T, 4};
    t[9] = {(void**)&a->ln2_rstd, L * B * T, 4};
    t[10] = {(void**)&a->fch, L * B * T * 4 * C, X};
    t[11] = {(void**)&a->fch_gelu, R < 1 ? L * B * T * 4 * C : B * T * 4 * C, X};
    t[12] = {(void**)&a->residual3, L * B * T * C, X};
    t[13] = {(void**)&a->lnf, B * T * C, X};
    t[14] = {(void**)&a->lnf_mean, B * T, 4};
    t[15] = {(void**)&a->lnf_rstd, B * T, 4};
    t[16] = {(void**)&a->losses, B * T, 4};
    t[17] = {(void**)&a->qkvr, L * B * T * 3 * C, X};
    t[18] = {(void**)&a->output, out_elems, X};
    t[19] = {(void**)&a->scratch_bt4c, B * T * 4 * C, X};
    t[20] = {(void**)&a->scratch_btc, B * T * C, X};
}

void* malloc_and_point_activations(LLMK_GPT2* m) {   // train_gpt2.cu:256
    size_t bytes = 0;
    for (int i = 0; i < NUM_ACTIVATION_TENSORS; i++) bytes += ceil_div(m->acts_specs[i].size * m->acts_specs[i].elem, 256) * 256;
    m->acts_bytes = bytes;
    printf("allocating %d MiB for activations\n", (int)round(bytes / (1024.0 * 1024.0)));
    void* mem;
    hipCheck(hipMalloc(&mem, bytes));
    hipCheck(hipMemset(mem, 0, bytes));
    char* it = (char*)mem;
    for (int i = 0; i < NUM_ACTIVATION_TENSORS; i++) {
        TensorSpec& s = m->acts_specs[i];
        if (s.size == 0) { *s.ptr = nullptr; continue; }
        *s.ptr = it;
        it += ceil_div(s.size * s.elem, 256) * 256;      // every tensor starts 256-byte aligned
    }
    return mem;
}

void set_hyperparameters_gpt2(GPT2Config* c, const char* depth_str) {   // train_gpt2.cu:519
    int depth = atoi(depth_str), ch = 0, nh = 0;
    if (depth == 6) { ch = 384; nh = 6; }
    else if (depth == 12) { ch = 768; nh = 12; }
    else if (depth == 24) { ch = 1024; nh = 16; }
    else if (depth == 36) { ch = 1280; nh = 20; }
    else if (depth == 48) { ch = 1600; nh = 25; }
    else if (depth == 60) { ch = 1920; nh = 30; }
    else if (depth == 72) { ch = 2880; nh = 30; }
    else if (depth == 84) { ch = 3456; nh = 36; }
    else { fprintf(stderr, "Unsupported GPT-2 depth: %d\n", depth); exit(EXIT_FAILURE); }
    c->num_layers = depth; c->channels = ch; c->num_heads = nh; c->max_seq_len = 1024;
}
void set_hyperparameters_gpt3(GPT2Config* c, const char* channels_str) {   // train_gpt2.cu:538
    int ch = atoi(channels_str), depth = 0, hsz = 0;
    if (ch == 384) { depth = 6; hsz = 64; }
    else if (ch == 768) { depth = 12; hsz = 64; }
    else if (ch == 1024) { depth = 24; hsz = 64; }
    else if (ch == 1536) { depth = 24; hsz = 96; }
    else if (ch == 2048) { depth = 24; hsz = 128; }
    else if (ch == 2560) { depth = 32; hsz = 80; }
    else if (ch == 4096) { depth = 32; hsz = 128; }
    else if (ch == 5140) { depth = 40; hsz = 128; }
    else if (ch == 12288) { depth = 96; hsz = 128; }
    else { fprintf(stderr, "Unsupported GPT-3 channels: %d\n", ch); exit(EXIT_FAILURE); }
    c->num_layers = depth; c->channels = ch; c->num_heads = ch / hsz; c->max_seq_len = 2048;
}

// train_gpt2.cu:587-637: N(0,0.02) in PyTorch module order, residual projections / sqrt(2L),
// LayerNorm weights 1, biases and padded wte rows 0; fp32 draw then round to the storage type.
void random_init(LLMK_GPT2* m, unsigned int seed) {
    const size_t L = m->config.num_layers;
    std::vector<float> cpu(m->num_parameters, 0.0f);
    size_t offs[NUM_PARAMETER_TENSORS], o = 0;
    for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) { offs[i] = o; o += m->param_elements[i]; }
    for (int i : {2, 8, 14}) std::fill(cpu.begin() + offs[i], cpu.begin() + offs[i] + m->param_elements[i], 1.0f);
    llmk::Mt19937 rng(seed);
    const float residual_scale = 1.0f / sqrtf(2.0f * (float)L);
    for (size_t l = 0; l < L; l++) {
        for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) {
            const bool embed = (l == 0 && (i == 0 || i == 1));
            const bool matrix = (i == 4 || i == 6 || i == 10 || i == 12);
            if (!embed && !matrix) continue;
            size_t n = m->param_elements[i], layer_off = 0;
            if (i == 0) n = (size_t)m->config.vocab_size * m->config.channels;
            if (matrix) { n /= L; layer_off = l * n; }
            const float std = (i == 6 || i == 12) ? 0.02f * residual_scale : 0.02f;
            rng.normal(cpu.data() + offs[i] + layer_off, (uint32_t)n, 0.0f, std);
        }
    }
    std::vector<char> stor(m->num_parameters_bytes);
    to_storage(stor.data(), cpu.data(), m->num_parameters, m->X);
    hipCheck(hipMemcpy(m->params_memory, stor.data(), m->num_parameters_bytes, hipMemcpyHostToDevice));
}

void token_check(const int* tokens, size_t n, int V) {   // llmc/utils.h tokenCheck
    for (size_t i = 0; i < n; i++) {
        if (tokens[i] < 0 || tokens[i] >= V) {
            fprintf(stderr, "Error: token %d at position %zu out of range [0, %d)\n", tokens[i], i, V);
            exit(EXIT_FAILURE);
        }
    }
}

// device <-> file through a pinned bounce buffer (llmc/cuda_common.h:130-207)
void device_to_file(FILE* f, const void* src, size_t bytes, hipStream_t st) {
    char* buf;
    hipCheck(hipHostMalloc((void**)&buf, IO_BUF_SIZE));
    for (size_t done = 0; done < bytes;) {
        size_t n = std::min(IO_BUF_SIZE, bytes - done);
        hipCheck(hipMemcpyAsync(buf, (const char*)src + done, n, hipMemcpyDeviceToHost, st));
        hipCheck(hipStreamSynchronize(st));
        if (fwrite(buf, 1, n, f) != n) { fprintf(stderr, "Error: file write failed\n"); exit(EXIT_FAILURE); }
        done += n;
    }
    hipCheck(hipHostFree(buf));
}
void file_to_device(void* dst, FILE* f, size_t bytes, hipStream_t st) {
    char* buf;
    hipCheck(hipHostMalloc((void**)&buf, IO_BUF_SIZE));
    for (size_t done = 0; done < bytes;) {
        size_t n = std::min(IO_BUF_SIZE, bytes - done);
        if (fread(buf, 1, n, f) != n) { fprintf(stderr, "Error: unexpected end of file\n"); exit(EXIT_FAILURE); }
        hipCheck(hipMemcpyAsync((char*)dst + done, buf, n, hipMemcpyHostToDevice, st));
        hipCheck(hipStreamSynchronize(st));
        done += n;
    }
    hipCheck(hipHostFree(buf));
}

struct ShardInfo { ptrdiff_t offset; size_t size; };
ShardInfo tensor_at_layer(const LLMK_GPT2* m, int layer_id, int id) {   // train_gpt2.cu:977
    ptrdiff_t offset = 0;
    for (int i = 0; i < id; i++) offset += (ptrdiff_t)m->param_elements[i];
    size_t size = m->param_elements[id];
    if (2 <= id && id <= 13) { size /= m->config.num_layers; offset += (ptrdiff_t)(layer_id * size); }
    return {offset, size};
}

}  // namespace

extern "C" {

LLMK_GPT2* gpt2_create(void) {
    LLMK_GPT2* m = new LLMK_GPT2();
    m->X = (size_t)llmk_sizeof_floatx();
    hipCheck(hipStreamCreate(&m->stream));
    return m;
}

// gelu_fusion 3 leaves gelu'(fch) in the fch tensor; recomputing fch_gelu in the backward pass (recompute >= 1) needs
// fch itself, so those runs take level 2
static int gelu_fusion_in_use(const LLMK_GPT2* m) { return (m->gelu_fusion >= 3 && m->recompute >= 1) ? 2 : m->gelu_fusion; }

void gpt2_set_options(LLMK_GPT2* m, int use_master_weights, int recompute, int gelu_fusion) {
    if (use_master_weights >= 0) m->use_master_weights = use_master_weights;
    if (recompute >= 0) m->recompute = recompute;
    if (gelu_fusion >= 0) m->gelu_fusion = gelu_fusion;
}

void gpt2_build_from_descriptor(LLMK_GPT2* m, const char* d) {
    assert(d != nullptr);
    size_t len = strlen(d);
    if (len > 1 && d[0] == 'd') set_hyperparameters_gpt2(&m->config, d + 1);
    else if (len > 6 && strncmp(d, "gpt2:d", 6) == 0) set_hyperparameters_gpt2(&m->config, d + 6);
    else if (len > 6 && strncmp(d, "gpt3:c", 6) == 0) set_hyperparameters_gpt3(&m->config, d + 6);
    else { fprintf(stderr, "Unsupported model descriptor: %s\n", d); exit(EXIT_FAILURE); }
    m->config.vocab_size = 50257;
    m->config.padded_vocab_size = 50304;
    gpt2_allocate_weights(m);
    random_init(m, 42);
}

void gpt2_build_from_config(LLMK_GPT2* m, int max_seq_len, int vocab_size, int padded_vocab_size, int num_layers,
                            int num_heads, int channels, unsigned int seed) {
    m->config = GPT2Config{max_seq_len, vocab_size, padded_vocab_size, num_layers, num_heads, channels};
    gpt2_allocate_weights(m);
    random_init(m, seed);
}

void gpt2_build_from_checkpoint(LLMK_GPT2* m, const char* path, int weight_init) {
    FILE* f = fopen(path, "rb");
    if (!f) { fprintf(stderr, "Error: Failed to open file '%s'\n", path); exit(EXIT_FAILURE); }
    int hdr[256];
    if (fread(hdr, sizeof(int), 256, f) != 256) { fprintf(stderr, "Error: short model header\n"); exit(EXIT_FAILURE); }
    if (hdr[0] != 20240326) { fprintf(stderr, "Bad magic model file\n"); exit(EXIT_FAILURE); }
    int version = hdr[1];
    if (!(version == 3 || version == 5)) { fprintf(stderr, "Bad version in model file\n"); exit(EXIT_FAILURE); }
    if (weight_init) {
        if (m->X == 2 && version != 5) {
            fprintf(stderr, "Precision is configured as BF16 but model at %s is not.\n", path);
            exit(EXIT_FAILURE);
        }
        if (m->X == 4 && version != 3) {
            fprintf(stderr, "Precision is configured as FP32 but model at %s is not.\n", path);
            exit(EXIT_FAILURE);
        }
    }
    m->config = GPT2Config{hdr[2], hdr[3], hdr[7], hdr[4], hdr[5], hdr[6]};
    gpt2_allocate_weights(m);
    if (weight_init) file_to_device(m->params_memory, f, m->num_parameters_bytes, m->stream);
    fclose(f);
    hipCheck(hipDeviceSynchronize());
}

void gpt2_write_to_checkpoint(LLMK_GPT2* m, const char* path) {
    FILE* f = fopen(path, "wb");
    if (!f) { fprintf(stderr, "Error: Failed to open file '%s'\n", path); exit(EXIT_FAILURE); }
    int hdr[256];
    memset(hdr, 0, sizeof hdr);
    hdr[0] = 20240326; hdr[1] = m->X == 4 ? 3 : 5;
    hdr[2] = m->config.max_seq_len; hdr[3] = m->config.vocab_size; hdr[4] = m->config.num_layers;
    hdr[5] = m->config.num_heads; hdr[6] = m->config.channels; hdr[7] = m->config.padded_vocab_size;
    fwrite(hdr, sizeof(int), 256, f);
    device_to_file(f, m->params_memory, m->num_parameters_bytes, m->stream);
    fclose(f);
}

void gpt2_allocate_state(LLMK_GPT2* m, int B, int T) {
    assert(m->grads_memory == nullptr);
    m->grads_memory = malloc_and_point_parameters(&m->grads, m->param_elements, m->X);
    m->batch_size = B; m->seq_len = T;
    fill_in_activation_sizes(m, B, T);
    m->acts_memory = malloc_and_point_activations(m);
    hipCheck(hipMalloc((void**)&m->inputs, (size_t)B * T * sizeof(int)));
    hipCheck(hipMalloc((void**)&m->targets, (size_t)B * T * sizeof(int)));
    hipCheck(hipMalloc((void**)&m->accumulated_mean_loss, sizeof(float)));
    hipCheck(hipHostMalloc((void**)&m->cpu_losses, (size_t)B * T * sizeof(float)));
    size_t ncg = ceil_div(m->config.channels, 64 * (16 / m->X));
    // pinned: the copies of the sorted buckets to the device (llmk_encoder_backward) are then queued without a wait, and the
    // kernel that reads them right behind
    hipCheck(hipHostMalloc((void**)&m->workload_indices, sizeof(int) * (size_t)B * T * ncg));
    hipCheck(hipHostMalloc((void**)&m->bucket_info, sizeof(int) * 4 * (size_t)B * T * ncg));
    hipCheck(hipMalloc((void**)&m->m_memory, m->num_parameters * sizeof(float)));
    hipCheck(hipMalloc((void**)&m->v_memory, m->num_parameters * sizeof(float)));
    if (m->use_master_weights == 1) hipCheck(hipMalloc((void**)&m->master_weights, m->num_parameters * sizeof(float)));
    // the library's workspace at its final size now, so that no training step allocates (the reference sizes its
    // cuBLASLt workspace once, llmc/cublas_common.h:28-31)
    const int C = m->config.channels, Vp = m->config.padded_vocab_size, NH = m->config.num_heads;
    size_t ws = llmk_attention_backward_workspace_bytes(B, T, NH);
    const int shapes[5][2] = {{C, 3 * C}, {C, C}, {C, 4 * C}, {4 * C, C}, {C, Vp}};
    for (const auto& sh : shapes) ws = std::max(ws, llmk_matmul_backward_workspace_bytes(B, T, sh[0], sh[1]));
    llmk_workspace_reserve(ws);
}

namespace {
void forward_impl(LLMK_GPT2* m, const int* inputs, size_t B, size_t T, bool wait) {
    if (m->params_memory == nullptr) { printf("Error: model was not initialized properly.\n"); exit(EXIT_FAILURE); }
    const size_t Vp = m->config.padded_vocab_size, L = m->config.num_layers, NH = m->config.num_heads,
                 C = m->config.channels, X = m->X;
    if (B > (size_t)m->batch_size || T > (size_t)m->seq_len) {
        printf("Model: B=%d T=%d, Desired: B=%d T=%d\n", m->batch_size, m->seq_len, (int)B, (int)T);
        exit(EXIT_FAILURE);
    }
    hipStream_t st = m->stream;
    hipCheck(hipMemcpyAsync(m->inputs, inputs, B * T * sizeof(int), hipMemcpyHostToDevice, st));
    token_check(inputs, B * T, m->config.vocab_size);

    ParameterTensors p = m->params;
    ActivationTensors a = m->acts;
    const int R = m->recompute;
    llmk_encoder_forward(a.encoded, m->inputs, p.wte, p.wpe, (int)B, (int)T, (int)C, st);
    llmk_layernorm_forward(R < 2 ? a.ln1 : a.lnf, a.ln1_mean, a.ln1_rstd, a.encoded, p.ln1w, p.ln1b, (int)B, (int)T, (int)C, st);

    for (size_t l = 0; l < L; l++) {
        xptr residual = l == 0 ? a.encoded : off(a.residual3, (l - 1) * B * T * C, X);
        xptr l_qkvw = off(p.qkvw, l * 3 * C * C, X), l_qkvb = off(p.qkvb, l * 3 * C, X);
        xptr l_attprojw = off(p.attprojw, l * C * C, X), l_attprojb = off(p.attprojb, l * C, X);
        xptr l_ln2w = off(p.ln2w, l * C, X), l_ln2b = off(p.ln2b, l * C, X);
        xptr l_fcw = off(p.fcw, l * 4 * C * C, X), l_fcb = off(p.fcb, l * 4 * C, X);
        xptr l_fcprojw = off(p.fcprojw, l * C * 4 * C, X), l_fcprojb = off(p.fcprojb, l * C, X);

        xptr l_ln1 = R < 2 ? off(a.ln1, l * B * T * C, X) : a.lnf;
        xptr l_qkvr = off(a.qkvr, l * B * T * 3 * C, X);
        xptr l_atty = off(a.atty, l * B * T * C, X);
        xptr l_residual2 = off(a.residual2, l * B * T * C, X);
        xptr l_ln2 = R < 2 ? off(a.ln2, l * B * T * C, X) : a.lnf;
        float* l_ln2_mean = a.ln2_mean + l * B * T;
        float* l_ln2_rstd = a.ln2_rstd + l * B * T;
        xptr l_fch = off(a.fch, l * B * T * 4 * C, X);
        xptr l_fch_gelu = R < 1 ? off(a.fch_gelu, l * B * T * 4 * C, X) : a.fch_gelu;
        xptr l_residual3 = off(a.residual3, l * B * T * C, X);
        xptr scratch = a.output;
        float* l_att = a.att + l * B * NH * T;

        llmk_matmul_forward(l_qkvr, l_ln1, l_qkvw, l_qkvb, (int)B, (int)T, (int)C, (int)(3 * C), st, nullptr, 1);
        llmk_attention_forward(l_atty, l_att, l_qkvr, (int)B, (int)T, (int)NH, (int)C, st);
        // The two projections into the residual stream. The reference runs matmul_forward into a scratch buffer and then
        // fused_residual_forward5 (train_gpt2.cu:713-727: residual add + LayerNorm); here the add is the projection's
        // epilogue (llmk_matmul_forward_residual: the same two roundings, the same bits) and a plain LayerNorm follows,
        // which reads and writes one tensor less per instance.
        xptr n_ln = l + 1 != L ? (R < 2 ? off(a.ln1, (l + 1) * B * T * C, X) : a.lnf) : a.lnf;
        float* n_mean = l + 1 != L ? a.ln1_mean + (l + 1) * B * T : a.lnf_mean;
        float* n_rstd = l + 1 != L ? a.ln1_rstd + (l + 1) * B * T : a.lnf_rstd;
        xptr n_w = l + 1 != L ? off(p.ln1w, (l + 1) * C, X) : p.lnfw, n_b = l + 1 != L ? off(p.ln1b, (l + 1) * C, X) : p.lnfb;
        // (Measured on whole steps, both call sequences in one process: 124M -0.80 ms of 58.3, 350M -0.55 ms of 79.0, 1558M
        // -0.9 ms of 183.9. Widths that are multiples of 64: a wave's 64 columns are then all inside the output or all
        // outside, which is what the epilogue's counted loads need on the ragged last tile column of the 1600-wide model.)
        const bool fuse_residual = LLMK_FUSE_RESIDUAL && C % 64 == 0 && X == 2;   // (the fp32 library has no such epilogue)
        if (fuse_residual) {
            llmk_matmul_forward_residual(l_residual2, l_atty, l_attprojw, l_attprojb, residual, (int)B, (int)T, (int)C, (int)C, st);
            llmk_layernorm_forward(l_ln2, l_ln2_mean, l_ln2_rstd, l_residual2, l_ln2w, l_ln2b, (int)B, (int)T, (int)C, st);
            llmk_matmul_forward(l_fch_gelu, l_ln2, l_fcw, l_fcb, (int)B, (int)T, (int)C, (int)(4 * C), st, l_fch, gelu_fusion_in_use(m));
            llmk_matmul_forward_residual(l_residual3, l_fch_gelu, l_fcprojw, l_fcprojb, l_residual2, (int)B, (int)T, (int)(4 * C), (int)C, st);
            llmk_layernorm_forward(n_ln, n_mean, n_rstd, l_residual3, n_w, n_b, (int)B, (int)T, (int)C, st);
        } else {
            llmk_matmul_forward(scratch, l_atty, l_attprojw, l_attprojb, (int)B, (int)T, (int)C, (int)C, st, nullptr, 1);
            llmk_fused_residual_forward5(l_residual2, l_ln2, l_ln2_mean, l_ln2_rstd, residual, scratch, l_ln2w, l_ln2b, (int)(B * T), (int)C, st);
            llmk_matmul_forward(l_fch_gelu, l_ln2, l_fcw, l_fcb, (int)B, (int)T, (int)C, (int)(4 * C), st, l_fch, gelu_fusion_in_use(m));
            llmk_matmul_forward(scratch, l_fch_gelu, l_fcprojw, l_fcprojb, (int)B, (int)T, (int)(4 * C), (int)C, st, nullptr, 1);
            llmk_fused_residual_forward5(l_residual3, n_ln, n_mean, n_rstd, l_residual2, scratch, n_w, n_b, (int)(B * T), (int)C, st);
        }
    }
    llmk_matmul_forward(a.output, a.lnf, p.wte, nullptr, (int)B, (int)T, (int)C, (int)Vp, st, nullptr, 1);
    if (wait) hipCheck(hipStreamSynchronize(st));
}
}  // namespace

void gpt2_forward(LLMK_GPT2* m, const int* inputs, size_t B, size_t T) { forward_impl(m, inputs, B, T, true); }

float gpt2_validate(LLMK_GPT2* m, const int* inputs, const int* targets, size_t B, size_t T) {
    assert(targets != nullptr);
    gpt2_forward(m, inputs, B, T);
    const int V = m->config.vocab_size, Vp = m->config.padded_vocab_size;
    hipStream_t st = m->stream;
    const float dloss = 1.0f / (float)(B * T);
    hipCheck(hipMemsetAsync(m->acts.losses, 0, B * T * sizeof(float), st));
    hipCheck(hipMemcpyAsync(m->targets, targets, B * T * sizeof(int), hipMemcpyHostToDevice, st));
    token_check(targets, B * T, V);
    // the reference passes its `False` constant, which is std::bool_constant<true> (llmc/cuda_common.h:46),
    // so its validate also overwrites the logits; here the flag means what it says
    llmk_fused_classifier(m->acts.output, m->acts.losses, dloss, m->targets, (int)B, (int)T, V, Vp, 0, st);
    hipCheck(hipMemcpyAsync(m->cpu_losses, m->acts.losses, B * T * sizeof(float), hipMemcpyDeviceToHost, st));
    hipCheck(hipStreamSynchronize(st));
    float mean_loss = 0.0f;
    for (size_t i = 0; i < B * T; i++) mean_loss += m->cpu_losses[i];
    return mean_loss / (float)(B * T);
}

// The generation loop of the reference's trainer (train_gpt2.cu:1751-1796), without the printing: every position of
// gen_tokens starts as eot_token, then positions 1..genT-1 are drawn one at a time from the model's distribution after
// the tokens before them. Each draw runs the forward pass on one sequence whose length is rounded up to a multiple of
// min(seq_len, 256) (no KV cache, as there), moves the logits of the last real position to the host and samples there
// with llmc/sampler.h's generator, whose state the caller owns (the reference starts it at 1337 for every generation).
void gpt2_generate(LLMK_GPT2* m, int* gen_tokens, int genT, int eot_token, unsigned long long* sample_rng_state) {
    const int B = m->batch_size, T = m->seq_len, V = m->config.vocab_size;
    const size_t Vp = m->config.padded_vocab_size;
    if (genT > T) { printf("gpt2_generate: genT=%d exceeds the sequence length %d\n", genT, T); exit(EXIT_FAILURE); }
    for (int i = 0; i < B * T; i++) gen_tokens[i] = eot_token;
    std::vector<char> raw((size_t)V * m->X);
    std::vector<float> cpu_logits(V);
    const int chunk = T < 256 ? T : 256;
    for (int t = 1; t < genT; t++) {
        gpt2_forward(m, gen_tokens, 1, (size_t)((t + chunk - 1) / chunk) * chunk);
        hipCheck(hipMemcpy(raw.data(), off(m->acts.output, (size_t)(t - 1) * Vp, m->X), (size_t)V * m->X, hipMemcpyDeviceToHost));
        from_storage(cpu_logits.data(), raw.data(), V, m->X);
        const float coin = llmk::random_f32(sample_rng_state);
        gen_tokens[t] = llmk::sample_softmax(cpu_logits.data(), V, coin);
    }
}

namespace {
// wait = false: everything is queued and nothing read back; the loss sum of the last micro-step stays in accumulated_mean_loss
void backward_impl(LLMK_GPT2* m, const int* inputs, const int* targets, int grad_accum_steps, int micro_step, bool wait) {
    if (m->grads_memory == nullptr) { fprintf(stderr, "Need to allocate gradients before backward"); exit(EXIT_FAILURE); }
    const bool last_step = micro_step == grad_accum_steps - 1;
    hipStream_t st = m->stream;
    const size_t B = m->batch_size, T = m->seq_len, V = m->config.vocab_size, Vp = m->config.padded_vocab_size,
                 L = m->config.num_layers, NH = m->config.num_heads, C = m->config.channels, X = m->X;
    if (micro_step == 0) {
        hipCheck(hipMemsetAsync(m->acts.losses, 0, B * T * sizeof(float), st));
        llmk_zero(m->grads_memory, m->num_parameters * X, st);
    }
    ParameterTensors p = m->params, g = m->grads;
    ActivationTensors a = m->acts;
    const int R = m->recompute;

    const float dloss = 1.0f / (float)(B * T * grad_accum_steps);
    // the clears run on the GPU while the host stages and checks the targets
    xptr dresidual = a.scratch_btc;
    llmk_zero(dresidual, B * T * C * X, st);
    hipCheck(hipMemcpyAsync(m->targets, targets, B * T * sizeof(int), hipMemcpyHostToDevice, st));
    token_check(targets, B * T, (int)V);
    llmk_fused_classifier(a.output, a.losses, dloss, m->targets, (int)B, (int)T, (int)V, (int)Vp, 1, st);
    float* scratchF = (float*)a.output;

    llmk_matmul_backward(a.scratch_bt4c, g.wte, nullptr, a.output, a.lnf, p.wte, nullptr, (int)B, (int)T, (int)C, (int)Vp, st, nullptr, 1);
    xptr residual = off(a.residual3, (L - 1) * B * T * C, X);
    llmk_layernorm_backward(dresidual, g.lnfw, g.lnfb, scratchF, a.scratch_bt4c, residual, p.lnfw, a.lnf_mean, a.lnf_rstd, (int)B, (int)T, (int)C, st);
    xptr dl_btc = residual;   // the last residual is dead from here on: generic (B,T,C) scratch

    for (int l = (int)L - 1; l >= 0; l--) {
        residual = l == 0 ? a.encoded : off(a.residual3, (size_t)(l - 1) * B * T * C, X);
        xptr l_ln1w = off(p.ln1w, l * C, X), l_ln1b = off(p.ln1b, l * C, X);
        xptr l_qkvw = off(p.qkvw, l * 3 * C * C, X), l_attprojw = off(p.attprojw, l * C * C, X);
        xptr l_ln2w = off(p.ln2w, l * C, X), l_ln2b = off(p.ln2b, l * C, X);
        xptr l_fcw = off(p.fcw, l * 4 * C * C, X), l_fcprojw = off(p.fcprojw, l * C * 4 * C, X);
        xptr dl_ln1w = off(g.ln1w, l * C, X), dl_ln1b = off(g.ln1b, l * C, X);
        xptr dl_qkvw = off(g.qkvw, l * 3 * C * C, X), dl_qkvb = off(g.qkvb, l * 3 * C, X);
        xptr dl_attprojw = off(g.attprojw, l * C * C, X), dl_attprojb = off(g.attprojb, l * C, X);
        xptr dl_ln2w = off(g.ln2w, l * C, X), dl_ln2b = off(g.ln2b, l * C, X);
        xptr dl_fcw = off(g.fcw, l * 4 * C * C, X), dl_fcb = off(g.fcb, l * 4 * C, X);
        xptr dl_fcprojw = off(g.fcprojw, l * C * 4 * C, X), dl_fcprojb = off(g.fcprojb, l * C, X);
        xptr l_ln1 = R < 2 ? off(a.ln1, l * B * T * C, X) : a.lnf;
        float *l_ln1_mean = a.ln1_mean + l * B * T, *l_ln1_rstd = a.ln1_rstd + l * B * T;
        xptr l_qkvr = off(a.qkvr, l * B * T * 3 * C, X);
        xptr l_atty = off(a.atty, l * B * T * C, X);
        xptr l_residual2 = off(a.residual2, l * B * T * C, X);
        xptr l_ln2 = R < 2 ? off(a.ln2, l * B * T * C, X) : a.lnf;
        float *l_ln2_mean = a.ln2_mean + l * B * T, *l_ln2_rstd = a.ln2_rstd + l * B * T;
        xptr l_fch_pre_gelu = off(a.fch, l * B * T * 4 * C, X);
        xptr l_fch_gelu = R < 1 ? off(a.fch_gelu, l * B * T * 4 * C, X) : a.fch_gelu;
        xptr dl_bt4c = a.scratch_bt4c;
        float* l_att = a.att + l * B * NH * T;

        if (R >= 1) llmk_gelu_forward(l_fch_gelu, l_fch_pre_gelu, (int)(B * T * 4 * C), st);
        // with gelu_fusion 2 the GELU backward is the epilogue of this GEMM's dinp; the bias gradient of the fc layer, whose
        // dout that produces, comes out of the fc weight-gradient GEMM below
        llmk_matmul_backward(dl_bt4c, dl_fcprojw, dl_fcprojb, dresidual, l_fch_gelu, l_fcprojw, scratchF, (int)B, (int)T, (int)(4 * C), (int)C, st, l_fch_pre_gelu, gelu_fusion_in_use(m));
        if (R >= 2) llmk_layernorm_forward(l_ln2, l_ln2_mean, l_ln2_rstd, l_residual2, l_ln2w, l_ln2b, (int)B, (int)T, (int)C, st);
        llmk_matmul_backward(dl_btc, dl_fcw, dl_fcb, dl_bt4c, l_ln2, l_fcw, scratchF, (int)B, (int)T, (int)C, (int)(4 * C), st, nullptr, 1);
        llmk_layernorm_backward(dresidual, dl_ln2w, dl_ln2b, scratchF, dl_btc, l_residual2, l_ln2w, l_ln2_mean, l_ln2_rstd, (int)B, (int)T, (int)C, st);
        llmk_matmul_backward(dl_btc, dl_attprojw, dl_attprojb, dresidual, l_atty, l_attprojw, scratchF, (int)B, (int)T, (int)C, (int)C, st, nullptr, 1);
        llmk_attention_backward(dl_bt4c, dl_btc, l_qkvr, l_atty, l_att, (int)B, (int)T, (int)NH, (int)C, st);
        if (R >= 2) llmk_layernorm_forward(l_ln1, l_ln1_mean, l_ln1_rstd, residual, l_ln1w, l_ln1b, (int)B, (int)T, (int)C, st);
        llmk_matmul_backward(dl_btc, dl_qkvw, dl_qkvb, dl_bt4c, l_ln1, l_qkvw, scratchF, (int)B, (int)T, (int)C, (int)(3 * C), st, nullptr, 1);
        llmk_layernorm_backward(dresidual, dl_ln1w, dl_ln1b, scratchF, dl_btc, residual, l_ln1w, l_ln1_mean, l_ln1_rstd, (int)B, (int)T, (int)C, st);
        // gradient exchange with other GPUs would be launched here (train_gpt2.cu:929-947); one GPU: nothing to do
    }
    llmk_encoder_backward(g.wte, g.wpe, a.output, m->workload_indices, m->bucket_info, dresidual, m->inputs, inputs,
                          (int)B, (int)T, (int)C, llmk::random_u32(&m->rng_state), st);
    if (last_step) llmk_global_sum_deterministic(m->accumulated_mean_loss, a.losses, (int)(B * T), st);
    if (!wait) return;
    if (last_step) hipCheck(hipMemcpyAsync(&m->mean_loss, m->accumulated_mean_loss, sizeof(float), hipMemcpyDeviceToHost, st));
    hipCheck(hipStreamSynchronize(st));
    if (last_step) m->mean_loss /= (float)(B * T * grad_accum_steps);
    else m->mean_loss = -1.0f;
}
}  // namespace

void gpt2_backward_and_reduce(LLMK_GPT2* m, const int* inputs, const int* targets, int grad_accum_steps, int micro_step) {
    backward_impl(m, inputs, targets, grad_accum_steps, micro_step, true);
}

namespace {
// the squared norm of all gradients, left in the first float of the logits buffer (free after the backward pass)
float* launch_grad_norm_squared(LLMK_GPT2* m) {
    hipStream_t st = m->stream;
    float* grad_norm_squared = (float*)m->acts.output;
    int num_slices[2] = {1, m->config.num_layers};
    int max_num_block_sums = llmk_get_max_num_block_sums(num_slices, 2);
    llmk_global_norm_squared(grad_norm_squared, m->grads_memory, m->num_parameters, 0, 1, max_num_block_sums, 1, st);
    llmk_global_sum_deterministic(grad_norm_squared, grad_norm_squared, max_num_block_sums, st);
    return grad_norm_squared;
}
}  // namespace

float gpt2_calculate_grad_norm(LLMK_GPT2* m) {
    hipStream_t st = m->stream;
    float* grad_norm_squared = launch_grad_norm_squared(m);
    float cpu = 0.0f;
    hipCheck(hipMemcpyAsync(&cpu, grad_norm_squared, sizeof(float), hipMemcpyDeviceToHost, st));
    hipCheck(hipStreamSynchronize(st));
    return sqrtf(cpu);
}

namespace {
// grad_norm_squared given: the clipping factor is formed on the device from it and grad_clip (grad_scale unused), and the
// call returns 0 without launching anything when the one-launch update does not take this model. wait = false: queued only.
int update_impl(LLMK_GPT2* m, float learning_rate, float beta1, float beta2, float eps, float weight_decay,
                float grad_scale, const float* grad_norm_squared, float grad_clip, int t, int init_from_master_only, bool wait) {
    if (m->grads_memory == nullptr || m->m_memory == nullptr || m->v_memory == nullptr) {
        fprintf(stderr, "Need to allocate optimizer state before update");
        exit(EXIT_FAILURE);
    }
    hipStream_t st = m->stream;
    const bool init_state = m->init_state;
    if (init_state) {
        m->init_state = false;
        hipCheck(hipMemsetAsync(m->m_memory, 0, m->num_parameters * sizeof(float), st));
        hipCheck(hipMemsetAsync(m->v_memory, 0, m->num_parameters * sizeof(float), st));
    }
    m->rng_state_last_update = m->rng_state;
    // every tensor in one launch where the library takes them so (same results as the per-tensor calls below, which the
    // reference makes: ten of the sixteen tensors are a few KB and cost a launch each); the seeds are drawn in the same order
    if (!init_from_master_only && !(init_state && m->master_weights != nullptr)) {
        size_t offsets[NUM_PARAMETER_TENSORS], sizes[NUM_PARAMETER_TENSORS];
        int slices[NUM_PARAMETER_TENSORS];
        float wds[NUM_PARAMETER_TENSORS];
        unsigned int seeds[NUM_PARAMETER_TENSORS];
        unsigned long long rng = m->rng_state;
        for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) {
            seeds[i] = llmk::random_u32(&rng);
            ShardInfo tensor = tensor_at_layer(m, 0, i);
            offsets[i] = tensor.offset; sizes[i] = tensor.size;
            slices[i] = (i < 2 || i > 13) ? 1 : m->config.num_layers;
            wds[i] = (i == 0 || i == 1 || i == 4 || i == 6 || i == 10 || i == 12) ? weight_decay : 0.0f;
        }
        const int launched = grad_norm_squared
            ? llmk_adamw_update_multi_clip(m->params_memory, m->master_weights, m->grads_memory, m->m_memory, m->v_memory,
                                           NUM_PARAMETER_TENSORS, offsets, sizes, slices, wds, seeds, learning_rate, beta1, beta2, t,
                                           eps, grad_norm_squared, grad_clip, st)
            : llmk_adamw_update_multi(m->params_memory, m->master_weights, m->grads_memory, m->m_memory, m->v_memory,
                                      NUM_PARAMETER_TENSORS, offsets, sizes, slices, wds, seeds, learning_rate, beta1, beta2, t,
                                      eps, grad_scale, st);
        if (launched) {
            m->rng_state = rng;
            if (wait) hipCheck(hipStreamSynchronize(st));
            return 1;
        }
    }
    if (grad_norm_squared) return 0;       // the per-tensor launches below take their factor from the host
    for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) {
        unsigned int seed = llmk::random_u32(&m->rng_state);
        int num_layers = (i < 2 || i > 13) ? 1 : m->config.num_layers;
        ShardInfo tensor = tensor_at_layer(m, 0, i);
        float wd = (i == 0 || i == 1 || i == 4 || i == 6 || i == 10 || i == 12) ? weight_decay : 0.0f;
        void* param_ptr = (char*)m->params_memory + tensor.offset * m->X;
        void* grad_ptr = (char*)m->grads_memory + tensor.offset * m->X;
        float* m_ptr = m->m_memory + tensor.offset;
        float* v_ptr = m->v_memory + tensor.offset;
        float* master_ptr = m->master_weights ? m->master_weights + tensor.offset : nullptr;
        if (init_state && m->master_weights != nullptr) {
            llmk_copy_and_cast_to_f32(master_ptr, param_ptr, tensor.size, (ptrdiff_t)tensor.size, (ptrdiff_t)tensor.size, num_layers, st);
        }
        if (init_from_master_only) {
            llmk_init_from_master(param_ptr, master_ptr, tensor.size, (ptrdiff_t)tensor.size, (ptrdiff_t)tensor.size, num_layers, seed, st);
        } else {
            llmk_adamw_update(param_ptr, master_ptr, grad_ptr, m_ptr, v_ptr, tensor.size, (ptrdiff_t)tensor.size,
                              (ptrdiff_t)tensor.size, (ptrdiff_t)tensor.size, num_layers, learning_rate, beta1, beta2, t,
                              eps, wd, grad_scale, seed, st);
        }
    }
    if (wait) hipCheck(hipStreamSynchronize(st));
    return 1;
}
}  // namespace

void gpt2_update(LLMK_GPT2* m, float learning_rate, float beta1, float beta2, float eps, float weight_decay,
                 float grad_scale, int t, int init_from_master_only) {
    update_impl(m, learning_rate, beta1, beta2, eps, weight_decay, grad_scale, nullptr, 0.f, t, init_from_master_only, true);
}

// One optimizer step (one micro-batch) with a single wait at its end: forward, backward, gradient norm, clipping and
// update are queued back to back, the clipping factor is formed on the device, and the loss and the norm come back
// together after the update has been queued. The same kernels on the same data as gpt2_forward +
// gpt2_backward_and_reduce(.., 1, 0) + gpt2_calculate_grad_norm + gpt2_update with the factor of train_gpt2.cu:1850, so the
// same bits; what is gone are the four places where the GPU waits for the host (the reference's loop has them:
// train_gpt2.cu:785, :975, :1021, :1148). No counterpart in the reference.
void gpt2_train_step(LLMK_GPT2* m, const int* inputs, const int* targets, float learning_rate, float beta1, float beta2,
                     float eps, float weight_decay, float grad_clip, int t, float* mean_loss, float* grad_norm) {
    const size_t B = m->batch_size, T = m->seq_len;
    hipStream_t st = m->stream;
    forward_impl(m, inputs, B, T, false);
    backward_impl(m, inputs, targets, 1, 0, false);
    // the first-step work of gpt2_update that has to precede the norm's use of the logits buffer: none; the moments are
    // cleared and the master copy taken inside update_impl, after the norm
    const bool first = m->init_state;
    float* norm2 = launch_grad_norm_squared(m);
    float gn = -1.0f;
    bool fused = false;
    if (!(first && m->master_weights != nullptr))
        fused = update_impl(m, learning_rate, beta1, beta2, eps, weight_decay, 1.0f, norm2, grad_clip, t, 0, false) != 0;
    if (!fused) {                                // first step with a master copy to take, or a model the one-launch update does not take
        float cpu = 0.0f;
        hipCheck(hipMemcpyAsync(&cpu, norm2, sizeof(float), hipMemcpyDeviceToHost, st));
        hipCheck(hipStreamSynchronize(st));
        gn = sqrtf(cpu);
        const float scale = (gn > grad_clip) ? grad_clip / gn : 1.0f;
        update_impl(m, learning_rate, beta1, beta2, eps, weight_decay, scale, nullptr, 0.f, t, 0, false);
    }
    float* back = m->cpu_losses;                 // pinned
    hipCheck(hipMemcpyAsync(&back[0], m->accumulated_mean_loss, sizeof(float), hipMemcpyDeviceToHost, st));
    if (fused) hipCheck(hipMemcpyAsync(&back[1], norm2, sizeof(float), hipMemcpyDeviceToHost, st));
    hipCheck(hipStreamSynchronize(st));
    m->mean_loss = back[0] / (float)(B * T);
    if (fused) gn = sqrtf(back[1]);
    if (mean_loss) *mean_loss = m->mean_loss;
    if (grad_norm) *grad_norm = gn;
}

float gpt2_estimate_mfu(LLMK_GPT2* m, int num_tokens, float dt) {
    size_t N = m->num_parameters;
    size_t L = m->config.num_layers, C = m->config.channels, T = m->seq_len;
    size_t flops_per_token = 6 * N + 6 * L * C * T;
    double flops_per_step = (double)flops_per_token * num_tokens;
    double achieved = flops_per_step / dt;
    double promised = (m->X == 2 ? MI355X_PEAK_BF16_TFLOPS : MI355X_PEAK_FP32_TFLOPS) * 1e12;
    return (float)(achieved / promised);
}

void gpt2_free(LLMK_GPT2* m) {
    if (!m) return;
    (void)hipDeviceSynchronize();
    void* dev[] = {m->params_memory, m->grads_memory, m->m_memory, m->v_memory, m->master_weights, m->acts_memory,
                   m->inputs, m->targets, m->accumulated_mean_loss};
    for (void* p : dev) if (p) (void)hipFree(p);
    if (m->cpu_losses) (void)hipHostFree(m->cpu_losses);
    if (m->workload_indices) (void)hipHostFree(m->workload_indices);
    if (m->bucket_info) (void)hipHostFree(m->bucket_info);
    if (m->stream) (void)hipStreamDestroy(m->stream);
    delete m;
}

void gpt2_save_state(LLMK_GPT2* m, const char* filename, int step) { gpt2_save_state_with_loader(filename, step, m, nullptr); }
void gpt2_load_state(LLMK_GPT2* m, const char* filename, int* step) { gpt2_load_state_with_loader(step, m, nullptr, filename); }

// save_state, train_gpt2.cu:1209: header, AdamW moments (+ master weights), and for a shuffling loader its
// permutations and generator. Without a loader the loader fields of the header stay zero.
void gpt2_save_state_with_loader(const char* filename, int step, LLMK_GPT2* m, LLMK_DataLoader* loader) {
    FILE* f = fopen(filename, "wb");
    if (!f) { fprintf(stderr, "Error: Failed to open file '%s'\n", filename); exit(EXIT_FAILURE); }
    int hdr[256];
    memset(hdr, 0, sizeof hdr);
    hdr[0] = 20240527; hdr[1] = 1; hdr[2] = 1; hdr[3] = 0; hdr[4] = m->use_master_weights;
    hdr[5] = loader ? dataloader_should_shuffle(loader) : 0;
    hdr[10] = step;
    memcpy(&hdr[20], &m->rng_state, 8);
    memcpy(&hdr[22], &m->rng_state_last_update, 8);
    if (loader) {
        const size_t shard = dataloader_current_shard_idx(loader), sample = dataloader_current_sample_idx(loader);
        memcpy(&hdr[30], &shard, sizeof(size_t));
        memcpy(&hdr[32], &sample, sizeof(size_t));
    }
    fwrite(hdr, sizeof(int), 256, f);
    device_to_file(f, m->m_memory, m->num_parameters * sizeof(float), m->stream);
    device_to_file(f, m->v_memory, m->num_parameters * sizeof(float), m->stream);
    if (m->use_master_weights) device_to_file(f, m->master_weights, m->num_parameters * sizeof(float), m->stream);
    if (loader && dataloader_should_shuffle(loader)) {
        std::vector<char> st(dataloader_get_shuffle_state(loader, nullptr));
        dataloader_get_shuffle_state(loader, st.data());
        fwrite(st.data(), 1, st.size(), f);
    }
    fclose(f);
}

// load_state, train_gpt2.cu:1250. The loader (already initialised on the same files) is put back where it was.
void gpt2_load_state_with_loader(int* step, LLMK_GPT2* m, LLMK_DataLoader* loader, const char* filename) {
    FILE* f = fopen(filename, "rb");
    if (!f) { fprintf(stderr, "Error: Failed to open file '%s'\n", filename); exit(EXIT_FAILURE); }
    int hdr[256];
    if (fread(hdr, sizeof(int), 256, f) != 256) { fprintf(stderr, "Error: short state header\n"); exit(EXIT_FAILURE); }
    if (hdr[0] != 20240527 || hdr[1] != 1) { fprintf(stderr, "Bad magic/version in state file\n"); exit(EXIT_FAILURE); }
    if (hdr[2] != 1 || hdr[3] != 0) { fprintf(stderr, "State file written by a multi-process run\n"); exit(EXIT_FAILURE); }
    int use_master = hdr[4];
    if (step) *step = hdr[10];
    unsigned long long final_rng;
    memcpy(&final_rng, &hdr[20], 8);
    memcpy(&m->rng_state_last_update, &hdr[22], 8);
    if (use_master == 0 && m->use_master_weights) {
        fprintf(stderr, "Error: Master weights requested, but not present in state file.");
        exit(EXIT_FAILURE);
    }
    m->init_state = false;
    assert(m->m_memory != nullptr && m->v_memory != nullptr);
    file_to_device(m->m_memory, f, m->num_parameters * sizeof(float), m->stream);
    file_to_device(m->v_memory, f, m->num_parameters * sizeof(float), m->stream);
    if (m->use_master_weights) {
        file_to_device(m->master_weights, f, m->num_parameters * sizeof(float), m->stream);
        // re-derive the low-precision weights from the master copy with the RNG state of the last update
        m->rng_state = m->rng_state_last_update;
        gpt2_update(m, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0, 1);
    } else if (use_master == 1) {
        // the file carries a master copy this run does not keep (train_gpt2.cu:1268-1270 warns and goes on): step over it,
        // so that what follows is read as what it is
        fprintf(stderr, "Warning: Master weights are present in state, but not enabled for current run.");
        fseek(f, (long)(m->num_parameters * sizeof(float)), SEEK_CUR);
    }
    m->rng_state = final_rng;
    if (loader) {
        if (hdr[5] != 1) dataloader_set_shuffle_state(loader, nullptr, 0);     // the loader takes the file's flag (train_gpt2.cu:1289)
        if (hdr[5] == 1) {
            const long at = ftell(f);
            fseek(f, 0, SEEK_END);
            std::vector<char> st((size_t)(ftell(f) - at));
            fseek(f, at, SEEK_SET);
            if (fread(st.data(), 1, st.size(), f) != st.size()) { fprintf(stderr, "Error: short read of the loader state\n"); exit(EXIT_FAILURE); }
            dataloader_set_shuffle_state(loader, st.data(), st.size());
        }
        size_t shard, sample;
        memcpy(&shard, &hdr[30], sizeof(size_t));
        memcpy(&sample, &hdr[32], sizeof(size_t));
        dataloader_resume(loader, shard, sample);
    }
    fclose(f);
}

float gpt2_mean_loss(const LLMK_GPT2* m) { return m->mean_loss; }
size_t gpt2_num_parameters(const LLMK_GPT2* m) { return m->num_parameters; }
void gpt2_get_config(const LLMK_GPT2* m, int* o) {
    o[0] = m->config.max_seq_len; o[1] = m->config.vocab_size; o[2] = m->config.padded_vocab_size;
    o[3] = m->config.num_layers; o[4] = m->config.num_heads; o[5] = m->config.channels;
}
void gpt2_param_sizes(const LLMK_GPT2* m, size_t* o) { for (int i = 0; i < NUM_PARAMETER_TENSORS; i++) o[i] = m->param_elements[i]; }
const float* gpt2_cpu_losses(const LLMK_GPT2* m) { return m->cpu_losses; }
void* gpt2_params_memory(LLMK_GPT2* m) { return m->params_memory; }
void* gpt2_grads_memory(LLMK_GPT2* m) { return m->grads_memory; }
void* gpt2_output_memory(LLMK_GPT2* m) { return m->acts.output; }

static void arena_to_f32(LLMK_GPT2* m, const void* dev, float* out, size_t n) {
    std::vector<char> tmp(n * m->X);
    hipCheck(hipMemcpy(tmp.data(), dev, n * m->X, hipMemcpyDeviceToHost));
    from_storage(out, tmp.data(), n, m->X);
}
void gpt2_get_params_f32(LLMK_GPT2* m, float* out) { arena_to_f32(m, m->params_memory, out, m->num_parameters); }
void gpt2_get_grads_f32(LLMK_GPT2* m, float* out) { arena_to_f32(m, m->grads_memory, out, m->num_parameters); }
void gpt2_set_params_f32(LLMK_GPT2* m, const float* in) {
    std::vector<char> tmp(m->num_parameters_bytes);
    to_storage(tmp.data(), in, m->num_parameters, m->X);
    hipCheck(hipMemcpy(m->params_memory, tmp.data(), m->num_parameters_bytes, hipMemcpyHostToDevice));
}
void gpt2_get_logits_f32(LLMK_GPT2* m, float* out, size_t B, size_t T) {
    arena_to_f32(m, m->acts.output, out, B * T * (size_t)m->config.padded_vocab_size);
}
unsigned long long gpt2_get_rng_state(const LLMK_GPT2* m) { return m->rng_state; }
void gpt2_set_rng_state(LLMK_GPT2* m, unsigned long long s) { m->rng_state = s; }
size_t gpt2_activation_bytes(const LLMK_GPT2* m) { return m->acts_bytes; }

}  // extern "C"
