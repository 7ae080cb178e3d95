/*
 * cpu_ref.c — CPU restatement of llm.c's fp32 GPT-2 training step.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the shipped library links, loads or calls this file.
 * It exists so that the HIP kernels can be checked against plain fp32 loops on a machine that
 * does not have the reference sources, and so that a CPU figure can be printed next to the
 * GPU one. Only tests/, the smoke check and the benchmark's CPU-baseline leg load it.
 *
 * Every function states which part of the reference it follows (paths relative to the
 * reference checkout). The arithmetic is the same; the loop nests and memory handling are
 * this file's own (activations of one layer at a time in backward, O(T^2*hs) attention
 * backward instead of the cubic softmax-Jacobian loop).
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   mt19937 / normal_        known-answer vectors printed in llmc/rand.h:48-80
 *   per-op forward/backward   the compiled reference (oracle/_ref) on random inputs, plus
 *                             closed forms (constant rows, T=1 attention, uniform logits,
 *                             AdamW first step) and central finite differences
 *   whole model               the compiled reference on a tiny GPT-2 (golden fixture committed)
 *   mixed-precision AdamW,    device code only in the reference (llmc/adamw.cuh, llmc/cuda_utils.cuh:238-278), so
 *   stochastic rounding       pinned by what fixes them without the reference running
 *                             (tests/test_oracle_optimizer_pins.py): SquirrelNoise5 by known answers worked through
 *                             by hand from the published constants, its inverse, injectivity and avalanche; the
 *                             noise word of an element by a walk over the reference's launch grid; the update by
 *                             bit-equality of its fp32 state with the fp32 update (itself held to train_gpt2.c's
 *                             AdamW over several steps) and of its bf16 parameter with the stochastic rounding of
 *                             that state; the rounding by its exact up-probability low16/65536.
 *   bf16 rounding,            cref_f32_to_bf16[_array]: an independent library cast on a million bit patterns, every
 *   sum of squares            exact tie of eight exponents in both parities, infinities, denormals, NaNs;
 *                             cref_sum_squares: numpy's float64 sum on inputs where a float accumulator differs in
 *                             the 6th digit, and the closed form of 1^2 + ... + n^2 (same test file).
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define CREF_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------
 * bf16 helpers (round-to-nearest-even, as __float2bfloat16_rn does)
 * ---------------------------------------------------------------------------------------- */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

CREF_API uint16_t cref_f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u); /* NaN stays NaN */
    uint32_t bias = 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)((u + bias) >> 16);
}
CREF_API float cref_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

CREF_API void cref_f32_to_bf16_array(uint16_t* dst, const float* src, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = cref_f32_to_bf16(src[i]);
}
CREF_API void cref_bf16_to_f32_array(float* dst, const uint16_t* src, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = cref_bf16_to_f32(src[i]);
}

/* ------------------------------------------------------------------------------------------
 * mt19937 + torch-compatible normal_  (follows llmc/rand.h:106-221)
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    uint32_t s[624];
    int left;
    int next;
} cref_mt;

CREF_API void cref_mt_seed(cref_mt* g, uint32_t seed) {
    g->s[0] = seed;
    for (uint32_t j = 1; j < 624; j++) g->s[j] = 1812433253u * (g->s[j - 1] ^ (g->s[j - 1] >> 30)) + j;
    g->left = 1;
    g->next = 0;
}
static void mt_refill(cref_mt* g) {
    static const uint32_t mag[2] = {0u, 0x9908b0dfu};
    uint32_t* s = g->s;
    for (int j = 0; j < 624; j++) {
        uint32_t y = (s[j] & 0x80000000u) | (s[(j + 1) % 624] & 0x7fffffffu);
        s[j] = s[(j + 397) % 624] ^ (y >> 1) ^ mag[y & 1u];
    }
    g->left = 624;
    g->next = 0;
}
CREF_API uint32_t cref_mt_u32(cref_mt* g) {
    if (--g->left <= 0) mt_refill(g);
    uint32_t y = g->s[g->next++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}
static inline uint64_t mt_u64(cref_mt* g) { uint64_t hi = cref_mt_u32(g); return (hi << 32) | cref_mt_u32(g); }
static inline float mt_f32(cref_mt* g) { return (float)(cref_mt_u32(g) & 0xffffffu) * (1.0f / 16777216.0f); }
static inline double mt_f64(cref_mt* g) { return (double)(mt_u64(g) & ((1ull << 53) - 1)) * (1.0 / 9007199254740992.0); }

/* Box-Muller on a block of 16 uniforms: first 8 are radii, last 8 are angles */
static void box_muller16(float* d, float mean, float std) {
    for (int t = 0; t < 8; t++) {
        float u1 = 1.0f - d[t], u2 = d[t + 8];
        float r = sqrtf(-2.0f * logf(u1 + 1e-12f));
        float th = (float)(2.0 * M_PI * u2);
        d[t] = r * cosf(th) * std + mean;
        d[t + 8] = r * sinf(th) * std + mean;
    }
}
CREF_API void cref_normal(float* d, uint32_t n, float mean, float std, cref_mt* g) {
    if (n >= 16) {
        for (uint32_t t = 0; t < n; t++) d[t] = mt_f32(g);
        for (uint32_t i = 0; i + 16 <= n; i += 16) box_muller16(d + i, mean, std);
        if (n % 16) { /* the tail block is redrawn, overlapping the previous one */
            float* tail = d + n - 16;
            for (int i = 0; i < 16; i++) tail[i] = mt_f32(g);
            box_muller16(tail, mean, std);
        }
        return;
    }
    int have = 0;
    double spare = 0.0;
    for (uint32_t t = 0; t < n; t++) {
        if (have) { d[t] = (float)(spare * std + mean); have = 0; continue; }
        float u1 = (float)mt_f64(g), u2 = (float)mt_f64(g);
        float r = sqrtf(-2.0f * logf(1.0f - u2 + 1e-12f));
        float th = (float)(2.0 * M_PI * u1);
        spare = r * sinf(th);
        have = 1;
        d[t] = r * cosf(th) * std + mean;
    }
}
/* convenience for ctypes callers: seed, skip `skip_u32` raw draws, then fill */
CREF_API void cref_mt_kat(uint32_t seed, uint32_t* ints5, float* n8, uint32_t* mid, float* n16, uint32_t* last) {
    cref_mt g; cref_mt_seed(&g, seed);
    for (int i = 0; i < 5; i++) ints5[i] = cref_mt_u32(&g);
    cref_normal(n8, 8, 0.f, 1.f, &g);
    *mid = cref_mt_u32(&g);
    cref_normal(n16, 16, 0.f, 1.f, &g);
    *last = cref_mt_u32(&g);
}

/* ------------------------------------------------------------------------------------------
 * Model shape helpers (follows train_gpt2.c:556-577 / train_gpt2.cu:118-139)
 * ---------------------------------------------------------------------------------------- */
typedef struct { int max_seq_len, vocab_size, padded_vocab_size, num_layers, num_heads, channels; } cref_config;
enum { CREF_NPARAM = 16 };

CREF_API size_t cref_param_sizes(size_t* sz, const cref_config* c) {
    size_t Vp = c->padded_vocab_size, C = c->channels, mT = c->max_seq_len, L = c->num_layers;
    size_t v[CREF_NPARAM] = {Vp * C, mT * C, L * C, L * C, L * 3 * C * C, L * 3 * C, L * C * C, L * C,
                             L * C, L * C, L * 4 * C * C, L * 4 * C, L * 4 * C * C, L * C, C, C};
    size_t tot = 0;
    for (int i = 0; i < CREF_NPARAM; i++) { sz[i] = v[i]; tot += v[i]; }
    return tot;
}

/* Random init in the order PyTorch constructs the modules (follows train_gpt2.cu:587-637):
 * layer loop outermost; wte (V rows only) and wpe drawn during layer 0 before that layer's
 * matrices; c_proj matrices scaled by 1/sqrt(2L); LN weights 1; everything else 0. */
CREF_API void cref_init_params(float* p, const cref_config* c, uint32_t seed) {
    size_t sz[CREF_NPARAM];
    size_t tot = cref_param_sizes(sz, c);
    memset(p, 0, tot * sizeof(float));
    size_t off[CREF_NPARAM];
    size_t o = 0;
    for (int i = 0; i < CREF_NPARAM; i++) { off[i] = o; o += sz[i]; }
    const int ln_w[3] = {2, 8, 14};
    for (int k = 0; k < 3; k++)
        for (size_t j = 0; j < sz[ln_w[k]]; j++) p[off[ln_w[k]] + j] = 1.0f;
    cref_mt g; cref_mt_seed(&g, seed);
    int L = c->num_layers;
    float rs = 1.0f / sqrtf(2.0f * (float)L);
    const int mats[4] = {4, 6, 10, 12};
    for (int l = 0; l < L; l++) {
        if (l == 0) {
            cref_normal(p + off[0], (uint32_t)((size_t)c->vocab_size * c->channels), 0.f, 0.02f, &g);
            cref_normal(p + off[1], (uint32_t)sz[1], 0.f, 0.02f, &g);
        }
        for (int k = 0; k < 4; k++) {
            int i = mats[k];
            size_t n = sz[i] / L;
            float std = (i == 6 || i == 12) ? 0.02f * rs : 0.02f;
            cref_normal(p + off[i] + (size_t)l * n, (uint32_t)n, 0.f, std, &g);
        }
    }
}

/* Checkpoint writer: 256-int header + flat fp32 params, version 3
 * (layout read by train_gpt2.c:707-750, written by train_gpt2.cu:430-452). */
CREF_API int cref_write_checkpoint_fp32(const char* path, const float* p, const cref_config* c) {
    size_t sz[CREF_NPARAM];
    size_t tot = cref_param_sizes(sz, c);
    int hdr[256];
    memset(hdr, 0, sizeof hdr);
    hdr[0] = 20240326; hdr[1] = 3; hdr[2] = c->max_seq_len; hdr[3] = c->vocab_size;
    hdr[4] = c->num_layers; hdr[5] = c->num_heads; hdr[6] = c->channels; hdr[7] = c->padded_vocab_size;
    FILE* f = fopen(path, "wb");
    if (!f) return -1;
    int ok = fwrite(hdr, sizeof(int), 256, f) == 256 && fwrite(p, sizeof(float), tot, f) == tot;
    fclose(f);
    return ok ? 0 : -2;
}

/* ------------------------------------------------------------------------------------------
 * Per-op forward / backward
 * ---------------------------------------------------------------------------------------- */

/* train_gpt2.c:35-58 */
CREF_API void cref_encoder_forward(float* out, const int* inp, const float* wte, const float* wpe, int B, int T, int C) {
    for (int bt = 0; bt < B * T; bt++) {
        const float* e = wte + (size_t)inp[bt] * C;
        const float* p = wpe + (size_t)(bt % T) * C;
        float* o = out + (size_t)bt * C;
        for (int c = 0; c < C; c++) o[c] = e[c] + p[c];
    }
}
/* train_gpt2.c:60-76 (accumulates) */
CREF_API void cref_encoder_backward(float* dwte, float* dwpe, const float* dout, const int* inp, int B, int T, int C) {
    for (int bt = 0; bt < B * T; bt++) {
        float* de = dwte + (size_t)inp[bt] * C;
        float* dp = dwpe + (size_t)(bt % T) * C;
        const float* d = dout + (size_t)bt * C;
        for (int c = 0; c < C; c++) { de[c] += d[c]; dp[c] += d[c]; }
    }
}

/* train_gpt2.c:78-118: two-pass mean / biased variance, eps 1e-5. mean/rstd may be NULL. */
CREF_API void cref_layernorm_forward(float* out, float* mean, float* rstd, const float* inp, const float* w,
                                     const float* b, int N, int C) {
    for (int r = 0; r < N; r++) {
        const float* x = inp + (size_t)r * C;
        float m = 0.f;
        for (int c = 0; c < C; c++) m += x[c];
        m /= C;
        float v = 0.f;
        for (int c = 0; c < C; c++) { float d = x[c] - m; v += d * d; }
        v /= C;
        float s = 1.0f / sqrtf(v + 1e-5f);
        float* o = out + (size_t)r * C;
        for (int c = 0; c < C; c++) o[c] = s * (x[c] - m) * w[c] + b[c];
        if (mean) mean[r] = m;
        if (rstd) rstd[r] = s;
    }
}
/* train_gpt2.c:120-161: dinp, dweight, dbias all accumulate */
CREF_API void cref_layernorm_backward(float* dinp, float* dw, float* db, const float* dout, const float* inp,
                                      const float* w, const float* mean, const float* rstd, int N, int C) {
    for (int r = 0; r < N; r++) {
        const float* g = dout + (size_t)r * C;
        const float* x = inp + (size_t)r * C;
        float* dx = dinp + (size_t)r * C;
        float m = mean[r], s = rstd[r];
        float a = 0.f, bsum = 0.f;
        for (int c = 0; c < C; c++) {
            float nh = (x[c] - m) * s, dn = w[c] * g[c];
            a += dn;
            bsum += dn * nh;
        }
        a /= C;
        bsum /= C;
        for (int c = 0; c < C; c++) {
            float nh = (x[c] - m) * s, dn = w[c] * g[c];
            db[c] += g[c];
            dw[c] += nh * g[c];
            dx[c] += (dn - a - nh * bsum) * s;
        }
    }
}

/* train_gpt2.c:163-229: out[r][o] = bias[o] + sum_i inp[r][i] * weight[o][i] */
CREF_API void cref_matmul_forward(float* out, const float* inp, const float* w, const float* bias, int N, int C, int OC) {
    #pragma omp parallel for schedule(static)
    for (int r0 = 0; r0 < N; r0 += 4) {
        int rn = N - r0 < 4 ? N - r0 : 4;
        for (int o = 0; o < OC; o++) {
            const float* wr = w + (size_t)o * C;
            float acc[4];
            for (int k = 0; k < 4; k++) acc[k] = bias ? bias[o] : 0.f;
            for (int k = 0; k < rn; k++) {
                const float* x = inp + (size_t)(r0 + k) * C;
                float s = 0.f;
                #pragma omp simd reduction(+:s)
                for (int i = 0; i < C; i++) s += x[i] * wr[i];
                acc[k] += s;
            }
            for (int k = 0; k < rn; k++) out[(size_t)(r0 + k) * OC + o] = acc[k];
        }
    }
}
/* train_gpt2.c:231-269: all three outputs accumulate; dbias / dinp may be NULL */
CREF_API void cref_matmul_backward(float* dinp, float* dw, float* dbias, const float* dout, const float* inp,
                                   const float* w, int N, int C, int OC) {
    if (dinp) {
        #pragma omp parallel for schedule(static)
        for (int r = 0; r < N; r++) {
            float* dx = dinp + (size_t)r * C;
            const float* g = dout + (size_t)r * OC;
            for (int o = 0; o < OC; o++) {
                const float* wr = w + (size_t)o * C;
                float d = g[o];
                for (int i = 0; i < C; i++) dx[i] += wr[i] * d;
            }
        }
    }
    #pragma omp parallel for schedule(static)
    for (int o = 0; o < OC; o++) {
        float* dwr = dw + (size_t)o * C;
        float bs = 0.f;
        for (int r = 0; r < N; r++) {
            float d = dout[(size_t)r * OC + o];
            const float* x = inp + (size_t)r * C;
            bs += d;
            for (int i = 0; i < C; i++) dwr[i] += x[i] * d;
        }
        if (dbias) dbias[o] += bs;
    }
}

/* train_gpt2.c:271-345. qkv is (B,T,3C) = (B,T,3,NH,hs). att is (B,NH,T,T) of probabilities with
 * zeros above the diagonal; may be NULL when the caller does not need it. lse (B,NH,T), optional,
 * receives max + log(sum exp) of the scaled scores — the row statistic a flash kernel stores. */
CREF_API void cref_attention_forward(float* out, float* att, float* lse, const float* qkv, int B, int T, int C, int NH) {
    int hs = C / NH, C3 = 3 * C;
    float scale = 1.0f / sqrtf((float)hs);
    #pragma omp parallel
    {
        float* p = (float*)malloc(sizeof(float) * T);
        #pragma omp for collapse(2) schedule(static)
        for (int b = 0; b < B; b++)
            for (int h = 0; h < NH; h++)
                for (int t = 0; t < T; t++) {
                    const float* q = qkv + ((size_t)b * T + t) * C3 + h * hs;
                    float mx = -10000.0f; /* train_gpt2.c:294 */
                    for (int t2 = 0; t2 <= t; t2++) {
                        const float* k = qkv + ((size_t)b * T + t2) * C3 + C + h * hs;
                        float s = 0.f;
                        #pragma omp simd reduction(+:s)
                        for (int i = 0; i < hs; i++) s += q[i] * k[i];
                        s *= scale;
                        p[t2] = s;
                        if (s > mx) mx = s;
                    }
                    float sum = 0.f;
                    for (int t2 = 0; t2 <= t; t2++) { p[t2] = expf(p[t2] - mx); sum += p[t2]; }
                    float inv = sum == 0.f ? 0.f : 1.0f / sum;
                    float* o = out + ((size_t)b * T + t) * C + h * hs;
                    for (int i = 0; i < hs; i++) o[i] = 0.f;
                    for (int t2 = 0; t2 <= t; t2++) {
                        float a = p[t2] * inv;
                        p[t2] = a;
                        const float* v = qkv + ((size_t)b * T + t2) * C3 + 2 * C + h * hs;
                        for (int i = 0; i < hs; i++) o[i] += a * v[i];
                    }
                    if (att) {
                        float* arow = att + (((size_t)b * NH + h) * T + t) * T;
                        for (int t2 = 0; t2 < T; t2++) arow[t2] = t2 <= t ? p[t2] : 0.f;
                    }
                    if (lse) lse[((size_t)b * NH + h) * T + t] = mx + logf(sum);
                }
        free(p);
    }
}

/* train_gpt2.c:347-405, with the softmax Jacobian product (the t2,t3 double loop at :382-388)
 * collapsed to dpre[j] = att[j] * (datt[j] - sum_k att[k] datt[k]). dqkv accumulates.
 * att == NULL: probabilities are recomputed from qkv. */
CREF_API void cref_attention_backward(float* dqkv, const float* dout, const float* qkv, const float* att, int B,
                                      int T, int C, int NH) {
    int hs = C / NH, C3 = 3 * C;
    float scale = 1.0f / sqrtf((float)hs);
    #pragma omp parallel
    {
        float* p = (float*)malloc(sizeof(float) * T);
        float* da = (float*)malloc(sizeof(float) * T);
        #pragma omp for collapse(2) schedule(static)
        for (int b = 0; b < B; b++)
            for (int h = 0; h < NH; h++)
                for (int t = 0; t < T; t++) {
                    const float* q = qkv + ((size_t)b * T + t) * C3 + h * hs;
                    float* dq = dqkv + ((size_t)b * T + t) * C3 + h * hs;
                    const float* go = dout + ((size_t)b * T + t) * C + h * hs;
                    if (att) {
                        const float* arow = att + (((size_t)b * NH + h) * T + t) * T;
                        for (int t2 = 0; t2 <= t; t2++) p[t2] = arow[t2];
                    } else {
                        float mx = -10000.0f, sum = 0.f;
                        for (int t2 = 0; t2 <= t; t2++) {
                            const float* k = qkv + ((size_t)b * T + t2) * C3 + C + h * hs;
                            float s = 0.f;
                            for (int i = 0; i < hs; i++) s += q[i] * k[i];
                            p[t2] = s * scale;
                            if (p[t2] > mx) mx = p[t2];
                        }
                        for (int t2 = 0; t2 <= t; t2++) { p[t2] = expf(p[t2] - mx); sum += p[t2]; }
                        for (int t2 = 0; t2 <= t; t2++) p[t2] /= sum;
                    }
                    float dot = 0.f;
                    for (int t2 = 0; t2 <= t; t2++) {
                        const float* v = qkv + ((size_t)b * T + t2) * C3 + 2 * C + h * hs;
                        float* dv = dqkv + ((size_t)b * T + t2) * C3 + 2 * C + h * hs;
                        float d = 0.f;
                        for (int i = 0; i < hs; i++) { d += v[i] * go[i]; dv[i] += p[t2] * go[i]; }
                        da[t2] = d;
                        dot += p[t2] * d;
                    }
                    for (int t2 = 0; t2 <= t; t2++) {
                        float dpre = p[t2] * (da[t2] - dot) * scale;
                        const float* k = qkv + ((size_t)b * T + t2) * C3 + C + h * hs;
                        float* dk = dqkv + ((size_t)b * T + t2) * C3 + C + h * hs;
                        for (int i = 0; i < hs; i++) { dq[i] += k[i] * dpre; dk[i] += q[i] * dpre; }
                    }
                }
        free(p);
        free(da);
    }
}

/* train_gpt2.c:407-415 */
CREF_API void cref_gelu_forward(float* out, const float* inp, size_t n) {
    const float k = sqrtf(2.0f / (float)M_PI);
    for (size_t i = 0; i < n; i++) {
        float x = inp[i];
        out[i] = 0.5f * x * (1.0f + tanhf(k * (x + 0.044715f * x * x * x)));
    }
}
/* train_gpt2.c:422-433 (accumulates into dinp). Kept out of fast-math like the reference does. */
__attribute__((optimize("no-fast-math")))
CREF_API void cref_gelu_backward(float* dinp, const float* inp, const float* dout, size_t n) {
    const float k = sqrtf(2.0f / (float)M_PI);
    for (size_t i = 0; i < n; i++) {
        float x = inp[i];
        float u = k * (x + 0.044715f * x * x * x);
        float th = tanhf(u);
        float ch = coshf(u);
        float sech2 = 1.0f / (ch * ch);
        float g = 0.5f * (1.0f + th) + x * 0.5f * sech2 * k * (1.0f + 3.0f * 0.044715f * x * x);
        dinp[i] += g * dout[i];
    }
}

/* train_gpt2.c:436-447 */
CREF_API void cref_residual_forward(float* out, const float* a, const float* b, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = a[i] + b[i];
}

/* train_gpt2.c:449-500: softmax over the first V of Vp columns, padded probs 0, then
 * losses[r] = -log(probs[r][target]). losses may be NULL (no targets). */
CREF_API void cref_softmax_crossentropy_forward(float* probs, float* losses, const float* logits, const int* targets,
                                                int N, int V, int Vp) {
    #pragma omp parallel for schedule(static)
    for (int r = 0; r < N; r++) {
        const float* z = logits + (size_t)r * Vp;
        float* p = probs + (size_t)r * Vp;
        float mx = -10000.0f;
        for (int i = 0; i < V; i++) if (z[i] > mx) mx = z[i];
        float sum = 0.f;
        for (int i = 0; i < V; i++) { p[i] = expf(z[i] - mx); sum += p[i]; }
        for (int i = 0; i < V; i++) p[i] /= sum;
        for (int i = V; i < Vp; i++) p[i] = 0.f;
        if (losses) losses[r] = -logf(p[targets[r]]);
    }
}
/* train_gpt2.c:502-521: dlogits[r][i] += (p - [i==target]) * dloss for i < V; pads untouched */
CREF_API void cref_crossentropy_softmax_backward(float* dlogits, const float* probs, const int* targets, float dloss,
                                                 int N, int V, int Vp) {
    for (int r = 0; r < N; r++) {
        float* d = dlogits + (size_t)r * Vp;
        const float* p = probs + (size_t)r * Vp;
        for (int i = 0; i < V; i++) d[i] += (p[i] - (i == targets[r] ? 1.0f : 0.0f)) * dloss;
    }
}

/* train_gpt2.c:1007-1033: plain fp32 AdamW, decay on every element */
CREF_API void cref_adamw(float* p, float* m, float* v, const float* g, size_t n, float lr, float b1, float b2,
                         float eps, float wd, int t) {
    float c1 = 1.0f - powf(b1, (float)t), c2 = 1.0f - powf(b2, (float)t);
    for (size_t i = 0; i < n; i++) {
        float mi = b1 * m[i] + (1.0f - b1) * g[i];
        float vi = b2 * v[i] + (1.0f - b2) * g[i] * g[i];
        m[i] = mi;
        v[i] = vi;
        p[i] -= lr * ((mi / c1) / (sqrtf(vi / c2) + eps) + wd * p[i]);
    }
}

/* Sum of squares in double (dev/cuda/global_norm.cu:21-28) */
CREF_API double cref_sum_squares(const float* x, size_t n) {
    double s = 0.0;
    for (size_t i = 0; i < n; i++) s += (double)x[i] * (double)x[i];
    return s;
}

/* ------------------------------------------------------------------------------------------
 * Mixed-precision optimiser pieces (CUDA-only in the reference)
 * ---------------------------------------------------------------------------------------- */

/* llmc/cuda_utils.cuh:238-256 */
CREF_API uint32_t cref_squirrel_noise5(uint32_t pos, uint32_t seed) {
    uint32_t x = pos;
    x *= 0xd2a80a3fu; x += seed; x ^= x >> 9;
    x += 0xa884f197u; x ^= x >> 11;
    x *= 0x6C736F4Bu; x ^= x >> 13;
    x += 0xB79F3ABBu; x ^= x >> 15;
    x *= 0x1b56c4f5u; x ^= x >> 17;
    return x;
}
/* llmc/cuda_utils.cuh:257-264 */
CREF_API uint32_t cref_noise_2d(int x, int y, uint32_t seed) {
    return cref_squirrel_noise5((uint32_t)x + 198491317u * (uint32_t)y, seed);
}
/* llmc/cuda_utils.cuh:267-278: keep the low 16 mantissa bits with probability low/65536 */
CREF_API uint16_t cref_stochastic_round_bf16(float x, uint32_t rnd) {
    uint32_t thr = rnd & 0xffffu, u = f2u(x), low = u & 0xffffu;
    u = low > thr ? (u | 0xffffu) : (u & ~0xffffu);
    return cref_f32_to_bf16(u2f(u));
}
/* Random word the reference's AdamW launch geometry gives element idx of slice `slice`
 * (block 512, grid (ceil(n/512), slices): threadIdx.x = idx%512, blockIdx.x = idx/512,
 * blockIdx.y = slice; llmc/cuda_utils.cuh:272, llmc/adamw.cuh:81-88). */
CREF_API uint32_t cref_adamw_noise(size_t idx, int slice, uint32_t seed) {
    return cref_noise_2d((int)(idx % 512), (int)((idx / 512) * 512 + (size_t)slice), seed);
}
static inline float lerpf(float a, float b, float w) { return fmaf(w, b, fmaf(-w, a, a)); }

/* llmc/adamw.cuh:18-47 over one slice: bf16 params/grads, fp32 m, v and optional master. */
CREF_API void cref_adamw_mixed(uint16_t* p, float* master, const uint16_t* g, float* m, float* v, size_t n,
                               float lr, float b1, float b2, int t, float eps, float wd, float grad_scale,
                               uint32_t seed, int slice) {
    float c1 = 1.0f - powf(b1, (float)t), c2 = 1.0f - powf(b2, (float)t);
    for (size_t i = 0; i < n; i++) {
        float gi = grad_scale * cref_bf16_to_f32(g[i]);
        float mi = lerpf(gi, m[i], b1);
        float vi = lerpf(gi * gi, v[i], b2);
        m[i] = mi;
        v[i] = vi;
        mi /= c1;
        vi /= c2;
        float old = master ? master[i] : cref_bf16_to_f32(p[i]);
        float np = old - lr * (mi / (sqrtf(vi) + eps) + wd * old);
        p[i] = cref_stochastic_round_bf16(np, cref_adamw_noise(i, slice, seed));
        if (master) master[i] = np;
    }
}
/* same update with fp32 params and fp32 grads (the library's FP32 build; rounding is the identity) */
CREF_API void cref_adamw_f32(float* p, float* master, const float* g, float* m, float* v, size_t n, float lr,
                             float b1, float b2, int t, float eps, float wd, float grad_scale) {
    float c1 = 1.0f - powf(b1, (float)t), c2 = 1.0f - powf(b2, (float)t);
    for (size_t i = 0; i < n; i++) {
        float gi = grad_scale * g[i];
        float mi = lerpf(gi, m[i], b1);
        float vi = lerpf(gi * gi, v[i], b2);
        m[i] = mi;
        v[i] = vi;
        mi /= c1;
        vi /= c2;
        float old = master ? master[i] : p[i];
        float np = old - lr * (mi / (sqrtf(vi) + eps) + wd * old);
        p[i] = np;
        if (master) master[i] = np;
    }
}

/* xorshift* used for per-tensor seeds (train_gpt2.c:1051-1057, llmc/sampler.h) */
CREF_API uint32_t cref_random_u32(uint64_t* state) {
    *state ^= *state >> 12;
    *state ^= *state << 25;
    *state ^= *state >> 27;
    return (uint32_t)((*state * 0x2545F4914F6CDD1Dull) >> 32);
}

/* ------------------------------------------------------------------------------------------
 * Whole model: forward + backward + AdamW on one fixed batch
 * (order of operations follows train_gpt2.c:765-891, :898-1005, :1007-1033)
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    float *ln1, *ln1_mean, *ln1_rstd, *qkv, *atty, *att, *res2, *ln2, *ln2_mean, *ln2_rstd, *fch, *fch_gelu, *res3;
} layer_acts;

static float* falloc(size_t n) {
    float* p = (float*)calloc(n ? n : 1, sizeof(float));
    if (!p) { fprintf(stderr, "cpu_ref: out of memory (%zu floats)\n", n); exit(1); }
    return p;
}
static double now_s(void) { struct timespec ts; clock_gettime(CLOCK_MONOTONIC, &ts); return ts.tv_sec + ts.tv_nsec * 1e-9; }

/* Runs `steps` optimisation steps on the batch (inputs, targets), all (B*T) ints.
 *  params        in/out, flat fp32 in parameter-tensor order
 *  losses_out    [steps]        mean loss of each step's forward
 *  grads_out     optional [num_params]: gradient of step `grad_step` (0-based)
 *  logits_out    optional [B*T*Vp]: logits of step 0's forward
 *  step_ms_out   optional [steps]: wall time of forward+backward+update
 *  grad_clip     <= 0: none (train_gpt2.c); > 0: scale grads by min(1, clip/||g||) like train_gpt2.cu:1850
 *  wd_mask_2d    0: decay every tensor (train_gpt2.c:1031); 1: only 2-D tensors (train_gpt2.cu:1080)
 * Returns 0. */
CREF_API int cref_gpt2_train(const cref_config* cfg, float* params, const int* inputs, const int* targets, int B,
                             int T, int steps, float lr, float b1, float b2, float eps, float wd, float grad_clip,
                             int wd_mask_2d, float* losses_out, float* grads_out, int grad_step, float* logits_out,
                             float* step_ms_out, float* gradnorm_out) {
    const int C = cfg->channels, L = cfg->num_layers, NH = cfg->num_heads, V = cfg->vocab_size, Vp = cfg->padded_vocab_size;
    const size_t N = (size_t)B * T;
    size_t sz[CREF_NPARAM], off[CREF_NPARAM];
    size_t np = cref_param_sizes(sz, cfg);
    { size_t o = 0; for (int i = 0; i < CREF_NPARAM; i++) { off[i] = o; o += sz[i]; } }
    float* grads = falloc(np);
    float* m = falloc(np);
    float* v = falloc(np);
    float* P[CREF_NPARAM];
    float* G[CREF_NPARAM];
    for (int i = 0; i < CREF_NPARAM; i++) { P[i] = params + off[i]; G[i] = grads + off[i]; }

    float* encoded = falloc(N * C);
    layer_acts* A = (layer_acts*)calloc(L, sizeof(layer_acts));
    for (int l = 0; l < L; l++) {
        A[l].ln1 = falloc(N * C); A[l].ln1_mean = falloc(N); A[l].ln1_rstd = falloc(N);
        A[l].qkv = falloc(N * 3 * C); A[l].atty = falloc(N * C); A[l].att = falloc((size_t)B * NH * T * T);
        A[l].res2 = falloc(N * C); A[l].ln2 = falloc(N * C); A[l].ln2_mean = falloc(N); A[l].ln2_rstd = falloc(N);
        A[l].fch = falloc(N * 4 * C); A[l].fch_gelu = falloc(N * 4 * C); A[l].res3 = falloc(N * C);
    }
    float* lnf = falloc(N * C); float* lnf_mean = falloc(N); float* lnf_rstd = falloc(N);
    float* logits = falloc(N * Vp); float* probs = falloc(N * Vp); float* losses = falloc(N);
    float* tmp_c = falloc(N * C);      /* branch output before the residual add */
    /* backward scratch (one layer's worth) */
    float* dlogits = falloc(N * Vp);
    float* dres = falloc(N * C);       /* gradient of the residual stream */
    float* d_c = falloc(N * C);        /* gradient wrt an (N,C) branch tensor */
    float* d_c2 = falloc(N * C);
    float* d_3c = falloc(N * 3 * C);
    float* d_4c = falloc(N * 4 * C);
    float* d_4c2 = falloc(N * 4 * C);

    for (int step = 0; step < steps; step++) {
        double t0 = now_s();
        /* ---- forward ---- */
        cref_encoder_forward(encoded, inputs, P[0], P[1], B, T, C);
        const float* res = encoded;
        for (int l = 0; l < L; l++) {
            layer_acts* a = &A[l];
            cref_layernorm_forward(a->ln1, a->ln1_mean, a->ln1_rstd, res, P[2] + (size_t)l * C, P[3] + (size_t)l * C, (int)N, C);
            cref_matmul_forward(a->qkv, a->ln1, P[4] + (size_t)l * 3 * C * C, P[5] + (size_t)l * 3 * C, (int)N, C, 3 * C);
            cref_attention_forward(a->atty, a->att, NULL, a->qkv, B, T, C, NH);
            cref_matmul_forward(tmp_c, a->atty, P[6] + (size_t)l * C * C, P[7] + (size_t)l * C, (int)N, C, C);
            cref_residual_forward(a->res2, res, tmp_c, N * C);
            cref_layernorm_forward(a->ln2, a->ln2_mean, a->ln2_rstd, a->res2, P[8] + (size_t)l * C, P[9] + (size_t)l * C, (int)N, C);
            cref_matmul_forward(a->fch, a->ln2, P[10] + (size_t)l * 4 * C * C, P[11] + (size_t)l * 4 * C, (int)N, C, 4 * C);
            cref_gelu_forward(a->fch_gelu, a->fch, N * 4 * C);
            cref_matmul_forward(tmp_c, a->fch_gelu, P[12] + (size_t)l * 4 * C * C, P[13] + (size_t)l * C, (int)N, 4 * C, C);
            cref_residual_forward(a->res3, a->res2, tmp_c, N * C);
            res = a->res3;
        }
        cref_layernorm_forward(lnf, lnf_mean, lnf_rstd, res, P[14], P[15], (int)N, C);
        cref_matmul_forward(logits, lnf, P[0], NULL, (int)N, C, Vp);
        cref_softmax_crossentropy_forward(probs, losses, logits, targets, (int)N, V, Vp);
        float mean_loss = 0.f;
        for (size_t i = 0; i < N; i++) mean_loss += losses[i];
        mean_loss /= (float)N;
        losses_out[step] = mean_loss;
        if (step == 0 && logits_out) memcpy(logits_out, logits, N * Vp * sizeof(float));

        /* ---- backward ---- */
        memset(grads, 0, np * sizeof(float));
        memset(dlogits, 0, N * Vp * sizeof(float));
        cref_crossentropy_softmax_backward(dlogits, probs, targets, 1.0f / (float)N, (int)N, V, Vp);
        memset(d_c, 0, N * C * sizeof(float));
        cref_matmul_backward(d_c, G[0], NULL, dlogits, lnf, P[0], (int)N, C, Vp);
        memset(dres, 0, N * C * sizeof(float));
        cref_layernorm_backward(dres, G[14], G[15], d_c, res, P[14], lnf_mean, lnf_rstd, (int)N, C);
        for (int l = L - 1; l >= 0; l--) {
            layer_acts* a = &A[l];
            const float* res_in = l == 0 ? encoded : A[l - 1].res3;
            /* MLP branch: dres is d(res3); it flows unchanged into d(res2) and into d(fcproj out) */
            memset(d_4c, 0, N * 4 * C * sizeof(float));
            cref_matmul_backward(d_4c, G[12] + (size_t)l * 4 * C * C, G[13] + (size_t)l * C, dres, a->fch_gelu,
                                 P[12] + (size_t)l * 4 * C * C, (int)N, 4 * C, C);
            memset(d_4c2, 0, N * 4 * C * sizeof(float));
            cref_gelu_backward(d_4c2, a->fch, d_4c, N * 4 * C);
            memset(d_c, 0, N * C * sizeof(float));
            cref_matmul_backward(d_c, G[10] + (size_t)l * 4 * C * C, G[11] + (size_t)l * 4 * C, d_4c2, a->ln2,
                                 P[10] + (size_t)l * 4 * C * C, (int)N, C, 4 * C);
            cref_layernorm_backward(dres, G[8] + (size_t)l * C, G[9] + (size_t)l * C, d_c, a->res2, P[8] + (size_t)l * C,
                                    a->ln2_mean, a->ln2_rstd, (int)N, C);
            /* attention branch: dres is now d(res2) */
            memset(d_c2, 0, N * C * sizeof(float));
            cref_matmul_backward(d_c2, G[6] + (size_t)l * C * C, G[7] + (size_t)l * C, dres, a->atty,
                                 P[6] + (size_t)l * C * C, (int)N, C, C);
            memset(d_3c, 0, N * 3 * C * sizeof(float));
            cref_attention_backward(d_3c, d_c2, a->qkv, a->att, B, T, C, NH);
            memset(d_c, 0, N * C * sizeof(float));
            cref_matmul_backward(d_c, G[4] + (size_t)l * 3 * C * C, G[5] + (size_t)l * 3 * C, d_3c, a->ln1,
                                 P[4] + (size_t)l * 3 * C * C, (int)N, C, 3 * C);
            cref_layernorm_backward(dres, G[2] + (size_t)l * C, G[3] + (size_t)l * C, d_c, res_in, P[2] + (size_t)l * C,
                                    a->ln1_mean, a->ln1_rstd, (int)N, C);
        }
        cref_encoder_backward(G[0], G[1], dres, inputs, B, T, C);
        if (grads_out && step == grad_step) memcpy(grads_out, grads, np * sizeof(float));

        /* ---- update ---- */
        float gscale = 1.0f;
        float gnorm = sqrtf((float)cref_sum_squares(grads, np));
        if (gradnorm_out) gradnorm_out[step] = gnorm;
        if (grad_clip > 0.f && gnorm > grad_clip) gscale = grad_clip / gnorm;
        if (gscale != 1.0f) for (size_t i = 0; i < np; i++) grads[i] *= gscale;
        for (int i = 0; i < CREF_NPARAM; i++) {
            int is2d = (i == 0 || i == 1 || i == 4 || i == 6 || i == 10 || i == 12);
            float w = (wd_mask_2d && !is2d) ? 0.f : wd;
            cref_adamw(P[i], m + off[i], v + off[i], G[i], sz[i], lr, b1, b2, eps, w, step + 1);
        }
        if (step_ms_out) step_ms_out[step] = (float)((now_s() - t0) * 1e3);
    }

    free(grads); free(m); free(v); free(encoded);
    for (int l = 0; l < L; l++) {
        free(A[l].ln1); free(A[l].ln1_mean); free(A[l].ln1_rstd); free(A[l].qkv); free(A[l].atty); free(A[l].att);
        free(A[l].res2); free(A[l].ln2); free(A[l].ln2_mean); free(A[l].ln2_rstd); free(A[l].fch); free(A[l].fch_gelu);
        free(A[l].res3);
    }
    free(A); free(lnf); free(lnf_mean); free(lnf_rstd); free(logits); free(probs); free(losses); free(tmp_c);
    free(dlogits); free(dres); free(d_c); free(d_c2); free(d_3c); free(d_4c); free(d_4c2);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Text generation: forward only + the sampler (train_gpt2.cu:1751-1796, llmc/sampler.h)
 * ---------------------------------------------------------------------------------------- */

/* random float32 in [0,1) (llmc/sampler.h:18-20) */
CREF_API float cref_random_f32(uint64_t* state) { return (cref_random_u32(state) >> 8) / 16777216.0f; }

/* index drawn from softmax(logits) with the uniform number coin (llmc/sampler.h:22-40) */
CREF_API int cref_sample_softmax(const float* logits, int n, float coin) {
    double norm = 0;
    for (int i = 0; i < n; i++) norm += expf(logits[i]);
    coin *= norm;
    float cdf = 0.0f;
    for (int i = 0; i < n; i++) {
        cdf += expf(logits[i]);
        if (coin < cdf) return i;
    }
    return n - 1;
}

/* logits[B*T*Vp] of the forward pass alone (same order of operations as cref_gpt2_train's forward half,
 * train_gpt2.c:765-880); one layer's activations are kept at a time */
CREF_API int cref_gpt2_logits(const cref_config* cfg, const float* params, const int* inputs, int B, int T, float* logits) {
    const int C = cfg->channels, L = cfg->num_layers, NH = cfg->num_heads, Vp = cfg->padded_vocab_size;
    const size_t N = (size_t)B * T;
    size_t sz[CREF_NPARAM];
    const float* P[CREF_NPARAM];
    cref_param_sizes(sz, cfg);
    { size_t o = 0; for (int i = 0; i < CREF_NPARAM; i++) { P[i] = params + o; o += sz[i]; } }
    float* res = falloc(N * C); float* res2 = falloc(N * C); float* ln = falloc(N * C); float* tmp_c = falloc(N * C);
    float* mean = falloc(N); float* rstd = falloc(N);
    float* qkv = falloc(N * 3 * C); float* atty = falloc(N * C); float* att = falloc((size_t)B * NH * T * T);
    float* fch = falloc(N * 4 * C); float* fch_gelu = falloc(N * 4 * C);
    cref_encoder_forward(res, inputs, P[0], P[1], B, T, C);
    for (int l = 0; l < L; l++) {
        cref_layernorm_forward(ln, mean, rstd, res, P[2] + (size_t)l * C, P[3] + (size_t)l * C, (int)N, C);
        cref_matmul_forward(qkv, ln, P[4] + (size_t)l * 3 * C * C, P[5] + (size_t)l * 3 * C, (int)N, C, 3 * C);
        cref_attention_forward(atty, att, NULL, qkv, B, T, C, NH);
        cref_matmul_forward(tmp_c, atty, P[6] + (size_t)l * C * C, P[7] + (size_t)l * C, (int)N, C, C);
        cref_residual_forward(res2, res, tmp_c, N * C);
        cref_layernorm_forward(ln, mean, rstd, res2, P[8] + (size_t)l * C, P[9] + (size_t)l * C, (int)N, C);
        cref_matmul_forward(fch, ln, P[10] + (size_t)l * 4 * C * C, P[11] + (size_t)l * 4 * C, (int)N, C, 4 * C);
        cref_gelu_forward(fch_gelu, fch, N * 4 * C);
        cref_matmul_forward(tmp_c, fch_gelu, P[12] + (size_t)l * 4 * C * C, P[13] + (size_t)l * C, (int)N, 4 * C, C);
        cref_residual_forward(res, res2, tmp_c, N * C);
    }
    cref_layernorm_forward(ln, mean, rstd, res, P[14], P[15], (int)N, C);
    cref_matmul_forward(logits, ln, P[0], NULL, (int)N, C, Vp);
    free(res); free(res2); free(ln); free(tmp_c); free(mean); free(rstd); free(qkv); free(atty); free(att);
    free(fch); free(fch_gelu);
    return 0;
}

/* The generation loop of train_gpt2.cu:1751-1796: tokens[0..T) start as eot_token; position t = 1..genT-1 is sampled
 * from the logits at position t-1 of a forward pass over one sequence of length ceil(t / min(T,256)) * min(T,256). */
CREF_API int cref_gpt2_generate(const cref_config* cfg, const float* params, int* tokens, int T, int genT, int eot_token,
                                uint64_t* rng_state) {
    const int V = cfg->vocab_size, Vp = cfg->padded_vocab_size;
    const int chunk = T < 256 ? T : 256;
    float* logits = falloc((size_t)T * Vp);
    for (int i = 0; i < T; i++) tokens[i] = eot_token;
    for (int t = 1; t < genT; t++) {
        const int Tr = (t + chunk - 1) / chunk * chunk;
        cref_gpt2_logits(cfg, params, tokens, 1, Tr, logits);
        const float coin = cref_random_f32(rng_state);
        tokens[t] = cref_sample_softmax(logits + (size_t)(t - 1) * Vp, V, coin);
    }
    free(logits);
    return 0;
}

CREF_API int cref_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
