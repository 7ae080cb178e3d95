// mt19937 with torch-compatible uniform / normal_ draws, for seeded weight init.
// Same streams as the reference's llmc/rand.h:106-221 (which follows PyTorch's CPU generator);
// known-answer values for seed 137 are printed there (rand.h:48-80) and checked in tests/.
#pragma once
#include <cmath>
#include <cstdint>

namespace llmk {

class Mt19937 {
public:
    explicit Mt19937(uint32_t seed) { reseed(seed); }
    void reseed(uint32_t seed) {
        s_[0] = seed;
        for (uint32_t j = 1; j < N; j++) s_[j] = 1812433253u * (s_[j - 1] ^ (s_[j - 1] >> 30)) + j;
        left_ = 1;
        next_ = 0;
    }
    uint32_t u32() {
        if (--left_ <= 0) refill();
        uint32_t y = s_[next_++];
        y ^= y >> 11;
        y ^= (y << 7) & 0x9d2c5680u;
        y ^= (y << 15) & 0xefc60000u;
        y ^= y >> 18;
        return y;
    }
    uint64_t u64() { uint64_t hi = u32(); return (hi << 32) | u32(); }
    float f32() { return (float)(u32() & 0xffffffu) * (1.0f / 16777216.0f); }
    double f64() { return (double)(u64() & ((1ull << 53) - 1)) * (1.0 / 9007199254740992.0); }

    // torch.Tensor.normal_ on a CPU float tensor of n elements
    void normal(float* d, uint32_t n, float mean, float std) {
        if (n >= 16) {
            for (uint32_t t = 0; t < n; t++) d[t] = f32();
            for (uint32_t i = 0; i + 16 <= n; i += 16) box_muller16(d + i, mean, std);
            if (n % 16) {
                float* tail = d + n - 16;
                for (int i = 0; i < 16; i++) tail[i] = f32();
                box_muller16(tail, mean, std);
            }
            return;
        }
        bool have = false;
        double spare = 0.0;
        for (uint32_t t = 0; t < n; t++) {
            if (have) { d[t] = (float)(spare * std + mean); have = false; continue; }
            float u1 = (float)f64(), u2 = (float)f64();
            float r = sqrtf(-2.0f * logf(1.0f - u2 + 1e-12f));
            float th = (float)(2.0 * M_PI * u1);
            spare = r * sinf(th);
            have = true;
            d[t] = r * cosf(th) * std + mean;
        }
    }

    // The generator's state in the order of the reference's struct (llmc/rand.h:98-104, after its unused first field):
    // left_, next_, the 624 state words. MATRIX_A there is the constant pair {0, 0x9908b0df}.
    static constexpr uint32_t STATE_WORDS = 624;
    void export_state(int32_t& left, uint32_t& next, uint32_t* words) const {
        left = left_; next = (uint32_t)next_;
        for (uint32_t j = 0; j < N; j++) words[j] = s_[j];
    }
    void import_state(int32_t left, uint32_t next, const uint32_t* words) {
        left_ = left; next_ = (int)next;
        for (uint32_t j = 0; j < N; j++) s_[j] = words[j];
    }

private:
    static constexpr uint32_t N = 624, M = 397;
    uint32_t s_[N];
    int left_ = 1, next_ = 0;
    void refill() {
        for (uint32_t j = 0; j < N; j++) {
            uint32_t y = (s_[j] & 0x80000000u) | (s_[(j + 1) % N] & 0x7fffffffu);
            s_[j] = s_[(j + M) % N] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
        }
        left_ = N;
        next_ = 0;
    }
    static void box_muller16(float* d, float mean, float std) {
        for (int t = 0; t < 8; t++) {
            float u1 = 1.0f - d[t], u2 = d[t + 8];
            float r = sqrtf(-2.0f * logf(u1 + 1e-12f));
            float th = (float)(2.0 * M_PI * u2);
            d[t] = r * cosf(th) * std + mean;
            d[t + 8] = r * sinf(th) * std + mean;
        }
    }
};

// xorshift* stream that hands out per-tensor seeds (reference: llmc/sampler.h:10-16)
inline uint32_t random_u32(unsigned long long* state) {
    *state ^= *state >> 12;
    *state ^= *state << 25;
    *state ^= *state >> 27;
    return (uint32_t)((*state * 0x2545F4914F6CDD1Dull) >> 32);
}

// random float32 in [0,1) from the same stream (reference: llmc/sampler.h:18-20)
inline float random_f32(unsigned long long* state) { return (random_u32(state) >> 8) / 16777216.0f; }

// Index drawn from softmax(logits) with the uniform number `coin` (reference: llmc/sampler.h:22-40): the
// normaliser is summed in double, the running distribution in float, and the coin is scaled instead of the terms.
inline int sample_softmax(const float* logits, int n, float coin) {
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

}  // namespace llmk
