// CPU restatement of the device's random draws. TEST INFRASTRUCTURE ONLY (see rlt_oracle.h).
//
// The reference draws on the device from per-thread curandState generators (devices/cuda.h:88-122,
// containers/tensor/operations_cuda.h:548-624) and on the CPU from std::mt19937; neither sequence is part of
// its contract (its CUDA and CPU runs of one seed differ). What is fixed here is therefore the published
// algorithm the HIP backend uses -- Philox4x32 with 10 rounds, Salmon, Moraes, Dror, Shaw, "Parallel random
// numbers: as easy as 1, 2, 3", SC'11, section 3.3 and the Random123 distribution's known-answer file -- and
// the mapping from (seed, stream, element) to counter and key that include/rlt_rocm.h documents.
//
// Pinning: rlt_oracle_philox4x32_10 is checked against the three published known-answer vectors of
// philox4x32-10 (tests/test_oracle_rng.py); the float conversions against closed forms (range, cell midpoints,
// moments, Kolmogorov-Smirnov distance to the uniform and normal distributions); that streams and seeds select
// different sequences by the absence of any repeated group among a million (seed, stream, index) triples.
#include <vector>
#include "rlt_oracle.h"
#include <cmath>
#include <cstdint>
#include <cstring>

namespace {

// one S-P round on the four counter words: two 32x32->64 multiplications, the high halves xored with the
// other words and the round key, the low halves passed through
void philox_round(uint32_t ctr[4], const uint32_t key[2]) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * ctr[0];
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * ctr[2];
    const uint32_t next[4] = {(uint32_t)(p1 >> 32) ^ ctr[1] ^ key[0], (uint32_t)p1, (uint32_t)(p0 >> 32) ^ ctr[3] ^ key[1], (uint32_t)p0};
    std::memcpy(ctr, next, sizeof next);
}

void philox(const uint32_t counter[4], const uint32_t key_in[2], uint32_t out[4]) {
    uint32_t ctr[4] = {counter[0], counter[1], counter[2], counter[3]};
    uint32_t key[2] = {key_in[0], key_in[1]};
    for (int round = 0; round < 10; round++) {
        if (round > 0) { key[0] += 0x9E3779B9u; key[1] += 0xBB67AE85u; }   // Weyl sequence on the key
        philox_round(ctr, key);
    }
    std::memcpy(out, ctr, sizeof ctr);
}

// group `index` of the sequence (seed, stream): key = seed, counter = (index low, index high, stream low, stream high)
void group(uint64_t seed, uint64_t stream, uint64_t index, uint32_t out[4]) {
    const uint32_t counter[4] = {(uint32_t)index, (uint32_t)(index >> 32), (uint32_t)stream, (uint32_t)(stream >> 32)};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    philox(counter, key, out);
}

// the midpoint of one of 2^24 equal cells of (0, 1), chosen by the upper 24 bits
float unit(uint32_t word) { return ((float)(word >> 8) + 0.5f) * (1.0f / 16777216.0f); }

}  // namespace

extern "C" {

int rlt_oracle_philox4x32_10(const uint32_t* counter, const uint32_t* key, uint32_t* out) {
    if (!counter || !key || !out) return RLT_E_INVALID_ARGUMENT;
    philox(counter, key, out);
    return 0;
}

int rlt_oracle_rand_bits_u32(uint32_t* dst, size_t count, uint64_t seed, uint64_t stream) {
    if (!dst) return RLT_E_INVALID_ARGUMENT;
    for (size_t i = 0; i < count; i++) { uint32_t g[4]; group(seed, stream, i / 4, g); dst[i] = g[i % 4]; }
    return 0;
}

int rlt_oracle_rand_f32(float* dst, size_t count, float low, float high, uint64_t seed, uint64_t stream) {
    if (!dst) return RLT_E_INVALID_ARGUMENT;
    for (size_t i = 0; i < count; i++) { uint32_t g[4]; group(seed, stream, i / 4, g); dst[i] = low + (high - low) * unit(g[i % 4]); }
    return 0;
}

// Box-Muller: words (0, 1) of a group give elements 0 (cosine) and 1 (sine), words (2, 3) elements 2 and 3
int rlt_oracle_randn_f32(float* dst, size_t count, uint64_t seed, uint64_t stream) {
    if (!dst) return RLT_E_INVALID_ARGUMENT;
    for (size_t i = 0; i < count; i++) {
        uint32_t g[4]; group(seed, stream, i / 4, g);
        const int pair = (int)(i % 4) / 2;
        const float radius = std::sqrt(-2.0f * std::log(unit(g[2 * pair])));
        const float angle = 6.283185307179586f * unit(g[2 * pair + 1]);
        dst[i] = radius * ((i % 2) ? std::sin(angle) : std::cos(angle));
    }
    return 0;
}

// (environment, offset) pairs uniform over the eligible rows of each ring (off_policy_runner/operations_generic.h:257,304,426 draw
// the same two numbers per sample): sample i takes words 0 and 1 of group i, each scaled by multiply-shift
int rlt_oracle_gather_draw(const rlt_replay_buffer* rb, int batch, uint64_t seed, uint64_t stream, uint32_t* env_indices, uint32_t* sample_offsets) {
    if (!rb || !env_indices || !sample_offsets || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int i = 0; i < batch; i++) {
        uint32_t g[4]; group(seed, stream, (uint64_t)i, g);
        const uint32_t env = (uint32_t)(((uint64_t)g[0] * (uint32_t)rb->n_envs) >> 32);
        const uint32_t eligible = rb->full[env] ? (uint32_t)rb->capacity : rb->position[env];
        env_indices[i] = env;
        sample_offsets[i] = eligible ? (uint32_t)(((uint64_t)g[1] * eligible) >> 32) : 0u;
    }
    return 0;
}

// the draws of a sequence batch (off_policy_runner/operations_generic.h:257-275,304,362-371,426), in the word order documented at
// rlt_rocm_gather_sequence_draw: environment, padded offsets, padded + 1 nominal decisions, padded + 1 lengths
int rlt_oracle_gather_sequence_draw(const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling, int max_episode_length, int batch, int sequence_length, uint64_t seed,
                                    uint64_t stream, uint32_t* env_indices, uint32_t* sample_offsets, uint8_t* nominal, uint32_t* lengths) {
    if (!rb || !sampling || !env_indices || !sample_offsets || !nominal || !lengths || batch <= 0 || sequence_length < 1) return RLT_E_INVALID_ARGUMENT;
    const int padded = sequence_length + 1, n_words = 3 * padded + 3, groups = (n_words + 3) / 4;
    std::vector<uint32_t> words((size_t)groups * 4);
    for (int b = 0; b < batch; b++) {
        for (int g = 0; g < groups; g++) group(seed, stream, (uint64_t)b * groups + g, &words[4 * (size_t)g]);
        const uint32_t env = (uint32_t)(((uint64_t)words[0] * (uint32_t)rb->n_envs) >> 32);
        env_indices[b] = env;
        const uint32_t eligible = rb->full[env] ? (uint32_t)(sampling->always_sample_from_initial_state ? rb->capacity - max_episode_length : rb->capacity) : rb->position[env];
        for (int k = 0; k < padded; k++) sample_offsets[(size_t)b * padded + k] = eligible ? (uint32_t)(((uint64_t)words[1 + k] * eligible) >> 32) : 0u;
        for (int k = 0; k <= padded; k++) {
            nominal[(size_t)b * (padded + 1) + k] = unit(words[1 + padded + k]) < sampling->nominal_sequence_length_probability ? 1 : 0;
            lengths[(size_t)b * (padded + 1) + k] = sequence_length > 1 ? 1u + (uint32_t)(((uint64_t)words[2 + 2 * padded + k] * (uint32_t)(sequence_length - 1)) >> 32) : 1u;
        }
    }
    return 0;
}

// initial states the runner's prologue draws for the environments that reset: theta ~ U(-pi, pi), theta_dot ~ U(-1, 1)
// (rl/environments/pendulum/operations_generic.h sample_initial_state), environment e from words 0 and 1 of group e
int rlt_oracle_pendulum_initial_states(float* states, int n_envs, uint64_t seed, uint64_t stream) {
    if (!states || n_envs <= 0) return RLT_E_INVALID_ARGUMENT;
    const float pi = 3.14159265358979323846f;
    for (int e = 0; e < n_envs; e++) {
        uint32_t g[4]; group(seed, stream, (uint64_t)e, g);
        states[2 * e] = -pi + 2.0f * pi * unit(g[0]);
        states[2 * e + 1] = -1.0f + 2.0f * unit(g[1]);
    }
    return 0;
}

// sum / sum of squares of a float tensor in index order with a double accumulator (gradient_norm's inner sum,
// nn/parameters/operations_generic.h; the reference accumulates in T)
int rlt_oracle_reduce_sum_f32(const float* x, size_t count, int squared, float* out_sum) {
    if (!x || !out_sum) return RLT_E_INVALID_ARGUMENT;
    double acc = 0.0;
    for (size_t i = 0; i < count; i++) acc += squared ? (double)x[i] * x[i] : (double)x[i];
    *out_sum = (float)acc;
    return 0;
}

}  // extern "C"
