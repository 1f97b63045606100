// Counter-based random numbers of the backend: Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy
// as 1, 2, 3", SC'11). The reference keeps a generator STATE per call site (curandState in devices/cuda.h:88-122,
// std::mt19937 on the CPU); here a draw is a pure function of three numbers, so no state array exists:
//   key     = seed                     (64 bits -> k0, k1)
//   counter = (index, stream)          index  -> c0, c1 : which group of four 32-bit values inside the stream
//                                      stream -> c2, c3 : which call / which kind of draw
// Two different (seed, stream) pairs select disjoint sequences of 2^64 groups each: Philox is a bijection of the counter for a
// fixed key, so no two (index, stream) pairs of one seed share a group.
#pragma once
#include <stdint.h>
#ifndef RLT_RNG_HOST
#include <hip/hip_runtime.h>
#define RLT_RNG_FN __host__ __device__ __forceinline__
#else
#define RLT_RNG_FN static inline
#endif

struct rlt_u32x4 { uint32_t x, y, z, w; };

RLT_RNG_FN uint32_t rlt_mulhi32(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * (uint64_t)b) >> 32); }

// The raw block function on explicit counter and key words (what the published known-answer vectors are stated on).
RLT_RNG_FN rlt_u32x4 rlt_philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
    const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int r = 0; r < 10; r++) {
        const uint32_t hi0 = rlt_mulhi32(M0, c0), lo0 = M0 * c0;
        const uint32_t hi1 = rlt_mulhi32(M1, c2), lo1 = M1 * c2;
        const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
        c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
        k0 += W0; k1 += W1;
    }
    rlt_u32x4 out = {c0, c1, c2, c3};
    return out;
}

// group `index` of stream `stream` under `seed`
RLT_RNG_FN rlt_u32x4 rlt_philox(uint64_t seed, uint64_t stream, uint64_t index) {
    return rlt_philox4x32_10((uint32_t)index, (uint32_t)(index >> 32), (uint32_t)stream, (uint32_t)(stream >> 32), (uint32_t)seed, (uint32_t)(seed >> 32));
}

// 24 random bits -> the midpoint of one of 2^24 equal cells of (0, 1): never 0 or 1, so log() and the scaling to [low, high) are safe
RLT_RNG_FN float rlt_u01(uint32_t x) { return ((float)(x >> 8) + 0.5f) * (1.0f / 16777216.0f); }

// a uniform integer in [0, n) from 32 random bits (multiply-shift; bias below n / 2^32)
RLT_RNG_FN uint32_t rlt_uniform_below(uint32_t x, uint32_t n) { return (uint32_t)(((uint64_t)x * (uint64_t)n) >> 32); }

#ifndef RLT_RNG_HOST
// Element i of a uniform stream as rlt_rocm_rand_f32 lays it out (word i % 4 of group i / 4), in (0, 1)
__device__ __forceinline__ float rlt_rand_element(uint64_t seed, uint64_t stream, uint64_t i) {
    const rlt_u32x4 r = rlt_philox(seed, stream, i >> 2);
    const uint32_t k = (uint32_t)(i & 3);
    return rlt_u01(k == 0 ? r.x : k == 1 ? r.y : k == 2 ? r.z : r.w);
}
// Element i of a standard-normal stream as rlt_rocm_randn_f32 lays it out: word i % 4 of group i / 4, Box-Muller on the word pairs
// (0, 1) and (2, 3) -- for kernels that take their noise from the stream directly instead of from an array filled beforehand.
__device__ __forceinline__ float rlt_randn_element(uint64_t seed, uint64_t stream, uint64_t i) {
    const rlt_u32x4 r = rlt_philox(seed, stream, i >> 2);
    const bool second = (i & 2) != 0;
    const float radius = sqrtf(-2.0f * logf(rlt_u01(second ? r.z : r.x)));
    float s, c;
    sincosf(6.283185307179586f * rlt_u01(second ? r.w : r.y), &s, &c);
    return (i & 1) ? radius * s : radius * c;
}
#endif
