// Shared declarations of the gfx950 backend: device handle, error plumbing, launch helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/rlt_rocm.h"

constexpr int RLT_SIDE_STREAMS = 2;
struct rlt_rocm_device {
    int hip_device;
    hipStream_t own_stream;
    hipStream_t stream;          // the stream work is enqueued on (own_stream unless the caller set one)
    int compute_units;
    int lds_bytes;
    char name[128];
    void* scratch;               // grow-only device workspace for split reductions and partial sums
    size_t scratch_bytes;
    void* pad_scratch;           // a second grow-only buffer: zero-padded copies of narrow networks (pad.hip)
    size_t pad_scratch_bytes;
    void* copy_scratch; size_t copy_scratch_bytes;      // weight copies in consumption order of the MLP calls on sixteen-row tiles: not the handle's scratch buffer, which callers of forward() / evaluate() may hold across the call
    void* counters;              // 8 KiB, zero between launches: [0,256) ticket counters, [256,..) per-workgroup partial sums
    unsigned* fault;             // [0]: set by a persistent kernel that gave up waiting for another workgroup; read back by check_status
    int fault_armed;             // a kernel that can set it was launched since the last check
    int xcd_stride;              // workgroups b and b + xcd_stride run on the same XCD (0: not established; consecutive workgroups go round the XCDs)
    int sticky_error;
    int sac_per_operation;       // rlt_rocm_sac_train_critic / _actor run one launch per reference operation even where the fused kernels fit
    int update_tail;             // the fused update kernels step the optimiser themselves (their last workgroup), instead of in launches after them
    int update_one_xcd;          // small grids of the fused update kernels are placed on one XCD
    unsigned wait_limit;         // polls after which a workgroup gives up waiting for another (rlt_rocm_set_wait_limit; about a second by default)
    int capturing;               // the stream is recording a graph: nothing may allocate, free or wait (rlt_rocm_graph_begin_capture)
    uint64_t* stream_offset;     // device word added to the stream number of every draw made on the device (rlt_rocm_advance_streams)
    // two more streams (default priority) for passes that do not depend on what the main stream does next (rlt_side_begin); side_stream[0] null: none could be made
    hipStream_t side_stream[RLT_SIDE_STREAMS];
    hipEvent_t fork_event[RLT_SIDE_STREAMS], join_event[RLT_SIDE_STREAMS];
    int side_pending[RLT_SIDE_STREAMS];      // work has gone to the stream since the main stream last waited for it
    hipStream_t side_return;     // the stream to switch back to while work goes to a side stream (null otherwise)
    int side_active;             // which side stream that is
    void* side_scratch[RLT_SIDE_STREAMS]; size_t side_scratch_bytes[RLT_SIDE_STREAMS];      // what rlt_scratch hands out while work goes to a side stream: passes that run at the same time do not share split sums
};

// Network passes that are independent of each other (the two target critics of a sequence update, a critic's forward pass and the actor's) overlap on up to
// three streams: between rlt_side_begin(device, which) and rlt_side_end every launch of the library goes to the handle's side stream `which`, which first waits
// for everything enqueued on the main stream so far; rlt_side_join makes the main stream wait for every side stream that has received work. While the main stream
// records a graph (or if the side streams could not be made) rlt_side_begin returns false and the work simply stays on the main stream, in order. Passes that run at the same time must not share a workspace;
// the handle's scratch buffer (rlt_scratch: split sums of weight gradients) has a second instance for the side stream. The ticket counters (rlt_counters) have not:
// optimiser steps stay on the main stream.
bool rlt_side_begin(rlt_rocm_device* device, int which = 0);
void rlt_side_end(rlt_rocm_device* device);
int rlt_side_join(rlt_rocm_device* device);

#define RLT_HIP(expr)                                                        \
    do {                                                                     \
        hipError_t _e = (expr);                                              \
        if (_e != hipSuccess) { if (device) device->sticky_error = (int)_e; return (int)_e; } \
    } while (0)

#define RLT_REQUIRE(cond) do { if (!(cond)) return RLT_E_INVALID_ARGUMENT; } while (0)
// for entry points that allocate, free, copy to or from the host or wait: not while the stream records a graph
#define RLT_NOT_WHILE_CAPTURING() do { if (device->capturing) return RLT_E_CAPTURING; } while (0)

// Grow-only scratch owned by the device handle.
int rlt_scratch(rlt_rocm_device* device, size_t bytes, void** out);
// 8 KiB of zero-initialised device memory for last-workgroup-done tickets and per-workgroup partials.
int rlt_counters(rlt_rocm_device* device, void** out);
// Returns hipGetLastError() folded into the return convention; called after every launch.
int rlt_launch_status(rlt_rocm_device* device);

static inline int rlt_div_up(int a, int b) { return (a + b - 1) / b; }

// ---- activation functions on the device (nn/activation_functions.h:25-90 of the reference)
__device__ __forceinline__ float rlt_fast_tanh(float x) {
    x = fminf(fmaxf(x, -3.0f), 3.0f);
    float x2 = x * x;
    return x * (27.0f + x2) / (27.0f + 9.0f * x2);
}
__device__ __forceinline__ float rlt_act(float x, int f) {
    switch (f) {
        case RLT_ACT_RELU: return x > 0.0f ? x : 0.0f;
        // the reference's GELU constant is FRAC_2_SQRTPI * SQRT1_2 * 0.5, half of the textbook sqrt(2/pi) (nn/activation_functions.h:33-36)
        case RLT_ACT_GELU: { const float a = 0.3989422804014327f; return 0.5f * (x + x * tanhf(a * (0.044715f * x * x * x + x))); }
        case RLT_ACT_TANH: return tanhf(x);
        case RLT_ACT_FAST_TANH: return rlt_fast_tanh(x);
        case RLT_ACT_SIGMOID: return 1.0f / (1.0f + expf(-x));
        default: return x;
    }
}
__device__ __forceinline__ float rlt_dact(float x, int f) {
    switch (f) {
        case RLT_ACT_RELU: return x > 0.0f ? 1.0f : 0.0f;
        case RLT_ACT_GELU: {
            const float a = 0.3989422804014327f, b = 0.044715f;
            float t = tanhf(a * (b * x * x * x + x));
            return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * a * (3.0f * b * x * x + 1.0f);
        }
        case RLT_ACT_TANH: { float t = tanhf(x); return 1.0f - t * t; }
        case RLT_ACT_FAST_TANH: { float t = rlt_fast_tanh(x); return 1.0f - t * t; }
        case RLT_ACT_SIGMOID: { float s = 1.0f / (1.0f + expf(-x)); return s * (1.0f - s); }
        default: return 1.0f;
    }
}

// the same derivative written in terms of the layer OUTPUT o = act(x), where that is possible (everything but GELU):
// relu: o > 0 <=> x > 0; tanh / fast_tanh: 1 - o^2; sigmoid: o (1 - o)
__device__ __forceinline__ float rlt_dact_from_output(float o, int f) {
    switch (f) {
        case RLT_ACT_RELU: return o > 0.0f ? 1.0f : 0.0f;
        case RLT_ACT_TANH: case RLT_ACT_FAST_TANH: return 1.0f - o * o;
        case RLT_ACT_SIGMOID: return o * (1.0f - o);
        default: return 1.0f;
    }
}

// Workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every global load and store the wavefront has in
// flight, which defeats prefetching across a barrier; kernels whose wavefronts exchange data through LDS alone use this one.
__device__ __forceinline__ void rlt_lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// 64-lane wavefront sum (butterfly over DPP/ds_swizzle via __shfl_xor)
// Every lane receives the same sum bit for bit (each exchange adds the same two numbers on both sides). The summand is pinned to a register first: otherwise the compiler may contract the multiplication that produced it into the first addition
// (fma(a_i, b_i, partner's rounded product)), and the two lanes of an exchange then round differently -- the lanes no longer hold the same sum bit for bit.
__device__ __forceinline__ float rlt_wave_sum(float v) {
    asm volatile("" : "+v"(v));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
