// Internal entry points of optim.hip, and the optimiser's arithmetic as device functions for the kernels that step a network at
// the end of the launch that produced its gradients.
#pragma once
#include "common.h"

// Gradients that are still blocks of partial sums (one block of `block_stride` floats per workgroup of the kernel that made them): the
// optimiser's launch adds them up, in the order of the small-MLP reduction kernel, stores the sums in the tensors' gradients and steps.
// offsets[t]: where tensor t's gradient starts within a block; scales[t]: factor on its sums.
struct rlt_adam_source { const float* partial; int groups, block_stride; const uint32_t* offsets; const float* scales; };

// rlt_rocm_adam_step for at most 12 tensors whose gradients are blocks of partial sums
int rlt_adam_step_from_partials(rlt_rocm_device* device, const rlt_adam_tensor* tensors, int n, const rlt_adam_parameters* parameters, uint32_t* age, const rlt_adam_source* source);

// rlt_rocm_adam_step for two optimisers (each with its own tensors, parameters and age) in one launch; each list at most 12 tensors
// where a source is given
int rlt_adam_step_pair(rlt_rocm_device* device, const rlt_adam_tensor* tensors_a, int n_a, const rlt_adam_parameters* parameters_a, uint32_t* age_a,
                       const rlt_adam_tensor* tensors_b, int n_b, const rlt_adam_parameters* parameters_b, uint32_t* age_b,
                       const rlt_adam_source* source_a = nullptr, const rlt_adam_source* source_b = nullptr);

// ---- device side -------------------------------------------------------------------------------------------------------------------
// Words of the device handle's counters block (uint32 index) that the kernels with an optimiser tail use as tickets; every user
// leaves its words zero. [0] and [16] belong to adam_kernel / adam_pair_kernel.
enum { RLT_TICKET_TAIL = 32 /* .. +7 */ };

// target <- polyak * target + (1 - polyak) * source (utils/polyak/operations_generic.h:11-27): one expression for every kernel
// (products rounded before the sum in every kernel that uses it, so that all of them leave the same bits)
__device__ __forceinline__ float rlt_polyak_value(float polyak, float target, float source) {
#pragma clang fp contract(off)
    const float a = polyak * target, b = (1.0f - polyak) * source;
    return a + b;
}

// 1 / (1 - beta^age) for both moments (nn/optimizers/adam/operations_generic.h:49-58: from the age before the step)
__device__ __forceinline__ void rlt_adam_bias_corrections(const rlt_adam_parameters& p, uint32_t age, float& bc1, float& bc2) {
    bc1 = 1.0f / (1.0f - powf(p.beta_1, (float)age));
    bc2 = 1.0f / (1.0f - powf(p.beta_2, (float)age));
}

// One element of a tensor: moments, step, optional fused soft update of a target (nn/optimizers/adam/instance/operations_generic.h:26-72).
// Returns the new parameter value.
__device__ __forceinline__ float rlt_adam_apply(const rlt_adam_parameters& p, const rlt_adam_tensor& T, uint32_t j, float g, float bc1, float bc2, float polyak) {
#pragma clang fp contract(off)      // no product is fused into a sum: every kernel that inlines this leaves the same bits
    if (p.enable_gradient_clipping) g = fminf(fmaxf(g, -p.gradient_clip_value), p.gradient_clip_value);
    float m = p.beta_1 * T.first_moment[j] + (1.0f - p.beta_1) * g;
    float v = p.beta_2 * T.second_moment[j] + (1.0f - p.beta_2) * g * g;
    T.first_moment[j] = m; T.second_moment[j] = v;
    float pre_sqrt = fmaxf(v * bc2, p.epsilon_sqrt);
    float update = p.alpha * bc1 * m / (sqrtf(pre_sqrt) + p.epsilon);
    float param = T.parameters[j];
    if ((T.flags & 2u) && p.enable_bias_lr_factor) update *= p.bias_lr_factor;
    if ((T.flags & 1u) && p.enable_weight_decay) update += param * p.weight_decay / 2.0f;
    param -= update;
    T.parameters[j] = param;
    if (T.polyak_target) T.polyak_target[j] = rlt_polyak_value(polyak, T.polyak_target[j], param);
    return param;
}

// A load of data that a workgroup on another compute unit wrote earlier in the same launch. SAME_XCD: all workgroups of the launch
// share one L2, the writer's stores have completed there (s_waitcnt before it announced them) and a non-temporal load reads the L2
// without allocating in this compute unit's vector cache. Otherwise the writer released at agent scope and the load bypasses the
// caches that are not coherent across XCDs.
template <bool SAME_XCD>
__device__ __forceinline__ float rlt_load_shared(const float* p) {
    if (SAME_XCD) return __builtin_nontemporal_load(p);
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sum over `groups` blocks of element p[g * stride], for E elements at once, in the order of the small-MLP reduction kernel: four
// quarters of the blocks, each in block order from zero, then (q0 + q1) + (q2 + q3). With at most 16 blocks every load of the E
// elements is issued before the first addition.
template <int E, bool SAME_XCD>
__device__ __forceinline__ void rlt_sum_of_blocks(const float* const (&p)[E], int groups, int stride, float (&out)[E]) {
    const int per = (groups + 3) / 4;
    if (per <= 4) {
        float v[E][16];
#pragma unroll
        for (int e = 0; e < E; e++)
#pragma unroll
            for (int qi = 0; qi < 4; qi++)
#pragma unroll
                for (int u = 0; u < 4; u++) v[e][4 * qi + u] = rlt_load_shared<SAME_XCD>(p[e] + (size_t)min(qi * per + u, groups - 1) * stride);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int e = 0; e < E; e++) {
            float q[4];
#pragma unroll
            for (int qi = 0; qi < 4; qi++) {
                const int g0 = qi * per, g1 = min(groups, g0 + per);
                float s = 0.f;
#pragma unroll
                for (int u = 0; u < 4; u++) s += (u < per && g0 + u < g1) ? v[e][4 * qi + u] : 0.f;
                q[qi] = s;
            }
            out[e] = (q[0] + q[1]) + (q[2] + q[3]);
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < E; e++) {
        float q[4];
        for (int qi = 0; qi < 4; qi++) {
            const int g0 = qi * per, g1 = min(groups, g0 + per);
            float s = 0.f;
            for (int gb = g0; gb < g1; gb += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = rlt_load_shared<SAME_XCD>(p[e] + (size_t)min(gb + u, g1 - 1) * stride);
#pragma unroll
                for (int u = 0; u < 8; u++) s += (gb + u < g1) ? v[u] : 0.f;
            }
            q[qi] = s;
        }
        out[e] = (q[0] + q[1]) + (q[2] + q[3]);
    }
}

// An optimiser that a kernel steps itself once its last workgroup has written its block of partial gradient sums.
constexpr int RLT_TAIL_TENSORS = 12;
struct rlt_tail_optimizer {
    rlt_adam_tensor t[RLT_TAIL_TENSORS];
    uint32_t prefix[RLT_TAIL_TENSORS + 1];      // first element of tensor i in the optimiser's element numbering
    uint32_t offset[RLT_TAIL_TENSORS];          // where tensor i's gradient starts within a block
    float scale[RLT_TAIL_TENSORS];              // factor on its sums
    int n;
    rlt_adam_parameters p;
    uint32_t* age;
};
// the host side of it: false unless every tensor is complete
inline bool rlt_tail_optimizer_fill(rlt_tail_optimizer& O, const rlt_adam_tensor* tensors, int n, const uint32_t* offsets, const float* scales, const rlt_adam_parameters* p, uint32_t* age) {
    if (!tensors || n < 1 || n > RLT_TAIL_TENSORS || !p || !age) return false;
    uint32_t total = 0;
    for (int i = 0; i < n; i++) {
        const rlt_adam_tensor& T = tensors[i];
        if (!T.first_moment || !T.second_moment || !T.parameters || !T.gradient || T.count == 0) return false;
        O.t[i] = T; O.prefix[i] = total; total += T.count; O.offset[i] = offsets[i]; O.scale[i] = scales ? scales[i] : 1.0f;
    }
    for (int i = n; i <= RLT_TAIL_TENSORS; i++) O.prefix[i] = total;
    O.n = n; O.p = *p; O.age = age;
    return true;
}

// The step, by every thread of ONE workgroup of THREADS threads: gradients = sums of the blocks (stored), then Adam. The age is
// incremented by thread 0 after a workgroup barrier. Bit for bit what adam_kernel makes of the same blocks.
template <int THREADS, bool SAME_XCD>
__device__ __forceinline__ void rlt_tail_adam(const rlt_tail_optimizer& O, const float* partial, int groups, int block_stride, int tid) {
    const uint32_t age = *O.age;
    float bc1, bc2;
    rlt_adam_bias_corrections(O.p, age, bc1, bc2);
    const uint32_t total = O.prefix[O.n];
    constexpr int E = 3;
    for (uint32_t base = 0; base < total; base += E * THREADS) {
        int ti[E]; uint32_t j[E]; bool ok[E]; const float* src[E]; float g[E];
#pragma unroll
        for (int e = 0; e < E; e++) {
            const uint32_t i = base + e * THREADS + tid;
            ok[e] = i < total;
            const uint32_t ic = ok[e] ? i : 0u;
            int t = 0;
#pragma unroll
            for (int k = 1; k < RLT_TAIL_TENSORS; k++) t += (k < O.n && ic >= O.prefix[k]) ? 1 : 0;
            ti[e] = t; j[e] = ic - O.prefix[t];
            src[e] = partial + O.offset[t] + j[e];
        }
        rlt_sum_of_blocks<E, SAME_XCD>(src, groups, block_stride, g);
#pragma unroll
        for (int e = 0; e < E; e++)
            if (ok[e]) {
                const rlt_adam_tensor& T = O.t[ti[e]];
                const float ge = g[e] * O.scale[ti[e]];
                T.gradient[j[e]] = ge;
                rlt_adam_apply(O.p, T, j[e], ge, bc1, bc2, 0.0f);
            }
    }
    __syncthreads();        // every thread has read the age
    if (tid == 0) *O.age = age + 1;
}
