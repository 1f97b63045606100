// Internal entry points of optim.hip, and the optimiser's arithmetic as device functions for the kernels that step a network at
// the end of the launch that produced its gradients.
#pragma once
#include "common.h"

// Gradients that are still blocks of partial sums (one block of `block_stride` floats per workgroup of the kernel that made them): the
// optimiser's launch adds them up, in the order of the small-MLP reduction kernel, stores the sums in the tensors' gradients and steps.
// offsets[t]: where tensor t's gradient starts within a block; scales[t]: factor on its sums; adds[t] (optional array): added after scaling.
// extra_out (optional): one more sum of the blocks, at extra_offset, times extra_scale, stored there (a loss that the kernel summed per block).
struct rlt_adam_source { const float* partial; int groups, block_stride; const uint32_t* offsets; const float* scales; const float* adds; float* extra_out; uint32_t extra_offset; float extra_scale; };

// rlt_rocm_adam_step for at most 12 tensors whose gradients are blocks of partial sums
int rlt_adam_step_from_partials(rlt_rocm_device* device, const rlt_adam_tensor* tensors, int n, const rlt_adam_parameters* parameters, uint32_t* age, const rlt_adam_source* source,
                                float polyak = 0.0f);

// rlt_rocm_adam_step for two optimisers (each with its own tensors, parameters and age) in one launch; each list at most 12 tensors
// where a source is given
int rlt_adam_step_pair(rlt_rocm_device* device, const rlt_adam_tensor* tensors_a, int n_a, const rlt_adam_parameters* parameters_a, uint32_t* age_a,
                       const rlt_adam_tensor* tensors_b, int n_b, const rlt_adam_parameters* parameters_b, uint32_t* age_b,
                       const rlt_adam_source* source_a = nullptr, const rlt_adam_source* source_b = nullptr, float polyak = 0.0f);      // polyak: for tensors that name a polyak_target

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

// a gradient from its summed partial values: the product is rounded before the sum in every kernel, so that all of them leave the same bits
__device__ __forceinline__ float rlt_scaled_sum(float sum, float scale, float add) {
#pragma clang fp contract(off)
    const float a = sum * scale;
    return a + add;
}

// 1 / (1 - beta^age) for both moments (nn/optimizers/adam/operations_generic.h:49-58: from the age before the step)
__device__ __forceinline__ void rlt_adam_bias_corrections(const rlt_adam_parameters& p, uint32_t age, float& bc1, float& bc2) {
    bc1 = 1.0f / (1.0f - powf(p.beta_1, (float)age));
    bc2 = 1.0f / (1.0f - powf(p.beta_2, (float)age));
}

// The arithmetic of one element (nn/optimizers/adam/instance/operations_generic.h:26-72): moments m, v and the parameter are updated in place
__device__ __forceinline__ void rlt_adam_values(const rlt_adam_parameters& p, uint32_t flags, float g, float bc1, float bc2, float& m, float& v, float& param) {
#pragma clang fp contract(off)      // no product is fused into a sum: every kernel that inlines this leaves the same bits
    if (p.enable_gradient_clipping) g = fminf(fmaxf(g, -p.gradient_clip_value), p.gradient_clip_value);
    m = p.beta_1 * m + (1.0f - p.beta_1) * g;
    v = p.beta_2 * v + (1.0f - p.beta_2) * g * g;
    float pre_sqrt = fmaxf(v * bc2, p.epsilon_sqrt);
    float update = p.alpha * bc1 * m / (sqrtf(pre_sqrt) + p.epsilon);
    if ((flags & 2u) && p.enable_bias_lr_factor) update *= p.bias_lr_factor;
    if ((flags & 1u) && p.enable_weight_decay) update += param * p.weight_decay / 2.0f;
    param -= update;
}
// One element of a tensor: moments, step, optional fused soft update of a target. Returns the new parameter value.
__device__ __forceinline__ float rlt_adam_apply(const rlt_adam_parameters& p, const rlt_adam_tensor& T, uint32_t j, float g, float bc1, float bc2, float polyak) {
    float m = T.first_moment[j], v = T.second_moment[j], param = T.parameters[j];
    rlt_adam_values(p, T.flags, g, bc1, bc2, m, v, param);
    T.first_moment[j] = m; T.second_moment[j] = v;
    T.parameters[j] = param;
    if (T.polyak_target) T.polyak_target[j] = rlt_polyak_value(polyak, T.polyak_target[j], param);
    return param;
}

// A load of data that a workgroup on another compute unit wrote. KIND 1 (same launch, same XCD): all workgroups of the launch share one
// L2, the writer's stores have completed there (s_waitcnt before it announced them) and a non-temporal load reads the L2 without
// allocating in this compute unit's vector cache. KIND 0 (same launch, any XCD): the writer released at agent scope and the load
// bypasses the caches that are not coherent across XCDs. KIND 2 (an earlier launch): a plain load.
template <int KIND>
__device__ __forceinline__ float rlt_load_shared(const float* p) {
    if (KIND == 1) return __builtin_nontemporal_load(p);
    if (KIND == 2) return *p;
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sum over `groups` blocks of element p[g * stride], for E elements at once, in the order of the small-MLP reduction kernel: four
// quarters of the blocks, each in block order from zero, then (q0 + q1) + (q2 + q3). With at most 16 blocks every load of the E
// elements is issued before the first addition.
template <int E, int SAME_XCD>
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

// ---- The optimiser's step as the last part of the kernel that produced the gradients.
// Every workgroup of the launch has written a block of partial sums [.. | extra] (block b of trained network y at
// partial + (y * G + b) * count). It announces the block (tickets[0]), waits until all workgroups of the launch have, and steps a
// slice of its trained network's elements: sum over the blocks in the order of the small-MLP reduction kernel, Adam, and the soft
// update of a target where a tensor names one (opt[].t[].polyak_target; targets are read by every workgroup of the launch, hence the
// wait for all of them). The grid must be resident as a whole: the host only asks for this with at most RLT_TAIL_MAX_WORKGROUPS
// workgroups. The wait is bounded; a workgroup that gives up sets *fault and leaves its slice undone. tickets[1] counts the workgroups
// that are through; the last one clears both words (they are zero between launches) and advances the ages.
// same_xcd: the working workgroups share one XCD (see rlt_load_shared).
constexpr int RLT_TAIL_MAX_WORKGROUPS = 64;
struct rlt_tail_args {
    int enabled, same_xcd;
    unsigned max_poll;                               // polls after which a waiting workgroup gives up (the device handle's wait limit)
    uint32_t* tickets; unsigned* fault;
    const float* partial; int count;                 // blocks of `count` floats
    rlt_tail_optimizer opt[2];                       // per trained network of the launch (blockIdx.y)
    float polyak;
    int has_second, second_offset;                   // a scalar whose gradient is block element second_offset times second_scale (log_alpha)
    rlt_adam_tensor second; rlt_adam_parameters second_p; uint32_t* second_age; float second_scale;
    unsigned long long* ticks;                       // optional (profiling builds): [0] workgroup 0's clock after the wait, [1] after its slice
};
// The kernels hand over their own arguments where they lie in the argument segment: constant address space, so that reads of them are
// scalar loads that no store can invalidate (through a generic pointer every read is a vector load the compiler has to wait for and to
// repeat after every store).
#define RLT_CONSTANT __attribute__((address_space(4)))
typedef const RLT_CONSTANT rlt_tail_args* rlt_tail_pointer;
__device__ __forceinline__ rlt_adam_parameters rlt_read_parameters(const RLT_CONSTANT rlt_adam_parameters* p) {
    rlt_adam_parameters q;
    q.alpha = p->alpha; q.beta_1 = p->beta_1; q.beta_2 = p->beta_2; q.epsilon = p->epsilon; q.epsilon_sqrt = p->epsilon_sqrt; q.weight_decay = p->weight_decay;
    q.bias_lr_factor = p->bias_lr_factor; q.enable_weight_decay = p->enable_weight_decay; q.enable_bias_lr_factor = p->enable_bias_lr_factor;
    q.enable_gradient_clipping = p->enable_gradient_clipping; q.gradient_clip_value = p->gradient_clip_value;
    return q;
}
// The slice of workgroup g: one element per thread and pass (slices are a few hundred elements: the kernels that end this way have
// small networks), the element's tensor looked up per lane, every load of a pass requested before the first is used.
template <int THREADS, bool SAME_XCD>
__device__ __forceinline__ void rlt_tail_slice(rlt_tail_pointer A, int y, int g, int G) {
    const RLT_CONSTANT rlt_tail_optimizer* O = &A->opt[y];
    const rlt_adam_parameters P = rlt_read_parameters(&O->p);
    const int count = A->count, n_tensors = O->n;
    const float polyak = A->polyak;
    const float* blocks = A->partial + (size_t)y * G * count;
    const uint32_t n = O->prefix[n_tensors], chunk = (n + G - 1) / G, begin = min(n, (uint32_t)g * chunk), end = min(n, begin + chunk);
    float bc1, bc2;
    rlt_adam_bias_corrections(P, *O->age, bc1, bc2);
    for (uint32_t base = begin; base < end; base += THREADS) {
        const uint32_t i = base + threadIdx.x;
        const bool ok = i < end;
        const uint32_t ic = ok ? i : begin;
        int t = 0;
#pragma unroll
        for (int k = 1; k < RLT_TAIL_TENSORS; k++) t += (k < n_tensors && ic >= O->prefix[k]) ? 1 : 0;
        const uint32_t j = ic - O->prefix[t];
        const RLT_CONSTANT rlt_adam_tensor* T = &O->t[t];
        float* const gp = T->gradient + j; float* const mp = T->first_moment + j; float* const vp = T->second_moment + j; float* const pp = T->parameters + j;
        float* const tp = T->polyak_target ? T->polyak_target + j : nullptr;
        const uint32_t flags = T->flags;
        const float scale = O->scale[t];
        const float* const src[1] = {blocks + O->offset[t] + j};
        float m = *mp, v = *vp, param = *pp;
        const float target = tp ? *tp : 0.f;
        float gs[1];
        rlt_sum_of_blocks<1, SAME_XCD>(src, G, count, gs);
        if (ok) {
            const float ge = gs[0] * scale;
            rlt_adam_values(P, flags, ge, bc1, bc2, m, v, param);
            *gp = ge; *mp = m; *vp = v; *pp = param;
            if (tp) *tp = rlt_polyak_value(polyak, target, param);
        }
    }
    if (A->has_second && g == G - 1 && threadIdx.x == THREADS - 1) {
        const float* const src[1] = {blocks + A->second_offset};
        float gs[1];
        rlt_sum_of_blocks<1, SAME_XCD>(src, G, count, gs);
        const rlt_adam_parameters Q = rlt_read_parameters(&A->second_p);
        const rlt_adam_tensor T = {A->second.parameters, A->second.gradient, A->second.first_moment, A->second.second_moment, nullptr, 1u, A->second.flags};
        float b1, b2;
        rlt_adam_bias_corrections(Q, *A->second_age, b1, b2);
        const float ge = gs[0] * A->second_scale;
        T.gradient[0] = ge;
        rlt_adam_apply(Q, T, 0, ge, b1, b2, 0.0f);
    }
}
// Called by every thread of every working workgroup after its last store of partial sums. `flag_word`: one LDS word of the workgroup.
// A: the tail's arguments inside the calling kernel's argument segment.
template <int THREADS>
__device__ __noinline__ void rlt_optimiser_tail(rlt_tail_pointer A, int y, int g, int G, __attribute__((address_space(3))) int* flag_word) {
    const unsigned total = (unsigned)G * gridDim.y;
    const int same_xcd = A->same_xcd;
    const unsigned max_poll = A->max_poll;
    uint32_t* const tickets = A->tickets;
    unsigned* const fault = A->fault;
    unsigned long long* const ticks = A->ticks;
    __builtin_amdgcn_s_waitcnt(0);            // this wavefront's stores have completed
    if (!same_xcd) __threadfence();           // and are visible beyond this XCD
    __syncthreads();
    if (threadIdx.x == 0) {
        // the last workgroup to arrive learns so from its own ticket and goes on at once; every other one sleeps, then looks at the
        // word, at most max_poll - 1 times (a bound of one poll makes all but the last give up without looking)
        int ok = 1;
        if (__hip_atomic_fetch_add(tickets, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u < total) {
            unsigned tries = 0;
            do {
                if (++tries >= max_poll || ((tries & 63u) == 0u && __hip_atomic_load(fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                    __hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ok = 0;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            } while (__hip_atomic_load(tickets, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < total);
        }
        *flag_word = ok;
    }
    __syncthreads();
    if (ticks && g == 0 && y == 0 && threadIdx.x == 0) ticks[0] = wall_clock64();
    if (*flag_word) {
        if (same_xcd) rlt_tail_slice<THREADS, true>(A, y, g, G);
        else { __threadfence(); rlt_tail_slice<THREADS, false>(A, y, g, G); }
    }
    __syncthreads();        // every thread has read the ages it needs
    if (ticks && g == 0 && y == 0 && threadIdx.x == 0) ticks[1] = wall_clock64();
    if (threadIdx.x == 0 && __hip_atomic_fetch_add(tickets + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == total - 1) {
        // the last workgroup through: nobody waits on the words any more, and every slice has been stepped with the old ages
        __hip_atomic_store(tickets, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(tickets + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (unsigned k = 0; k < gridDim.y; k++) *A->opt[k].age += 1;
        if (A->has_second) *A->second_age += 1;
    }
}
