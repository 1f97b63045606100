// Adam step (moments, bias correction, parameter update, optional polyak target and gradient norm) for a list of
// parameter tensors in one launch, and the polyak soft update.
// reference: nn/optimizers/adam/operations_generic.h:43-66, instance/operations_generic.h:26-72,
//            utils/polyak/operations_generic.h:11-43; CUDA counterparts adam/operations_cuda.h:18-68 (scalar kernel for the
//            bias corrections), nn/layers/dense/operations_cuda.h:195-233 (one launch per layer).
#include "common.h"
#include "optim.h"

namespace {

constexpr int MAX_T = 12;
struct AdamLaunch {
    rlt_adam_tensor t[MAX_T];
    uint32_t prefix[MAX_T + 1];
    int n;
    rlt_adam_parameters p;
    float polyak;
    uint32_t* age;
    uint32_t* done_counter;      // zero between launches
    float* block_partials;       // [gridDim.x] sums of squared gradients
    float* out_sq_norm;          // optional
    int increment_age;
    int accumulate_norm;         // add to *out_sq_norm instead of overwriting (later chunks of one step)
    // optional: the gradients are still blocks of partial sums. Element j of tensor t is source_scale[t] times the sum over `groups`
    // blocks of `block_stride` floats of source[g * block_stride + source_offset[t] + j], added up in the order of the small-MLP
    // reduction kernel (four quarters of the blocks, each in block order, then (q0 + q1) + (q2 + q3)); it is stored in the tensor's
    // gradient before it is used
    const float* source;
    int groups, block_stride;
    uint32_t source_offset[MAX_T];
    float source_scale[MAX_T], source_add[MAX_T];
    float* extra_out; uint32_t extra_offset; float extra_scale;      // optional: one more sum of the blocks, stored scaled (not a gradient)
    uint32_t vec_end;            // elements [0, vec_end) can be stepped four at a time (16-byte loads of the blocks, moments and values): see vector_end()
};

// sum over the blocks of one element, every load in flight at once where there are at most 16 blocks
__device__ __forceinline__ float sum_of_blocks(const float* __restrict__ p, int groups, int stride) {
    const float* const src[1] = {p};
    float out[1];
    rlt_sum_of_blocks<1, 2>(src, groups, stride, out);
    return out[0];
}

// the step for one optimiser by workgroups [0, n_blocks) numbered `block`
__device__ __forceinline__ void adam_body(const AdamLaunch& a, uint32_t block, uint32_t n_blocks) {
    const uint32_t age = *a.age;
    // bias corrections from the un-incremented age (adam/operations_generic.h:49-58)
    float bc1, bc2;
    rlt_adam_bias_corrections(a.p, age, bc1, bc2);
    const uint32_t total = a.prefix[a.n];
    float sq = 0.0f;
    if (a.source && a.groups > 16) {
        // many blocks: 64 elements per pass of a workgroup, four threads per element each add up a quarter of the blocks (the order of
        // rlt_sum_of_blocks) with all of a quarter's loads of up to 32 blocks in flight at once
        __shared__ float quarter[4][64];
        const uint32_t el = threadIdx.x & 63u, qtr = threadIdx.x >> 6;
        const int per = (a.groups + 3) / 4, g0 = qtr * per, g1 = min(a.groups, g0 + per);
        for (uint32_t base = block * 64u; base < total; base += n_blocks * 64u) {
            const uint32_t i = min(base + el, total - 1u);
            int ti = 0;
#pragma unroll
            for (int k = 1; k < MAX_T; k++) ti += (k < a.n && i >= a.prefix[k]) ? 1 : 0;
            const uint32_t j = i - a.prefix[ti];
            const float* __restrict__ p = a.source + a.source_offset[ti] + j;
            // the element's moments and value travel while the blocks are added up
            const rlt_adam_tensor& T = a.t[ti];
            float m = 0.f, v2 = 0.f, param = 0.f, target = 0.f;
            if (qtr == 0) { m = T.first_moment[j]; v2 = T.second_moment[j]; param = T.parameters[j]; if (T.polyak_target) target = T.polyak_target[j]; }
            float s = 0.f;
            int gb = g0;
            for (; g1 - gb > 8; gb += 32) {
                float v[32];
#pragma unroll
                for (int u = 0; u < 32; u++) v[u] = p[(size_t)min(gb + u, g1 - 1) * a.block_stride];
#pragma unroll
                for (int u = 0; u < 32; u++) s += (gb + u < g1) ? v[u] : 0.f;
            }
            for (; gb < g1; gb += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = p[(size_t)min(gb + u, g1 - 1) * a.block_stride];
#pragma unroll
                for (int u = 0; u < 8; u++) s += (gb + u < g1) ? v[u] : 0.f;
            }
            quarter[qtr][el] = s;
            __syncthreads();
            if (qtr == 0 && base + el < total) {
                const float g = rlt_scaled_sum((quarter[0][el] + quarter[1][el]) + (quarter[2][el] + quarter[3][el]), a.source_scale[ti], a.source_add[ti]);
                T.gradient[j] = g;
                sq += g * g;
                rlt_adam_values(a.p, T.flags, g, bc1, bc2, m, v2, param);
                T.first_moment[j] = m; T.second_moment[j] = v2; T.parameters[j] = param;
                if (T.polyak_target) T.polyak_target[j] = rlt_polyak_value(a.polyak, target, param);
            }
            __syncthreads();
        }
    } else {
    // at most 16 blocks, four neighbouring elements per thread: every load is 16 bytes per lane (the same sums in the same order per element)
    typedef float f4 __attribute__((ext_vector_type(4)));
    for (uint32_t i = (block * blockDim.x + threadIdx.x) * 4u; i < a.vec_end; i += n_blocks * blockDim.x * 4u) {
        int ti = 0;
#pragma unroll
        for (int k = 1; k < MAX_T; k++) ti += (k < a.n && i >= a.prefix[k]) ? 1 : 0;
        const rlt_adam_tensor& T = a.t[ti];
        const uint32_t j = i - a.prefix[ti];
        f4 m = *reinterpret_cast<const f4*>(T.first_moment + j), v = *reinterpret_cast<const f4*>(T.second_moment + j), param = *reinterpret_cast<const f4*>(T.parameters + j);
        f4 target = {0.f, 0.f, 0.f, 0.f};
        if (T.polyak_target) target = *reinterpret_cast<const f4*>(T.polyak_target + j);
        const float* __restrict__ p = a.source + a.source_offset[ti] + j;
        const int per = (a.groups + 3) / 4;
        f4 blk[16];
#pragma unroll
        for (int qi = 0; qi < 4; qi++)
#pragma unroll
            for (int u = 0; u < 4; u++) blk[4 * qi + u] = *reinterpret_cast<const f4*>(p + (size_t)min(qi * per + u, a.groups - 1) * a.block_stride);
        __builtin_amdgcn_sched_barrier(0);
        f4 q[4];
#pragma unroll
        for (int qi = 0; qi < 4; qi++) {
            const int g0 = qi * per, g1 = min(a.groups, g0 + per);
            f4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < 4; u++) if (u < per && g0 + u < g1) sum += blk[4 * qi + u];
            q[qi] = sum;
        }
        const f4 total4 = (q[0] + q[1]) + (q[2] + q[3]);
        f4 g;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            g[c] = rlt_scaled_sum(total4[c], a.source_scale[ti], a.source_add[ti]);
            sq += g[c] * g[c];
            float mc = m[c], vc = v[c], pc = param[c];
            rlt_adam_values(a.p, T.flags, g[c], bc1, bc2, mc, vc, pc);
            m[c] = mc; v[c] = vc; param[c] = pc;
            if (T.polyak_target) target[c] = rlt_polyak_value(a.polyak, target[c], pc);
        }
        *reinterpret_cast<f4*>(T.gradient + j) = g;
        *reinterpret_cast<f4*>(T.first_moment + j) = m; *reinterpret_cast<f4*>(T.second_moment + j) = v; *reinterpret_cast<f4*>(T.parameters + j) = param;
        if (T.polyak_target) *reinterpret_cast<f4*>(T.polyak_target + j) = target;
    }
    for (uint32_t i = a.vec_end + block * blockDim.x + threadIdx.x; i < total; i += n_blocks * blockDim.x) {
        int ti = 0;
#pragma unroll
        for (int k = 1; k < MAX_T; k++) ti += (k < a.n && i >= a.prefix[k]) ? 1 : 0;
        const rlt_adam_tensor& T = a.t[ti];
        const uint32_t j = i - a.prefix[ti];
        // the element's moments, value and target travel together with its gradient (or the blocks that add up to it)
        float m = T.first_moment[j], v = T.second_moment[j], param = T.parameters[j];
        const float target = T.polyak_target ? T.polyak_target[j] : 0.f;
        float g;
        if (a.source) {
            g = rlt_scaled_sum(sum_of_blocks(a.source + a.source_offset[ti] + j, a.groups, a.block_stride), a.source_scale[ti], a.source_add[ti]);
            T.gradient[j] = g;
        } else g = T.gradient[j];
        sq += g * g;
        rlt_adam_values(a.p, T.flags, g, bc1, bc2, m, v, param);
        T.first_moment[j] = m; T.second_moment[j] = v; T.parameters[j] = param;
        if (T.polyak_target) T.polyak_target[j] = rlt_polyak_value(a.polyak, target, param);
    }
    }
    if (a.extra_out && block == n_blocks - 1 && threadIdx.x == blockDim.x - 1) *a.extra_out = sum_of_blocks(a.source + a.extra_offset, a.groups, a.block_stride) * a.extra_scale;
    // gradient norm + age increment: the last workgroup to finish has seen every other one read `age`
    __shared__ float partial[4];
    __shared__ bool last;
    sq = rlt_wave_sum(sq);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sq;
    __syncthreads();
    if (threadIdx.x == 0) {
        a.block_partials[block] = partial[0] + partial[1] + partial[2] + partial[3];
        __threadfence();
        uint32_t ticket = atomicAdd(a.done_counter, 1u);
        last = (ticket == n_blocks - 1);
    }
    __syncthreads();
    if (last && threadIdx.x == 0) {
        __threadfence();
        if (a.out_sq_norm) {
            float s = a.accumulate_norm ? *a.out_sq_norm : 0.0f;
            for (uint32_t b = 0; b < n_blocks; b++) s += ((volatile float*)a.block_partials)[b];
            *a.out_sq_norm = s;
        }
        if (a.increment_age) *a.age = age + 1;
        *a.done_counter = 0;
    }
}

__global__ __launch_bounds__(256) void adam_kernel(AdamLaunch a) { adam_body(a, blockIdx.x, gridDim.x); }
// two optimisers in one launch: workgroups [0, blocks_a) take the first
__global__ __launch_bounds__(256) void adam_pair_kernel(AdamLaunch a, AdamLaunch b, uint32_t blocks_a) {
    if (blockIdx.x < blocks_a) adam_body(a, blockIdx.x, blocks_a);
    else adam_body(b, blockIdx.x - blocks_a, gridDim.x - blocks_a);
}

__global__ __launch_bounds__(256) void adam_reset_kernel(AdamLaunch a) {
    const uint32_t total = a.prefix[a.n];
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        int ti = 0;
#pragma unroll
        for (int k = 1; k < MAX_T; k++) ti += (k < a.n && i >= a.prefix[k]) ? 1 : 0;
        const uint32_t j = i - a.prefix[ti];
        a.t[ti].first_moment[j] = 0.0f; a.t[ti].second_moment[j] = 0.0f;
    }
    if (a.increment_age && blockIdx.x == 0 && threadIdx.x == 0) *a.age = 1;
}

__global__ __launch_bounds__(256) void polyak_kernel(const float* __restrict__ source, float* __restrict__ target, size_t count, float polyak, int squared) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
        float s = source[i];
        target[i] = squared ? polyak * target[i] + (1.0f - polyak) * s * s : rlt_polyak_value(polyak, target[i], s);
    }
}

}  // namespace

// Layout of the device handle's scratch for this file: [0,256) the done counter, [256, ...) block partials.
static int adam_launch(rlt_rocm_device* device, const rlt_adam_tensor* tensors, int n_tensors, const rlt_adam_parameters* p, uint32_t* age,
                       float polyak, float* out_sq_norm, bool reset) {
    void* counters = nullptr;
    int rc = rlt_counters(device, &counters);
    if (rc) return rc;
    for (int base = 0; base < n_tensors; base += MAX_T) {
        AdamLaunch a = {};
        a.n = n_tensors - base < MAX_T ? n_tensors - base : MAX_T;
        uint32_t total = 0;
        for (int i = 0; i < a.n; i++) {
            const rlt_adam_tensor& T = tensors[base + i];
            if (!T.first_moment || !T.second_moment || (!reset && (!T.parameters || !T.gradient)) || T.count == 0) return RLT_E_INVALID_ARGUMENT;
            a.t[i] = T; a.prefix[i] = total; total += T.count;
        }
        for (int i = a.n; i <= MAX_T; i++) a.prefix[i] = total;
        if (p) a.p = *p;
        a.polyak = polyak; a.age = age;
        a.done_counter = (uint32_t*)counters; a.block_partials = (float*)((char*)counters + 256);
        a.out_sq_norm = out_sq_norm; a.accumulate_norm = base > 0;
        a.increment_age = (base + MAX_T >= n_tensors);
        int blocks = (int)((total + 255) / 256); if (blocks > 960) blocks = 960; if (blocks < 1) blocks = 1;
        if (reset) hipLaunchKernelGGL(adam_reset_kernel, dim3(blocks), dim3(256), 0, device->stream, a);
        else hipLaunchKernelGGL(adam_kernel, dim3(blocks), dim3(256), 0, device->stream, a);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    return 0;
}

// how far the elements can be stepped four at a time: up to the first tensor whose start, pointers or place in the blocks is not a multiple of 16 bytes, or that
// ends off one (then its last one to three elements and everything behind them are stepped one by one)
static uint32_t vector_end(const AdamLaunch& a) {
    auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    if (!a.source || a.groups > 16 || a.block_stride % 4 != 0 || !aligned(a.source)) return 0;
    uint32_t end = 0;
    for (int i = 0; i < a.n; i++) {
        const rlt_adam_tensor& T = a.t[i];
        if (a.prefix[i] % 4 != 0 || a.source_offset[i] % 4 != 0 || !aligned(T.parameters) || !aligned(T.gradient) || !aligned(T.first_moment) || !aligned(T.second_moment) ||
            (T.polyak_target && !aligned(T.polyak_target))) break;
        end = a.prefix[i] + (T.count & ~3u);
        if (T.count % 4 != 0) break;
    }
    return end;
}
static void set_source(AdamLaunch& a, const rlt_adam_source* source) {
    if (!source) return;
    a.source = source->partial; a.groups = source->groups; a.block_stride = source->block_stride;
    for (int i = 0; i < a.n; i++) { a.source_offset[i] = source->offsets[i]; a.source_scale[i] = source->scales[i]; a.source_add[i] = source->adds ? source->adds[i] : 0.0f; }
    a.extra_out = source->extra_out; a.extra_offset = source->extra_offset; a.extra_scale = source->extra_scale;
    a.vec_end = vector_end(a);
}
// workgroups for an optimiser of `total` elements: 64 elements per workgroup pass on the many-block path, 256 threads of four elements each where those apply
static uint32_t blocks_for(const AdamLaunch& a, uint32_t total, const rlt_adam_source* source) {
    if (source && source->groups > 16) return (total + 63) / 64;
    const uint32_t threads = a.vec_end / 4 > total - a.vec_end ? a.vec_end / 4 : total - a.vec_end;
    return (threads + 255) / 256;
}

int rlt_adam_step_from_partials(rlt_rocm_device* device, const rlt_adam_tensor* tensors, int n, const rlt_adam_parameters* parameters, uint32_t* age, const rlt_adam_source* source, float polyak) {
    RLT_REQUIRE(tensors && n > 0 && n <= MAX_T && parameters && age && source && source->partial && source->groups > 0);
    void* counters = nullptr;
    int rc = rlt_counters(device, &counters);
    if (rc) return rc;
    AdamLaunch a = {};
    a.n = n;
    uint32_t total = 0;
    for (int i = 0; i < n; i++) {
        const rlt_adam_tensor& T = tensors[i];
        if (!T.first_moment || !T.second_moment || !T.parameters || !T.gradient || T.count == 0) return RLT_E_INVALID_ARGUMENT;
        a.t[i] = T; a.prefix[i] = total; total += T.count;
    }
    for (int i = n; i <= MAX_T; i++) a.prefix[i] = total;
    a.p = *parameters; a.age = age; a.polyak = polyak;
    a.done_counter = (uint32_t*)counters; a.block_partials = (float*)((char*)counters + 256);
    a.increment_age = 1;
    set_source(a, source);
    int blocks = (int)blocks_for(a, total, source); if (blocks > 960) blocks = 960; if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(adam_kernel, dim3(blocks), dim3(256), 0, device->stream, a);
    return rlt_launch_status(device);
}

int rlt_adam_step_pair(rlt_rocm_device* device, const rlt_adam_tensor* tensors_a, int n_a, const rlt_adam_parameters* parameters_a, uint32_t* age_a,
                       const rlt_adam_tensor* tensors_b, int n_b, const rlt_adam_parameters* parameters_b, uint32_t* age_b,
                       const rlt_adam_source* source_a, const rlt_adam_source* source_b, float polyak) {
    RLT_REQUIRE(tensors_a && tensors_b && n_a > 0 && n_b > 0 && parameters_a && parameters_b && age_a && age_b);
    if (n_a > MAX_T || n_b > MAX_T) {
        RLT_REQUIRE(!source_a && !source_b);
        const int rc = adam_launch(device, tensors_a, n_a, parameters_a, age_a, 0.0f, nullptr, false);
        return rc ? rc : adam_launch(device, tensors_b, n_b, parameters_b, age_b, 0.0f, nullptr, false);
    }
    void* counters = nullptr;
    int rc = rlt_counters(device, &counters);
    if (rc) return rc;
    AdamLaunch L[2] = {};
    uint32_t blocks[2];
    for (int k = 0; k < 2; k++) {
        AdamLaunch& a = L[k];
        const rlt_adam_tensor* tensors = k ? tensors_b : tensors_a;
        a.n = k ? n_b : n_a;
        uint32_t total = 0;
        for (int i = 0; i < a.n; i++) {
            const rlt_adam_tensor& T = tensors[i];
            if (!T.first_moment || !T.second_moment || !T.parameters || !T.gradient || T.count == 0) return RLT_E_INVALID_ARGUMENT;
            a.t[i] = T; a.prefix[i] = total; total += T.count;
        }
        for (int i = a.n; i <= MAX_T; i++) a.prefix[i] = total;
        a.p = k ? *parameters_b : *parameters_a;
        a.age = k ? age_b : age_a; a.polyak = polyak;
        // the second optimiser's ticket counter and partial sums sit in their own part of the counters block
        a.done_counter = (uint32_t*)((char*)counters + (k ? 64 : 0)); a.block_partials = (float*)((char*)counters + 256) + (k ? 480 : 0);
        a.increment_age = 1;
        const rlt_adam_source* source = k ? source_b : source_a;
        set_source(a, source);
        blocks[k] = blocks_for(a, total, source); if (blocks[k] > 480) blocks[k] = 480; if (blocks[k] < 1) blocks[k] = 1;
    }
    hipLaunchKernelGGL(adam_pair_kernel, dim3(blocks[0] + blocks[1]), dim3(256), 0, device->stream, L[0], L[1], blocks[0]);
    return rlt_launch_status(device);
}

extern "C" {

int rlt_rocm_adam_step(rlt_rocm_device* device, const rlt_adam_tensor* tensors_host, int n_tensors, const rlt_adam_parameters* parameters_host,
                       uint32_t* age, float polyak, float* out_gradient_squared_norm) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(tensors_host && n_tensors > 0 && parameters_host && age);
    return adam_launch(device, tensors_host, n_tensors, parameters_host, age, polyak, out_gradient_squared_norm, false);
}
int rlt_rocm_adam_reset(rlt_rocm_device* device, const rlt_adam_tensor* tensors_host, int n_tensors, uint32_t* age) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(tensors_host && n_tensors > 0 && age);
    return adam_launch(device, tensors_host, n_tensors, nullptr, age, 0.0f, nullptr, true);
}
int rlt_rocm_polyak_update(rlt_rocm_device* device, const float* source, float* target, size_t count, float polyak, int squared) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(source && target);
    if (count == 0) return 0;
    size_t b = (count + 255) / 256; if (b > 960) b = 960;
    hipLaunchKernelGGL(polyak_kernel, dim3((int)b), dim3(256), 0, device->stream, source, target, count, polyak, squared);
    return rlt_launch_status(device);
}

}  // extern "C"
