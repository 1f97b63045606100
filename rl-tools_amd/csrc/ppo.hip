// PPO: generalized advantage estimation and the minibatch update.
// reference: rl/algorithms/ppo/operations_generic.h:60-95 (GAE: serial double loop on the host; rows are step-major,
// row = step * n_envs + env, rl/components/on_policy_runner/on_policy_runner.h:38-72) and :96-330 (train: per-sample loops on the
// host around the networks' forward / backward passes).
#include "common.h"
#include <cstdlib>
#include "mlp_small.h"
#include "pad.h"
#include "optim.h"

namespace {
// Generalized advantage estimation as a two-level reverse scan. The recurrence over the steps of one environment,
//     A_t = c_t A_{t+1} + d_t,   c_t = lambda gamma (0 where step t is truncated),   d_t = r_t + gamma V_{t+1} [not terminated] - V_t (0 where truncated but not terminated),
// is linear in A_{t+1}, so a run of steps composes into one pair (a, b) with A_first = a A_in + b. A thread takes GAE_CHUNK consecutive steps of one
// environment: all its loads are independent of the recurrence and are in flight together (the dataset is step-major: row = step * n_envs + env, so at
// a fixed step the lanes of neighbouring environments read neighbouring rows). It scans its chunk from zero, keeping per step the advantage so far and
// the product of the coefficients up to the chunk's end; the chunks of an environment are then chained through LDS, and every step adds its product
// times the advantage that enters its chunk. One round trip to memory instead of one per step.
constexpr int GAE_THREADS = 256;
template <int GAE_CHUNK>
__global__ __launch_bounds__(GAE_THREADS) void gae_kernel(const float* __restrict__ rewards, const float* __restrict__ terminated, const float* __restrict__ truncated,
                                                          const float* __restrict__ all_values, float* __restrict__ advantages, float* __restrict__ target_values,
                                                          int ld, int n_envs, int steps, float gamma, float lambda, int ignore_termination, int n_chunks, int envs_per_block) {
    __shared__ float chunk_b[GAE_THREADS], chunk_a[GAE_THREADS];      // per (chunk, environment): advantage at the chunk's first step for zero input, and its coefficient product
    const int chunk = threadIdx.x / envs_per_block, env_local = threadIdx.x - chunk * envs_per_block;
    const int env = blockIdx.x * envs_per_block + env_local;
    const bool live = chunk < n_chunks && env < n_envs;
    const int first = chunk * GAE_CHUNK;                             // steps [first, first + count) in forward numbering
    const int count = live ? min(GAE_CHUNK, steps - first) : 0;
    float value[GAE_CHUNK + 1], reward[GAE_CHUNK], term[GAE_CHUNK], trunc[GAE_CHUNK];
#pragma unroll
    for (int j = 0; j < GAE_CHUNK; j++) {
        const bool in = j < count;
        const size_t pos = ((size_t)(first + (in ? j : 0)) * n_envs + (live ? env : 0)) * ld;
        value[j] = in ? all_values[pos] : 0.f; reward[j] = in ? rewards[pos] : 0.f; term[j] = in ? terminated[pos] : 0.f; trunc[j] = in ? truncated[pos] : 0.f;
    }
    // the value that follows the chunk's last step: the next chunk's first row, or the bootstrap row after the last step
    float value_after = live ? all_values[((size_t)(first + count) * n_envs + env) * ld] : 0.f;
    float adv[GAE_CHUNK], prod[GAE_CHUNK];
    float previous_advantage = 0.f, previous_value = value_after, product = 1.f;
#pragma unroll
    for (int j = GAE_CHUNK - 1; j >= 0; j--) {
        if (j < count) {
            const bool tm = term[j] != 0.f, tr = trunc[j] != 0.f;
            const float next_value = (tm && !ignore_termination) ? 0.f : previous_value;
            float td_error = reward[j] + gamma * next_value - value[j];
            float coefficient = lambda * gamma;
            if (tr) { if (!tm) td_error = 0.f; previous_advantage = 0.f; coefficient = 0.f; }
            const float advantage = lambda * gamma * previous_advantage + td_error;
            product *= coefficient;
            adv[j] = advantage; prod[j] = product;
            previous_advantage = advantage; previous_value = value[j];
        } else { adv[j] = 0.f; prod[j] = 0.f; }
    }
    chunk_b[threadIdx.x] = previous_advantage; chunk_a[threadIdx.x] = product;
    __syncthreads();
    // the advantage that enters this chunk: chain the later chunks of the same environment, last one first
    float incoming = 0.f;
    if (live) for (int k = n_chunks - 1; k > chunk; k--) incoming = chunk_b[k * envs_per_block + env_local] + chunk_a[k * envs_per_block + env_local] * incoming;
#pragma unroll
    for (int j = 0; j < GAE_CHUNK; j++) {
        if (j < count) {
            const size_t pos = ((size_t)(first + j) * n_envs + env) * ld;
            const float advantage = adv[j] + prod[j] * incoming;
            advantages[pos] = advantage;
            target_values[pos] = advantage + value[j];
        }
    }
}
// one lane per environment, serial over the steps (any number of steps)
__global__ __launch_bounds__(64) void gae_serial_kernel(const float* __restrict__ rewards, const float* __restrict__ terminated, const float* __restrict__ truncated,
                                                       const float* __restrict__ all_values, float* __restrict__ advantages, float* __restrict__ target_values,
                                                       int ld, int n_envs, int steps, float gamma, float lambda, int ignore_termination) {
    for (int env = blockIdx.x * blockDim.x + threadIdx.x; env < n_envs; env += gridDim.x * blockDim.x) {
        float previous_value = all_values[((size_t)steps * n_envs + env) * ld];
        float previous_advantage = 0.0f;
        for (int s = steps - 1; s >= 0; s--) {
            const size_t pos = ((size_t)s * n_envs + env) * ld;
            const bool term = terminated[pos] != 0.0f, trunc = truncated[pos] != 0.0f;
            const float value = all_values[pos];
            const float next_value = (term && !ignore_termination) ? 0.0f : previous_value;
            float td_error = rewards[pos] + gamma * next_value - value;
            if (trunc) { if (!term) td_error = 0.0f; previous_advantage = 0.0f; }
            const float advantage = lambda * gamma * previous_advantage + td_error;
            advantages[pos] = advantage;
            target_values[pos] = advantage + value;
            previous_advantage = advantage;
            previous_value = value;
        }
    }
}

// ---- minibatch update (train(), rl/algorithms/ppo/operations_generic.h:156-318)

// rows of the dataset selected by row_indices (or [0, batch)) into packed minibatch buffers; 16 lanes per row
__global__ __launch_bounds__(256) void ppo_gather_kernel(const float* __restrict__ observations, const float* __restrict__ observations_privileged,
                                                         const float* __restrict__ actions, const float* __restrict__ log_probs, const float* __restrict__ advantages,
                                                         const float* __restrict__ targets, int ld, const uint32_t* __restrict__ row_indices, int batch, int O, int OP, int A,
                                                         float* __restrict__ obs, float* __restrict__ obsp, float* __restrict__ act, float* __restrict__ lp,
                                                         float* __restrict__ adv, float* __restrict__ tgt,
                                                         const float* __restrict__ actor_mean, const float* __restrict__ actor_precision,
                                                         const float* __restrict__ critic_mean, const float* __restrict__ critic_precision) {
    const int sub = threadIdx.x & 15;
    for (int b = (blockIdx.x * blockDim.x + threadIdx.x) >> 4; b < batch; b += (gridDim.x * blockDim.x) >> 4) {
        const size_t row = row_indices ? row_indices[b] : (size_t)b;
        // the optional standardize layers in front of the networks (nn/layers/standardize/operations_generic.h:68-86) are applied here
        for (int c = sub; c < O; c += 16) {
            float v = observations[row * ld + c];
            if (actor_mean) { v -= actor_mean[c]; const float p = actor_precision[c]; if (p != 0.f) v *= p; }
            obs[(size_t)b * O + c] = v;
        }
        for (int c = sub; c < OP; c += 16) {
            float v = observations_privileged[row * ld + c];
            if (critic_mean) { v -= critic_mean[c]; const float p = critic_precision[c]; if (p != 0.f) v *= p; }
            obsp[(size_t)b * OP + c] = v;
        }
        for (int c = sub; c < A; c += 16) act[(size_t)b * A + c] = actions[row * ld + c];
        if (sub == 0) { lp[b] = log_probs[row * ld]; adv[b] = advantages[row * ld]; tgt[b] = targets[row * ld]; }
    }
}

// advantage mean and standard deviation over the minibatch (:170-180): stats = {mean, std}. Minibatch row b is dataset row rows[b] (rows == NULL: b).
// Shuffled rows of a large dataset sit on as many pages as there are rows, so the rows are spread over up to STAT_GROUPS workgroups; each leaves
// {sum, sum of squares} of its rows in `partial`, and they are added up in workgroup order: the result does not depend on scheduling.
constexpr int STAT_GROUPS = 64, EPOCH_CHUNK = 32;
// thread 0 of workgroup `block` of `n_blocks` returns the sums over the workgroup's share of the rows
__device__ __forceinline__ void advantage_block_sums(const float* __restrict__ advantages, int ld, int batch, const uint32_t* __restrict__ rows, int block, int n_blocks,
                                                     float& sum, float& sum_sq) {
    __shared__ float s1[4], s2[4];
    float a = 0.f, q = 0.f;
    // four rows per lane at a time: their indices are requested together, then their values
    const int stride = n_blocks * 256;
    for (int base = block * 256; base < batch; base += 4 * stride) {
        size_t row[4]; float v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) { const int b = min(base + u * stride + (int)threadIdx.x, batch - 1); row[u] = rows ? rows[b] : (size_t)b; }
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = advantages[row[u] * ld];
#pragma unroll
        for (int u = 0; u < 4; u++) if (base + u * stride + (int)threadIdx.x < batch) { a += v[u]; q += v[u] * v[u]; }
    }
    a = rlt_wave_sum(a); q = rlt_wave_sum(q);
    if ((threadIdx.x & 63) == 0) { s1[threadIdx.x >> 6] = a; s2[threadIdx.x >> 6] = q; }
    __syncthreads();
    sum = (s1[0] + s1[1]) + (s1[2] + s1[3]); sum_sq = (s2[0] + s2[1]) + (s2[2] + s2[3]);
}
__device__ __forceinline__ void advantage_stats_from_partials(const float* partial, int groups, int batch, int normalize, float* __restrict__ stats) {
    float m = 0.f, v = 0.f;
    for (int g = 0; g < groups; g++) { m += ((const volatile float*)partial)[2 * g]; v += ((const volatile float*)partial)[2 * g + 1]; }
    m /= (float)batch; v /= (float)batch;
    stats[0] = normalize ? m : 0.f;
    stats[1] = normalize ? sqrtf(fmaxf(0.f, v - m * m)) : 0.f;
}
// one minibatch: the last workgroup to finish (ticket counter, zero between launches) adds the partial sums up
__global__ __launch_bounds__(256) void ppo_advantage_stats_kernel(const float* __restrict__ advantages, int ld, int batch, int normalize, float* __restrict__ stats,
                                                                  const uint32_t* __restrict__ rows, float* __restrict__ partial, uint32_t* __restrict__ ticket) {
    __shared__ bool last;
    float a = 0.f, q = 0.f;
    if (normalize) advantage_block_sums(advantages, ld, batch, rows, blockIdx.x, gridDim.x, a, q);
    if (threadIdx.x == 0) {
        partial[2 * blockIdx.x] = a; partial[2 * blockIdx.x + 1] = q;
        __threadfence();
        last = atomicAdd(ticket, 1u) == gridDim.x - 1;
    }
    __syncthreads();
    if (last && threadIdx.x == 0) {
        __threadfence();
        advantage_stats_from_partials(partial, gridDim.x, batch, normalize, stats);
        *ticket = 0;
    }
}
// the minibatches of an epoch at once: blockIdx.y = minibatch, rows = its `batch` entries of the epoch's permutation; then one lane per minibatch
__global__ __launch_bounds__(256) void ppo_epoch_stats_partial_kernel(const float* __restrict__ advantages, int ld, int batch, const uint32_t* __restrict__ rows,
                                                                      float* __restrict__ partial) {
    float a, q;
    advantage_block_sums(advantages, ld, batch, rows + (size_t)blockIdx.y * batch, blockIdx.x, gridDim.x, a, q);
    if (threadIdx.x == 0) { float* p = partial + ((size_t)blockIdx.y * STAT_GROUPS + blockIdx.x) * 2; p[0] = a; p[1] = q; }
}
__global__ void ppo_epoch_stats_final_kernel(const float* __restrict__ partial, int groups, int batch, int normalize, int n_minibatches, float* __restrict__ stats) {
    const int mb = blockIdx.x * blockDim.x + threadIdx.x;
    if (mb < n_minibatches) advantage_stats_from_partials(partial + (size_t)mb * STAT_GROUPS * 2, normalize ? groups : 0, batch, normalize, stats + 2 * mb);
}
int stat_groups(int batch) { const int g = (batch + 255) / 256; return g > STAT_GROUPS ? STAT_GROUPS : g; }
// stats = scratch[0..1]; the workgroups' partial sums sit behind the surrogate kernel's own partials
int ppo_advantage_stats(rlt_rocm_device* device, const float* advantages, int ld, int batch, int normalize, float* scratch, int action_dim, const uint32_t* rows) {
    void* counters = nullptr;
    int rc = rlt_counters(device, &counters);
    if (rc) return rc;
    float* partial = scratch + 2 + (size_t)((batch + 255) / 256) * action_dim;
    hipLaunchKernelGGL(ppo_advantage_stats_kernel, dim3(stat_groups(batch)), dim3(256), 0, device->stream, advantages, ld, batch, normalize, scratch, rows, partial,
                       (uint32_t*)((char*)counters + 192));
    return rlt_launch_status(device);
}

// per sample (:205-269): log-probability of the rollout action under the current policy, ratio, clipping, d loss / d mean; the
// surrogate part of the log_std gradient as per-workgroup partial sums partial[block][action]
constexpr int PPO_MAX_ACTION_DIM = 64;
__global__ __launch_bounds__(256) void ppo_surrogate_kernel(const float* __restrict__ means, int ld_means, const float* __restrict__ log_std,
                                                            const float* __restrict__ actions, int ld_actions, const float* __restrict__ log_probs, int ld_lp,
                                                            const float* __restrict__ advantages, int ld_adv, rlt_ppo_parameters P, const float* __restrict__ stats,
                                                            float* __restrict__ d_means, int ld_d, float* __restrict__ partial, int batch, int A) {
    __shared__ float red[4][PPO_MAX_ACTION_DIM];
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    const bool ok = b < batch;
    float d_loss_d_lp = 0.f;
    if (ok) {
        float lp = 0.f;
        for (int a = 0; a < A; a++) {
            const float mean = means[(size_t)b * ld_means + a], ls = log_std[a], value = actions[(size_t)b * ld_actions + a];
            const float pre = (value - mean) / expf(ls);
            lp += (-0.9189385332046727f - ls) - 0.5f * pre * pre;        // random/operations_generic.h:73-81
        }
        float advantage = advantages[(size_t)b * ld_adv];
        if (P.normalize_advantage) advantage = (advantage - stats[0]) / (stats[1] + P.advantage_epsilon);
        const float ratio = expf(lp - log_probs[(size_t)b * ld_lp]);
        const float clipped_ratio = fminf(fmaxf(ratio, 1.0f - P.epsilon_clip), 1.0f + P.epsilon_clip);
        const bool clipped = ratio != clipped_ratio;
        const bool ratio_min_switch = ratio * advantage - clipped_ratio * advantage <= 0.0f;
        const float d_surrogate_d_ratio = ratio_min_switch ? advantage : (clipped ? 0.0f : advantage);
        d_loss_d_lp = (-1.0f / (float)batch) * d_surrogate_d_ratio * ratio;
    }
    for (int a = 0; a < A; a++) {
        float g_ls = 0.f;
        if (ok) {
            const float mean = means[(size_t)b * ld_means + a], ls = log_std[a], value = actions[(size_t)b * ld_actions + a];
            const float sd = expf(ls), pre = (value - mean) / sd;
            d_means[(size_t)b * ld_d + a] = d_loss_d_lp * (pre / sd);     // d log_prob / d mean (:82-88)
            g_ls = d_loss_d_lp * (pre * pre - 1.0f);                      // d log_prob / d log_std (:89-96)
        }
        g_ls = rlt_wave_sum(g_ls);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6][a] = g_ls;
    }
    __syncthreads();
    if ((int)threadIdx.x < A) partial[(size_t)blockIdx.x * A + threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}
// d_log_std[a] += sum of the partials (workgroup order) + the entropy term batch * (-1/batch * coefficient) (:229-233)
__global__ void ppo_log_std_gradient_kernel(const float* __restrict__ partial, int blocks, int A, float entropy_coefficient, float* __restrict__ d_log_std) {
    const int a = blockIdx.x * blockDim.x + threadIdx.x;
    if (a >= A) return;
    float s = 0.f;
    for (int i = 0; i < blocks; i++) s += partial[(size_t)i * A + a];
    d_log_std[a] += s - entropy_coefficient;
}

// RLT_MLP_SINGLE_PASS=0 keeps the actor on the per-layer kernels (tests compare the two paths with each other)
bool narrow_pass_enabled() { const char* v = std::getenv("RLT_MLP_SINGLE_PASS"); return !(v && v[0] == '0'); }
bool ppo_agent_ok(const rlt_ppo_agent* A) {
    return A && A->actor && A->critic && A->n_actor_layers >= 1 && A->n_critic_layers >= 1 && A->log_std && A->actor_adam_tensors && A->critic_adam_tensors &&
           A->actor_age && A->critic_age && A->observation_dim >= 1 && A->observation_privileged_dim >= 1 && A->action_dim >= 1 && A->action_dim <= PPO_MAX_ACTION_DIM &&
           A->batch >= 1 && A->actor[0].in_dim == A->observation_dim && A->actor[A->n_actor_layers - 1].out_dim == A->action_dim &&
           A->critic[0].in_dim == A->observation_privileged_dim && A->critic[A->n_critic_layers - 1].out_dim == 1 && A->actor[A->n_actor_layers - 1].output &&
           !A->actor_standardize_mean == !A->actor_standardize_precision && !A->critic_standardize_mean == !A->critic_standardize_precision;
}
size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
// stats, surrogate partials, stats partials, then for an epoch's minibatches in chunks: their stats and stats partials
size_t ppo_surrogate_scratch_floats(int batch, int A) { return 2 + (size_t)((batch + 255) / 256) * A + 2 * STAT_GROUPS + (size_t)EPOCH_CHUNK * (2 + 2 * STAT_GROUPS); }
}  // namespace

extern "C" int rlt_rocm_ppo_gae(rlt_rocm_device* device, const float* rewards, const float* terminated, const float* truncated, const float* all_values,
                                float* advantages, float* target_values, int ld, int n_envs, int steps, float gamma, float lambda, int ignore_termination) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rewards && terminated && truncated && all_values && advantages && target_values && ld >= 1 && n_envs > 0 && steps > 0);
    // short chunks put more threads (and more loads) in flight; 16 steps a thread reach 4,096 steps
    const int chunk_steps = steps <= 8 * GAE_THREADS ? 8 : 16;
    const int n_chunks = (steps + chunk_steps - 1) / chunk_steps;
    const char* serial = std::getenv("RLT_GAE_SERIAL");
    if (n_chunks <= GAE_THREADS && !(serial && serial[0] == '1')) {
        int envs_per_block = GAE_THREADS / n_chunks;                  // threads of a block: n_chunks x envs_per_block, neighbouring lanes = neighbouring environments
        if (envs_per_block > 64) envs_per_block = 64;
        if (envs_per_block > n_envs) envs_per_block = n_envs;
        const int blocks = (n_envs + envs_per_block - 1) / envs_per_block;
        if (chunk_steps == 8)
            hipLaunchKernelGGL(gae_kernel<8>, dim3(blocks), dim3(GAE_THREADS), 0, device->stream, rewards, terminated, truncated, all_values, advantages, target_values, ld, n_envs, steps,
                               gamma, lambda, ignore_termination, n_chunks, envs_per_block);
        else
            hipLaunchKernelGGL(gae_kernel<16>, dim3(blocks), dim3(GAE_THREADS), 0, device->stream, rewards, terminated, truncated, all_values, advantages, target_values, ld, n_envs, steps,
                               gamma, lambda, ignore_termination, n_chunks, envs_per_block);
    } else {
        int blocks = (n_envs + 63) / 64; if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(gae_serial_kernel, dim3(blocks), dim3(64), 0, device->stream, rewards, terminated, truncated, all_values, advantages, target_values, ld, n_envs, steps,
                           gamma, lambda, ignore_termination);
    }
    return rlt_launch_status(device);
}

extern "C" size_t rlt_rocm_ppo_workspace_bytes(const rlt_ppo_agent* A) {
    if (!ppo_agent_ok(A)) return 0;
    const size_t B = (size_t)A->batch;
    size_t floats = B * (A->observation_dim + A->observation_privileged_dim + 2 * A->action_dim + 4) + ppo_surrogate_scratch_floats(A->batch, A->action_dim) + 64;
    const size_t mlp_a = rlt_rocm_mlp_workspace_bytes(A->actor, A->n_actor_layers, A->batch), mlp_c = rlt_rocm_mlp_workspace_bytes(A->critic, A->n_critic_layers, A->batch);
    return align256(floats * sizeof(float)) + align256(mlp_a > mlp_c ? mlp_a : mlp_c) + 256;
}

static int ppo_surrogate_impl(rlt_rocm_device* device, const float* means, int ld_means, const float* log_std, const float* actions, int ld_actions, const float* log_probs,
                              int ld_lp, const float* advantages, int ld_adv, const rlt_ppo_parameters* P, float* d_means, int ld_d, float* d_log_std, int batch, int A,
                              float* scratch) {
    float* stats = scratch; float* partial = scratch + 2;
    const int blocks = (batch + 255) / 256;
    int rc = ppo_advantage_stats(device, advantages, ld_adv, batch, P->normalize_advantage, scratch, A, nullptr);
    if (rc) return rc;
    hipLaunchKernelGGL(ppo_surrogate_kernel, dim3(blocks), dim3(256), 0, device->stream, means, ld_means, log_std, actions, ld_actions, log_probs, ld_lp, advantages, ld_adv, *P,
                       stats, d_means, ld_d, partial, batch, A);
    if ((rc = rlt_launch_status(device))) return rc;
    if (P->learn_action_std) {
        hipLaunchKernelGGL(ppo_log_std_gradient_kernel, dim3(1), dim3(64), 0, device->stream, partial, blocks, A, P->action_entropy_coefficient, d_log_std);
        rc = rlt_launch_status(device);
    }
    return rc;
}

extern "C" int rlt_rocm_ppo_surrogate_gradient(rlt_rocm_device* device, const float* action_means, int ld_means, const float* log_std, const float* actions, int ld_actions,
                                               const float* action_log_probs, int ld_log_probs, const float* advantages, int ld_advantages, const rlt_ppo_parameters* P,
                                               float* d_action_means, int ld_d, float* d_log_std, int batch, int action_dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(action_means && log_std && actions && action_log_probs && advantages && P && d_action_means && batch > 0 && action_dim > 0 && action_dim <= PPO_MAX_ACTION_DIM);
    RLT_REQUIRE(ld_means >= action_dim && ld_actions >= action_dim && ld_d >= action_dim && ld_log_probs >= 1 && ld_advantages >= 1 && (!P->learn_action_std || d_log_std));
    void* scratch = nullptr;
    int rc = rlt_scratch(device, ppo_surrogate_scratch_floats(batch, action_dim) * sizeof(float), &scratch);
    if (rc) return rc;
    return ppo_surrogate_impl(device, action_means, ld_means, log_std, actions, ld_actions, action_log_probs, ld_log_probs, advantages, ld_advantages, P, d_action_means, ld_d,
                              d_log_std, batch, action_dim, (float*)scratch);
}

// Which way the pair of networks takes: 1 = both are in -> 64 -> 64 -> out and share the one-launch pass; 2 = they do once their hidden width (below 64) is padded
// to 64 with zero rows and columns (pad.h); 0 = the per-layer kernels.
static int pair_mode(const rlt_ppo_agent* A) {
    if (!narrow_pass_enabled()) return 0;
    if (rlt_mlp3s_pair_supported(A->actor, A->n_actor_layers, A->critic, A->n_critic_layers)) return 1;
    const bool pad_a = rlt_pad_eligible(A->actor, A->n_actor_layers), pad_c = rlt_pad_eligible(A->critic, A->n_critic_layers);
    if (!pad_a && !pad_c) return 0;
    if (A->n_actor_layers != 3 || A->n_critic_layers != 3) return 0;
    rlt_dense_layer a[3], c[3];
    for (int l = 0; l < 3; l++) { a[l] = A->actor[l]; c[l] = A->critic[l]; }
    if (pad_a) { a[0].out_dim = 64; a[1].in_dim = 64; a[1].out_dim = 64; a[2].in_dim = 64; }
    if (pad_c) { c[0].out_dim = 64; c[1].in_dim = 64; c[1].out_dim = 64; c[2].in_dim = 64; }
    return rlt_mlp3s_pair_supported(a, 3, c, 3) ? 2 : 0;
}

// actor and critic of the supported narrow shape in one launch (stats = {advantage mean, std} of the minibatch on the device), then both Adam steps in one
static int ppo_pair_update(rlt_rocm_device* device, const rlt_ppo_agent* A, const rlt_ppo_parameters* P, const float* observations, const float* observations_privileged,
                           const float* actions, const float* action_log_probs, const float* advantages, const float* target_values, int ld, const uint32_t* row_indices,
                           const float* stats, float* values, float* out_critic_loss) {
    const int B = A->batch, AD = A->action_dim;
    int rc;
    const rlt_dense_layer* actor = A->actor; const rlt_dense_layer* critic = A->critic;
    rlt_padded_net padded_actor, padded_critic;
    const bool pad_a = rlt_pad_eligible(A->actor, A->n_actor_layers), pad_c = rlt_pad_eligible(A->critic, A->n_critic_layers);
    if (pad_a || pad_c) {       // the parameters change with every minibatch's Adam step: the padded copies are made anew
        const size_t floats_a = pad_a ? rlt_pad_floats(A->actor, true) : 0, floats_c = pad_c ? rlt_pad_floats(A->critic, true) : 0;
        void* memory = nullptr;
        if ((rc = rlt_pad_scratch(device, (floats_a + floats_c) * sizeof(float), &memory))) return rc;
        if (pad_a) { if ((rc = rlt_pad_parameters(device, A->actor, (float*)memory, true, &padded_actor))) return rc; actor = padded_actor.L; }
        if (pad_c) { if ((rc = rlt_pad_parameters(device, A->critic, (float*)memory + floats_a, true, &padded_critic))) return rc; critic = padded_critic.L; }
    }
    // the optimisers' launch adds up the kernel's partial sums itself where it can (:305-306); not for padded copies, whose gradients are copied back first
    const rlt_mlp3s_step steps[2] = {{A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age}, {A->critic_adam_tensors, A->n_critic_adam_tensors, &A->critic_adam, A->critic_age}};
    const bool fuse_steps = !pad_a && !pad_c && (P->learn_action_std || !A->d_log_std);
    bool stepped = false;
    rc = rlt_mlp3s_ppo_actor_critic(device, actor, A->n_actor_layers, observations, A->actor[A->n_actor_layers - 1].output, AD, A->log_std, actions,
                                    action_log_probs, advantages, stats, P, P->learn_action_std ? A->d_log_std : nullptr, -P->action_entropy_coefficient,
                                    critic, A->n_critic_layers, observations_privileged, values, 1, target_values, 1.0f / (float)B, out_critic_loss,   // :303
                                    ld, row_indices, B, A->actor_standardize_mean, A->actor_standardize_precision, A->critic_standardize_mean,
                                    A->critic_standardize_precision, fuse_steps ? steps : nullptr, &stepped);
    if (rc || stepped) return rc;
    if (pad_a) if ((rc = rlt_unpad_gradients(device, A->actor, &padded_actor))) return rc;
    if (pad_c) if ((rc = rlt_unpad_gradients(device, A->critic, &padded_critic))) return rc;
    if (A->d_log_std && !P->learn_action_std) if ((rc = rlt_rocm_fill_f32(device, A->d_log_std, 1, AD, AD, 0.0f))) return rc;
    return rlt_adam_step_pair(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age,                                            // :305-306
                              A->critic_adam_tensors, A->n_critic_adam_tensors, &A->critic_adam, A->critic_age);
}

extern "C" int rlt_rocm_ppo_train_minibatch(rlt_rocm_device* device, const rlt_ppo_agent* A, const rlt_ppo_parameters* P, const float* observations,
                                            const float* observations_privileged, const float* actions, const float* action_log_probs, const float* advantages,
                                            const float* target_values, int ld, const uint32_t* row_indices, float* out_critic_loss) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(ppo_agent_ok(A) && P && observations && observations_privileged && actions && action_log_probs && advantages && target_values && ld >= 1);
    RLT_REQUIRE(!P->learn_action_std || A->d_log_std);
    RLT_REQUIRE(A->workspace && A->workspace_bytes >= rlt_rocm_ppo_workspace_bytes(A));
    const int B = A->batch, O = A->observation_dim, OP = A->observation_privileged_dim, AD = A->action_dim;
    // carve the workspace: packed minibatch, gradient at the actor output, critic output, surrogate scratch, then the networks' own workspace
    float* w = (float*)A->workspace;
    float* obs = w; w += (size_t)B * O; float* obsp = w; w += (size_t)B * OP; float* act = w; w += (size_t)B * AD; float* d_act = w; w += (size_t)B * AD;
    float* lp = w; w += B; float* adv = w; w += B; float* tgt = w; w += B; float* values = w; w += B;
    float* scratch = w; w += ppo_surrogate_scratch_floats(B, AD);
    char* mlp_ws = (char*)A->workspace + align256((size_t)((char*)w - (char*)A->workspace) + 64 * sizeof(float));
    const size_t mlp_ws_bytes = A->workspace_bytes - (size_t)(mlp_ws - (char*)A->workspace);
    int rc;
    if (pair_mode(A)) {
        // both networks in -> 64 -> 64 -> out (or narrower and padded to that): one launch runs the actor (forward, surrogate gradient, backward, :203-285) on half of the compute units
        // and the critic (forward, MSE gradient with loss weight 0.5 = (v - target) / batch, backward, :289-300) on the other half, reading the
        // minibatch's rows straight out of the dataset; its gradients replace the old ones, which is what zero_gradient (:158-159) followed by
        // backward leaves. The means still land in the actor's last output buffer; the hidden layers' buffers are not written.
        if ((rc = ppo_advantage_stats(device, advantages, ld, B, P->normalize_advantage, scratch, AD, row_indices))) return rc;
        return ppo_pair_update(device, A, P, observations, observations_privileged, actions, action_log_probs, advantages, target_values, ld, row_indices, scratch,
                               values, out_critic_loss);
    }
    int blocks = (B * 16 + 255) / 256; if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(ppo_gather_kernel, dim3(blocks), dim3(256), 0, device->stream, observations, observations_privileged, actions, action_log_probs, advantages, target_values,
                       ld, row_indices, B, O, OP, AD, obs, obsp, act, lp, adv, tgt, A->actor_standardize_mean, A->actor_standardize_precision,
                       A->critic_standardize_mean, A->critic_standardize_precision);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_mlp_zero_gradient(device, A->critic, A->n_critic_layers))) return rc;                      // :158
    if ((rc = rlt_rocm_mlp_zero_gradient(device, A->actor, A->n_actor_layers))) return rc;                        // :159 (clears the log_std gradient too)
    if (A->d_log_std) if ((rc = rlt_rocm_fill_f32(device, A->d_log_std, 1, AD, AD, 0.0f))) return rc;
    rc = RLT_E_UNSUPPORTED;
    if (narrow_pass_enabled() && rlt_mlp3s_supported(A->actor, A->n_actor_layers)) {       // the actor alone in one kernel
        if ((rc = ppo_advantage_stats(device, adv, 1, B, P->normalize_advantage, scratch, AD, nullptr))) return rc;
        rc = rlt_mlp3s_ppo_actor(device, A->actor, A->n_actor_layers, obs, O, A->actor[A->n_actor_layers - 1].output, AD, A->log_std, act, AD, lp, 1, adv, 1, scratch, P,
                                 P->learn_action_std ? A->d_log_std : nullptr, -P->action_entropy_coefficient, B);
        if (rc && rc != RLT_E_UNSUPPORTED) return rc;
    }
    if (rc == RLT_E_UNSUPPORTED) {
        if ((rc = rlt_rocm_mlp_forward(device, A->actor, A->n_actor_layers, obs, O, B))) return rc;                    // :203
        const float* means = A->actor[A->n_actor_layers - 1].output;
        if ((rc = ppo_surrogate_impl(device, means, AD, A->log_std, act, AD, lp, 1, adv, 1, P, d_act, AD, A->d_log_std, B, AD, scratch))) return rc;
        if ((rc = rlt_rocm_mlp_backward(device, A->actor, A->n_actor_layers, obs, O, d_act, AD, nullptr, 0, B, 1, mlp_ws, mlp_ws_bytes))) return rc;   // :285
    }
    // critic: forward, MSE gradient with loss weight 0.5 (= (v - target)/batch), backward in one pass (:289-300)
    if ((rc = rlt_rocm_mlp_forward_backward(device, A->critic, A->n_critic_layers, obsp, OP, values, 1, nullptr, 0, tgt, 1, 1.0f / (float)B, B, mlp_ws, mlp_ws_bytes))) return rc;
    if (out_critic_loss) if ((rc = rlt_rocm_mse_evaluate(device, values, 1, tgt, 1, B, 1, 1.0f, out_critic_loss))) return rc;                      // :303
    if ((rc = rlt_rocm_adam_step(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, 0.0f, nullptr))) return rc;  // :305
    return rlt_rocm_adam_step(device, A->critic_adam_tensors, A->n_critic_adam_tensors, &A->critic_adam, A->critic_age, 0.0f, nullptr);             // :306
}

extern "C" int rlt_rocm_ppo_train_epoch(rlt_rocm_device* device, const rlt_ppo_agent* A, const rlt_ppo_parameters* P, const float* observations,
                                        const float* observations_privileged, const float* actions, const float* action_log_probs, const float* advantages,
                                        const float* target_values, int ld, const uint32_t* row_indices, int n_minibatches, float* out_critic_losses) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(ppo_agent_ok(A) && P && observations && observations_privileged && actions && action_log_probs && advantages && target_values && ld >= 1);
    RLT_REQUIRE(row_indices && n_minibatches >= 1 && (!P->learn_action_std || A->d_log_std));
    RLT_REQUIRE(A->workspace && A->workspace_bytes >= rlt_rocm_ppo_workspace_bytes(A));
    const int B = A->batch, O = A->observation_dim, OP = A->observation_privileged_dim, AD = A->action_dim;
    if (!pair_mode(A)) {
        for (int mb = 0; mb < n_minibatches; mb++) {
            const int rc = rlt_rocm_ppo_train_minibatch(device, A, P, observations, observations_privileged, actions, action_log_probs, advantages, target_values, ld,
                                                        row_indices + (size_t)mb * B, out_critic_losses ? out_critic_losses + mb : nullptr);
            if (rc) return rc;
        }
        return 0;
    }
    // same carving of the workspace as the minibatch call; the advantage statistics of up to EPOCH_CHUNK minibatches are formed by one pair of launches
    float* w = (float*)A->workspace;
    w += (size_t)B * O; w += (size_t)B * OP; w += (size_t)B * AD; w += (size_t)B * AD; w += 3 * (size_t)B;
    float* values = w; w += B;
    float* stats_all = w + 2 + (size_t)((B + 255) / 256) * AD + 2 * STAT_GROUPS; float* partial_all = stats_all + 2 * EPOCH_CHUNK;
    const int groups = stat_groups(B);
    for (int first = 0; first < n_minibatches; first += EPOCH_CHUNK) {
        const int n = n_minibatches - first < EPOCH_CHUNK ? n_minibatches - first : EPOCH_CHUNK;
        int rc;
        if (P->normalize_advantage) {
            hipLaunchKernelGGL(ppo_epoch_stats_partial_kernel, dim3(groups, n), dim3(256), 0, device->stream, advantages, ld, B, row_indices + (size_t)first * B, partial_all);
            if ((rc = rlt_launch_status(device))) return rc;
        }
        hipLaunchKernelGGL(ppo_epoch_stats_final_kernel, dim3(1), dim3(EPOCH_CHUNK), 0, device->stream, partial_all, groups, B, P->normalize_advantage, n, stats_all);
        if ((rc = rlt_launch_status(device))) return rc;
        for (int mb = first; mb < first + n; mb++)
            if ((rc = ppo_pair_update(device, A, P, observations, observations_privileged, actions, action_log_probs, advantages, target_values, ld,
                                      row_indices + (size_t)mb * B, stats_all + 2 * (mb - first), values, out_critic_losses ? out_critic_losses + mb : nullptr))) return rc;
    }
    return 0;
}
