// TD3: the actor's clipped-Gaussian sampling layer, target-policy smoothing noise, TD target, and train_critic / train_actor /
// target updates assembled from them and the shared network kernels.
// reference: nn/layers/td3_sampling/operations_generic.h:75-163,
//            rl/algorithms/td3/operations_generic.h:116-325 (CUDA: operations_cuda.h:8-110).
#include "common.h"
#include "sac_update.h"
#include "mlp_rows.h"

namespace {

__device__ __forceinline__ float clampf(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }
// a * b + c rounded twice, as the reference's CPU build computes it (keeps the compiler from contracting into one fused operation)
__device__ __forceinline__ float mul_add(float a, float b, float c) {
#pragma clang fp contract(off)
    float product = a * b;
    return product + c;
}

__global__ __launch_bounds__(256) void td3_sampling_forward_kernel(const float* __restrict__ input, int ldin, const float* __restrict__ noise, int ldn, float std,
                                                                   float* __restrict__ pre_clip, int ldp, float* __restrict__ output, int ldo, int batch, int dim) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * dim; i += gridDim.x * blockDim.x) {
        int r = i / dim, c = i % dim;
        float mean = input[(size_t)r * ldin + c];
        float sample = noise ? mul_add(noise[(size_t)r * ldn + c], std, mean) : mean;
        if (pre_clip) pre_clip[(size_t)r * ldp + c] = sample;
        output[(size_t)r * ldo + c] = clampf(sample, -1.0f, 1.0f);
    }
}

__global__ __launch_bounds__(256) void td3_sampling_backward_kernel(const float* __restrict__ pre_clip, int ldp, const float* __restrict__ d_output, int lddo,
                                                                    float* __restrict__ d_input, int lddi, int batch, int dim) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * dim; i += gridDim.x * blockDim.x) {
        int r = i / dim, c = i % dim;
        float pc = pre_clip[(size_t)r * ldp + c];
        d_input[(size_t)r * lddi + c] = (pc < -1.0f || pc > 1.0f) ? 0.0f : d_output[(size_t)r * lddo + c];
    }
}

__global__ __launch_bounds__(256) void td3_target_action_noise_kernel(const float* __restrict__ z, float std, float clip, float* __restrict__ out, size_t count) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        out[i] = clampf(mul_add(z[i], std, 0.0f), -clip, clip);
}

__global__ __launch_bounds__(256) void td3_noisy_next_actions_kernel(float* __restrict__ a, int lda, const float* __restrict__ noise, int ldn, int batch, int dim) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * dim; i += gridDim.x * blockDim.x) {
        int r = i / dim, c = i % dim;
        a[(size_t)r * lda + c] = clampf(a[(size_t)r * lda + c] + noise[(size_t)r * ldn + c], -1.0f, 1.0f);
    }
}

__global__ __launch_bounds__(256) void td3_target_q_kernel(const float* __restrict__ q1, const float* __restrict__ q2, const float* __restrict__ rewards,
                                                           const uint8_t* __restrict__ terminated, float gamma, int ignore_termination,
                                                           float* __restrict__ target, int batch) {
    for (int b = blockIdx.x * blockDim.x + threadIdx.x; b < batch; b += gridDim.x * blockDim.x) {
        float m = fminf(q1[b], q2[b]);
        float future = (ignore_termination || !terminated[b]) ? gamma * m : 0.0f;
        target[b] = mul_add(1.0f, rewards[b], future);
    }
}

// The input of the target critics in one pass over the rows (td3/operations_generic.h:191-196): the target actor's mean through the
// sampling layer, the smoothing noise, the mask that keeps the stored next action on non-final steps, and the observation copy.
__global__ __launch_bounds__(256) void td3_next_input_kernel(const float* __restrict__ mean, const float* __restrict__ sampling_noise, float std,
                                                             const float* __restrict__ target_noise, const uint8_t* __restrict__ next_final_step_mask,
                                                             const float* __restrict__ obs_next, float* __restrict__ next_input, int batch, int obs, int act) {
    const int D = obs + act;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * D; i += gridDim.x * blockDim.x) {
        int r = i / D, c = i % D;
        float v = obs_next[i];
        if (c >= obs && (!next_final_step_mask || next_final_step_mask[r])) {
            int a = c - obs;
            float sample = mul_add(sampling_noise[(size_t)r * act + a], std, mean[(size_t)r * act + a]);
            v = clampf(clampf(sample, -1.0f, 1.0f) + target_noise[(size_t)r * act + a], -1.0f, 1.0f);
        }
        next_input[i] = v;
    }
}

// The input of critic 0 in train_actor (:255-259): sampled action (or the stored one on non-final steps) beside the observation.
__global__ __launch_bounds__(256) void td3_actor_input_kernel(const float* __restrict__ mean, const float* __restrict__ sampling_noise, float std,
                                                              const uint8_t* __restrict__ final_step_mask, const float* __restrict__ obs_act,
                                                              float* __restrict__ pre_clip, float* __restrict__ input, int batch, int obs, int act) {
    const int D = obs + act;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * D; i += gridDim.x * blockDim.x) {
        int r = i / D, c = i % D;
        float v = obs_act[i];
        if (c >= obs) {
            int a = c - obs;
            float sample = mul_add(sampling_noise[(size_t)r * act + a], std, mean[(size_t)r * act + a]);
            pre_clip[(size_t)r * act + a] = sample;
            if (!final_step_mask || final_step_mask[r]) v = clampf(sample, -1.0f, 1.0f);
        }
        input[i] = v;
    }
}

// One workgroup: n = count(final_step_mask) (or rows), then
//   critic (:200-227): y = r + gamma * min(q1', q2') unless terminated; d = (q - y) * 2/rows * (rows/n); where the mask is clear d, q and y
//                      are zeroed (the reference zeroes the latter two in its logging block);
//   actor  (:262-267): d = -1/n, zeroed where the mask is clear.
__global__ __launch_bounds__(1024) void td3_d_output_kernel(float* __restrict__ q, const float* __restrict__ q1n, const float* __restrict__ q2n,
                                                            const float* __restrict__ rewards, const uint8_t* __restrict__ terminated, float gamma,
                                                            int ignore_termination, float* __restrict__ y, const uint8_t* __restrict__ mask,
                                                            float* __restrict__ d, int rows, int actor) {
    __shared__ float partial[16];
    __shared__ float n_final;
    float cnt = 0.0f;
    for (int i = threadIdx.x; i < rows; i += blockDim.x) cnt += mask ? (float)(mask[i] != 0) : 1.0f;
    cnt = rlt_wave_sum(cnt);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = cnt;
    __syncthreads();
    if (threadIdx.x == 0) { float s = 0.0f; for (int i = 0; i < 16; i++) s += partial[i]; n_final = s; }
    __syncthreads();
    if (actor) {
        const float v = -1.0f / n_final;
        for (int i = threadIdx.x; i < rows; i += blockDim.x) d[i] = (!mask || mask[i]) ? v : 0.0f;
        return;
    }
    float loss_weight = 1.0f; loss_weight *= (float)rows / n_final;
    const float constant = 2.0f / (float)rows * loss_weight;
    for (int i = threadIdx.x; i < rows; i += blockDim.x) {
        float m = fminf(q1n[i], q2n[i]);
        float future = (ignore_termination || !terminated[i]) ? gamma * m : 0.0f;
        float target = mul_add(1.0f, rewards[i], future);
        float diff = q[i] - target;
        if (!mask || mask[i]) { y[i] = target; d[i] = diff * constant; }
        else { y[i] = 0.0f; d[i] = 0.0f; q[i] = 0.0f; }
    }
}

// d_actions (columns obs.. of d_critic_input) through the mask and the sampling layer's backward (:272-278)
__global__ __launch_bounds__(256) void td3_actor_d_output_kernel(float* __restrict__ d_critic_input, const float* __restrict__ pre_clip,
                                                                 const uint8_t* __restrict__ final_step_mask, float* __restrict__ d_actor_output,
                                                                 int batch, int obs, int act) {
    const int D = obs + act;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * act; i += gridDim.x * blockDim.x) {
        int r = i / act, a = i % act;
        float g = d_critic_input[(size_t)r * D + obs + a];
        float pc = pre_clip[i];
        if (final_step_mask && !final_step_mask[r]) { g = 0.0f; d_critic_input[(size_t)r * D + obs + a] = 0.0f; }   // mask_gradient works in place
        d_actor_output[i] = (pc < -1.0f || pc > 1.0f) ? 0.0f : g;
    }
}

int grid1(long n) { long b = (n + 255) / 256; return (int)(b > 1024 ? 1024 : (b < 1 ? 1 : b)); }

bool agent_ok(const rlt_td3_agent* A) {
    return A && A->batch > 0 && A->observation_dim > 0 && A->action_dim > 0 && A->n_actor_layers >= 1 && A->n_critic_layers >= 1 && A->actor && A->actor_target &&
           A->critics[0] && A->critics[1] && A->critics_target[0] && A->critics_target[1] && A->observations_actions_base && A->rewards && A->terminated &&
           A->workspace && A->actor[A->n_actor_layers - 1].out_dim == A->action_dim && A->critics[0][0].in_dim == A->observation_dim + A->action_dim;
}

int polyak_mlp(rlt_rocm_device* device, const rlt_dense_layer* source, const rlt_dense_layer* target, int n, float polyak) {
    for (int l = 0; l < n; l++) {
        int rc;
        if ((rc = rlt_rocm_polyak_update(device, source[l].weights, target[l].weights, (size_t)source[l].in_dim * source[l].out_dim, polyak, 0))) return rc;
        if ((rc = rlt_rocm_polyak_update(device, source[l].biases, target[l].biases, (size_t)source[l].out_dim, polyak, 0))) return rc;
    }
    return 0;
}

}  // namespace

extern "C" {

int rlt_rocm_td3_sampling_forward(rlt_rocm_device* device, const float* input, int ldin, const float* noise, int ldn, float std, float* pre_clip, int ldp,
                                  float* output, int ldo, int batch, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(input && output && batch > 0 && dim > 0 && ldin >= dim && ldo >= dim && (!noise || ldn >= dim) && (!pre_clip || ldp >= dim));
    hipLaunchKernelGGL(td3_sampling_forward_kernel, dim3(grid1((long)batch * dim)), dim3(256), 0, device->stream, input, ldin, noise, ldn, std, pre_clip, ldp, output, ldo, batch, dim);
    return rlt_launch_status(device);
}

int rlt_rocm_td3_sampling_backward(rlt_rocm_device* device, const float* pre_clip, int ldp, const float* d_output, int lddo, float* d_input, int lddi, int batch, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(pre_clip && d_output && d_input && batch > 0 && dim > 0 && ldp >= dim && lddo >= dim && lddi >= dim);
    hipLaunchKernelGGL(td3_sampling_backward_kernel, dim3(grid1((long)batch * dim)), dim3(256), 0, device->stream, pre_clip, ldp, d_output, lddo, d_input, lddi, batch, dim);
    return rlt_launch_status(device);
}

int rlt_rocm_td3_target_action_noise(rlt_rocm_device* device, const float* standard_normal, float std, float clip, float* out, size_t count) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(standard_normal && out && count > 0 && clip >= 0.0f);
    hipLaunchKernelGGL(td3_target_action_noise_kernel, dim3(grid1((long)count)), dim3(256), 0, device->stream, standard_normal, std, clip, out, count);
    return rlt_launch_status(device);
}

int rlt_rocm_td3_noisy_next_actions(rlt_rocm_device* device, float* next_actions, int lda, const float* noise, int ldn, int batch, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(next_actions && noise && batch > 0 && dim > 0 && lda >= dim && ldn >= dim);
    hipLaunchKernelGGL(td3_noisy_next_actions_kernel, dim3(grid1((long)batch * dim)), dim3(256), 0, device->stream, next_actions, lda, noise, ldn, batch, dim);
    return rlt_launch_status(device);
}

int rlt_rocm_td3_target_action_values(rlt_rocm_device* device, const float* q1_next, const float* q2_next, const float* rewards, const uint8_t* terminated,
                                      float gamma, int ignore_termination, float* target, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(q1_next && q2_next && rewards && terminated && target && batch > 0);
    hipLaunchKernelGGL(td3_target_q_kernel, dim3(grid1(batch)), dim3(256), 0, device->stream, q1_next, q2_next, rewards, terminated, gamma, ignore_termination, target, batch);
    return rlt_launch_status(device);
}


// rl/algorithms/td3/operations_generic.h:170-235. The elementwise steps between the network passes are folded into two launches.
int rlt_rocm_td3_train_critic(rlt_rocm_device* device, const rlt_td3_agent* A, int ci, const float* sampling_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && (ci == 0 || ci == 1) && sampling_noise);
    RLT_REQUIRE(A->target_next_action_noise && A->next_state_action_value_input && A->next_q[0] && A->next_q[1] && A->target_action_value && A->d_output_critic);
    RLT_REQUIRE(A->critic_adam_tensors[ci] && A->critic_age[ci]);
    if (!device->sac_per_operation && rlt_td3_update_supported(device, A)) return rlt_td3_update_critic(device, A, ci, sampling_noise);
    if (!device->sac_per_operation && rlt_td3_wide_supported(device, A)) return rlt_td3_wide_update_critic(device, A, ci, sampling_noise);
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const rlt_dense_layer* critic = A->critics[ci];
    const size_t mean_bytes = ((size_t)B * ACT * sizeof(float) + 255) & ~(size_t)255;
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(critic, A->n_critic_layers, B) + mean_bytes);
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(A->actor_target, A->n_actor_layers, B) + mean_bytes);
    float* mean = (float*)A->workspace;
    void* ws = (char*)A->workspace + mean_bytes;
    const size_t ws_bytes = A->workspace_bytes - mean_bytes;
    int rc;
    if ((rc = rlt_rocm_mlp_zero_gradient(device, critic, A->n_critic_layers))) return rc;
    const float* obs_next = A->observations_actions_base + (size_t)B * D;
    if ((rc = rlt_rocm_mlp_evaluate(device, A->actor_target, A->n_actor_layers, obs_next, D, mean, ACT, B, ws, ws_bytes))) return rc;
    hipLaunchKernelGGL(td3_next_input_kernel, dim3(grid1((long)B * D)), dim3(256), 0, device->stream, (const float*)mean, sampling_noise, A->sampling_std,
                       (const float*)A->target_next_action_noise, A->next_final_step_mask, obs_next, A->next_state_action_value_input, B, OBS, ACT);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_mlp_forward_pair(device, A->critics_target[0], A->critics_target[1], A->n_critic_layers, A->next_state_action_value_input, D, A->next_q[0], A->next_q[1], 1, B, false, ws, ws_bytes))) return rc;
    if ((rc = rlt_rocm_mlp_forward(device, critic, A->n_critic_layers, A->observations_actions_base, D, B))) return rc;
    float* q = critic[A->n_critic_layers - 1].output;
    hipLaunchKernelGGL(td3_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, q, (const float*)A->next_q[0], (const float*)A->next_q[1], (const float*)A->rewards,
                       (const uint8_t*)A->terminated, A->gamma, A->ignore_termination, A->target_action_value, A->final_step_mask, A->d_output_critic, B, 0);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_mlp_backward(device, critic, A->n_critic_layers, A->observations_actions_base, D, A->d_output_critic, 1, nullptr, 0, B, 1, ws, ws_bytes))) return rc;
    return rlt_rocm_adam_step(device, A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], 0.0f, nullptr);
}

// train_critic for critic 0 with sampling_noise_first, then for critic 1 with sampling_noise_second, on the agent's batch and target noise (the loop's shared batch,
// rl/algorithms/td3/loop/core/operations_generic.h:98-112): for hidden widths up to 256 both run in one launch, side by side; otherwise the two calls
int rlt_rocm_td3_train_critics(rlt_rocm_device* device, const rlt_td3_agent* A, const float* sampling_noise_first, const float* sampling_noise_second) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && sampling_noise_first && sampling_noise_second);
    if (!device->sac_per_operation && rlt_td3_update_supported(device, A)) {
        RLT_REQUIRE(A->target_next_action_noise && A->target_action_value);
        for (int k = 0; k < 2; k++) RLT_REQUIRE(A->critic_adam_tensors[k] && A->critic_age[k]);
        return rlt_td3_update_critics(device, A, sampling_noise_first, sampling_noise_second, nullptr, false);
    }
    if (!device->sac_per_operation && rlt_td3_wide_supported(device, A)) {
        RLT_REQUIRE(A->target_next_action_noise && A->target_action_value);
        for (int k = 0; k < 2; k++) RLT_REQUIRE(A->critic_adam_tensors[k] && A->critic_age[k]);
        return rlt_td3_wide_update_critics(device, A, sampling_noise_first, sampling_noise_second, nullptr, false);
    }
    const int rc = rlt_rocm_td3_train_critic(device, A, 0, sampling_noise_first);
    return rc ? rc : rlt_rocm_td3_train_critic(device, A, 1, sampling_noise_second);
}

// the critic update of a shared batch with its draws: inside the one launch where that path applies, by three rlt_rocm_randn_f32 calls otherwise
int rlt_rocm_td3_train_critics_drawn(rlt_rocm_device* device, const rlt_td3_agent* A, const rlt_td3_critic_draws* draws, float* sampling_noise, int update_targets) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && draws && A->target_next_action_noise && draws->target_noise_std >= 0.0f && draws->target_noise_clip >= 0.0f);
    if (!device->sac_per_operation && rlt_td3_update_supported(device, A)) {
        RLT_REQUIRE(A->target_action_value);
        for (int k = 0; k < 2; k++) RLT_REQUIRE(A->critic_adam_tensors[k] && A->critic_age[k]);
        return rlt_td3_update_critics(device, A, nullptr, nullptr, draws, update_targets != 0);
    }
    if (!device->sac_per_operation && rlt_td3_wide_supported(device, A)) {
        RLT_REQUIRE(A->target_action_value);
        for (int k = 0; k < 2; k++) RLT_REQUIRE(A->critic_adam_tensors[k] && A->critic_age[k]);
        return rlt_td3_wide_update_critics(device, A, nullptr, nullptr, draws, update_targets != 0);
    }
    RLT_REQUIRE(sampling_noise);
    const size_t count = (size_t)A->batch * A->action_dim;
    int rc = rlt_rocm_randn_f32(device, A->target_next_action_noise, count, draws->seed, draws->target_noise_stream);
    if (!rc) rc = rlt_rocm_td3_target_action_noise(device, A->target_next_action_noise, draws->target_noise_std, draws->target_noise_clip, A->target_next_action_noise, count);
    for (int k = 0; k < 2 && !rc; k++) rc = rlt_rocm_randn_f32(device, sampling_noise + k * count, count, draws->seed, draws->sampling_stream[k]);
    if (!rc) rc = rlt_rocm_td3_train_critics(device, A, sampling_noise, sampling_noise + count);
    return (rc || !update_targets) ? rc : rlt_rocm_td3_update_critic_targets(device, A);
}

int rlt_rocm_td3_train_actor_drawn(rlt_rocm_device* device, const rlt_td3_agent* A, uint64_t seed, uint64_t stream, float* sampling_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A));
    if (!device->sac_per_operation && (rlt_td3_update_supported(device, A) || rlt_td3_wide_supported(device, A))) {
        RLT_REQUIRE(A->state_action_value_input && A->actor_pre_clip && A->d_output_actor && A->d_critic_input && A->d_actor_output && A->actor_adam_tensors && A->actor_age);
        return rlt_td3_update_supported(device, A) ? rlt_td3_update_actor(device, A, nullptr, seed, stream) : rlt_td3_wide_update_actor(device, A, nullptr, seed, stream);
    }
    RLT_REQUIRE(sampling_noise);
    const int rc = rlt_rocm_randn_f32(device, sampling_noise, (size_t)A->batch * A->action_dim, seed, stream);
    return rc ? rc : rlt_rocm_td3_train_actor(device, A, sampling_noise);
}

// rl/algorithms/td3/operations_generic.h:236-281
int rlt_rocm_td3_train_actor(rlt_rocm_device* device, const rlt_td3_agent* A, const float* sampling_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && sampling_noise);
    RLT_REQUIRE(A->state_action_value_input && A->actor_pre_clip && A->d_output_actor && A->d_critic_input && A->d_actor_output && A->actor_adam_tensors && A->actor_age);
    if (!device->sac_per_operation && rlt_td3_update_supported(device, A)) return rlt_td3_update_actor(device, A, sampling_noise, 0, 0);
    if (!device->sac_per_operation && rlt_td3_wide_supported(device, A)) return rlt_td3_wide_update_actor(device, A, sampling_noise, 0, 0);
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(A->critics[0], A->n_critic_layers, B));
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(A->actor, A->n_actor_layers, B));
    void* ws = A->workspace; const size_t ws_bytes = A->workspace_bytes;
    const float* obs = A->observations_actions_base;
    const rlt_dense_layer* critic = A->critics[0];
    int rc;
    if ((rc = rlt_rocm_mlp_forward(device, A->actor, A->n_actor_layers, obs, D, B))) return rc;
    const float* mean = A->actor[A->n_actor_layers - 1].output;
    hipLaunchKernelGGL(td3_actor_input_kernel, dim3(grid1((long)B * D)), dim3(256), 0, device->stream, mean, sampling_noise, A->sampling_std, A->final_step_mask, obs,
                       A->actor_pre_clip, A->state_action_value_input, B, OBS, ACT);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_mlp_forward(device, critic, A->n_critic_layers, A->state_action_value_input, D, B))) return rc;
    hipLaunchKernelGGL(td3_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, (float*)nullptr, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr,
                       (const uint8_t*)nullptr, 0.0f, 0, (float*)nullptr, A->final_step_mask, A->d_output_actor, B, 1);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_mlp_backward(device, critic, A->n_critic_layers, nullptr, 0, A->d_output_actor, 1, A->d_critic_input, D, B, 0, ws, ws_bytes))) return rc;
    hipLaunchKernelGGL(td3_actor_d_output_kernel, dim3(grid1((long)B * ACT)), dim3(256), 0, device->stream, A->d_critic_input, (const float*)A->actor_pre_clip,
                       A->final_step_mask, A->d_actor_output, B, OBS, ACT);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_mlp_zero_gradient(device, A->actor, A->n_actor_layers))) return rc;
    if ((rc = rlt_rocm_mlp_backward(device, A->actor, A->n_actor_layers, obs, D, A->d_actor_output, ACT, nullptr, 0, B, 1, ws, ws_bytes))) return rc;
    return rlt_rocm_adam_step(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, 0.0f, nullptr);
}

// rl/algorithms/td3/operations_generic.h:317-321
int rlt_rocm_td3_update_critic_targets(rlt_rocm_device* device, const rlt_td3_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A));
    for (int k = 0; k < 2; k++) { int rc = polyak_mlp(device, A->critics[k], A->critics_target[k], A->n_critic_layers, A->critic_polyak); if (rc) return rc; }
    return 0;
}

// rl/algorithms/td3/operations_generic.h:322-325
int rlt_rocm_td3_update_actor_target(rlt_rocm_device* device, const rlt_td3_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A));
    return polyak_mlp(device, A->actor, A->actor_target, A->n_actor_layers, A->actor_polyak);
}

}  // extern "C"

// ------------------------------------------------------------------------------------------------ TD3 on sequence batches
namespace {
__global__ __launch_bounds__(256) void td3_copy_columns_kernel(const float* __restrict__ src, int lds, float* __restrict__ dst, int ldd, int rows, int cols) {
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < (long)rows * cols; i += (long)gridDim.x * blockDim.x) {
        const long r = i / cols; const int c = (int)(i - r * cols);
        dst[r * ldd + c] = src[r * lds + c];
    }
}
int copy_columns(rlt_rocm_device* device, const float* src, int lds, float* dst, int ldd, int rows, int cols) {
    long blocks = ((long)rows * cols + 255) / 256; if (blocks > 4096) blocks = 4096; if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(td3_copy_columns_kernel, dim3((unsigned)blocks), dim3(256), 0, device->stream, src, lds, dst, ldd, rows, cols);
    return rlt_launch_status(device);
}
inline const float* seq_last_output(const rlt_seq_layer* layers, int n) { const rlt_seq_layer& L = layers[n - 1]; return L.kind ? L.gru.output : L.dense.output; }
inline int seq_last_dim(const rlt_seq_layer* layers, int n) { const rlt_seq_layer& L = layers[n - 1]; return L.kind ? L.gru.hidden_dim : L.dense.out_dim; }
// every tensor of a target network in one launch per sixteen tensors
int polyak_seq(rlt_rocm_device* device, const rlt_seq_layer* source, const rlt_seq_layer* target, int n, float polyak) {
    RLT_REQUIRE(n <= RLT_SEQ_MAX_LAYERS);
    const float* sources[5 * RLT_SEQ_MAX_LAYERS]; float* targets[5 * RLT_SEQ_MAX_LAYERS]; uint32_t counts[5 * RLT_SEQ_MAX_LAYERS];
    int m = 0;
    auto pair = [&](const float* from, float* to, size_t count) { sources[m] = from; targets[m] = to; counts[m++] = (uint32_t)count; };
    for (int l = 0; l < n; l++) {
        const rlt_seq_layer& s = source[l]; const rlt_seq_layer& t = target[l];
        RLT_REQUIRE(s.kind == t.kind);
        if (s.kind == 0) {
            pair(s.dense.weights, t.dense.weights, (size_t)s.dense.in_dim * s.dense.out_dim); pair(s.dense.biases, t.dense.biases, (size_t)s.dense.out_dim);
        } else {
            const size_t H = s.gru.hidden_dim, I = s.gru.input_dim;
            pair(s.gru.weights_input, t.gru.weights_input, 3 * H * I); pair(s.gru.biases_input, t.gru.biases_input, 3 * H);
            pair(s.gru.weights_hidden, t.gru.weights_hidden, 3 * H * H); pair(s.gru.biases_hidden, t.gru.biases_hidden, 3 * H);
            pair(s.gru.initial_hidden_state, t.gru.initial_hidden_state, H);
        }
    }
    for (int i = 0; i < m; i++) RLT_REQUIRE(sources[i] && targets[i]);
    return rlt_sac_polyak_list(device, sources, targets, counts, m, polyak);
}
bool td3_sequence_agent_ok(const rlt_td3_sequence_agent* A) {
    if (!A || A->observation_dim <= 0 || A->action_dim <= 0 || A->n_actor_layers < 1 || A->n_critic_layers < 1) return false;
    if (!A->actor || !A->actor_target || !A->critics[0] || !A->critics[1] || !A->critics_target[0] || !A->critics_target[1]) return false;
    const rlt_sequence_batch& K = A->batch;
    if (K.batch <= 0 || K.sequence_length <= 0 || !K.observations_actions_base || !K.rewards || !K.terminated || !K.reset || !K.next_reset_base || !K.final_step_mask ||
        !K.next_final_step_mask_base) return false;
    if (seq_last_dim(A->actor, A->n_actor_layers) != A->action_dim || seq_last_dim(A->actor_target, A->n_actor_layers) != A->action_dim) return false;
    for (int k = 0; k < 2; k++) if (seq_last_dim(A->critics[k], A->n_critic_layers) != 1 || seq_last_dim(A->critics_target[k], A->n_critic_layers) != 1) return false;
    if (!A->actor_input || !A->d_output) return false;
    return A->workspace && A->workspace_bytes >= rlt_rocm_td3_sequence_workspace_bytes(A);
}
}  // namespace

extern "C" {

// what one pass of any of the agent's networks needs, rounded up so that the second half of a doubled workspace is aligned like the first
static size_t td3_sequence_pass_workspace_bytes(const rlt_td3_sequence_agent* A) {
    const int T = A->batch.sequence_length + 1, B = A->batch.batch;
    size_t n = rlt_rocm_seq_workspace_bytes(A->actor, A->n_actor_layers, T, B);
    n = std::max(n, rlt_rocm_seq_workspace_bytes(A->actor_target, A->n_actor_layers, T, B));
    n = std::max(n, rlt_rocm_seq_workspace_bytes(A->critics[0], A->n_critic_layers, T, B));
    n = std::max(n, rlt_rocm_seq_workspace_bytes(A->critics_target[0], A->n_critic_layers, T, B));
    return (n + 255) & ~(size_t)255;
}
size_t rlt_rocm_td3_sequence_workspace_bytes(const rlt_td3_sequence_agent* A) {
    if (!A || !A->actor || !A->actor_target || !A->critics[0] || !A->critics_target[0]) return 0;
    // three passes may run at the same time (rlt_side_begin), each in its own part; behind them the first critic's loss gradient of rlt_rocm_td3_sequence_train_critics
    return 3 * td3_sequence_pass_workspace_bytes(A) + (((size_t)A->batch.sequence_length * A->batch.batch * sizeof(float) + 255) & ~(size_t)255);
}

// rl/algorithms/td3/operations_generic.h:170-235 on a sequence batch, one launch per reference operation
int rlt_rocm_td3_sequence_train_critic(rlt_rocm_device* device, const rlt_td3_sequence_agent* A, int ci) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(td3_sequence_agent_ok(A) && (ci == 0 || ci == 1));
    RLT_REQUIRE(A->target_next_action_noise && A->next_state_action_value_input && A->next_q[0] && A->next_q[1] && A->target_action_value);
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const int first = A->include_first_step_in_targets ? 1 : 0, T = S + first, next_offset = first ? 0 : 1;   // off_policy_runner/operations_generic.h:85-92
    const rlt_seq_layer* critic = A->critics[ci];
    // passes that do not depend on each other run at the same time, one on the handle's side stream, each in its own half of the workspace: the trained critic's
    // forward pass next to the target actor's, then the second target critic next to the first
    const size_t ws_bytes = td3_sequence_pass_workspace_bytes(A);
    void* ws = A->workspace; void* ws_side = (char*)A->workspace + ws_bytes;
    const bool overlap = S >= 48;      // short sequences: a pass is shorter than the two events that fork and join a stream cost on the host
    int rc;
    if ((rc = rlt_rocm_seq_zero_gradient(device, critic, A->n_critic_layers))) return rc;                                                  // :185
    {
        const bool side = overlap && rlt_side_begin(device);
        rc = rlt_rocm_seq_forward(device, critic, A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B, side ? ws_side : ws, ws_bytes);   // :205
        rlt_side_end(device);
        if (rc) return rc;
    }
    const float* base_next = K.observations_actions_base + (size_t)next_offset * B * D;
    const uint8_t* next_reset = K.next_reset_base + (size_t)next_offset * B;
    const uint8_t* next_final = K.next_final_step_mask_base + (size_t)next_offset * B;
    if ((rc = copy_columns(device, base_next, D, A->actor_input, OBS, T * B, OBS))) return rc;                                             // the observation columns, contiguous
    if ((rc = rlt_rocm_seq_forward(device, A->actor_target, A->n_actor_layers, A->actor_input, OBS, next_reset, T, B, ws, ws_bytes))) return rc;   // :191
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = copy_columns(device, seq_last_output(A->actor_target, A->n_actor_layers), ACT, next_actions, D, T * B, ACT))) return rc;
    if ((rc = rlt_rocm_td3_noisy_next_actions(device, next_actions, D, A->target_next_action_noise, ACT, T * B, ACT))) return rc;          // :192
    if ((rc = rlt_rocm_mask_copy(device, base_next + OBS, D, next_actions, D, next_final, 1, T * B, ACT))) return rc;                      // :193-195
    if ((rc = copy_columns(device, base_next, D, A->next_state_action_value_input, D, T * B, OBS))) return rc;                             // :196
    for (int k = 1; k >= 0; k--) {                                                                                                         // :197-198 (target critic 1 on the side stream)
        const bool side = k == 1 && overlap && rlt_side_begin(device);
        rc = rlt_rocm_seq_forward(device, A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, next_reset, T, B, side ? ws_side : ws, ws_bytes);
        if (!rc) rc = rlt_rocm_memcpy_d2d(device, A->next_q[k], seq_last_output(A->critics_target[k], A->n_critic_layers), sizeof(float) * T * B);
        rlt_side_end(device);
        if (rc) return rc;
    }
    if (overlap && (rc = rlt_side_join(device))) return rc;
    // :200-227: targets from the value of the step after (offset B where the first step is included), reweighted and masked gradient
    hipLaunchKernelGGL(td3_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, const_cast<float*>(seq_last_output(critic, A->n_critic_layers)),
                       (const float*)(A->next_q[0] + (size_t)first * B), (const float*)(A->next_q[1] + (size_t)first * B), (const float*)K.rewards, (const uint8_t*)K.terminated,
                       A->gamma, A->ignore_termination, A->target_action_value, (const uint8_t*)K.final_step_mask, A->d_output, S * B, 0);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_seq_backward(device, critic, A->n_critic_layers, K.observations_actions_base, D, A->d_output, nullptr, K.reset, S, B, 1, 0, ws, ws_bytes))) return rc;   // :233
    return rlt_rocm_adam_step(device, A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], 0.0f, nullptr);   // :234
}

// rlt_rocm_td3_sequence_train_critic for critic 0 and then for critic 1 on one batch and one target noise (the loop's shared batch, td3/loop/core/operations_generic.h:98-112):
// what the second call would repeat (the target actor's pass, the noisy next actions, both target critics' passes, the targets) is computed once, and the passes that do
// not depend on each other run side by side: critic 0's forward pass and then target critic 1 on one side stream, critic 1's forward pass on the other, the target actor
// and target critic 0 on the main stream; then the two backward passes side by side. Same results bit for bit (every pass is the same launches on the same inputs).
int rlt_rocm_td3_sequence_train_critics(rlt_rocm_device* device, const rlt_td3_sequence_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(td3_sequence_agent_ok(A));
    RLT_REQUIRE(A->target_next_action_noise && A->next_state_action_value_input && A->next_q[0] && A->next_q[1] && A->target_action_value);
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const int first = A->include_first_step_in_targets ? 1 : 0, T = S + first, next_offset = first ? 0 : 1;
    const size_t ws_bytes = td3_sequence_pass_workspace_bytes(A);
    void* ws = A->workspace; void* ws_side = (char*)A->workspace + ws_bytes; void* ws_second = (char*)A->workspace + 2 * ws_bytes;
    float* d_output_first = (float*)((char*)A->workspace + 3 * ws_bytes);      // critic 0's loss gradient; critic 1's goes to the agent's buffer, where two single calls leave it
    const bool overlap = S >= 48;
    int rc;
    for (int k = 0; k < 2; k++) if ((rc = rlt_rocm_seq_zero_gradient(device, A->critics[k], A->n_critic_layers))) return rc;
    {
        if (overlap) rlt_side_begin(device);      // (without a second stream everything below simply runs in order on the one stream)
        rc = rlt_rocm_seq_forward(device, A->critics[0], A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B, device->side_return ? ws_side : ws, ws_bytes);
        rlt_side_end(device);
        if (rc) return rc;
        if (overlap) rlt_side_begin(device, 1);
        rc = rlt_rocm_seq_forward(device, A->critics[1], A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B, device->side_return ? ws_second : ws, ws_bytes);
        rlt_side_end(device);
        if (rc) return rc;
    }
    const float* base_next = K.observations_actions_base + (size_t)next_offset * B * D;
    const uint8_t* next_reset = K.next_reset_base + (size_t)next_offset * B;
    const uint8_t* next_final = K.next_final_step_mask_base + (size_t)next_offset * B;
    if ((rc = copy_columns(device, base_next, D, A->actor_input, OBS, T * B, OBS))) return rc;
    if ((rc = rlt_rocm_seq_forward(device, A->actor_target, A->n_actor_layers, A->actor_input, OBS, next_reset, T, B, ws, ws_bytes))) return rc;
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = copy_columns(device, seq_last_output(A->actor_target, A->n_actor_layers), ACT, next_actions, D, T * B, ACT))) return rc;
    if ((rc = rlt_rocm_td3_noisy_next_actions(device, next_actions, D, A->target_next_action_noise, ACT, T * B, ACT))) return rc;
    if ((rc = rlt_rocm_mask_copy(device, base_next + OBS, D, next_actions, D, next_final, 1, T * B, ACT))) return rc;
    if ((rc = copy_columns(device, base_next, D, A->next_state_action_value_input, D, T * B, OBS))) return rc;
    for (int k = 1; k >= 0; k--) {      // target critic 1 behind critic 0's forward pass on the side stream (it waits for the copies above), target critic 0 on the main stream
        if (k == 1 && overlap) rlt_side_begin(device);
        rc = rlt_rocm_seq_forward(device, A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, next_reset, T, B, device->side_return ? ws_side : ws, ws_bytes);
        if (!rc) rc = rlt_rocm_memcpy_d2d(device, A->next_q[k], seq_last_output(A->critics_target[k], A->n_critic_layers), sizeof(float) * T * B);
        rlt_side_end(device);
        if (rc) return rc;
    }
    if (overlap && (rc = rlt_side_join(device))) return rc;
    for (int k = 0; k < 2; k++) {
        hipLaunchKernelGGL(td3_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, const_cast<float*>(seq_last_output(A->critics[k], A->n_critic_layers)),
                           (const float*)(A->next_q[0] + (size_t)first * B), (const float*)(A->next_q[1] + (size_t)first * B), (const float*)K.rewards, (const uint8_t*)K.terminated,
                           A->gamma, A->ignore_termination, A->target_action_value, (const uint8_t*)K.final_step_mask, k ? A->d_output : d_output_first, S * B, 0);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    {
        if (overlap) rlt_side_begin(device);
        rc = rlt_rocm_seq_backward(device, A->critics[1], A->n_critic_layers, K.observations_actions_base, D, A->d_output, nullptr, K.reset, S, B, 1, 0, device->side_return ? ws_side : ws, ws_bytes);
        rlt_side_end(device);
        if (rc) return rc;
    }
    if ((rc = rlt_rocm_seq_backward(device, A->critics[0], A->n_critic_layers, K.observations_actions_base, D, d_output_first, nullptr, K.reset, S, B, 1, 0, ws, ws_bytes))) return rc;
    if (overlap && (rc = rlt_side_join(device))) return rc;
    for (int k = 0; k < 2; k++)
        if ((rc = rlt_rocm_adam_step(device, A->critic_adam_tensors[k], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[k], 0.0f, nullptr))) return rc;
    return 0;
}

// td3/operations_generic.h:236-281 on a sequence batch
int rlt_rocm_td3_sequence_train_actor(rlt_rocm_device* device, const rlt_td3_sequence_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(td3_sequence_agent_ok(A) && A->state_action_value_input && A->d_critic_input && A->d_actor_output && A->actor_adam_tensors && A->actor_age);
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT, R = S * B;
    const float* obs = K.observations_actions_base;
    void* ws = A->workspace; const size_t ws_bytes = A->workspace_bytes;
    int rc;
    if ((rc = copy_columns(device, obs, D, A->actor_input, OBS, R, OBS))) return rc;
    if ((rc = rlt_rocm_seq_forward(device, A->actor, A->n_actor_layers, A->actor_input, OBS, K.reset, S, B, ws, ws_bytes))) return rc;      // :255
    float* sav_actions = A->state_action_value_input + OBS;
    if ((rc = copy_columns(device, seq_last_output(A->actor, A->n_actor_layers), ACT, sav_actions, D, R, ACT))) return rc;
    if ((rc = rlt_rocm_mask_copy(device, obs + OBS, D, sav_actions, D, K.final_step_mask, 1, R, ACT))) return rc;                          // :256-258
    if ((rc = copy_columns(device, obs, D, A->state_action_value_input, D, R, OBS))) return rc;                                            // :259
    const rlt_seq_layer* critic = A->critics[0];
    if ((rc = rlt_rocm_seq_forward(device, critic, A->n_critic_layers, A->state_action_value_input, D, K.reset, S, B, ws, ws_bytes))) return rc;   // :261
    hipLaunchKernelGGL(td3_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, (float*)nullptr, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr,
                       (const uint8_t*)nullptr, 0.0f, 0, (float*)nullptr, (const uint8_t*)K.final_step_mask, A->d_output, R, 1);           // :262-267
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_seq_backward(device, critic, A->n_critic_layers, nullptr, 0, A->d_output, A->d_critic_input, K.reset, S, B, 0, 0, ws, ws_bytes))) return rc;   // :271
    if ((rc = copy_columns(device, A->d_critic_input + OBS, D, A->d_actor_output, ACT, R, ACT))) return rc;                                // :272
    if ((rc = rlt_rocm_mask_zero(device, A->d_actor_output, ACT, K.final_step_mask, 1, R, ACT))) return rc;                                // :273-275
    if ((rc = rlt_rocm_seq_zero_gradient(device, A->actor, A->n_actor_layers))) return rc;                                                 // :277
    if ((rc = rlt_rocm_seq_backward(device, A->actor, A->n_actor_layers, A->actor_input, OBS, A->d_actor_output, nullptr, K.reset, S, B, 1, 0, ws, ws_bytes))) return rc;   // :278
    return rlt_rocm_adam_step(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, 0.0f, nullptr);        // :280
}

// td3/operations_generic.h:283-325
int rlt_rocm_td3_sequence_update_critic_targets(rlt_rocm_device* device, const rlt_td3_sequence_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(td3_sequence_agent_ok(A));
    int rc;
    for (int k = 0; k < 2; k++)
        if ((rc = polyak_seq(device, A->critics[k], A->critics_target[k], A->n_critic_layers, A->critic_polyak))) return rc;
    return 0;
}
int rlt_rocm_td3_sequence_update_actor_target(rlt_rocm_device* device, const rlt_td3_sequence_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(td3_sequence_agent_ok(A));
    return polyak_seq(device, A->actor, A->actor_target, A->n_actor_layers, A->actor_polyak);
}

}  // extern "C"
