// Replay buffer add / gather_batch, batched Pendulum dynamics and the off-policy runner step.
// reference: rl/components/replay_buffer/operations_generic.h:54-78, rl/components/off_policy_runner/operations_generic.h:183-430
//            (CUDA :14-230), operations_generic_per_env.h:8-108, rl/environments/pendulum/operations_generic.h:14-160.
#include "common.h"

namespace {

__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }

struct Transition { float obs[3]; float next_obs[3]; float action, reward; float theta, theta_dot; };

// pendulum/operations_generic.h:79-101 (step), :131-139 (reward from the pre-step state and the un-clamped action),
// :142-160 (Fourier observation)
__device__ __forceinline__ void pendulum_transition(const rlt_pendulum_parameters& p, float theta, float theta_dot, float action, Transition& t) {
    sincosf(theta, &t.obs[1], &t.obs[0]);
    t.obs[2] = theta_dot;
    float u = p.max_torque * clampf(action, -1.0f, 1.0f);
    u = clampf(u, -p.max_torque, p.max_torque);
    float newthdot = theta_dot + (3.0f * p.g / (2.0f * p.l) * t.obs[1] + 3.0f / (p.m * p.l * p.l) * u) * p.dt;
    newthdot = clampf(newthdot, -p.max_speed, p.max_speed);
    float newth = theta + newthdot * p.dt;
    const float PI = 3.14159265358979323846f;
    float a = theta + PI, b = 2.0f * PI;
    float angle_norm = (a - b * floorf(a / b)) - PI;
    float ur = p.max_torque * action;
    t.reward = -(angle_norm * angle_norm + 0.1f * theta_dot * theta_dot + 0.001f * (ur * ur));
    sincosf(newth, &t.next_obs[1], &t.next_obs[0]);
    t.next_obs[2] = newthdot;
    t.theta = newth; t.theta_dot = newthdot; t.action = action;
}

__global__ __launch_bounds__(256) void pendulum_step_kernel(rlt_pendulum_parameters p, float* __restrict__ states, const float* __restrict__ actions,
                                                            float* __restrict__ observations, float* __restrict__ next_observations, float* __restrict__ rewards, int n) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        Transition t;
        pendulum_transition(p, states[2 * e], states[2 * e + 1], actions[e], t);
        if (observations) { observations[3 * (size_t)e] = t.obs[0]; observations[3 * (size_t)e + 1] = t.obs[1]; observations[3 * (size_t)e + 2] = t.obs[2]; }
        if (next_observations) { next_observations[3 * (size_t)e] = t.next_obs[0]; next_observations[3 * (size_t)e + 1] = t.next_obs[1]; next_observations[3 * (size_t)e + 2] = t.next_obs[2]; }
        if (rewards) rewards[e] = t.reward;
        states[2 * e] = t.theta; states[2 * e + 1] = t.theta_dot;
    }
}

// replay_buffer/operations_generic.h:54-78, thread per environment (each environment owns its ring)
__global__ __launch_bounds__(256) void replay_add_kernel(rlt_replay_buffer rb, const float* __restrict__ obs, const float* __restrict__ actions, const float* __restrict__ rewards,
                                                         const float* __restrict__ next_obs, const uint8_t* __restrict__ terminated, const uint8_t* __restrict__ truncated) {
    const int OBS = rb.observation_dim, ACT = rb.action_dim, R = 2 * OBS + ACT + 3;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rb.n_envs; e += gridDim.x * blockDim.x) {
        uint32_t pos = rb.position[e];
        float* row = rb.data + ((size_t)e * rb.capacity + pos) * R;
        for (int i = 0; i < OBS; i++) { row[i] = obs[(size_t)e * OBS + i]; row[OBS + ACT + 1 + i] = next_obs[(size_t)e * OBS + i]; }
        for (int i = 0; i < ACT; i++) row[OBS + i] = actions[(size_t)e * ACT + i];
        row[OBS + ACT] = rewards[e];
        row[2 * OBS + ACT + 1] = terminated[e] ? 1.0f : 0.0f;
        row[2 * OBS + ACT + 2] = truncated[e] ? 1.0f : 0.0f;
        rb.episode_start[(size_t)e * rb.capacity + pos] = rb.current_episode_start[e];
        pos = (pos + 1) % (uint32_t)rb.capacity;
        rb.position[e] = pos;
        if (truncated[e]) rb.current_episode_start[e] = pos;
        if (pos == 0 && !rb.full[e]) rb.full[e] = 1;
    }
}

// off_policy_runner/operations_generic.h:240-430 for SEQUENCE_LENGTH = 1: 16 lanes cooperate on one sample so that a replay
// row (2*obs+act+3 floats) is read as one contiguous segment and each batch row is written contiguously.
__global__ __launch_bounds__(256) void gather_kernel(rlt_replay_buffer rb, const uint32_t* __restrict__ env_indices, const uint32_t* __restrict__ sample_offsets,
                                                     int deterministic, int max_episode_length, int batch, float* __restrict__ oab, float* __restrict__ rewards,
                                                     uint8_t* __restrict__ terminated, uint8_t* __restrict__ reset, uint8_t* __restrict__ next_reset_base,
                                                     uint8_t* __restrict__ final_step_mask, uint8_t* __restrict__ next_final_step_mask_base, int* __restrict__ error_flag) {
    const int OBS = rb.observation_dim, ACT = rb.action_dim, R = 2 * OBS + ACT + 3, D = OBS + ACT;
    const int sub = threadIdx.x & 15;
    for (int i = (blockIdx.x * blockDim.x + threadIdx.x) >> 4; i < batch; i += (gridDim.x * blockDim.x) >> 4) {
        uint32_t e = deterministic ? 0u : env_indices[i];
        uint32_t offset = deterministic ? (uint32_t)i : sample_offsets[i];
        if (e >= (uint32_t)rb.n_envs) { if (sub == 0) *error_flag = 1; continue; }
        uint32_t index = rb.full[e] ? (rb.position[e] + (uint32_t)max_episode_length + offset) % (uint32_t)rb.capacity : offset;
        if (index >= (uint32_t)rb.capacity) { if (sub == 0) *error_flag = 1; continue; }
        const float* row = rb.data + ((size_t)e * rb.capacity + index) * R;
        float* step0 = oab + (size_t)i * D; float* step1 = oab + ((size_t)batch + i) * D;
        for (int j = sub; j < R; j += 16) {
            float v = row[j];
            if (j < D) step0[j] = v;                                   // observation and action of padded step 0
            else if (j == D) rewards[i] = v;
            else if (j < D + 1 + OBS) step1[j - D - 1] = v;            // next observation into padded step 1
            else if (j == D + 1 + OBS) terminated[i] = v != 0.0f;
        }
        for (int j = sub; j < ACT; j += 16) step1[OBS + j] = 0.0f;     // next action zeroed
        if (sub == 0) {
            if (reset) reset[i] = 1;
            if (next_reset_base) { next_reset_base[i] = 1; next_reset_base[batch + i] = 1; }
            if (final_step_mask) final_step_mask[i] = 1;
            if (next_final_step_mask_base) { next_final_step_mask_base[i] = 0; next_final_step_mask_base[batch + i] = 1; }
        }
    }
}

__device__ __forceinline__ uint32_t mix32(uint64_t x) {   // splitmix64 finaliser
    x += 0x9E3779B97F4A7C15ull; x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull; x = (x ^ (x >> 27)) * 0x94D049BB133111EBull; x ^= x >> 31;
    return (uint32_t)(x >> 32);
}
__global__ __launch_bounds__(256) void gather_draw_kernel(rlt_replay_buffer rb, int batch, uint64_t seed, uint64_t offset, uint32_t* __restrict__ env_indices, uint32_t* __restrict__ sample_offsets) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch; i += gridDim.x * blockDim.x) {
        uint32_t r0 = mix32(seed ^ ((offset + (uint64_t)i) * 2u)), r1 = mix32(seed ^ ((offset + (uint64_t)i) * 2u + 1u));
        uint32_t e = (uint32_t)(((uint64_t)r0 * (uint32_t)rb.n_envs) >> 32);
        uint32_t eligible = rb.full[e] ? (uint32_t)rb.capacity : rb.position[e];
        env_indices[i] = e;
        sample_offsets[i] = eligible ? (uint32_t)(((uint64_t)r1 * eligible) >> 32) : 0u;
    }
}

// prologue of the runner step (operations_generic_per_env.h:8-66): reset where truncated, flag the previous replay row, observe
__global__ __launch_bounds__(256) void runner_prologue_kernel(rlt_pendulum_runner rn, rlt_replay_buffer rb, const float* __restrict__ initial_states, uint64_t seed, uint64_t offset,
                                                              float* __restrict__ observations) {
    const int R = 2 * rb.observation_dim + rb.action_dim + 3;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        if (rn.truncated[e]) {
            float th, thd;
            if (initial_states) { th = initial_states[2 * e]; thd = initial_states[2 * e + 1]; }
            else {
                const float PI = 3.14159265358979323846f;
                float u0 = ((mix32(seed ^ ((offset + (uint64_t)e) * 2u)) >> 8) + 0.5f) * (1.0f / 16777216.0f);
                float u1 = ((mix32(seed ^ ((offset + (uint64_t)e) * 2u + 1u)) >> 8) + 0.5f) * (1.0f / 16777216.0f);
                th = -PI + 2.0f * PI * u0; thd = -1.0f + 2.0f * u1;
            }
            rn.states[2 * e] = th; rn.states[2 * e + 1] = thd;
            rn.episode_step[e] = 0; rn.episode_return[e] = 0.0f;
            if (rb.full[e] || rb.position[e] > 0) {
                uint32_t prev = rb.position[e] == 0 ? (uint32_t)rb.capacity - 1 : rb.position[e] - 1;
                rb.data[((size_t)e * rb.capacity + prev) * R + (R - 1)] = 1.0f;
                rb.current_episode_start[e] = rb.position[e];
            }
        }
        float s, c;
        sincosf(rn.states[2 * e], &s, &c);
        observations[3 * (size_t)e] = c; observations[3 * (size_t)e + 1] = s; observations[3 * (size_t)e + 2] = rn.states[2 * e + 1];
    }
}
// epilogue (operations_generic_per_env.h:67-108): env step, reward, next observation, truncation, replay add
__global__ __launch_bounds__(256) void runner_epilogue_kernel(rlt_pendulum_runner rn, rlt_replay_buffer rb, const float* __restrict__ actions) {
    const int R = 10;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        Transition t;
        pendulum_transition(rn.env, rn.states[2 * e], rn.states[2 * e + 1], actions[e], t);
        uint32_t step = rn.episode_step[e] + 1;
        rn.episode_step[e] = step;
        rn.episode_return[e] += t.reward;
        const bool truncated = step == (uint32_t)rn.episode_step_limit;
        rn.truncated[e] = truncated;
        rn.states[2 * e] = t.theta; rn.states[2 * e + 1] = t.theta_dot;
        uint32_t pos = rb.position[e];
        float* row = rb.data + ((size_t)e * rb.capacity + pos) * R;
        row[0] = t.obs[0]; row[1] = t.obs[1]; row[2] = t.obs[2]; row[3] = t.action; row[4] = t.reward;
        row[5] = t.next_obs[0]; row[6] = t.next_obs[1]; row[7] = t.next_obs[2]; row[8] = 0.0f; row[9] = truncated ? 1.0f : 0.0f;
        rb.episode_start[(size_t)e * rb.capacity + pos] = rb.current_episode_start[e];
        pos = (pos + 1) % (uint32_t)rb.capacity;
        rb.position[e] = pos;
        if (truncated) rb.current_episode_start[e] = pos;
        if (pos == 0 && !rb.full[e]) rb.full[e] = 1;
    }
}

int grid1(int n) { int b = (n + 255) / 256; return b > 2048 ? 2048 : (b < 1 ? 1 : b); }
bool rb_ok(const rlt_replay_buffer* rb) {
    return rb && rb->data && rb->episode_start && rb->position && rb->current_episode_start && rb->full && rb->n_envs > 0 && rb->capacity > 0 &&
           rb->observation_dim > 0 && rb->action_dim > 0;
}

}  // namespace

extern "C" {

int rlt_rocm_replay_add(rlt_rocm_device* device, const rlt_replay_buffer* rb, const float* observations, const float* actions, const float* rewards,
                        const float* next_observations, const uint8_t* terminated, const uint8_t* truncated) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && observations && actions && rewards && next_observations && terminated && truncated);
    hipLaunchKernelGGL(replay_add_kernel, dim3(grid1(rb->n_envs)), dim3(256), 0, device->stream, *rb, observations, actions, rewards, next_observations, terminated, truncated);
    return rlt_launch_status(device);
}

int rlt_rocm_gather_batch(rlt_rocm_device* device, const rlt_replay_buffer* rb, const uint32_t* env_indices, const uint32_t* sample_offsets, int deterministic,
                          int max_episode_length, int batch, float* observations_actions_base, float* rewards, uint8_t* terminated,
                          uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && batch > 0 && observations_actions_base && rewards && terminated && max_episode_length >= 0);
    RLT_REQUIRE(deterministic || (env_indices && sample_offsets));
    void* counters; int rc = rlt_counters(device, &counters); if (rc) return rc;
    int* error_flag = (int*)((char*)counters + 128);
    hipLaunchKernelGGL(gather_kernel, dim3(grid1(batch * 16)), dim3(256), 0, device->stream, *rb, env_indices, sample_offsets, deterministic, max_episode_length, batch,
                       observations_actions_base, rewards, terminated, reset, next_reset_base, final_step_mask, next_final_step_mask_base, error_flag);
    return rlt_launch_status(device);
}

int rlt_rocm_gather_draw(rlt_rocm_device* device, const rlt_replay_buffer* rb, int batch, uint64_t seed, uint64_t offset, uint32_t* env_indices, uint32_t* sample_offsets) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && batch > 0 && env_indices && sample_offsets);
    hipLaunchKernelGGL(gather_draw_kernel, dim3(grid1(batch)), dim3(256), 0, device->stream, *rb, batch, seed, offset, env_indices, sample_offsets);
    return rlt_launch_status(device);
}

int rlt_rocm_pendulum_step(rlt_rocm_device* device, const rlt_pendulum_parameters* p, float* states, const float* actions, float* observations,
                           float* next_observations, float* rewards, int n_envs) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(p && states && actions && n_envs > 0);
    hipLaunchKernelGGL(pendulum_step_kernel, dim3(grid1(n_envs)), dim3(256), 0, device->stream, *p, states, actions, observations, next_observations, rewards, n_envs);
    return rlt_launch_status(device);
}

int rlt_rocm_pendulum_runner_step(rlt_rocm_device* device, const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, int policy_kind,
                                  const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas, const float* actions_in, const float* action_noise,
                                  const float* initial_states, uint64_t seed, uint64_t offset) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rn->states && rn->episode_step && rn->episode_return && rn->truncated && rn->n_envs > 0 && rb_ok(rb));
    RLT_REQUIRE(rn->n_envs == rb->n_envs && rb->observation_dim == 3 && rb->action_dim == 1 && policy_kind >= 0 && policy_kind <= 2);
    RLT_REQUIRE(policy_kind != 0 || actions_in);
    RLT_REQUIRE(policy_kind == 0 || (actor && n_actor_layers >= 1 && actor[0].in_dim == 3 && actor[n_actor_layers - 1].out_dim == (policy_kind == 2 ? 2 : 1)));
    RLT_REQUIRE(policy_kind != 2 || (sas && action_noise));
    const int N = rn->n_envs;
    // scratch: observations [N x 3], actor output [N x 2], actions [N], log-probs [N], then the MLP workspace
    size_t mlp_ws = policy_kind ? rlt_rocm_mlp_workspace_bytes(actor, n_actor_layers, N) : 0;
    size_t head = (((size_t)N * 7 * sizeof(float)) + 255) & ~(size_t)255;
    void* scratch; int rc = rlt_scratch(device, head + mlp_ws, &scratch); if (rc) return rc;
    float* obs = (float*)scratch; float* actor_out = obs + (size_t)N * 3; float* actions = actor_out + (size_t)N * 2; float* lp = actions + N;
    void* ws = (char*)scratch + head;
    hipLaunchKernelGGL(runner_prologue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *rb, initial_states, seed, offset, obs);
    if ((rc = rlt_launch_status(device))) return rc;
    const float* act_ptr = actions;
    if (policy_kind == 0) act_ptr = actions_in;
    else if (policy_kind == 1) { if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, obs, 3, actions, 1, N, ws, mlp_ws))) return rc; }
    else {
        if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, obs, 3, actor_out, 2, N, ws, mlp_ws))) return rc;
        if ((rc = rlt_rocm_sas_forward(device, sas, actor_out, 2, action_noise, 1, actions, 1, nullptr, 0, lp, N, 1))) return rc;
    }
    hipLaunchKernelGGL(runner_epilogue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *rb, act_ptr);
    return rlt_launch_status(device);
}

}  // extern "C"
