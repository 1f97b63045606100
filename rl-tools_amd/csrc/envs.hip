// Analytic environments other than the Pendulum as batched kernels, one lane per environment: the Acrobot and the Car.
// Acrobot / AcrobotSwingup: rl/environments/acrobot/operations_generic.h:56-117 (dsdt, rk4), :118-144 (step), :145-171 (reward),
// :173-193 (observe, terminated). The reference evaluates parts of dsdt in double (double literals and the double cos / sin); the kernel computes in
// fp32 throughout, which stays within 1e-5 relative of it per step. 4 Runge-Kutta stages of ~60 flop: the kernel is bound by its 52 bytes per
// environment (state in and out, observations, reward, flag) once there are enough environments to fill the device.
#include "common.h"
#include "pendulum.h"
#include "rng.h"
#include "sac_heads.h"

namespace {
struct Acrobot4 { float v[4]; };
__device__ __forceinline__ float angle_normalize(float x) {
    const float PI = 3.14159265358979323846f;
    const float a = x + PI, b = 2.0f * PI;
    return (a - b * floorf(a / b)) - PI;
}
__device__ __forceinline__ Acrobot4 acrobot_dsdt(const rlt_acrobot_parameters& P, const Acrobot4& s, float action) {
    const float m1 = P.link_mass_1, m2 = P.link_mass_2, l1 = P.link_length_1, lc1 = P.link_com_pos_1, lc2 = P.link_com_pos_2, I1 = P.link_moi, I2 = P.link_moi;
    const float g = 9.8f, HALF_PI = 1.57079632679489661923f;
    const float theta1 = s.v[0], theta2 = s.v[1], dtheta1 = s.v[2], dtheta2 = s.v[3];
    float s2, c2;
    sincosf(theta2, &s2, &c2);
    const float d1 = m1 * lc1 * lc1 + m2 * (l1 * l1 + lc2 * lc2 + 2.0f * l1 * lc2 * c2) + I1 + I2;
    const float d2 = m2 * (lc2 * lc2 + l1 * lc2 * c2) + I2;
    const float phi2 = m2 * lc2 * g * cosf(theta1 + theta2 - HALF_PI);
    const float phi1 = -m2 * l1 * lc2 * dtheta2 * dtheta2 * s2 - 2.0f * m2 * l1 * lc2 * dtheta2 * dtheta1 * s2 + (m1 * lc1 + m2 * l1) * g * cosf(theta1 - HALF_PI) + phi2;
    const float ddtheta2 = (action + d2 / d1 * phi1 - m2 * l1 * lc2 * dtheta1 * dtheta1 * s2 - phi2) / (m2 * lc2 * lc2 + I2 - d2 * d2 / d1);
    const float ddtheta1 = -(d2 * ddtheta2 + phi1) / d1;
    return {{dtheta1, dtheta2, ddtheta1, ddtheta2}};
}
__device__ __forceinline__ Acrobot4 axpy(const Acrobot4& s, float a, const Acrobot4& k) { return {{s.v[0] + a * k.v[0], s.v[1] + a * k.v[1], s.v[2] + a * k.v[2], s.v[3] + a * k.v[3]}}; }
__device__ __forceinline__ void acrobot_observe(const Acrobot4& s, float* __restrict__ o) {
    float sn, cs;
    sincosf(s.v[0], &sn, &cs); o[0] = cs; o[1] = sn;
    sincosf(s.v[1], &sn, &cs); o[2] = cs; o[3] = sn;
    o[4] = s.v[2]; o[5] = s.v[3];
}

// one environment's step: Runge-Kutta over one time step (:98-117), reward, flag, observations
__device__ __forceinline__ void acrobot_step_one(const rlt_acrobot_parameters& P, int swingup, float* __restrict__ states, const float* __restrict__ actions,
                                                 float* __restrict__ observations, float* __restrict__ next_observations, float* __restrict__ rewards,
                                                 uint8_t* __restrict__ terminated, int e) {
    const float PI = 3.14159265358979323846f;
    const float4 raw = reinterpret_cast<const float4*>(states)[e];
    const Acrobot4 s = {{raw.x, raw.y, raw.z, raw.w}};
    if (observations) acrobot_observe(s, observations + 6 * (size_t)e);
    const float action = (clampf(actions[e], -1.0f, 1.0f) + 1.0f) / 2.0f * (P.max_torque - P.min_torque) + P.min_torque;
    const Acrobot4 k1 = acrobot_dsdt(P, s, action);
    const Acrobot4 k2 = acrobot_dsdt(P, axpy(s, P.dt / 2.0f, k1), action);
    const Acrobot4 k3 = acrobot_dsdt(P, axpy(s, P.dt / 2.0f, k2), action);
    const Acrobot4 k4 = acrobot_dsdt(P, axpy(s, P.dt, k3), action);
    Acrobot4 next;
#pragma unroll
    for (int i = 0; i < 4; i++) next.v[i] = s.v[i] + P.dt / 6.0f * (k1.v[i] + 2.0f * k2.v[i] + 2.0f * k3.v[i] + k4.v[i]);
    next.v[0] = angle_normalize(next.v[0]); next.v[1] = angle_normalize(next.v[1]);
    next.v[2] = clampf(next.v[2], -P.max_vel_1, P.max_vel_1); next.v[3] = clampf(next.v[3], -P.max_vel_2, P.max_vel_2);
    if (rewards) rewards[e] = swingup ? (-fabsf(angle_normalize(next.v[0] - PI)) - fabsf(angle_normalize(next.v[1]))) / 100.0f * P.dt / 0.02f : -1.0f;
    if (terminated) terminated[e] = swingup ? 0 : ((-cosf(next.v[0]) - cosf(next.v[1] + next.v[0])) > 1.0f);
    if (next_observations) acrobot_observe(next, next_observations + 6 * (size_t)e);
    reinterpret_cast<float4*>(states)[e] = make_float4(next.v[0], next.v[1], next.v[2], next.v[3]);
}
__global__ __launch_bounds__(256) void acrobot_step_kernel(rlt_acrobot_parameters P, int swingup, float* __restrict__ states, const float* __restrict__ actions,
                                                           float* __restrict__ observations, float* __restrict__ next_observations, float* __restrict__ rewards,
                                                           uint8_t* __restrict__ terminated, int n) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x)
        acrobot_step_one(P, swingup, states, actions, observations, next_observations, rewards, terminated, e);
}

// Car: single-track model with Pacejka tire forces, explicit Euler over dt (rl/environments/car/operations_generic.h:99-127)
struct Car6 { float x, y, mu, vx, vy, omega; };
__device__ __forceinline__ Car6 car_dynamics(const rlt_car_parameters& p, const Car6& s, float2 a) {
    const float throttle_break = clampf(a.x, -1.0f, 1.0f), delta = clampf(a.y, -1.0f, 1.0f);
    const float alpha_f = atan2f(s.vy + p.lf * s.omega, s.vx) - delta;
    const float alpha_r = atan2f(s.vy - p.lr * s.omega, s.vx);
    const float FnF = p.lr / (p.lf + p.lr) * p.m * p.g, FnR = p.lf / (p.lf + p.lr) * p.m * p.g;
    const bool moving = s.vx > p.vt || s.vy > p.vt;
    const float FyF = moving ? FnF * p.tf_D * sinf(p.tf_C * atanf(p.tf_B * (-alpha_f))) : 0.0f;
    const float FyR = moving ? FnR * p.tr_D * sinf(p.tr_C * atanf(p.tr_B * (-alpha_r))) : 0.0f;
    const float Fx = p.cm * throttle_break - p.cr0 - p.cr2 * s.vx * s.vx;
    float sm, cm_, sd, cd;
    sincosf(s.mu, &sm, &cm_);
    sincosf(delta, &sd, &cd);
    Car6 n;
    n.x = s.x + p.dt * (cm_ * s.vx - sm * s.vy);
    n.y = s.y + p.dt * (sm * s.vx + cm_ * s.vy);
    n.mu = s.mu + p.dt * s.omega;
    n.vx = s.vx + p.dt * (1.0f / p.m * (Fx - FyF * sd) + s.omega * s.vy);
    n.vy = s.vy + p.dt * (1.0f / p.m * (FyF * cd + FyR) - s.omega * s.vx);
    n.omega = s.omega + p.dt * (1.0f / p.I * (FyF * p.lf * cd - FyR * p.lr));
    return n;
}
__device__ __forceinline__ Car6 car_load(const float* __restrict__ states, int e) {
    const float2* sp = reinterpret_cast<const float2*>(states) + 3 * (size_t)e;
    const float2 s0 = sp[0], s1 = sp[1], s2 = sp[2];
    return {s0.x, s0.y, s1.x, s1.y, s2.x, s2.y};
}
__device__ __forceinline__ void car_store(float* __restrict__ rows, size_t row_floats, int e, const Car6& s) {       // the state as the first six values of row e (rows start 8-byte aligned)
    float2* o = reinterpret_cast<float2*>(rows + row_floats * (size_t)e);
    o[0] = make_float2(s.x, s.y); o[1] = make_float2(s.mu, s.vx); o[2] = make_float2(s.vy, s.omega);
}

// without a track: the reward comes from the pre-step state (:128-135), terminated from the next one (:80-84), the observation is the state (:143-155)
__device__ __forceinline__ void car_step_one(const rlt_car_parameters& p, float* __restrict__ states, const float* __restrict__ actions, float* __restrict__ observations,
                                             float* __restrict__ next_observations, float* __restrict__ rewards, uint8_t* __restrict__ terminated, int e) {
    const Car6 s = car_load(states, e);
    if (observations) car_store(observations, 6, e, s);
    const Car6 nx = car_dynamics(p, s, reinterpret_cast<const float2*>(actions)[e]);
    if (rewards) { const float an = angle_normalize(s.mu); rewards[e] = expf(-5.0f * (0.1f * an * an + s.x * s.x + s.y * s.y)); }
    if (terminated) terminated[e] = nx.x > 1.0f || nx.x < -1.0f || nx.y > 1.0f || nx.y < -1.0f;
    if (next_observations) car_store(next_observations, 6, e, nx);
    car_store(states, 6, e, nx);
}
__global__ __launch_bounds__(256) void car_step_kernel(rlt_car_parameters p, float* __restrict__ states, const float* __restrict__ actions, float* __restrict__ observations,
                                                       float* __restrict__ next_observations, float* __restrict__ rewards, uint8_t* __restrict__ terminated, int n) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) car_step_one(p, states, actions, observations, next_observations, rewards, terminated, e);
}

// on a track (:85-98 terminated, :136-141 reward, :156-190 observe): cell coordinates in double, as the reference's double literal makes them
struct TrackMap { const uint8_t* track; int height, width; float scale; };
__device__ __forceinline__ bool track_cell(const TrackMap& M, float x_coord, float y_coord) {
    if (!(x_coord > 0.0f && x_coord < (float)M.width && y_coord > 0.0f && y_coord < (float)M.height)) return false;       // beyond the bitmap: not drivable
    return M.track[(size_t)y_coord * M.width + (size_t)x_coord] != 0;
}
__device__ __forceinline__ void track_observe(const TrackMap& M, const Car6& s, float* __restrict__ o) {
    const float step_size = M.scale / 2.0f;
    const float directions[3] = {(float)(-20 / 180.0 * 3.14159274101257324), 0.0f, (float)(20 / 180.0 * 3.14159274101257324)};      // 20 degrees of the float pi
    const int NUM_STEPS = 50;
#pragma unroll
    for (int d = 0; d < 3; d++) {
        float sn, cs;
        sincosf(s.mu + directions[d], &sn, &cs);
        const float direction_x = cs * step_size, direction_y = sn * step_size;
        float distance = NUM_STEPS * step_size;
        for (int step_i = 0; step_i < NUM_STEPS; step_i++) {
            const float x_coord = (float)(((double)(s.x + direction_x * (float)step_i) + (double)(M.scale * (float)M.width) / 2.0) / (double)M.scale);
            const float y_coord = (float)(((double)(-s.y - direction_y * (float)step_i) + (double)(M.scale * (float)M.height) / 2.0) / (double)M.scale);
            if (!track_cell(M, x_coord, y_coord)) { distance = (float)step_i * step_size; break; }
        }
        o[6 + d] = distance / (NUM_STEPS * step_size);
    }
}
__global__ __launch_bounds__(256) void car_track_step_kernel(rlt_car_parameters p, TrackMap M, float* __restrict__ states, const float* __restrict__ actions,
                                                             float* __restrict__ observations, float* __restrict__ next_observations, float* __restrict__ rewards,
                                                             uint8_t* __restrict__ terminated, int n) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        const Car6 s = car_load(states, e);
        if (observations) { float* o = observations + 9 * (size_t)e; o[0] = s.x; o[1] = s.y; o[2] = s.mu; o[3] = s.vx; o[4] = s.vy; o[5] = s.omega; track_observe(M, s, o); }
        const Car6 nx = car_dynamics(p, s, reinterpret_cast<const float2*>(actions)[e]);
        if (rewards) rewards[e] = s.vx;
        if (terminated) {
            const float x_coord = (float)(((double)nx.x + (double)(M.scale * (float)M.width) / 2.0) / (double)M.scale);
            const float y_coord = (float)(((double)(-nx.y) + (double)(M.scale * (float)M.height) / 2.0) / (double)M.scale);
            terminated[e] = !track_cell(M, x_coord, y_coord);
        }
        if (next_observations) { float* o = next_observations + 9 * (size_t)e; o[0] = nx.x; o[1] = nx.y; o[2] = nx.mu; o[3] = nx.vx; o[4] = nx.vy; o[5] = nx.omega; track_observe(M, nx, o); }
        car_store(states, 6, e, nx);
    }
}
}  // namespace

extern "C" int rlt_rocm_car_step(rlt_rocm_device* device, const rlt_car_parameters* p, float* states, const float* actions, float* observations, float* next_observations,
                                 float* rewards, uint8_t* terminated, int n_envs) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(p && states && actions && n_envs > 0);
    RLT_REQUIRE((((uintptr_t)states | (uintptr_t)actions | (uintptr_t)observations | (uintptr_t)next_observations) & 7) == 0);      // rows move as 8-byte pairs
    int blocks = (n_envs + 255) / 256; if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(car_step_kernel, dim3(blocks), dim3(256), 0, device->stream, *p, states, actions, observations, next_observations, rewards, terminated, n_envs);
    return rlt_launch_status(device);
}

extern "C" int rlt_rocm_car_track_step(rlt_rocm_device* device, const rlt_car_parameters* p, const uint8_t* track, int height, int width, float track_scale, float* states,
                                       const float* actions, float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n_envs) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(p && track && height >= 1 && width >= 1 && track_scale > 0.0f && states && actions && n_envs > 0);
    RLT_REQUIRE((((uintptr_t)states | (uintptr_t)actions) & 7) == 0);      // states and actions move as 8-byte pairs
    int blocks = (n_envs + 255) / 256; if (blocks > 4096) blocks = 4096;
    const TrackMap M = {track, height, width, track_scale};
    hipLaunchKernelGGL(car_track_step_kernel, dim3(blocks), dim3(256), 0, device->stream, *p, M, states, actions, observations, next_observations, rewards, terminated, n_envs);
    return rlt_launch_status(device);
}

extern "C" int rlt_rocm_acrobot_step(rlt_rocm_device* device, const rlt_acrobot_parameters* p, int swingup, float* states, const float* actions, float* observations,
                                     float* next_observations, float* rewards, uint8_t* terminated, int n_envs) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(p && states && actions && n_envs > 0 && ((uintptr_t)states & 15) == 0);
    int blocks = (n_envs + 255) / 256; if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(acrobot_step_kernel, dim3(blocks), dim3(256), 0, device->stream, *p, swingup, states, actions, observations, next_observations, rewards, terminated, n_envs);
    return rlt_launch_status(device);
}

// ---- the off-policy runner over any of these environments (rl/components/off_policy_runner/operations_generic_per_env.h:8-108)
namespace {
struct EnvDims { int state, obs, act; };
__host__ __device__ inline EnvDims env_dims(int kind) {
    switch (kind) {
        case RLT_ENV_PENDULUM: return {2, 3, 1};
        case RLT_ENV_ACROBOT: case RLT_ENV_ACROBOT_SWINGUP: return {4, 6, 1};
        case RLT_ENV_CAR: return {6, 6, 2};
        case RLT_ENV_PENDULUM_POSITION: return {3, 2, 1};
        default: return {0, 0, 0};
    }
}
// The Pendulum whose observation is the position only and whose state also remembers the last action (rl/environments/pendulum/pendulum.h:117-124,
// step operations_generic.h:102-108, observe :168-181): states [n x 3] = (theta, theta_dot, last_action), observations [n x 2] = (cos, sin)
__device__ __forceinline__ void pendulum_position_step_one(const rlt_pendulum_parameters& p, float* __restrict__ states, const float* __restrict__ actions,
                                                           float* __restrict__ next_observations, float* __restrict__ rewards, uint8_t* __restrict__ terminated, int e) {
    Transition t;
    pendulum_transition(p, states[3 * (size_t)e], states[3 * (size_t)e + 1], actions[e], t);
    if (next_observations) { next_observations[2 * (size_t)e] = t.next_obs[0]; next_observations[2 * (size_t)e + 1] = t.next_obs[1]; }
    if (rewards) rewards[e] = t.reward;
    if (terminated) terminated[e] = 0;      // the Pendulum has no terminal states
    states[3 * (size_t)e] = t.theta; states[3 * (size_t)e + 1] = t.theta_dot; states[3 * (size_t)e + 2] = actions[e];
}
__global__ __launch_bounds__(256) void pendulum_position_step_kernel(rlt_pendulum_parameters p, float* __restrict__ states, const float* __restrict__ actions,
                                                                     float* __restrict__ next_observations, float* __restrict__ rewards, uint8_t* __restrict__ terminated, int n) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) pendulum_position_step_one(p, states, actions, next_observations, rewards, terminated, e);
}
int pendulum_position_step(rlt_rocm_device* device, const rlt_env_runner* rn, float* next_observations) {
    int blocks = (rn->n_envs + 255) / 256; if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(pendulum_position_step_kernel, dim3(blocks), dim3(256), 0, device->stream, rn->pendulum, rn->states, (const float*)rn->actions, next_observations, rn->rewards,
                       rn->terminated, rn->n_envs);
    return rlt_launch_status(device);
}
// prologue_per_env (:8-62): reset where the last step truncated (state from the caller's draw, counters, the ring's last row marked truncated,
// a new episode start), then observe
__device__ __forceinline__ void env_observe_one(int kind, const float* __restrict__ state, float* __restrict__ o) {
    if (kind == RLT_ENV_PENDULUM) { float sn, cs; sincosf(state[0], &sn, &cs); o[0] = cs; o[1] = sn; o[2] = state[1]; }
    else if (kind == RLT_ENV_PENDULUM_POSITION) { float sn, cs; sincosf(state[0], &sn, &cs); o[0] = cs; o[1] = sn; }
    else if (kind == RLT_ENV_CAR) { for (int i = 0; i < 6; i++) o[i] = state[i]; }
    else { const Acrobot4 s4 = {{state[0], state[1], state[2], state[3]}}; acrobot_observe(s4, o); }
}
// `initial`: the state this environment starts its next episode from
__device__ __forceinline__ void env_prologue_one(const rlt_env_runner& rn, const rlt_replay_buffer& rb, const float* initial, int e) {
    const EnvDims d = env_dims(rn.env_kind);
    const int R = 2 * rb.observation_dim + rb.action_dim + 3;
    float* state = rn.states + (size_t)e * d.state;
    if (rn.truncated[e]) {
        for (int i = 0; i < d.state; i++) state[i] = initial[i];
        rn.episode_step[e] = 0; rn.episode_return[e] = 0.0f;
        if (rb.full[e] || rb.position[e] > 0) {
            const uint32_t prev = rb.position[e] == 0 ? (uint32_t)rb.capacity - 1 : rb.position[e] - 1;
            rb.data[((size_t)e * rb.capacity + prev) * R + (R - 1)] = 1.0f;
            rb.current_episode_start[e] = rb.position[e];
        }
    }
    env_observe_one(rn.env_kind, state, rn.observations + (size_t)e * d.obs);
}
__global__ __launch_bounds__(256) void env_prologue_kernel(rlt_env_runner rn, rlt_replay_buffer rb, const float* __restrict__ initial_states) {
    const int state_dim = env_dims(rn.env_kind).state;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) env_prologue_one(rn, rb, initial_states + (size_t)e * state_dim, e);
}
// the rest of epilogue_per_env after the environment's own step (:88-104): counters, truncation, replay add (replay_buffer/operations_generic.h:54-78)
__device__ __forceinline__ void env_epilogue_one(const rlt_env_runner& rn, const rlt_replay_buffer& rb, int e) {
    const EnvDims d = env_dims(rn.env_kind);
    const int OBS = d.obs, ACT = d.act, R = 2 * OBS + ACT + 3;
    const float reward = rn.rewards[e];
    const bool terminated = rn.terminated[e] != 0;
    const uint32_t step = rn.episode_step[e] + 1;
    rn.episode_step[e] = step;
    rn.episode_return[e] += reward;
    const bool truncated = terminated || step == (uint32_t)rn.episode_step_limit;
    rn.truncated[e] = truncated;
    uint32_t pos = rb.position[e];
    float* row = rb.data + ((size_t)e * rb.capacity + pos) * R;
    for (int i = 0; i < OBS; i++) row[i] = rn.observations[(size_t)e * OBS + i];
    for (int i = 0; i < ACT; i++) row[OBS + i] = rn.actions[(size_t)e * ACT + i];
    row[OBS + ACT] = reward;
    for (int i = 0; i < OBS; i++) row[OBS + ACT + 1 + i] = rn.next_observations[(size_t)e * OBS + i];
    row[R - 2] = terminated ? 1.0f : 0.0f; row[R - 1] = truncated ? 1.0f : 0.0f;
    rb.episode_start[(size_t)e * rb.capacity + pos] = rb.current_episode_start[e];
    pos = (pos + 1) % (uint32_t)rb.capacity;
    rb.position[e] = pos;
    if (truncated) rb.current_episode_start[e] = pos;
    if (pos == 0 && !rb.full[e]) rb.full[e] = 1;
}
__global__ __launch_bounds__(256) void env_epilogue_kernel(rlt_env_runner rn, rlt_replay_buffer rb) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) env_epilogue_one(rn, rb, e);
}
// one environment's own step, whatever its kind
__device__ __forceinline__ void env_step_one(const rlt_env_runner& rn, float* __restrict__ next_observations, int e) {
    switch (rn.env_kind) {
        case RLT_ENV_PENDULUM: {
            Transition t;
            pendulum_transition(rn.pendulum, rn.states[2 * (size_t)e], rn.states[2 * (size_t)e + 1], rn.actions[e], t);
            if (next_observations) for (int i = 0; i < 3; i++) next_observations[3 * (size_t)e + i] = t.next_obs[i];
            rn.rewards[e] = t.reward; rn.terminated[e] = 0;
            rn.states[2 * (size_t)e] = t.theta; rn.states[2 * (size_t)e + 1] = t.theta_dot;
            break;
        }
        case RLT_ENV_PENDULUM_POSITION: pendulum_position_step_one(rn.pendulum, rn.states, rn.actions, next_observations, rn.rewards, rn.terminated, e); break;
        case RLT_ENV_CAR: car_step_one(rn.car, rn.states, rn.actions, nullptr, next_observations, rn.rewards, rn.terminated, e); break;
        default: acrobot_step_one(rn.acrobot, rn.env_kind == RLT_ENV_ACROBOT_SWINGUP, rn.states, rn.actions, nullptr, next_observations, rn.rewards, rn.terminated, e);
    }
}

// ---- The runner's whole step in ONE launch for a handful of environments and a policy of dense layers (rl/components/off_policy_runner/operations_generic.h:183-238 over
// operations_generic_per_env.h:8-108): reset and observe, the policy's layers, its head, the environment's step, counters and the replay add. One workgroup of sixteen
// wavefronts: a wavefront forms the dot products of its sixteen output units (lanes across the input width, the weights' rows read coalesced and all at once, the
// sums folded across the lanes), the activations of a layer wait in LDS for the next. For the loops that step one or a few environments per training step, where the
// launches of the separate kernels (nine of them) are the whole cost.
__device__ __forceinline__ float mul_add_twice_rounded(float a, float b, float c) {
#pragma clang fp contract(off)
    const float product = a * b;
    return product + c;
}
constexpr int FUSED_MAX_ENVS = 16, FUSED_MAX_WIDTH = 256, FUSED_MAX_LAYERS = 8, FUSED_THREADS = 1024;
struct FusedLayer { const float* weights; const float* biases; int in_dim, out_dim, activation; };
struct EnvFusedArgs {
    rlt_env_runner rn; rlt_replay_buffer rb;
    FusedLayer L[FUSED_MAX_LAYERS]; int n_layers;
    int head_kind;              // 0: the actions are given (no policy); 1: the policy's output is the action; 2: sample_and_squash; 3: clamp(output + std * noise, -1, 1)
    rlt_sas_parameters sas; float noise_std;
    const float* noise;         // [n_envs x action_dim] standard normal draws (head kinds 2 and 3) or the caller's actions (head kind 0)
    const float* initial_states;
    // the kernel's own draws where both arrays are NULL: element e * action_dim + c of the noise stream (standard normal for head kinds 2 and 3; for head kind 0 the
    // action itself, uniform in (-1, 1)), and for an environment that starts an episode state component i = low[i] + (high[i] - low[i]) * element e * state_dim + i
    // of the initial-state stream (rng.h: the elements rlt_rocm_randn_f32 / rlt_rocm_rand_f32 would write)
    int draw; uint64_t seed, noise_stream, initial_stream; const uint64_t* stream_offset;
    float initial_low[8], initial_high[8];
    float* drawn_noise;         // optional: the noise (or uniform actions) drawn
};
__global__ __launch_bounds__(FUSED_THREADS) void env_runner_fused_kernel(EnvFusedArgs A) {
    __shared__ float act[2][FUSED_MAX_ENVS][FUSED_MAX_WIDTH + 1];
    const int N = A.rn.n_envs, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const EnvDims d = env_dims(A.rn.env_kind);
    __shared__ float drawn[FUSED_MAX_ENVS][8];      // this step's initial states, then its noise, where the kernel draws them
    if (tid < N) {
        const float* initial = A.initial_states ? A.initial_states + (size_t)tid * d.state : nullptr;
        if (A.draw) {
            const uint64_t stream = A.initial_stream + *A.stream_offset;
            if (A.rn.truncated[tid])
                for (int i = 0; i < d.state; i++) drawn[tid][i] = A.initial_low[i] + (A.initial_high[i] - A.initial_low[i]) * rlt_rand_element(A.seed, stream, (uint64_t)tid * d.state + i);
            initial = &drawn[tid][0];
        }
        env_prologue_one(A.rn, A.rb, initial, tid);
        for (int i = 0; i < d.obs; i++) act[0][tid][i] = A.rn.observations[(size_t)tid * d.obs + i];
        if (A.draw) {
            const uint64_t stream = A.noise_stream + *A.stream_offset;
            for (int c = 0; c < d.act; c++) {
                const uint64_t i = (uint64_t)tid * d.act + c;
                const float v = A.head_kind == 0 ? -1.0f + 2.0f * rlt_rand_element(A.seed, stream, i) : rlt_randn_element(A.seed, stream, i);
                drawn[tid][c] = v;
                if (A.drawn_noise) A.drawn_noise[i] = v;
            }
        }
    }
    __syncthreads();
    int cur = 0;
    // A layer: wavefront w owns output units 16 w .. 16 w + 15. All of their rows of W are requested at once, with addresses clamped into the matrix instead of
    // branches (a launch of one workgroup finds nothing of the weights in its caches: one trip to memory per layer, not one per unit; and straight-line code,
    // because the instructions come from memory as well). Lanes hold the input positions lane + 64 j; positions beyond the layer's width meet zero activations,
    // units beyond it are not stored. After the sums over the lanes, lane q of the first sixteen keeps unit q, adds the bias and applies the activation.
    constexpr int UNITS = 16, CHUNKS = FUSED_MAX_WIDTH / 64;
    static_assert(UNITS * (FUSED_THREADS / 64) == FUSED_MAX_WIDTH, "a wavefront's units times the wavefronts cover the widest layer");
    for (int l = 0; l < A.n_layers; l++) {
        const FusedLayer& L = A.L[l];
        const int in = L.in_dim, out = L.out_dim;
        if (UNITS * wave < out) {
            float w[UNITS][CHUNKS];
#pragma unroll
            for (int q = 0; q < UNITS; q++) {
                const float* row = L.weights + (size_t)min(UNITS * wave + q, out - 1) * in;
#pragma unroll
                for (int j = 0; j < CHUNKS; j++) w[q][j] = row[min(lane + 64 * j, in - 1)];
            }
            const int mine = UNITS * wave + (lane & 15);
            const float bias = L.biases[min(mine, out - 1)];
            for (int r = 0; r < N; r++) {
                float a[CHUNKS];
#pragma unroll
                for (int j = 0; j < CHUNKS; j++) a[j] = lane + 64 * j < in ? act[cur][r][lane + 64 * j] : 0.f;
                float kept = 0.f;
#pragma unroll
                for (int q = 0; q < UNITS; q++) {
                    float sum = w[q][0] * a[0];
#pragma unroll
                    for (int j = 1; j < CHUNKS; j++) sum += w[q][j] * a[j];
                    sum = rlt_sac::groups_sum(rlt_sac::row16_sum(sum));
                    kept = (lane & 15) == q ? sum : kept;
                }
                if (lane < 16 && mine < out) act[cur ^ 1][r][mine] = rlt_act(kept + bias, L.activation);
            }
        }
        __syncthreads();
        cur ^= 1;
    }
    if (tid < N) {
        const int e = tid;
        const float* noise_row = A.draw ? &drawn[e][0] : (A.noise ? A.noise + (size_t)e * d.act : nullptr);
        if (A.head_kind == 0) { for (int c = 0; c < d.act; c++) A.rn.actions[(size_t)e * d.act + c] = noise_row[c]; }      // the caller's actions, or uniform draws
        else if (A.head_kind == 1) { for (int c = 0; c < d.act; c++) A.rn.actions[(size_t)e * d.act + c] = act[cur][e][c]; }
        else if (A.head_kind == 2) {       // nn/layers/sample_and_squash/operations_generic.h:149-195 in rollout mode
            for (int c = 0; c < d.act; c++) {
                const float mean = act[cur][e][c];
                const float log_std = fminf(fmaxf(act[cur][e][d.act + c], A.sas.log_std_lower_bound), A.sas.log_std_upper_bound);
                A.rn.actions[(size_t)e * d.act + c] = tanhf(mean + noise_row[c] * expf(log_std));
            }
        } else if (A.head_kind == 3) {     // nn/layers/td3_sampling/operations_generic.h:75-128
            for (int c = 0; c < d.act; c++) {
                const float sample = mul_add_twice_rounded(noise_row[c], A.noise_std, act[cur][e][c]);
                A.rn.actions[(size_t)e * d.act + c] = sample < -1.0f ? -1.0f : (sample > 1.0f ? 1.0f : sample);
            }
        }
        env_step_one(A.rn, A.rn.next_observations, e);
        env_epilogue_one(A.rn, A.rb, e);
    }
}
__global__ __launch_bounds__(256) void env_copy_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}
inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
}  // namespace

namespace {
// the one-launch step where it applies: a few environments, dense layers of moderate width (or no policy at all); false: the caller takes the separate kernels
struct EnvDraws { uint64_t seed, noise_stream, initial_stream; const float* low; const float* high; float* drawn_noise; };
bool env_runner_fused(rlt_rocm_device* device, const rlt_env_runner* rn, const rlt_replay_buffer* rb, const rlt_dense_layer* const* layers, int n_layers, int head_kind,
                      const rlt_sas_parameters* sas, float noise_std, const float* noise, const float* initial_states, int* rc, const EnvDraws* draws = nullptr) {
    if (rn->n_envs > FUSED_MAX_ENVS || n_layers > FUSED_MAX_LAYERS) return false;
    const EnvDims d = env_dims(rn->env_kind);
    if (n_layers > 0 && (layers[0]->in_dim != d.obs || layers[n_layers - 1]->out_dim != (head_kind == 2 ? 2 : 1) * d.act)) return false;      // the separate kernels report it
    EnvFusedArgs A = {};
    for (int l = 0; l < n_layers; l++) {
        const rlt_dense_layer& L = *layers[l];
        if (L.in_dim < 1 || L.out_dim < 1 || L.in_dim > FUSED_MAX_WIDTH || L.out_dim > FUSED_MAX_WIDTH || !L.weights || !L.biases || (l > 0 && L.in_dim != layers[l - 1]->out_dim)) return false;
        A.L[l] = FusedLayer{L.weights, L.biases, L.in_dim, L.out_dim, L.activation};
    }
    A.rn = *rn; A.rb = *rb; A.n_layers = n_layers; A.head_kind = head_kind; A.noise_std = noise_std; A.noise = noise; A.initial_states = initial_states;
    if (sas) A.sas = *sas;
    if (draws) {
        A.draw = 1; A.seed = draws->seed; A.noise_stream = draws->noise_stream; A.initial_stream = draws->initial_stream; A.stream_offset = (const uint64_t*)device->stream_offset;
        for (int i = 0; i < d.state && i < 8; i++) { A.initial_low[i] = draws->low[i]; A.initial_high[i] = draws->high[i]; }
        A.drawn_noise = draws->drawn_noise;
    }
    hipLaunchKernelGGL(env_runner_fused_kernel, dim3(1), dim3(FUSED_THREADS), 0, device->stream, A);
    *rc = rlt_launch_status(device);
    return true;
}
}  // namespace

extern "C" int rlt_rocm_env_dims(int env_kind, int* state_dim, int* observation_dim, int* action_dim) {
    const EnvDims d = env_dims(env_kind);
    if (!d.state) return RLT_E_INVALID_ARGUMENT;
    if (state_dim) *state_dim = d.state;
    if (observation_dim) *observation_dim = d.obs;
    if (action_dim) *action_dim = d.act;
    return 0;
}

extern "C" size_t rlt_rocm_env_runner_step_workspace_bytes(const rlt_env_runner* rn, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers) {
    if (!rn || rn->n_envs < 1) return 0;
    const EnvDims d = env_dims(rn->env_kind);
    const size_t head = align256((size_t)rn->n_envs * (2 * d.act + 1) * sizeof(float));      // actor output [n x 2 act], log-probabilities [n]
    return head + (policy_kind ? rlt_rocm_mlp_workspace_bytes(actor, n_actor_layers, rn->n_envs) : 0) + 256;
}

extern "C" int rlt_rocm_env_runner_step(rlt_rocm_device* device, const rlt_env_runner* rn, const rlt_replay_buffer* rb, int policy_kind, const rlt_dense_layer* actor,
                                        int n_actor_layers, const rlt_sas_parameters* sas, const float* actions_in, const float* action_noise, const float* initial_states,
                                        void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rb && rn->n_envs > 0 && rn->states && rn->episode_step && rn->episode_return && rn->truncated && initial_states);
    RLT_REQUIRE(rn->observations && rn->actions && rn->next_observations && rn->rewards && rn->terminated);
    RLT_REQUIRE(rb->data && rb->episode_start && rb->position && rb->current_episode_start && rb->full && rb->capacity > 0);
    const EnvDims d = env_dims(rn->env_kind);
    RLT_REQUIRE(d.state && rn->n_envs == rb->n_envs && rb->observation_dim == d.obs && rb->action_dim == d.act && policy_kind >= 0 && policy_kind <= 2);
    RLT_REQUIRE(policy_kind != 0 || actions_in);
    RLT_REQUIRE(policy_kind == 0 || (actor && n_actor_layers >= 1 && actor[0].in_dim == d.obs && actor[n_actor_layers - 1].out_dim == (policy_kind == 2 ? 2 : 1) * d.act));
    RLT_REQUIRE(policy_kind != 2 || (sas && action_noise));
    RLT_REQUIRE(policy_kind == 0 || (workspace && workspace_bytes >= rlt_rocm_env_runner_step_workspace_bytes(rn, policy_kind, actor, n_actor_layers)));
    {
        const rlt_dense_layer* list[FUSED_MAX_LAYERS];
        const int n_list = policy_kind == 0 ? 0 : n_actor_layers;
        for (int l = 0; l < n_list && l < FUSED_MAX_LAYERS; l++) list[l] = actor + l;
        int frc = 0;
        if (env_runner_fused(device, rn, rb, list, n_list, policy_kind, sas, 0.0f, policy_kind == 0 ? actions_in : action_noise, initial_states, &frc)) return frc;
    }
    const int N = rn->n_envs;
    const int blocks = rlt_div_up(N, 256) > 1024 ? 1024 : rlt_div_up(N, 256);
    int rc;
    hipLaunchKernelGGL(env_prologue_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *rb, initial_states);
    if ((rc = rlt_launch_status(device))) return rc;
    if (policy_kind == 0) {
        hipLaunchKernelGGL(env_copy_kernel, dim3(blocks), dim3(256), 0, device->stream, actions_in, rn->actions, (size_t)N * d.act);
        if ((rc = rlt_launch_status(device))) return rc;
    } else {
        char* w = reinterpret_cast<char*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
        float* actor_out = (float*)w; float* log_probabilities = actor_out + (size_t)N * 2 * d.act;
        const size_t head = align256((size_t)N * (2 * d.act + 1) * sizeof(float));
        void* mlp_ws = w + head; const size_t mlp_ws_bytes = rlt_rocm_mlp_workspace_bytes(actor, n_actor_layers, N);
        if (policy_kind == 1) { if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, rn->observations, d.obs, rn->actions, d.act, N, mlp_ws, mlp_ws_bytes))) return rc; }
        else {
            if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, rn->observations, d.obs, actor_out, 2 * d.act, N, mlp_ws, mlp_ws_bytes))) return rc;
            if ((rc = rlt_rocm_sas_forward(device, sas, actor_out, 2 * d.act, action_noise, d.act, rn->actions, d.act, nullptr, 0, log_probabilities, N, d.act))) return rc;
        }
    }
    switch (rn->env_kind) {
        case RLT_ENV_PENDULUM:
            if ((rc = rlt_rocm_pendulum_step(device, &rn->pendulum, rn->states, rn->actions, nullptr, rn->next_observations, rn->rewards, N))) return rc;
            if ((rc = rlt_rocm_fill_u8(device, rn->terminated, (size_t)N, 0))) return rc;      // the Pendulum has no terminal states
            break;
        case RLT_ENV_PENDULUM_POSITION: if ((rc = pendulum_position_step(device, rn, rn->next_observations))) return rc; break;
        case RLT_ENV_CAR: if ((rc = rlt_rocm_car_step(device, &rn->car, rn->states, rn->actions, nullptr, rn->next_observations, rn->rewards, rn->terminated, N))) return rc; break;
        default:
            if ((rc = rlt_rocm_acrobot_step(device, &rn->acrobot, rn->env_kind == RLT_ENV_ACROBOT_SWINGUP, rn->states, rn->actions, nullptr, rn->next_observations, rn->rewards,
                                            rn->terminated, N))) return rc;
    }
    hipLaunchKernelGGL(env_epilogue_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *rb);
    return rlt_launch_status(device);
}

extern "C" int rlt_rocm_env_runner_step_drawn(rlt_rocm_device* device, const rlt_env_runner* rn, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n_policy_layers,
                                              int head_kind, const rlt_sas_parameters* sas, float exploration_noise_std, const float* initial_low, const float* initial_high,
                                              float* drawn_noise, uint64_t seed, uint64_t noise_stream, uint64_t initial_state_stream) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rb && rn->n_envs > 0 && rn->states && rn->episode_step && rn->episode_return && rn->truncated && initial_low && initial_high);
    RLT_REQUIRE(rn->observations && rn->actions && rn->next_observations && rn->rewards && rn->terminated);
    RLT_REQUIRE(rb->data && rb->episode_start && rb->position && rb->current_episode_start && rb->full && rb->capacity > 0);
    const EnvDims d = env_dims(rn->env_kind);
    RLT_REQUIRE(d.state && d.state <= 8 && rn->n_envs == rb->n_envs && rb->observation_dim == d.obs && rb->action_dim == d.act && head_kind >= 0 && head_kind <= 3);
    RLT_REQUIRE((head_kind == 0) == (n_policy_layers == 0) && n_policy_layers >= 0 && n_policy_layers <= RLT_SEQ_MAX_LAYERS && (n_policy_layers == 0 || policy) && (head_kind != 2 || sas));
    const rlt_dense_layer* list[RLT_SEQ_MAX_LAYERS];
    for (int l = 0; l < n_policy_layers; l++) {
        if (policy[l].kind != 0) return RLT_E_UNSUPPORTED;
        list[l] = &policy[l].dense;
    }
    if (n_policy_layers > 0) RLT_REQUIRE(list[0]->in_dim == d.obs && list[n_policy_layers - 1]->out_dim == (head_kind == 2 ? 2 : 1) * d.act);
    const EnvDraws draws = {seed, noise_stream, initial_state_stream, initial_low, initial_high, drawn_noise};
    int rc = 0;
    if (!env_runner_fused(device, rn, rb, list, n_policy_layers, head_kind, sas, exploration_noise_std, nullptr, nullptr, &rc, &draws)) return RLT_E_UNSUPPORTED;
    return rc;
}

// ---- on-policy collection over any of these environments (rl/components/on_policy_runner/operations_generic_per_env.h:8-74)
namespace {
__device__ __forceinline__ void observe_any(int kind, const float* __restrict__ state, float* __restrict__ o) {
    if (kind == RLT_ENV_PENDULUM) { float sn, cs; sincosf(state[0], &sn, &cs); o[0] = cs; o[1] = sn; o[2] = state[1]; }
    else if (kind == RLT_ENV_PENDULUM_POSITION) { float sn, cs; sincosf(state[0], &sn, &cs); o[0] = cs; o[1] = sn; }
    else if (kind == RLT_ENV_CAR) { for (int i = 0; i < 6; i++) o[i] = state[i]; }
    else { const Acrobot4 s4 = {{state[0], state[1], state[2], state[3]}}; acrobot_observe(s4, o); }
}
// prologue of step `step` (:8-35): reset where truncated (the flag is cleared), observe into the dataset row of this step; final: only the observation
__global__ __launch_bounds__(256) void env_collect_prologue_kernel(rlt_env_runner rn, rlt_on_policy_dataset D, const float* __restrict__ initial_states, int step, int final) {
    const EnvDims d = env_dims(rn.env_kind);
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        const size_t row = (size_t)step * rn.n_envs + e;
        float* state = rn.states + (size_t)e * d.state;
        if (!final) {
            const bool truncated = rn.truncated[e] != 0;
            if (step == 0) D.all_reset[(size_t)e * D.ld] = truncated ? 1.0f : 0.0f;      // reset aliases the first rows of all_reset
            if (truncated) {
                rn.truncated[e] = 0; rn.episode_step[e] = 0; rn.episode_return[e] = 0.0f;
                for (int i = 0; i < d.state; i++) state[i] = initial_states[row * d.state + i];
            }
        }
        observe_any(rn.env_kind, state, D.observations + row * D.ld);
    }
}
// first half of the epilogue (:37-58): the action around the mean, its log-probability (random/operations_generic.h:73-97); the action also packed for the step kernel
__global__ __launch_bounds__(256) void env_collect_sample_kernel(rlt_env_runner rn, rlt_on_policy_dataset D, const float* __restrict__ log_std, const float* __restrict__ action_noise, int step) {
    const int ACT = env_dims(rn.env_kind).act;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        const size_t row = (size_t)step * rn.n_envs + e;
        float log_prob = 0.0f;
        for (int a = 0; a < ACT; a++) {
            const float ls = log_std[a], sd = expf(ls);
            const float mean = D.actions_mean[row * D.ld + a];
            const float action = mul_add_twice_rounded(action_noise[row * ACT + a], sd, mean);      // z * std + mean, rounded twice as the reference's CPU build does
            const float pre = (action - mean) / sd;
            log_prob += (-0.9189385332046727f - ls) - 0.5f * pre * pre;
            D.actions[row * D.ld + a] = action;
            rn.actions[(size_t)e * ACT + a] = action;
        }
        D.action_log_probs[row * D.ld] = log_prob;
    }
}
// second half of the epilogue (:59-74) after the environment's own step: flags, reward, counters, the delayed reset flag
__global__ __launch_bounds__(256) void env_collect_epilogue_kernel(rlt_env_runner rn, rlt_on_policy_dataset D, int step) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        const size_t row = (size_t)step * rn.n_envs + e;
        const bool terminated = rn.terminated[e] != 0;
        const float reward = rn.rewards[e];
        D.terminated[row * D.ld] = terminated ? 1.0f : 0.0f;
        rn.episode_return[e] += reward;
        D.rewards[row * D.ld] = reward;
        const uint32_t n = rn.episode_step[e] + 1;
        rn.episode_step[e] = n;
        const bool truncated = terminated || (rn.episode_step_limit > 0 && n >= (uint32_t)rn.episode_step_limit);
        D.truncated[row * D.ld] = truncated ? 1.0f : 0.0f;
        D.all_reset[(row + rn.n_envs) * D.ld] = truncated ? 1.0f : 0.0f;
        rn.truncated[e] = truncated;
    }
}
int env_step_launch(rlt_rocm_device* device, const rlt_env_runner* rn, float* next_observations) {
    const int N = rn->n_envs;
    int rc;
    switch (rn->env_kind) {
        case RLT_ENV_PENDULUM:
            if ((rc = rlt_rocm_pendulum_step(device, &rn->pendulum, rn->states, rn->actions, nullptr, next_observations, rn->rewards, N))) return rc;
            return rlt_rocm_fill_u8(device, rn->terminated, (size_t)N, 0);      // the Pendulum has no terminal states
        case RLT_ENV_PENDULUM_POSITION: return pendulum_position_step(device, rn, next_observations);
        case RLT_ENV_CAR: return rlt_rocm_car_step(device, &rn->car, rn->states, rn->actions, nullptr, next_observations, rn->rewards, rn->terminated, N);
        default: return rlt_rocm_acrobot_step(device, &rn->acrobot, rn->env_kind == RLT_ENV_ACROBOT_SWINGUP, rn->states, rn->actions, nullptr, next_observations, rn->rewards, rn->terminated, N);
    }
}
}  // namespace

extern "C" size_t rlt_rocm_env_on_policy_collect_workspace_bytes(const rlt_env_runner* rn, const rlt_seq_layer* policy, int n_policy_layers) {
    if (!rn || rn->n_envs < 1 || !policy || n_policy_layers < 1) return 0;
    const EnvDims d = env_dims(rn->env_kind);
    return align256((size_t)rn->n_envs * d.obs * sizeof(float)) + rlt_rocm_seq_evaluate_step_workspace_bytes(policy, n_policy_layers, rn->n_envs) + 512;
}

extern "C" int rlt_rocm_env_on_policy_collect(rlt_rocm_device* device, const rlt_env_runner* rn, const rlt_on_policy_dataset* D, const rlt_seq_layer* policy, int n_policy_layers,
                                              const rlt_seq_state* policy_state, int auto_reset_period, const float* log_std, const float* standardize_mean,
                                              const float* standardize_precision, const float* action_noise, const float* initial_states, int truncate_on_each_iteration,
                                              void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rn->n_envs > 0 && rn->states && rn->episode_step && rn->episode_return && rn->truncated && rn->actions && rn->rewards && rn->terminated);
    const EnvDims d = env_dims(rn->env_kind);
    RLT_REQUIRE(d.state && D && D->steps_per_env > 0 && D->ld >= d.obs && D->ld >= d.act);
    RLT_REQUIRE(D->observations && D->actions_mean && D->actions && D->action_log_probs && D->rewards && D->terminated && D->truncated && D->all_reset);
    RLT_REQUIRE(policy && n_policy_layers >= 1 && n_policy_layers <= RLT_SEQ_MAX_LAYERS && log_std && action_noise && initial_states);
    RLT_REQUIRE((standardize_mean == nullptr) == (standardize_precision == nullptr));
    bool recurrent = false;
    for (int l = 0; l < n_policy_layers; l++) recurrent = recurrent || policy[l].kind != 0;
    RLT_REQUIRE(!recurrent || policy_state);
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_env_on_policy_collect_workspace_bytes(rn, policy, n_policy_layers));
    const int N = rn->n_envs, blocks = rlt_div_up(N, 256) > 1024 ? 1024 : rlt_div_up(N, 256);
    float* standardized = reinterpret_cast<float*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    char* step_ws = (char*)standardized + align256((size_t)N * d.obs * sizeof(float));
    const size_t step_ws_bytes = workspace_bytes - (size_t)(step_ws - (char*)workspace);
    int rc;
    const rlt_seq_state no_state = {};      // a policy of dense layers keeps no state
    const rlt_seq_state* step_state = policy_state ? policy_state : &no_state;
    if (truncate_on_each_iteration && (rc = rlt_rocm_fill_u8(device, rn->truncated, (size_t)N, 1))) return rc;      // :112-114
    for (int step = 0; step < D->steps_per_env; step++) {
        if (policy_state && (rc = rlt_rocm_seq_reset_state(device, policy, n_policy_layers, policy_state, rn->truncated, N))) return rc;
        hipLaunchKernelGGL(env_collect_prologue_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *D, initial_states, step, 0);
        if ((rc = rlt_launch_status(device))) return rc;
        const float* obs = D->observations + (size_t)step * N * D->ld; int ldo = D->ld;
        if (standardize_mean) {
            if ((rc = rlt_rocm_standardize_forward(device, standardize_mean, standardize_precision, obs, D->ld, standardized, d.obs, N, d.obs))) return rc;
            obs = standardized; ldo = d.obs;
        }
        if ((rc = rlt_rocm_seq_evaluate_step(device, policy, n_policy_layers, obs, ldo, step_state, auto_reset_period, D->actions_mean + (size_t)step * N * D->ld, D->ld, N,
                                             step_ws, step_ws_bytes))) return rc;
        hipLaunchKernelGGL(env_collect_sample_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *D, log_std, action_noise, step);
        if ((rc = rlt_launch_status(device))) return rc;
        if ((rc = env_step_launch(device, rn, nullptr))) return rc;
        hipLaunchKernelGGL(env_collect_epilogue_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *D, step);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    hipLaunchKernelGGL(env_collect_prologue_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *D, initial_states, D->steps_per_env, 1);
    return rlt_launch_status(device);
}

extern "C" size_t rlt_rocm_env_runner_step_sequential_workspace_bytes(const rlt_env_runner* rn, const rlt_seq_layer* policy, int n_policy_layers) {
    if (!rn || rn->n_envs < 1 || !policy || n_policy_layers < 1) return 0;
    const EnvDims d = env_dims(rn->env_kind);
    return align256((size_t)rn->n_envs * (2 * d.act + 1) * sizeof(float)) + rlt_rocm_seq_evaluate_step_workspace_bytes(policy, n_policy_layers, rn->n_envs) + 512;
}

extern "C" int rlt_rocm_env_runner_step_sequential(rlt_rocm_device* device, const rlt_env_runner* rn, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n_policy_layers,
                                                   const rlt_seq_state* policy_state, int auto_reset_period, int head_kind, const rlt_sas_parameters* sas, float exploration_noise_std,
                                                   const float* action_noise, const float* initial_states, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rb && rn->n_envs > 0 && rn->states && rn->episode_step && rn->episode_return && rn->truncated && initial_states);
    RLT_REQUIRE(rn->observations && rn->actions && rn->next_observations && rn->rewards && rn->terminated);
    RLT_REQUIRE(rb->data && rb->episode_start && rb->position && rb->current_episode_start && rb->full && rb->capacity > 0);
    const EnvDims d = env_dims(rn->env_kind);
    RLT_REQUIRE(d.state && rn->n_envs == rb->n_envs && rb->observation_dim == d.obs && rb->action_dim == d.act && head_kind >= 1 && head_kind <= 3);
    RLT_REQUIRE(policy && n_policy_layers >= 1 && n_policy_layers <= RLT_SEQ_MAX_LAYERS && (head_kind == 1 || action_noise) && (head_kind != 2 || sas));
    bool recurrent = false;
    for (int l = 0; l < n_policy_layers; l++) recurrent = recurrent || policy[l].kind != 0;
    RLT_REQUIRE(!recurrent || policy_state);
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_env_runner_step_sequential_workspace_bytes(rn, policy, n_policy_layers));
    if (!recurrent) {
        const rlt_dense_layer* list[RLT_SEQ_MAX_LAYERS];
        for (int l = 0; l < n_policy_layers; l++) list[l] = &policy[l].dense;
        int frc = 0;
        if (env_runner_fused(device, rn, rb, list, n_policy_layers, head_kind, sas, exploration_noise_std, action_noise, initial_states, &frc)) return frc;
    }
    const int N = rn->n_envs, blocks = rlt_div_up(N, 256) > 1024 ? 1024 : rlt_div_up(N, 256);
    float* policy_out = reinterpret_cast<float*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    float* log_probabilities = policy_out + (size_t)N * 2 * d.act;
    char* step_ws = (char*)policy_out + align256((size_t)N * (2 * d.act + 1) * sizeof(float));
    const size_t step_ws_bytes = workspace_bytes - (size_t)(step_ws - (char*)workspace);
    const rlt_seq_state no_state = {};
    int rc;
    hipLaunchKernelGGL(env_prologue_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *rb, initial_states);
    if ((rc = rlt_launch_status(device))) return rc;
    if (policy_state && (rc = rlt_rocm_seq_reset_state(device, policy, n_policy_layers, policy_state, rn->truncated, N))) return rc;
    const int out_dim = (head_kind == 2 ? 2 : 1) * d.act;
    float* out = head_kind == 1 ? rn->actions : policy_out;
    if ((rc = rlt_rocm_seq_evaluate_step(device, policy, n_policy_layers, rn->observations, d.obs, policy_state ? policy_state : &no_state, auto_reset_period, out, out_dim, N,
                                         step_ws, step_ws_bytes))) return rc;
    if (head_kind == 2) { if ((rc = rlt_rocm_sas_forward(device, sas, policy_out, 2 * d.act, action_noise, d.act, rn->actions, d.act, nullptr, 0, log_probabilities, N, d.act))) return rc; }
    else if (head_kind == 3) { if ((rc = rlt_rocm_td3_sampling_forward(device, policy_out, d.act, action_noise, d.act, exploration_noise_std, nullptr, 0, rn->actions, d.act, N, d.act))) return rc; }
    if ((rc = env_step_launch(device, rn, rn->next_observations))) return rc;
    hipLaunchKernelGGL(env_epilogue_kernel, dim3(blocks), dim3(256), 0, device->stream, *rn, *rb);
    return rlt_launch_status(device);
}

// ---- rl::utils::evaluation::evaluate over any of these environments (rl/utils/evaluation/operations_generic.h:113-233)
namespace {
__global__ __launch_bounds__(256) void env_evaluate_observe_kernel(int kind, const float* __restrict__ states, float* __restrict__ obs, int n) {
    const EnvDims d = env_dims(kind);
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) observe_any(kind, states + (size_t)e * d.state, obs + (size_t)e * d.obs);
}
// the standardize layer in front of a policy (nn/layers/standardize/operations_generic.h:69-135)
__global__ __launch_bounds__(256) void env_evaluate_standardize_kernel(const float* __restrict__ raw, float* __restrict__ obs, const float* __restrict__ mean,
                                                                       const float* __restrict__ precision, int n, int dim) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n * dim; i += gridDim.x * blockDim.x) obs[i] = (raw[i] - mean[i % dim]) * precision[i % dim];
}
// sample_and_squash in Evaluation mode (nn/layers/sample_and_squash/operations_generic.h:149-195 with zero noise): action = tanh(mean)
__global__ __launch_bounds__(256) void env_evaluate_squash_kernel(const float* __restrict__ out, float* __restrict__ actions, int n, int act) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n * act; i += gridDim.x * blockDim.x) actions[i] = tanhf(out[(size_t)(i / act) * 2 * act + i % act]);
}
// :187-197: an episode counts its steps and rewards up to and including the step that terminates it
__global__ __launch_bounds__(256) void env_evaluate_accumulate_kernel(const float* __restrict__ rewards, const uint8_t* __restrict__ terminated, uint8_t* __restrict__ done,
                                                                      float* __restrict__ returns, uint32_t* __restrict__ episode_length, int n) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        if (done[e]) continue;
        returns[e] += rewards[e]; episode_length[e] += 1;
        if (terminated[e]) done[e] = 1;
    }
}
// :213-228, sums in episode order as the reference makes them
__global__ void env_evaluate_summary_kernel(const float* __restrict__ returns, const uint32_t* __restrict__ episode_length, const uint8_t* __restrict__ done, int n,
                                            float* __restrict__ summary) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    float rm = 0.f, rs = 0.f, lm = 0.f, ls = 0.f;
    uint32_t num_terminated = 0;
    for (int e = 0; e < n; e++) {
        rm += returns[e]; rs += returns[e] * returns[e]; lm += (float)episode_length[e]; ls += (float)(episode_length[e] * episode_length[e]);
        num_terminated += done[e] ? 1 : 0;
    }
    rm /= (float)n; lm /= (float)n;
    summary[0] = rm; summary[1] = sqrtf(fmaxf(0.f, rs / (float)n - rm * rm));
    summary[2] = lm; summary[3] = sqrtf(fmaxf(0.f, ls / (float)n - lm * lm));
    summary[4] = (float)num_terminated; summary[5] = (float)num_terminated / (float)n;
}
struct EvaluateLayout { size_t states, raw, obs, out, actions, rewards, terminated, done, step_ws, total; };
EvaluateLayout evaluate_layout(const EnvDims& d, const rlt_seq_layer* policy, int n_layers, int N) {
    EvaluateLayout L;
    size_t at = 0;
    auto take = [&](size_t bytes) { const size_t here = at; at += align256(bytes); return here; };
    L.states = take((size_t)N * d.state * sizeof(float)); L.raw = take((size_t)N * d.obs * sizeof(float)); L.obs = take((size_t)N * d.obs * sizeof(float));
    L.out = take((size_t)N * 2 * d.act * sizeof(float)); L.actions = take((size_t)N * d.act * sizeof(float)); L.rewards = take((size_t)N * sizeof(float));
    L.terminated = take((size_t)N); L.done = take((size_t)N);
    L.step_ws = at; L.total = at + rlt_rocm_seq_evaluate_step_workspace_bytes(policy, n_layers, N) + 512;
    return L;
}
}  // namespace

extern "C" size_t rlt_rocm_env_evaluate_workspace_bytes(int env_kind, const rlt_seq_layer* policy, int n_policy_layers, int n_episodes) {
    const EnvDims d = env_dims(env_kind);
    if (!d.state || !policy || n_policy_layers < 1 || n_episodes < 1) return 0;
    return evaluate_layout(d, policy, n_policy_layers, n_episodes).total;
}

// Episodes that have terminated keep being stepped (their rows are never read again: every episode is a row of its own in the environment kernels and in the policy),
// where the reference leaves their state as it was (:166-170); returns, lengths and the terminated count stop at the terminating step as there.
extern "C" int rlt_rocm_env_evaluate(rlt_rocm_device* device, const rlt_env_runner* env, int policy_kind, const rlt_seq_layer* policy, int n_policy_layers,
                                     const rlt_seq_state* policy_state, int auto_reset_period, const float* observation_mean, const float* observation_precision,
                                     const float* initial_states, int n_episodes, int step_limit, float* returns, uint32_t* episode_length, float* summary,
                                     void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(env && policy && n_policy_layers >= 1 && n_policy_layers <= RLT_SEQ_MAX_LAYERS && initial_states && n_episodes >= 1 && step_limit >= 1 && returns && episode_length && summary);
    RLT_REQUIRE((policy_kind == 1 || policy_kind == 2) && (observation_mean == nullptr) == (observation_precision == nullptr) && auto_reset_period >= 0);
    const EnvDims d = env_dims(env->env_kind);
    RLT_REQUIRE(d.state != 0);
    bool recurrent = false;
    for (int l = 0; l < n_policy_layers; l++) recurrent = recurrent || policy[l].kind != 0;
    RLT_REQUIRE(!recurrent || policy_state);
    const rlt_seq_layer& first = policy[0]; const rlt_seq_layer& last = policy[n_policy_layers - 1];
    RLT_REQUIRE((first.kind == 0 ? first.dense.in_dim : first.gru.input_dim) == d.obs && (last.kind == 0 ? last.dense.out_dim : last.gru.hidden_dim) == policy_kind * d.act);
    const int N = n_episodes, blocks = rlt_div_up(N, 256) > 1024 ? 1024 : rlt_div_up(N, 256);
    const EvaluateLayout L = evaluate_layout(d, policy, n_policy_layers, N);
    RLT_REQUIRE(workspace && workspace_bytes >= L.total);
    char* w = reinterpret_cast<char*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    float* states = (float*)(w + L.states); float* raw = (float*)(w + L.raw); float* obs = (float*)(w + L.obs); float* out = (float*)(w + L.out);
    float* actions = (float*)(w + L.actions); uint8_t* done = (uint8_t*)(w + L.done);
    const size_t step_ws_bytes = workspace_bytes - (size_t)((w + L.step_ws) - (char*)workspace);
    rlt_env_runner rn = *env;
    rn.n_envs = N; rn.states = states; rn.actions = actions; rn.rewards = (float*)(w + L.rewards); rn.terminated = (uint8_t*)(w + L.terminated);
    float* next_obs = observation_mean ? raw : obs;      // the environment's step kernel leaves the observation of the state it arrives at
    const rlt_seq_state no_state = {};
    int rc;
    hipLaunchKernelGGL(env_copy_kernel, dim3(blocks), dim3(256), 0, device->stream, initial_states, states, (size_t)N * d.state);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_fill_f32(device, returns, 1, N, N, 0.0f))) return rc;
    if ((rc = rlt_rocm_fill_f32(device, (float*)episode_length, 1, N, N, 0.0f))) return rc;      // the bit pattern of 0.0f is the integer 0
    if ((rc = rlt_rocm_fill_u8(device, done, (size_t)N, 0))) return rc;
    if (policy_state && (rc = rlt_rocm_seq_reset_state(device, policy, n_policy_layers, policy_state, nullptr, N))) return rc;      // :135
    hipLaunchKernelGGL(env_evaluate_observe_kernel, dim3(blocks), dim3(256), 0, device->stream, (int)env->env_kind, (const float*)states, next_obs, N);
    if ((rc = rlt_launch_status(device))) return rc;
    for (int step = 0; step < step_limit; step++) {
        if (observation_mean) {
            hipLaunchKernelGGL(env_evaluate_standardize_kernel, dim3(blocks), dim3(256), 0, device->stream, (const float*)raw, obs, observation_mean, observation_precision, N, d.obs);
            if ((rc = rlt_launch_status(device))) return rc;
        }
        float* y = policy_kind == 1 ? actions : out;
        if ((rc = rlt_rocm_seq_evaluate_step(device, policy, n_policy_layers, obs, d.obs, policy_state ? policy_state : &no_state, auto_reset_period, y, policy_kind * d.act, N,
                                             w + L.step_ws, step_ws_bytes))) return rc;
        if (policy_kind == 2) {
            hipLaunchKernelGGL(env_evaluate_squash_kernel, dim3(blocks), dim3(256), 0, device->stream, (const float*)out, actions, N, d.act);
            if ((rc = rlt_launch_status(device))) return rc;
        }
        if ((rc = env_step_launch(device, &rn, next_obs))) return rc;
        hipLaunchKernelGGL(env_evaluate_accumulate_kernel, dim3(blocks), dim3(256), 0, device->stream, (const float*)rn.rewards, (const uint8_t*)rn.terminated, done, returns,
                           episode_length, N);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    hipLaunchKernelGGL(env_evaluate_summary_kernel, dim3(1), dim3(64), 0, device->stream, (const float*)returns, (const uint32_t*)episode_length, (const uint8_t*)done, N, summary);
    return rlt_launch_status(device);
}
