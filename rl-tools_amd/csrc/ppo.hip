// PPO generalized advantage estimation.
// reference: rl/algorithms/ppo/operations_generic.h:60-95 (serial double loop on the host; rows are step-major,
// row = step * n_envs + env, rl/components/on_policy_runner/on_policy_runner.h:38-72).
#include "common.h"

namespace {
// one lane per environment, reverse scan over the steps; at a fixed step adjacent lanes touch adjacent dataset rows
__global__ __launch_bounds__(256) void gae_kernel(const float* __restrict__ rewards, const float* __restrict__ terminated, const float* __restrict__ truncated,
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
}  // namespace

extern "C" int rlt_rocm_ppo_gae(rlt_rocm_device* device, const float* rewards, const float* terminated, const float* truncated, const float* all_values,
                                float* advantages, float* target_values, int ld, int n_envs, int steps, float gamma, float lambda, int ignore_termination) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rewards && terminated && truncated && all_values && advantages && target_values && ld >= 1 && n_envs > 0 && steps > 0);
    int blocks = (n_envs + 63) / 64; if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(gae_kernel, dim3(blocks), dim3(64), 0, device->stream, rewards, terminated, truncated, all_values, advantages, target_values, ld, n_envs, steps,
                       gamma, lambda, ignore_termination);
    return rlt_launch_status(device);
}
