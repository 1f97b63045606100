// Pieces that the fused SAC update kernels share: lane reductions of the matrix-instruction layouts and the per-row arithmetic of the
// sample_and_squash head (nn/layers/sample_and_squash/operations_generic.h:148-398).
// Lane l = r + 16 kk of a wavefront: r = row (or column) of a 16-wide tile, kk = lane group.
#pragma once
#include "common.h"

namespace rlt_sac {
typedef __attribute__((address_space(3))) float* lptr;

template <int CTRL>
__device__ __forceinline__ float dpp(float x) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true)); }
// sum over the 16 lanes of a row (r = 0..15), every lane of the row receives it
__device__ __forceinline__ float row16_sum(float x) { asm volatile("" : "+v"(x)); x += dpp<0xB1>(x); x += dpp<0x4E>(x); x += dpp<0x141>(x); x += dpp<0x140>(x); return x; }
// sum over the four lane groups (lanes r, r + 16, r + 32, r + 48), in a fixed order
__device__ __forceinline__ float groups_sum(float v) { asm volatile("" : "+v"(v)); v += __shfl_xor(v, 16, 64); v += __shfl_xor(v, 32, 64); return v; }
// lanes of one wavefront exchange data through LDS: the hardware executes a wavefront's LDS instructions in order, the fences keep
// the compiler from moving them across
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }
__device__ __forceinline__ float normal_log_prob(float mean, float log_std, float sd, float value) {
    const float z = (value - mean) / sd;
    return -0.9189385332046727f - log_std - 0.5f * z * z;
}

// sample_and_squash forward for the items of a lane of the wavefront that does the per-row work: row r, actions kk and kk + 4.
// d3s [16][D3S]: the actor's output rows [mean | log_std]; the action goes into columns OBS.. of xs [16][SX]. Returns the row's
// log-probability (in every lane of the row's four).
struct HeadItem { float mean, log_std_raw, noise, sample, action; };
__device__ __forceinline__ float head_forward(const rlt_sas_parameters& sas, int OBS, int ACT, lptr d3s, int D3S, lptr xs, int SX, const float (&noise)[2], int r, int kk, HeadItem (&item)[2]) {
    float log_prob = 0.f;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int a = kk + 4 * j;
        HeadItem& I = item[j];
        I = {0.f, 0.f, 0.f, 0.f, 0.f};
        if (a < ACT) {
            I.mean = d3s[r * D3S + a];
            I.log_std_raw = d3s[r * D3S + ACT + a];
            const float log_std = clampf(I.log_std_raw, sas.log_std_lower_bound, sas.log_std_upper_bound);
            const float sd = expf(log_std);
            I.noise = noise[j];
            I.sample = I.mean + I.noise * sd;
            I.action = tanhf(I.sample);
            xs[r * SX + OBS + a] = I.action;
            log_prob += normal_log_prob(I.mean, log_std, sd, I.sample) - logf(1.0f - I.action * I.action + sas.log_probability_epsilon);
        }
    }
    return groups_sum(log_prob);
}

// sample_and_squash backward for one item (nn/layers/sample_and_squash/operations_generic.h:262-398): d_out = the loss gradient at
// the action; returns the gradients at the mean and the raw log_std and adds the item's share of the row's entropy
__device__ __forceinline__ void head_backward(const rlt_sas_parameters& sas, const HeadItem& I, float d_out, float alpha_over_batch, float& d_mu, float& d_ls, float& entropy) {
    const float g = d_out * (1.0f - I.action * I.action);
    const float log_std = clampf(I.log_std_raw, sas.log_std_lower_bound, sas.log_std_upper_bound);
    const float sd = expf(log_std);
    const float z = (I.sample - I.mean) / sd;
    const float dlp_dmean = z / sd, dlp_dsample = -z / sd, dlp_dlogstd = z * z - 1.0f;
    d_mu = g + alpha_over_batch * (dlp_dmean + dlp_dsample + 2.0f * I.action);
    d_ls = sd * (g * I.noise) + alpha_over_batch * (dlp_dlogstd + dlp_dsample * I.noise * sd + 2.0f * I.action * I.noise * sd);
    if (I.log_std_raw < sas.log_std_lower_bound || I.log_std_raw > sas.log_std_upper_bound) d_ls = 0.0f;
    entropy -= normal_log_prob(I.mean, log_std, sd, I.sample) - logf(1.0f - I.action * I.action + sas.log_probability_epsilon);
}

// TD3's actor head for the items of a lane: tanh of the MLP's output, the td3_sampling layer (action = clamp(tanh(output) + sampling_std * noise, -1, 1),
// nn/layers/td3_sampling/operations_generic.h:75-128), and in the critic update the smoothing noise of the target action
// (rl/algorithms/td3/operations_generic.h:129-145). mean = tanh(output), sample = value before the clamp.
__device__ __forceinline__ void td3_head_forward(int OBS, int ACT, float sampling_std, lptr d3s, int D3S, lptr xs, int SX, const float (&noise)[2], const float (&target_noise)[2],
                                                 bool critic_update, int r, int kk, HeadItem (&item)[2]) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int a = kk + 4 * j;
        HeadItem& I = item[j];
        I = {0.f, 0.f, 0.f, 0.f, 0.f};
        if (a < ACT) {
            I.mean = tanhf(d3s[r * D3S + a]);
            I.noise = noise[j];
            float scaled = I.noise * sampling_std;
            asm volatile("" : "+v"(scaled));        // the product is rounded before the addition, as the per-operation kernels and the reference's CPU build do
            I.sample = scaled + I.mean;
            I.action = clampf(I.sample, -1.0f, 1.0f);
            if (critic_update) I.action = clampf(I.action + target_noise[j], -1.0f, 1.0f);
            xs[r * SX + OBS + a] = I.action;
        }
    }
}
}  // namespace rlt_sac
