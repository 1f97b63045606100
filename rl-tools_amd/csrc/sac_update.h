// Internal entry points of sac_update.hip: the fused SAC updates for 3-layer networks of hidden width 64.
#pragma once
#include "common.h"

// true if the agent fits the fused kernels: every network 3 layers in -> 64 -> 64 -> out with one hidden activation (not GELU), at most 128
// critic inputs and 8 actions, no sequence masks
bool rlt_sac_update_supported(const rlt_rocm_device* device, const rlt_sac_agent* agent);
// The N(0, 1) noise of an update: an array [batch x action_dim] filled beforehand (values), or, with values == NULL, the elements of
// the stream (seed, stream) that rlt_rocm_randn_f32 would have put there, drawn by the kernel itself; `drawn` (optional) then receives them.
struct rlt_update_noise { const float* values; uint64_t seed, stream; float* drawn; };
// train_critic / train_actor with the contracts of rlt_rocm_sac_train_critic / rlt_rocm_sac_train_actor; of the training buffers only
// next_log_probabilities and target_action_value / actor_log_probabilities, actor_actions and actor_pre_squashing are written.
// One launch each where the Adam tensors are the networks' gradient buffers (the last workgroup to finish adds up the partial
// gradients and steps), else the optimiser follows as launches of its own. RLT_E_UNSUPPORTED unless rlt_sac_update_supported.
int rlt_sac_update_critic(rlt_rocm_device* device, const rlt_sac_agent* agent, int critic_index, const rlt_update_noise& noise);
int rlt_sac_update_actor(rlt_rocm_device* device, const rlt_sac_agent* agent, const rlt_update_noise& noise);
// both train_critic calls on the agent's batch with the same noise in ONE launch and, if update_targets, update_critic_targets after them
int rlt_sac_update_critics(rlt_rocm_device* device, const rlt_sac_agent* agent, const rlt_update_noise& noise, bool update_targets);
// The same updates for three-layer networks of any hidden width up to 256 (sac_wide.hip): a launch that lays the second layers' weights out for the
// wavefronts, the update kernel, and the optimisers' launch, which adds up the workgroups' blocks of partial sums; batches of at most 2,048 rows, no masks.
// `first`, `count`: the critics trained by the launch (one of them, or both on the same batch and noise; update_targets only with both).
bool rlt_sac_wide_supported(const rlt_rocm_device* device, const rlt_sac_agent* agent);
int rlt_sac_wide_update_critics(rlt_rocm_device* device, const rlt_sac_agent* agent, int first, int count, const rlt_update_noise& noise, bool update_targets);
int rlt_sac_wide_update_actor(rlt_rocm_device* device, const rlt_sac_agent* agent, const rlt_update_noise& noise);
// target[i] = polyak * target[i] + (1 - polyak) * source[i] for a list of tensors, one launch per 16 tensors
int rlt_sac_polyak_list(rlt_rocm_device* device, const float* const* sources, float* const* targets, const uint32_t* counts, int n, float polyak);

// The same for TD3 (rl/algorithms/td3/operations_generic.h:170-281): actors obs -> 64 -> 64 -> act with a tanh output followed by the
// td3_sampling layer, critics as above, no masks.
bool rlt_td3_update_supported(const rlt_rocm_device* device, const rlt_td3_agent* agent);
int rlt_td3_update_critic(rlt_rocm_device* device, const rlt_td3_agent* agent, int critic_index, const float* sampling_noise);
// both critics in one launch; draws != NULL: the noise tensors are drawn inside it; update_targets: update_critic_targets afterwards
int rlt_td3_update_critics(rlt_rocm_device* device, const rlt_td3_agent* agent, const float* sampling_noise_first, const float* sampling_noise_second, const rlt_td3_critic_draws* draws, bool update_targets);
// sampling_noise NULL: drawn inside the launch from (seed, stream)
int rlt_td3_update_actor(rlt_rocm_device* device, const rlt_td3_agent* agent, const float* sampling_noise, uint64_t seed, uint64_t stream);
// and at hidden widths up to 256 (sac_wide.hip)
bool rlt_td3_wide_supported(const rlt_rocm_device* device, const rlt_td3_agent* agent);
int rlt_td3_wide_update_critic(rlt_rocm_device* device, const rlt_td3_agent* agent, int critic_index, const float* sampling_noise);
// draws != NULL: the two sampling noises and the smoothing noise are drawn inside the launch
int rlt_td3_wide_update_critics(rlt_rocm_device* device, const rlt_td3_agent* agent, const float* sampling_noise_first, const float* sampling_noise_second, const rlt_td3_critic_draws* draws, bool update_targets);
// (update_targets: update_critic_targets after the two updates, in the optimisers' launch where the tensors correspond)
// sampling_noise NULL: drawn inside the launch from (seed, stream)
int rlt_td3_wide_update_actor(rlt_rocm_device* device, const rlt_td3_agent* agent, const float* sampling_noise, uint64_t seed, uint64_t stream);

// forward + backward (with weight gradients, added onto the layers' gradients) of one three-layer network of hidden width up to 256 over at most RLT_MLP_WIDE_MAX_BATCH
// rows on the wide update kernels' machinery (sac_wide.hip): input width up to 128, output width up to 16, no output activation. d_output or target (the MSE's
// gradient (y - target) * mse_scale) as in rlt_rocm_mlp_forward_backward. RLT_E_UNSUPPORTED for any other network.
constexpr int RLT_MLP_WIDE_MAX_BATCH = 4096;
int rlt_mlp_wide_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy,
                                  const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch);
// the backward pass alone (weight gradients, no input gradient) from the outputs that a forward() left in layers 1 and 2; d_pre_last [batch x out] is the gradient at the last
// layer's pre-activations, whatever that layer's activation
int rlt_mlp_wide_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, const float* d_pre_last, int ldd, int batch);
// forward() alone, storing every layer's pre-activations and outputs (those of the layers that have the buffers) where `keep` is set, and the network's output into y
// (optional, leading dimension ldy); any output activation
int rlt_mlp_wide_forward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy, int batch, bool keep);
