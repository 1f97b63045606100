// Single-pass forward + backward of a 3-layer MLP in -> 64 -> 64 -> out (mlp_small.hip).
#pragma once
#include "common.h"

// true if the network has a shape the kernel is built for: in -> 64 -> 64 -> out or in -> 64 -> out, in <= 128, hidden activation relu, tanh or
// fast_tanh (the same in both hidden layers), out <= 16 with an activation whose derivative follows from the output
bool rlt_mlp3s_supported(const rlt_dense_layer* layers, int n_layers);

// same contract as rlt_rocm_mlp_forward_backward (partial sums live in the device handle's scratch), plus the optional gradient with respect to x
// into d_input [batch x in]; RLT_E_UNSUPPORTED if the shape does not fit
int rlt_mlp3s_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy,
                               const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch, float* d_input = nullptr, int ldi = 0);

// PPO actor pass (rl/algorithms/ppo/operations_generic.h:203-285): forward, the clipped-surrogate gradient per sample, backward. `stats` =
// {advantage mean, advantage std} on the device. Means go to `means` [batch x action_dim]; weight gradients are accumulated into the layers,
// the surrogate part of the log_std gradient plus `log_std_gradient_offset` into d_log_std (if non-NULL).
int rlt_mlp3s_ppo_actor(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* means, int ld_means,
                        const float* log_std, const float* actions, int ld_actions, const float* log_probs, int ld_lp, const float* advantages, int ld_adv,
                        const float* stats, const rlt_ppo_parameters* P, float* d_log_std, float log_std_gradient_offset, int batch);

// true if the two networks can share a launch: both of the supported shape, the same hidden activation, input widths on the same side of 32
bool rlt_mlp3s_pair_supported(const rlt_dense_layer* a, int n_a, const rlt_dense_layer* b, int n_b);

// steps[0] (actor), steps[1] (critic), optional: the optimisers' steps (nn/optimizers/adam/operations_generic.h:43-66) follow in ONE launch that adds the
// workgroups' blocks of partial gradient sums up itself, where each optimiser's tensors are exactly the network's gradient buffers (the actor's plus
// d_log_std); *stepped then is true. Otherwise the gradients are formed as without `steps` and the caller steps the optimisers.
struct rlt_mlp3s_step { const rlt_adam_tensor* tensors; int n; const rlt_adam_parameters* parameters; uint32_t* age; };

// The same actor pass and the critic's forward + MSE gradient + backward (:289-300) in ONE launch, each network on half of the compute units,
// straight from the dataset: every input column has the dataset's row stride `ld`, and minibatch row b is dataset row rows[b] (rows == NULL: b).
// Means [batch x action_dim] and values [batch] are written packed; out_critic_loss (optional, critic output width 1) receives
// mse::evaluate(values, targets) = sum((v - t)^2) / batch. The gradients are OVERWRITTEN (what zero_gradient followed by backward
// leaves), so the caller skips zeroing them. RLT_E_UNSUPPORTED unless rlt_mlp3s_pair_supported. The optional standardize constants
// ([in] floats each) put a standardize layer in front of the network: it reads (x - mean) * precision (the factor where it is not 0).
int rlt_mlp3s_ppo_actor_critic(rlt_rocm_device* device, const rlt_dense_layer* actor, int n_actor, const float* x, float* means, int ld_means,
                               const float* log_std, const float* actions, const float* log_probs, const float* advantages,
                               const float* stats, const rlt_ppo_parameters* P, float* d_log_std, float log_std_gradient_offset,
                               const rlt_dense_layer* critic, int n_critic, const float* x_critic, float* values, int ld_values,
                               const float* target_values, float mse_scale, float* out_critic_loss, int ld, const uint32_t* rows, int batch,
                               const float* actor_std_mean = nullptr, const float* actor_std_precision = nullptr,
                               const float* critic_std_mean = nullptr, const float* critic_std_precision = nullptr,
                               const rlt_mlp3s_step* steps = nullptr, bool* stepped = nullptr);

// For kernels that write blocks of partial sums in this file's layout (dW1 [64 x in], db1 [64], dW2 [64 x 64], db2 [64], dW3 [out x 64], db3 [out],
// extra [16]): the floats per block, and the launch that adds `groups` blocks up in block order into the layers' gradients (overwrite != 0:
// gradient = sum) and, if `extra` is given, extra[i] = sum_i * extra_scale + extra_offset for i < n_extra.
int rlt_mlp3s_partial_count(int in_dim, int out_dim);
int rlt_mlp3s_reduce(rlt_rocm_device* device, const rlt_dense_layer* layers, const float* partial, int groups, int overwrite, float* extra, int n_extra,
                     float extra_scale, float extra_offset);
