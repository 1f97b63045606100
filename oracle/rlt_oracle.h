/*
 * rlt_oracle.h -- CPU restatement of the reference algorithms of the dense-network training hot path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing shipped may call into this library: it exists so that tests,
 * the smoke check and the benchmark's cpu_baseline leg can check / time the HIP path against a plain
 * CPU statement of what the reference computes. Every function cites the reference file:line it follows.
 *
 * The entry points mirror include/rlt_rocm.h one to one (same structs, same argument meaning) with
 * host pointers instead of device pointers and no device handle.
 *
 * Pinning status of each function (what, other than this file, fixes its answers):
 *   dense/mlp forward+backward, adam, polyak, mse, sample_and_squash, sac target/min-q/train_*,
 *   replay add, gather_batch, pendulum, gae: checked against the reference itself compiled from
 *   /root/reference (oracle/_ref) and against golden vectors written by it (tests/golden), plus the
 *   closed-form / finite-difference checks in tests/test_oracle_*.py.
 *   ppo surrogate/train, gru forward/backward, td3 (sampling layer, noise, targets, train_*, target updates):
 *   checked bit for bit against the reference's own PPO loop, GRU layer and TD3 loop compiled from
 *   /root/reference (oracle/_ref), and against golden vectors written by them (tests/golden).
 *   on-policy collect (with the reference's RNG order), running normaliser, standardize statistics: bit for bit against the
 *   reference's PPO loop with observation normalisation on (oracle/_ref), golden vectors, and closed forms in numpy.
 *   pendulum evaluate (evaluation episodes): returns, episode lengths and summary statistics bit for bit against the reference's
 *   rl::utils::evaluation::evaluate on the SAC loop's actor at three stages of training (oracle/_ref), golden vectors, and the
 *   identity between the two policy kinds on a mean-only copy of the actor.
 *   acrobot step (dsdt, Runge-Kutta, reward, terminated, observe): bit for bit against the reference's Acrobot, AcrobotSwingup and EasyParameters
 *   environments (oracle/_ref/librlt_ref_envs_generic.so) on random states and closed chains, golden vectors, and energy conservation /
 *   integration order / work-energy checks that do not involve the reference.
 *   car step (single-track model, reward, terminated; no track): bit for bit against the reference's Car (oracle/_ref/librlt_ref_envs_generic.so),
 *   golden vectors, and closed forms (straight rolling, pose equivariance, no tire force below the speed threshold). On a track: bit for bit against
 *   the reference's CarTrack on its default track where the reference is mounted (the bitmap is not kept as a fixture), closed-form ray lengths in a
 *   straight corridor.
 *   gather for sequence batches: all seven tensors of the batch entry for entry against the reference's gather_batch on its own runner's rings
 *   (oracle/_ref/librlt_ref_gather_seq_generic.so; sequence length 8 with and without the default sampling switches, and 1), draws made on the
 *   reference's std::mt19937 in its order; golden vectors; structural invariants on synthetic rings.
 *   ppo train_epoch: the loop over ppo train_minibatch (pinned above) that the reference's train() runs per epoch.
 *   sequential models (dense / GRU layers, FAST_TANH gates) and sac train_critic / train_actor / target update on sequence batches
 *   (rlt_oracle_seq.cpp): every parameter bit for bit against the reference's SAC loop with its recurrent approximators over 400 loop steps at two
 *   depths (oracle/_ref/librlt_ref_sac_gru{3,5}_generic.so), the FAST_TANH gates also on the GRU layer alone (librlt_ref_gru_fast_generic.so);
 *   golden vectors; equality with the single-step update at sequence length 1, finite differences of a dense-GRU-GRU-dense model.
 *   seq reset_state / evaluate_step / pendulum runner step with a recurrent policy: runner, policy state and replay rings bit for bit against the
 *   same loop over 300 steps at two depths, the step's draws taken from a copy of the reference's engine; golden vectors; a chain of single steps
 *   equals the sequence forward pass.
 *   td3_sequence_*: every parameter and Adam age bit for bit against the reference's TD3 loop with its recurrent approximators over 300 loop steps at two
 *   depths (oracle/_ref/librlt_ref_td3_gru{4,5}_generic.so), target values and d_output too.
 *   philox4x32_10, rand_bits / rand / randn / gather_draw / gather_sequence_draw / pendulum_initial_states (rlt_oracle_rng.cpp): the block function against the three
 *   published known-answer vectors of Philox4x32-10; the conversions by range, moments and Kolmogorov-Smirnov distance; no reference counterpart
 *   fixes the sequence itself (the reference's CUDA and CPU generators differ from each other).
 *   reduce_sum_f32, adam_reset: against numpy closed forms (tests/test_oracle_rng.py, tests/test_oracle_closed_forms.py).
 *   pendulum_evaluate_recurrent: returns, lengths and summary bit for bit against rl::utils::evaluation::evaluate on that loop's recurrent actor at two
 *   depths, untrained and trained; golden vectors; equality with pendulum_evaluate for a policy of dense layers only.
 *   pendulum_evaluate_standardized: identity statistics give pendulum_evaluate's results exactly; other statistics give those of the network with the
 *   statistics folded into its first layer (tests/test_oracle_closed_forms.py). The layer itself, (x - mean) * precision, is the one the PPO loop's
 *   standardize pins cover (ppo_train_minibatch with standardize layers, on_policy_collect).
 *   env_evaluate: with the Pendulum it reproduces the reference's evaluation vectors bit for bit (the loop shared with pendulum_evaluate); with the Acrobot, whose
 *   episodes terminate, every episode equals that episode run alone through acrobot_step (pinned against the reference's own step) until its first terminated
 *   flag, the terminating step's reward counted and nothing after it, and the terminated count and share follow (tests/test_oracle_golden.py). The reference's
 *   evaluate was not run on an environment that terminates: the bookkeeping after a termination (rl/utils/evaluation/operations_generic.h:166-197) is restated
 *   from its text and pinned by that per-episode construction only.
 */
#ifndef RLT_ORACLE_H
#define RLT_ORACLE_H
#include "../include/rlt_rocm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* 0: accumulate dot products in fp32 in the reference's loop order (default, the faithful restatement);
 * 1: accumulate in fp64 and round once (used as ground truth when judging fp32 summation error). */
void rlt_oracle_set_f64_accumulate(int enabled);
/* 1: route the three GEMMs of a dense layer through cblas_sgemm of the given shared library
 * (the reference's CPU_BLAS device does this); 0: plain loops. Returns 0 on success. */
int rlt_oracle_use_cblas(const char* library_path);
const char* rlt_oracle_cblas_name(void);

float rlt_oracle_activation(float x, int activation);
float rlt_oracle_d_activation(float x, int activation);

int rlt_oracle_dense_evaluate(const rlt_dense_layer* layer, const float* x, int ldx, float* y, int ldy, int batch);
int rlt_oracle_dense_forward(const rlt_dense_layer* layer, const float* x, int ldx, float* y, int ldy, int batch);
int rlt_oracle_dense_backward_input(const rlt_dense_layer* layer, float* d_output, int ldd, float* d_input, int ldi, int batch);
int rlt_oracle_dense_backward(const rlt_dense_layer* layer, const float* x, int ldx, float* d_output, int ldd, int batch);
int rlt_oracle_dense_backward_full(const rlt_dense_layer* layer, const float* x, int ldx, float* d_output, int ldd, float* d_input, int ldi, int batch);

int rlt_oracle_mlp_evaluate(const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy, int batch);
int rlt_oracle_mlp_forward(const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, int batch);
int rlt_oracle_mlp_backward(const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* d_output, int ldd,
                            float* d_input, int ldi, int batch, int want_weight_gradients);
int rlt_oracle_mlp_zero_gradient(const rlt_dense_layer* layers, int n_layers);
int rlt_oracle_mlp_forward_backward(const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy,
                                    const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch);

int rlt_oracle_adam_step(const rlt_adam_tensor* tensors, int n_tensors, const rlt_adam_parameters* parameters, uint32_t* age,
                         float polyak, float* out_gradient_squared_norm);
int rlt_oracle_adam_reset(const rlt_adam_tensor* tensors, int n_tensors, uint32_t* age);
int rlt_oracle_polyak_update(const float* source, float* target, size_t count, float polyak, int squared);

int rlt_oracle_mse_gradient(const float* a, int lda, const float* b, int ldb, float* d_a, int ldda, int rows, int cols,
                            float loss_weight, const float* loss_weight_ptr);
int rlt_oracle_mse_evaluate(const float* a, int lda, const float* b, int ldb, int rows, int cols, float loss_weight, float* out_loss);

int rlt_oracle_sas_forward(const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                           float* actions, int lda, float* pre_squashing, int ldp, float* log_probabilities, int batch, int dim);
int rlt_oracle_sas_backward(const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                            const float* actions, int lda, const float* pre_squashing, int ldp,
                            const float* d_output, int lddo, float* d_input, int lddi,
                            const float* log_alpha, float* d_log_alpha, int batch, int dim);

int rlt_oracle_sac_target_action_values(const float* q1_next, const float* q2_next, const float* rewards, const uint8_t* terminated,
                                        const float* next_log_probabilities, const float* log_alpha, float gamma, int ignore_termination,
                                        float* target, int batch);
int rlt_oracle_sac_min_value_d_output(const float* q1, const float* q2, const float* d_critic_1_input, const float* d_critic_2_input,
                                      int ld_critic_input, int critic_input_dim, int action_dim, float* d_actor_output, int ldo, int batch);
int rlt_oracle_mask_copy(const float* source, int lds, float* target, int ldt, const uint8_t* mask, int invert, int rows, int cols);
int rlt_oracle_mask_zero(float* gradient, int ld, const uint8_t* mask, int invert, int rows, int cols);
int rlt_oracle_scale_f32(float* x, size_t count, float s, int reciprocal);
int rlt_oracle_cast_reduce_sum_u8(const uint8_t* mask, size_t count, float* out_sum);
/* squared_sum / sum of a tensor (containers/tensor/operations_generic.h:497-520,803; gradient_norm of a parameter,
 * nn/parameters/operations_generic.h:85-87), accumulated in double and rounded once */
int rlt_oracle_reduce_sum_f32(const float* x, size_t count, int squared, float* out_sum);

/* ---- random draws (rlt_oracle_rng.cpp): Philox4x32-10 and the (seed, stream, element) mapping of include/rlt_rocm.h */
int rlt_oracle_philox4x32_10(const uint32_t* counter, const uint32_t* key, uint32_t* out);   /* the block function on explicit words */
int rlt_oracle_rand_bits_u32(uint32_t* dst, size_t count, uint64_t seed, uint64_t stream);
int rlt_oracle_rand_f32(float* dst, size_t count, float low, float high, uint64_t seed, uint64_t stream);
int rlt_oracle_randn_f32(float* dst, size_t count, uint64_t seed, uint64_t stream);
int rlt_oracle_gather_draw(const rlt_replay_buffer* rb, int batch, uint64_t seed, uint64_t stream, uint32_t* env_indices, uint32_t* sample_offsets);
int rlt_oracle_gather_sequence_draw(const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling, int max_episode_length, int batch, int sequence_length, uint64_t seed,
                                    uint64_t stream, uint32_t* env_indices, uint32_t* sample_offsets, uint8_t* nominal, uint32_t* lengths);
int rlt_oracle_pendulum_initial_states(float* states, int n_envs, uint64_t seed, uint64_t stream);

int rlt_oracle_sac_train_critic(const rlt_sac_agent* agent, int critic_index, const float* action_noise);
int rlt_oracle_sac_update_critic_targets(const rlt_sac_agent* agent);
int rlt_oracle_sac_train_actor(const rlt_sac_agent* agent, const float* action_noise);
int rlt_oracle_sas_backward_reset(const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                                  const float* actions, int lda, const float* pre_squashing, int ldp,
                                  const float* d_output, int lddo, float* d_input, int lddi,
                                  const float* log_alpha, float* d_log_alpha, const uint8_t* reset, int batch, int dim);
/* sequential (recurrent) models and SAC on sequence batches: oracle/rlt_oracle_seq.cpp */
int rlt_oracle_seq_forward(const rlt_seq_layer* layers, int n_layers, const float* x, int ldx, const uint8_t* reset, int steps, int batch);
int rlt_oracle_seq_backward(const rlt_seq_layer* layers, int n_layers, const float* x, int ldx, float* d_output, float* d_input, const uint8_t* reset,
                            int steps, int batch, int want_weight_gradients, int reset_in_backward_input);
int rlt_oracle_seq_zero_gradient(const rlt_seq_layer* layers, int n_layers);
int rlt_oracle_seq_reset_state(const rlt_seq_layer* layers, int n_layers, const rlt_seq_state* state, const uint8_t* mask, int batch);
int rlt_oracle_seq_evaluate_step(const rlt_seq_layer* layers, int n_layers, const float* x, int ldx, const rlt_seq_state* state, int auto_reset_period,
                                 float* y, int ldy, int batch);
int rlt_oracle_pendulum_runner_prologue(const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb, const float* initial_states, float* observations);
int rlt_oracle_pendulum_runner_epilogue(const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb, const float* observations, const float* actions);
int rlt_oracle_pendulum_runner_step_recurrent(const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n_policy_layers,
                                              const rlt_seq_state* policy_state, int auto_reset_period, const rlt_sas_parameters* sas, const float* action_noise,
                                              const float* initial_states);
int rlt_oracle_sac_sequence_train_critic(const rlt_sac_sequence_agent* agent, int critic_index, const float* action_noise);
int rlt_oracle_sac_sequence_update_critic_targets(const rlt_sac_sequence_agent* agent);
int rlt_oracle_sac_sequence_train_actor(const rlt_sac_sequence_agent* agent, const float* action_noise);

int rlt_oracle_replay_add(const rlt_replay_buffer* rb, const float* observations, const float* actions, const float* rewards,
                          const float* next_observations, const uint8_t* terminated, const uint8_t* truncated);
int rlt_oracle_gather_batch(const rlt_replay_buffer* rb, const uint32_t* env_indices, const uint32_t* sample_offsets, int deterministic,
                            int max_episode_length, int batch, float* observations_actions_base, float* rewards, uint8_t* terminated,
                            uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base);

int rlt_oracle_pendulum_step(const rlt_pendulum_parameters* p, float* states, const float* actions, float* observations,
                             float* next_observations, float* rewards, int n_envs);
int rlt_oracle_pendulum_runner_step(const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb, int policy_kind,
                                    const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas,
                                    const float* actions_in, const float* action_noise, const float* initial_states);

int rlt_oracle_ppo_gae(const float* rewards, const float* terminated, const float* truncated, const float* all_values,
                       float* advantages, float* target_values, int ld, int n_envs, int steps, float gamma, float lambda,
                       int ignore_termination);

/* gather_batch for sequence batches, rl/components/off_policy_runner/operations_generic.h:239-430; the second form makes the draws itself on the
 * reference's std::mt19937 (text form in, text form out) and returns them in the layout of rlt_sequence_draws */
int rlt_oracle_gather_sequence_batch(const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling, const rlt_sequence_draws* draws, int max_episode_length,
                                     const rlt_sequence_batch* batch);
int rlt_oracle_gather_sequence_batch_with_rng(const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling, int max_episode_length, const rlt_sequence_batch* batch,
                                              char* rng_state, int rng_capacity, uint32_t* env_indices, uint32_t* sample_offsets, uint8_t* nominal, uint32_t* lengths);
/* rl/environments/acrobot/operations_generic.h:56-193 */
int rlt_oracle_env_runner_step(const rlt_env_runner* runner, const rlt_replay_buffer* rb, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers,
                               const rlt_sas_parameters* sas, const float* actions_in, const float* action_noise, const float* initial_states);
int rlt_oracle_env_on_policy_collect(const rlt_env_runner* runner, const rlt_on_policy_dataset* dataset, const rlt_seq_layer* policy, int n_policy_layers,
                                     const rlt_seq_state* policy_state, int auto_reset_period, const float* log_std, const float* standardize_mean,
                                     const float* standardize_precision, const float* action_noise, const float* initial_states, int truncate_on_each_iteration);
int rlt_oracle_env_runner_step_sequential(const rlt_env_runner* runner, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n_policy_layers,
                                          const rlt_seq_state* policy_state, int auto_reset_period, int head_kind, const rlt_sas_parameters* sas, float exploration_noise_std,
                                          const float* action_noise, const float* initial_states);
int rlt_oracle_env_evaluate(const rlt_env_runner* env, int policy_kind, const rlt_seq_layer* policy, int n_policy_layers, const rlt_seq_state* policy_state, int auto_reset_period,
                            const float* observation_mean, const float* observation_precision, const float* initial_states, int n_episodes, int step_limit, float* returns,
                            uint32_t* episode_length, float* summary);
int rlt_oracle_unary_f32(int operation, float parameter, const float* src, int ld_src, float* dst, int ld_dst, int rows, int cols);
int rlt_oracle_binary_f32(int operation, const float* a, int lda, const float* b, int ldb, float* dst, int ld_dst, int rows, int cols);
int rlt_oracle_multiply_accumulate_f32(const float* a, int lda, const float* b, int ldb, const float* accumulator, int ldc, float* dst, int ld_dst, int rows, int cols);
int rlt_oracle_reduce_abs_max_f32(const float* x, size_t count, float* out_max);
int rlt_oracle_mlp_forward_backward_input(const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy, const float* d_output, int ldd,
                                          const float* target, int ldt, float mse_scale, float* d_input, int ldi, int batch);
int rlt_oracle_acrobot_step(const rlt_acrobot_parameters* p, int swingup, float* states, const float* actions, float* observations, float* next_observations,
                            float* rewards, uint8_t* terminated, int n_envs);
/* rl/environments/car/operations_generic.h:80-155 (the Car without a track) */
int rlt_oracle_car_step(const rlt_car_parameters* p, float* states, const float* actions, float* observations, float* next_observations, float* rewards,
                        uint8_t* terminated, int n_envs);
int rlt_oracle_car_track_step(const rlt_car_parameters* p, const uint8_t* track, int height, int width, float track_scale, float* states, const float* actions,
                              float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n_envs);
/* rl::utils::evaluation::evaluate with the Pendulum environment (rl/utils/evaluation/operations_generic.h:106-233) */
int rlt_oracle_pendulum_evaluate(const rlt_pendulum_parameters* env, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers, const float* initial_states,
                                 int n_episodes, int step_limit, float* returns, uint32_t* episode_length, float* summary);
/* the same with a sequential (recurrent) policy: state reset before the first step, evaluate_step per step (:135,:163) */
int rlt_oracle_pendulum_evaluate_standardized(const rlt_pendulum_parameters* env, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers, const float* observation_mean,
                                              const float* observation_precision, const float* initial_states, int n_episodes, int step_limit, float* returns,
                                              uint32_t* episode_length, float* summary);
int rlt_oracle_pendulum_evaluate_recurrent(const rlt_pendulum_parameters* env, int policy_kind, const rlt_seq_layer* policy, int n_layers, const rlt_seq_state* state,
                                           int auto_reset_period, const float* initial_states, int n_episodes, int step_limit, float* returns,
                                           uint32_t* episode_length, float* summary);
int rlt_oracle_ppo_surrogate_gradient(const float* action_means, int ld_means, const float* log_std, const float* actions, int ld_actions,
                                      const float* action_log_probs, int ld_log_probs, const float* advantages, int ld_advantages,
                                      const rlt_ppo_parameters* parameters, float* d_action_means, int ld_d, float* d_log_std, int batch, int action_dim);
int rlt_oracle_ppo_train_minibatch(const rlt_ppo_agent* agent, const rlt_ppo_parameters* parameters, const float* observations,
                                   const float* observations_privileged, const float* actions, const float* action_log_probs,
                                   const float* advantages, const float* target_values, int ld, const uint32_t* row_indices, float* out_critic_loss);
/* the batch loop of train() (rl/algorithms/ppo/operations_generic.h:156-318) over one epoch's permutation */
int rlt_oracle_ppo_train_epoch(const rlt_ppo_agent* agent, const rlt_ppo_parameters* parameters, const float* observations,
                               const float* observations_privileged, const float* actions, const float* action_log_probs,
                               const float* advantages, const float* target_values, int ld, const uint32_t* row_indices, int n_minibatches,
                               float* out_critic_losses);
int rlt_oracle_gru_forward(const rlt_gru_layer* layer, const float* input, const uint8_t* reset, int sequence_length, int batch);
int rlt_oracle_gru_backward(const rlt_gru_layer* layer, const float* input, float* d_output, float* d_input, const uint8_t* reset,
                            int sequence_length, int batch, int want_weight_gradients);
/* the reference's per-epoch in-place dataset shuffle as row permutations, driven by the text form of its std::mt19937 */
int rlt_oracle_ppo_shuffle(char* rng_state, int rng_state_capacity, int n, int epochs, uint32_t* permutations);

int rlt_oracle_td3_sampling_forward(const float* input, int ldin, const float* noise, int ldn, float std, float* pre_clip, int ldp,
                                    float* output, int ldo, int batch, int dim);
int rlt_oracle_td3_sampling_backward(const float* pre_clip, int ldp, const float* d_output, int lddo, float* d_input, int lddi, int batch, int dim);
int rlt_oracle_td3_target_action_noise(const float* standard_normal, float std, float clip, float* out, size_t count);
int rlt_oracle_td3_noisy_next_actions(float* next_actions, int lda, const float* noise, int ldn, int batch, int dim);
int rlt_oracle_td3_target_action_values(const float* q1_next, const float* q2_next, const float* rewards, const uint8_t* terminated,
                                        float gamma, int ignore_termination, float* target, int batch);
int rlt_oracle_td3_train_critic(const rlt_td3_agent* agent, int critic_index, const float* sampling_noise);
int rlt_oracle_td3_train_actor(const rlt_td3_agent* agent, const float* sampling_noise);
int rlt_oracle_td3_update_critic_targets(const rlt_td3_agent* agent);
int rlt_oracle_td3_update_actor_target(const rlt_td3_agent* agent);
/* TD3 on sequence batches with sequential (recurrent) networks: rl/algorithms/td3/operations_generic.h:170-325 */
int rlt_oracle_td3_sequence_train_critic(const rlt_td3_sequence_agent* agent, int critic_index);
int rlt_oracle_td3_sequence_train_actor(const rlt_td3_sequence_agent* agent);
int rlt_oracle_td3_sequence_update_critic_targets(const rlt_td3_sequence_agent* agent);
int rlt_oracle_td3_sequence_update_actor_target(const rlt_td3_sequence_agent* agent);

int rlt_oracle_standardize_set_statistics(const float* mean, const float* std, float* layer_mean, float* layer_precision, int dim);
int rlt_oracle_standardize_forward(const float* layer_mean, const float* layer_precision, const float* input, int ldin, float* output, int ldo, int batch, int dim);
int rlt_oracle_standardize_backward_input(const float* layer_precision, const float* d_output, int ldd, float* d_input, int ldi, int batch, int dim);
int rlt_oracle_running_normalizer_update(const float* data, int ld, int rows, int dim, float* mean, float* std, uint32_t* age);
int rlt_oracle_on_policy_collect(const rlt_pendulum_runner* runner, const rlt_on_policy_dataset* dataset, const rlt_dense_layer* actor, int n_actor_layers,
                                 const float* log_std, const float* standardize_mean, const float* standardize_precision, const float* action_noise,
                                 const float* initial_states, int truncate_on_each_iteration);
/* The draws collect() takes from the reference's std::mt19937, in its order, without running the networks' arithmetic twice: the engine (text
 * form, advanced in place) is consumed exactly as the reference's collect consumes it -- per step, per environment that resets two uniform
 * draws (initial theta, theta_dot), then per environment and action dimension one normal draw -- which needs the truncation pattern, so this
 * runs the collection itself with the drawn values and also returns them: action_noise receives the N(0,1) value behind every N(mean, std)
 * draw, initial_states the drawn states (rows of environments that do not reset are left untouched). */
int rlt_oracle_on_policy_collect_with_rng(const rlt_pendulum_runner* runner, const rlt_on_policy_dataset* dataset, const rlt_dense_layer* actor, int n_actor_layers,
                                          const float* log_std, const float* standardize_mean, const float* standardize_precision, float* action_noise,
                                          float* initial_states, int truncate_on_each_iteration, char* rng_state, int rng_state_capacity);

#ifdef __cplusplus
}
#endif
#endif
