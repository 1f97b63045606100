// PPO on devices::ROCM: estimate_generalized_advantages and train (the generic versions, rl/algorithms/ppo/operations_generic.h:60-95
// and :97-336, are host loops over samples; the reference has no CUDA version of them). malloc / free / init are the generic ones over
// the leaf overloads of this backend.
//
// train hands each epoch to the library (rlt_rocm_ppo_train_epoch): the reference shuffles the dataset's rows in place with its
// generator (:129-156) and then walks it in minibatches; here an epoch's shuffle is a permutation of row indices, drawn on the host by
// the same Fisher-Yates walk from a generator that is seeded from the device generator's stream, and the minibatches gather their rows
// through it (the dataset is left in place). The overload takes part for what the library's update covers: actor = [standardize ->]
// MLP with a state-independent log_std, critic = [standardize ->] MLP, fp32, stateless, no adaptive learning rate.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/algorithms/ppo/ppo.h>
#include <rl_tools/rl/algorithms/ppo/operations_generic.h>
#include <rl_tools/rl/components/on_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>
#include <rl_tools/nn/optimizers/adam/operations_rocm.h>
#include <random>
#include <vector>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    // estimate_generalized_advantages   rl/algorithms/ppo/operations_generic.h:60-95
    template <typename DEV_SPEC, typename DATASET_SPEC, typename PPO_PARAMETERS>
    void estimate_generalized_advantages(devices::ROCM<DEV_SPEC>& device, rl::components::on_policy_runner::Dataset<DATASET_SPEC>& dataset, PPO_PARAMETERS ppo_parameters_tag){
        using DATASET = rl::components::on_policy_runner::Dataset<DATASET_SPEC>;
        static_assert(utils::typing::is_same_v<typename DATASET::T, float>);
        static_assert(decltype(dataset.data)::SPEC::COL_PITCH == 1 && decltype(dataset.data)::SPEC::ROW_PITCH == DATASET::DATA_DIM);
        devices::rocm::check(rlt_rocm_ppo_gae(device.handle, dataset.rewards._data, dataset.terminated._data, dataset.truncated._data, dataset.all_values._data, dataset.advantages._data,
                                              dataset.target_values._data, (int)DATASET::DATA_DIM, (int)DATASET_SPEC::SPEC::N_ENVIRONMENTS, (int)DATASET_SPEC::STEPS_PER_ENV,
                                              (float)PPO_PARAMETERS::GAMMA, (float)PPO_PARAMETERS::LAMBDA, PPO_PARAMETERS::IGNORE_TERMINATION ? 1 : 0), "estimate_generalized_advantages");
    }
    // train                   rl/algorithms/ppo/operations_generic.h:97-336
    template <typename DEV_SPEC, typename PPO_SPEC, typename DATASET_SPEC, typename ACTOR_OPTIMIZER, typename CRITIC_OPTIMIZER, typename BUFFERS_SPEC, typename ACTOR_BUFFER, typename CRITIC_BUFFER, typename RNG>
    void train(devices::ROCM<DEV_SPEC>& device, rl::algorithms::PPO<PPO_SPEC>& ppo, rl::components::on_policy_runner::Dataset<DATASET_SPEC>& dataset, ACTOR_OPTIMIZER& actor_optimizer, CRITIC_OPTIMIZER& critic_optimizer, rl::algorithms::ppo::Buffers<BUFFERS_SPEC>& ppo_buffers, ACTOR_BUFFER& actor_buffers, CRITIC_BUFFER& critic_buffers, RNG& rng){
#ifdef RL_TOOLS_DEBUG_RL_ALGORITHMS_PPO_CHECK_INIT
        utils::assert_exit(device, ppo.initialized, "PPO not initialized");
#endif
        using DEVICE = devices::ROCM<DEV_SPEC>;
        using TI = typename PPO_SPEC::TI;
        using PARAMETERS = typename PPO_SPEC::PARAMETERS;
        using ENVIRONMENT = typename PPO_SPEC::ENVIRONMENT;
        using DATASET = rl::components::on_policy_runner::Dataset<DATASET_SPEC>;
        static_assert(utils::typing::is_same_v<typename PPO_SPEC::ENVIRONMENT, typename DATASET_SPEC::SPEC::ENVIRONMENT>, "environment mismatch");
        static_assert(utils::typing::is_same_v<typename PPO_SPEC::TYPE_POLICY::DEFAULT, float>, "the ROCM backend computes in fp32");
        static_assert(!PARAMETERS::STATEFUL_ACTOR_AND_CRITIC && !PARAMETERS::ADAPTIVE_LEARNING_RATE && ENVIRONMENT::N_AGENTS == 1, "the library's PPO update is the stateless single-agent one with a fixed learning rate");
        static_assert(decltype(dataset.data)::SPEC::COL_PITCH == 1 && decltype(dataset.data)::SPEC::ROW_PITCH == DATASET::DATA_DIM);
        constexpr TI N_EPOCHS = PARAMETERS::N_EPOCHS, BATCH_SIZE = PARAMETERS::BATCH_SIZE, N_BATCHES = DATASET::STEPS_TOTAL / BATCH_SIZE;
        static_assert(DATASET::STEPS_TOTAL > 1 && N_BATCHES > 0);
        namespace opr = rl::components::on_policy_runner::rocm;
        opr::ActorDescription actor, critic;
        opr::describe(ppo.actor, actor);
        opr::describe(ppo.critic, critic);
        utils::assert_exit(device, actor.n_layers > 0 && critic.n_layers > 0 && actor.log_std && actor.d_log_std, "train: the actor and the critic are not [standardize ->] mlp_unconditional_stddev models");
        std::vector<rlt_adam_tensor> actor_tensors = nn::optimizers::adam::rocm::collect<DEVICE, typename ACTOR_OPTIMIZER::SPEC>(device, ppo.actor, false);
        std::vector<rlt_adam_tensor> critic_tensors = nn::optimizers::adam::rocm::collect<DEVICE, typename CRITIC_OPTIMIZER::SPEC>(device, ppo.critic, false);
        rlt_ppo_agent agent = {};
        agent.actor = actor.layers; agent.n_actor_layers = actor.n_layers; agent.critic = critic.layers; agent.n_critic_layers = critic.n_layers;
        agent.log_std = actor.log_std; agent.d_log_std = actor.d_log_std;
        agent.actor_adam_tensors = actor_tensors.data(); agent.n_actor_adam_tensors = (int)actor_tensors.size();
        agent.critic_adam_tensors = critic_tensors.data(); agent.n_critic_adam_tensors = (int)critic_tensors.size();
        agent.actor_adam = rl::algorithms::sac::rocm::adam_parameters(actor_optimizer); agent.critic_adam = rl::algorithms::sac::rocm::adam_parameters(critic_optimizer);
        agent.actor_age = (uint32_t*)actor_optimizer.age._data; agent.critic_age = (uint32_t*)critic_optimizer.age._data;
        agent.observation_dim = ENVIRONMENT::Observation::DIM; agent.observation_privileged_dim = ENVIRONMENT::ObservationPrivileged::DIM; agent.action_dim = ENVIRONMENT::ACTION_DIM;
        agent.batch = BATCH_SIZE;
        agent.actor_standardize_mean = actor.standardize_mean; agent.actor_standardize_precision = actor.standardize_precision;
        agent.critic_standardize_mean = critic.standardize_mean; agent.critic_standardize_precision = critic.standardize_precision;
        rlt_ppo_parameters parameters = {};
        parameters.epsilon_clip = PARAMETERS::EPSILON_CLIP; parameters.action_entropy_coefficient = PARAMETERS::ACTION_ENTROPY_COEFFICIENT; parameters.advantage_epsilon = PARAMETERS::ADVANTAGE_EPSILON;
        parameters.normalize_advantage = PARAMETERS::NORMALIZE_ADVANTAGE ? 1 : 0; parameters.learn_action_std = PARAMETERS::LEARN_ACTION_STD ? 1 : 0;
        // device memory for this call: the library's workspace, one epoch's row indices, the minibatches' critic losses
        const size_t workspace_bytes = (rlt_rocm_ppo_workspace_bytes(&agent) + 255) / 256 * 256, index_bytes = ((size_t)N_BATCHES * BATCH_SIZE * sizeof(uint32_t) + 255) / 256 * 256;
        char* memory = (char*)devices::rocm::scratch(device, workspace_bytes + index_bytes + N_BATCHES * sizeof(float));
        agent.workspace = memory; agent.workspace_bytes = workspace_bytes;
        uint32_t* row_indices = (uint32_t*)(memory + workspace_bytes);
        float* critic_losses = (float*)(memory + workspace_bytes + index_bytes);
        std::vector<uint32_t> permutation(DATASET::STEPS_TOTAL);
        for(TI i = 0; i < DATASET::STEPS_TOTAL; i++){ permutation[i] = (uint32_t)i; }
        std::mt19937_64 shuffle_generator(((uint64_t)rng.seed << 32) ^ (uint64_t)random::next_stream(rng));
        for(TI epoch_i = 0; epoch_i < N_EPOCHS; epoch_i++){
            if constexpr(PARAMETERS::SHUFFLE_EPOCH){     // the same walk as :130-155, on indices: successive epochs shuffle the previous epoch's order
                for(TI dataset_i = 0; dataset_i < DATASET::STEPS_TOTAL; dataset_i++){
                    const TI sample_index = dataset_i + (TI)(shuffle_generator() % (uint64_t)(DATASET::STEPS_TOTAL - dataset_i));
                    std::swap(permutation[dataset_i], permutation[sample_index]);
                }
            }
            devices::rocm::check(rlt_rocm_memcpy_h2d(device.handle, row_indices, permutation.data(), (size_t)N_BATCHES * BATCH_SIZE * sizeof(uint32_t)), "train (row indices)");
            devices::rocm::check(rlt_rocm_ppo_train_epoch(device.handle, &agent, &parameters, dataset.observations._data, dataset.all_observations_privileged._data, dataset.actions._data,
                                                          dataset.action_log_probs._data, dataset.advantages._data, dataset.target_values._data, (int)DATASET::DATA_DIM, row_indices, (int)N_BATCHES,
                                                          critic_losses), "train");
        }
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
