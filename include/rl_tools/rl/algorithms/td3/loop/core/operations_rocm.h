// One step of the TD3 training loop on devices::ROCM (the reference's is rl/algorithms/td3/loop/core/operations_generic.h:78-133; it has no counterpart in the CUDA
// backend). For loops that share one batch among the updates: the generic step's operations in its order on its random streams, with the two train_critic calls as
// one call of the library that also makes target_action_noise (rlt_rocm_td3_train_critics_drawn: one launch for both critics at hidden widths up to 256,
// the smoothing noise and each critic's sampling noise drawn inside it on the streams the separate calls would have taken). Same bits as the generic step. Every other configuration resolves to the reference's generic step.
// Include after rl/algorithms/td3/loop/core/operations_generic.h.
#pragma once
#include <rl_tools/rl/algorithms/td3/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/td3/loop/core/state.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::algorithms::td3::loop::core::rocm{
        template <typename CONFIG>
        constexpr bool shared_batch_updates(){
            return CONFIG::CORE_PARAMETERS::SHARED_BATCH && rl::algorithms::td3::rocm::describable<typename CONFIG::ACTOR_CRITIC_SPEC, typename CONFIG::CRITIC_BATCH_SPEC>();
        }
    }
    template <typename DEV_SPEC, typename T_CONFIG, utils::typing::enable_if_t<rl::algorithms::td3::loop::core::rocm::shared_batch_updates<T_CONFIG>(), int> = 0>
    bool step(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::loop::core::State<T_CONFIG>& ts){
        using CORE = typename T_CONFIG::CORE_PARAMETERS;
        using TD3 = typename CORE::TD3_PARAMETERS;
        set_step(device, device.logger, ts.step);
        bool finished = false;
        if(ts.step >= CORE::N_WARMUP_STEPS){
            step<1>(device, ts.off_policy_runner, get_actor(ts), ts.actor_buffers_eval, ts.rng);
        }
        else{
            typename T_CONFIG::EXPLORATION_POLICY exploration_policy;
            typename T_CONFIG::EXPLORATION_POLICY::template Buffer<> exploration_policy_buffer;
            step<0>(device, ts.off_policy_runner, exploration_policy, exploration_policy_buffer, ts.rng);
        }
        const bool critics_due = ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % TD3::CRITIC_TRAINING_INTERVAL == 0;
        const bool critic_targets_due = ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % TD3::CRITIC_TARGET_UPDATE_INTERVAL == 0;
        const bool actor_due = ts.step >= CORE::N_WARMUP_STEPS_ACTOR && ts.step % TD3::ACTOR_TRAINING_INTERVAL == 0;
        const bool actor_target_due = ts.step >= CORE::N_WARMUP_STEPS_ACTOR && ts.step % TD3::ACTOR_TARGET_UPDATE_INTERVAL == 0;
        bool critics_done = false;
        if(critics_due || actor_due){
            gather_batch(device, ts.off_policy_runner, ts.critic_batch, ts.rng);
            // the smoothing noise, both critic updates and (when due) the targets' soft update as one call with its three draws, on the streams the separate calls take in this order
            critics_done = critics_due && rl::algorithms::td3::rocm::train_critics<true>(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.critic_optimizers, ts.critic_training_buffers, ts.rng, critic_targets_due);
            if(!critics_done){
                auto action_noise_matrix_view = matrix_view(device, ts.critic_training_buffers.target_next_action_noise);
                target_action_noise(device, ts.actor_critic, action_noise_matrix_view, ts.rng);
            }
        }
        if(critics_due && !critics_done){
            if(!rl::algorithms::td3::rocm::train_critics(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.critic_optimizers, ts.critic_training_buffers, ts.rng)){
                for(int critic_i = 0; critic_i < 2; critic_i++){
                    train_critic(device, ts.actor_critic, ts.actor_critic.critics[critic_i], ts.critic_batch, ts.actor_critic.critic_optimizers[critic_i], ts.actor_buffers[critic_i], ts.actor_target_buffers[critic_i], ts.critic_buffers[critic_i], ts.critic_target_buffers[critic_i], ts.critic_training_buffers, ts.rng);
                }
            }
        }
        if(critic_targets_due && !critics_done){
            update_critic_targets(device, ts.actor_critic);
        }
        if(actor_due){
            train_actor(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.actor_optimizer, ts.actor_buffers[0], ts.critic_buffers[0], ts.actor_training_buffers, ts.rng);
        }
        if(actor_target_due){
            update_actor_target(device, ts.actor_critic);
        }
        ts.step++;
        if(ts.step > CORE::STEP_LIMIT){
            return true;
        }
        return finished;
    }
}
// The same for recurrent agents on sequence batches (rl/algorithms/td3/operations_rocm_sequence.h): the generic step with the two train_critic calls of a shared batch as one
// rlt_rocm_td3_sequence_train_critics. Same bits as the generic step.
#include <rl_tools/rl/algorithms/td3/operations_rocm_sequence.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::algorithms::td3::loop::core::rocm{
        template <typename CONFIG>
        constexpr bool shared_sequence_updates(){
            return CONFIG::CORE_PARAMETERS::SHARED_BATCH && rl::algorithms::td3::rocm::sequence_describable<typename CONFIG::ACTOR_CRITIC_SPEC, typename CONFIG::CRITIC_BATCH_SPEC>();
        }
    }
    template <typename DEV_SPEC, typename T_CONFIG, utils::typing::enable_if_t<rl::algorithms::td3::loop::core::rocm::shared_sequence_updates<T_CONFIG>(), char> = 0>
    bool step(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::loop::core::State<T_CONFIG>& ts){
        using CORE = typename T_CONFIG::CORE_PARAMETERS;
        using TD3 = typename CORE::TD3_PARAMETERS;
        set_step(device, device.logger, ts.step);
        bool finished = false;
        if(ts.step >= CORE::N_WARMUP_STEPS){
            step<1>(device, ts.off_policy_runner, get_actor(ts), ts.actor_buffers_eval, ts.rng);
        }
        else{
            typename T_CONFIG::EXPLORATION_POLICY exploration_policy;
            typename T_CONFIG::EXPLORATION_POLICY::template Buffer<> exploration_policy_buffer;
            step<0>(device, ts.off_policy_runner, exploration_policy, exploration_policy_buffer, ts.rng);
        }
        const bool critics_due = ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % TD3::CRITIC_TRAINING_INTERVAL == 0;
        const bool actor_due = ts.step >= CORE::N_WARMUP_STEPS_ACTOR && ts.step % TD3::ACTOR_TRAINING_INTERVAL == 0;
        if(critics_due || actor_due){
            gather_batch(device, ts.off_policy_runner, ts.critic_batch, ts.rng);
            auto action_noise_matrix_view = matrix_view(device, ts.critic_training_buffers.target_next_action_noise);
            target_action_noise(device, ts.actor_critic, action_noise_matrix_view, ts.rng);
        }
        if(critics_due){
            if(!rl::algorithms::td3::rocm::train_critics_on_sequences(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.critic_optimizers, ts.critic_training_buffers)){
                for(int critic_i = 0; critic_i < 2; critic_i++){
                    train_critic(device, ts.actor_critic, ts.actor_critic.critics[critic_i], ts.critic_batch, ts.actor_critic.critic_optimizers[critic_i], ts.actor_buffers[critic_i], ts.actor_target_buffers[critic_i], ts.critic_buffers[critic_i], ts.critic_target_buffers[critic_i], ts.critic_training_buffers, ts.rng);
                }
            }
        }
        if(ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % TD3::CRITIC_TARGET_UPDATE_INTERVAL == 0){
            update_critic_targets(device, ts.actor_critic);
        }
        if(actor_due){
            train_actor(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.actor_optimizer, ts.actor_buffers[0], ts.critic_buffers[0], ts.actor_training_buffers, ts.rng);
        }
        if(ts.step >= CORE::N_WARMUP_STEPS_ACTOR && ts.step % TD3::ACTOR_TARGET_UPDATE_INTERVAL == 0){
            update_actor_target(device, ts.actor_critic);
        }
        ts.step++;
        if(ts.step > CORE::STEP_LIMIT){
            return true;
        }
        return finished;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
