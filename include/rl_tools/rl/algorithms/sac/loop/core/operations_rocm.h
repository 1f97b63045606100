// One step of the SAC training loop on devices::ROCM (the reference's is rl/algorithms/sac/loop/core/operations_generic.h:110-155; it has no
// counterpart in the CUDA backend, whose example captures the generic step's launches into graphs: src/rl/environments/pendulum/sac/cuda/sac.cu:122-164).
// Same operations in the same order on the same random streams as the generic step makes through this backend's overloads, but issued as the
// library's widest calls: the runner step draws its exploration noise itself, gather_batch draws its indices itself, both train_critic calls of
// a shared batch and update_critic_targets are one launch that also draws the critics' action noise, train_actor draws its own: four launches
// per loop step for agents the fused update kernels serve (three-layer networks of hidden width 64), against ten through the leaf overloads.
// Takes part for loops with a shared batch of single steps and an agent that rl::algorithms::sac::rocm::describable accepts; every other
// configuration resolves to the reference's generic step.
// Include after rl/algorithms/sac/loop/core/operations_generic.h.
#pragma once
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/loop/core/state.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::algorithms::sac::loop::core::rocm{
        template <typename CONFIG>
        constexpr bool one_launch_updates(){
            using BATCH_SPEC = typename CONFIG::CRITIC_BATCH_SPEC;
            return CONFIG::CORE_PARAMETERS::SHARED_BATCH && !BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS
                && rl::algorithms::sac::rocm::describable<typename CONFIG::ACTOR_CRITIC_SPEC, BATCH_SPEC>();
        }
    }
    template <typename DEV_SPEC, typename T_CONFIG, typename = utils::typing::enable_if_t<rl::algorithms::sac::loop::core::rocm::one_launch_updates<T_CONFIG>()>>
    bool step(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::loop::core::State<T_CONFIG>& ts){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        using CORE = typename T_CONFIG::CORE_PARAMETERS;
        using SAC = typename CORE::SAC_PARAMETERS;
        using AC_SPEC = typename T_CONFIG::ACTOR_CRITIC_SPEC;
        if(ts.step >= CORE::STEP_LIMIT){
            return true;
        }
        set_step(device, device.logger, ts.step);
        // one environment step per environment of the runner: the actor past the warm-up, uniform actions before
        if(ts.step < CORE::N_WARMUP_STEPS){
            typename T_CONFIG::EXPLORATION_POLICY uniform_policy;
            typename T_CONFIG::EXPLORATION_POLICY::template Buffer<> uniform_policy_buffer;
            step<0>(device, ts.off_policy_runner, uniform_policy, uniform_policy_buffer, ts.rng);
        }
        else{
            step<1>(device, ts.off_policy_runner, get_actor(ts), ts.actor_buffers_eval, ts.rng);
        }
        const bool critics_due = ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % SAC::CRITIC_TRAINING_INTERVAL == 0;
        const bool targets_due = ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % SAC::CRITIC_TARGET_UPDATE_INTERVAL == 0;
        const bool actor_due = ts.step >= CORE::N_WARMUP_STEPS_ACTOR && ts.step % SAC::ACTOR_TRAINING_INTERVAL == 0;
        if(critics_due || actor_due){
            gather_batch(device, ts.off_policy_runner, ts.critic_batch, ts.rng);
            rl::algorithms::sac::rocm::Description<DEVICE, AC_SPEC> d(device, ts.actor_critic);
            d.set_batch(device, ts.critic_batch);
            // the stream the generic step's randn(device, ts.action_noise_critic, ts.rng) would take, whether or not the critics train this step
            const uint64_t critic_noise_stream = random::next_stream(ts.rng);
            if(critics_due){
                // both critics' training buffers would receive the same values (same batch, same noise): the first one's are written
                auto& buffers = ts.critic_training_buffers[0];
                d.agent.critic_adam = rl::algorithms::sac::rocm::adam_parameters(ts.actor_critic.critic_optimizers[0]);
                d.agent.next_state_action_value_input = buffers.next_state_action_value_input._data;
                d.agent.next_q[0] = buffers.next_state_action_value_critic_1._data; d.agent.next_q[1] = buffers.next_state_action_value_critic_2._data;
                d.agent.next_log_probabilities = buffers.next_action_log_probs._data;
                d.agent.target_action_value = buffers.target_action_value._data;
                d.agent.d_output_critic[0] = buffers.d_output._data; d.agent.d_output_critic[1] = ts.critic_training_buffers[1].d_output._data;
                devices::rocm::check(rlt_rocm_sac_train_critics_drawn(device.handle, &d.agent, ts.action_noise_critic._data, ts.rng.seed, critic_noise_stream, targets_due ? 1 : 0), "step (train_critic x 2)");
            }
            else{
                constexpr size_t COUNT = decltype(ts.action_noise_critic)::SPEC::ROWS * decltype(ts.action_noise_critic)::SPEC::COLS;
                devices::rocm::check(rlt_rocm_randn_f32(device.handle, ts.action_noise_critic._data, COUNT, ts.rng.seed, critic_noise_stream), "step (critic noise)");
            }
            if(targets_due && !critics_due){
                update_critic_targets(device, ts.actor_critic);
            }
            if(actor_due){
                auto& buffers = ts.actor_training_buffers;
                d.agent.actor_adam = rl::algorithms::sac::rocm::adam_parameters(ts.actor_critic.actor_optimizer);
                d.agent.state_action_value_input = buffers.state_action_value_input._data;
                d.agent.d_output_actor_critics = buffers.d_output._data;
                d.agent.d_critic_input[0] = buffers.d_critic_1_input._data; d.agent.d_critic_input[1] = buffers.d_critic_2_input._data;
                d.agent.d_actor_output_squashing = buffers.d_actor_output_squashing._data; d.agent.d_actor_output = buffers.d_actor_output._data;
                devices::rocm::check(rlt_rocm_sac_train_actor_drawn(device.handle, &d.agent, ts.action_noise_actor._data, ts.rng.seed, random::next_stream(ts.rng)), "step (train_actor)");
            }
        }
        else if(targets_due){
            update_critic_targets(device, ts.actor_critic);
        }
        ts.step++;
        return false;
    }
    // The same loop step for recurrent agents on sequence batches (rl/algorithms/sac/operations_rocm_sequence.h) where the loop shares one batch among the updates: the
    // generic step's operations in its order on its random streams, with the two train_critic calls as one call of the library (what the second would recompute on
    // unchanged inputs is computed once, the two critics' passes run side by side). Same bits as the generic step.
    namespace rl::algorithms::sac::loop::core::rocm{
        template <typename CONFIG>
        constexpr bool shared_sequence_updates(){
            return CONFIG::CORE_PARAMETERS::SHARED_BATCH && rl::algorithms::sac::rocm::sequence_describable<typename CONFIG::ACTOR_CRITIC_SPEC, typename CONFIG::CRITIC_BATCH_SPEC>();
        }
    }
    template <typename DEV_SPEC, typename T_CONFIG, utils::typing::enable_if_t<rl::algorithms::sac::loop::core::rocm::shared_sequence_updates<T_CONFIG>(), int> = 0>
    bool step(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::loop::core::State<T_CONFIG>& ts){
        using CORE = typename T_CONFIG::CORE_PARAMETERS;
        using SAC = typename CORE::SAC_PARAMETERS;
        if(ts.step >= CORE::STEP_LIMIT){
            return true;
        }
        set_step(device, device.logger, ts.step);
        if(ts.step >= CORE::N_WARMUP_STEPS){
            step<1>(device, ts.off_policy_runner, get_actor(ts), ts.actor_buffers_eval, ts.rng);
        }
        else{
            typename T_CONFIG::EXPLORATION_POLICY exploration_policy;
            typename T_CONFIG::EXPLORATION_POLICY::template Buffer<> exploration_policy_buffer;
            step<0>(device, ts.off_policy_runner, exploration_policy, exploration_policy_buffer, ts.rng);
        }
        const bool critics_due = ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % SAC::CRITIC_TRAINING_INTERVAL == 0;
        const bool targets_due = ts.step >= CORE::N_WARMUP_STEPS_CRITIC && ts.step % SAC::CRITIC_TARGET_UPDATE_INTERVAL == 0;
        const bool actor_due = ts.step >= CORE::N_WARMUP_STEPS_ACTOR && ts.step % SAC::ACTOR_TRAINING_INTERVAL == 0;
        if(critics_due || actor_due){
            gather_batch(device, ts.off_policy_runner, ts.critic_batch, ts.rng);
            randn(device, ts.action_noise_critic, ts.rng);
        }
        if(critics_due){
            if(!rl::algorithms::sac::rocm::train_critics(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.critic_optimizers, ts.critic_training_buffers[0], ts.action_noise_critic)){
                for(int critic_i = 0; critic_i < 2; critic_i++){
                    train_critic(device, ts.actor_critic, ts.actor_critic.critics[critic_i], ts.critic_batch, ts.actor_critic.critic_optimizers[critic_i], ts.actor_target_buffers[critic_i], ts.critic_buffers[critic_i], ts.critic_target_buffers[critic_i], ts.critic_training_buffers[critic_i], ts.action_noise_critic, ts.rng);
                }
            }
        }
        if(targets_due){
            update_critic_targets(device, ts.actor_critic);
        }
        if(actor_due){
            randn(device, ts.action_noise_actor, ts.rng);
            train_actor(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.actor_optimizer, ts.actor_buffers[0], ts.critic_buffers[0], ts.actor_training_buffers, ts.action_noise_actor, ts.rng);
        }
        ts.step++;
        return false;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
