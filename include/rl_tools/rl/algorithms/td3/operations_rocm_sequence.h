// TD3's updates on sequence batches (SEQUENCE_LENGTH > 1) with sequential networks of dense and GRU layers on devices::ROCM:
// train_critic / train_actor / update_critic_targets / update_actor_target (rl/algorithms/td3/operations_generic.h:170-235, 236-281, 283-325) as one call each of
// the library's entry points for sequence batches (rlt_rocm_td3_sequence_train_critic, _train_actor, _update_critic_targets, _update_actor_target). The networks
// are the recurrent approximators of rl/algorithms/td3/loop/core/approximators_gru.h:9-75 (GRU [-> GRU] [-> dense] -> dense, no sampling layer).
//
// As for SAC (rl/algorithms/sac/operations_rocm_sequence.h), what the entry points need beyond what the reference's objects hold comes from the device's scratch
// memory for the duration of a call: the kept intermediates of the target actor and the target critics on the `next` views, the observation columns of the
// batch laid out back to back for an actor whose first layer is a GRU, and the library's workspace.
#pragma once
#include <cstring>
#include <rl_tools/rl/algorithms/td3/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/operations_rocm_sequence.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::algorithms::td3::rocm{
        template <typename SPEC, typename BATCH_SPEC>
        constexpr bool sequence_describable(){
            using P = typename SPEC::PARAMETERS;
            if constexpr(BATCH_SPEC::SEQUENCE_LENGTHH > 1 && P::SEQUENCE_LENGTH == BATCH_SPEC::SEQUENCE_LENGTHH){
                return sac_rocm::is_sequence_model<typename SPEC::ACTOR_TYPE, false>::value && sac_rocm::is_sequence_model<typename SPEC::ACTOR_TARGET_TYPE, false>::value
                    && sac_rocm::is_sequence_model<typename SPEC::CRITIC_TYPE, false>::value && sac_rocm::is_sequence_model<typename SPEC::CRITIC_TARGET_TYPE, false>::value
                    && utils::typing::is_same_v<typename SPEC::TYPE_POLICY::DEFAULT, float> && P::MASK_NON_TERMINAL && !BATCH_SPEC::SPEC::PARAMETERS::ASYMMETRIC_OBSERVATIONS;
            }
            else{ return false; }
        }
        template <typename SPEC>
        constexpr bool sequence_targets_describable(){
            return sac_rocm::is_sequence_model<typename SPEC::ACTOR_TYPE, false>::value && sac_rocm::is_sequence_model<typename SPEC::ACTOR_TARGET_TYPE, false>::value
                && sac_rocm::is_sequence_model<typename SPEC::CRITIC_TYPE, false>::value && sac_rocm::is_sequence_model<typename SPEC::CRITIC_TARGET_TYPE, false>::value
                && !is_mlp_td3_model<typename SPEC::ACTOR_TYPE>::value && utils::typing::is_same_v<typename SPEC::TYPE_POLICY::DEFAULT, float>;
        }
        // everything of the agent that the updates need; the descriptors and tensor lists live in this object for the duration of the call
        template <typename DEVICE, typename SPEC>
        struct SequenceDescription{
            rlt_td3_sequence_agent agent = {};
            sac_rocm::SequenceModel actor, actor_target, critics[2], targets[2];
            std::vector<rlt_adam_tensor> actor_tensors, critic_tensors[2];
            SequenceDescription(DEVICE& device, rl::algorithms::td3::ActorCritic<SPEC>& ac){
                using P = typename SPEC::PARAMETERS;
                agent.observation_dim = get_last(typename SPEC::ACTOR_TYPE::INPUT_SHAPE{});
                agent.action_dim = SPEC::ENVIRONMENT::ACTION_DIM;
                agent.ignore_termination = P::IGNORE_TERMINATION ? 1 : 0;
                agent.gamma = ac.gamma; agent.actor_polyak = P::ACTOR_POLYAK; agent.critic_polyak = P::CRITIC_POLYAK;
                sac_rocm::describe_model(ac.actor, actor); sac_rocm::describe_model(ac.actor_target, actor_target);
                agent.actor = actor.layers; agent.actor_target = actor_target.layers; agent.n_actor_layers = actor.n;
                bool too_deep = actor.too_deep || actor_target.too_deep;
                for(int k = 0; k < 2; k++){
                    sac_rocm::describe_model(ac.critics[k], critics[k]); sac_rocm::describe_model(ac.critics_target[k], targets[k]);
                    too_deep = too_deep || critics[k].too_deep || targets[k].too_deep;
                    agent.critics[k] = critics[k].layers; agent.critics_target[k] = targets[k].layers;
                    critic_tensors[k] = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::OPTIMIZER::SPEC>(device, ac.critics[k], false);
                    agent.critic_adam_tensors[k] = critic_tensors[k].data(); agent.critic_age[k] = (uint32_t*)ac.critic_optimizers[k].age._data;
                }
                utils::assert_exit(device, !too_deep, "TD3 on sequence batches: a network has more layers than the library's sequence entry points take");
                agent.n_critic_layers = critics[0].n;
                agent.n_critic_adam_tensors = (int32_t)critic_tensors[0].size();
                actor_tensors = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::OPTIMIZER::SPEC>(device, ac.actor, false);
                agent.actor_adam_tensors = actor_tensors.data(); agent.n_actor_adam_tensors = (int32_t)actor_tensors.size();
                agent.actor_age = (uint32_t*)ac.actor_optimizer.age._data;
                agent.actor_adam = sac_rocm::adam_parameters(ac.actor_optimizer); agent.critic_adam = sac_rocm::adam_parameters(ac.critic_optimizers[0]);
            }
            template <typename BATCH_SPEC>
            void set_batch(rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch){
                rlt_sequence_batch& b = agent.batch;
                b.observations_actions_base = batch.observations_actions_base._data; b.rewards = batch.rewards._data; b.terminated = (uint8_t*)batch.terminated._data;
                b.reset = (uint8_t*)batch.reset._data; b.next_reset_base = (uint8_t*)batch.next_reset_base._data; b.final_step_mask = (uint8_t*)batch.final_step_mask._data;
                b.next_final_step_mask_base = (uint8_t*)batch.next_final_step_mask_base._data; b.batch = BATCH_SPEC::BATCH_SIZE; b.sequence_length = BATCH_SPEC::SEQUENCE_LENGTHH;
                agent.include_first_step_in_targets = BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? 1 : 0;
            }
            // scratch memory behind `head_bytes` of the caller's own: the staging buffer of the actor's input (T x B rows) and the library's workspace
            char* attach_workspace(DEVICE& device, size_t head_bytes, size_t rows){
                const size_t input_bytes = sac_rocm::align256(rows * agent.observation_dim * sizeof(float));
                const size_t workspace_bytes = rlt_rocm_td3_sequence_workspace_bytes(&agent);      // depends on the networks' widths and the batch only
                char* memory = (char*)devices::rocm::scratch(device, head_bytes + input_bytes + workspace_bytes + 256);
                agent.actor_input = (float*)(memory + head_bytes);
                agent.workspace = memory + head_bytes + input_bytes; agent.workspace_bytes = workspace_bytes;
                return memory;
            }
        };
        template <typename DEVICE>
        void polyak_sequence_models(DEVICE& device, const sac_rocm::SequenceModel* source, const sac_rocm::SequenceModel* target, int n_models, float polyak, const char* what){
            constexpr int MAX = 2 * 5 * RLT_SEQ_MAX_LAYERS;
            const float* sources[MAX]; float* targets[MAX]; uint32_t counts[MAX];
            int n = 0;
            auto pair = [&](const float* s, float* t, size_t count){ sources[n] = s; targets[n] = t; counts[n++] = (uint32_t)count; };
            for(int k = 0; k < n_models; k++){
                utils::assert_exit(device, !source[k].too_deep && source[k].n == target[k].n, what);
                for(int l = 0; l < source[k].n; l++){
                    const rlt_seq_layer& s = source[k].layers[l]; const rlt_seq_layer& t = target[k].layers[l];
                    if(s.kind == 0){
                        pair(s.dense.weights, t.dense.weights, (size_t)s.dense.in_dim * s.dense.out_dim); pair(s.dense.biases, t.dense.biases, s.dense.out_dim);
                    }
                    else{
                        const size_t H = s.gru.hidden_dim, I = s.gru.input_dim;
                        pair(s.gru.weights_input, t.gru.weights_input, 3 * H * I); pair(s.gru.biases_input, t.gru.biases_input, 3 * H);
                        pair(s.gru.weights_hidden, t.gru.weights_hidden, 3 * H * H); pair(s.gru.biases_hidden, t.gru.biases_hidden, 3 * H);
                        pair(s.gru.initial_hidden_state, t.gru.initial_hidden_state, H);
                    }
                }
            }
            devices::rocm::check(rlt_rocm_polyak_update_list(device.handle, sources, targets, counts, n, polyak), what);
        }
    }
    // train_critic            rl/algorithms/td3/operations_generic.h:170-235 on a sequence batch; training_buffers.target_next_action_noise holds the clamped noise (target_action_noise)
    template <typename DEV_SPEC, typename SPEC, typename CRITIC_TYPE, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename ACTOR_TARGET_BUFFERS, typename CRITIC_BUFFERS, typename CRITIC_TARGET_BUFFERS, typename TRAINING_BUFFERS_SPEC, typename RNG,
              std::enable_if_t<rl::algorithms::td3::rocm::sequence_describable<SPEC, BATCH_SPEC>(), int> = 0>
    void train_critic(devices::ROCM<DEV_SPEC>& device, const rl::algorithms::td3::ActorCritic<SPEC>& actor_critic, CRITIC_TYPE& critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_buffers, ACTOR_TARGET_BUFFERS& actor_target_buffers, CRITIC_BUFFERS& critic_buffers, CRITIC_TARGET_BUFFERS& critic_target_buffers, rl::algorithms::td3::CriticTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        namespace rocm = rl::algorithms::td3::rocm;
        namespace sac_rocm = rl::algorithms::sac::rocm;
        constexpr size_t S = BATCH_SPEC::SEQUENCE_LENGTHH, B = BATCH_SPEC::BATCH_SIZE;
        constexpr size_t T = S + (BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? 1 : 0);
        auto& ac = const_cast<rl::algorithms::td3::ActorCritic<SPEC>&>(actor_critic);       // described, not modified: the critic arrives through `critic`
        rocm::SequenceDescription<DEVICE, SPEC> d(device, ac);
        d.set_batch(batch);
        rlt_td3_sequence_agent& a = d.agent;
        a.critic_adam = sac_rocm::adam_parameters(optimizer);
        a.target_next_action_noise = training_buffers.target_next_action_noise._data;
        a.next_state_action_value_input = training_buffers.next_state_action_value_input._data;
        a.next_q[0] = training_buffers.next_state_action_value_critic_1._data; a.next_q[1] = training_buffers.next_state_action_value_critic_2._data;
        a.target_action_value = training_buffers.target_action_value._data;
        a.d_output = training_buffers.d_output._data;
        // on the `next` views the target actor and the target critics run over T steps: their kept intermediates go to scratch memory
        const size_t intermediates = sac_rocm::intermediates_bytes(d.actor_target, T * B) + sac_rocm::intermediates_bytes(d.targets[0], T * B) + sac_rocm::intermediates_bytes(d.targets[1], T * B);
        char* memory = d.attach_workspace(device, intermediates, T * B);
        memory = sac_rocm::attach_intermediates(d.actor_target, T * B, memory);
        memory = sac_rocm::attach_intermediates(d.targets[0], T * B, memory);
        memory = sac_rocm::attach_intermediates(d.targets[1], T * B, memory);
        const int critic_index = &critic == &actor_critic.critics[1] ? 1 : 0;
        devices::rocm::check(rlt_rocm_td3_sequence_train_critic(device.handle, &a, critic_index), "train_critic (sequences)");
    }
    namespace rl::algorithms::td3::rocm{
        // train_critic for critic 0 and then for critic 1 on one sequence batch and one target noise, the loop's SHARED_BATCH case (rl/algorithms/td3/loop/core/operations_generic.h:98-112),
        // as one call of the library: the second train_critic would repeat the target actor's pass, the noisy next actions, both target critics and the target values on
        // unchanged inputs; the library computes them once and runs the two critics' passes side by side. Same bits as the two calls; d_output holds critic 1's loss
        // gradient (critic 0's stays in the library's workspace). false: the two optimisers differ in their parameters; the caller makes the two calls.
        template <typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename OPTIMIZER, typename TRAINING_BUFFERS_SPEC>
        bool train_critics_on_sequences(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER (&optimizers)[2],
                                        rl::algorithms::td3::CriticTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers){
            using DEVICE = devices::ROCM<DEV_SPEC>;
            namespace sac_rocm = rl::algorithms::sac::rocm;
            constexpr size_t S = BATCH_SPEC::SEQUENCE_LENGTHH, B = BATCH_SPEC::BATCH_SIZE;
            constexpr size_t T = S + (BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? 1 : 0);
            const rlt_adam_parameters first = sac_rocm::adam_parameters(optimizers[0]), second = sac_rocm::adam_parameters(optimizers[1]);
            if(std::memcmp(&first, &second, sizeof(first)) != 0){ return false; }
            SequenceDescription<DEVICE, SPEC> d(device, actor_critic);
            d.set_batch(batch);
            rlt_td3_sequence_agent& a = d.agent;
            a.critic_adam = first;
            a.target_next_action_noise = training_buffers.target_next_action_noise._data;
            a.next_state_action_value_input = training_buffers.next_state_action_value_input._data;
            a.next_q[0] = training_buffers.next_state_action_value_critic_1._data; a.next_q[1] = training_buffers.next_state_action_value_critic_2._data;
            a.target_action_value = training_buffers.target_action_value._data;
            a.d_output = training_buffers.d_output._data;
            const size_t intermediates = sac_rocm::intermediates_bytes(d.actor_target, T * B) + sac_rocm::intermediates_bytes(d.targets[0], T * B) + sac_rocm::intermediates_bytes(d.targets[1], T * B);
            char* memory = d.attach_workspace(device, intermediates, T * B);
            memory = sac_rocm::attach_intermediates(d.actor_target, T * B, memory);
            memory = sac_rocm::attach_intermediates(d.targets[0], T * B, memory);
            memory = sac_rocm::attach_intermediates(d.targets[1], T * B, memory);
            devices::rocm::check(rlt_rocm_td3_sequence_train_critics(device.handle, &a), "train_critic x 2 (sequences)");
            return true;
        }
    }
    // train_actor             rl/algorithms/td3/operations_generic.h:236-281 on a sequence batch (through critic 0)
    template <typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename CRITIC_BUFFERS, typename TRAINING_BUFFER_SPEC, typename RNG,
              std::enable_if_t<rl::algorithms::td3::rocm::sequence_describable<SPEC, BATCH_SPEC>(), int> = 0>
    void train_actor(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_buffers, CRITIC_BUFFERS& critic_buffers, rl::algorithms::td3::ActorTrainingBuffers<TRAINING_BUFFER_SPEC>& training_buffers, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        namespace rocm = rl::algorithms::td3::rocm;
        constexpr size_t S = BATCH_SPEC::SEQUENCE_LENGTHH, B = BATCH_SPEC::BATCH_SIZE;
        constexpr size_t T = S + (BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? 1 : 0);
        rocm::SequenceDescription<DEVICE, SPEC> d(device, actor_critic);
        d.set_batch(batch);
        rlt_td3_sequence_agent& a = d.agent;
        a.actor_adam = rl::algorithms::sac::rocm::adam_parameters(optimizer);
        a.state_action_value_input = training_buffers.state_action_value_input._data;
        a.d_output = training_buffers.d_output._data;
        a.d_critic_input = training_buffers.d_critic_input._data;
        a.d_actor_output = training_buffers.d_actor_output._data;
        d.attach_workspace(device, 0, T * B);      // the target networks take no part here: their descriptions stay without intermediates
        devices::rocm::check(rlt_rocm_td3_sequence_train_actor(device.handle, &a), "train_actor (sequences)");
    }
    // update_critic_targets / update_actor_target   rl/algorithms/td3/operations_generic.h:283-325 for networks of dense and GRU layers: every tensor in one launch
    template <typename DEV_SPEC, typename SPEC, std::enable_if_t<rl::algorithms::td3::rocm::sequence_targets_describable<SPEC>(), int> = 0>
    void update_critic_targets(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic){
        namespace sac_rocm = rl::algorithms::sac::rocm;
        sac_rocm::SequenceModel source[2], target[2];
        for(int k = 0; k < 2; k++){ sac_rocm::describe_model(actor_critic.critics[k], source[k]); sac_rocm::describe_model(actor_critic.critics_target[k], target[k]); }
        rl::algorithms::td3::rocm::polyak_sequence_models(device, source, target, 2, (float)SPEC::PARAMETERS::CRITIC_POLYAK, "update_critic_targets (sequences)");
    }
    template <typename DEV_SPEC, typename SPEC, std::enable_if_t<rl::algorithms::td3::rocm::sequence_targets_describable<SPEC>(), int> = 0>
    void update_actor_target(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic){
        namespace sac_rocm = rl::algorithms::sac::rocm;
        sac_rocm::SequenceModel source, target;
        sac_rocm::describe_model(actor_critic.actor, source); sac_rocm::describe_model(actor_critic.actor_target, target);
        rl::algorithms::td3::rocm::polyak_sequence_models(device, &source, &target, 1, (float)SPEC::PARAMETERS::ACTOR_POLYAK, "update_actor_target (sequences)");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
