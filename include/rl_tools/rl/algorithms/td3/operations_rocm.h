// TD3 on devices::ROCM: target_action_noise, train_critic, train_actor, update_critic_targets, update_actor_target (the counterpart of
// rl/algorithms/td3/operations_cuda.h:8-110, which covers the element-wise steps of an older interface; the generic versions,
// rl/algorithms/td3/operations_generic.h:116-325, loop over elements on the host).
//
// The updates are calls of the library's own TD3 entry points (rlt_rocm_td3_train_critic, ...). These overloads take part only for agents
// they can describe: single-step batches, actor = MLP followed by td3_sampling, critics = MLPs, fp32, symmetric observations. The noise
// that the reference draws inside evaluate / forward of the td3_sampling layer is drawn on the device into a buffer first.
#pragma once
#include <cstring>
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/algorithms/td3/td3.h>
#include <rl_tools/rl/components/off_policy_runner/off_policy_runner.h>
#include <rl_tools/nn/layers/td3_sampling/layer.h>
#include <rl_tools/nn/layers/dense/operations_rocm.h>
#include <rl_tools/nn/optimizers/adam/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>
#include <type_traits>
#include <utility>
#include <vector>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::algorithms::td3::rocm{
        namespace sac_rocm = rl::algorithms::sac::rocm;
        template <typename T, typename = void> struct is_td3_sampling: std::false_type{};
        template <typename T> struct is_td3_sampling<T, std::void_t<decltype(T::SPEC::PARAMETERS::STD), typename T::SPEC::PARAMETERS, decltype(std::declval<T&>().pre_clip)>>: std::true_type{};
        template <typename MODEL, typename = void> struct is_mlp_td3_model: std::false_type{};    // an MLP followed by td3_sampling
        template <typename MODEL> struct is_mlp_td3_model<MODEL, std::void_t<typename MODEL::CONTENT, typename MODEL::NEXT_MODULE::CONTENT>>:
            std::integral_constant<bool, sac_rocm::is_mlp<typename MODEL::CONTENT>::value && is_td3_sampling<typename MODEL::NEXT_MODULE::CONTENT>::value && sac_rocm::is_final_module<typename MODEL::NEXT_MODULE>>{};
        template <typename SPEC, typename BATCH_SPEC>
        constexpr bool describable(){
            using P = typename SPEC::PARAMETERS;
            return BATCH_SPEC::SEQUENCE_LENGTHH == 1 && P::SEQUENCE_LENGTH == 1 && is_mlp_td3_model<typename SPEC::ACTOR_TYPE>::value && sac_rocm::is_mlp_model<typename SPEC::CRITIC_TYPE>::value
                && sac_rocm::is_mlp_model<typename SPEC::CRITIC_TARGET_TYPE>::value && utils::typing::is_same_v<typename SPEC::TYPE_POLICY::DEFAULT, float>
                && P::MASK_NON_TERMINAL && !BATCH_SPEC::SPEC::PARAMETERS::ASYMMETRIC_OBSERVATIONS && !BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS;
        }
        template <typename MLP>
        int describe_forward_mlp(MLP& mlp, rlt_dense_layer* out){
            static_assert(MLP::NUM_HIDDEN_LAYERS + 2 <= sac_rocm::MAX_LAYERS);
            int n = 0;
            out[n++] = nn::layers::dense::rocm::describe_forward(mlp.input_layer);
            for(int i = 0; i < (int)MLP::NUM_HIDDEN_LAYERS; i++){ out[n++] = nn::layers::dense::rocm::describe_forward(mlp.hidden_layers[i]); }
            out[n++] = nn::layers::dense::rocm::describe_forward(mlp.output_layer);
            return n;
        }
        // everything of the agent that the updates need; the descriptor arrays and tensor lists live in this object for the duration of the call
        template <typename DEVICE, typename SPEC>
        struct Description{
            rlt_td3_agent agent = {};
            rlt_dense_layer actor[sac_rocm::MAX_LAYERS], actor_target[sac_rocm::MAX_LAYERS], critics[2][sac_rocm::MAX_LAYERS], targets[2][sac_rocm::MAX_LAYERS];
            std::vector<rlt_adam_tensor> actor_tensors, critic_tensors[2];
            Description(DEVICE& device, rl::algorithms::td3::ActorCritic<SPEC>& ac){
                using P = typename SPEC::PARAMETERS;
                using SAMPLING = utils::typing::remove_reference_t<decltype(ac.actor.next_module.content)>;
                agent.observation_dim = get_last(typename SPEC::ACTOR_TYPE::INPUT_SHAPE{});
                agent.action_dim = SPEC::ENVIRONMENT::ACTION_DIM;
                agent.ignore_termination = P::IGNORE_TERMINATION ? 1 : 0;
                agent.gamma = ac.gamma; agent.actor_polyak = P::ACTOR_POLYAK; agent.critic_polyak = P::CRITIC_POLYAK;
                agent.sampling_std = SAMPLING::SPEC::PARAMETERS::STD;
                agent.n_actor_layers = sac_rocm::describe_mlp(ac.actor.content, actor); agent.actor = actor;
                describe_forward_mlp(ac.actor_target.content, actor_target); agent.actor_target = actor_target;
                for(int k = 0; k < 2; k++){
                    agent.n_critic_layers = sac_rocm::describe_mlp(ac.critics[k].content, critics[k]); agent.critics[k] = critics[k];
                    describe_forward_mlp(ac.critics_target[k].content, targets[k]); agent.critics_target[k] = targets[k];
                    critic_tensors[k] = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::OPTIMIZER::SPEC>(device, ac.critics[k].content, false);
                    agent.critic_adam_tensors[k] = critic_tensors[k].data(); agent.critic_age[k] = (uint32_t*)ac.critic_optimizers[k].age._data;
                }
                agent.n_critic_adam_tensors = (int32_t)critic_tensors[0].size();
                actor_tensors = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::OPTIMIZER::SPEC>(device, ac.actor.content, false);
                agent.actor_adam_tensors = actor_tensors.data(); agent.n_actor_adam_tensors = (int32_t)actor_tensors.size();
                agent.actor_age = (uint32_t*)ac.actor_optimizer.age._data;
                agent.actor_adam = sac_rocm::adam_parameters(ac.actor_optimizer); agent.critic_adam = sac_rocm::adam_parameters(ac.critic_optimizers[0]);
                agent.actor_pre_clip = ac.actor.next_module.content.pre_clip._data;
            }
            template <typename BATCH_SPEC>
            void set_batch(DEVICE& device, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, size_t extra_bytes){
                agent.batch = BATCH_SPEC::BATCH_SIZE;
                agent.observations_actions_base = batch.observations_actions_base._data;
                agent.rewards = batch.rewards._data; agent.terminated = (uint8_t*)batch.terminated._data;
                // single-step batches: every step is final for the purposes of the update (both masks all true), which NULL states
                size_t bytes = rlt_rocm_mlp_workspace_bytes(agent.actor, agent.n_actor_layers, agent.batch), critic_bytes = rlt_rocm_mlp_workspace_bytes(agent.critics[0], agent.n_critic_layers, agent.batch);
                bytes = ((bytes > critic_bytes ? bytes : critic_bytes) + (size_t)agent.batch * agent.action_dim * sizeof(float) + 1024 + 255) / 256 * 256;
                agent.workspace = devices::rocm::scratch(device, bytes + extra_bytes); agent.workspace_bytes = bytes;
            }
            float* extra(){ return (float*)((char*)agent.workspace + agent.workspace_bytes); }      // the `extra_bytes` behind the library's workspace
        };
    }
    // target_action_noise     rl/algorithms/td3/operations_generic.h:116-128, operations_cuda.h:8-44: clamp(N(0, std), -clip, clip)
    template <typename DEV_SPEC, typename SPEC, typename OUTPUT_SPEC, typename RNG>
    void target_action_noise(devices::ROCM<DEV_SPEC>& device, const rl::algorithms::td3::ActorCritic<SPEC>& actor_critic, Matrix<OUTPUT_SPEC>& target_action_noise, RNG& rng){
        static_assert(OUTPUT_SPEC::COLS == SPEC::ENVIRONMENT::ACTION_DIM && utils::typing::is_same_v<typename OUTPUT_SPEC::T, float>);
        static_assert(OUTPUT_SPEC::COL_PITCH == 1 && OUTPUT_SPEC::ROW_PITCH == OUTPUT_SPEC::COLS, "the noise rows lie back to back");
        constexpr size_t COUNT = (size_t)OUTPUT_SPEC::ROWS * OUTPUT_SPEC::COLS;
        devices::rocm::check(rlt_rocm_randn_f32(device.handle, target_action_noise._data, COUNT, rng.seed, random::next_stream(rng)), "target_action_noise");
        devices::rocm::check(rlt_rocm_td3_target_action_noise(device.handle, target_action_noise._data, (float)actor_critic.target_next_action_noise_std, (float)actor_critic.target_next_action_noise_clip,
                                                              target_action_noise._data, COUNT), "target_action_noise");
    }
    // train_critic            rl/algorithms/td3/operations_generic.h:170-235
    template <typename DEV_SPEC, typename SPEC, typename CRITIC_TYPE, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename ACTOR_TARGET_BUFFERS, typename CRITIC_BUFFERS, typename CRITIC_TARGET_BUFFERS, typename TRAINING_BUFFERS_SPEC, typename RNG,
              typename = utils::typing::enable_if_t<rl::algorithms::td3::rocm::describable<SPEC, BATCH_SPEC>()>>
    void train_critic(devices::ROCM<DEV_SPEC>& device, const rl::algorithms::td3::ActorCritic<SPEC>& actor_critic, CRITIC_TYPE& critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_buffers, ACTOR_TARGET_BUFFERS& actor_target_buffers, CRITIC_BUFFERS& critic_buffers, CRITIC_TARGET_BUFFERS& critic_target_buffers, rl::algorithms::td3::CriticTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        constexpr size_t BATCH_SIZE = BATCH_SPEC::BATCH_SIZE, ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
        auto& ac = const_cast<rl::algorithms::td3::ActorCritic<SPEC>&>(actor_critic);       // described, not modified: the critic arrives through `critic`
        rl::algorithms::td3::rocm::Description<DEVICE, SPEC> d(device, ac);
        d.set_batch(device, batch, BATCH_SIZE * ACTION_DIM * sizeof(float));
        const int critic_index = &critic == &actor_critic.critics[1] ? 1 : 0;
        d.agent.critic_adam = rl::algorithms::sac::rocm::adam_parameters(optimizer);
        d.agent.target_next_action_noise = training_buffers.target_next_action_noise._data;
        d.agent.next_state_action_value_input = training_buffers.next_state_action_value_input._data;
        d.agent.next_q[0] = training_buffers.next_state_action_value_critic_1._data; d.agent.next_q[1] = training_buffers.next_state_action_value_critic_2._data;
        d.agent.target_action_value = training_buffers.target_action_value._data;
        d.agent.d_output_critic = training_buffers.d_output._data;
        // the exploration noise of the target actor's td3_sampling layer (evaluate in the default mode samples it, nn/layers/td3_sampling/operations_generic.h:75-128)
        float* sampling_noise = d.extra();
        if(device.td3_sampling_noise_override){ devices::rocm::check(rlt_rocm_memcpy_d2d(device.handle, sampling_noise, device.td3_sampling_noise_override, BATCH_SIZE * ACTION_DIM * sizeof(float)), "train_critic (sampling noise)"); }
        else{ devices::rocm::check(rlt_rocm_randn_f32(device.handle, sampling_noise, BATCH_SIZE * ACTION_DIM, rng.seed, random::next_stream(rng)), "train_critic (sampling noise)"); }
        devices::rocm::check(rlt_rocm_td3_train_critic(device.handle, &d.agent, critic_index, sampling_noise), "train_critic");
    }
    namespace rl::algorithms::td3::rocm{
        // train_critic for critic 0 and then for critic 1 on one batch and one target noise, the loop's SHARED_BATCH case (rl/algorithms/td3/loop/core/operations_generic.h:98-112),
        // as one call of the library (one launch for hidden widths up to 256: the two updates side by side). The sampling noise of the target actor's
        // td3_sampling layer is drawn for critic 0 and then for critic 1 from the streams the two calls would take. Same bits as the two calls.
        // DRAW_TARGET_NOISE: target_action_noise into the training buffers first (the stream before the two sampling noises', as the loop step calls it), all three draws
        // made by the library inside the launch where it is one; update_targets (with DRAW_TARGET_NOISE only): update_critic_targets afterwards, in the same call.
        // false, before any stream is taken: the two optimisers differ in their parameters, or the sampling noise is given; the caller makes the separate calls.
        template <bool DRAW_TARGET_NOISE = false, typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename OPTIMIZER, typename TRAINING_BUFFERS_SPEC, typename RNG>
        bool train_critics(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER (&optimizers)[2],
                           rl::algorithms::td3::CriticTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers, RNG& rng, bool update_targets = false){
            using DEVICE = devices::ROCM<DEV_SPEC>;
            constexpr size_t BATCH_SIZE = BATCH_SPEC::BATCH_SIZE, ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM, NOISE = BATCH_SIZE * ACTION_DIM;
            const rlt_adam_parameters first = rl::algorithms::sac::rocm::adam_parameters(optimizers[0]), second = rl::algorithms::sac::rocm::adam_parameters(optimizers[1]);
            if(std::memcmp(&first, &second, sizeof(first)) != 0 || device.td3_sampling_noise_override){ return false; }
            Description<DEVICE, SPEC> d(device, actor_critic);
            d.set_batch(device, batch, 2 * NOISE * sizeof(float));
            d.agent.critic_adam = first;
            d.agent.target_next_action_noise = training_buffers.target_next_action_noise._data;
            d.agent.next_state_action_value_input = training_buffers.next_state_action_value_input._data;
            d.agent.next_q[0] = training_buffers.next_state_action_value_critic_1._data; d.agent.next_q[1] = training_buffers.next_state_action_value_critic_2._data;
            d.agent.target_action_value = training_buffers.target_action_value._data;
            d.agent.d_output_critic = training_buffers.d_output._data;
            float* sampling_noise = d.extra();
            if(DRAW_TARGET_NOISE){
                rlt_td3_critic_draws draws;
                draws.seed = rng.seed;
                draws.target_noise_stream = random::next_stream(rng);
                for(int k = 0; k < 2; k++){ draws.sampling_stream[k] = random::next_stream(rng); }
                draws.target_noise_std = (float)actor_critic.target_next_action_noise_std; draws.target_noise_clip = (float)actor_critic.target_next_action_noise_clip;
                devices::rocm::check(rlt_rocm_td3_train_critics_drawn(device.handle, &d.agent, &draws, sampling_noise, update_targets ? 1 : 0), "target_action_noise, train_critic x 2");
                return true;
            }
            for(int k = 0; k < 2; k++){
                devices::rocm::check(rlt_rocm_randn_f32(device.handle, sampling_noise + k * NOISE, NOISE, rng.seed, random::next_stream(rng)), "train_critic x 2 (sampling noise)");
            }
            devices::rocm::check(rlt_rocm_td3_train_critics(device.handle, &d.agent, sampling_noise, sampling_noise + NOISE), "train_critic x 2");
            return true;
        }
    }
    // train_actor             rl/algorithms/td3/operations_generic.h:236-281
    template <typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename CRITIC_BUFFERS, typename TRAINING_BUFFER_SPEC, typename RNG,
              typename = utils::typing::enable_if_t<rl::algorithms::td3::rocm::describable<SPEC, BATCH_SPEC>()>>
    void train_actor(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_buffers, CRITIC_BUFFERS& critic_buffers, rl::algorithms::td3::ActorTrainingBuffers<TRAINING_BUFFER_SPEC>& training_buffers, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        constexpr size_t BATCH_SIZE = BATCH_SPEC::BATCH_SIZE, ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
        static_assert(BATCH_SIZE == SPEC::PARAMETERS::ACTOR_BATCH_SIZE);
        rl::algorithms::td3::rocm::Description<DEVICE, SPEC> d(device, actor_critic);
        d.set_batch(device, batch, BATCH_SIZE * ACTION_DIM * sizeof(float));
        d.agent.actor_adam = rl::algorithms::sac::rocm::adam_parameters(optimizer);
        d.agent.state_action_value_input = training_buffers.state_action_value_input._data;
        d.agent.d_output_actor = training_buffers.d_output._data;
        d.agent.d_critic_input = training_buffers.d_critic_input._data;
        d.agent.d_actor_output = training_buffers.d_actor_output._data;
        float* sampling_noise = d.extra();
        if(device.td3_sampling_noise_override){ devices::rocm::check(rlt_rocm_memcpy_d2d(device.handle, sampling_noise, device.td3_sampling_noise_override, BATCH_SIZE * ACTION_DIM * sizeof(float)), "train_actor (sampling noise)"); }
        else{       // the draw inside the update's launch where the library has one
            devices::rocm::check(rlt_rocm_td3_train_actor_drawn(device.handle, &d.agent, rng.seed, random::next_stream(rng), sampling_noise), "train_actor");
            return;
        }
        devices::rocm::check(rlt_rocm_td3_train_actor(device.handle, &d.agent, sampling_noise), "train_actor");
    }
    // update_critic_targets / update_actor_target   rl/algorithms/td3/operations_generic.h:317-325
    namespace rl::algorithms::td3::rocm{
        template <typename SPEC>
        constexpr bool targets_describable(){
            return is_mlp_td3_model<typename SPEC::ACTOR_TYPE>::value && sac_rocm::is_mlp_model<typename SPEC::CRITIC_TYPE>::value && sac_rocm::is_mlp_model<typename SPEC::CRITIC_TARGET_TYPE>::value
                && utils::typing::is_same_v<typename SPEC::TYPE_POLICY::DEFAULT, float>;
        }
        template <typename DEVICE, typename SOURCE, typename TARGET>
        void polyak_mlp(DEVICE& device, SOURCE& source, TARGET& target, float polyak, const char* what){
            rlt_dense_layer s[sac_rocm::MAX_LAYERS], t[sac_rocm::MAX_LAYERS];
            const int n = describe_forward_mlp(source, s);
            describe_forward_mlp(target, t);
            const float* sources[2 * sac_rocm::MAX_LAYERS]; float* targets[2 * sac_rocm::MAX_LAYERS]; uint32_t counts[2 * sac_rocm::MAX_LAYERS];
            for(int l = 0; l < n; l++){
                sources[2 * l] = s[l].weights; targets[2 * l] = t[l].weights; counts[2 * l] = (uint32_t)(s[l].in_dim * s[l].out_dim);
                sources[2 * l + 1] = s[l].biases; targets[2 * l + 1] = t[l].biases; counts[2 * l + 1] = (uint32_t)s[l].out_dim;
            }
            devices::rocm::check(rlt_rocm_polyak_update_list(device.handle, sources, targets, counts, 2 * n, polyak), what);
        }
    }
    template <typename DEV_SPEC, typename SPEC, typename = utils::typing::enable_if_t<rl::algorithms::td3::rocm::targets_describable<SPEC>()>>
    void update_critic_targets(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic){
        for(int k = 0; k < 2; k++){
            rl::algorithms::td3::rocm::polyak_mlp(device, actor_critic.critics[k].content, actor_critic.critics_target[k].content, (float)SPEC::PARAMETERS::CRITIC_POLYAK, "update_critic_targets");
        }
    }
    template <typename DEV_SPEC, typename SPEC, typename = utils::typing::enable_if_t<rl::algorithms::td3::rocm::targets_describable<SPEC>()>>
    void update_actor_target(devices::ROCM<DEV_SPEC>& device, rl::algorithms::td3::ActorCritic<SPEC>& actor_critic){
        rl::algorithms::td3::rocm::polyak_mlp(device, actor_critic.actor.content, actor_critic.actor_target.content, (float)SPEC::PARAMETERS::ACTOR_POLYAK, "update_actor_target");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
#include <rl_tools/rl/algorithms/td3/operations_rocm_sequence.h>      // the same functions for sequence batches and recurrent networks
