// SAC's element-wise steps on devices::ROCM: target_action_values, min_value_d_output, mask_actions, mask_gradient (the counterpart of
// rl/algorithms/sac/operations_cuda.h:9-128). train_critic / train_actor / update_critic_targets are the reference's generic functions
// (rl/algorithms/sac/operations_generic.h:243-337,395-468,524-527): with these overloads and those of the layers, the optimiser and
// the containers every call they make resolves to this backend.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/algorithms/sac/sac.h>
#include <rl_tools/rl/components/off_policy_runner/off_policy_runner.h>
#include <rl_tools/nn/layers/dense/operations_rocm.h>
#include <rl_tools/nn/optimizers/adam/operations_rocm.h>
#include <type_traits>
#include <utility>
#include <vector>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    // train_critic / train_actor / update_critic_targets as calls of the library's own SAC entry points (rlt_rocm_sac_train_critic, ...), which run an
    // update as two launches for 3-layer networks of hidden width 64 and as one launch per operation otherwise. These overloads take part only for
    // agents they can describe: single-step batches, actor = MLP followed by sample_and_squash, critics = MLPs, fp32, the reference's default
    // entropy handling. Any other agent goes through the reference's generic functions and the leaf overloads of this backend.
    namespace rl::algorithms::sac::rocm{
        template <typename T, typename = void> struct is_mlp: std::false_type{};
        template <typename T> struct is_mlp<T, std::void_t<decltype(T::NUM_HIDDEN_LAYERS), decltype(std::declval<T&>().input_layer), decltype(std::declval<T&>().hidden_layers), decltype(std::declval<T&>().output_layer)>>: std::true_type{};
        template <typename T, typename = void> struct is_sample_and_squash: std::false_type{};
        template <typename T> struct is_sample_and_squash<T, std::void_t<decltype(std::declval<T&>().log_alpha), decltype(std::declval<T&>().pre_squashing), decltype(std::declval<T&>().log_probabilities)>>: std::true_type{};
        template <typename MODULE> constexpr bool is_final_module = utils::typing::is_same_v<typename MODULE::NEXT_MODULE, nn_models::sequential::OutputModule>;
        template <typename MODEL, typename = void> struct is_mlp_model: std::false_type{};        // a sequential model that is one MLP
        template <typename MODEL> struct is_mlp_model<MODEL, std::void_t<typename MODEL::CONTENT, typename MODEL::NEXT_MODULE>>: std::integral_constant<bool, is_mlp<typename MODEL::CONTENT>::value && is_final_module<MODEL>>{};
        template <typename MODEL, typename = void> struct is_mlp_sas_model: std::false_type{};    // an MLP followed by sample_and_squash
        template <typename MODEL> struct is_mlp_sas_model<MODEL, std::void_t<typename MODEL::CONTENT, typename MODEL::NEXT_MODULE::CONTENT>>:
            std::integral_constant<bool, is_mlp<typename MODEL::CONTENT>::value && is_sample_and_squash<typename MODEL::NEXT_MODULE::CONTENT>::value && is_final_module<typename MODEL::NEXT_MODULE>>{};
        template <typename SPEC, typename BATCH_SPEC>
        constexpr bool describable(){
            using P = typename SPEC::PARAMETERS;
            return BATCH_SPEC::SEQUENCE_LENGTHH == 1 && P::SEQUENCE_LENGTH == 1 && is_mlp_sas_model<typename SPEC::ACTOR_NETWORK_TYPE>::value && is_mlp_model<typename SPEC::CRITIC_NETWORK_TYPE>::value
                && is_mlp_model<typename SPEC::CRITIC_TARGET_NETWORK_TYPE>::value && utils::typing::is_same_v<typename SPEC::TYPE_POLICY::DEFAULT, float>
                && P::ENTROPY_BONUS && P::ENTROPY_BONUS_NEXT_STEP && P::ADAPTIVE_ALPHA && !P::IGNORE_TERMINATION && P::MASK_NON_TERMINAL && !BATCH_SPEC::SPEC::PARAMETERS::ASYMMETRIC_OBSERVATIONS;
        }
        constexpr int MAX_LAYERS = 16;
        template <typename MLP>
        int describe_mlp(MLP& mlp, rlt_dense_layer* out){
            static_assert(MLP::NUM_HIDDEN_LAYERS + 2 <= MAX_LAYERS);
            int n = 0;
            out[n++] = nn::layers::dense::rocm::describe(mlp.input_layer);
            for(int i = 0; i < (int)MLP::NUM_HIDDEN_LAYERS; i++){ out[n++] = nn::layers::dense::rocm::describe(mlp.hidden_layers[i]); }
            out[n++] = nn::layers::dense::rocm::describe(mlp.output_layer);
            return n;
        }
        template <typename OPTIMIZER>
        rlt_adam_parameters adam_parameters(const OPTIMIZER& optimizer){
            using OSPEC = typename OPTIMIZER::SPEC;
            using DEFAULTS = typename OSPEC::DEFAULT_PARAMETERS;
            const auto& hp = optimizer.parameters._data[0];
            rlt_adam_parameters p = {};
            p.alpha = hp.alpha; p.beta_1 = hp.beta_1; p.beta_2 = hp.beta_2; p.epsilon = hp.epsilon; p.epsilon_sqrt = hp.epsilon_sqrt;
            p.weight_decay = hp.weight_decay; p.bias_lr_factor = hp.bias_lr_factor;
            p.enable_weight_decay = OSPEC::ENABLE_WEIGHT_DECAY; p.enable_bias_lr_factor = OSPEC::ENABLE_BIAS_LR_FACTOR;
            p.enable_gradient_clipping = DEFAULTS::ENABLE_GRADIENT_CLIPPING; p.gradient_clip_value = DEFAULTS::GRADIENT_CLIP_VALUE;
            return p;
        }
        // everything of the agent that both updates need; the descriptor arrays and tensor lists live in this object for the duration of the call
        template <typename DEVICE, typename SPEC>
        struct Description{
            rlt_sac_agent agent = {};
            rlt_dense_layer actor[MAX_LAYERS], critics[2][MAX_LAYERS], targets[2][MAX_LAYERS];
            std::vector<rlt_adam_tensor> actor_tensors, critic_tensors[2];
            Description(DEVICE& device, rl::algorithms::sac::ActorCritic<SPEC>& ac){
                using P = typename SPEC::PARAMETERS;
                auto& sas = ac.actor.next_module.content;
                using SAS_P = typename utils::typing::remove_reference_t<decltype(sas)>::SPEC::PARAMETERS;
                agent.observation_dim = get_last(typename SPEC::ACTOR_NETWORK_TYPE::INPUT_SHAPE{});
                agent.action_dim = SPEC::ENVIRONMENT::ACTION_DIM;
                agent.gamma = P::GAMMA; agent.polyak = P::CRITIC_POLYAK;
                agent.sas.log_std_lower_bound = SAS_P::LOG_STD_LOWER_BOUND; agent.sas.log_std_upper_bound = SAS_P::LOG_STD_UPPER_BOUND;
                agent.sas.log_probability_epsilon = SAS_P::LOG_PROBABILITY_EPSILON; agent.sas.target_entropy = SAS_P::TARGET_ENTROPY;
                agent.n_actor_layers = describe_mlp(ac.actor.content, actor); agent.actor = actor;
                for(int k = 0; k < 2; k++){
                    agent.n_critic_layers = describe_mlp(ac.critics[k].content, critics[k]); agent.critics[k] = critics[k];
                    describe_mlp(ac.critics_target[k].content, targets[k]); agent.critics_target[k] = targets[k];
                    critic_tensors[k] = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::CRITIC_OPTIMIZER::SPEC>(device, ac.critics[k].content, false);
                    agent.critic_adam_tensors[k] = critic_tensors[k].data(); agent.critic_age[k] = (uint32_t*)ac.critic_optimizers[k].age._data;
                }
                agent.n_critic_adam_tensors = (int32_t)critic_tensors[0].size();
                actor_tensors = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::ACTOR_OPTIMIZER::SPEC>(device, ac.actor.content, false);
                agent.actor_adam_tensors = actor_tensors.data(); agent.n_actor_adam_tensors = (int32_t)actor_tensors.size();
                agent.log_alpha = nn::optimizers::adam::rocm::describe(sas.log_alpha);
                agent.actor_age = (uint32_t*)ac.actor_optimizer.age._data; agent.alpha_age = (uint32_t*)ac.alpha_optimizer.age._data;
                agent.actor_adam = adam_parameters(ac.actor_optimizer); agent.critic_adam = adam_parameters(ac.critic_optimizers[0]); agent.alpha_adam = adam_parameters(ac.alpha_optimizer);
                agent.actor_pre_squashing = sas.pre_squashing._data; agent.actor_log_probabilities = sas.log_probabilities._data; agent.actor_actions = sas.output._data;
            }
            template <typename BATCH_SPEC>
            void set_batch(DEVICE& device, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch){
                agent.batch = BATCH_SPEC::BATCH_SIZE;
                agent.observations_actions_base = batch.observations_actions_base._data;
                agent.rewards = batch.rewards._data; agent.terminated = (uint8_t*)batch.terminated._data;
                // single-step batches: every step is final and starts an episode for the purposes of the update (all three masks all true), which NULL states
                size_t bytes = rlt_rocm_mlp_workspace_bytes(agent.actor, agent.n_actor_layers, agent.batch), critic_bytes = rlt_rocm_mlp_workspace_bytes(agent.critics[0], agent.n_critic_layers, agent.batch);
                bytes = (bytes > critic_bytes ? bytes : critic_bytes) + (size_t)agent.batch * 2 * agent.action_dim * sizeof(float) + 1024;
                agent.workspace = devices::rocm::scratch(device, bytes); agent.workspace_bytes = bytes;
            }
        };
    }
    // train_critic            rl/algorithms/sac/operations_generic.h:243-337
    template <typename DEV_SPEC, typename SPEC, typename CRITIC_TYPE, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename CRITIC_BUFFERS, typename CRITIC_TARGET_BUFFERS, typename TRAINING_BUFFER_SPEC, typename ACTION_NOISE_SPEC, typename RNG,
              typename = utils::typing::enable_if_t<rl::algorithms::sac::rocm::describable<SPEC, BATCH_SPEC>()>>
    void train_critic(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic, CRITIC_TYPE& critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_target_buffers, CRITIC_BUFFERS& critic_buffers, CRITIC_TARGET_BUFFERS& critic_target_buffers, rl::algorithms::sac::CriticTrainingBuffers<TRAINING_BUFFER_SPEC>& training_buffers, Matrix<ACTION_NOISE_SPEC>& action_noise, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        constexpr int BATCH_SIZE = BATCH_SPEC::BATCH_SIZE, ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM, D = decltype(batch.observations_actions_base)::SPEC::SHAPE::template GET<2>;
        constexpr int TARGET_OFFSET = BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? BATCH_SIZE : 0;       // the targets of the single step are the values of the `next` rows
        static_assert(ACTION_NOISE_SPEC::COL_PITCH == 1 && ACTION_NOISE_SPEC::ROW_PITCH == ACTION_DIM, "the noise rows lie back to back");
        rl::algorithms::sac::rocm::Description<DEVICE, SPEC> d(device, actor_critic);
        d.set_batch(device, batch);
        const int critic_index = &critic == &actor_critic.critics[1] ? 1 : 0;
        d.agent.critic_adam = rl::algorithms::sac::rocm::adam_parameters(optimizer);
        d.agent.next_state_action_value_input = training_buffers.next_state_action_value_input._data + (size_t)TARGET_OFFSET * D;
        d.agent.next_q[0] = training_buffers.next_state_action_value_critic_1._data + TARGET_OFFSET; d.agent.next_q[1] = training_buffers.next_state_action_value_critic_2._data + TARGET_OFFSET;
        d.agent.next_log_probabilities = training_buffers.next_action_log_probs._data + TARGET_OFFSET;
        d.agent.target_action_value = training_buffers.target_action_value._data;
        d.agent.d_output_critic[0] = d.agent.d_output_critic[1] = training_buffers.d_output._data;
        devices::rocm::check(rlt_rocm_sac_train_critic(device.handle, &d.agent, critic_index, action_noise._data + (size_t)TARGET_OFFSET * ACTION_DIM), "train_critic");
    }
    // train_actor             rl/algorithms/sac/operations_generic.h:395-468
    template <typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename CRITIC_BUFFERS, typename TRAINING_BUFFERS_SPEC, typename ACTION_NOISE_SPEC, typename RNG,
              typename = utils::typing::enable_if_t<rl::algorithms::sac::rocm::describable<SPEC, BATCH_SPEC>()>>
    void train_actor(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_buffers, CRITIC_BUFFERS& critic_buffers, rl::algorithms::sac::ActorTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers, Matrix<ACTION_NOISE_SPEC>& action_noise, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        constexpr int ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
        static_assert(ACTION_NOISE_SPEC::COL_PITCH == 1 && ACTION_NOISE_SPEC::ROW_PITCH == ACTION_DIM, "the noise rows lie back to back");
        rl::algorithms::sac::rocm::Description<DEVICE, SPEC> d(device, actor_critic);
        d.set_batch(device, batch);
        d.agent.actor_adam = rl::algorithms::sac::rocm::adam_parameters(optimizer);
        d.agent.state_action_value_input = training_buffers.state_action_value_input._data;
        d.agent.d_output_actor_critics = training_buffers.d_output._data;
        d.agent.d_critic_input[0] = training_buffers.d_critic_1_input._data; d.agent.d_critic_input[1] = training_buffers.d_critic_2_input._data;
        d.agent.d_actor_output_squashing = training_buffers.d_actor_output_squashing._data; d.agent.d_actor_output = training_buffers.d_actor_output._data;
        devices::rocm::check(rlt_rocm_sac_train_actor(device.handle, &d.agent, action_noise._data), "train_actor");
    }
    // update_critic_targets   rl/algorithms/sac/operations_generic.h:524-527: every tensor of both target critics in one launch
    template <typename DEV_SPEC, typename SPEC, typename = utils::typing::enable_if_t<rl::algorithms::sac::rocm::is_mlp_model<typename SPEC::CRITIC_NETWORK_TYPE>::value && rl::algorithms::sac::rocm::is_mlp_model<typename SPEC::CRITIC_TARGET_NETWORK_TYPE>::value>>
    void update_critic_targets(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic){
        constexpr int MAX = rl::algorithms::sac::rocm::MAX_LAYERS;
        rlt_dense_layer source[MAX], target[MAX];
        const float* sources[4 * MAX]; float* targets[4 * MAX]; uint32_t counts[4 * MAX];
        int n = 0;
        for(int k = 0; k < 2; k++){
            const int layers = rl::algorithms::sac::rocm::describe_mlp(actor_critic.critics[k].content, source);
            rl::algorithms::sac::rocm::describe_mlp(actor_critic.critics_target[k].content, target);
            for(int l = 0; l < layers; l++){
                sources[n] = source[l].weights; targets[n] = target[l].weights; counts[n++] = (uint32_t)source[l].in_dim * source[l].out_dim;
                sources[n] = source[l].biases; targets[n] = target[l].biases; counts[n++] = (uint32_t)source[l].out_dim;
            }
        }
        devices::rocm::check(rlt_rocm_polyak_update_list(device.handle, sources, targets, counts, n, (float)SPEC::PARAMETERS::CRITIC_POLYAK), "update_critic_targets");
    }
    // target_action_values    sac/operations_cuda.h:10-43: y = r + gamma * (1 - terminated) * (min(Q1', Q2') - alpha * log pi(a'|s'))
    template <typename DEV_SPEC, typename BATCH_SPEC, typename TRAINING_BUFFER_SPEC, typename NEXT_ACTION_LOG_PROBS_SPEC, typename LOG_ALPHA_PARAMETER>
    void target_action_values(devices::ROCM<DEV_SPEC>& device, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, rl::algorithms::sac::CriticTrainingBuffers<TRAINING_BUFFER_SPEC>& training_buffers, const Matrix<NEXT_ACTION_LOG_PROBS_SPEC>& next_action_log_probs, LOG_ALPHA_PARAMETER& log_alpha){
        using SPEC = typename TRAINING_BUFFER_SPEC::SPEC;
        using BUFFERS = rl::algorithms::sac::CriticTrainingBuffers<TRAINING_BUFFER_SPEC>;
        constexpr auto BATCH_SIZE = BATCH_SPEC::BATCH_SIZE;
        constexpr auto SEQUENCE_LENGTH = BATCH_SPEC::SEQUENCE_LENGTHH;
        static_assert(BATCH_SIZE == BUFFERS::BATCH_SIZE);
        static_assert(SPEC::PARAMETERS::ENTROPY_BONUS && SPEC::PARAMETERS::ENTROPY_BONUS_NEXT_STEP, "the ROCM kernel adds the entropy bonus of the next step inside the discounted term");
        static_assert(NEXT_ACTION_LOG_PROBS_SPEC::COL_PITCH == 1);
        constexpr auto TARGET_OFFSET = BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? BATCH_SIZE : 0;      // the target of step t takes the target critics' value at t + 1 ...
        devices::rocm::check(rlt_rocm_sac_target_action_values(device.handle, training_buffers.next_state_action_value_critic_1._data + TARGET_OFFSET, training_buffers.next_state_action_value_critic_2._data + TARGET_OFFSET,
                                                               batch.rewards._data, (const uint8_t*)batch.terminated._data, next_action_log_probs._data /* ... and the log-probability at index t */, log_alpha.parameters._data,
                                                               (float)SPEC::PARAMETERS::GAMMA, SPEC::PARAMETERS::IGNORE_TERMINATION ? 1 : 0, training_buffers.target_action_value._data, SEQUENCE_LENGTH * BATCH_SIZE), "target_action_values");
    }
    // min_value_d_output      sac/operations_cuda.h:45-72: per sample, the action columns of the input gradient of the critic with the smaller value
    template <typename DEV_SPEC, typename SPEC, typename TRAINING_BUFFERS_SPEC>
    void min_value_d_output(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic, rl::algorithms::sac::ActorTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers){
        using BUFFERS = rl::algorithms::sac::ActorTrainingBuffers<TRAINING_BUFFERS_SPEC>;
        constexpr int ROWS = BUFFERS::BATCH_SIZE * SPEC::PARAMETERS::SEQUENCE_LENGTH;
        constexpr int CRITIC_INPUT_DIM = get_last(typename SPEC::CRITIC_NETWORK_TYPE::INPUT_SHAPE{});
        constexpr int ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
        auto critic_1_output = output(device, actor_critic.critics[0]);
        auto critic_2_output = output(device, actor_critic.critics[1]);
        devices::rocm::check(rlt_rocm_sac_min_value_d_output(device.handle, critic_1_output._data, critic_2_output._data, training_buffers.d_critic_1_input._data, training_buffers.d_critic_2_input._data,
                                                             CRITIC_INPUT_DIM, CRITIC_INPUT_DIM, ACTION_DIM, training_buffers.d_actor_output_squashing._data, ACTION_DIM, ROWS), "min_value_d_output");
    }
    // mask_actions            sac/operations_cuda.h:73-99: rows of `source` replace rows of `target` where the mask (or its inverse) is set
    template <typename DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC, typename MASK_SPEC>
    void mask_actions(devices::ROCM<DEV_SPEC>& device, Tensor<SOURCE_SPEC>& source, Tensor<TARGET_SPEC>& target, Tensor<MASK_SPEC>& mask, bool invert_mask = false){
        static_assert(SOURCE_SPEC::SHAPE::LENGTH == 3 && tensor::same_dimensions<SOURCE_SPEC, TARGET_SPEC>());
        static_assert(tensor::dense_row_major_layout<MASK_SPEC>() && sizeof(typename MASK_SPEC::T) == 1);
        constexpr int ROWS = SOURCE_SPEC::SHAPE::template GET<0> * SOURCE_SPEC::SHAPE::template GET<1>, COLS = SOURCE_SPEC::SHAPE::template GET<2>;
        static_assert(SOURCE_SPEC::STRIDE::template GET<2> == 1 && TARGET_SPEC::STRIDE::template GET<2> == 1);
        static_assert(SOURCE_SPEC::STRIDE::template GET<0> == SOURCE_SPEC::STRIDE::template GET<1> * SOURCE_SPEC::SHAPE::template GET<1> && TARGET_SPEC::STRIDE::template GET<0> == TARGET_SPEC::STRIDE::template GET<1> * TARGET_SPEC::SHAPE::template GET<1>,
                      "sequence steps follow each other with the row stride");
        devices::rocm::check(rlt_rocm_mask_copy(device.handle, source._data, SOURCE_SPEC::STRIDE::template GET<1>, target._data, TARGET_SPEC::STRIDE::template GET<1>, (const uint8_t*)mask._data, invert_mask ? 1 : 0, ROWS, COLS), "mask_actions");
    }
    // mask_gradient           sac/operations_cuda.h:100-128: rows are zeroed where the mask (or its inverse) is set
    template <typename DEV_SPEC, typename SOURCE_SPEC, typename MASK_SPEC>
    void mask_gradient(devices::ROCM<DEV_SPEC>& device, Tensor<SOURCE_SPEC>& source, Tensor<MASK_SPEC>& mask, bool invert_mask = false){
        static_assert(SOURCE_SPEC::SHAPE::LENGTH == 3);
        static_assert(tensor::dense_row_major_layout<MASK_SPEC>() && sizeof(typename MASK_SPEC::T) == 1);
        constexpr int ROWS = SOURCE_SPEC::SHAPE::template GET<0> * SOURCE_SPEC::SHAPE::template GET<1>, COLS = SOURCE_SPEC::SHAPE::template GET<2>;
        static_assert(SOURCE_SPEC::STRIDE::template GET<2> == 1 && SOURCE_SPEC::STRIDE::template GET<0> == SOURCE_SPEC::STRIDE::template GET<1> * SOURCE_SPEC::SHAPE::template GET<1>);
        devices::rocm::check(rlt_rocm_mask_zero(device.handle, source._data, SOURCE_SPEC::STRIDE::template GET<1>, (const uint8_t*)mask._data, invert_mask ? 1 : 0, ROWS, COLS), "mask_gradient");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
#include <rl_tools/rl/algorithms/sac/operations_rocm_sequence.h>      // the same three functions for sequence batches and recurrent networks
