// SAC's updates on sequence batches (SEQUENCE_LENGTH > 1) with sequential networks of dense and GRU layers on devices::ROCM:
// train_critic / train_actor / update_critic_targets (rl/algorithms/sac/operations_generic.h:243-337, 395-468, 486-527) as one call each of the
// library's entry points for sequence batches (rlt_rocm_sac_sequence_train_critic, _train_actor, _update_critic_targets). The networks are the
// recurrent approximators of rl/algorithms/sac/loop/core/approximators_gru.h: dense -> GRU(s) -> dense(s), the actor's followed by sample_and_squash.
//
// What the entry points need beyond what the reference's objects hold is taken from the device's scratch memory for the duration of a call: the
// kept intermediates of the actor and of the target critics on the `next` views (one step longer than the networks' own buffers when the batch
// includes the first step in its targets; the target critics, of Forward capability, keep none at all), and the library's workspace.
// Agents these overloads cannot describe take the reference's generic functions over the layer overloads of this backend.
#pragma once
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_rocm.h>
#include <type_traits>
#include <cstring>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::algorithms::sac::rocm{
        template <typename T> struct IsDenseLayer: std::false_type{};
        template <typename S> struct IsDenseLayer<nn::layers::dense::LayerForward<S>>: std::true_type{};
        template <typename S> struct IsDenseLayer<nn::layers::dense::LayerBackward<S>>: std::true_type{};
        template <typename S> struct IsDenseLayer<nn::layers::dense::LayerGradient<S>>: std::true_type{};
        template <typename T> struct IsGruLayer: std::false_type{};
        template <typename S> struct IsGruLayer<nn::layers::gru::LayerForward<S>>: std::true_type{};
        template <typename S> struct IsGruLayer<nn::layers::gru::LayerBackward<S>>: std::true_type{};
        template <typename S> struct IsGruLayer<nn::layers::gru::LayerGradient<S>>: std::true_type{};
        template <typename T> struct IsSasLayer: std::false_type{};
        template <typename S> struct IsSasLayer<nn::layers::sample_and_squash::LayerForward<S>>: std::true_type{};
        template <typename S> struct IsSasLayer<nn::layers::sample_and_squash::LayerBackward<S>>: std::true_type{};
        template <typename S> struct IsSasLayer<nn::layers::sample_and_squash::LayerGradient<S>>: std::true_type{};
        // dense and GRU layers, the actor's closed by a sample_and_squash layer
        template <typename MODULE, bool ACTOR>
        constexpr bool sequence_layers_ok(){
            using C = typename MODULE::CONTENT;
            if constexpr(is_final_module<MODULE>){ return ACTOR ? IsSasLayer<C>::value : (IsDenseLayer<C>::value || IsGruLayer<C>::value); }
            else{ return (IsDenseLayer<C>::value || IsGruLayer<C>::value) && sequence_layers_ok<typename MODULE::NEXT_MODULE, ACTOR>(); }
        }
        template <typename MODEL, bool ACTOR, typename = void> struct is_sequence_model: std::false_type{};
        template <typename MODEL, bool ACTOR> struct is_sequence_model<MODEL, ACTOR, std::void_t<typename MODEL::CONTENT, typename MODEL::NEXT_MODULE>>: std::integral_constant<bool, sequence_layers_ok<MODEL, ACTOR>()>{};
        template <typename SPEC, typename BATCH_SPEC>
        constexpr bool sequence_describable(){
            using P = typename SPEC::PARAMETERS;
            if constexpr(BATCH_SPEC::SEQUENCE_LENGTHH > 1 && P::SEQUENCE_LENGTH == BATCH_SPEC::SEQUENCE_LENGTHH){
                return is_sequence_model<typename SPEC::ACTOR_NETWORK_TYPE, true>::value && is_sequence_model<typename SPEC::CRITIC_NETWORK_TYPE, false>::value
                    && is_sequence_model<typename SPEC::CRITIC_TARGET_NETWORK_TYPE, false>::value && utils::typing::is_same_v<typename SPEC::TYPE_POLICY::DEFAULT, float>
                    && P::ENTROPY_BONUS && P::ENTROPY_BONUS_NEXT_STEP && P::ADAPTIVE_ALPHA && !P::IGNORE_TERMINATION && P::MASK_NON_TERMINAL && !BATCH_SPEC::SPEC::PARAMETERS::ASYMMETRIC_OBSERVATIONS;
            }
            else{ return false; }
        }
        // the layers of one network as the library's entry points take them
        struct SequenceModel{
            rlt_seq_layer layers[RLT_SEQ_MAX_LAYERS] = {};
            int n = 0;
            bool too_deep = false;
        };
        inline rlt_seq_layer* next_layer(SequenceModel& m){
            if(m.n >= RLT_SEQ_MAX_LAYERS){ m.too_deep = true; return nullptr; }
            return &m.layers[m.n++];
        }
        template <typename S> void describe_layer(nn::layers::dense::LayerGradient<S>& layer, SequenceModel& m){ if(auto* l = next_layer(m)){ l->kind = 0; l->dense = nn::layers::dense::rocm::describe(layer); } }
        template <typename S> void describe_layer(const nn::layers::dense::LayerForward<S>& layer, SequenceModel& m){ if(auto* l = next_layer(m)){ l->kind = 0; l->dense = nn::layers::dense::rocm::describe_forward(layer); } }
        template <typename S> void describe_layer(nn::layers::gru::LayerGradient<S>& layer, SequenceModel& m){ if(auto* l = next_layer(m)){ l->kind = 1; l->gru = nn::layers::gru::rocm::describe(layer); } }
        template <typename S> void describe_layer(const nn::layers::gru::LayerForward<S>& layer, SequenceModel& m){ if(auto* l = next_layer(m)){ l->kind = 1; l->gru = nn::layers::gru::rocm::describe_forward(layer); } }
        template <typename S> void describe_layer(const nn::layers::sample_and_squash::LayerForward<S>&, SequenceModel&){}      // the head lives in the agent, not in the layer list
        template <typename MODULE>
        void describe_model(MODULE& module, SequenceModel& m){
            describe_layer(module.content, m);
            if constexpr(!is_final_module<MODULE>){ describe_model(module.next_module, m); }
        }
        inline size_t align256(size_t bytes){ return (bytes + 255) / 256 * 256; }
        // bytes of kept intermediates for `rows` rows of every layer (dense: pre_activations, output; GRU: post_activation, n_pre_pre_activation, output)
        inline size_t intermediates_bytes(const SequenceModel& m, size_t rows){
            size_t bytes = 0;
            for(int l = 0; l < m.n; l++){
                if(m.layers[l].kind == 0){ bytes += 2 * align256(rows * m.layers[l].dense.out_dim * sizeof(float)); }
                else{ const size_t H = m.layers[l].gru.hidden_dim; bytes += align256(rows * 3 * H * sizeof(float)) + 2 * align256(rows * H * sizeof(float)); }
            }
            return bytes;
        }
        inline char* attach_intermediates(SequenceModel& m, size_t rows, char* memory){
            for(int l = 0; l < m.n; l++){
                if(m.layers[l].kind == 0){
                    const size_t bytes = align256(rows * m.layers[l].dense.out_dim * sizeof(float));
                    m.layers[l].dense.pre_activations = (float*)memory; memory += bytes;
                    m.layers[l].dense.output = (float*)memory; memory += bytes;
                }
                else{
                    const size_t H = m.layers[l].gru.hidden_dim;
                    m.layers[l].gru.post_activation = (float*)memory; memory += align256(rows * 3 * H * sizeof(float));
                    m.layers[l].gru.n_pre_pre_activation = (float*)memory; memory += align256(rows * H * sizeof(float));
                    m.layers[l].gru.output = (float*)memory; memory += align256(rows * H * sizeof(float));
                }
            }
            return memory;
        }
        // everything of the agent that the updates need; the descriptors and tensor lists live in this object for the duration of the call
        template <typename DEVICE, typename SPEC>
        struct SequenceDescription{
            rlt_sac_sequence_agent agent = {};
            SequenceModel actor, critics[2], targets[2];
            std::vector<rlt_adam_tensor> actor_tensors, critic_tensors[2];
            SequenceDescription(DEVICE& device, rl::algorithms::sac::ActorCritic<SPEC>& ac){
                using P = typename SPEC::PARAMETERS;
                auto& sas = get_last_layer(ac.actor);
                using SAS_P = typename utils::typing::remove_reference_t<decltype(sas)>::SPEC::PARAMETERS;
                agent.observation_dim = get_last(typename SPEC::ACTOR_NETWORK_TYPE::INPUT_SHAPE{});
                agent.action_dim = SPEC::ENVIRONMENT::ACTION_DIM;
                agent.gamma = P::GAMMA; agent.polyak = P::CRITIC_POLYAK;
                agent.sas.log_std_lower_bound = SAS_P::LOG_STD_LOWER_BOUND; agent.sas.log_std_upper_bound = SAS_P::LOG_STD_UPPER_BOUND;
                agent.sas.log_probability_epsilon = SAS_P::LOG_PROBABILITY_EPSILON; agent.sas.target_entropy = SAS_P::TARGET_ENTROPY;
                describe_model(ac.actor, actor);
                agent.actor = actor.layers; agent.n_actor_layers = actor.n;
                bool too_deep = actor.too_deep;
                for(int k = 0; k < 2; k++){
                    describe_model(ac.critics[k], critics[k]); describe_model(ac.critics_target[k], targets[k]);
                    too_deep = too_deep || critics[k].too_deep || targets[k].too_deep;
                    agent.critics[k] = critics[k].layers; agent.critics_target[k] = targets[k].layers;
                    critic_tensors[k] = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::CRITIC_OPTIMIZER::SPEC>(device, ac.critics[k], false);
                    agent.critic_adam_tensors[k] = critic_tensors[k].data(); agent.critic_age[k] = (uint32_t*)ac.critic_optimizers[k].age._data;
                }
                utils::assert_exit(device, !too_deep, "SAC on sequence batches: a network has more layers than the library's sequence entry points take");
                agent.n_critic_layers = critics[0].n;
                agent.n_critic_adam_tensors = (int32_t)critic_tensors[0].size();
                actor_tensors = nn::optimizers::adam::rocm::collect<DEVICE, typename SPEC::ACTOR_OPTIMIZER::SPEC>(device, ac.actor, false);
                agent.actor_adam_tensors = actor_tensors.data(); agent.n_actor_adam_tensors = (int32_t)actor_tensors.size();
                agent.log_alpha = nn::optimizers::adam::rocm::describe(sas.log_alpha);
                agent.actor_age = (uint32_t*)ac.actor_optimizer.age._data; agent.alpha_age = (uint32_t*)ac.alpha_optimizer.age._data;
                agent.actor_adam = adam_parameters(ac.actor_optimizer); agent.critic_adam = adam_parameters(ac.critic_optimizers[0]); agent.alpha_adam = adam_parameters(ac.alpha_optimizer);
                agent.actor_pre_squashing = sas.pre_squashing._data; agent.actor_log_probabilities = sas.log_probabilities._data; agent.actor_actions = sas.output._data;
            }
            template <typename BATCH_SPEC>
            void set_batch(rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch){
                rlt_sequence_batch& b = agent.batch;
                b.observations_actions_base = batch.observations_actions_base._data; b.rewards = batch.rewards._data; b.terminated = (uint8_t*)batch.terminated._data;
                b.reset = (uint8_t*)batch.reset._data; b.next_reset_base = (uint8_t*)batch.next_reset_base._data; b.final_step_mask = (uint8_t*)batch.final_step_mask._data;
                b.next_final_step_mask_base = (uint8_t*)batch.next_final_step_mask_base._data; b.batch = BATCH_SPEC::BATCH_SIZE; b.sequence_length = BATCH_SPEC::SEQUENCE_LENGTHH;
                agent.include_first_step_in_targets = BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? 1 : 0;
            }
        };
    }
    // train_critic            rl/algorithms/sac/operations_generic.h:243-337 on a sequence batch
    template <typename DEV_SPEC, typename SPEC, typename CRITIC_TYPE, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename CRITIC_BUFFERS, typename CRITIC_TARGET_BUFFERS, typename TRAINING_BUFFER_SPEC, typename ACTION_NOISE_SPEC, typename RNG,
              std::enable_if_t<rl::algorithms::sac::rocm::sequence_describable<SPEC, BATCH_SPEC>(), int> = 0>
    void train_critic(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic, CRITIC_TYPE& critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_target_buffers, CRITIC_BUFFERS& critic_buffers, CRITIC_TARGET_BUFFERS& critic_target_buffers, rl::algorithms::sac::CriticTrainingBuffers<TRAINING_BUFFER_SPEC>& training_buffers, Matrix<ACTION_NOISE_SPEC>& action_noise, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        namespace rocm = rl::algorithms::sac::rocm;
        constexpr size_t S = BATCH_SPEC::SEQUENCE_LENGTHH, B = BATCH_SPEC::BATCH_SIZE, ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
        constexpr size_t T = S + (BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? 1 : 0);
        static_assert(ACTION_NOISE_SPEC::ROWS == T * B && ACTION_NOISE_SPEC::COLS == ACTION_DIM && ACTION_NOISE_SPEC::COL_PITCH == 1 && ACTION_NOISE_SPEC::ROW_PITCH == ACTION_DIM, "one row of noise per evaluated `next` step, back to back");
        rocm::SequenceDescription<DEVICE, SPEC> d(device, actor_critic);
        d.set_batch(batch);
        rlt_sac_sequence_agent& a = d.agent;
        a.critic_adam = rocm::adam_parameters(optimizer);
        a.next_state_action_value_input = training_buffers.next_state_action_value_input._data;
        a.next_q[0] = training_buffers.next_state_action_value_critic_1._data; a.next_q[1] = training_buffers.next_state_action_value_critic_2._data;
        a.next_log_probabilities = training_buffers.next_action_log_probs._data;
        a.target_action_value = training_buffers.target_action_value._data;
        a.d_output = training_buffers.d_output._data;
        // on the `next` views the actor and the target critics run over T steps: their kept intermediates go to scratch memory
        const size_t intermediates = rocm::intermediates_bytes(d.actor, T * B) + rocm::intermediates_bytes(d.targets[0], T * B) + rocm::intermediates_bytes(d.targets[1], T * B);
        // the workspace's size depends on the networks' widths and the batch only, not on the pointers that are still to be carved out of the same block
        const size_t workspace_bytes = rlt_rocm_sac_sequence_workspace_bytes(&a);
        char* memory = (char*)devices::rocm::scratch(device, intermediates + workspace_bytes + 256);
        memory = rocm::attach_intermediates(d.actor, T * B, memory);
        memory = rocm::attach_intermediates(d.targets[0], T * B, memory);
        memory = rocm::attach_intermediates(d.targets[1], T * B, memory);
        a.workspace = memory; a.workspace_bytes = workspace_bytes;
        const int critic_index = &critic == &actor_critic.critics[1] ? 1 : 0;
        devices::rocm::check(rlt_rocm_sac_sequence_train_critic(device.handle, &a, critic_index, action_noise._data), "train_critic (sequences)");
    }
    namespace rl::algorithms::sac::rocm{
        // train_critic for critic 0 and then for critic 1 on one batch and one set of noise, the loop's SHARED_BATCH case (rl/algorithms/sac/loop/core/operations_generic.h:127-138),
        // as one call of the library: the second train_critic would repeat the actor's pass over the next steps, its sample, both target critics and the target values on
        // unchanged inputs; the library computes them once and runs the two critics' passes side by side. Same bits as the two calls. The training buffers of critic 0
        // receive what both calls would write there except d_output, which holds critic 1's loss gradient (critic 0's stays in the library's workspace).
        // false: the two optimisers differ in their parameters; the caller makes the two calls.
        template <typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename OPTIMIZER, typename TRAINING_BUFFER_SPEC, typename ACTION_NOISE_SPEC>
        bool train_critics(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER (&optimizers)[2],
                           rl::algorithms::sac::CriticTrainingBuffers<TRAINING_BUFFER_SPEC>& training_buffers, Matrix<ACTION_NOISE_SPEC>& action_noise){
            using DEVICE = devices::ROCM<DEV_SPEC>;
            constexpr size_t S = BATCH_SPEC::SEQUENCE_LENGTHH, B = BATCH_SPEC::BATCH_SIZE, ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
            constexpr size_t T = S + (BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? 1 : 0);
            static_assert(ACTION_NOISE_SPEC::ROWS == T * B && ACTION_NOISE_SPEC::COLS == ACTION_DIM && ACTION_NOISE_SPEC::COL_PITCH == 1 && ACTION_NOISE_SPEC::ROW_PITCH == ACTION_DIM, "one row of noise per evaluated `next` step, back to back");
            const rlt_adam_parameters first = adam_parameters(optimizers[0]), second = adam_parameters(optimizers[1]);
            if(std::memcmp(&first, &second, sizeof(first)) != 0){ return false; }
            SequenceDescription<DEVICE, SPEC> d(device, actor_critic);
            d.set_batch(batch);
            rlt_sac_sequence_agent& a = d.agent;
            a.critic_adam = first;
            a.next_state_action_value_input = training_buffers.next_state_action_value_input._data;
            a.next_q[0] = training_buffers.next_state_action_value_critic_1._data; a.next_q[1] = training_buffers.next_state_action_value_critic_2._data;
            a.next_log_probabilities = training_buffers.next_action_log_probs._data;
            a.target_action_value = training_buffers.target_action_value._data;
            a.d_output = training_buffers.d_output._data;
            const size_t intermediates = intermediates_bytes(d.actor, T * B) + intermediates_bytes(d.targets[0], T * B) + intermediates_bytes(d.targets[1], T * B);
            const size_t workspace_bytes = rlt_rocm_sac_sequence_workspace_bytes(&a);
            char* memory = (char*)devices::rocm::scratch(device, intermediates + workspace_bytes + 256);
            memory = attach_intermediates(d.actor, T * B, memory);
            memory = attach_intermediates(d.targets[0], T * B, memory);
            memory = attach_intermediates(d.targets[1], T * B, memory);
            a.workspace = memory; a.workspace_bytes = workspace_bytes;
            devices::rocm::check(rlt_rocm_sac_sequence_train_critics(device.handle, &a, action_noise._data), "train_critic x 2 (sequences)");
            return true;
        }
    }
    // train_actor             rl/algorithms/sac/operations_generic.h:395-468 on a sequence batch
    template <typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename OPTIMIZER, typename ACTOR_BUFFERS, typename CRITIC_BUFFERS, typename TRAINING_BUFFERS_SPEC, typename ACTION_NOISE_SPEC, typename RNG,
              std::enable_if_t<rl::algorithms::sac::rocm::sequence_describable<SPEC, BATCH_SPEC>(), int> = 0>
    void train_actor(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, OPTIMIZER& optimizer, ACTOR_BUFFERS& actor_buffers, CRITIC_BUFFERS& critic_buffers, rl::algorithms::sac::ActorTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers, Matrix<ACTION_NOISE_SPEC>& action_noise, RNG& rng){
        using DEVICE = devices::ROCM<DEV_SPEC>;
        namespace rocm = rl::algorithms::sac::rocm;
        constexpr size_t S = BATCH_SPEC::SEQUENCE_LENGTHH, B = BATCH_SPEC::BATCH_SIZE, ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
        static_assert(ACTION_NOISE_SPEC::ROWS == S * B && ACTION_NOISE_SPEC::COLS == ACTION_DIM && ACTION_NOISE_SPEC::COL_PITCH == 1 && ACTION_NOISE_SPEC::ROW_PITCH == ACTION_DIM, "one row of noise per step, back to back");
        rocm::SequenceDescription<DEVICE, SPEC> d(device, actor_critic);
        d.set_batch(batch);
        rlt_sac_sequence_agent& a = d.agent;
        a.actor_adam = rocm::adam_parameters(optimizer);
        a.state_action_value_input = training_buffers.state_action_value_input._data;
        a.d_output = training_buffers.d_output._data;
        a.d_critic_input[0] = training_buffers.d_critic_1_input._data; a.d_critic_input[1] = training_buffers.d_critic_2_input._data;
        a.d_actor_output_squashing = training_buffers.d_actor_output_squashing._data; a.d_actor_output = training_buffers.d_actor_output._data;
        const size_t workspace_bytes = rlt_rocm_sac_sequence_workspace_bytes(&a);      // the target critics take no part here: their descriptions stay without intermediates
        a.workspace = devices::rocm::scratch(device, workspace_bytes + 256); a.workspace_bytes = workspace_bytes;
        devices::rocm::check(rlt_rocm_sac_sequence_train_actor(device.handle, &a, action_noise._data), "train_actor (sequences)");
    }
    // update_critic_targets   rl/algorithms/sac/operations_generic.h:486-527 for critics of dense and GRU layers: every tensor of both target critics in one launch
    template <typename DEV_SPEC, typename SPEC, std::enable_if_t<rl::algorithms::sac::rocm::is_sequence_model<typename SPEC::CRITIC_NETWORK_TYPE, false>::value && rl::algorithms::sac::rocm::is_sequence_model<typename SPEC::CRITIC_TARGET_NETWORK_TYPE, false>::value, int> = 0>
    void update_critic_targets(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic){
        namespace rocm = rl::algorithms::sac::rocm;
        constexpr int MAX = 2 * 5 * RLT_SEQ_MAX_LAYERS;
        const float* sources[MAX]; float* targets[MAX]; uint32_t counts[MAX];
        int n = 0;
        for(int k = 0; k < 2; k++){
            rocm::SequenceModel source, target;
            rocm::describe_model(actor_critic.critics[k], source); rocm::describe_model(actor_critic.critics_target[k], target);
            utils::assert_exit(device, !source.too_deep && source.n == target.n, "update_critic_targets: a network has more layers than the library's sequence entry points take");
            auto pair = [&](const float* s, float* t, size_t count){ sources[n] = s; targets[n] = t; counts[n++] = (uint32_t)count; };
            for(int l = 0; l < source.n; l++){
                const rlt_seq_layer& s = source.layers[l]; const rlt_seq_layer& t = target.layers[l];
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
        devices::rocm::check(rlt_rocm_polyak_update_list(device.handle, sources, targets, counts, n, (float)SPEC::PARAMETERS::CRITIC_POLYAK), "update_critic_targets (sequences)");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
