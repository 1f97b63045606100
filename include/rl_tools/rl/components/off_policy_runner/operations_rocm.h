// The off-policy runner on devices::ROCM: malloc / free / init / truncate_all / step / gather_batch (the counterpart of
// rl/components/off_policy_runner/operations_cuda.h:9-237).
//
// The CUDA backend compiles the environment's generic step into its prologue / epilogue kernels. This backend ships precompiled
// kernels, so the runner steps the environments the C ABI has a kernel for (rl/environments/operations_rocm.h: the Pendulum, the Acrobot and
// the AcrobotSwingup). On the Pendulum one step of all environments -- reset where truncated, observe, the actor (an MLP with or without a
// sample_and_squash head, or given actions), dynamics, reward, truncation and the replay add -- is ONE launch
// (rlt_rocm_pendulum_runner_step); on the others it is a prologue kernel, the actor's layers, its head, the environment's step kernel and an
// epilogue kernel (rlt_rocm_env_runner_step_sequential), as the CUDA backend launches them.
//
// Memory. runner.replay_buffers is, on every device, the block that holds the replay rings. Host code never looks inside it on a GPU
// backend; here it holds the backend's own layout: the rings of all environments in one allocation (ring e = rows [e * capacity,
// (e + 1) * capacity) of `data`, a row being [observation | action | reward | next observation | terminated | truncated] as in
// rl/components/replay_buffer/replay_buffer.h:32-62), then episode_start, then the device-resident cursors position,
// current_episode_start and full of every ring. runner.envs / env_parameters / episode_stats stay in host memory (host code reads them).
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/components/off_policy_runner/off_policy_runner.h>
#include <rl_tools/rl/components/off_policy_runner/operations_generic.h>
#include <rl_tools/rl/environments/operations_rocm.h>
#include <rl_tools/nn_models/mlp/network.h>
#include <rl_tools/nn_models/sequential/model.h>
#include <rl_tools/nn_models/random_uniform/model.h>
#include <rl_tools/nn/layers/dense/operations_rocm.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_rocm.h>
#include <rl_tools/nn/layers/td3_sampling/layer.h>
#include <rl_tools/nn/layers/standardize/layer.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::components::off_policy_runner::rocm{
        template <typename SPEC>
        struct Layout{
            using T = typename SPEC::TYPE_POLICY::DEFAULT;
            using ENVIRONMENT = typename SPEC::ENVIRONMENT;
            static_assert(utils::typing::is_same_v<T, float>, "the ROCM backend computes in fp32");
            static_assert(!SPEC::PARAMETERS::ASYMMETRIC_OBSERVATIONS, "asymmetric observations are not available on devices::ROCM");
            static constexpr size_t N = SPEC::PARAMETERS::N_ENVIRONMENTS, CAPACITY = SPEC::PARAMETERS::REPLAY_BUFFER_CAPACITY;
            static constexpr size_t OBS = ENVIRONMENT::Observation::DIM, ACT = ENVIRONMENT::ACTION_DIM, ROW = 2 * OBS + ACT + 3;
            static constexpr size_t align(size_t x){ return (x + 255) / 256 * 256; }
            static constexpr size_t DATA = 0;
            static constexpr size_t EPISODE_START = align(DATA + N * CAPACITY * ROW * sizeof(float));
            static constexpr size_t POSITION = align(EPISODE_START + N * CAPACITY * sizeof(uint32_t));
            static constexpr size_t CURRENT_EPISODE_START = POSITION + align(N * sizeof(uint32_t));
            static constexpr size_t FULL = CURRENT_EPISODE_START + align(N * sizeof(uint32_t));
            static constexpr size_t BYTES = FULL + align(N);
        };
        template <typename SPEC>
        rlt_replay_buffer replay(rl::components::OffPolicyRunner<SPEC>& runner){
            using L = Layout<SPEC>;
            char* base = (char*)runner.replay_buffers._data;
            rlt_replay_buffer rb = {};
            rb.data = (float*)(base + L::DATA); rb.episode_start = (uint32_t*)(base + L::EPISODE_START); rb.position = (uint32_t*)(base + L::POSITION);
            rb.current_episode_start = (uint32_t*)(base + L::CURRENT_EPISODE_START); rb.full = (uint8_t*)(base + L::FULL);
            rb.n_envs = (int32_t)L::N; rb.capacity = (int32_t)L::CAPACITY; rb.observation_dim = (int32_t)L::OBS; rb.action_dim = (int32_t)L::ACT;
            return rb;
        }
        template <typename SPEC>
        rlt_pendulum_runner pendulum(rl::components::OffPolicyRunner<SPEC>& runner){
            using ENVIRONMENT = typename SPEC::ENVIRONMENT;
            using T = typename SPEC::TYPE_POLICY::DEFAULT;
            using TI = typename SPEC::TI;
            static_assert(utils::typing::is_same_v<ENVIRONMENT, rl::environments::Pendulum<typename ENVIRONMENT::SPEC>>);
            static_assert(sizeof(typename ENVIRONMENT::State) == 2 * sizeof(T) && sizeof(TI) == 4 && sizeof(bool) == 1);
            rlt_pendulum_runner r = {};
            r.states = (float*)runner.states._data; r.episode_step = (uint32_t*)runner.episode_step._data; r.episode_return = (float*)runner.episode_return._data;
            r.truncated = (uint8_t*)runner.truncated._data;
            r.n_envs = SPEC::PARAMETERS::N_ENVIRONMENTS; r.episode_step_limit = SPEC::PARAMETERS::EPISODE_STEP_LIMIT;
            r.env = rl::environments::rocm::Description<ENVIRONMENT>::parameters();
            return r;
        }
        // one step of the runner through the library's entry points for any environment: head_kind 0 uniform actions in [-1, 1] (the warm-up policy),
        // 1 / 2 / 3 a sequential policy (its output is the action / sample_and_squash / td3_sampling with noise_std). Initial states, exploration noise and
        // uniform actions are drawn on the device first.
        template <typename DEV_SPEC, typename SPEC, typename RNG>
        void env_step(devices::ROCM<DEV_SPEC>& device, rl::components::OffPolicyRunner<SPEC>& runner, int head_kind, const rlt_seq_layer* layers, int n_layers,
                      const rlt_seq_state* policy_state, int auto_reset_period, const rlt_sas_parameters* sas, float noise_std, RNG& rng){
            using ENVIRONMENT = typename SPEC::ENVIRONMENT;
            using DESCRIPTION = rl::environments::rocm::Description<ENVIRONMENT>;
            static_assert(DESCRIPTION::SUPPORTED, "the ROCM backend's runner steps the environments that rl/environments/operations_rocm.h describes");
            static_assert(sizeof(typename ENVIRONMENT::State) == DESCRIPTION::STATE_DIM * sizeof(float) && sizeof(typename SPEC::TI) == 4 && sizeof(bool) == 1);
            constexpr size_t N = SPEC::PARAMETERS::N_ENVIRONMENTS, ACT = ENVIRONMENT::ACTION_DIM, STATE = DESCRIPTION::STATE_DIM;
            const rlt_replay_buffer rb = replay(runner);
            rlt_env_runner e = {};
            DESCRIPTION::set_parameters(e);
            e.n_envs = (int32_t)N; e.episode_step_limit = (int32_t)SPEC::PARAMETERS::EPISODE_STEP_LIMIT;
            e.states = (float*)runner.states._data; e.episode_step = (uint32_t*)runner.episode_step._data; e.episode_return = (float*)runner.episode_return._data;
            e.truncated = (uint8_t*)runner.truncated._data;
            e.observations = runner.buffers.observations._data; e.actions = runner.buffers.actions._data; e.next_observations = runner.buffers.next_observations._data;
            auto align = [](size_t bytes){ return (bytes + 255) / 256 * 256; };
            const size_t rewards_bytes = align(N * sizeof(float)), terminated_bytes = align(N), noise_bytes = align(N * ACT * sizeof(float)), initial_bytes = align(N * STATE * sizeof(float));
            // the workspace size depends on the runner's widths only, not on the pointers that are still to be carved out of the same block
            const size_t workspace_bytes = head_kind == 0 ? 0 : rlt_rocm_env_runner_step_sequential_workspace_bytes(&e, layers, n_layers);
            char* memory = (char*)devices::rocm::scratch(device, rewards_bytes + terminated_bytes + noise_bytes + initial_bytes + workspace_bytes);
            e.rewards = (float*)memory; e.terminated = (uint8_t*)(memory + rewards_bytes);
            float* noise = (float*)(memory + rewards_bytes + terminated_bytes); float* initial = (float*)(memory + rewards_bytes + terminated_bytes + noise_bytes);
            void* workspace = memory + rewards_bytes + terminated_bytes + noise_bytes + initial_bytes;
            if(N <= 16 && policy_state == nullptr){
                // few environments and a policy of dense layers: ONE launch that draws its own initial states and noise (the same stream numbers, taken in the
                // same order, as the draws into arrays below); the library declines (RLT_E_UNSUPPORTED) a policy it cannot hold in one workgroup
                float low[8], high[8];
                DESCRIPTION::initial_ranges(low, high);
                const uint64_t counter = rng.counter;
                const uint64_t initial_stream = random::next_stream(rng);
                const uint64_t noise_stream = head_kind == 1 ? 0 : random::next_stream(rng);
                const int rc = rlt_rocm_env_runner_step_drawn(device.handle, &e, &rb, layers, n_layers, head_kind, sas, noise_std, low, high, noise, rng.seed, noise_stream, initial_stream);
                if(rc != RLT_E_UNSUPPORTED){
                    devices::rocm::check(rc, "step(runner, one launch)");
                    return;
                }
                rng.counter = counter;
            }
            DESCRIPTION::sample_initial_states(device, initial, N, rng);
            if(head_kind == 0){
                devices::rocm::check(rlt_rocm_rand_f32(device.handle, noise, N * ACT, -1.0f, 1.0f, rng.seed, random::next_stream(rng)), "step(runner, uniform actions)");
                devices::rocm::check(rlt_rocm_env_runner_step(device.handle, &e, &rb, 0, nullptr, 0, nullptr, noise, nullptr, initial, nullptr, 0), "step(runner, uniform policy)");
            }
            else{
                if(head_kind != 1){
                    devices::rocm::check(rlt_rocm_randn_f32(device.handle, noise, N * ACT, rng.seed, random::next_stream(rng)), "step(runner, noise)");
                }
                devices::rocm::check(rlt_rocm_env_runner_step_sequential(device.handle, &e, &rb, layers, n_layers, policy_state, auto_reset_period, head_kind, sas, noise_std, noise, initial,
                                                                         workspace, workspace_bytes), "step(runner, policy)");
            }
        }
        // the dense layers of a policy in evaluation order, and whether it ends in a sample_and_squash head
        struct PolicyDescription{
            static constexpr int MAX_LAYERS = 16;
            rlt_dense_layer layers[MAX_LAYERS];
            int n_layers = 0;
            bool has_head = false;
            rlt_sas_parameters head = {};
            bool has_td3_sampling = false;      // the policy ends in a td3_sampling layer: action = clamp(output + std * noise, -1, 1)
            float td3_sampling_std = 0;
            const float* standardize_mean = nullptr;        // the policy starts with a standardize layer: its statistics [input width], on the device
            const float* standardize_precision = nullptr;
            bool standardize_misplaced = false;             // ... anywhere else: no entry point of the library runs that
        };
        template <typename LAYER_SPEC>
        void describe(const nn::layers::standardize::LayerForward<LAYER_SPEC>& layer, PolicyDescription& d){
            d.standardize_misplaced = d.standardize_misplaced || d.n_layers != 0 || d.standardize_mean != nullptr;
            d.standardize_mean = layer.mean.parameters._data; d.standardize_precision = layer.precision.parameters._data;
        }
        template <typename LAYER_SPEC>
        void describe(const nn::layers::dense::LayerForward<LAYER_SPEC>& layer, PolicyDescription& d){
            d.layers[d.n_layers++] = nn::layers::dense::rocm::describe_forward(layer);
        }
        template <typename LAYER_SPEC>
        void describe(const nn::layers::sample_and_squash::LayerForward<LAYER_SPEC>& layer, PolicyDescription& d){
            d.has_head = true;
            d.head = nn::layers::sample_and_squash::rocm::parameters<LAYER_SPEC>();
        }
        template <typename LAYER_SPEC>
        void describe(const nn::layers::td3_sampling::LayerForward<LAYER_SPEC>& layer, PolicyDescription& d){
            d.has_td3_sampling = true;
            d.td3_sampling_std = (float)LAYER_SPEC::PARAMETERS::STD;
        }
        template <typename MODEL_SPEC>
        void describe(const nn_models::mlp::NeuralNetworkForward<MODEL_SPEC>& model, PolicyDescription& d){
            static_assert(MODEL_SPEC::NUM_HIDDEN_LAYERS + 2 <= PolicyDescription::MAX_LAYERS);
            describe(model.input_layer, d);
            for(typename MODEL_SPEC::TI i = 0; i < MODEL_SPEC::NUM_HIDDEN_LAYERS; i++){ describe(model.hidden_layers[i], d); }
            describe(model.output_layer, d);
        }
        template <typename MODULE_SPEC>
        void describe(const nn_models::sequential::ModuleForward<MODULE_SPEC>& module, PolicyDescription& d){
            describe(module.content, d);
            if constexpr(!utils::typing::is_same_v<typename MODULE_SPEC::NEXT_MODULE, nn_models::sequential::OutputModule>){
                describe(module.next_module, d);
            }
        }
    }
    namespace rl::components::off_policy_runner::rocm{
        // a sequential policy with GRU layers and the state it carries between rollout steps, as the library's recurrent entry points take them
        struct RecurrentPolicyDescription{
            rlt_seq_layer layers[RLT_SEQ_MAX_LAYERS] = {};
            rlt_seq_state state = {};
            int n_layers = 0;
            bool has_gru = false, has_head = false, unsupported = false;
            rlt_sas_parameters head = {};
        };
        template <typename LAYER_SPEC, typename STATE>
        void describe_recurrent(const nn::layers::dense::LayerForward<LAYER_SPEC>& layer, STATE&, RecurrentPolicyDescription& d){
            if(d.n_layers >= RLT_SEQ_MAX_LAYERS){ d.unsupported = true; return; }
            d.layers[d.n_layers].kind = 0; d.layers[d.n_layers].dense = nn::layers::dense::rocm::describe_forward(layer);
            d.n_layers++;
        }
        template <typename LAYER_SPEC, typename STATE_SPEC>
        void describe_recurrent(const nn::layers::gru::LayerForward<LAYER_SPEC>& layer, nn::layers::gru::State<STATE_SPEC>& state, RecurrentPolicyDescription& d){
            static_assert(sizeof(typename LAYER_SPEC::TI) == 4, "the step counters of a GRU state are 32-bit on devices::ROCM");
            if(d.n_layers >= RLT_SEQ_MAX_LAYERS){ d.unsupported = true; return; }
            d.layers[d.n_layers].kind = 1; d.layers[d.n_layers].gru = nn::layers::gru::rocm::describe_forward(layer);
            d.state.hidden[d.n_layers] = state.state._data; d.state.step[d.n_layers] = (uint32_t*)state.step._data;
            d.has_gru = true;
            d.n_layers++;
        }
        template <typename LAYER_SPEC, typename STATE>
        void describe_recurrent(const nn::layers::sample_and_squash::LayerForward<LAYER_SPEC>& layer, STATE&, RecurrentPolicyDescription& d){
            d.has_head = true;
            d.head = nn::layers::sample_and_squash::rocm::parameters<LAYER_SPEC>();
        }
        template <typename MODULE_SPEC, typename CONTENT_STATE>
        void describe_recurrent(const nn_models::sequential::ModuleForward<MODULE_SPEC>& module, CONTENT_STATE& state, RecurrentPolicyDescription& d){
            describe_recurrent(module.content, state.state, d);
            if constexpr(!utils::typing::is_same_v<typename MODULE_SPEC::NEXT_MODULE, nn_models::sequential::OutputModule>){
                describe_recurrent(module.next_module, state.next_content_state, d);
            }
        }
        // whether a policy type has a GRU layer (such policies take the recurrent runner step)
        template <typename T> struct IsGru{ static constexpr bool value = false; };
        template <typename SPEC> struct IsGru<nn::layers::gru::LayerForward<SPEC>>{ static constexpr bool value = true; };
        template <typename SPEC> struct IsGru<nn::layers::gru::LayerBackward<SPEC>>{ static constexpr bool value = true; };
        template <typename SPEC> struct IsGru<nn::layers::gru::LayerGradient<SPEC>>{ static constexpr bool value = true; };
        template <typename MODULE_SPEC>
        constexpr bool module_has_gru(){
            if constexpr(IsGru<typename MODULE_SPEC::CONTENT>::value){ return true; }
            else if constexpr(utils::typing::is_same_v<typename MODULE_SPEC::NEXT_MODULE, nn_models::sequential::OutputModule>){ return false; }
            else{ return module_has_gru<typename MODULE_SPEC::NEXT_MODULE::SPEC>(); }
        }
        template <typename...> using void_t = void;
        template <typename POLICY, typename = void> struct HasGru{ static constexpr bool value = false; };
        // sequential models (nn_models::sequential::Build derives from its first module, so the module's SPEC is looked at, not the type)
        template <typename POLICY> struct HasGru<POLICY, void_t<typename POLICY::SPEC::CONTENT, typename POLICY::SPEC::NEXT_MODULE>>{ static constexpr bool value = module_has_gru<typename POLICY::SPEC>(); };
    }
    // malloc / free           off_policy_runner/operations_cuda.h:100-133
    template<typename DEV_SPEC, typename SPEC>
    void malloc(devices::ROCM<DEV_SPEC>& device, rl::components::OffPolicyRunner<SPEC>& runner){
        using RUNNER = rl::components::OffPolicyRunner<SPEC>;
        using L = rl::components::off_policy_runner::rocm::Layout<SPEC>;
        static_assert(SPEC::DYNAMIC_ALLOCATION, "runners on devices::ROCM are dynamically allocated");
        malloc(device, runner.buffers);
        void* states = nullptr;     // the kernels' [N_ENVIRONMENTS x state width] float array
        devices::rocm::check(rlt_rocm_malloc(device.handle, &states, sizeof(typename SPEC::ENVIRONMENT::State) * SPEC::PARAMETERS::N_ENVIRONMENTS), "malloc(runner)");
        runner.states._data = (typename SPEC::ENVIRONMENT::State*)states;
        malloc(device, runner.episode_return);
        malloc(device, runner.episode_step);
        malloc(device, runner.truncated);
        void* block = nullptr;
        devices::rocm::check(rlt_rocm_malloc(device.handle, &block, L::BYTES), "malloc(runner)");
        runner.replay_buffers._data = (typename RUNNER::REPLAY_BUFFER_TYPE*)block;
        count_malloc(device, L::BYTES);
        runner.envs._data = new typename SPEC::ENVIRONMENT[SPEC::PARAMETERS::N_ENVIRONMENTS];
        runner.env_parameters._data = new typename SPEC::ENVIRONMENT::Parameters[SPEC::PARAMETERS::N_ENVIRONMENTS];
        runner.episode_stats._data = nullptr;       // episode statistics are not collected on the device
        malloc(device, runner.policy_states);
    }
    template<typename DEV_SPEC, typename SPEC>
    void free(devices::ROCM<DEV_SPEC>& device, rl::components::OffPolicyRunner<SPEC>& runner){
        free(device, runner.buffers);
        devices::rocm::check(rlt_rocm_free(device.handle, (void*)runner.states._data), "free(runner)");
        runner.states._data = nullptr;
        free(device, runner.episode_return);
        free(device, runner.episode_step);
        free(device, runner.truncated);
        devices::rocm::check(rlt_rocm_free(device.handle, (void*)runner.replay_buffers._data), "free(runner)");
        runner.replay_buffers._data = nullptr;
        delete[] runner.envs._data; runner.envs._data = nullptr;
        delete[] runner.env_parameters._data; runner.env_parameters._data = nullptr;
        free(device, runner.policy_states);
    }
    // init                    off_policy_runner/operations_cuda.h:134-151: every environment starts a new episode at the next step, empty rings
    template<typename DEV_SPEC, typename SPEC>
    void init(devices::ROCM<DEV_SPEC>& device, rl::components::OffPolicyRunner<SPEC>& runner){
        using L = rl::components::off_policy_runner::rocm::Layout<SPEC>;
        truncate_all(device, runner);
        set_all(device, runner.episode_step, 0);
        set_all(device, runner.episode_return, 0);
        devices::rocm::check(rlt_rocm_fill_u8(device.handle, (uint8_t*)runner.replay_buffers._data + L::POSITION, L::BYTES - L::POSITION, 0), "init(runner)");
        for(typename SPEC::TI env_i = 0; env_i < SPEC::PARAMETERS::N_ENVIRONMENTS; env_i++){
            auto& env = runner.envs._data[env_i];
            init(device, env);
            initial_parameters(device, env, runner.env_parameters._data[env_i]);
        }
        runner.previous_policy_set = false;
        runner.previous_policy = 0;
#ifdef RL_TOOLS_DEBUG_RL_COMPONENTS_OFF_POLICY_RUNNER_CHECK_INIT
        runner.initialized = true;
#endif
    }
    // step                    off_policy_runner/operations_cuda.h:164-185 (prologue + interlude + epilogue), one launch
    template<auto POLICY_INDEX, typename DEV_SPEC, typename SPEC, typename POLICY, typename POLICY_BUFFERS, typename RNG>
    void step(devices::ROCM<DEV_SPEC>& device, rl::components::OffPolicyRunner<SPEC>& runner, POLICY& policy, POLICY_BUFFERS& policy_eval_buffers, RNG& rng){
        using TI = typename SPEC::TI;
        constexpr TI N = SPEC::PARAMETERS::N_ENVIRONMENTS;
        constexpr TI POLICY_INPUT_DIM = get_last(typename POLICY::INPUT_SHAPE{});
        constexpr TI POLICY_OUTPUT_DIM = get_last(typename POLICY::OUTPUT_SHAPE{});
        static_assert(POLICY_INPUT_DIM == SPEC::ENVIRONMENT::Observation::DIM, "The policy's input dimension must match the environment's observation dimension.");
        static_assert(POLICY_OUTPUT_DIM == SPEC::ENVIRONMENT::ACTION_DIM, "The policy's output dimension must match the environment's action dimension.");
        const bool policy_switch = runner.previous_policy_set && (POLICY_INDEX != runner.previous_policy);
        if(policy_switch){
            truncate_all(device, runner);
        }
        namespace rocm = rl::components::off_policy_runner::rocm;
        using ENVIRONMENT = typename SPEC::ENVIRONMENT;
        // the Pendulum has a runner step of its own (one launch); the other environments take the library's step for any environment
        constexpr bool PENDULUM = utils::typing::is_same_v<ENVIRONMENT, rl::environments::Pendulum<typename ENVIRONMENT::SPEC>>;
        if constexpr(utils::typing::is_same_v<POLICY, nn_models::RandomUniform<typename POLICY::SPEC>>){
            // the exploration policy of the warm-up phase: uniform actions (nn_models/random_uniform/operations_generic.h:28-44), drawn on the device
            static_assert(POLICY::SPEC::RANGE == nn_models::random_uniform::Range::MINUS_ONE_TO_ONE);
            if constexpr(PENDULUM){
                const rlt_pendulum_runner r = rocm::pendulum(runner);
                const rlt_replay_buffer rb = rocm::replay(runner);
                auto actions = to_tensor(device, runner.buffers.actions);
                rand(device, actions, rng, -1.0f, 1.0f);
                devices::rocm::check(rlt_rocm_pendulum_runner_step(device.handle, &r, &rb, 0, nullptr, 0, nullptr, runner.buffers.actions._data, nullptr, nullptr, rng.seed, random::next_stream(rng)), "step(runner, uniform policy)");
            }
            else{
                rocm::env_step(device, runner, 0, nullptr, 0, nullptr, 0, nullptr, 0.0f, rng);
            }
        }
        else if constexpr(rocm::HasGru<POLICY>::value){
            // a recurrent actor (off_policy_runner/operations_generic.h:189-206): the policy state of the environments that start an episode is reset, then one
            // evaluate_step in Rollout mode; GRU layers restart by themselves every SEQUENCE_LENGTH steps of their input shape (nn/layers/gru/operations_generic.h:406-413)
            rocm::RecurrentPolicyDescription d;
            rocm::describe_recurrent(policy, get<POLICY_INDEX>(runner.policy_states).content_state, d);
            utils::assert_exit(device, !d.unsupported, "step(runner): a recurrent policy is dense and GRU layers, optionally followed by sample_and_squash");
            constexpr int AUTO_RESET_PERIOD = (int)get<0>(typename POLICY::INPUT_SHAPE{});
            if(!d.has_head){
                // TD3's recurrent actor (rl/algorithms/td3/loop/core/approximators_gru.h:13-40) has no sampling layer: its output is the action
                rocm::env_step(device, runner, 1, d.layers, d.n_layers, &d.state, AUTO_RESET_PERIOD, nullptr, 0.0f, rng);
            }
            else if constexpr(PENDULUM){
                const rlt_pendulum_runner r = rocm::pendulum(runner);
                const rlt_replay_buffer rb = rocm::replay(runner);
                constexpr size_t ACT = ENVIRONMENT::ACTION_DIM;
                auto align = [](size_t bytes){ return (bytes + 255) / 256 * 256; };
                const size_t noise_bytes = align(N * ACT * sizeof(float)), initial_bytes = align(N * 2 * sizeof(float));
                const size_t workspace_bytes = rlt_rocm_pendulum_runner_step_recurrent_workspace_bytes(d.layers, d.n_layers, (int)N);
                char* memory = (char*)devices::rocm::scratch(device, noise_bytes + initial_bytes + workspace_bytes);
                float* noise = (float*)memory; float* initial = (float*)(memory + noise_bytes);
                devices::rocm::check(rlt_rocm_randn_f32(device.handle, noise, N * ACT, rng.seed, random::next_stream(rng)), "step(runner, noise)");
                rl::environments::rocm::Description<ENVIRONMENT>::sample_initial_states(device, initial, N, rng);
                devices::rocm::check(rlt_rocm_pendulum_runner_step_recurrent(device.handle, &r, &rb, d.layers, d.n_layers, &d.state, AUTO_RESET_PERIOD, &d.head, noise, initial,
                                                                             memory + noise_bytes + initial_bytes, workspace_bytes), "step(runner, recurrent actor)");
            }
            else{
                rocm::env_step(device, runner, 2, d.layers, d.n_layers, &d.state, AUTO_RESET_PERIOD, &d.head, 0.0f, rng);
            }
        }
        else{
            rocm::PolicyDescription d;
            rocm::describe(policy, d);
            utils::assert_exit(device, d.standardize_mean == nullptr && !d.standardize_misplaced, "step(runner): the library's off-policy runner steps have no standardize layer");
            if(d.has_td3_sampling || !PENDULUM){
                // the library's runner step for any environment and any sequential policy: reset, observe, the policy's layers, its head (TD3's exploring actor:
                // clamp(output + std * noise); SAC's: sample_and_squash; else the output is the action), dynamics, reward, replay add: a handful of launches
                rlt_seq_layer layers[rocm::PolicyDescription::MAX_LAYERS] = {};
                for(int l = 0; l < d.n_layers; l++){ layers[l].kind = 0; layers[l].dense = d.layers[l]; }
                rocm::env_step(device, runner, d.has_td3_sampling ? 3 : (d.has_head ? 2 : 1), layers, d.n_layers, nullptr, 0, &d.head, d.td3_sampling_std, rng);
            }
            else if constexpr(PENDULUM){
                const rlt_pendulum_runner r = rocm::pendulum(runner);
                const rlt_replay_buffer rb = rocm::replay(runner);
                if(d.has_head){
                    auto& noise = get_last_buffer(policy_eval_buffers).noise;
                    static_assert(utils::typing::remove_reference_t<decltype(noise)>::ROWS == N);
                    // the noise (what randn(device, noise, rng) leaves in the buffer) is drawn by the step's own launch
                    const uint64_t noise_stream = random::next_stream(rng), initial_state_stream = random::next_stream(rng);
                    devices::rocm::check(rlt_rocm_pendulum_runner_step_drawn(device.handle, &r, &rb, d.layers, d.n_layers, &d.head, noise._data, rng.seed, noise_stream, initial_state_stream), "step(runner, stochastic actor)");
                }
                else{
                    devices::rocm::check(rlt_rocm_pendulum_runner_step(device.handle, &r, &rb, 1, d.layers, d.n_layers, nullptr, nullptr, nullptr, nullptr, rng.seed, random::next_stream(rng)), "step(runner, deterministic actor)");
                }
            }
        }
        runner.previous_policy = POLICY_INDEX;
        runner.previous_policy_set = true;
    }
    // gather_batch            off_policy_runner/operations_cuda.h:152-163: draws (environment, row) pairs on the device and copies the rows
    template <typename DEV_SPEC, typename SPEC, typename BATCH_SPEC, typename RNG, bool DETERMINISTIC = false>
    void gather_batch(devices::ROCM<DEV_SPEC>& device, rl::components::OffPolicyRunner<SPEC>& runner, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, RNG& rng){
        static_assert(utils::typing::is_same_v<SPEC, typename BATCH_SPEC::SPEC>);
        constexpr int BATCH_SIZE = BATCH_SPEC::BATCH_SIZE;
        const rlt_replay_buffer rb = rl::components::off_policy_runner::rocm::replay(runner);
        if constexpr(BATCH_SPEC::SEQUENCE_LENGTHH > 1){
            // gather_batch's multi-step branch (off_policy_runner/operations_generic.h:239-430): the per-sample draws are made on the device first
            static_assert(!DETERMINISTIC, "deterministic sequence batches are not available on devices::ROCM");
            using BP = typename BATCH_SPEC::PARAMETERS;
            constexpr int S = BATCH_SPEC::SEQUENCE_LENGTHH, PADDED = S + 1;
            rlt_sequence_sampling sampling = {};
            sampling.always_sample_from_initial_state = BP::ALWAYS_SAMPLE_FROM_INITIAL_STATE; sampling.random_seq_length = BP::RANDOM_SEQ_LENGTH;
            sampling.enable_nominal_sequence_length_probability = BP::ENABLE_NOMINAL_SEQUENCE_LENGTH_PROBABILITY;
            sampling.nominal_sequence_length_probability = (float)BP::NOMINAL_SEQUENCE_LENGTH_PROBABILITY;
            sampling.include_first_step_in_targets = BP::INCLUDE_FIRST_STEP_IN_TARGETS;
            auto align = [](size_t bytes){ return (bytes + 255) / 256 * 256; };
            const size_t env_bytes = align(sizeof(uint32_t) * BATCH_SIZE), offset_bytes = align(sizeof(uint32_t) * BATCH_SIZE * PADDED), nominal_bytes = align((size_t)BATCH_SIZE * (PADDED + 1));
            const size_t length_bytes = align(sizeof(uint32_t) * BATCH_SIZE * (PADDED + 1));
            char* memory = (char*)devices::rocm::scratch(device, env_bytes + offset_bytes + nominal_bytes + length_bytes);
            uint32_t* env_indices = (uint32_t*)memory; uint32_t* offsets = (uint32_t*)(memory + env_bytes);
            uint8_t* nominal = (uint8_t*)(memory + env_bytes + offset_bytes); uint32_t* lengths = (uint32_t*)(memory + env_bytes + offset_bytes + nominal_bytes);
            devices::rocm::check(rlt_rocm_gather_sequence_draw(device.handle, &rb, &sampling, SPEC::MAX_EPISODE_LENGTH, BATCH_SIZE, S, rng.seed, random::next_stream(rng), env_indices, offsets,
                                                               nominal, lengths), "gather_batch (draw)");
            const rlt_sequence_draws draws = {env_indices, offsets, nominal, lengths};
            rlt_sequence_batch b = {};
            b.observations_actions_base = batch.observations_actions_base._data; b.rewards = batch.rewards._data; b.terminated = (uint8_t*)batch.terminated._data;
            b.reset = (uint8_t*)batch.reset._data; b.next_reset_base = (uint8_t*)batch.next_reset_base._data; b.final_step_mask = (uint8_t*)batch.final_step_mask._data;
            b.next_final_step_mask_base = (uint8_t*)batch.next_final_step_mask_base._data; b.batch = BATCH_SIZE; b.sequence_length = S;
            devices::rocm::check(rlt_rocm_gather_sequence_batch(device.handle, &rb, &sampling, &draws, SPEC::MAX_EPISODE_LENGTH, &b), "gather_batch (sequences)");
            return;
        }
        if constexpr(!DETERMINISTIC){
            // the (environment, row) pairs are drawn by the launch that copies the rows
            devices::rocm::check(rlt_rocm_gather_batch_drawn(device.handle, &rb, rng.seed, random::next_stream(rng), nullptr, nullptr, SPEC::MAX_EPISODE_LENGTH, BATCH_SIZE,
                                                             batch.observations_actions_base._data, batch.rewards._data, (uint8_t*)batch.terminated._data, (uint8_t*)batch.reset._data,
                                                             (uint8_t*)batch.next_reset_base._data, (uint8_t*)batch.final_step_mask._data, (uint8_t*)batch.next_final_step_mask_base._data), "gather_batch");
        }
        else{
            devices::rocm::check(rlt_rocm_gather_batch(device.handle, &rb, nullptr, nullptr, 1, SPEC::MAX_EPISODE_LENGTH, BATCH_SIZE,
                                                       batch.observations_actions_base._data, batch.rewards._data, (uint8_t*)batch.terminated._data, (uint8_t*)batch.reset._data,
                                                       (uint8_t*)batch.next_reset_base._data, (uint8_t*)batch.final_step_mask._data, (uint8_t*)batch.next_final_step_mask_base._data), "gather_batch");
        }
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
