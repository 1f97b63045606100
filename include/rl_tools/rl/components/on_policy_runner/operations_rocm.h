// The on-policy runner on devices::ROCM: malloc / free / collect (the generic versions, rl/components/on_policy_runner/
// operations_generic.h:50-146 with operations_generic_per_env.h:8-74, are host loops over environments and steps; the CPU backend's
// operations_cpu.h:17-64 spreads the environments over threads; the reference has no CUDA version of this component).
//
// This backend ships precompiled kernels, so the runner steps the environments the C ABI has kernels for (rl/environments/operations_rocm.h describes them:
// the Pendulum, the PendulumPosition, the Acrobot, the AcrobotSwingup, the Car), with an actor that is a sequential model of a standardize layer followed by an
// MLP with a state-independent action standard deviation (the loop's ConfigApproximatorsSequential, rl/algorithms/ppo/loop/core/config.h:51-66).
// One call of collect is STEPS_PER_ENV + 1 launches per stage (reset and observe, the actor, sample and step) on the device; the noise
// of all steps and the initial states of all possible resets are drawn beforehand, by a few launches. The Pendulum takes rlt_rocm_on_policy_collect (its step and
// the sampling share a launch), the other environments rlt_rocm_env_on_policy_collect.
//
// Memory. runner.environments and runner.env_parameters hold structs that only host code reads: host memory (containers of structs
// are host memory on this backend). runner.states is the kernels' [N_ENVIRONMENTS x 2] float array (angle, angular velocity): device
// memory; the other members are device matrices.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/components/on_policy_runner/on_policy_runner.h>
#include <rl_tools/rl/components/on_policy_runner/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/pendulum.h>
#include <rl_tools/rl/environments/operations_rocm.h>
#include <rl_tools/nn_models/mlp/network.h>
#include <rl_tools/nn_models/mlp_unconditional_stddev/network.h>
#include <rl_tools/nn_models/sequential/model.h>
#include <rl_tools/nn/layers/standardize/layer.h>
#include <rl_tools/nn/layers/dense/operations_rocm.h>
#include <rl_tools/containers/tensor/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace rl::components::on_policy_runner::rocm{
        template <typename SPEC>
        rlt_pendulum_runner pendulum(rl::components::OnPolicyRunner<SPEC>& runner){
            using ENVIRONMENT = typename SPEC::ENVIRONMENT;
            using T = typename SPEC::TYPE_POLICY::DEFAULT;
            using TI = typename SPEC::TI;
            static_assert(utils::typing::is_same_v<ENVIRONMENT, rl::environments::Pendulum<typename ENVIRONMENT::SPEC>>, "the ROCM backend's on-policy runner steps the Pendulum; other environments are collected through rlt_rocm_env_on_policy_collect");
            static_assert(utils::typing::is_same_v<T, float> && sizeof(typename ENVIRONMENT::State) == 2 * sizeof(T) && sizeof(TI) == 4 && sizeof(bool) == 1);
            static_assert(!SPEC::ASYMMETRIC_OBSERVATIONS && SPEC::N_AGENTS_PER_ENV == 1);
            using P = typename ENVIRONMENT::SPEC::PARAMETERS;
            rlt_pendulum_runner r = {};
            r.states = (float*)runner.states._data; r.episode_step = (uint32_t*)runner.episode_step._data; r.episode_return = (float*)runner.episode_return._data;
            r.truncated = (uint8_t*)runner.truncated._data;
            r.n_envs = SPEC::N_ENVIRONMENTS; r.episode_step_limit = SPEC::STEP_LIMIT;
            r.env = rlt_pendulum_parameters{(float)P::g, (float)P::max_speed, (float)P::max_torque, (float)P::dt, (float)P::m, (float)P::l};
            return r;
        }
        // an actor the library's collect and PPO update can run: [standardize ->] MLP with a state-independent log_std
        constexpr int MAX_LAYERS = 16;
        struct ActorDescription{
            rlt_dense_layer layers[MAX_LAYERS];
            int n_layers = 0;
            const float* standardize_mean = nullptr; const float* standardize_precision = nullptr;
            float* log_std = nullptr; float* d_log_std = nullptr;
        };
        template <typename LAYER> auto describe_dense(LAYER& layer, int) -> decltype(nn::layers::dense::rocm::describe(layer)){ return nn::layers::dense::rocm::describe(layer); }
        template <typename LAYER> rlt_dense_layer describe_dense(LAYER& layer, long){ return nn::layers::dense::rocm::describe_forward(layer); }
        template <typename SPEC, template <typename> typename BASE>
        void describe(nn_models::mlp_unconditional_stddev::NeuralNetworkForward<SPEC, BASE>& model, ActorDescription& d){
            static_assert(SPEC::NUM_HIDDEN_LAYERS + 2 <= MAX_LAYERS);
            d.layers[d.n_layers++] = describe_dense(model.input_layer, 0);
            for(typename SPEC::TI i = 0; i < SPEC::NUM_HIDDEN_LAYERS; i++){ d.layers[d.n_layers++] = describe_dense(model.hidden_layers[i], 0); }
            d.layers[d.n_layers++] = describe_dense(model.output_layer, 0);
            d.log_std = model.log_std.parameters._data;
            if constexpr(SPEC::CAPABILITY::TAG == nn::LayerCapability::Gradient){ d.d_log_std = model.log_std.gradient._data; }
        }
        template <typename LAYER_SPEC>
        void describe(nn::layers::standardize::LayerForward<LAYER_SPEC>& layer, ActorDescription& d){
            d.standardize_mean = layer.mean.parameters._data; d.standardize_precision = layer.precision.parameters._data;
        }
        template <typename MODULE_SPEC>
        void describe(nn_models::sequential::ModuleForward<MODULE_SPEC>& module, ActorDescription& d){
            describe(module.content, d);
            if constexpr(!utils::typing::is_same_v<typename MODULE_SPEC::NEXT_MODULE, nn_models::sequential::OutputModule>){
                describe(module.next_module, d);
            }
        }
    }
    // malloc / free           rl/components/on_policy_runner/operations_generic.h:50-69
    template <typename DEV_SPEC, typename SPEC>
    void malloc(devices::ROCM<DEV_SPEC>& device, rl::components::OnPolicyRunner<SPEC>& runner){
        using RUNNER = rl::components::OnPolicyRunner<SPEC>;
        malloc(device, runner.environments);
        malloc(device, runner.env_parameters);
        void* states = nullptr;
        devices::rocm::check(rlt_rocm_malloc(device.handle, &states, sizeof(typename SPEC::ENVIRONMENT::State) * SPEC::N_ENVIRONMENTS), "malloc(on-policy runner)");
        runner.states._data = (typename SPEC::ENVIRONMENT::State*)states;
        count_malloc(device, sizeof(typename SPEC::ENVIRONMENT::State) * SPEC::N_ENVIRONMENTS);
        malloc(device, runner.policy_state);
        malloc(device, runner.episode_step);
        malloc(device, runner.episode_return);
        malloc(device, runner.truncated);
    }
    template <typename DEV_SPEC, typename SPEC>
    void free(devices::ROCM<DEV_SPEC>& device, rl::components::OnPolicyRunner<SPEC>& runner){
        free(device, runner.environments);
        free(device, runner.env_parameters);
        devices::rocm::check(rlt_rocm_free(device.handle, (void*)runner.states._data), "free(on-policy runner)");
        runner.states._data = nullptr;
        free(device, runner.policy_state);
        free(device, runner.episode_step);
        free(device, runner.episode_return);
        free(device, runner.truncated);
    }
    // collect                 rl/components/on_policy_runner/operations_generic.h:105-146
    template <typename DEV_SPEC, typename DATASET_SPEC, typename ACTOR, typename ACTOR_BUFFER, typename RNG>
    void collect(devices::ROCM<DEV_SPEC>& device, rl::components::on_policy_runner::Dataset<DATASET_SPEC>& dataset, rl::components::OnPolicyRunner<typename DATASET_SPEC::SPEC>& runner, ACTOR& actor, ACTOR_BUFFER& policy_eval_buffers, RNG& rng){
#ifdef RL_TOOLS_DEBUG_RL_COMPONENTS_ON_POLICY_RUNNER_CHECK_INIT
        utils::assert_exit(device, runner.initialized, "rl::components::on_policy_runner::collect: runner not initialized");
#endif
        using SPEC = typename DATASET_SPEC::SPEC;
        using ENVIRONMENT = typename SPEC::ENVIRONMENT;
        using DATASET = rl::components::on_policy_runner::Dataset<DATASET_SPEC>;
        using DESCRIPTION = rl::environments::rocm::Description<ENVIRONMENT>;
        static_assert(DESCRIPTION::SUPPORTED, "the ROCM backend's on-policy runner steps the environments that rl/environments/operations_rocm.h describes");
        constexpr size_t N = SPEC::N_ENVIRONMENTS, S = DATASET_SPEC::STEPS_PER_ENV, A = ENVIRONMENT::ACTION_DIM, STATE = DESCRIPTION::STATE_DIM;
        constexpr bool PENDULUM = utils::typing::is_same_v<ENVIRONMENT, rl::environments::Pendulum<typename ENVIRONMENT::SPEC>>;
        static_assert(decltype(dataset.data)::SPEC::COL_PITCH == 1 && decltype(dataset.data)::SPEC::ROW_PITCH == DATASET::DATA_DIM);
        static_assert(sizeof(typename ENVIRONMENT::State) == STATE * sizeof(float) && sizeof(typename SPEC::TI) == 4 && sizeof(bool) == 1);
        static_assert(!SPEC::ASYMMETRIC_OBSERVATIONS && SPEC::N_AGENTS_PER_ENV == 1);
        rl::components::on_policy_runner::rocm::ActorDescription d;
        rl::components::on_policy_runner::rocm::describe(actor, d);
        utils::assert_exit(device, d.n_layers > 0 && d.log_std, "collect: the actor is not a [standardize ->] mlp_unconditional_stddev model");
        rlt_on_policy_dataset columns = {};
        columns.observations = dataset.observations._data; columns.actions_mean = dataset.actions_mean._data; columns.actions = dataset.actions._data;
        columns.action_log_probs = dataset.action_log_probs._data; columns.rewards = dataset.rewards._data; columns.terminated = dataset.terminated._data;
        columns.truncated = dataset.truncated._data; columns.all_reset = dataset.all_reset._data;
        columns.ld = (int32_t)DATASET::DATA_DIM; columns.steps_per_env = (int32_t)S;
        auto align = [](size_t bytes){ return (bytes + 255) / 256 * 256; };
        // device memory for this call: the noise of every step, the initial state of every possible reset (sample_initial_state of the environment), the library's workspace
        const size_t noise_bytes = align(S * N * A * sizeof(float)), initial_bytes = align(S * N * STATE * sizeof(float));
        if constexpr(PENDULUM){
            const rlt_pendulum_runner r = rl::components::on_policy_runner::rocm::pendulum(runner);
            const size_t workspace_bytes = rlt_rocm_on_policy_collect_workspace_bytes(&r, d.layers, d.n_layers);
            char* memory = (char*)devices::rocm::scratch(device, noise_bytes + initial_bytes + workspace_bytes);
            float* noise = (float*)memory; float* initial = (float*)(memory + noise_bytes); void* workspace = memory + noise_bytes + initial_bytes;
            devices::rocm::check(rlt_rocm_randn_f32(device.handle, noise, S * N * A, rng.seed, random::next_stream(rng)), "collect (noise)");
            DESCRIPTION::sample_initial_states(device, initial, S * N, rng);
            devices::rocm::check(rlt_rocm_on_policy_collect(device.handle, &r, &columns, d.layers, d.n_layers, d.log_std, d.standardize_mean, d.standardize_precision, noise, initial,
                                                            SPEC::TRUNCATE_ON_EACH_ITERATION ? 1 : 0, workspace, workspace_bytes), "collect");
        }
        else{
            rlt_env_runner e = {};
            DESCRIPTION::set_parameters(e);
            e.n_envs = (int32_t)N; e.episode_step_limit = (int32_t)SPEC::STEP_LIMIT;
            e.states = (float*)runner.states._data; e.episode_step = (uint32_t*)runner.episode_step._data; e.episode_return = (float*)runner.episode_return._data;
            e.truncated = (uint8_t*)runner.truncated._data;
            rlt_seq_layer layers[rl::components::on_policy_runner::rocm::MAX_LAYERS] = {};
            for(int l = 0; l < d.n_layers; l++){ layers[l].kind = 0; layers[l].dense = d.layers[l]; }
            // the per-step staging buffers of the library's runner description (observations and next observations are written into the dataset)
            constexpr size_t OBS = ENVIRONMENT::Observation::DIM;
            const size_t staging_bytes = align(N * A * sizeof(float)) + align(N * sizeof(float)) + align(N) + 2 * align(N * OBS * sizeof(float));
            const size_t workspace_bytes = rlt_rocm_env_on_policy_collect_workspace_bytes(&e, layers, d.n_layers);
            char* memory = (char*)devices::rocm::scratch(device, noise_bytes + initial_bytes + staging_bytes + workspace_bytes);
            float* noise = (float*)memory; float* initial = (float*)(memory + noise_bytes);
            char* staging = memory + noise_bytes + initial_bytes;
            e.actions = (float*)staging; staging += align(N * A * sizeof(float));
            e.rewards = (float*)staging; staging += align(N * sizeof(float));
            e.terminated = (uint8_t*)staging; staging += align(N);
            e.observations = (float*)staging; staging += align(N * OBS * sizeof(float));
            e.next_observations = (float*)staging; staging += align(N * OBS * sizeof(float));
            void* workspace = staging;
            devices::rocm::check(rlt_rocm_randn_f32(device.handle, noise, S * N * A, rng.seed, random::next_stream(rng)), "collect (noise)");
            DESCRIPTION::sample_initial_states(device, initial, S * N, rng);
            devices::rocm::check(rlt_rocm_env_on_policy_collect(device.handle, &e, &columns, layers, d.n_layers, nullptr, 0, d.log_std, d.standardize_mean, d.standardize_precision, noise, initial,
                                                                SPEC::TRUNCATE_ON_EACH_ITERATION ? 1 : 0, workspace, workspace_bytes), "collect");
        }
        runner.step += SPEC::N_ENVIRONMENTS * DATASET_SPEC::STEPS_PER_ENV;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
