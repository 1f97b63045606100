// The on-policy runner on devices::ROCM: malloc / free / collect (the generic versions, rl/components/on_policy_runner/
// operations_generic.h:50-146 with operations_generic_per_env.h:8-74, are host loops over environments and steps; the CPU backend's
// operations_cpu.h:17-64 spreads the environments over threads; the reference has no CUDA version of this component).
//
// This backend ships precompiled kernels, so the runner steps the environment the C ABI's collect has a kernel for: the Pendulum
// (rl/environments/pendulum), with an actor that is a sequential model of a standardize layer followed by an MLP with a
// state-independent action standard deviation (the loop's ConfigApproximatorsSequential, rl/algorithms/ppo/loop/core/config.h:51-66).
// One call of collect is STEPS_PER_ENV + 1 launches per stage (reset and observe, the actor, sample and step) on the device; the noise
// of all steps and the initial states of all possible resets are drawn beforehand, by two launches.
//
// Memory. runner.environments and runner.env_parameters hold structs that only host code reads: host memory (containers of structs
// are host memory on this backend). runner.states is the kernels' [N_ENVIRONMENTS x 2] float array (angle, angular velocity): device
// memory; the other members are device matrices.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/components/on_policy_runner/on_policy_runner.h>
#include <rl_tools/rl/components/on_policy_runner/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/pendulum.h>
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
        using P = typename ENVIRONMENT::SPEC::PARAMETERS;
        using DATASET = rl::components::on_policy_runner::Dataset<DATASET_SPEC>;
        constexpr size_t N = SPEC::N_ENVIRONMENTS, S = DATASET_SPEC::STEPS_PER_ENV, A = ENVIRONMENT::ACTION_DIM;
        static_assert(P::initial_state_min_angle == -P::initial_state_max_angle && P::initial_state_min_speed == -P::initial_state_max_speed, "initial states are drawn from ranges that are symmetric about zero");
        static_assert(P::OBSERVATION_NOISE_POSITION == 0 && P::OBSERVATION_NOISE_VELOCITY == 0);
        static_assert(decltype(dataset.data)::SPEC::COL_PITCH == 1 && decltype(dataset.data)::SPEC::ROW_PITCH == DATASET::DATA_DIM);
        const rlt_pendulum_runner r = rl::components::on_policy_runner::rocm::pendulum(runner);
        rl::components::on_policy_runner::rocm::ActorDescription d;
        rl::components::on_policy_runner::rocm::describe(actor, d);
        utils::assert_exit(device, d.n_layers > 0 && d.log_std, "collect: the actor is not a [standardize ->] mlp_unconditional_stddev model");
        // device memory for this call: the noise of every step, the initial state of every possible reset, the library's workspace
        const size_t workspace_bytes = rlt_rocm_on_policy_collect_workspace_bytes(&r, d.layers, d.n_layers);
        const size_t noise_bytes = (S * N * A * sizeof(float) + 255) / 256 * 256, initial_bytes = (S * N * 2 * sizeof(float) + 255) / 256 * 256;
        char* memory = (char*)devices::rocm::scratch(device, noise_bytes + initial_bytes + workspace_bytes);
        float* noise = (float*)memory; float* initial = (float*)(memory + noise_bytes); void* workspace = memory + noise_bytes + initial_bytes;
        devices::rocm::check(rlt_rocm_randn_f32(device.handle, noise, S * N * A, rng.seed, random::next_stream(rng)), "collect (noise)");
        // sample_initial_state (rl/environments/pendulum/operations_generic.h:58-61): uniform in +- the largest angle and speed
        devices::rocm::check(rlt_rocm_rand_f32(device.handle, initial, S * N * 2, -1.0f, 1.0f, rng.seed, random::next_stream(rng)), "collect (initial states)");
        devices::rocm::check(rlt_rocm_unary_f32(device.handle, RLT_UNARY_SCALE, (float)P::initial_state_max_angle, initial, 2, initial, 2, (int)(S * N), 1), "collect (initial states)");
        if constexpr(P::initial_state_max_speed != 1){
            devices::rocm::check(rlt_rocm_unary_f32(device.handle, RLT_UNARY_SCALE, (float)P::initial_state_max_speed, initial + 1, 2, initial + 1, 2, (int)(S * N), 1), "collect (initial states)");
        }
        rlt_on_policy_dataset columns = {};
        columns.observations = dataset.observations._data; columns.actions_mean = dataset.actions_mean._data; columns.actions = dataset.actions._data;
        columns.action_log_probs = dataset.action_log_probs._data; columns.rewards = dataset.rewards._data; columns.terminated = dataset.terminated._data;
        columns.truncated = dataset.truncated._data; columns.all_reset = dataset.all_reset._data;
        columns.ld = (int32_t)DATASET::DATA_DIM; columns.steps_per_env = (int32_t)S;
        devices::rocm::check(rlt_rocm_on_policy_collect(device.handle, &r, &columns, d.layers, d.n_layers, d.log_std, d.standardize_mean, d.standardize_precision, noise, initial,
                                                        SPEC::TRUNCATE_ON_EACH_ITERATION ? 1 : 0, workspace, workspace_bytes), "collect");
        runner.step += SPEC::N_ENVIRONMENTS * DATASET_SPEC::STEPS_PER_ENV;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
