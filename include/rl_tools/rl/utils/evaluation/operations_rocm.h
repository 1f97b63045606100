// rl::utils::evaluation::evaluate on devices::ROCM (the generic version, rl/utils/evaluation/operations_generic.h:113-234, steps the
// episodes one call at a time from the host; the reference's CUDA programs copy the actor to the CPU device and evaluate there,
// src/rl/environments/pendulum/sac/cuda/sac.cu:6-27). With this overload the evaluation loop step
// (rl/loop/steps/evaluation/operations_generic.h:56-92) runs on the device: all episodes of an evaluation are one call of the library
// (rlt_rocm_pendulum_evaluate; actors 3 -> H -> H -> out with H <= 64 run every step of every episode in one launch). The other environments
// that rl/environments/operations_rocm.h describes (Acrobot, AcrobotSwingup) take rlt_rocm_env_evaluate: per step the actor's layers, its head,
// the environment's step kernel and one that keeps the episodes' returns, lengths and terminated flags.
//
// Covered: an actor that is an MLP, alone or followed by sample_and_squash (SAC: action = tanh(mean) in evaluation
// mode) or td3_sampling (TD3: the tanh output, no noise in evaluation mode), or preceded by a standardize layer (PPO: the action is the
// mean of mlp_unconditional_stddev, nn_models/mlp_unconditional_stddev/operations_generic.h:23-49), or a sequential model with GRU layers (the
// recurrent approximators of SAC and TD3: rlt_rocm_pendulum_evaluate_recurrent, about ten launches per step); no per-step data collection.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/utils/evaluation/evaluation.h>
#include <rl_tools/rl/utils/evaluation/operations_generic.h>
#include <rl_tools/rl/environments/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    template<typename DEV_SPEC, typename ENVIRONMENT, typename UI, typename POLICY, typename POLICY_STATE, typename POLICY_EVALUATION_BUFFERS, typename BUFFER_SPEC, typename DATA_SPEC, typename RNG, typename SPEC, typename MODE>
    void evaluate(devices::ROCM<DEV_SPEC>& device, ENVIRONMENT& env_init, UI& ui, const POLICY& policy, POLICY_STATE& policy_state, POLICY_EVALUATION_BUFFERS& policy_evaluation_buffers, rl::utils::evaluation::Buffer<BUFFER_SPEC>& evaluation_buffers, rl::utils::evaluation::Result<SPEC>& results, rl::utils::evaluation::NoData<DATA_SPEC>& data, RNG& rng, const Mode<MODE>& mode){
        using T = typename SPEC::T;
        using TI = typename SPEC::TI;
        using DESCRIPTION = rl::environments::rocm::Description<ENVIRONMENT>;
        static_assert(DESCRIPTION::SUPPORTED, "the ROCM backend evaluates on the environments that rl/environments/operations_rocm.h describes");
        static_assert(utils::typing::is_same_v<T, float> && sizeof(TI) == 4 && ENVIRONMENT::N_AGENTS == 1);
        static_assert(mode::is<MODE, mode::Evaluation>, "the library's evaluation runs the actor in evaluation mode (no exploration noise)");
        constexpr bool PENDULUM = utils::typing::is_same_v<ENVIRONMENT, rl::environments::Pendulum<typename ENVIRONMENT::SPEC>>;
        constexpr size_t N = SPEC::N_EPISODES, STATE = DESCRIPTION::STATE_DIM;
        constexpr bool RECURRENT = rl::components::off_policy_runner::rocm::HasGru<POLICY>::value;
        constexpr int AUTO_RESET_PERIOD = RECURRENT ? (int)get<0>(typename POLICY::INPUT_SHAPE{}) : 0;
        rl::components::off_policy_runner::rocm::PolicyDescription d;
        rl::components::off_policy_runner::rocm::RecurrentPolicyDescription rd;
        rlt_env_runner env = {};
        DESCRIPTION::set_parameters(env);
        size_t workspace_bytes = 0;
        if constexpr(RECURRENT){
            // policy_state holds N_EPISODES rows; it is reset before the first step and left as the last step left it (rl/utils/evaluation/operations_generic.h:135,163)
            rl::components::off_policy_runner::rocm::describe_recurrent(policy, policy_state.content_state, rd);
            utils::assert_exit(device, !rd.unsupported, "evaluate: a recurrent policy is dense and GRU layers, with or without a sample_and_squash head");
            workspace_bytes = PENDULUM ? rlt_rocm_pendulum_evaluate_recurrent_workspace_bytes(rd.layers, rd.n_layers, (int)N) : rlt_rocm_env_evaluate_workspace_bytes(env.env_kind, rd.layers, rd.n_layers, (int)N);
        }
        else{
            rl::components::off_policy_runner::rocm::describe(policy, d);
            utils::assert_exit(device, !d.standardize_misplaced, "evaluate: a standardize layer is supported in front of the first dense layer only");
            if constexpr(!PENDULUM){
                utils::assert_exit(device, d.n_layers <= RLT_SEQ_MAX_LAYERS, "evaluate: too many layers");
                rd.n_layers = d.n_layers; rd.has_head = d.has_head;
                for(int l = 0; l < d.n_layers && l < RLT_SEQ_MAX_LAYERS; l++){ rd.layers[l].kind = 0; rd.layers[l].dense = d.layers[l]; }
                workspace_bytes = rlt_rocm_env_evaluate_workspace_bytes(env.env_kind, rd.layers, rd.n_layers, (int)N);
            }
        }
        auto align = [](size_t bytes){ return (bytes + 255) / 256 * 256; };
        const size_t initial_bytes = align(N * STATE * sizeof(float)), returns_bytes = align(N * sizeof(float)), length_bytes = align(N * sizeof(uint32_t));
        char* memory = (char*)devices::rocm::scratch(device, initial_bytes + returns_bytes + length_bytes + 256 + workspace_bytes);
        float* initial = (float*)memory; float* returns = (float*)(memory + initial_bytes); uint32_t* episode_length = (uint32_t*)(memory + initial_bytes + returns_bytes);
        float* summary = (float*)(memory + initial_bytes + returns_bytes + length_bytes);
        void* workspace = memory + initial_bytes + returns_bytes + length_bytes + 256;
        if constexpr(SPEC::DETERMINISTIC_INITIAL_STATE){
            float host[STATE * N];
            for(size_t e = 0; e < N; e++){ DESCRIPTION::initial_state(host + STATE * e); }
            devices::rocm::check(rlt_rocm_memcpy_h2d(device.handle, initial, host, sizeof(host)), "evaluate (initial states)");
        }
        else{
            DESCRIPTION::sample_initial_states(device, initial, N, rng);
        }
        if constexpr(!PENDULUM){
            devices::rocm::check(rlt_rocm_env_evaluate(device.handle, &env, rd.has_head ? 2 : 1, rd.layers, rd.n_layers, RECURRENT ? &rd.state : nullptr, AUTO_RESET_PERIOD, d.standardize_mean,
                                                       d.standardize_precision, initial, (int)N, (int)SPEC::STEP_LIMIT, returns, episode_length, summary, workspace, workspace_bytes), "evaluate");
        }
        else if constexpr(RECURRENT){
            devices::rocm::check(rlt_rocm_pendulum_evaluate_recurrent(device.handle, &env.pendulum, rd.has_head ? 2 : 1, rd.layers, rd.n_layers, &rd.state, AUTO_RESET_PERIOD, initial, (int)N,
                                                                      (int)SPEC::STEP_LIMIT, returns, episode_length, summary, workspace, workspace_bytes), "evaluate (recurrent)");
        }
        else{
            devices::rocm::check(rlt_rocm_pendulum_evaluate_standardized(device.handle, &env.pendulum, d.has_head ? 2 : 1, d.layers, d.n_layers, d.standardize_mean, d.standardize_precision, initial, (int)N, (int)SPEC::STEP_LIMIT, returns, episode_length, summary), "evaluate");
        }
        float host_summary[6];
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, results.returns, returns, N * sizeof(float)), "evaluate (results)");
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, results.episode_length, episode_length, N * sizeof(uint32_t)), "evaluate (results)");
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, host_summary, summary, sizeof(host_summary)), "evaluate (results)");
        results.returns_mean = host_summary[0]; results.returns_std = host_summary[1];
        results.episode_length_mean = host_summary[2]; results.episode_length_std = host_summary[3];
        results.num_terminated = (TI)host_summary[4]; results.share_terminated = host_summary[5];
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
