// The reference's own PPO training loop (rl/algorithms/ppo/loop/core: malloc, init, step = collect, critic evaluation, generalized
// advantage estimation, train) instantiated on devices::ROCM for the Pendulum, the program a maintainer would write to use the backend
// (the CPU counterpart is src/rl/environments/pendulum/ppo/cpu/training.cpp:1-120 with config.h:1-52). Only the device type and the
// ROCM includes differ from a CPU program; every operation the loop calls resolves to an overload of this backend. Evaluation runs on
// the CPU device on a copy of the actor.
//
// With -DPPO_ACROBOT_SWINGUP the environment is the AcrobotSwingup (rl/environments/acrobot, EasyParameters): collect then goes through the library's collection for
// any environment, the rest of the program is the same.
//
// Usage: rocm_ppo_pendulum [n_steps [seed]] ; prints "step <n> mean_return <r>" lines and a last line "final <r> ...".
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#ifdef PPO_ACROBOT_SWINGUP
#include <rl_tools/rl/environments/acrobot/operations_generic.h>
#endif
#include <rl_tools/nn/layers/standardize/operations_generic.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/mlp_unconditional_stddev/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/standardize/operations_rocm.h>
#include <rl_tools/rl/components/running_normalizer/operations_rocm.h>
#include <rl_tools/rl/components/on_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/ppo/operations_rocm.h>

#include <rl_tools/rl/algorithms/ppo/loop/core/config.h>
#include <rl_tools/rl/algorithms/ppo/loop/core/operations_generic.h>
#include <rl_tools/rl/utils/evaluation/operations_generic.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using DEVICE_EVALUATION = rlt::devices::DEVICE_FACTORY<>;
using TI = typename DEVICE::index_t;
using T = float;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;

using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
#ifdef PPO_ACROBOT_SWINGUP
using ACROBOT_SPEC = rlt::rl::environments::acrobot::Specification<float, TI, rlt::rl::environments::acrobot::EasyParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::AcrobotSwingup<ACROBOT_SPEC>;
#else
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
#endif
#ifndef NORMALIZE
#define NORMALIZE true
#endif
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::ppo::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    static constexpr TI N_ENVIRONMENTS = 64;
    static constexpr TI ON_POLICY_RUNNER_STEPS_PER_ENV = 128;
    static constexpr TI BATCH_SIZE = 1024;
    static constexpr TI ACTOR_HIDDEN_DIM = 64;
    static constexpr TI CRITIC_HIDDEN_DIM = 64;
    static constexpr auto ACTOR_ACTIVATION_FUNCTION = rlt::nn::activation_functions::ActivationFunction::TANH;
    static constexpr auto CRITIC_ACTIVATION_FUNCTION = rlt::nn::activation_functions::ActivationFunction::TANH;
    static constexpr TI STEP_LIMIT = 200;
    static constexpr TI EPISODE_STEP_LIMIT = 200;
    static constexpr bool NORMALIZE_OBSERVATIONS = NORMALIZE;
    struct ACTOR_OPTIMIZER_PARAMETERS: rlt::nn::optimizers::adam::DEFAULT_PARAMETERS_TENSORFLOW<TYPE_POLICY>{
        static constexpr T ALPHA = 0.001;
    };
    using CRITIC_OPTIMIZER_PARAMETERS = ACTOR_OPTIMIZER_PARAMETERS;
    struct PPO_PARAMETERS: rlt::rl::algorithms::ppo::DefaultParameters<TYPE_POLICY, TI, BATCH_SIZE>{
        static constexpr T ACTION_ENTROPY_COEFFICIENT = 0.0;
        static constexpr TI N_EPOCHS = 2;
        static constexpr T GAMMA = 0.9;
        static constexpr T INITIAL_ACTION_STD = 2.0;
    };
};
using LOOP_CORE_CONFIG = rlt::rl::algorithms::ppo::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
using LOOP_STATE = typename LOOP_CORE_CONFIG::template State<LOOP_CORE_CONFIG>;

constexpr TI NUM_EVALUATION_EPISODES = 100;

int main(int argc, char** argv){
    const TI n_steps = argc > 1 ? (TI)std::atoi(argv[1]) : LOOP_CORE_PARAMETERS::STEP_LIMIT;
    const TI seed = argc > 2 ? (TI)std::atoi(argv[2]) : 0;
    DEVICE device;
    DEVICE_EVALUATION device_evaluation;
    LOOP_STATE ts;
    DEVICE_EVALUATION::SPEC::RANDOM::ENGINE<> rng_evaluation;
    rlt::init(device_evaluation, rng_evaluation, seed);
    using ACTOR_TYPE_ORIG = rlt::utils::typing::remove_reference_t<decltype(rlt::get_actor(ts))>;
    using ACTOR_TYPE_INFERENCE = ACTOR_TYPE_ORIG::template CHANGE_CAPABILITY<rlt::nn::capability::Forward<>>;
    using ACTOR_TYPE_EVALUATION = ACTOR_TYPE_INFERENCE::template CHANGE_BATCH_SIZE<TI, NUM_EVALUATION_EPISODES>;
    ACTOR_TYPE_EVALUATION actor_evaluation;
    ENVIRONMENT env_evaluation;
    rlt::rl::environments::DummyUI ui;
    rlt::init(device);
    rlt::malloc(device, ts);
    rlt::malloc(device_evaluation, actor_evaluation);
    rlt::init(device, ts, seed);

    auto evaluate = [&](){
        rlt::copy(device, device_evaluation, rlt::get_actor(ts), actor_evaluation);
        using RESULT_SPEC = rlt::rl::utils::evaluation::Specification<TYPE_POLICY, TI, ENVIRONMENT, NUM_EVALUATION_EPISODES, LOOP_CORE_PARAMETERS::EPISODE_STEP_LIMIT>;
        rlt::rl::utils::evaluation::Result<RESULT_SPEC> result;
        rlt::evaluate(device_evaluation, env_evaluation, ui, actor_evaluation, result, rng_evaluation, rlt::Mode<rlt::mode::Evaluation<>>{});
        return result.returns_mean;
    };
    std::printf("step 0 mean_return %f\n", (double)evaluate());
    rlt::check_status(device);
    const auto start = std::chrono::steady_clock::now();
    double training_seconds = 0;
    for(TI step = 0; step < n_steps; step++){
        const bool finished = rlt::step(device, ts);
        if((step + 1) % 20 == 0 || step + 1 == n_steps || finished){
            rlt::check_status(device);
            training_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
            std::printf("step %u mean_return %f\n", (unsigned)(step + 1), (double)evaluate());
            std::fflush(stdout);
        }
        if(finished){ break; }
    }
    constexpr double ENV_STEPS_PER_LOOP_STEP = (double)LOOP_CORE_PARAMETERS::N_ENVIRONMENTS * LOOP_CORE_PARAMETERS::ON_POLICY_RUNNER_STEPS_PER_ENV;
    std::printf("final %f environment_steps_per_second_including_evaluations %f\n", (double)evaluate(), (double)ts.step * ENV_STEPS_PER_LOOP_STEP / training_seconds);
    rlt::free(device, ts);
    rlt::free(device_evaluation, actor_evaluation);
    rlt::free(device);
    return 0;
}
