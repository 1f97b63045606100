// The reference's own TD3 training loop (rl/algorithms/td3/loop/core: malloc, init, step) instantiated on devices::ROCM for the Pendulum, the
// program a maintainer would write to use the backend (the CPU counterpart is src/rl/environments/pendulum/td3/cpu/standalone.cpp; the SAC
// program's CUDA counterpart is src/rl/environments/pendulum/sac/cuda/sac.cu:6-27,122-164).
// Only the device type and the two ROCM includes differ from a CPU program; every operation the loop calls resolves to an overload of this
// backend. Evaluation runs on the CPU device on a copy of the actor, as in the CUDA program.
//
// Usage: rocm_td3_pendulum [n_steps [seed [batch-size tag ignored]]] ; prints "step <n> mean_return <r>" lines and a last line "final <r>".
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/td3_sampling/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/td3/operations_rocm.h>

#include <rl_tools/rl/algorithms/td3/loop/core/config.h>
#include <rl_tools/rl/algorithms/td3/loop/core/operations_generic.h>
#include <rl_tools/rl/algorithms/td3/loop/core/operations_rocm.h>
#include <rl_tools/rl/utils/evaluation/operations_generic.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using DEVICE_EVALUATION = rlt::devices::DEVICE_FACTORY<>;
using TI = typename DEVICE::index_t;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;

using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
#ifndef BATCH_SIZE
#define BATCH_SIZE 256
#endif
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::td3::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct TD3_PARAMETERS: rlt::rl::algorithms::td3::DefaultParameters<TYPE_POLICY, TI>{
        static constexpr TI ACTOR_BATCH_SIZE = BATCH_SIZE;
        static constexpr TI CRITIC_BATCH_SIZE = BATCH_SIZE;
    };
    static constexpr TI N_WARMUP_STEPS = BATCH_SIZE;
    static constexpr TI N_WARMUP_STEPS_CRITIC = BATCH_SIZE;
    static constexpr TI N_WARMUP_STEPS_ACTOR = BATCH_SIZE;
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 64;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 64;
    static constexpr bool COLLECT_EPISODE_STATS = false;
    static constexpr TI EPISODE_STATS_BUFFER_SIZE = 0;
};
using LOOP_CORE_CONFIG = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
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
        if((step + 1) % 1000 == 0 || step + 1 == n_steps || finished){
            rlt::check_status(device);
            training_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
            std::printf("step %u mean_return %f\n", (unsigned)(step + 1), (double)evaluate());
            std::fflush(stdout);
        }
        if(finished){ break; }
    }
    std::printf("final %f loop_steps_per_second_including_evaluations %f\n", (double)evaluate(), (double)ts.step / training_seconds);
    rlt::free(device, ts);
    rlt::free(device_evaluation, actor_evaluation);
    rlt::free(device);
    return 0;
}
