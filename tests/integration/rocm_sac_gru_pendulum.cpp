// The reference's SAC loop with its recurrent approximators (rl/algorithms/sac/loop/core/approximators_gru.h: dense -> GRU -> dense actor with a
// sample_and_squash head, dense -> GRU -> dense critics) and sequence batches (SEQUENCE_LENGTH > 1: gather_batch's multi-step branch,
// rl/components/off_policy_runner/operations_generic.h:239-430) instantiated on devices::ROCM for the Pendulum; the CPU counterpart is the zoo's
// src/rl/zoo/pendulum-position-v1/sac.h:8-52 (same approximators, same batch sampling parameters; that configuration hides the velocity from the
// observation, this one does not, and is smaller so that it trains in seconds). Only the device type and the ROCM includes differ from a CPU program.
//
// With -DSAC_GRU_DEVICE_CPU the same program runs on the reference's CPU device (generic operations, one thread): the figure the device's is read against.
//
// Usage: rocm_sac_gru_pendulum [n_steps [seed]] ; prints "step <n> mean_return <r>" lines and a last line "final <r> loop_steps_per_second <x>".
#include <rl_tools/operations/cpu_mux.h>
#ifndef SAC_GRU_DEVICE_CPU
#include <rl_tools/operations/rocm.h>
#endif
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_generic.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#ifndef SAC_GRU_DEVICE_CPU
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>
#endif

#include <rl_tools/rl/algorithms/sac/loop/core/config.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#include <rl_tools/rl/utils/evaluation/operations_generic.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

#ifndef SAC_GRU_DEVICE_CPU
using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
#else
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
#endif
using DEVICE_EVALUATION = rlt::devices::DEVICE_FACTORY<>;
using TI = typename DEVICE::index_t;
using T = float;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;

using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct SAC_PARAMETERS: rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM>{
        static constexpr TI ACTOR_BATCH_SIZE = 32;
        static constexpr TI CRITIC_BATCH_SIZE = 32;
        static constexpr TI SEQUENCE_LENGTH = 16;
    };
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 32;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 32;
    static constexpr T ALPHA = 1.0;
    static constexpr TI N_ENVIRONMENTS = 4;
    static constexpr bool COLLECT_EPISODE_STATS = false;
    static constexpr TI EPISODE_STATS_BUFFER_SIZE = 0;
    struct BATCH_SAMPLING_PARAMETERS{
        static constexpr bool INCLUDE_FIRST_STEP_IN_TARGETS = true;
        static constexpr bool ALWAYS_SAMPLE_FROM_INITIAL_STATE = false;
        static constexpr bool RANDOM_SEQ_LENGTH = true;
        static constexpr bool ENABLE_NOMINAL_SEQUENCE_LENGTH_PROBABILITY = false;
        static constexpr T NOMINAL_SEQUENCE_LENGTH_PROBABILITY = 0.1;
    };
};
using LOOP_CORE_CONFIG = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS, rlt::rl::algorithms::sac::loop::core::ConfigApproximatorsGRU>;
using LOOP_STATE = typename LOOP_CORE_CONFIG::template State<LOOP_CORE_CONFIG>;

constexpr TI NUM_EVALUATION_EPISODES = 50;

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
        using RESULT_SPEC = rlt::rl::utils::evaluation::Specification<TYPE_POLICY, TI, ENVIRONMENT, NUM_EVALUATION_EPISODES, 200>;
        rlt::rl::utils::evaluation::Result<RESULT_SPEC> result;
        rlt::evaluate(device_evaluation, env_evaluation, ui, actor_evaluation, result, rng_evaluation, rlt::Mode<rlt::mode::Evaluation<>>{});
        return result.returns_mean;
    };
    std::printf("step 0 mean_return %f\n", (double)evaluate());
    const auto start = std::chrono::steady_clock::now();
    double seconds = 0;
    for(TI step = 0; step < n_steps; step++){
        const bool finished = rlt::step(device, ts);
        if((step + 1) % 1000 == 0 || step + 1 == n_steps || finished){
#ifndef SAC_GRU_DEVICE_CPU
            rlt::check_status(device);
#endif
            seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
            std::printf("step %u mean_return %f\n", (unsigned)(step + 1), (double)evaluate());
            std::fflush(stdout);
        }
        if(finished){ break; }
    }
    std::printf("final %f loop_steps_per_second_including_evaluations %f\n", (double)evaluate(), (double)ts.step / seconds);
    rlt::free(device, ts);
    rlt::free(device_evaluation, actor_evaluation);
    rlt::free(device);
    return 0;
}
