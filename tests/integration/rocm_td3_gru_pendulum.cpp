// The reference's TD3 loop with its recurrent approximators (rl/algorithms/td3/loop/core/approximators_gru.h: GRU -> dense actor without a sampling layer, GRU -> dense
// critics) and sequence batches (SEQUENCE_LENGTH > 1) instantiated on devices::ROCM for the Pendulum, inside the reference's evaluation and timing loop steps: the runner
// steps the recurrent actor with its kept state (the actor's output is the action), train_critic / train_actor / both target updates resolve to the library's entry
// points for sequence batches, the evaluations run on the device. Only the device type and the ROCM includes differ from a CPU program.
//
// With -DTD3_GRU_DEVICE_CPU the same program runs on the reference's CPU device (generic operations, one thread).
//
// Usage: rocm_td3_gru_pendulum [n_steps [seed]] ; prints "step <n> mean_return <r>" for the evaluation made at loop step n and a last line
// "final <r> loop_steps_per_second_including_evaluations <x>" (r: the last evaluation made).
#include <rl_tools/operations/cpu_mux.h>
#ifndef TD3_GRU_DEVICE_CPU
#include <rl_tools/operations/rocm.h>
#endif
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/td3_sampling/operations_generic.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#ifndef TD3_GRU_DEVICE_CPU
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/td3/operations_rocm.h>
#include <rl_tools/rl/utils/evaluation/operations_rocm.h>
#else
#include <rl_tools/rl/utils/evaluation/operations_cpu.h>
#endif

#include <rl_tools/rl/algorithms/td3/loop/core/config.h>
#include <rl_tools/rl/loop/steps/evaluation/config.h>
#include <rl_tools/rl/loop/steps/timing/config.h>
#include <rl_tools/rl/algorithms/td3/loop/core/operations_generic.h>
#ifndef TD3_GRU_DEVICE_CPU
#include <rl_tools/rl/algorithms/td3/loop/core/operations_rocm.h>       // the loop step with both critic updates of the shared sequence batch as one call
#endif
#include <rl_tools/rl/loop/steps/evaluation/operations_generic.h>
#include <rl_tools/rl/loop/steps/timing/operations_cpu.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

#ifndef TD3_GRU_DEVICE_CPU
using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
#else
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
#endif
using TI = typename DEVICE::index_t;
using T = float;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;

using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::td3::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct TD3_PARAMETERS: rlt::rl::algorithms::td3::DefaultParameters<TYPE_POLICY, TI>{
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
using LOOP_CORE_CONFIG = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS, rlt::rl::algorithms::td3::loop::core::ConfigApproximatorsGRU>;
struct LOOP_EVAL_PARAMETERS: rlt::rl::loop::steps::evaluation::Parameters<TYPE_POLICY, TI, LOOP_CORE_CONFIG>{
    static constexpr TI EVALUATION_INTERVAL = 1000;
    static constexpr TI NUM_EVALUATION_EPISODES = 50;
    static constexpr TI N_EVALUATIONS = LOOP_CORE_PARAMETERS::STEP_LIMIT / EVALUATION_INTERVAL;
};
using LOOP_EVAL_CONFIG = rlt::rl::loop::steps::evaluation::Config<LOOP_CORE_CONFIG, LOOP_EVAL_PARAMETERS>;
using LOOP_CONFIG = rlt::rl::loop::steps::timing::Config<LOOP_EVAL_CONFIG>;
using LOOP_STATE = typename LOOP_CONFIG::template State<LOOP_CONFIG>;

int main(int argc, char** argv){
    const TI n_steps = argc > 1 ? (TI)std::atoi(argv[1]) : LOOP_CORE_PARAMETERS::STEP_LIMIT;
    const TI seed = argc > 2 ? (TI)std::atoi(argv[2]) : 0;
    DEVICE device;
    LOOP_STATE ts;
    rlt::init(device);
    rlt::malloc(device, ts);
    rlt::init(device, ts, seed);
    const auto start = std::chrono::steady_clock::now();
    while(ts.step < n_steps && !rlt::step(device, ts)){
    }
#ifndef TD3_GRU_DEVICE_CPU
    rlt::check_status(device);
#endif
    const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
    const TI made = (ts.step + LOOP_EVAL_PARAMETERS::EVALUATION_INTERVAL - 1) / LOOP_EVAL_PARAMETERS::EVALUATION_INTERVAL;
    double last = 0;
    for(TI i = 0; i < made && i < LOOP_EVAL_PARAMETERS::N_EVALUATIONS; i++){
        last = (double)rlt::get(ts.evaluation_results, 0, i).returns_mean;
        std::printf("step %u mean_return %f\n", (unsigned)(i * LOOP_EVAL_PARAMETERS::EVALUATION_INTERVAL), last);
    }
    std::printf("final %f loop_steps_per_second_including_evaluations %f\n", last, (double)ts.step / seconds);
    rlt::free(device, ts);
    rlt::free(device);
    return 0;
}
