// The reference's zoo configurations of the Pendulum (src/rl/zoo/pendulum-v1/{sac,td3,ppo}.h) and of the AcrobotSwingup
// (src/rl/zoo/acrobot-swingup-v0/sac.h), included as they are and instantiated on
// devices::ROCM the way src/rl/zoo/zoo.cpp:135-268 instantiates them on the CPU device: FACTORY<DEVICE, ...>::LOOP_CORE_CONFIG inside the
// evaluation and timing loop steps (the experiment tracking, checkpoint and trajectory steps of zoo.cpp write files and are left out),
// then `while(!step(device, ts))`. One source, four programs: -DZOO_SAC, -DZOO_TD3 or -DZOO_PPO selects the algorithm on the Pendulum as
// RL_TOOLS_RL_ZOO_ALGORITHM_* does there, -DZOO_ACROBOT_SWINGUP_SAC the AcrobotSwingup with SAC (RL_TOOLS_RL_ZOO_ENVIRONMENT_ACROBOT_SWINGUP_V0),
// -DZOO_PENDULUM_POSITION_SAC the Pendulum without velocity observations with SAC's recurrent approximators on sequences of 100 steps (src/rl/zoo/pendulum-position-v1/sac.h). Nothing of the configuration is restated here: batch sizes, widths, activation functions,
// step limits and optimizer parameters are the zoo's.
//
// With -DZOO_DEVICE_CPU the same program runs on the reference's CPU device (its generic operations, one thread): the figure the device's is read against.
//
// Usage: rocm_zoo_<environment>_<algorithm> [seed [step_limit]] ; prints "evaluation <i> step <s> mean_return <r>" for every evaluation the
// loop made and a last line "final <r> best <r> loop_steps <n> seconds <s>".
#include <rl_tools/operations/cpu_mux.h>
#ifndef ZOO_DEVICE_CPU
#include <rl_tools/operations/rocm.h>
#endif
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_generic.h>
#include <rl_tools/nn/layers/td3_sampling/operations_generic.h>
#include <rl_tools/nn/layers/standardize/operations_generic.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/mlp_unconditional_stddev/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/rl/environments/acrobot/operations_cpu.h>
#ifndef ZOO_DEVICE_CPU
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/standardize/operations_rocm.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>
#include <rl_tools/rl/components/running_normalizer/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/components/on_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>
#include <rl_tools/rl/algorithms/td3/operations_rocm.h>
#include <rl_tools/rl/algorithms/ppo/operations_rocm.h>
#include <rl_tools/rl/utils/evaluation/operations_rocm.h>
#else
#include <rl_tools/rl/components/on_policy_runner/operations_cpu.h>
#include <rl_tools/rl/utils/evaluation/operations_cpu.h>
#endif

#if defined(ZOO_SAC)
#include <pendulum-v1/sac.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#ifndef ZOO_DEVICE_CPU
#include <rl_tools/rl/algorithms/sac/loop/core/operations_rocm.h>
#endif
#elif defined(ZOO_TD3)
#include <pendulum-v1/td3.h>
#include <rl_tools/rl/algorithms/td3/loop/core/operations_generic.h>
#ifndef ZOO_DEVICE_CPU
#include <rl_tools/rl/algorithms/td3/loop/core/operations_rocm.h>
#endif
#elif defined(ZOO_PPO)
#include <pendulum-v1/ppo.h>
#include <rl_tools/rl/algorithms/ppo/loop/core/operations_generic.h>
#elif defined(ZOO_ACROBOT_SWINGUP_SAC)
#include <acrobot-swingup-v0/sac.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#ifndef ZOO_DEVICE_CPU
#include <rl_tools/rl/algorithms/sac/loop/core/operations_rocm.h>
#endif
#elif defined(ZOO_PENDULUM_POSITION_SAC)
#include <pendulum-position-v1/sac.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#ifndef ZOO_DEVICE_CPU
#include <rl_tools/rl/algorithms/sac/loop/core/operations_rocm.h>
#endif
#else
#error "define ZOO_SAC, ZOO_TD3, ZOO_PPO, ZOO_ACROBOT_SWINGUP_SAC or ZOO_PENDULUM_POSITION_SAC"
#endif
#include <rl_tools/rl/loop/steps/evaluation/config.h>
#include <rl_tools/rl/loop/steps/timing/config.h>
#include <rl_tools/rl/loop/steps/evaluation/operations_generic.h>
#include <rl_tools/rl/loop/steps/timing/operations_cpu.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

#ifndef ZOO_DEVICE_CPU
using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
#else
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
#endif
using TI = typename DEVICE::index_t;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;
constexpr bool DYNAMIC_ALLOCATION = true;

#if defined(ZOO_SAC)
using LOOP_CORE_CONFIG = rlt::rl::zoo::pendulum_v1::sac::FACTORY<DEVICE, TYPE_POLICY, TI, RNG, DYNAMIC_ALLOCATION>::LOOP_CORE_CONFIG;
constexpr TI TIMING_INTERVAL = 10000;
#elif defined(ZOO_TD3)
using LOOP_CORE_CONFIG = rlt::rl::zoo::pendulum_v1::td3::FACTORY<DEVICE, TYPE_POLICY, TI, RNG, DYNAMIC_ALLOCATION>::LOOP_CORE_CONFIG;
constexpr TI TIMING_INTERVAL = 10000;
#elif defined(ZOO_ACROBOT_SWINGUP_SAC)
using LOOP_CORE_CONFIG = rlt::rl::zoo::acrobot_swingup_v0::sac::FACTORY<DEVICE, TYPE_POLICY, TI, RNG, DYNAMIC_ALLOCATION>::LOOP_CORE_CONFIG;
constexpr TI TIMING_INTERVAL = 100000;
#elif defined(ZOO_PENDULUM_POSITION_SAC)
using LOOP_CORE_CONFIG = rlt::rl::zoo::pendulum_position_v1::sac::FACTORY<DEVICE, TYPE_POLICY, TI, RNG, DYNAMIC_ALLOCATION>::LOOP_CORE_CONFIG;
constexpr TI TIMING_INTERVAL = 100000;
#else
using LOOP_CORE_CONFIG = rlt::rl::zoo::pendulum_v1::ppo::FACTORY<DEVICE, TYPE_POLICY, TI, RNG, DYNAMIC_ALLOCATION>::LOOP_CORE_CONFIG;
constexpr TI TIMING_INTERVAL = 100;
#endif

constexpr TI NUM_EVALUATIONS = 100;      // src/rl/zoo/zoo.cpp:252
using LOOP_TIMING_CONFIG = rlt::rl::loop::steps::timing::Config<LOOP_CORE_CONFIG, rlt::rl::loop::steps::timing::Parameters<TI, TIMING_INTERVAL>>;
struct LOOP_EVALUATION_PARAMETERS: rlt::rl::loop::steps::evaluation::Parameters<TYPE_POLICY, TI, LOOP_TIMING_CONFIG>{
    static constexpr TI EVALUATION_INTERVAL = LOOP_CORE_CONFIG::CORE_PARAMETERS::STEP_LIMIT / NUM_EVALUATIONS == 0 ? 1 : LOOP_CORE_CONFIG::CORE_PARAMETERS::STEP_LIMIT / NUM_EVALUATIONS;
    static constexpr TI NUM_EVALUATION_EPISODES = 100;
    static constexpr TI N_EVALUATIONS = NUM_EVALUATIONS;
};
using LOOP_CONFIG = rlt::rl::loop::steps::evaluation::Config<LOOP_TIMING_CONFIG, LOOP_EVALUATION_PARAMETERS>;
using LOOP_STATE = typename LOOP_CONFIG::template State<LOOP_CONFIG>;

int main(int argc, char** argv){
    const TI seed = argc > 1 ? (TI)std::atoi(argv[1]) : 0;
    const TI step_limit = argc > 2 ? (TI)std::atoi(argv[2]) : LOOP_CORE_CONFIG::CORE_PARAMETERS::STEP_LIMIT;
    DEVICE device;
    LOOP_STATE ts;
    rlt::init(device);
    rlt::malloc(device, ts);
    rlt::init(device, ts, seed);
    const auto start = std::chrono::steady_clock::now();
    while(ts.step < step_limit && !rlt::step(device, ts)){
    }
#ifndef ZOO_DEVICE_CPU
    rlt::check_status(device);
#endif
    const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
    const TI made = (ts.step + LOOP_EVALUATION_PARAMETERS::EVALUATION_INTERVAL - 1) / LOOP_EVALUATION_PARAMETERS::EVALUATION_INTERVAL;
    double last = 0, best = -1e30;
    for(TI i = 0; i < made && i < LOOP_EVALUATION_PARAMETERS::N_EVALUATIONS; i++){
        last = (double)rlt::get(ts.evaluation_results, 0, i).returns_mean;
        best = last > best ? last : best;
        std::printf("evaluation %u step %u mean_return %f\n", (unsigned)i, (unsigned)(i * LOOP_EVALUATION_PARAMETERS::EVALUATION_INTERVAL), last);
    }
    std::printf("final %f best %f loop_steps %u seconds %f\n", last, best, (unsigned)ts.step, seconds);
    rlt::free(device, ts);
    rlt::free(device);
    return 0;
}
