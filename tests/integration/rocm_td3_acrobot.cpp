// The configuration of the reference's TD3 program for the AcrobotSwingup (src/rl/environments/acrobot/td3/acrobot.cpp: EasyParameters, the loop's default TD3
// parameters, actor and critics 3 layers x 256, 100,000 loop steps) instantiated on devices::ROCM inside the reference's evaluation loop step: the runner steps the
// environment through the library's step for any environment (td3_sampling head: clamp(actor output + std * noise)), train_critic / train_actor are the TD3 overloads,
// the evaluations run on the device. With -DTD3_ACROBOT_DEVICE_CPU the same program runs on the reference's CPU device.
//
// Usage: rocm_td3_acrobot [seed [step_limit]] ; prints "evaluation <i> step <s> mean_return <r>" per evaluation and a last line
// "final <r> best <r> loop_steps <n> seconds <s>".
#include <rl_tools/operations/cpu_mux.h>
#ifndef TD3_ACROBOT_DEVICE_CPU
#include <rl_tools/operations/rocm.h>
#endif
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/td3_sampling/operations_generic.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/rl/environments/acrobot/operations_generic.h>
#ifndef TD3_ACROBOT_DEVICE_CPU
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/td3/operations_rocm.h>
#include <rl_tools/rl/utils/evaluation/operations_rocm.h>
#else
#include <rl_tools/rl/utils/evaluation/operations_cpu.h>
#endif
#include <rl_tools/rl/algorithms/td3/loop/core/config.h>
#include <rl_tools/rl/loop/steps/evaluation/config.h>
#include <rl_tools/rl/algorithms/td3/loop/core/operations_generic.h>
#if !defined(TD3_ACROBOT_DEVICE_CPU) && !defined(TD3_ACROBOT_GENERIC_STEP)
#include <rl_tools/rl/algorithms/td3/loop/core/operations_rocm.h>       // the loop step with the smoothing noise and both critic updates as one call
#endif
#include <rl_tools/rl/loop/steps/evaluation/operations_generic.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

#ifndef TD3_ACROBOT_DEVICE_CPU
using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
#else
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
#endif
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using TI = typename DEVICE::index_t;

using ENVIRONMENT_SPEC = rlt::rl::environments::acrobot::Specification<float, TI, rlt::rl::environments::acrobot::EasyParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::AcrobotSwingup<ENVIRONMENT_SPEC>;
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::td3::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    static constexpr TI STEP_LIMIT = 100000;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 256;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 256;
};
using LOOP_CORE_CONFIG = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
using LOOP_CONFIG = rlt::rl::loop::steps::evaluation::Config<LOOP_CORE_CONFIG>;
using LOOP_STATE = typename LOOP_CONFIG::template State<LOOP_CONFIG>;
using EVALUATION_PARAMETERS = typename LOOP_CONFIG::EVALUATION_PARAMETERS;

int main(int argc, char** argv){
    const TI seed = argc > 1 ? (TI)std::atoi(argv[1]) : 0;
    const TI step_limit = argc > 2 ? (TI)std::atoi(argv[2]) : LOOP_CORE_PARAMETERS::STEP_LIMIT;
    DEVICE device;
    LOOP_STATE ts;
#ifndef TD3_ACROBOT_DEVICE_CPU
    rlt::init(device);
#endif
    rlt::malloc(device, ts);
    rlt::init(device, ts, seed);
    const auto start = std::chrono::steady_clock::now();
    while(ts.step < step_limit && !rlt::step(device, ts)){
    }
#ifndef TD3_ACROBOT_DEVICE_CPU
    rlt::check_status(device);
#endif
    const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
    const TI made = (ts.step + EVALUATION_PARAMETERS::EVALUATION_INTERVAL - 1) / EVALUATION_PARAMETERS::EVALUATION_INTERVAL;
    double last = 0, best = -1e30;
    for(TI i = 0; i < made && i < EVALUATION_PARAMETERS::N_EVALUATIONS; i++){
        last = (double)rlt::get(ts.evaluation_results, 0, i).returns_mean;
        best = last > best ? last : best;
        std::printf("evaluation %u step %u mean_return %f\n", (unsigned)i, (unsigned)(i * EVALUATION_PARAMETERS::EVALUATION_INTERVAL), last);
    }
    std::printf("final %f best %f loop_steps %u seconds %f\n", last, best, (unsigned)ts.step, seconds);
    rlt::free(device, ts);
#ifndef TD3_ACROBOT_DEVICE_CPU
    rlt::free(device);
#endif
    return 0;
}
