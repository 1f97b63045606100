// The reference's SAC loop (rl/algorithms/sac/loop/core) inside its evaluation loop step on the Car without a track (rl/environments/car: single-track model with
// Pacejka tire forces, terminated when the car leaves the unit square, reward exp(-5 (0.1 heading^2 + x^2 + y^2)) so that a car that stays at the origin collects
// one unit per step), instantiated on devices::ROCM: the runner steps the environment through the library's step for any environment from the description in
// rl/environments/operations_rocm.h, the evaluations run on the device.
//
// Usage: rocm_sac_car [seed [step_limit]] ; prints "evaluation <i> step <s> mean_return <r>" per evaluation and a last line
// "final <r> best <r> loop_steps <n> seconds <s>".
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_generic.h>
#include <rl_tools/rl/environments/car/operations_generic.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>
#include <rl_tools/rl/utils/evaluation/operations_rocm.h>

#include <rl_tools/rl/algorithms/sac/loop/core/config.h>
#include <rl_tools/rl/loop/steps/evaluation/config.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_rocm.h>
#include <rl_tools/rl/loop/steps/evaluation/operations_generic.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using TI = typename DEVICE::index_t;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;

using ENVIRONMENT_SPEC = rlt::rl::environments::car::Specification<float, TI>;
// the reference's Car predates the EPISODE_STEP_LIMIT member that its runner reads from the environment type (rl/components/off_policy_runner/off_policy_runner.h:41):
// the program's environment type adds it and takes over the Car's description
struct ENVIRONMENT: rlt::rl::environments::Car<ENVIRONMENT_SPEC>{
    static constexpr TI EPISODE_STEP_LIMIT = 200;
};
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools::rl::environments::rocm{
    template <> struct Description<::ENVIRONMENT>: Description<rl::environments::Car<ENVIRONMENT_SPEC>>{};
}
RL_TOOLS_NAMESPACE_WRAPPER_END
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct SAC_PARAMETERS: rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM>{
        static constexpr TI ACTOR_BATCH_SIZE = 256;
        static constexpr TI CRITIC_BATCH_SIZE = 256;
    };
    static constexpr TI N_WARMUP_STEPS = 1000;
    static constexpr TI N_WARMUP_STEPS_CRITIC = 1000;
    static constexpr TI N_WARMUP_STEPS_ACTOR = 1000;
    static constexpr TI STEP_LIMIT = 20000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
    static constexpr TI EPISODE_STEP_LIMIT = 200;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 64;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 64;
    static constexpr bool COLLECT_EPISODE_STATS = false;
    static constexpr TI EPISODE_STATS_BUFFER_SIZE = 0;
};
using LOOP_CORE_CONFIG = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
struct LOOP_EVAL_PARAMETERS: rlt::rl::loop::steps::evaluation::Parameters<TYPE_POLICY, TI, LOOP_CORE_CONFIG>{
    static constexpr TI EVALUATION_INTERVAL = 2000;
    static constexpr TI NUM_EVALUATION_EPISODES = 100;
    static constexpr TI N_EVALUATIONS = LOOP_CORE_PARAMETERS::STEP_LIMIT / EVALUATION_INTERVAL;
};
using LOOP_CONFIG = rlt::rl::loop::steps::evaluation::Config<LOOP_CORE_CONFIG, LOOP_EVAL_PARAMETERS>;
using LOOP_STATE = typename LOOP_CONFIG::template State<LOOP_CONFIG>;

int main(int argc, char** argv){
    const TI seed = argc > 1 ? (TI)std::atoi(argv[1]) : 0;
    const TI step_limit = argc > 2 ? (TI)std::atoi(argv[2]) : LOOP_CORE_PARAMETERS::STEP_LIMIT;
    DEVICE device;
    LOOP_STATE ts;
    rlt::init(device);
    rlt::malloc(device, ts);
    rlt::init(device, ts, seed);
    const auto start = std::chrono::steady_clock::now();
    bool finished = false;
    while(!finished && ts.step < step_limit){
        finished = rlt::step(device, ts);
    }
    rlt::check_status(device);
    const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
    double best = -1e30, last = 0;
    for(TI i = 0; i < LOOP_EVAL_PARAMETERS::N_EVALUATIONS && i * LOOP_EVAL_PARAMETERS::EVALUATION_INTERVAL < ts.step; i++){
        last = (double)rlt::get(ts.evaluation_results, 0, i).returns_mean;
        best = last > best ? last : best;
        std::printf("evaluation %u step %u mean_return %f\n", (unsigned)i, (unsigned)(i * LOOP_EVAL_PARAMETERS::EVALUATION_INTERVAL), last);
    }
    std::printf("final %f best %f loop_steps %u seconds %f\n", last, best, (unsigned)ts.step, seconds);
    rlt::free(device, ts);
    rlt::free(device);
    return 0;
}
