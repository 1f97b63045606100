// The reference's SAC loop wrapped in its evaluation and timing loop steps (rl/loop/steps/evaluation, rl/loop/steps/timing), as its training
// programs build it (src/rl/environments/pendulum/sac/cpu/training.h:31-84), instantiated on devices::ROCM: `while(!step(device, ts))` is
// the whole program, and the evaluations run on the device through the evaluate overload of this backend
// (rl/utils/evaluation/operations_rocm.h) instead of on a CPU copy of the actor as in src/rl/environments/pendulum/sac/cuda/sac.cu.
//
// Usage: rocm_sac_pendulum_loop_steps [seed] ; prints "evaluation <i> mean_return <r>" lines for the loop's evaluation results and a last
// line "final <r> loop_steps_per_second_including_evaluations <x>".
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
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
#include <rl_tools/rl/loop/steps/timing/config.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_rocm.h>
#include <rl_tools/rl/loop/steps/evaluation/operations_generic.h>
#include <rl_tools/rl/loop/steps/timing/operations_cpu.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

namespace rlt = rl_tools;

using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using TI = typename DEVICE::index_t;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;

using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct SAC_PARAMETERS: rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM>{
        static constexpr TI ACTOR_BATCH_SIZE = 256;
        static constexpr TI CRITIC_BATCH_SIZE = 256;
    };
    static constexpr TI N_WARMUP_STEPS = 256;
    static constexpr TI N_WARMUP_STEPS_CRITIC = 256;
    static constexpr TI N_WARMUP_STEPS_ACTOR = 256;
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 64;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 64;
    static constexpr bool COLLECT_EPISODE_STATS = false;
    static constexpr TI EPISODE_STATS_BUFFER_SIZE = 0;
};
using LOOP_CORE_CONFIG = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
struct LOOP_EVAL_PARAMETERS: rlt::rl::loop::steps::evaluation::Parameters<TYPE_POLICY, TI, LOOP_CORE_CONFIG>{
    static constexpr TI EVALUATION_INTERVAL = 1000;
    static constexpr TI NUM_EVALUATION_EPISODES = 100;
    static constexpr TI N_EVALUATIONS = LOOP_CORE_PARAMETERS::STEP_LIMIT / EVALUATION_INTERVAL;
};
using LOOP_EVAL_CONFIG = rlt::rl::loop::steps::evaluation::Config<LOOP_CORE_CONFIG, LOOP_EVAL_PARAMETERS>;
using LOOP_CONFIG = rlt::rl::loop::steps::timing::Config<LOOP_EVAL_CONFIG>;
using LOOP_STATE = typename LOOP_CONFIG::template State<LOOP_CONFIG>;

int main(int argc, char** argv){
    const TI seed = argc > 1 ? (TI)std::atoi(argv[1]) : 0;
    DEVICE device;
    LOOP_STATE ts;
    rlt::init(device);
    rlt::malloc(device, ts);
    rlt::init(device, ts, seed);
    const auto start = std::chrono::steady_clock::now();
    while(!rlt::step(device, ts)){
    }
    rlt::check_status(device);
    const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
    for(TI i = 0; i < LOOP_EVAL_PARAMETERS::N_EVALUATIONS; i++){
        std::printf("evaluation %u mean_return %f\n", (unsigned)i, (double)rlt::get(ts.evaluation_results, 0, i).returns_mean);
    }
    std::printf("final %f loop_steps_per_second_including_evaluations %f\n", (double)rlt::get(ts.evaluation_results, 0, LOOP_EVAL_PARAMETERS::N_EVALUATIONS - 1).returns_mean, (double)ts.step / seconds);
    rlt::free(device, ts);
    rlt::free(device);
    return 0;
}
