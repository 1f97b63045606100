// The reference's own SAC training loop (rl/algorithms/sac/loop/core: malloc, init, step) instantiated on devices::ROCM for the Pendulum, the
// program a maintainer would write to use the backend (the CUDA counterpart is src/rl/environments/pendulum/sac/cuda/sac.cu:6-27,122-164).
// Only the device type and the two ROCM includes differ from a CPU program; every operation the loop calls resolves to an overload of this
// backend. Evaluation runs on the CPU device on a copy of the actor, as in the CUDA program.
//
// Built with -DSAC_LOOP_GRAPH the loop step past the warm-up is recorded once into a graph and replayed (the counterpart of the CUDA program's three
// graphs, sac.cu:122-164); -DSAC_LOOP_HIDDEN_WIDTH=<n> sets the width of all networks (64 unless given).
//
// Usage: rocm_sac_pendulum [n_steps [seed [batch-size tag ignored]]] ; prints "step <n> mean_return <r>" lines and a last line "final <r>".
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

#include <rl_tools/rl/algorithms/sac/loop/core/config.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_rocm.h>
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
#ifndef SAC_LOOP_HIDDEN_WIDTH
#define SAC_LOOP_HIDDEN_WIDTH 64
#endif
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct SAC_PARAMETERS: rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM>{
        static constexpr TI ACTOR_BATCH_SIZE = BATCH_SIZE;
        static constexpr TI CRITIC_BATCH_SIZE = BATCH_SIZE;
    };
    static constexpr TI N_WARMUP_STEPS = BATCH_SIZE;
    static constexpr TI N_WARMUP_STEPS_CRITIC = BATCH_SIZE;
    static constexpr TI N_WARMUP_STEPS_ACTOR = BATCH_SIZE;
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = SAC_LOOP_HIDDEN_WIDTH;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = SAC_LOOP_HIDDEN_WIDTH;
    static constexpr bool COLLECT_EPISODE_STATS = false;
    static constexpr TI EPISODE_STATS_BUFFER_SIZE = 0;
};
using LOOP_CORE_CONFIG = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
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
    auto stretch_start = start;
    double training_seconds = 0, training_only_seconds = 0;
#ifdef SAC_LOOP_GRAPH
    rlt_rocm_graph* step_graph = nullptr;
#endif
    for(TI step = 0; step < n_steps; step++){
#ifdef SAC_LOOP_GRAPH
        // past the warm-up every loop step issues the same launches: the first few run as they are (which also sizes every workspace), one is
        // recorded, the rest are replays of it; the step counter, which the recorded calls do not read, advances on the host
        bool finished = false;
        if(ts.step < LOOP_CORE_PARAMETERS::N_WARMUP_STEPS + 3){
            finished = rlt::step(device, ts);
        }
        else{
            if(!step_graph){
                const TI recorded_at = ts.step;
                rlt::devices::rocm::begin_capture(device);
                rlt::step(device, ts);
                step_graph = rlt::devices::rocm::end_capture(device);
                ts.step = recorded_at;      // recorded, not run
            }
            finished = ts.step >= LOOP_CORE_PARAMETERS::STEP_LIMIT;
            if(!finished){
                rlt::devices::rocm::replay(device, step_graph);
                ts.step++;
            }
        }
#else
        const bool finished = rlt::step(device, ts);
#endif
        if((step + 1) % 1000 == 0 || step + 1 == n_steps || finished){
            rlt::check_status(device);
            training_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
            training_only_seconds += std::chrono::duration<double>(std::chrono::steady_clock::now() - stretch_start).count();
            std::printf("step %u mean_return %f\n", (unsigned)(step + 1), (double)evaluate());
            std::fflush(stdout);
            stretch_start = std::chrono::steady_clock::now();
        }
        if(finished){ break; }
    }
    std::printf("final %f loop_steps_per_second_including_evaluations %f loop_steps_per_second_between_evaluations %f\n", (double)evaluate(), (double)ts.step / training_seconds,
                (double)ts.step / training_only_seconds);
#ifdef SAC_LOOP_GRAPH
    rlt::devices::rocm::free_graph(device, step_graph);
#endif
    rlt::free(device, ts);
    rlt::free(device_evaluation, actor_evaluation);
    rlt::free(device);
    return 0;
}
