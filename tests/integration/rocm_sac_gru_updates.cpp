// SAC's updates with the recurrent approximators (dense -> GRU -> dense actor and critics, rl/algorithms/sac/loop/core/approximators_gru.h) on sequence batches
// on devices::ROCM next to the reference's own on its CPU device, in one program (the recurrent counterpart of rocm_sac_updates.cpp): the agent is initialised on
// the CPU and copied over, the CPU side fills the replay buffers of four environments and gathers the sequence batches (16 steps x 32 samples), and every update
// (train_critic for both critics, update_critic_targets, train_actor: rl/algorithms/sac/operations_generic.h:243-527 -- on devices::ROCM the reference's generic
// code over the GRU, dense, sample_and_squash, loss and tensor overloads of this backend) is made on both devices from the same batch and action noise. After each
// loop step's worth of updates the device's networks are copied back and compared tensor by tensor (mean absolute difference / largest magnitude): the parameters,
// bound 1e-5 (measured 8e-8), and the gradients the last backward pass left, bound 5e-5 (measured 9e-6 on the actor's output bias, whose gradient is a sum of
// cancelling terms, 2e-6 and below elsewhere). Exit code 0 if both bounds hold after each of 10 such steps.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_generic.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/sac/operations_rocm.h>

#include <rl_tools/rl/algorithms/sac/loop/core/config.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>

#include <cmath>
#include <cstdio>

namespace rlt = rl_tools;

using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using DEVICE_CPU = rlt::devices::DEVICE_FACTORY<>;
using TI = typename DEVICE::index_t;
using T = float;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;

using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct SAC_PARAMETERS: rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM>{
        static constexpr TI ACTOR_BATCH_SIZE = 32;
        static constexpr TI CRITIC_BATCH_SIZE = 32;
        static constexpr TI SEQUENCE_LENGTH = 16;
    };
    static constexpr TI N_WARMUP_STEPS = 400;
    static constexpr TI N_WARMUP_STEPS_CRITIC = 400;
    static constexpr TI N_WARMUP_STEPS_ACTOR = 400;
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
using CONFIG_CPU = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, DEVICE_CPU::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS, rlt::rl::algorithms::sac::loop::core::ConfigApproximatorsGRU>;
using CONFIG_DEV = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, DEVICE::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS, rlt::rl::algorithms::sac::loop::core::ConfigApproximatorsGRU>;
using STATE_CPU = typename CONFIG_CPU::template State<CONFIG_CPU>;
using STATE_DEV = typename CONFIG_DEV::template State<CONFIG_DEV>;

T worst = 0, worst_gradient = 0;
// mean |difference| / largest magnitude of a parameter tensor, and of its gradient (what the last update's backward pass left there)
template <bool GRADIENT, typename PARAMETER>
void compare_parameter(DEVICE_CPU& cpu, PARAMETER& from_device, PARAMETER& reference, const char* what, bool print){
    using SPEC = typename decltype(reference.parameters)::SPEC;
    const T scale = rlt::abs_max(cpu, reference.parameters);
    const T e = rlt::abs_diff(cpu, from_device.parameters, reference.parameters) / (T)SPEC::SIZE / (scale > 0 ? scale : 1);
    if(std::isnan(e) || e > worst){ worst = std::isnan(e) ? 1 : e; }
    if constexpr(GRADIENT){
        const T gradient_scale = rlt::abs_max(cpu, reference.gradient);
        const T g = rlt::abs_diff(cpu, from_device.gradient, reference.gradient) / (T)SPEC::SIZE / (gradient_scale > 0 ? gradient_scale : 1);
        if(std::isnan(g) || g > worst_gradient){ worst_gradient = std::isnan(g) ? 1 : g; }
        if(print){ std::printf("  %s %.1e (gradient %.1e)", what, e, g); }
    }
    else if(print){ std::printf("  %s %.1e", what, e); }
}
// dense -> GRU -> dense; target networks carry no gradients
template <bool GRADIENT, typename MODEL>
void compare_model(DEVICE_CPU& cpu, MODEL& a, MODEL& b, const char* name, bool print){
    if(print){ std::printf("%s:", name); }
    compare_parameter<GRADIENT>(cpu, a.content.weights, b.content.weights, "W in", print);
    compare_parameter<GRADIENT>(cpu, a.content.biases, b.content.biases, "b in", print);
    compare_parameter<GRADIENT>(cpu, a.next_module.content.weights_input, b.next_module.content.weights_input, "W_i", print);
    compare_parameter<GRADIENT>(cpu, a.next_module.content.biases_input, b.next_module.content.biases_input, "b_i", print);
    compare_parameter<GRADIENT>(cpu, a.next_module.content.weights_hidden, b.next_module.content.weights_hidden, "W_h", print);
    compare_parameter<GRADIENT>(cpu, a.next_module.content.biases_hidden, b.next_module.content.biases_hidden, "b_h", print);
    compare_parameter<GRADIENT>(cpu, a.next_module.content.initial_hidden_state, b.next_module.content.initial_hidden_state, "h0", print);
    compare_parameter<GRADIENT>(cpu, a.next_module.next_module.content.weights, b.next_module.next_module.content.weights, "W out", print);
    compare_parameter<GRADIENT>(cpu, a.next_module.next_module.content.biases, b.next_module.next_module.content.biases, "b out", print);
    if(print){ std::printf("\n"); }
}

int main(){
    DEVICE device; DEVICE_CPU cpu;
    rlt::init(device);
    static STATE_CPU ts_cpu;
    static STATE_DEV ts_dev;
    static typename CONFIG_CPU::ACTOR_CRITIC_TYPE back;
    rlt::malloc(cpu, ts_cpu); rlt::malloc(device, ts_dev); rlt::malloc(cpu, back);
    rlt::init(cpu, ts_cpu, 4); rlt::init(device, ts_dev, 4);
    // the same agent on both devices (the optimisers are in their initial state on both: age 1, zero moments)
    auto networks_to_device = [&](){
        rlt::copy(cpu, device, ts_cpu.actor_critic.actor, ts_dev.actor_critic.actor);
        for(int k = 0; k < 2; k++){
            rlt::copy(cpu, device, ts_cpu.actor_critic.critics[k], ts_dev.actor_critic.critics[k]);
            rlt::copy(cpu, device, ts_cpu.actor_critic.critics_target[k], ts_dev.actor_critic.critics_target[k]);
        }
    };
    auto networks_from_device = [&](){
        rlt::copy(device, cpu, ts_dev.actor_critic.actor, back.actor);
        for(int k = 0; k < 2; k++){
            rlt::copy(device, cpu, ts_dev.actor_critic.critics[k], back.critics[k]);
            rlt::copy(device, cpu, ts_dev.actor_critic.critics_target[k], back.critics_target[k]);
        }
    };
    networks_to_device();
    // the reference's loop on the CPU through its warm-up: 400 transitions in each of the four replay buffers
    for(TI step = 0; step < LOOP_CORE_PARAMETERS::N_WARMUP_STEPS; step++){ rlt::step(cpu, ts_cpu); }
    constexpr int STEPS = 10;
    for(int step = 0; step < STEPS; step++){
        const bool print = step == 0 || step == STEPS - 1;
        for(int critic_i = 0; critic_i < 2; critic_i++){
            rlt::gather_batch(cpu, ts_cpu.off_policy_runner, ts_cpu.critic_batch, ts_cpu.rng);
            rlt::randn(cpu, ts_cpu.action_noise_critic, ts_cpu.rng);
            rlt::copy(cpu, device, ts_cpu.critic_batch, ts_dev.critic_batch);
            rlt::copy(cpu, device, ts_cpu.action_noise_critic, ts_dev.action_noise_critic);
            rlt::train_critic(cpu, ts_cpu.actor_critic, ts_cpu.actor_critic.critics[critic_i], ts_cpu.critic_batch, ts_cpu.actor_critic.critic_optimizers[critic_i], ts_cpu.actor_target_buffers[critic_i], ts_cpu.critic_buffers[critic_i], ts_cpu.critic_target_buffers[critic_i], ts_cpu.critic_training_buffers[critic_i], ts_cpu.action_noise_critic, ts_cpu.rng);
            rlt::train_critic(device, ts_dev.actor_critic, ts_dev.actor_critic.critics[critic_i], ts_dev.critic_batch, ts_dev.actor_critic.critic_optimizers[critic_i], ts_dev.actor_target_buffers[critic_i], ts_dev.critic_buffers[critic_i], ts_dev.critic_target_buffers[critic_i], ts_dev.critic_training_buffers[critic_i], ts_dev.action_noise_critic, ts_dev.rng);
        }
        rlt::update_critic_targets(cpu, ts_cpu.actor_critic);
        rlt::update_critic_targets(device, ts_dev.actor_critic);
        rlt::gather_batch(cpu, ts_cpu.off_policy_runner, ts_cpu.actor_batch, ts_cpu.rng);
        rlt::randn(cpu, ts_cpu.action_noise_actor, ts_cpu.rng);
        rlt::copy(cpu, device, ts_cpu.actor_batch, ts_dev.actor_batch);
        rlt::copy(cpu, device, ts_cpu.action_noise_actor, ts_dev.action_noise_actor);
        rlt::train_actor(cpu, ts_cpu.actor_critic, ts_cpu.actor_batch, ts_cpu.actor_critic.actor_optimizer, ts_cpu.actor_buffers[0], ts_cpu.critic_buffers[0], ts_cpu.actor_training_buffers, ts_cpu.action_noise_actor, ts_cpu.rng);
        rlt::train_actor(device, ts_dev.actor_critic, ts_dev.actor_batch, ts_dev.actor_critic.actor_optimizer, ts_dev.actor_buffers[0], ts_dev.critic_buffers[0], ts_dev.actor_training_buffers, ts_dev.action_noise_actor, ts_dev.rng);
        networks_from_device();
        if(print){ std::printf("after %d loop steps of updates: mean |difference| / largest magnitude per tensor\n", step + 1); }
        compare_model<true>(cpu, back.actor, ts_cpu.actor_critic.actor, "actor", print);
        compare_model<true>(cpu, back.critics[0], ts_cpu.actor_critic.critics[0], "critic 0", print);
        compare_model<true>(cpu, back.critics[1], ts_cpu.actor_critic.critics[1], "critic 1", print);
        compare_model<false>(cpu, back.critics_target[0], ts_cpu.actor_critic.critics_target[0], "critic target 0", print);
        compare_model<false>(cpu, back.critics_target[1], ts_cpu.actor_critic.critics_target[1], "critic target 1", print);
    }
    rlt::check_status(device);
    std::printf("worst %.2e worst_gradient %.2e\n", worst, worst_gradient);
    return worst <= 1e-5f && worst_gradient <= 5e-5f ? 0 : 1;
}
