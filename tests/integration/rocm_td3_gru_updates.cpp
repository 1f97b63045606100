// TD3's updates with the recurrent approximators (rl/algorithms/td3/loop/core/approximators_gru.h: GRU -> dense actor and critics, no sampling layer) on sequence
// batches on devices::ROCM next to the reference's own on its CPU device, in one program (the TD3 counterpart of rocm_sac_gru_updates.cpp): the agent is initialised on
// the CPU and copied over, the CPU side runs the reference's loop through its warm-up to fill the replay buffers, gathers the sequence batches and draws the clipped
// target-policy noise, and every update (train_critic for both critics, update_critic_targets, train_actor, update_actor_target:
// rl/algorithms/td3/operations_generic.h:170-325) is then made on both devices from the same batch and noise; on devices::ROCM they resolve to the library's entry
// points for sequence batches. After each loop step's worth of updates the device's networks are copied back and compared with the CPU's. Exit code 0 if every parameter
// tensor of the six networks agrees to 1e-5 of its largest magnitude (mean absolute difference), and the gradients the last backward passes left to 5e-5.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/td3_sampling/operations_generic.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>
#include <rl_tools/rl/components/off_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/td3/operations_rocm.h>

#include <rl_tools/rl/algorithms/td3/loop/core/config.h>
#include <rl_tools/rl/algorithms/td3/loop/core/operations_generic.h>

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
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::td3::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    struct TD3_PARAMETERS: rlt::rl::algorithms::td3::DefaultParameters<TYPE_POLICY, TI>{
        static constexpr TI ACTOR_BATCH_SIZE = 32;
        static constexpr TI CRITIC_BATCH_SIZE = 32;
        static constexpr TI SEQUENCE_LENGTH = 16;
    };
    static constexpr TI N_WARMUP_STEPS = 400;
    static constexpr TI N_WARMUP_STEPS_CRITIC = 400;
    static constexpr TI N_WARMUP_STEPS_ACTOR = 400;
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = 4;       // GRU -> GRU -> dense
    static constexpr TI ACTOR_HIDDEN_DIM = 32;
    static constexpr TI CRITIC_NUM_LAYERS = 4;
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
using CONFIG_CPU = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, DEVICE_CPU::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS, rlt::rl::algorithms::td3::loop::core::ConfigApproximatorsGRU>;
using CONFIG_DEV = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, DEVICE::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS, rlt::rl::algorithms::td3::loop::core::ConfigApproximatorsGRU>;
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
template <bool GRADIENT, typename GRU>
void compare_gru(DEVICE_CPU& cpu, GRU& a, GRU& b, const char* name, bool print){
    if(print){ std::printf(" [%s]", name); }
    compare_parameter<GRADIENT>(cpu, a.weights_input, b.weights_input, "W_i", print);
    compare_parameter<GRADIENT>(cpu, a.biases_input, b.biases_input, "b_i", print);
    compare_parameter<GRADIENT>(cpu, a.weights_hidden, b.weights_hidden, "W_h", print);
    compare_parameter<GRADIENT>(cpu, a.biases_hidden, b.biases_hidden, "b_h", print);
    compare_parameter<GRADIENT>(cpu, a.initial_hidden_state, b.initial_hidden_state, "h0", print);
}
// GRU -> GRU -> dense; target networks carry no gradients
template <bool GRADIENT, typename MODEL>
void compare_model(DEVICE_CPU& cpu, MODEL& a, MODEL& b, const char* name, bool print){
    if(print){ std::printf("%s:", name); }
    compare_gru<GRADIENT>(cpu, a.content, b.content, "GRU 1", print);
    compare_gru<GRADIENT>(cpu, a.next_module.content, b.next_module.content, "GRU 2", print);
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
    rlt::copy(cpu, device, ts_cpu.actor_critic.actor, ts_dev.actor_critic.actor);
    rlt::copy(cpu, device, ts_cpu.actor_critic.actor_target, ts_dev.actor_critic.actor_target);
    for(int k = 0; k < 2; k++){
        rlt::copy(cpu, device, ts_cpu.actor_critic.critics[k], ts_dev.actor_critic.critics[k]);
        rlt::copy(cpu, device, ts_cpu.actor_critic.critics_target[k], ts_dev.actor_critic.critics_target[k]);
    }
    auto networks_from_device = [&](){
        rlt::copy(device, cpu, ts_dev.actor_critic.actor, back.actor);
        rlt::copy(device, cpu, ts_dev.actor_critic.actor_target, back.actor_target);
        for(int k = 0; k < 2; k++){
            rlt::copy(device, cpu, ts_dev.actor_critic.critics[k], back.critics[k]);
            rlt::copy(device, cpu, ts_dev.actor_critic.critics_target[k], back.critics_target[k]);
        }
    };
    // the reference's loop on the CPU through its warm-up: 400 transitions in each of the four replay buffers
    for(TI step = 0; step < LOOP_CORE_PARAMETERS::N_WARMUP_STEPS; step++){ rlt::step(cpu, ts_cpu); }
    constexpr int STEPS = 10;
    for(int step = 0; step < STEPS; step++){
        const bool print = step == 0 || step == STEPS - 1;
        for(int critic_i = 0; critic_i < 2; critic_i++){
            rlt::gather_batch(cpu, ts_cpu.off_policy_runner, ts_cpu.critic_batch, ts_cpu.rng);
            auto noise_cpu = rlt::matrix_view(cpu, ts_cpu.critic_training_buffers.target_next_action_noise);
            rlt::target_action_noise(cpu, ts_cpu.actor_critic, noise_cpu, ts_cpu.rng);
            rlt::copy(cpu, device, ts_cpu.critic_batch, ts_dev.critic_batch);
            rlt::copy(cpu, device, ts_cpu.critic_training_buffers.target_next_action_noise, ts_dev.critic_training_buffers.target_next_action_noise);
            rlt::train_critic(cpu, ts_cpu.actor_critic, ts_cpu.actor_critic.critics[critic_i], ts_cpu.critic_batch, ts_cpu.actor_critic.critic_optimizers[critic_i], ts_cpu.actor_buffers[critic_i], ts_cpu.actor_target_buffers[critic_i], ts_cpu.critic_buffers[critic_i], ts_cpu.critic_target_buffers[critic_i], ts_cpu.critic_training_buffers, ts_cpu.rng);
            rlt::train_critic(device, ts_dev.actor_critic, ts_dev.actor_critic.critics[critic_i], ts_dev.critic_batch, ts_dev.actor_critic.critic_optimizers[critic_i], ts_dev.actor_buffers[critic_i], ts_dev.actor_target_buffers[critic_i], ts_dev.critic_buffers[critic_i], ts_dev.critic_target_buffers[critic_i], ts_dev.critic_training_buffers, ts_dev.rng);
        }
        rlt::update_critic_targets(cpu, ts_cpu.actor_critic);
        rlt::update_critic_targets(device, ts_dev.actor_critic);
        rlt::gather_batch(cpu, ts_cpu.off_policy_runner, ts_cpu.actor_batch, ts_cpu.rng);
        rlt::copy(cpu, device, ts_cpu.actor_batch, ts_dev.actor_batch);
        rlt::train_actor(cpu, ts_cpu.actor_critic, ts_cpu.actor_batch, ts_cpu.actor_critic.actor_optimizer, ts_cpu.actor_buffers[0], ts_cpu.critic_buffers[0], ts_cpu.actor_training_buffers, ts_cpu.rng);
        rlt::train_actor(device, ts_dev.actor_critic, ts_dev.actor_batch, ts_dev.actor_critic.actor_optimizer, ts_dev.actor_buffers[0], ts_dev.critic_buffers[0], ts_dev.actor_training_buffers, ts_dev.rng);
        rlt::update_actor_target(cpu, ts_cpu.actor_critic);
        rlt::update_actor_target(device, ts_dev.actor_critic);
        networks_from_device();
        if(print){ std::printf("after %d loop steps of updates: mean |difference| / largest magnitude per tensor\n", step + 1); }
        compare_model<true>(cpu, back.actor, ts_cpu.actor_critic.actor, "actor", print);
        compare_model<false>(cpu, back.actor_target, ts_cpu.actor_critic.actor_target, "actor target", print);
        compare_model<true>(cpu, back.critics[0], ts_cpu.actor_critic.critics[0], "critic 0", print);
        compare_model<true>(cpu, back.critics[1], ts_cpu.actor_critic.critics[1], "critic 1", print);
        compare_model<false>(cpu, back.critics_target[0], ts_cpu.actor_critic.critics_target[0], "critic target 0", print);
        compare_model<false>(cpu, back.critics_target[1], ts_cpu.actor_critic.critics_target[1], "critic target 1", print);
    }
    rlt::check_status(device);
    std::printf("worst %.2e worst_gradient %.2e\n", worst, worst_gradient);
    return worst <= 1e-5f && worst_gradient <= 5e-5f ? 0 : 1;
}
