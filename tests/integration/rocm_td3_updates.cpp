// TD3's updates on devices::ROCM next to the reference's own on its CPU device, in one program (the TD3 counterpart of rocm_sac_updates.cpp): the
// agent is initialised on the CPU and copied over, the CPU side runs the reference's loop through its warm-up to fill a replay buffer, gathers the
// batches and draws the clipped target-policy noise (target_action_noise, rl/algorithms/td3/operations_generic.h:117-131), and every update
// (train_critic for both critics, update_critic_targets, train_actor, update_actor_target: :170-325) is then made on both devices from the same
// batch and noise -- also the N(0, 1) draws the reference makes INSIDE the td3_sampling layer of the (target) actor's forward pass: they are replayed
// from a copy of the CPU generator's state and handed to the device through devices::ROCM::td3_sampling_noise_override. After each loop step's worth of updates the device's networks are copied back and compared with the CPU's. Exit code 0 if every
// parameter tensor of the six networks agrees to 1e-5 of its largest magnitude (mean absolute difference) after each of 20 such steps.
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
        static constexpr TI ACTOR_BATCH_SIZE = 256;
        static constexpr TI CRITIC_BATCH_SIZE = 256;
    };
    static constexpr TI N_WARMUP_STEPS = 600;
    static constexpr TI N_WARMUP_STEPS_CRITIC = 600;
    static constexpr TI N_WARMUP_STEPS_ACTOR = 600;
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 64;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 64;
    static constexpr bool COLLECT_EPISODE_STATS = false;
    static constexpr TI EPISODE_STATS_BUFFER_SIZE = 0;
};
using CONFIG_CPU = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, DEVICE_CPU::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
using CONFIG_DEV = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, DEVICE::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
using STATE_CPU = typename CONFIG_CPU::template State<CONFIG_CPU>;
using STATE_DEV = typename CONFIG_DEV::template State<CONFIG_DEV>;

T worst = 0;
template <typename TENSOR>
void compare(DEVICE_CPU& cpu, TENSOR& from_device, TENSOR& reference, const char* what, bool print){
    const T scale = rlt::abs_max(cpu, reference);
    const T e = rlt::abs_diff(cpu, from_device, reference) / (T)TENSOR::SPEC::SIZE / (scale > 0 ? scale : 1);
    if(print){ std::printf("  %s %.2e", what, e); }
    if(std::isnan(e) || e > worst){ worst = std::isnan(e) ? 1 : e; }
}
template <typename MLP>
void compare_mlp(DEVICE_CPU& cpu, MLP& from_device, MLP& reference, const char* name, bool print){
    if(print){ std::printf("%s:", name); }
    compare(cpu, from_device.input_layer.weights.parameters, reference.input_layer.weights.parameters, "W1", print);
    compare(cpu, from_device.hidden_layers[0].weights.parameters, reference.hidden_layers[0].weights.parameters, "W2", print);
    compare(cpu, from_device.output_layer.weights.parameters, reference.output_layer.weights.parameters, "W3", print);
    compare(cpu, from_device.output_layer.biases.parameters, reference.output_layer.biases.parameters, "b3", print);
    if(print){ std::printf("\n"); }
}

int main(){
    DEVICE device; DEVICE_CPU cpu;
    rlt::init(device);
    static STATE_CPU ts_cpu;
    static STATE_DEV ts_dev;
    static typename CONFIG_CPU::ACTOR_CRITIC_TYPE back;
    rlt::malloc(cpu, ts_cpu); rlt::malloc(device, ts_dev); rlt::malloc(cpu, back);
    rlt::init(cpu, ts_cpu, 5); rlt::init(device, ts_dev, 5);
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
    // what the td3_sampling layer will draw in the next forward pass on the CPU (one N(0, 1) per row and action, in row order,
    // nn/layers/td3_sampling/operations_generic.h:75-128), replayed from a copy of the generator and put where the device's update reads it
    rlt::Matrix<rlt::matrix::Specification<T, TI, 256, ENVIRONMENT::ACTION_DIM>> sampling_noise_cpu;
    rlt::Matrix<rlt::matrix::Specification<T, DEVICE::index_t, 256, ENVIRONMENT::ACTION_DIM>> sampling_noise_dev;
    rlt::malloc(cpu, sampling_noise_cpu); rlt::malloc(device, sampling_noise_dev);
    auto replay_sampling_noise = [&](){
        auto rng_copy = ts_cpu.rng;
        for(TI row = 0; row < 256; row++){
            for(TI col = 0; col < ENVIRONMENT::ACTION_DIM; col++){ rlt::set(sampling_noise_cpu, row, col, rlt::random::normal_distribution::sample(cpu.random, (T)0, (T)1, rng_copy)); }
        }
        rlt::copy(cpu, device, sampling_noise_cpu, sampling_noise_dev);
        device.td3_sampling_noise_override = sampling_noise_dev._data;
    };
    // the reference's loop on the CPU through its warm-up: 600 transitions in the replay buffer
    for(TI step = 0; step < LOOP_CORE_PARAMETERS::N_WARMUP_STEPS; step++){ rlt::step(cpu, ts_cpu); }
    constexpr int STEPS = 20;
    for(int step = 0; step < STEPS; step++){
        const bool print = step == 0 || step == STEPS - 1;
        for(int critic_i = 0; critic_i < 2; critic_i++){
            rlt::gather_batch(cpu, ts_cpu.off_policy_runner, ts_cpu.critic_batch, ts_cpu.rng);
            auto noise_cpu = rlt::matrix_view(cpu, ts_cpu.critic_training_buffers.target_next_action_noise);
            rlt::target_action_noise(cpu, ts_cpu.actor_critic, noise_cpu, ts_cpu.rng);
            rlt::copy(cpu, device, ts_cpu.critic_batch, ts_dev.critic_batch);
            rlt::copy(cpu, device, ts_cpu.critic_training_buffers.target_next_action_noise, ts_dev.critic_training_buffers.target_next_action_noise);
            replay_sampling_noise();
            rlt::train_critic(cpu, ts_cpu.actor_critic, ts_cpu.actor_critic.critics[critic_i], ts_cpu.critic_batch, ts_cpu.actor_critic.critic_optimizers[critic_i], ts_cpu.actor_buffers[critic_i], ts_cpu.actor_target_buffers[critic_i], ts_cpu.critic_buffers[critic_i], ts_cpu.critic_target_buffers[critic_i], ts_cpu.critic_training_buffers, ts_cpu.rng);
            rlt::train_critic(device, ts_dev.actor_critic, ts_dev.actor_critic.critics[critic_i], ts_dev.critic_batch, ts_dev.actor_critic.critic_optimizers[critic_i], ts_dev.actor_buffers[critic_i], ts_dev.actor_target_buffers[critic_i], ts_dev.critic_buffers[critic_i], ts_dev.critic_target_buffers[critic_i], ts_dev.critic_training_buffers, ts_dev.rng);
        }
        rlt::update_critic_targets(cpu, ts_cpu.actor_critic);
        rlt::update_critic_targets(device, ts_dev.actor_critic);
        rlt::gather_batch(cpu, ts_cpu.off_policy_runner, ts_cpu.actor_batch, ts_cpu.rng);
        rlt::copy(cpu, device, ts_cpu.actor_batch, ts_dev.actor_batch);
        replay_sampling_noise();
        rlt::train_actor(cpu, ts_cpu.actor_critic, ts_cpu.actor_batch, ts_cpu.actor_critic.actor_optimizer, ts_cpu.actor_buffers[0], ts_cpu.critic_buffers[0], ts_cpu.actor_training_buffers, ts_cpu.rng);
        rlt::train_actor(device, ts_dev.actor_critic, ts_dev.actor_batch, ts_dev.actor_critic.actor_optimizer, ts_dev.actor_buffers[0], ts_dev.critic_buffers[0], ts_dev.actor_training_buffers, ts_dev.rng);
        rlt::update_actor_target(cpu, ts_cpu.actor_critic);
        rlt::update_actor_target(device, ts_dev.actor_critic);
        networks_from_device();
        if(print){ std::printf("after %d loop steps of updates: mean |difference| / largest magnitude per tensor\n", step + 1); }
        compare_mlp(cpu, back.actor.content, ts_cpu.actor_critic.actor.content, "actor", print);
        compare_mlp(cpu, back.actor_target.content, ts_cpu.actor_critic.actor_target.content, "actor target", print);
        compare_mlp(cpu, back.critics[0].content, ts_cpu.actor_critic.critics[0].content, "critic 0", print);
        compare_mlp(cpu, back.critics[1].content, ts_cpu.actor_critic.critics[1].content, "critic 1", print);
        compare_mlp(cpu, back.critics_target[0].content, ts_cpu.actor_critic.critics_target[0].content, "critic target 0", print);
        compare_mlp(cpu, back.critics_target[1].content, ts_cpu.actor_critic.critics_target[1].content, "critic target 1", print);
    }
    rlt::check_status(device);
    std::printf("worst %.2e\n", worst);
    return worst <= 1e-5f ? 0 : 1;
}
