// SAC's updates on devices::ROCM next to the reference's own on its CPU device, in one program: the agent is initialised on the CPU and
// copied over, the CPU side runs the reference's loop through its warm-up to fill a replay buffer and gathers batches, and every update
// (train_critic for both critics, update_critic_targets, train_actor: rl/algorithms/sac/operations_generic.h:243-527) is then made on both
// devices from the same batch and the same action noise. After each loop step's worth of updates the device's networks are copied back
// and compared with the CPU's. Exit code 0 if every parameter tensor of the five networks and log_alpha agrees to 1e-5 of its largest
// magnitude (mean absolute difference) after each of 20 such steps; the differences are fp32 summation orders.
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
using CONFIG_CPU = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, DEVICE_CPU::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
using CONFIG_DEV = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, DEVICE::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
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
    rlt::init(cpu, ts_cpu, 3); rlt::init(device, ts_dev, 3);
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
    // the reference's loop on the CPU through its warm-up: 600 transitions in the replay buffer
    for(TI step = 0; step < LOOP_CORE_PARAMETERS::N_WARMUP_STEPS; step++){ rlt::step(cpu, ts_cpu); }
    constexpr int STEPS = 20;
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
        compare_mlp(cpu, back.actor.content, ts_cpu.actor_critic.actor.content, "actor", print);
        compare_mlp(cpu, back.critics[0].content, ts_cpu.actor_critic.critics[0].content, "critic 0", print);
        compare_mlp(cpu, back.critics[1].content, ts_cpu.actor_critic.critics[1].content, "critic 1", print);
        compare_mlp(cpu, back.critics_target[0].content, ts_cpu.actor_critic.critics_target[0].content, "critic target 0", print);
        compare_mlp(cpu, back.critics_target[1].content, ts_cpu.actor_critic.critics_target[1].content, "critic target 1", print);
        if(print){ std::printf("log_alpha:"); }
        compare(cpu, back.actor.next_module.content.log_alpha.parameters, ts_cpu.actor_critic.actor.next_module.content.log_alpha.parameters, "", print);
        if(print){ std::printf("\n"); }
    }
    rlt::check_status(device);
    // the whole agent CPU -> ROCM -> CPU, optimisers included (their hyper-parameters are a container of structs, which stays in host memory on the device side)
    bool optimisers_ok = true;
    {
        static typename CONFIG_DEV::ACTOR_CRITIC_TYPE there;
        static typename CONFIG_CPU::ACTOR_CRITIC_TYPE and_back;
        rlt::malloc(device, there); rlt::malloc(cpu, and_back);
        ts_cpu.actor_critic.actor_optimizer.parameters._data[0].alpha = 0.0123f;
        ts_cpu.actor_critic.critic_optimizers[1].parameters._data[0].beta_2 = 0.987f;
        rlt::copy(cpu, device, ts_cpu.actor_critic, there);
        rlt::copy(device, device, there, ts_dev.actor_critic);
        rlt::copy(device, cpu, ts_dev.actor_critic, and_back);
        rlt::check_status(device);
        auto same = [&](auto& a, auto& b){
            const auto& p = a.parameters._data[0]; const auto& q = b.parameters._data[0];
            return p.alpha == q.alpha && p.beta_1 == q.beta_1 && p.beta_2 == q.beta_2 && p.epsilon == q.epsilon && p.epsilon_sqrt == q.epsilon_sqrt && p.bias_lr_factor == q.bias_lr_factor
                && rlt::get(cpu, a.age, 0) == rlt::get(cpu, b.age, 0);
        };
        optimisers_ok = same(and_back.actor_optimizer, ts_cpu.actor_critic.actor_optimizer) && same(and_back.critic_optimizers[0], ts_cpu.actor_critic.critic_optimizers[0])
                     && same(and_back.critic_optimizers[1], ts_cpu.actor_critic.critic_optimizers[1]) && same(and_back.alpha_optimizer, ts_cpu.actor_critic.alpha_optimizer)
                     && and_back.actor_optimizer.parameters._data[0].alpha == 0.0123f && rlt::get(cpu, and_back.actor_optimizer.age, 0) == 21;
        T worst_copy = 0;
        auto compare_copy = [&](auto& a, auto& b){ const T d = rlt::abs_diff(cpu, a, b); worst_copy = d > worst_copy ? d : worst_copy; };
        compare_copy(and_back.actor.content.hidden_layers[0].weights.parameters, ts_cpu.actor_critic.actor.content.hidden_layers[0].weights.parameters);
        compare_copy(and_back.critics[1].content.input_layer.weights.gradient_first_order_moment, ts_cpu.actor_critic.critics[1].content.input_layer.weights.gradient_first_order_moment);
        compare_copy(and_back.critics_target[0].content.output_layer.biases.parameters, ts_cpu.actor_critic.critics_target[0].content.output_layer.biases.parameters);
        optimisers_ok = optimisers_ok && worst_copy == 0;
        std::printf("whole-agent round trip: %s\n", optimisers_ok ? "identical" : "DIFFERENT");
        rlt::free(device, there); rlt::free(cpu, and_back);
    }
    std::printf("worst %.2e\n", worst);
    return (worst <= 1e-5f && optimisers_ok) ? 0 : 1;
}
