// PPO's advantage estimation and training on devices::ROCM next to the reference's own on its CPU device, in one program: the agent is initialised
// on the CPU and copied over, every iteration's dataset is collected by the reference's on-policy runner on the CPU and copied to the device, and
// then the critic's pass over the dataset, estimate_generalized_advantages and train (rl/algorithms/ppo/operations_generic.h:60-336, called as
// rl/algorithms/ppo/loop/core/operations_generic.h:126-135 calls them) run on both devices. One epoch of one minibatch that spans the whole dataset
// (8,192 rows), so that the order in which each side shuffles the rows only changes summation orders. After every iteration the device's value,
// advantage and target columns and all parameters of actor and critic (standardize statistics set to the same non-trivial values on both sides)
// are copied back and compared. Exit code 0 if every tensor agrees to 1e-5 of its largest magnitude (mean absolute difference) in each of 5 iterations.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn/layers/standardize/operations_generic.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/mlp_unconditional_stddev/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/standardize/operations_rocm.h>
#include <rl_tools/rl/components/running_normalizer/operations_rocm.h>
#include <rl_tools/rl/components/on_policy_runner/operations_cpu.h>
#include <rl_tools/rl/components/on_policy_runner/operations_rocm.h>
#include <rl_tools/rl/algorithms/ppo/operations_rocm.h>

#include <rl_tools/rl/algorithms/ppo/loop/core/config.h>
#include <rl_tools/rl/algorithms/ppo/loop/core/operations_generic.h>

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
struct LOOP_CORE_PARAMETERS: rlt::rl::algorithms::ppo::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT>{
    static constexpr TI N_ENVIRONMENTS = 64;
    static constexpr TI ON_POLICY_RUNNER_STEPS_PER_ENV = 128;
    static constexpr TI BATCH_SIZE = N_ENVIRONMENTS * ON_POLICY_RUNNER_STEPS_PER_ENV;
    static constexpr TI ACTOR_HIDDEN_DIM = 64;
    static constexpr TI CRITIC_HIDDEN_DIM = 64;
    static constexpr auto ACTOR_ACTIVATION_FUNCTION = rlt::nn::activation_functions::ActivationFunction::TANH;
    static constexpr auto CRITIC_ACTIVATION_FUNCTION = rlt::nn::activation_functions::ActivationFunction::TANH;
    static constexpr TI STEP_LIMIT = 200;
    static constexpr TI EPISODE_STEP_LIMIT = 200;
    static constexpr bool NORMALIZE_OBSERVATIONS = true;
    struct PPO_PARAMETERS: rlt::rl::algorithms::ppo::DefaultParameters<TYPE_POLICY, TI, BATCH_SIZE>{
        static constexpr T ACTION_ENTROPY_COEFFICIENT = 0.01;
        static constexpr TI N_EPOCHS = 1;
        static constexpr T GAMMA = 0.9;
        static constexpr T INITIAL_ACTION_STD = 2.0;
    };
};
using CONFIG_CPU = rlt::rl::algorithms::ppo::loop::core::Config<TYPE_POLICY, TI, DEVICE_CPU::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
using CONFIG_DEV = rlt::rl::algorithms::ppo::loop::core::Config<TYPE_POLICY, TI, DEVICE::SPEC::RANDOM::ENGINE<>, ENVIRONMENT, LOOP_CORE_PARAMETERS>;
using STATE_CPU = typename CONFIG_CPU::template State<CONFIG_CPU>;
using STATE_DEV = typename CONFIG_DEV::template State<CONFIG_DEV>;

T worst = 0;
template <typename A, typename B>
void compare(DEVICE_CPU& cpu, A& from_device, B& reference, const char* what, bool print){
    const T scale = rlt::abs_max(cpu, reference);
    const T e = rlt::abs_diff(cpu, from_device, reference) / (T)A::SPEC::SIZE / (scale > 0 ? scale : 1);
    if(print){ std::printf("  %s %.2e", what, e); }
    if(std::isnan(e) || e > worst){ worst = std::isnan(e) ? 1 : e; }
}
template <typename A, typename B>
void compare_column(A& from_device, B& reference, const char* what, bool print){
    T scale = 0, sum = 0;
    for(TI r = 0; r < A::ROWS; r++){
        const T a = rlt::get(from_device, r, 0), b = rlt::get(reference, r, 0);
        scale = std::fabs(b) > scale ? std::fabs(b) : scale; sum += std::fabs(a - b);
    }
    const T e = sum / (T)A::ROWS / (scale > 0 ? scale : 1);
    if(print){ std::printf("  %s %.2e", what, e); }
    if(std::isnan(e) || e > worst){ worst = std::isnan(e) ? 1 : e; }
}
template <typename MLP>
void compare_mlp(DEVICE_CPU& cpu, MLP& from_device, MLP& reference, const char* name, bool print){
    if(print){ std::printf("%s:", name); }
    compare(cpu, from_device.input_layer.weights.parameters, reference.input_layer.weights.parameters, "W1", print);
    compare(cpu, from_device.input_layer.biases.parameters, reference.input_layer.biases.parameters, "b1", print);
    compare(cpu, from_device.hidden_layers[0].weights.parameters, reference.hidden_layers[0].weights.parameters, "W2", print);
    compare(cpu, from_device.output_layer.weights.parameters, reference.output_layer.weights.parameters, "W3", print);
    compare(cpu, from_device.output_layer.biases.parameters, reference.output_layer.biases.parameters, "b3", print);
}
// the critic's pass over the whole dataset and the advantage estimation, as the loop's step makes them
template <typename DEV, typename STATE>
void values_and_advantages(DEV& device, STATE& ts){
    using CONFIG = typename STATE::CONFIG;
    constexpr TI FORWARD_BATCH_SIZE = CONFIG::ON_POLICY_RUNNER_DATASET_SPEC::STEPS_TOTAL_ALL;
    auto observations = rlt::to_tensor(device, ts.on_policy_runner_dataset.all_observations_privileged);
    auto observations_reshaped = rlt::reshape_row_major(device, observations, rlt::tensor::Shape<TI, 1, FORWARD_BATCH_SIZE, decltype(observations)::SHAPE::LAST>{});
    auto values = rlt::to_tensor(device, ts.on_policy_runner_dataset.all_values);
    auto values_reshaped = rlt::reshape_row_major(device, values, rlt::tensor::Shape<TI, 1, FORWARD_BATCH_SIZE, 1>{});
    rlt::evaluate(device, ts.ppo.critic, observations_reshaped, values_reshaped, ts.critic_buffers_gae, ts.rng, rlt::Mode<rlt::mode::Rollout<>>{});
    rlt::estimate_generalized_advantages(device, ts.on_policy_runner_dataset, typename CONFIG::PPO_TYPE::SPEC::PARAMETERS{});
}

int main(){
    DEVICE device; DEVICE_CPU cpu;
    rlt::init(device);
    static STATE_CPU ts_cpu;
    static STATE_DEV ts_dev;
    static STATE_CPU back;      // host copies of what the device holds
    rlt::malloc(cpu, ts_cpu); rlt::malloc(device, ts_dev); rlt::malloc(cpu, back);
    rlt::init(cpu, ts_cpu, 7); rlt::init(device, ts_dev, 7); rlt::init(cpu, back, 7);
    // observation statistics other than (0, 1) in the standardize layers of actor and critic, the same on both sides
    {
        auto& mean = ts_cpu.observation_normalizer.mean; auto& std_dev = ts_cpu.observation_normalizer.std;
        const T m[3] = {0.1f, -0.2f, 0.3f}, s[3] = {0.7f, 0.6f, 2.5f};
        for(TI i = 0; i < 3; i++){ rlt::set(mean, 0, i, m[i]); rlt::set(std_dev, 0, i, s[i]); }
        rlt::set_statistics(cpu, rlt::get_first_layer(ts_cpu.ppo.actor), mean, std_dev);
        rlt::set_statistics(cpu, ts_cpu.ppo.critic.content, mean, std_dev);
    }
    rlt::copy(cpu, device, ts_cpu.ppo.actor, ts_dev.ppo.actor);
    rlt::copy(cpu, device, ts_cpu.ppo.critic, ts_dev.ppo.critic);
    constexpr int ITERATIONS = 5;
    for(int iteration = 0; iteration < ITERATIONS; iteration++){
        const bool print = iteration == 0 || iteration == ITERATIONS - 1;
        rlt::collect(cpu, ts_cpu.on_policy_runner_dataset, ts_cpu.on_policy_runner, ts_cpu.ppo.actor, ts_cpu.actor_eval_buffers, ts_cpu.rng);
        rlt::copy(cpu, device, ts_cpu.on_policy_runner_dataset.data, ts_dev.on_policy_runner_dataset.data);
        values_and_advantages(cpu, ts_cpu);
        values_and_advantages(device, ts_dev);
        rlt::copy(device, cpu, ts_dev.on_policy_runner_dataset.data, back.on_policy_runner_dataset.data);
        if(print){ std::printf("iteration %d: mean |difference| / largest magnitude per tensor\ndataset:", iteration); }
        compare_column(back.on_policy_runner_dataset.all_values, ts_cpu.on_policy_runner_dataset.all_values, "values", print);
        compare_column(back.on_policy_runner_dataset.advantages, ts_cpu.on_policy_runner_dataset.advantages, "advantages", print);
        compare_column(back.on_policy_runner_dataset.target_values, ts_cpu.on_policy_runner_dataset.target_values, "target values", print);
        if(print){ std::printf("\n"); }
        rlt::train(cpu, ts_cpu.ppo, ts_cpu.on_policy_runner_dataset, ts_cpu.actor_optimizer, ts_cpu.critic_optimizer, ts_cpu.ppo_buffers, ts_cpu.actor_buffers, ts_cpu.critic_buffers, ts_cpu.rng);
        rlt::train(device, ts_dev.ppo, ts_dev.on_policy_runner_dataset, ts_dev.actor_optimizer, ts_dev.critic_optimizer, ts_dev.ppo_buffers, ts_dev.actor_buffers, ts_dev.critic_buffers, ts_dev.rng);
        rlt::copy(device, cpu, ts_dev.ppo.actor, back.ppo.actor);
        rlt::copy(device, cpu, ts_dev.ppo.critic, back.ppo.critic);
        compare_mlp(cpu, back.ppo.actor.next_module.content, ts_cpu.ppo.actor.next_module.content, "actor", print);
        compare(cpu, back.ppo.actor.next_module.content.log_std.parameters, ts_cpu.ppo.actor.next_module.content.log_std.parameters, "log_std", print);
        if(print){ std::printf("\n"); }
        compare_mlp(cpu, back.ppo.critic.next_module.content, ts_cpu.ppo.critic.next_module.content, "critic", print);
        if(print){ std::printf("\n"); }
    }
    rlt::check_status(device);
    std::printf("worst %.2e\n", worst);
    return worst <= 1e-5f ? 0 : 1;
}
