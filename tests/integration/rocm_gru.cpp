// A sequence model of the reference (GRU -> dense, nn_models::sequential, as its recurrent approximators are built:
// rl/algorithms/sac/loop/core/approximators_gru.h:9-75) on devices::ROCM next to the same model on the CPU device: identical weights
// (initialised on the CPU, copied over), identical inputs and output gradients, with and without per-step resets; forward, backward_full
// and an Adam step on both, compared on the host. Exit code 0 if outputs, input gradients, parameter gradients and updated parameters
// agree to 1e-4 relative to their largest magnitude. Then a rollout: evaluate_step of the model with the state a policy carries between environment steps
// (nn_models/sequential/operations_generic.h:303-327), for more steps than the sequence length so that rows restart by themselves, with a reset of some rows through
// a ResetMask on the way; every step's output next to the CPU device's.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/gru/operations_rocm.h>

#include <cmath>
#include <cstdio>

namespace rlt = rl_tools;
using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using DEVICE_CPU = rlt::devices::DEVICE_FACTORY<>;
using TI = DEVICE::index_t;
using T = float;
using TYPE_POLICY = rlt::numeric_types::Policy<T>;

constexpr TI SEQUENCE_LENGTH = 24, BATCH_SIZE = 40, INPUT_DIM = 11, HIDDEN_DIM = 32, OUTPUT_DIM = 3;
using INPUT_SHAPE = rlt::tensor::Shape<TI, SEQUENCE_LENGTH, BATCH_SIZE, INPUT_DIM>;
using GRU_CONFIG = rlt::nn::layers::gru::Configuration<TYPE_POLICY, TI, HIDDEN_DIM, rlt::nn::parameters::groups::Normal, false>;
using GRU = rlt::nn::layers::gru::BindConfiguration<GRU_CONFIG>;
using DENSE_CONFIG = rlt::nn::layers::dense::Configuration<TYPE_POLICY, TI, OUTPUT_DIM, rlt::nn::activation_functions::ActivationFunction::TANH, rlt::nn::layers::dense::DefaultInitializer<TYPE_POLICY, TI>, rlt::nn::parameters::groups::Output>;
using DENSE = rlt::nn::layers::dense::BindConfiguration<DENSE_CONFIG>;
template <typename T_CONTENT, typename T_NEXT_MODULE = rlt::nn_models::sequential::OutputModule>
using Module = typename rlt::nn_models::sequential::Module<T_CONTENT, T_NEXT_MODULE>;
using MODULE_CHAIN = Module<GRU, Module<DENSE>>;
using CAPABILITY = rlt::nn::capability::Gradient<rlt::nn::parameters::Adam>;
using MODEL = rlt::nn_models::sequential::Build<CAPABILITY, MODULE_CHAIN, INPUT_SHAPE>;
using OPTIMIZER = rlt::nn::optimizers::Adam<rlt::nn::optimizers::adam::Specification<TYPE_POLICY, TI>>;

int main(){
    DEVICE device; DEVICE_CPU cpu;
    rlt::init(device);
    DEVICE_CPU::SPEC::RANDOM::ENGINE<> rng_cpu;
    DEVICE::SPEC::RANDOM::ENGINE<> rng;
    rlt::malloc(device, rng); rlt::init(device, rng, 5);
    rlt::init(cpu, rng_cpu, 7);
    MODEL model_cpu, model_dev, model_back;
    MODEL::Buffer<> buffer_cpu, buffer_dev;
    OPTIMIZER optimizer_cpu, optimizer_dev;
    rlt::malloc(cpu, model_cpu); rlt::malloc(cpu, model_back); rlt::malloc(device, model_dev);
    rlt::malloc(cpu, buffer_cpu); rlt::malloc(device, buffer_dev);
    rlt::malloc(cpu, optimizer_cpu); rlt::malloc(device, optimizer_dev);
    rlt::init(cpu, optimizer_cpu); rlt::init(device, optimizer_dev);
    rlt::init_weights(cpu, model_cpu, rng_cpu);
    rlt::reset_optimizer_state(cpu, optimizer_cpu, model_cpu);
    rlt::copy(cpu, device, model_cpu, model_dev);
    rlt::reset_optimizer_state(device, optimizer_dev, model_dev);

    rlt::Tensor<rlt::tensor::Specification<T, TI, INPUT_SHAPE>> input_cpu, input_dev, d_input_cpu, d_input_dev, d_input_back;
    using OUTPUT_SHAPE = rlt::tensor::Shape<TI, SEQUENCE_LENGTH, BATCH_SIZE, OUTPUT_DIM>;
    rlt::Tensor<rlt::tensor::Specification<T, TI, OUTPUT_SHAPE>> d_output_cpu, d_output_dev, output_back, d_output_original;
    rlt::Tensor<rlt::tensor::Specification<bool, TI, rlt::tensor::Shape<TI, SEQUENCE_LENGTH, BATCH_SIZE, 1>>> reset_cpu, reset_dev;
    rlt::malloc(cpu, input_cpu); rlt::malloc(device, input_dev); rlt::malloc(cpu, d_input_cpu); rlt::malloc(device, d_input_dev); rlt::malloc(cpu, d_input_back);
    rlt::malloc(cpu, d_output_cpu); rlt::malloc(device, d_output_dev); rlt::malloc(cpu, output_back); rlt::malloc(cpu, d_output_original);
    rlt::malloc(cpu, reset_cpu); rlt::malloc(device, reset_dev);
    rlt::randn(cpu, input_cpu, rng_cpu);
    rlt::randn(cpu, d_output_original, rng_cpu);
    for(TI step = 0; step < SEQUENCE_LENGTH; step++){
        for(TI sample = 0; sample < BATCH_SIZE; sample++){
            rlt::set(cpu, reset_cpu, step == 0 || (step * 7 + sample * 3) % 11 == 0, step, sample, 0);
        }
    }
    rlt::copy(cpu, device, input_cpu, input_dev);
    rlt::copy(cpu, device, reset_cpu, reset_dev);

    T worst = 0;
    auto relative = [&](T difference_sum, T count, T scale){ return difference_sum / count / (scale > 0 ? scale : 1); };
    auto run = [&](auto& mode_cpu, auto& mode_dev, const char* name){
        rlt::copy(cpu, cpu, d_output_original, d_output_cpu);
        rlt::copy(cpu, device, d_output_original, d_output_dev);
        rlt::zero_gradient(cpu, model_cpu); rlt::zero_gradient(device, model_dev);
        rlt::forward(cpu, model_cpu, input_cpu, buffer_cpu, rng_cpu, mode_cpu);
        rlt::forward(device, model_dev, input_dev, buffer_dev, rng, mode_dev);
        auto output_cpu = rlt::output(cpu, model_cpu);
        auto output_dev = rlt::output(device, model_dev);
        rlt::copy(device, cpu, output_dev, output_back);
        const T e_output = relative(rlt::abs_diff(cpu, output_back, output_cpu), (T)(SEQUENCE_LENGTH * BATCH_SIZE * OUTPUT_DIM), rlt::abs_max(cpu, output_cpu));
        rlt::backward_full(cpu, model_cpu, input_cpu, d_output_cpu, d_input_cpu, buffer_cpu, mode_cpu);
        rlt::backward_full(device, model_dev, input_dev, d_output_dev, d_input_dev, buffer_dev, mode_dev);
        rlt::copy(device, cpu, d_input_dev, d_input_back);
        const T e_d_input = relative(rlt::abs_diff(cpu, d_input_back, d_input_cpu), (T)(SEQUENCE_LENGTH * BATCH_SIZE * INPUT_DIM), rlt::abs_max(cpu, d_input_cpu));
        rlt::copy(device, cpu, model_dev, model_back);
        auto& gru_cpu = model_cpu.content; auto& gru_back = model_back.content;
        const T e_dwi = relative(rlt::abs_diff(cpu, gru_back.weights_input.gradient, gru_cpu.weights_input.gradient), (T)(3 * HIDDEN_DIM * INPUT_DIM), rlt::abs_max(cpu, gru_cpu.weights_input.gradient));
        const T e_dwh = relative(rlt::abs_diff(cpu, gru_back.weights_hidden.gradient, gru_cpu.weights_hidden.gradient), (T)(3 * HIDDEN_DIM * HIDDEN_DIM), rlt::abs_max(cpu, gru_cpu.weights_hidden.gradient));
        const T e_dbi = relative(rlt::abs_diff(cpu, gru_back.biases_input.gradient, gru_cpu.biases_input.gradient), (T)(3 * HIDDEN_DIM), rlt::abs_max(cpu, gru_cpu.biases_input.gradient));
        const T e_dbh = relative(rlt::abs_diff(cpu, gru_back.biases_hidden.gradient, gru_cpu.biases_hidden.gradient), (T)(3 * HIDDEN_DIM), rlt::abs_max(cpu, gru_cpu.biases_hidden.gradient));
        rlt::step(cpu, optimizer_cpu, model_cpu);
        rlt::step(device, optimizer_dev, model_dev);
        rlt::copy(device, cpu, model_dev, model_back);
        const T e_wi = relative(rlt::abs_diff(cpu, gru_back.weights_input.parameters, gru_cpu.weights_input.parameters), (T)(3 * HIDDEN_DIM * INPUT_DIM), rlt::abs_max(cpu, gru_cpu.weights_input.parameters));
        const T e_wh = relative(rlt::abs_diff(cpu, gru_back.weights_hidden.parameters, gru_cpu.weights_hidden.parameters), (T)(3 * HIDDEN_DIM * HIDDEN_DIM), rlt::abs_max(cpu, gru_cpu.weights_hidden.parameters));
        std::printf("%s: mean |difference| / largest magnitude: output %.2e d_input %.2e dW_i %.2e dW_h %.2e db_i %.2e db_h %.2e W_i %.2e W_h %.2e\n", name, e_output, e_d_input, e_dwi, e_dwh, e_dbi, e_dbh, e_wi, e_wh);
        for(T e: {e_output, e_d_input, e_dwi, e_dwh, e_dbi, e_dbh, e_wi, e_wh}){ worst = (std::isnan(e) || e > worst) ? (std::isnan(e) ? 1 : e) : worst; }
    };
    {
        rlt::Mode<rlt::mode::Default<>> mode;
        run(mode, mode, "whole sequences");
    }
    {
        // (the index type of the specification has to be the device's: the reference's reset_sample overload for ResetMode takes MODE_SPEC::TI, and
        // with another type the call resolves to the overload that never resets, nn/layers/gru/operations_generic.h:205-212)
        rlt::Mode<rlt::nn::layers::gru::ResetMode<rlt::mode::Default<>, rlt::nn::layers::gru::ResetModeSpecification<DEVICE_CPU::index_t, decltype(reset_cpu)>>> mode_cpu;
        rlt::Mode<rlt::nn::layers::gru::ResetMode<rlt::mode::Default<>, rlt::nn::layers::gru::ResetModeSpecification<TI, decltype(reset_dev)>>> mode_dev;
        mode_cpu.reset_container = reset_cpu; mode_dev.reset_container = reset_dev;
        run(mode_cpu, mode_dev, "with per-step resets");
    }
    {
        MODEL::State<> state_cpu, state_dev;
        rlt::malloc(cpu, state_cpu); rlt::malloc(device, state_dev);
        rlt::Mode<rlt::mode::Evaluation<>> mode;
        rlt::reset(cpu, model_cpu, state_cpu, rng_cpu);
        rlt::reset(device, model_dev, state_dev, rng);
        rlt::Tensor<rlt::tensor::Specification<T, TI, rlt::tensor::Shape<TI, BATCH_SIZE, INPUT_DIM>>> step_input_cpu, step_input_dev;
        rlt::Tensor<rlt::tensor::Specification<T, TI, rlt::tensor::Shape<TI, BATCH_SIZE, OUTPUT_DIM>>> step_output_cpu, step_output_dev, step_output_back;
        rlt::Matrix<rlt::matrix::Specification<bool, TI, 1, BATCH_SIZE>> mask_cpu, mask_dev;
        rlt::malloc(cpu, step_input_cpu); rlt::malloc(device, step_input_dev); rlt::malloc(cpu, step_output_cpu); rlt::malloc(device, step_output_dev); rlt::malloc(cpu, step_output_back);
        rlt::malloc(cpu, mask_cpu); rlt::malloc(device, mask_dev);
        T e_rollout = 0;
        for(TI step = 0; step < 2 * SEQUENCE_LENGTH + 5; step++){
            if(step == 9){      // some environments start a new episode: their rows of the state start again
                for(TI sample = 0; sample < BATCH_SIZE; sample++){ rlt::set(mask_cpu, 0, sample, sample % 3 == 1); }
                rlt::copy(cpu, device, mask_cpu, mask_dev);
                rlt::Mode<rlt::mode::sequential::ResetMask<rlt::mode::Default<>, rlt::mode::sequential::ResetMaskSpecification<decltype(mask_cpu)>>> reset_cpu_mode;
                rlt::Mode<rlt::mode::sequential::ResetMask<rlt::mode::Default<>, rlt::mode::sequential::ResetMaskSpecification<decltype(mask_dev)>>> reset_dev_mode;
                reset_cpu_mode.mask = mask_cpu; reset_dev_mode.mask = mask_dev;
                rlt::reset(cpu, model_cpu, state_cpu, rng_cpu, reset_cpu_mode);
                rlt::reset(device, model_dev, state_dev, rng, reset_dev_mode);
            }
            rlt::randn(cpu, step_input_cpu, rng_cpu);
            rlt::copy(cpu, device, step_input_cpu, step_input_dev);
            rlt::evaluate_step(cpu, model_cpu, step_input_cpu, state_cpu, step_output_cpu, buffer_cpu, rng_cpu, mode);
            rlt::evaluate_step(device, model_dev, step_input_dev, state_dev, step_output_dev, buffer_dev, rng, mode);
            rlt::copy(device, cpu, step_output_dev, step_output_back);
            const T e = relative(rlt::abs_diff(cpu, step_output_back, step_output_cpu), (T)(BATCH_SIZE * OUTPUT_DIM), rlt::abs_max(cpu, step_output_cpu));
            e_rollout = (std::isnan(e) || e > e_rollout) ? (std::isnan(e) ? 1 : e) : e_rollout;
        }
        std::printf("rollout of %u steps (evaluate_step): worst mean |difference| / largest magnitude of a step's output %.2e\n", (unsigned)(2 * SEQUENCE_LENGTH + 5), e_rollout);
        worst = e_rollout > worst ? e_rollout : worst;
    }
    rlt::check_status(device);
    std::printf("worst %.2e\n", worst);
    return worst <= 1e-4f ? 0 : 1;
}
