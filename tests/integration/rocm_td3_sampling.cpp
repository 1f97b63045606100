// The td3_sampling layer of the reference behind a dense layer (nn_models::sequential, as TD3's actor is built: rl/algorithms/td3/loop/core/approximators_mlp.h:15-31)
// on devices::ROCM next to the same model on the CPU device: identical weights, inputs, output gradients and -- through the layer's ExternalNoise mode -- identical
// noise, with a noise scale large enough that a third of the samples are clipped; forward, backward_full, and evaluate in Evaluation mode. In the Default mode, where
// the layer draws its own noise, the device's output is checked against clamp(mean + std * noise) for the noise it left in the buffer. Exit code 0 if outputs, input
// gradients and the dense layer's parameter gradients agree to 1e-5 relative to their largest magnitude.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/td3_sampling/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/nn/operations_rocm.h>
#include <rl_tools/nn/layers/td3_sampling/operations_rocm.h>

#include <cmath>
#include <cstdio>

namespace rlt = rl_tools;
using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using DEVICE_CPU = rlt::devices::DEVICE_FACTORY<>;
using TI = DEVICE::index_t;
using T = float;
using TYPE_POLICY = rlt::numeric_types::Policy<T>;

constexpr TI BATCH_SIZE = 200, INPUT_DIM = 5, ACTION_DIM = 3;
using INPUT_SHAPE = rlt::tensor::Shape<TI, 1, BATCH_SIZE, INPUT_DIM>;
using DENSE_CONFIG = rlt::nn::layers::dense::Configuration<TYPE_POLICY, TI, ACTION_DIM, rlt::nn::activation_functions::ActivationFunction::TANH, rlt::nn::layers::dense::DefaultInitializer<TYPE_POLICY, TI>, rlt::nn::parameters::groups::Output>;
using DENSE = rlt::nn::layers::dense::BindConfiguration<DENSE_CONFIG>;
struct SAMPLING_PARAMETERS{ static constexpr T STD = 0.8; };
using SAMPLING_CONFIG = rlt::nn::layers::td3_sampling::Configuration<TYPE_POLICY, TI, SAMPLING_PARAMETERS>;
using SAMPLING = rlt::nn::layers::td3_sampling::BindConfiguration<SAMPLING_CONFIG>;
template <typename T_CONTENT, typename T_NEXT_MODULE = rlt::nn_models::sequential::OutputModule>
using Module = typename rlt::nn_models::sequential::Module<T_CONTENT, T_NEXT_MODULE>;
using CAPABILITY = rlt::nn::capability::Gradient<rlt::nn::parameters::Adam>;
using MODEL = rlt::nn_models::sequential::Build<CAPABILITY, Module<DENSE, Module<SAMPLING>>, INPUT_SHAPE>;

int main(){
    DEVICE device; DEVICE_CPU cpu;
    rlt::init(device);
    DEVICE_CPU::SPEC::RANDOM::ENGINE<> rng_cpu;
    DEVICE::SPEC::RANDOM::ENGINE<> rng;
    rlt::malloc(device, rng); rlt::init(device, rng, 5);
    rlt::init(cpu, rng_cpu, 7);
    MODEL model_cpu, model_dev, model_back;
    MODEL::Buffer<> buffer_cpu, buffer_dev, buffer_back;
    rlt::malloc(cpu, model_cpu); rlt::malloc(cpu, model_back); rlt::malloc(device, model_dev);
    rlt::malloc(cpu, buffer_cpu); rlt::malloc(device, buffer_dev); rlt::malloc(cpu, buffer_back);
    rlt::init_weights(cpu, model_cpu, rng_cpu);
    rlt::copy(cpu, device, model_cpu, model_dev);
    using OUTPUT_SHAPE = rlt::tensor::Shape<TI, 1, BATCH_SIZE, ACTION_DIM>;
    rlt::Tensor<rlt::tensor::Specification<T, TI, INPUT_SHAPE>> input_cpu, input_dev, d_input_cpu, d_input_dev, d_input_back;
    rlt::Tensor<rlt::tensor::Specification<T, TI, OUTPUT_SHAPE>> d_output_cpu, d_output_dev, output_cpu, output_dev, output_back;
    rlt::malloc(cpu, input_cpu); rlt::malloc(device, input_dev); rlt::malloc(cpu, d_input_cpu); rlt::malloc(device, d_input_dev); rlt::malloc(cpu, d_input_back);
    rlt::malloc(cpu, d_output_cpu); rlt::malloc(device, d_output_dev); rlt::malloc(cpu, output_cpu); rlt::malloc(device, output_dev); rlt::malloc(cpu, output_back);
    rlt::randn(cpu, input_cpu, rng_cpu); rlt::randn(cpu, d_output_cpu, rng_cpu);
    rlt::copy(cpu, device, input_cpu, input_dev); rlt::copy(cpu, device, d_output_cpu, d_output_dev);
    auto& noise_cpu = rlt::get_last_buffer(buffer_cpu).noise; auto& noise_dev = rlt::get_last_buffer(buffer_dev).noise; auto& noise_back = rlt::get_last_buffer(buffer_back).noise;
    rlt::randn(cpu, noise_cpu, rng_cpu);
    rlt::copy(cpu, device, noise_cpu, noise_dev);

    T worst = 0;
    auto note = [&](const char* what, T difference_sum, T count, T scale){
        const T e = difference_sum / count / (scale > 0 ? scale : 1);
        std::printf("  %s %.2e", what, e);
        worst = (std::isnan(e) || e > worst) ? (std::isnan(e) ? 1 : e) : worst;
    };
    {
        std::printf("external noise:");
        rlt::Mode<rlt::nn::layers::td3_sampling::mode::ExternalNoise<rlt::mode::Default<>>> mode;
        rlt::zero_gradient(cpu, model_cpu); rlt::zero_gradient(device, model_dev);
        rlt::forward(cpu, model_cpu, input_cpu, output_cpu, buffer_cpu, rng_cpu, mode);
        rlt::forward(device, model_dev, input_dev, output_dev, buffer_dev, rng, mode);
        rlt::copy(device, cpu, output_dev, output_back);
        note("output", rlt::abs_diff(cpu, output_back, output_cpu), (T)(BATCH_SIZE * ACTION_DIM), rlt::abs_max(cpu, output_cpu));
        TI clipped = 0;
        for(TI row = 0; row < BATCH_SIZE; row++){ for(TI col = 0; col < ACTION_DIM; col++){ clipped += std::fabs(rlt::get(cpu, output_cpu, 0, row, col)) == 1 ? 1 : 0; } }
        std::printf("  (%u of %u samples clipped)", (unsigned)clipped, (unsigned)(BATCH_SIZE * ACTION_DIM));
        if(clipped < BATCH_SIZE * ACTION_DIM / 10){ worst = 1; }
        rlt::backward_full(cpu, model_cpu, input_cpu, d_output_cpu, d_input_cpu, buffer_cpu, mode);
        rlt::backward_full(device, model_dev, input_dev, d_output_dev, d_input_dev, buffer_dev, mode);
        rlt::copy(device, cpu, d_input_dev, d_input_back);
        note("d_input", rlt::abs_diff(cpu, d_input_back, d_input_cpu), (T)(BATCH_SIZE * INPUT_DIM), rlt::abs_max(cpu, d_input_cpu));
        rlt::copy(device, cpu, model_dev, model_back);
        note("dW", rlt::abs_diff(cpu, model_back.content.weights.gradient, model_cpu.content.weights.gradient), (T)(ACTION_DIM * INPUT_DIM), rlt::abs_max(cpu, model_cpu.content.weights.gradient));
        note("db", rlt::abs_diff(cpu, model_back.content.biases.gradient, model_cpu.content.biases.gradient), (T)ACTION_DIM, rlt::abs_max(cpu, model_cpu.content.biases.gradient));
        std::printf("\n");
    }
    {
        std::printf("evaluation mode:");
        rlt::Mode<rlt::mode::Evaluation<>> mode;
        rlt::evaluate(cpu, model_cpu, input_cpu, output_cpu, buffer_cpu, rng_cpu, mode);
        rlt::evaluate(device, model_dev, input_dev, output_dev, buffer_dev, rng, mode);
        rlt::copy(device, cpu, output_dev, output_back);
        note("output", rlt::abs_diff(cpu, output_back, output_cpu), (T)(BATCH_SIZE * ACTION_DIM), rlt::abs_max(cpu, output_cpu));
        std::printf("\n");
    }
    {
        // the layer draws: the output must be clamp(mean + std * noise) for the noise the device left in the buffer, and that noise must be new
        std::printf("default mode (noise drawn on the device):");
        rlt::Mode<rlt::mode::Default<>> mode;
        rlt::evaluate(device, model_dev, input_dev, output_dev, buffer_dev, rng, mode);
        rlt::copy(device, cpu, output_dev, output_back);
        rlt::copy(device, cpu, noise_dev, noise_back);
        T difference = 0, moved = 0;
        for(TI row = 0; row < BATCH_SIZE; row++){
            for(TI col = 0; col < ACTION_DIM; col++){
                const T mean = rlt::get(cpu, output_cpu, 0, row, col);        // the Evaluation-mode output: the dense layer's tanh
                T expected = mean + SAMPLING_PARAMETERS::STD * rlt::get(noise_back, row, col);
                expected = expected < -1 ? -1 : (expected > 1 ? 1 : expected);
                difference += std::fabs(expected - rlt::get(cpu, output_back, 0, row, col));
                moved += std::fabs(rlt::get(noise_back, row, col) - rlt::get(noise_cpu, row, col));
            }
        }
        note("output", difference, (T)(BATCH_SIZE * ACTION_DIM), 1);
        std::printf("  (mean |noise - the external noise| %.2f)\n", moved / (BATCH_SIZE * ACTION_DIM));
        if(moved / (BATCH_SIZE * ACTION_DIM) < 0.5f){ worst = 1; }
    }
    rlt::check_status(device);
    std::printf("worst %.2e\n", worst);
    return worst <= 1e-5f ? 0 : 1;
}
