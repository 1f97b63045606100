// The sample_and_squash layer (tanh-Gaussian policy head with entropy bonus) on devices::ROCM: evaluate, forward, backward_full (the
// counterpart of nn/layers/sample_and_squash/operations_cuda.h:17-115). One launch each; the CUDA backend's backward_full needs a
// second, single-thread kernel to sum the per-sample log_alpha gradients, here the sum is part of the launch.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/nn/layers/sample_and_squash/layer.h>
#include <rl_tools/containers/matrix/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace nn::layers::sample_and_squash::rocm{
        template <typename SPEC>
        rlt_sas_parameters parameters(){
            using P = typename SPEC::PARAMETERS;
            return rlt_sas_parameters{(float)P::LOG_STD_LOWER_BOUND, (float)P::LOG_STD_UPPER_BOUND, (float)P::LOG_PROBABILITY_EPSILON, (float)P::TARGET_ENTROPY};
        }
        // where the noise of a pass comes from (sample_and_squash/operations_generic.h:159-176): the buffer as the caller filled it (ExternalNoise),
        // a fresh draw into the buffer (Default / Rollout), or none (Evaluation: the action is tanh(mean))
        template <typename DEVICE, typename BUFFER, typename RNG, typename MODE>
        const float* noise_for(DEVICE& device, BUFFER& buffer, RNG& rng, const Mode<MODE>&){
            if constexpr(rl_tools::mode::is<MODE, nn::layers::sample_and_squash::mode::ExternalNoise>){
                return buffer.noise._data;
            }
            else if constexpr(rl_tools::mode::is<MODE, rl_tools::mode::Evaluation>){
                return nullptr;
            }
            else{
                static_assert(rl_tools::mode::is<MODE, rl_tools::mode::Default> || rl_tools::mode::is<MODE, rl_tools::mode::Rollout>, "Invalid mode");
                randn(device, buffer.noise, rng);
                return buffer.noise._data;
            }
        }
    }
    // evaluate                sample_and_squash/operations_cuda.h:17-39: actions and log-probabilities (into the buffer)
    template <typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void evaluate(devices::ROCM<DEV_SPEC>& device, const nn::layers::sample_and_squash::LayerForward<SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::sample_and_squash::Buffer<BUFFER_SPEC>& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(INPUT_SPEC::COLS == 2 * SPEC::DIM && OUTPUT_SPEC::COLS == SPEC::DIM && INPUT_SPEC::ROWS == OUTPUT_SPEC::ROWS);
        static_assert(INPUT_SPEC::COL_PITCH == 1 && OUTPUT_SPEC::COL_PITCH == 1);
        static_assert(INPUT_SPEC::ROWS <= decltype(buffer.noise)::ROWS);
        const rlt_sas_parameters p = nn::layers::sample_and_squash::rocm::parameters<SPEC>();
        const float* noise = nn::layers::sample_and_squash::rocm::noise_for(device, buffer, rng, mode);
        devices::rocm::check(rlt_rocm_sas_forward(device.handle, &p, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, noise, containers::rocm::leading_dimension<typename decltype(buffer.noise)::SPEC>, output._data, containers::rocm::leading_dimension<OUTPUT_SPEC>, nullptr, 0,
                                                  buffer.log_probabilities._data, INPUT_SPEC::ROWS, SPEC::DIM), "evaluate(sample_and_squash)");
    }
    // forward                 sample_and_squash/operations_cuda.h:40-67: keeps noise, pre-squashing values, actions and log-probabilities in the layer
    template <typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::sample_and_squash::LayerGradient<SPEC>& layer, const Matrix<INPUT_SPEC>& input, nn::layers::sample_and_squash::Buffer<BUFFER_SPEC>& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(INPUT_SPEC::COLS == 2 * SPEC::DIM && INPUT_SPEC::ROWS == SPEC::INTERNAL_BATCH_SIZE && INPUT_SPEC::COL_PITCH == 1);
        const rlt_sas_parameters p = nn::layers::sample_and_squash::rocm::parameters<SPEC>();
        const float* noise = nn::layers::sample_and_squash::rocm::noise_for(device, buffer, rng, mode);
        if(noise){ copy(device, device, buffer.noise, layer.noise); } else { set_all(device, layer.noise, 0); }
        devices::rocm::check(rlt_rocm_sas_forward(device.handle, &p, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, noise ? layer.noise._data : nullptr, containers::rocm::leading_dimension<typename decltype(layer.noise)::SPEC>,
                                                  layer.output._data, containers::rocm::leading_dimension<typename decltype(layer.output)::SPEC>, layer.pre_squashing._data, containers::rocm::leading_dimension<typename decltype(layer.pre_squashing)::SPEC>,
                                                  layer.log_probabilities._data, INPUT_SPEC::ROWS, SPEC::DIM), "forward(sample_and_squash)");
    }
    template <typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::sample_and_squash::LayerGradient<SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::sample_and_squash::Buffer<BUFFER_SPEC>& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        forward(device, layer, input, buffer, rng, mode);
        copy(device, device, layer.output, output);
    }
    // backward_full           sample_and_squash/operations_cuda.h:68-115: d_input [batch x 2 dim], and the mean over the batch of the log_alpha gradient
    // added to layer.log_alpha.gradient
    template<typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename D_OUTPUT_SPEC, typename D_INPUT_SPEC, typename BUFFER_SPEC, typename MODE = mode::Default<>>
    void backward_full(devices::ROCM<DEV_SPEC>& device, nn::layers::sample_and_squash::LayerGradient<SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<D_OUTPUT_SPEC>& d_output, Matrix<D_INPUT_SPEC>& d_input, nn::layers::sample_and_squash::Buffer<BUFFER_SPEC>& buffer, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(INPUT_SPEC::COLS == 2 * SPEC::DIM && D_INPUT_SPEC::COLS == 2 * SPEC::DIM && D_OUTPUT_SPEC::COLS == SPEC::DIM && INPUT_SPEC::ROWS == SPEC::INTERNAL_BATCH_SIZE);
        static_assert(INPUT_SPEC::COL_PITCH == 1 && D_OUTPUT_SPEC::COL_PITCH == 1 && D_INPUT_SPEC::COL_PITCH == 1);
        static_assert(!mode::is<MODE, nn::layers::sample_and_squash::mode::DisableEntropy>, "the entropy term is part of the ROCM kernel");
        const rlt_sas_parameters p = nn::layers::sample_and_squash::rocm::parameters<SPEC>();
        devices::rocm::check(rlt_rocm_sas_backward(device.handle, &p, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, layer.noise._data, containers::rocm::leading_dimension<typename decltype(layer.noise)::SPEC>, layer.output._data, containers::rocm::leading_dimension<typename decltype(layer.output)::SPEC>,
                                                   layer.pre_squashing._data, containers::rocm::leading_dimension<typename decltype(layer.pre_squashing)::SPEC>, d_output._data, containers::rocm::leading_dimension<D_OUTPUT_SPEC>, d_input._data, containers::rocm::leading_dimension<D_INPUT_SPEC>,
                                                   layer.log_alpha.parameters._data, layer.log_alpha.gradient._data, INPUT_SPEC::ROWS, SPEC::DIM), "backward_full(sample_and_squash)");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
