// The td3_sampling layer on devices::ROCM: evaluate, forward, backward_full (the reference's layer, nn/layers/td3_sampling/operations_generic.h:75-163,
// walks the rows on the host and draws its noise from the host generator one value at a time; its CUDA build has no counterpart, TD3 on CUDA stops at
// rl/algorithms/td3/operations_cuda.h). The reference's Tensor proxies (:187-240) reach these through matrix_view.
//
// action = clamp(mean + std * noise, -1, 1). Where the reference samples inside the layer (the Default and Rollout modes), the draws are made on the device
// into the layer buffer's noise matrix first; ExternalNoise takes what that matrix holds; Evaluation adds nothing.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/nn/layers/td3_sampling/layer.h>
#include <rl_tools/containers/matrix/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace nn::layers::td3_sampling::rocm{
        // the noise the step adds, or nullptr: drawn into buffer.noise unless given from outside (or overridden for a parity run, devices/rocm.h)
        template <typename DEVICE, typename BUFFER_SPEC, typename RNG, typename MODE>
        const float* noise(DEVICE& device, nn::layers::td3_sampling::Buffer<BUFFER_SPEC>& buffer, RNG& rng, const Mode<MODE>&, size_t rows, size_t dim){
            using NOISE = decltype(buffer.noise);
            static_assert(NOISE::SPEC::COL_PITCH == 1 && NOISE::SPEC::ROW_PITCH == NOISE::SPEC::COLS, "the noise rows lie back to back");
            if constexpr(rl_tools::mode::is<MODE, nn::layers::td3_sampling::mode::ExternalNoise>){ return buffer.noise._data; }
            else if constexpr(rl_tools::mode::is<MODE, rl_tools::mode::Evaluation>){ return nullptr; }
            else{
                static_assert(rl_tools::mode::is<MODE, rl_tools::mode::Default> || rl_tools::mode::is<MODE, rl_tools::mode::Rollout>, "td3_sampling: invalid mode");
                if(device.td3_sampling_noise_override){ return device.td3_sampling_noise_override; }
                devices::rocm::check(rlt_rocm_randn_f32(device.handle, buffer.noise._data, rows * dim, rng.seed, random::next_stream(rng)), "td3_sampling (noise)");
                return buffer.noise._data;
            }
        }
    }
    template <typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void evaluate(devices::ROCM<DEV_SPEC>& device, const nn::layers::td3_sampling::LayerForward<SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::td3_sampling::Buffer<BUFFER_SPEC>& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(INPUT_SPEC::COLS == SPEC::DIM && OUTPUT_SPEC::COLS == SPEC::DIM && INPUT_SPEC::ROWS == OUTPUT_SPEC::ROWS);
        static_assert(INPUT_SPEC::COL_PITCH == 1 && OUTPUT_SPEC::COL_PITCH == 1 && INPUT_SPEC::ROWS <= decltype(buffer.noise)::SPEC::ROWS);
        const float* noise = nn::layers::td3_sampling::rocm::noise(device, buffer, rng, mode, INPUT_SPEC::ROWS, SPEC::DIM);
        devices::rocm::check(rlt_rocm_td3_sampling_forward(device.handle, input._data, (int)INPUT_SPEC::ROW_PITCH, noise, (int)SPEC::DIM, (float)layer.std, nullptr, 0, output._data,
                                                           (int)OUTPUT_SPEC::ROW_PITCH, (int)INPUT_SPEC::ROWS, (int)SPEC::DIM), "evaluate(td3_sampling)");
    }
    template <typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::td3_sampling::LayerGradient<SPEC>& layer, const Matrix<INPUT_SPEC>& input, nn::layers::td3_sampling::Buffer<BUFFER_SPEC>& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        using OUT = decltype(layer.output); using PRE = decltype(layer.pre_clip);
        static_assert(INPUT_SPEC::COLS == SPEC::DIM && INPUT_SPEC::ROWS == OUT::SPEC::ROWS && INPUT_SPEC::COL_PITCH == 1 && INPUT_SPEC::ROWS <= decltype(buffer.noise)::SPEC::ROWS);
        const float* noise = nn::layers::td3_sampling::rocm::noise(device, buffer, rng, mode, INPUT_SPEC::ROWS, SPEC::DIM);
        devices::rocm::check(rlt_rocm_td3_sampling_forward(device.handle, input._data, (int)INPUT_SPEC::ROW_PITCH, noise, (int)SPEC::DIM, (float)layer.std, layer.pre_clip._data,
                                                           (int)PRE::SPEC::ROW_PITCH, layer.output._data, (int)OUT::SPEC::ROW_PITCH, (int)INPUT_SPEC::ROWS, (int)SPEC::DIM), "forward(td3_sampling)");
    }
    template <typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::td3_sampling::LayerGradient<SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::td3_sampling::Buffer<BUFFER_SPEC>& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        forward(device, layer, input, buffer, rng, mode);
        copy(device, device, layer.output, output);
    }
    // backward_full           :139-163: the gradient passes where the sample was not clipped
    template<typename DEV_SPEC, typename SPEC, typename INPUT_SPEC, typename D_OUTPUT_SPEC, typename D_INPUT_SPEC, typename BUFFER_SPEC, typename MODE = mode::Default<>>
    void backward_full(devices::ROCM<DEV_SPEC>& device, nn::layers::td3_sampling::LayerGradient<SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<D_OUTPUT_SPEC>& d_output, Matrix<D_INPUT_SPEC>& d_input, nn::layers::td3_sampling::Buffer<BUFFER_SPEC>& buffer, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        using PRE = decltype(layer.pre_clip);
        static_assert(D_OUTPUT_SPEC::COLS == SPEC::DIM && D_INPUT_SPEC::COLS == SPEC::DIM && D_OUTPUT_SPEC::ROWS == PRE::SPEC::ROWS && D_INPUT_SPEC::ROWS == PRE::SPEC::ROWS);
        static_assert(D_OUTPUT_SPEC::COL_PITCH == 1 && D_INPUT_SPEC::COL_PITCH == 1);
        devices::rocm::check(rlt_rocm_td3_sampling_backward(device.handle, layer.pre_clip._data, (int)PRE::SPEC::ROW_PITCH, d_output._data, (int)D_OUTPUT_SPEC::ROW_PITCH, d_input._data,
                                                            (int)D_INPUT_SPEC::ROW_PITCH, (int)PRE::SPEC::ROWS, (int)SPEC::DIM), "backward_full(td3_sampling)");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
