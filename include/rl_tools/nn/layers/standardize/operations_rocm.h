// The standardize layer on devices::ROCM: set_statistics, evaluate / forward, backward_input (the counterpart of
// nn/layers/standardize/operations_cuda.h:13-156; the generic versions, operations_generic.h:54-120, are host loops over elements).
// backward is a no-op there (the layer has no trainable parameters) and needs no overload.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/nn/layers/standardize/layer.h>
#include <rl_tools/nn/layers/standardize/operations_generic.h>
#include <rl_tools/containers/matrix/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    // set_statistics          nn/layers/standardize/operations_generic.h:54-67: mean as given, precision = 1 / std (0 where std is 0)
    template<typename DEV_SPEC, typename LAYER_SPEC, typename MEAN_SPEC, typename STD_SPEC>
    void set_statistics(devices::ROCM<DEV_SPEC>& device, nn::layers::standardize::LayerForward<LAYER_SPEC>& layer, const Matrix<MEAN_SPEC>& mean, const Matrix<STD_SPEC>& std){
        static_assert(MEAN_SPEC::ROWS == 1 && STD_SPEC::ROWS == 1 && MEAN_SPEC::COLS == LAYER_SPEC::INPUT_DIM && STD_SPEC::COLS == LAYER_SPEC::INPUT_DIM);
        static_assert(utils::typing::is_same_v<typename MEAN_SPEC::T, float> && MEAN_SPEC::COL_PITCH == 1 && STD_SPEC::COL_PITCH == 1);
        devices::rocm::check(rlt_rocm_standardize_set_statistics(device.handle, mean._data, std._data, layer.mean.parameters._data, layer.precision.parameters._data, (int)LAYER_SPEC::INPUT_DIM), "set_statistics(standardize)");
    }
    // evaluate / forward      nn/layers/standardize/operations_generic.h:68-98
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename RNG, typename MODE = mode::Default<>>
    void evaluate(devices::ROCM<DEV_SPEC>& device, const nn::layers::standardize::LayerForward<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::standardize::Buffer& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::standardize::check_input_output<LAYER_SPEC, INPUT_SPEC, OUTPUT_SPEC>);
        static_assert(utils::typing::is_same_v<typename INPUT_SPEC::T, float> && INPUT_SPEC::COL_PITCH == 1 && OUTPUT_SPEC::COL_PITCH == 1);
        devices::rocm::check(rlt_rocm_standardize_forward(device.handle, layer.mean.parameters._data, layer.precision.parameters._data, input._data, containers::rocm::leading_dimension<INPUT_SPEC>,
                                                          output._data, containers::rocm::leading_dimension<OUTPUT_SPEC>, (int)INPUT_SPEC::ROWS, (int)LAYER_SPEC::INPUT_DIM), "evaluate(standardize)");
    }
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::standardize::LayerBackward<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::standardize::Buffer& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        evaluate(device, layer, input, output, buffer, rng, mode);
    }
    // backward_input          nn/layers/standardize/operations_generic.h:101-120
    template<typename DEV_SPEC, typename LAYER_SPEC, typename D_OUTPUT_SPEC, typename D_INPUT_SPEC, typename MODE = mode::Default<>>
    void backward_input(devices::ROCM<DEV_SPEC>& device, nn::layers::standardize::LayerBackward<LAYER_SPEC>& layer, const Matrix<D_OUTPUT_SPEC>& d_output, Matrix<D_INPUT_SPEC>& d_input, nn::layers::standardize::Buffer& buffer, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::standardize::check_input_output<LAYER_SPEC, D_INPUT_SPEC, D_OUTPUT_SPEC>);
        static_assert(utils::typing::is_same_v<typename D_OUTPUT_SPEC::T, float> && D_OUTPUT_SPEC::COL_PITCH == 1 && D_INPUT_SPEC::COL_PITCH == 1);
        devices::rocm::check(rlt_rocm_standardize_backward_input(device.handle, layer.precision.parameters._data, d_output._data, containers::rocm::leading_dimension<D_OUTPUT_SPEC>,
                                                                 d_input._data, containers::rocm::leading_dimension<D_INPUT_SPEC>, (int)D_OUTPUT_SPEC::ROWS, (int)LAYER_SPEC::INPUT_DIM), "backward_input(standardize)");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
