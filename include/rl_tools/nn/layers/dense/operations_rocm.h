// Dense layers on devices::ROCM: init_weights, evaluate, forward, backward_input, backward, backward_full (the counterpart of
// nn/layers/dense/operations_cuda.h:53-413). Each call is one launch of the per-layer contraction kernels behind the C ABI
// (fp32 MFMA tiles with bias, activation and the stores of pre-activations / outputs in the epilogue); the CUDA backend spends a
// bias kernel, a cuBLAS call, a copy and an activation kernel on the same work.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/containers/matrix/operations_rocm.h>
#include <rl_tools/nn/layers/dense/layer.h>
#include <rl_tools/containers/tensor/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace nn::layers::dense::rocm{
        // The C ABI's view of a layer (rlt_dense_layer): pointers into the layer's own tensors. Members a capability does not have stay NULL.
        template <typename LAYER>
        rlt_dense_layer describe_forward(const LAYER& layer){
            static_assert(utils::typing::is_same_v<typename decltype(layer.weights.parameters)::T, float>, "the ROCM backend computes in fp32");
            rlt_dense_layer d = {};
            d.weights = const_cast<float*>(layer.weights.parameters._data);
            d.biases = const_cast<float*>(layer.biases.parameters._data);
            d.in_dim = LAYER::INPUT_DIM; d.out_dim = LAYER::OUTPUT_DIM;
            d.activation = (int32_t)LAYER::SPEC::ACTIVATION_FUNCTION;        // rlt_activation keeps the numbering of nn/activation_functions.h:11-18
            return d;
        }
        template <typename SPEC>
        rlt_dense_layer describe(const nn::layers::dense::LayerForward<SPEC>& layer){ return describe_forward(layer); }
        template <typename SPEC>
        rlt_dense_layer describe(const nn::layers::dense::LayerBackward<SPEC>& layer){
            rlt_dense_layer d = describe_forward(layer);
            d.pre_activations = const_cast<float*>(layer.pre_activations._data);
            return d;
        }
        template <typename SPEC>
        rlt_dense_layer describe(const nn::layers::dense::LayerGradient<SPEC>& layer){
            rlt_dense_layer d = describe_forward(layer);
            d.pre_activations = const_cast<float*>(layer.pre_activations._data);
            d.output = const_cast<float*>(layer.output._data);
            d.d_weights = const_cast<float*>(layer.weights.gradient._data);
            d.d_biases = const_cast<float*>(layer.biases.gradient._data);
            return d;
        }
        template <typename SPEC>
        constexpr bool rows_contiguous = SPEC::COL_PITCH == 1 && utils::typing::is_same_v<utils::typing::remove_cv_t<typename SPEC::T>, float>;
    }
    // init_weights            nn/layers/dense/operations_generic.h:59-92, operations_cuda.h:53-68: uniform in +- bound, drawn on the device
    template<typename DEV_SPEC, typename SPEC, typename INITIALIZER_SPEC, typename RNG>
    void init_weights(devices::ROCM<DEV_SPEC>& device, nn::layers::dense::LayerForward<SPEC>& layer, const nn::layers::dense::KaimingUniform<INITIALIZER_SPEC>& initializer, RNG& rng){
        using T = typename SPEC::TYPE_POLICY::DEFAULT;
        T gain;
        if constexpr(INITIALIZER_SPEC::INIT_LEGACY){
            T negative_slope = math::sqrt(device.math, (T)5);
            gain = math::sqrt(device.math, (T)2.0 / (1 + negative_slope * negative_slope));
        }
        else{
            gain = math::sqrt(device.math, (T)2.0) * INITIALIZER_SPEC::SCALE;
        }
        T fan = SPEC::INPUT_DIM;
        T std = gain / math::sqrt(device.math, fan);
        T weight_bound = math::sqrt(device.math, (T)3.0) * std;
        T bias_bound = 1/math::sqrt(device.math, (T)SPEC::INPUT_DIM);
        if constexpr(INITIALIZER_SPEC::INIT_LEGACY){
            rand(device, layer.biases.parameters, rng, -bias_bound, bias_bound);
        }
        else{
            set_all(device, layer.biases.parameters, 0);
        }
        rand(device, layer.weights.parameters, rng, -weight_bound, weight_bound);
    }
    template<typename DEV_SPEC, typename SPEC, typename RNG>
    void init_weights(devices::ROCM<DEV_SPEC>& device, nn::layers::dense::LayerForward<SPEC>& layer, RNG& rng){
        init_weights(device, layer, typename SPEC::INITIALIZER{}, rng);
    }
    // evaluate                nn/layers/dense/operations_cuda.h:236-275
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename RNG, typename MODE = mode::Default<>>
    void evaluate(devices::ROCM<DEV_SPEC>& device, const nn::layers::dense::LayerForward<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::dense::Buffer&, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::dense::check_input_output<LAYER_SPEC, INPUT_SPEC, OUTPUT_SPEC>);
        static_assert(nn::layers::dense::rocm::rows_contiguous<INPUT_SPEC> && nn::layers::dense::rocm::rows_contiguous<OUTPUT_SPEC>);
        const rlt_dense_layer d = nn::layers::dense::rocm::describe_forward(layer);
        devices::rocm::check(rlt_rocm_dense_evaluate(device.handle, &d, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, output._data, containers::rocm::leading_dimension<OUTPUT_SPEC>, INPUT_SPEC::ROWS), "evaluate(dense)");
    }
    // forward                 nn/layers/dense/operations_cuda.h:276-316: also keeps the pre-activations
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::dense::LayerBackward<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::dense::Buffer& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::dense::check_input_output<LAYER_SPEC, INPUT_SPEC, OUTPUT_SPEC>);
        static_assert(nn::layers::dense::rocm::rows_contiguous<INPUT_SPEC> && nn::layers::dense::rocm::rows_contiguous<OUTPUT_SPEC>);
        static_assert(INPUT_SPEC::ROWS == LAYER_SPEC::INTERNAL_BATCH_SIZE);
        rlt_dense_layer d = nn::layers::dense::rocm::describe_forward(layer);
        d.pre_activations = layer.pre_activations._data;
        devices::rocm::check(rlt_rocm_dense_forward(device.handle, &d, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, output._data, containers::rocm::leading_dimension<OUTPUT_SPEC>, INPUT_SPEC::ROWS), "forward(dense)");
    }
    // forward into the layer's own output: one launch writes pre-activations and output (the generic route is forward + copy, operations_generic.h:132-144)
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::dense::LayerGradient<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, nn::layers::dense::Buffer& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::dense::rocm::rows_contiguous<INPUT_SPEC>);
        static_assert(INPUT_SPEC::ROWS == LAYER_SPEC::INTERNAL_BATCH_SIZE && INPUT_SPEC::COLS == LAYER_SPEC::INPUT_DIM);
        const rlt_dense_layer d = nn::layers::dense::rocm::describe(layer);
        devices::rocm::check(rlt_rocm_dense_forward(device.handle, &d, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, nullptr, 0, INPUT_SPEC::ROWS), "forward(dense)");
    }
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename RNG, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::dense::LayerGradient<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<OUTPUT_SPEC>& output, nn::layers::dense::Buffer& buffer, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::dense::check_input_output<LAYER_SPEC, INPUT_SPEC, OUTPUT_SPEC>);
        static_assert(nn::layers::dense::rocm::rows_contiguous<INPUT_SPEC> && nn::layers::dense::rocm::rows_contiguous<OUTPUT_SPEC>);
        const rlt_dense_layer d = nn::layers::dense::rocm::describe(layer);
        devices::rocm::check(rlt_rocm_dense_forward(device.handle, &d, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, output._data, containers::rocm::leading_dimension<OUTPUT_SPEC>, INPUT_SPEC::ROWS), "forward(dense)");
    }
    // backward_input          nn/layers/dense/operations_cuda.h:409-413: d_output becomes d_pre = act'(pre) * d_output in place (as in the
    // reference's BLAS and CUDA backends, which write through the const), d_input = d_pre W
    template<typename DEV_SPEC, typename LAYER_SPEC, typename D_OUTPUT_SPEC, typename D_INPUT_SPEC, typename MODE = mode::Default<>>
    void backward_input(devices::ROCM<DEV_SPEC>& device, const nn::layers::dense::LayerBackward<LAYER_SPEC>& layer, const Matrix<D_OUTPUT_SPEC>& d_output, Matrix<D_INPUT_SPEC>& d_input, nn::layers::dense::Buffer&, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::dense::check_input_output<LAYER_SPEC, D_INPUT_SPEC, D_OUTPUT_SPEC>);
        static_assert(nn::layers::dense::rocm::rows_contiguous<D_OUTPUT_SPEC> && nn::layers::dense::rocm::rows_contiguous<D_INPUT_SPEC>);
        rlt_dense_layer d = nn::layers::dense::rocm::describe_forward(layer);
        d.pre_activations = const_cast<float*>(layer.pre_activations._data);
        devices::rocm::check(rlt_rocm_dense_backward_input(device.handle, &d, const_cast<float*>(d_output._data), containers::rocm::leading_dimension<D_OUTPUT_SPEC>, d_input._data, containers::rocm::leading_dimension<D_INPUT_SPEC>, D_OUTPUT_SPEC::ROWS), "backward_input(dense)");
    }
    // backward                nn/layers/dense/operations_cuda.h:358-403: d_biases += column sums of d_pre, d_weights += d_pre^T input
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename D_OUTPUT_SPEC, typename MODE = mode::Default<>>
    void backward(devices::ROCM<DEV_SPEC>& device, nn::layers::dense::LayerGradient<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<D_OUTPUT_SPEC>& d_output, nn::layers::dense::Buffer&, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::dense::check_input_output<LAYER_SPEC, INPUT_SPEC, D_OUTPUT_SPEC>);
        static_assert(nn::layers::dense::rocm::rows_contiguous<INPUT_SPEC> && nn::layers::dense::rocm::rows_contiguous<D_OUTPUT_SPEC>);
        const rlt_dense_layer d = nn::layers::dense::rocm::describe(layer);
        devices::rocm::check(rlt_rocm_dense_backward(device.handle, &d, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, d_output._data, containers::rocm::leading_dimension<D_OUTPUT_SPEC>, INPUT_SPEC::ROWS), "backward(dense)");
    }
    // backward_full           nn/layers/dense/operations_cuda.h:404-408
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename D_OUTPUT_SPEC, typename D_INPUT_SPEC, typename MODE = mode::Default<>>
    void backward_full(devices::ROCM<DEV_SPEC>& device, nn::layers::dense::LayerGradient<LAYER_SPEC>& layer, const Matrix<INPUT_SPEC>& input, Matrix<D_OUTPUT_SPEC>& d_output, Matrix<D_INPUT_SPEC>& d_input, nn::layers::dense::Buffer& buffer, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::dense::check_input_output<LAYER_SPEC, INPUT_SPEC, D_OUTPUT_SPEC>);
        static_assert(nn::layers::dense::rocm::rows_contiguous<INPUT_SPEC> && nn::layers::dense::rocm::rows_contiguous<D_OUTPUT_SPEC> && nn::layers::dense::rocm::rows_contiguous<D_INPUT_SPEC>);
        const rlt_dense_layer d = nn::layers::dense::rocm::describe(layer);
        devices::rocm::check(rlt_rocm_dense_backward_full(device.handle, &d, input._data, containers::rocm::leading_dimension<INPUT_SPEC>, d_output._data, containers::rocm::leading_dimension<D_OUTPUT_SPEC>, d_input._data, containers::rocm::leading_dimension<D_INPUT_SPEC>, INPUT_SPEC::ROWS), "backward_full(dense)");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
