// GRU layers on devices::ROCM: evaluate, forward, backward, backward_full, backward_input over whole sequences (the counterpart of
// nn/layers/gru/operations_cuda.h, helper_operations_cuda.h:14-240; the generic versions, nn/layers/gru/operations_generic.h:231-341 and
// :594-795, walk the sequence on the host with 3-4 matrix products and several element-wise operations per step). Here a pass over the
// sequence is one call of the library (rlt_rocm_gru_forward / rlt_rocm_gru_backward: the input projection of all steps as one matrix
// product, the recurrence in one launch, the weight gradients as matrix products over all steps).
//
// A rollout step (evaluate_step with the State a policy carries from one environment step to the next, and reset of that State) is one call of the library too
// (rlt_rocm_seq_evaluate_step / rlt_rocm_seq_reset_state on a one-layer description); the generic versions (:87-120, :348-416) loop over the batch rows on the host.
//
// malloc / free / init_weights / zero_gradient / update / copy are the generic functions over this backend's container and optimiser
// overloads. LEARN_INITIAL_HIDDEN_STATE = false (the reference's configuration, nn/layers/gru/layer.h:14-24).
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/nn/layers/gru/layer.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/containers/tensor/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace nn::layers::gru::rocm{
        template <typename SPEC>
        rlt_gru_layer describe_forward(const nn::layers::gru::LayerForward<SPEC>& layer){
            static_assert(utils::typing::is_same_v<typename SPEC::TYPE_POLICY::DEFAULT, float>, "the ROCM backend computes in fp32");
            rlt_gru_layer d = {};
            d.weights_input = layer.weights_input.parameters._data; d.biases_input = layer.biases_input.parameters._data;
            d.weights_hidden = layer.weights_hidden.parameters._data; d.biases_hidden = layer.biases_hidden.parameters._data;
            d.initial_hidden_state = layer.initial_hidden_state.parameters._data;
            d.input_dim = SPEC::INPUT_DIM; d.hidden_dim = SPEC::HIDDEN_DIM; d.fast_tanh = SPEC::FAST_TANH ? 1 : 0;
            return d;
        }
        template <typename SPEC>
        rlt_gru_layer describe(nn::layers::gru::LayerGradient<SPEC>& layer){
            rlt_gru_layer d = describe_forward(layer);
            d.d_weights_input = layer.weights_input.gradient._data; d.d_biases_input = layer.biases_input.gradient._data;
            d.d_weights_hidden = layer.weights_hidden.gradient._data; d.d_biases_hidden = layer.biases_hidden.gradient._data;
            d.post_activation = layer.post_activation._data; d.n_pre_pre_activation = layer.n_pre_pre_activation._data; d.output = layer.output._data;
            return d;
        }
        // the per-step reset flags of a ResetMode (nn/layers/gru/layer.h:56-68), or NULL: every sequence starts at step 0 only
        template <typename MODE, typename MODE_SPEC>
        const uint8_t* reset_flags(const Mode<nn::layers::gru::ResetMode<MODE, MODE_SPEC>>& mode){
            using CONTAINER = utils::typing::remove_reference_t<decltype(mode.reset_container)>;
            static_assert(sizeof(typename CONTAINER::T) == 1 && tensor::dense_row_major_layout<typename CONTAINER::SPEC>(), "the reset flags are one byte per (step, sample), dense");
            return (const uint8_t*)mode.reset_container._data;
        }
        template <typename MODE>
        const uint8_t* reset_flags(const Mode<MODE>&){ return nullptr; }
        template <typename SPEC>
        constexpr bool dense(){ return tensor::dense_row_major_layout<SPEC>(); }
    }
    // evaluate                nn/layers/gru/operations_generic.h:342-347: the intermediates of the steps go to scratch memory
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename OUTPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void evaluate(devices::ROCM<DEV_SPEC>& device, const nn::layers::gru::LayerForward<LAYER_SPEC>& layer, const Tensor<INPUT_SPEC>& input, Tensor<OUTPUT_SPEC>& output, nn::layers::gru::buffers::Evaluation<BUFFER_SPEC>& buffers, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::gru::check_input_output<LAYER_SPEC, INPUT_SPEC, OUTPUT_SPEC>, "Input and output spec not matching");
        static_assert(nn::layers::gru::rocm::dense<INPUT_SPEC>() && nn::layers::gru::rocm::dense<OUTPUT_SPEC>(), "sequences are dense [steps x batch x features] tensors");
        constexpr size_t S = get<0>(typename INPUT_SPEC::SHAPE{}), B = get<1>(typename INPUT_SPEC::SHAPE{}), H = LAYER_SPEC::HIDDEN_DIM;
        rlt_gru_layer d = nn::layers::gru::rocm::describe_forward(layer);
        d.output = output._data;
        const size_t workspace_bytes = rlt_rocm_gru_workspace_bytes(&d, (int)S, (int)B), post_bytes = (S * B * 3 * H * sizeof(float) + 255) / 256 * 256, pre_bytes = (S * B * H * sizeof(float) + 255) / 256 * 256;
        char* memory = (char*)devices::rocm::scratch(device, post_bytes + pre_bytes + workspace_bytes);
        d.post_activation = (float*)memory; d.n_pre_pre_activation = (float*)(memory + post_bytes);
        devices::rocm::check(rlt_rocm_gru_forward(device.handle, &d, input._data, nn::layers::gru::rocm::reset_flags(mode), (int)S, (int)B, memory + post_bytes + pre_bytes, workspace_bytes), "evaluate(gru)");
    }
    // forward                 nn/layers/gru/operations_generic.h:418-421: keeps the intermediates in the layer
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename RNG, typename BUFFER_SPEC, typename MODE = mode::Default<>>
    void forward(devices::ROCM<DEV_SPEC>& device, nn::layers::gru::LayerGradient<LAYER_SPEC>& layer, const Tensor<INPUT_SPEC>& input, nn::layers::gru::buffers::Evaluation<BUFFER_SPEC>& buffers, RNG& rng, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::gru::rocm::dense<INPUT_SPEC>(), "sequences are dense [steps x batch x features] tensors");
        constexpr size_t S = get<0>(typename INPUT_SPEC::SHAPE{}), B = get<1>(typename INPUT_SPEC::SHAPE{});
        static_assert(S == LAYER_SPEC::SEQUENCE_LENGTH && get<2>(typename INPUT_SPEC::SHAPE{}) == LAYER_SPEC::INPUT_DIM);
        const rlt_gru_layer d = nn::layers::gru::rocm::describe(layer);
        const size_t workspace_bytes = rlt_rocm_gru_workspace_bytes(&d, (int)S, (int)B);
        void* workspace = devices::rocm::scratch(device, workspace_bytes);
        devices::rocm::check(rlt_rocm_gru_forward(device.handle, &d, input._data, nn::layers::gru::rocm::reset_flags(mode), (int)S, (int)B, workspace, workspace_bytes), "forward(gru)");
    }
    namespace nn::layers::gru::rocm{
        template<typename DEVICE, typename LAYER_SPEC, typename MODE>
        void backward(DEVICE& device, nn::layers::gru::LayerGradient<LAYER_SPEC>& layer, const float* input, float* d_output, float* d_input, size_t S, size_t B, bool weight_gradients, const Mode<MODE>& mode, const char* what){
            const rlt_gru_layer d = describe(layer);
            const size_t workspace_bytes = rlt_rocm_gru_workspace_bytes(&d, (int)S, (int)B);
            void* workspace = devices::rocm::scratch(device, workspace_bytes);
            devices::rocm::check(rlt_rocm_gru_backward(device.handle, &d, input, d_output, d_input, reset_flags(mode), (int)S, (int)B, weight_gradients ? 1 : 0, workspace, workspace_bytes), what);
        }
    }
    // backward_full / backward / backward_input through time   nn/layers/gru/operations_generic.h:771-795. d_output is modified, as in the
    // reference (the gradient that flows back through the hidden state is accumulated into it).
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename D_OUTPUT_SPEC, typename D_INPUT_SPEC, typename BUFFER_SPEC, typename MODE = mode::Default<>>
    void backward_full(devices::ROCM<DEV_SPEC>& device, nn::layers::gru::LayerGradient<LAYER_SPEC>& layer, const Tensor<INPUT_SPEC>& input, Tensor<D_OUTPUT_SPEC>& d_output, Tensor<D_INPUT_SPEC>& d_input, nn::layers::gru::buffers::Backward<BUFFER_SPEC>& buffers, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::gru::rocm::dense<INPUT_SPEC>() && nn::layers::gru::rocm::dense<D_OUTPUT_SPEC>() && nn::layers::gru::rocm::dense<D_INPUT_SPEC>(), "sequences are dense [steps x batch x features] tensors");
        nn::layers::gru::rocm::backward(device, layer, input._data, d_output._data, d_input._data, get<0>(typename INPUT_SPEC::SHAPE{}), get<1>(typename INPUT_SPEC::SHAPE{}), true, mode, "backward_full(gru)");
    }
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename D_OUTPUT_SPEC, typename BUFFER_SPEC, typename MODE = mode::Default<>>
    void backward(devices::ROCM<DEV_SPEC>& device, nn::layers::gru::LayerGradient<LAYER_SPEC>& layer, const Tensor<INPUT_SPEC>& input, Tensor<D_OUTPUT_SPEC>& d_output, nn::layers::gru::buffers::Backward<BUFFER_SPEC>& buffers, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::gru::rocm::dense<INPUT_SPEC>() && nn::layers::gru::rocm::dense<D_OUTPUT_SPEC>(), "sequences are dense [steps x batch x features] tensors");
        nn::layers::gru::rocm::backward(device, layer, input._data, d_output._data, nullptr, get<0>(typename INPUT_SPEC::SHAPE{}), get<1>(typename INPUT_SPEC::SHAPE{}), true, mode, "backward(gru)");
    }
    template<typename DEV_SPEC, typename LAYER_SPEC, typename D_OUTPUT_SPEC, typename D_INPUT_SPEC, typename BUFFER_SPEC, typename MODE = mode::Default<>>
    void backward_input(devices::ROCM<DEV_SPEC>& device, nn::layers::gru::LayerGradient<LAYER_SPEC>& layer, Tensor<D_OUTPUT_SPEC>& d_output, Tensor<D_INPUT_SPEC>& d_input, nn::layers::gru::buffers::Backward<BUFFER_SPEC>& buffers, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(nn::layers::gru::rocm::dense<D_OUTPUT_SPEC>() && nn::layers::gru::rocm::dense<D_INPUT_SPEC>(), "sequences are dense [steps x batch x features] tensors");
        nn::layers::gru::rocm::backward(device, layer, nullptr, d_output._data, d_input._data, get<0>(typename D_INPUT_SPEC::SHAPE{}), get<1>(typename D_INPUT_SPEC::SHAPE{}), false, mode, "backward_input(gru)");
    }
    // reset(layer, state)     nn/layers/gru/operations_generic.h:87-120: all rows (Default mode) or the rows of a ResetMask start again from the initial hidden state, step 0
    template<typename DEV_SPEC, typename SPEC, typename STATE_SPEC, typename RNG, typename MODE = mode::Default<>>
    void reset(devices::ROCM<DEV_SPEC>& device, const nn::layers::gru::LayerForward<SPEC>& layer, nn::layers::gru::State<STATE_SPEC>& state, RNG&, Mode<MODE> mode = Mode<mode::Default<>>{}){
        constexpr size_t B = get<0>(typename decltype(state.state)::SPEC::SHAPE{});
        static_assert(sizeof(typename decltype(state.step)::T) == 4, "the step counters of a GRU state are 32-bit on devices::ROCM");
        rlt_seq_layer l = {}; l.kind = 1; l.gru = nn::layers::gru::rocm::describe_forward(layer);
        rlt_seq_state s = {}; s.hidden[0] = state.state._data; s.step[0] = (uint32_t*)state.step._data;
        const uint8_t* mask = nullptr;
        if constexpr(mode::is<MODE, mode::sequential::ResetMask>){
            static_assert(sizeof(typename decltype(mode.mask)::T) == 1 && decltype(mode.mask)::ROWS == 1 && decltype(mode.mask)::COLS == B && decltype(mode.mask)::SPEC::COL_PITCH == 1, "the reset mask is one byte per batch row");
            mask = (const uint8_t*)mode.mask._data;
        }
        else{
            static_assert(mode::is<MODE, mode::Default>, "reset(gru state): Default mode or a ResetMask");
        }
        devices::rocm::check(rlt_rocm_seq_reset_state(device.handle, &l, 1, &s, mask, (int)B), "reset(gru state)");
    }
    // evaluate_step           nn/layers/gru/operations_generic.h:348-416: one step of the recurrence on the state's rows; rows that have run SEQUENCE_LENGTH steps start
    //                         again from the initial hidden state (before the step and after it), unless the mode is NoAutoResetMode
    template<typename DEV_SPEC, typename LAYER_SPEC, typename INPUT_SPEC, typename STATE_SPEC, typename OUTPUT_SPEC, typename BUFFER_SPEC, typename RNG, typename MODE = mode::Default<>>
    void evaluate_step(devices::ROCM<DEV_SPEC>& device, const nn::layers::gru::LayerForward<LAYER_SPEC>& layer, const Tensor<INPUT_SPEC>& input, nn::layers::gru::State<STATE_SPEC>& state, Tensor<OUTPUT_SPEC>& output, nn::layers::gru::buffers::Evaluation<BUFFER_SPEC>&, RNG&, const Mode<MODE>& mode = Mode<mode::Default<>>{}){
        static_assert(length(typename INPUT_SPEC::SHAPE{}) == 2 && length(typename OUTPUT_SPEC::SHAPE{}) == 2, "evaluate_step has no sequence dimension (batch x features)");
        static_assert(nn::layers::gru::rocm::dense<INPUT_SPEC>() && nn::layers::gru::rocm::dense<OUTPUT_SPEC>());
        static_assert(sizeof(typename decltype(state.step)::T) == 4, "the step counters of a GRU state are 32-bit on devices::ROCM");
        constexpr size_t B = get<0>(typename INPUT_SPEC::SHAPE{});
        static_assert(get<1>(typename INPUT_SPEC::SHAPE{}) == LAYER_SPEC::INPUT_DIM && get<0>(typename OUTPUT_SPEC::SHAPE{}) == B && get<1>(typename OUTPUT_SPEC::SHAPE{}) == LAYER_SPEC::HIDDEN_DIM);
        rlt_seq_layer l = {}; l.kind = 1; l.gru = nn::layers::gru::rocm::describe_forward(layer);
        rlt_seq_state s = {}; s.hidden[0] = state.state._data; s.step[0] = (uint32_t*)state.step._data;
        const int auto_reset_period = mode::is<MODE, nn::layers::gru::NoAutoResetMode> ? 0 : (int)LAYER_SPEC::SEQUENCE_LENGTH;
        const size_t workspace_bytes = rlt_rocm_seq_evaluate_step_workspace_bytes(&l, 1, (int)B);
        void* workspace = devices::rocm::scratch(device, workspace_bytes);
        devices::rocm::check(rlt_rocm_seq_evaluate_step(device.handle, &l, 1, input._data, (int)LAYER_SPEC::INPUT_DIM, &s, auto_reset_period, output._data, (int)LAYER_SPEC::HIDDEN_DIM, (int)B,
                                                        workspace, workspace_bytes), "evaluate_step(gru)");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
