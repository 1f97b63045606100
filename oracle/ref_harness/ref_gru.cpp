// Harness around the REAL reference's GRU layer (compiled from /root/reference/include where it lies; nothing of it is copied here):
// forward and backward-through-time of one layer on caller-supplied weights and inputs, with and without per-sample resets, so that
// tests can pin the CPU restatement (oracle/) against it. Shapes are compile-time in the reference: one small fixed shape is built.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>

#include <cstdint>
#include <cstring>

namespace rlt = rl_tools;

namespace {
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using TI = typename DEVICE::index_t;
constexpr TI S = 7, B = 5, I = 6, H = 8;
using CAPABILITY = rlt::nn::capability::Gradient<rlt::nn::parameters::Adam>;
using INPUT_SHAPE = rlt::tensor::Shape<TI, S, B, I>;
#ifdef RLT_REF_GRU_FAST_TANH   // the switch the reference's SAC / TD3 GRU approximators set
using GRU_CONFIG = rlt::nn::layers::gru::Configuration<TYPE_POLICY, TI, H, rlt::nn::parameters::groups::Normal, true>;
#else
using GRU_CONFIG = rlt::nn::layers::gru::Configuration<TYPE_POLICY, TI, H>;
#endif
using GRU = rlt::nn::layers::gru::Layer<GRU_CONFIG, CAPABILITY, INPUT_SHAPE>;
using RESET = rlt::Tensor<rlt::tensor::Specification<bool, TI, rlt::tensor::Shape<TI, S, B, 1>>>;
using RESET_MODE_SPEC = rlt::nn::layers::gru::ResetModeSpecification<TI, RESET>;
using RESET_MODE = rlt::nn::layers::gru::ResetMode<rlt::mode::Default<>, RESET_MODE_SPEC>;

template <typename TENSOR> void put(TENSOR& t, const float* src, size_t n) { std::memcpy(rlt::data(t), src, n * sizeof(float)); }
template <typename TENSOR> void get(TENSOR& t, float* dst, size_t n) { std::memcpy(dst, rlt::data(t), n * sizeof(float)); }
}  // namespace

extern "C" {

// [S, B, I, H]
void rlt_ref_gru_dims(int* out) { out[0] = S; out[1] = B; out[2] = I; out[3] = H; }

// weights: W_i [3H x I], b_i [3H], W_h [3H x H], b_h [3H], h0 [H]; reset may be NULL.
// outputs: output [S x B x H], post_activation [S x B x 3H], n_pre_pre_activation [S x B x H], d_input [S x B x I], the gradients in the
// same order as the weights (without h0), and d_output after the pass (the reference accumulates into it).
int rlt_ref_gru_forward_backward(const float* W_i, const float* b_i, const float* W_h, const float* b_h, const float* h0, const float* input,
                                 const uint8_t* reset_flags, const float* d_output_in, float* output, float* post_activation, float* n_pre_pre_activation,
                                 float* d_input_out, float* dW_i, float* db_i, float* dW_h, float* db_h, float* d_output_after) {
    DEVICE device;
    GRU gru;
    typename GRU::template Buffer<true> buffer;
    typename DEVICE::SPEC::RANDOM::ENGINE<> rng;
    rlt::Tensor<rlt::tensor::Specification<float, TI, INPUT_SHAPE>> x, dx;
    rlt::Tensor<rlt::tensor::Specification<float, TI, rlt::tensor::Shape<TI, S, B, H>>> dy;
    RESET reset;
    rlt::malloc(device, gru); rlt::malloc(device, buffer); rlt::malloc(device, x); rlt::malloc(device, dx); rlt::malloc(device, dy); rlt::malloc(device, reset);
    rlt::init(device, rng, 0);
    rlt::init_weights(device, gru, rng);
    put(gru.weights_input.parameters, W_i, 3 * H * I); put(gru.biases_input.parameters, b_i, 3 * H);
    put(gru.weights_hidden.parameters, W_h, 3 * H * H); put(gru.biases_hidden.parameters, b_h, 3 * H);
    put(gru.initial_hidden_state.parameters, h0, H);
    put(x, input, S * B * I); put(dy, d_output_in, S * B * H);
    rlt::zero_gradient(device, gru);
    if (reset_flags) {
        for (TI t = 0; t < S; t++) for (TI b = 0; b < B; b++) rlt::set(device, reset, reset_flags[t * B + b] != 0, t, b, 0);
        rlt::Mode<RESET_MODE> mode;
        mode.reset_container = reset;
        rlt::forward(device, gru, x, buffer, rng, mode);
        get(gru.output, output, S * B * H); get(gru.post_activation, post_activation, S * B * 3 * H); get(gru.n_pre_pre_activation, n_pre_pre_activation, S * B * H);
        rlt::backward_full(device, gru, x, dy, dx, buffer, mode);
    } else {
        rlt::forward(device, gru, x, buffer, rng);
        get(gru.output, output, S * B * H); get(gru.post_activation, post_activation, S * B * 3 * H); get(gru.n_pre_pre_activation, n_pre_pre_activation, S * B * H);
        rlt::backward_full(device, gru, x, dy, dx, buffer);
    }
    get(dx, d_input_out, S * B * I); get(dy, d_output_after, S * B * H);
    get(gru.weights_input.gradient, dW_i, 3 * H * I); get(gru.biases_input.gradient, db_i, 3 * H);
    get(gru.weights_hidden.gradient, dW_h, 3 * H * H); get(gru.biases_hidden.gradient, db_h, 3 * H);
    rlt::free(device, gru); rlt::free(device, buffer); rlt::free(device, x); rlt::free(device, dx); rlt::free(device, dy); rlt::free(device, reset);
    return 0;
}

}  // extern "C"
