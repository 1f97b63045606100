// Harness around the REAL reference (compiled from /root/reference/include where it lies; nothing of it is copied here): the reference's own
// TD3 loop on the Pendulum with its recurrent approximators (rl/algorithms/td3/loop/core/approximators_gru.h: GRU [-> GRU] [-> dense] -> dense)
// on sequence batches: three environments, episodes of 30 steps, 260-row replay rings, sequences of 6 steps with the first step included in the
// targets, batches of 16 sequences. After every loop step it exposes every parameter of the six networks, the Adam ages, the batch the step
// trained on and the clamped target-action noise it drew, so that tests can pin the CPU restatement of TD3's train_critic / train_actor on
// sequence batches (oracle/) against it. The training operations draw nothing themselves, so the loop's own step() is used as it is.
// RLT_REF_TD3_GRU_LAYERS (3, 4 or 5) selects the depth; built by oracle/Makefile into oracle/_ref/librlt_ref_td3_gru<N>_generic.so.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/nn/layers/td3_sampling/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/rl/algorithms/td3/loop/core/config.h>
#include <rl_tools/rl/algorithms/td3/loop/core/operations_generic.h>

#include <cstdint>
#include <cstring>
#include <vector>

#ifndef RLT_REF_TD3_GRU_LAYERS
#define RLT_REF_TD3_GRU_LAYERS 4
#endif

namespace rlt = rl_tools;

namespace {
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;
using TI = typename DEVICE::index_t;
using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
constexpr TI N_ENVS = 3, CAPACITY = 260, EPISODE_LIMIT = 30, BATCH = 16, SEQ = 6, HIDDEN = 16;

struct LoopParameters : rlt::rl::algorithms::td3::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT> {
    struct TD3_PARAMETERS : rlt::rl::algorithms::td3::DefaultParameters<TYPE_POLICY, TI> {
        static constexpr TI ACTOR_BATCH_SIZE = BATCH;
        static constexpr TI CRITIC_BATCH_SIZE = BATCH;
        static constexpr TI SEQUENCE_LENGTH = SEQ;
    };
    struct BATCH_SAMPLING_PARAMETERS {
        static constexpr bool INCLUDE_FIRST_STEP_IN_TARGETS = true;
        static constexpr bool ALWAYS_SAMPLE_FROM_INITIAL_STATE = false;
        static constexpr bool RANDOM_SEQ_LENGTH = true;
        static constexpr bool ENABLE_NOMINAL_SEQUENCE_LENGTH_PROBABILITY = true;
        static constexpr float NOMINAL_SEQUENCE_LENGTH_PROBABILITY = 0.5;
    };
    static constexpr TI N_ENVIRONMENTS = N_ENVS;
    static constexpr TI N_WARMUP_STEPS = 100;
    static constexpr TI N_WARMUP_STEPS_CRITIC = 100;
    static constexpr TI N_WARMUP_STEPS_ACTOR = 100;
    static constexpr TI STEP_LIMIT = 100000;
    static constexpr TI REPLAY_BUFFER_CAP = CAPACITY;
    static constexpr TI EPISODE_STEP_LIMIT = EPISODE_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = RLT_REF_TD3_GRU_LAYERS;
    static constexpr TI ACTOR_HIDDEN_DIM = HIDDEN;
    static constexpr TI CRITIC_NUM_LAYERS = RLT_REF_TD3_GRU_LAYERS;
    static constexpr TI CRITIC_HIDDEN_DIM = HIDDEN;
};
using CONFIG = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LoopParameters, rlt::rl::algorithms::td3::loop::core::ConfigApproximatorsGRU>;
using STATE = typename CONFIG::template State<CONFIG>;

struct Loop {
    DEVICE device;
    STATE ts;
    explicit Loop(uint32_t seed) {
        rlt::malloc(device, ts); rlt::init(device, ts, seed);
        // The reference allocates the batch without clearing it, and gather_batch never writes some entries (reward and terminated flag of the
        // padding step after a sequence end): they are masked out of the update, but would make the exported batches differ from run to run.
        auto& b = ts.critic_batch;
        std::memset(b.observations_actions_base._data, 0, sizeof(float) * (SEQ + 1) * BATCH * 4);
        std::memset(b.rewards._data, 0, sizeof(float) * SEQ * BATCH);
        std::memset(b.terminated._data, 0, sizeof(bool) * SEQ * BATCH); std::memset(b.reset._data, 0, sizeof(bool) * SEQ * BATCH);
        std::memset(b.final_step_mask._data, 0, sizeof(bool) * SEQ * BATCH);
        std::memset(b.next_reset_base._data, 0, sizeof(bool) * (SEQ + 1) * BATCH); std::memset(b.next_final_step_mask_base._data, 0, sizeof(bool) * (SEQ + 1) * BATCH);
    }
    ~Loop() { rlt::free(device, ts); }
};

// flat parameter export of a sequential model, layer after layer: dense [W | b], GRU [W_i | b_i | W_h | b_h | h0]
template <typename T> void append(std::vector<float>& out, T& tensor, size_t n) { const float* p = rlt::data(tensor); out.insert(out.end(), p, p + n); }
template <typename L> auto layer_parameters(L& l, std::vector<float>& out, int) -> decltype(l.weights_hidden, void()) {
    constexpr size_t H = L::SPEC::HIDDEN_DIM, I = L::SPEC::INPUT_DIM;
    append(out, l.weights_input.parameters, 3 * H * I); append(out, l.biases_input.parameters, 3 * H);
    append(out, l.weights_hidden.parameters, 3 * H * H); append(out, l.biases_hidden.parameters, 3 * H);
    append(out, l.initial_hidden_state.parameters, H);
}
template <typename L> auto layer_parameters(L& l, std::vector<float>& out, int) -> decltype(l.weights, void()) {
    append(out, l.weights.parameters, (size_t)L::INPUT_DIM * L::OUTPUT_DIM); append(out, l.biases.parameters, (size_t)L::OUTPUT_DIM);
}
template <typename L> auto layer_dims(L& l, std::vector<int>& out, int) -> decltype(l.weights_hidden, void()) { out.push_back(1); out.push_back(L::SPEC::INPUT_DIM); out.push_back(L::SPEC::HIDDEN_DIM); out.push_back(0); }
template <typename L> auto layer_dims(L& l, std::vector<int>& out, int) -> decltype(l.weights, void()) { out.push_back(0); out.push_back(L::INPUT_DIM); out.push_back(L::OUTPUT_DIM); out.push_back((int)L::SPEC::ACTIVATION_FUNCTION); }
template <typename M> void model_parameters(M& m, std::vector<float>& out) {
    layer_parameters(m.content, out, 0);
    if constexpr (!rlt::utils::typing::is_same_v<typename M::NEXT_MODULE, rlt::nn_models::sequential::OutputModule>) model_parameters(m.next_module, out);
}
template <typename L> auto layer_gradients(L& l, std::vector<float>& out, int) -> decltype(l.weights_hidden, void()) {
    constexpr size_t H = L::SPEC::HIDDEN_DIM, I = L::SPEC::INPUT_DIM;
    append(out, l.weights_input.gradient, 3 * H * I); append(out, l.biases_input.gradient, 3 * H);
    append(out, l.weights_hidden.gradient, 3 * H * H); append(out, l.biases_hidden.gradient, 3 * H);
    append(out, l.initial_hidden_state.gradient, H);
}
template <typename L> auto layer_gradients(L& l, std::vector<float>& out, int) -> decltype(l.weights, void()) {
    append(out, l.weights.gradient, (size_t)L::INPUT_DIM * L::OUTPUT_DIM); append(out, l.biases.gradient, (size_t)L::OUTPUT_DIM);
}
template <typename M> void model_gradients(M& m, std::vector<float>& out) {
    layer_gradients(m.content, out, 0);
    if constexpr (!rlt::utils::typing::is_same_v<typename M::NEXT_MODULE, rlt::nn_models::sequential::OutputModule>) model_gradients(m.next_module, out);
}
template <typename M> void model_dims(M& m, std::vector<int>& out) {
    layer_dims(m.content, out, 0);
    if constexpr (!rlt::utils::typing::is_same_v<typename M::NEXT_MODULE, rlt::nn_models::sequential::OutputModule>) model_dims(m.next_module, out);
}
std::vector<float> all_parameters(Loop& L) {
    auto& ac = L.ts.actor_critic;
    std::vector<float> out;
    model_parameters(ac.actor, out); model_parameters(ac.critics[0], out); model_parameters(ac.critics[1], out);
    model_parameters(ac.actor_target, out); model_parameters(ac.critics_target[0], out); model_parameters(ac.critics_target[1], out);
    return out;
}
}  // namespace

extern "C" {

void* rlt_ref_td3_gru_create(uint32_t seed) { return new Loop(seed); }
void rlt_ref_td3_gru_destroy(void* h) { delete static_cast<Loop*>(h); }
void rlt_ref_td3_gru_step(void* h) { auto& L = *static_cast<Loop*>(h); rlt::step(L.device, L.ts); }
uint32_t rlt_ref_td3_gru_step_count(void* h) { return (uint32_t)static_cast<Loop*>(h)->ts.step; }

// [batch, sequence length, n_warmup_steps, observation dim, action dim, include_first_step_in_targets, critic training interval, critic target update
//  interval, actor training interval, actor target update interval, ignore_termination]
void rlt_ref_td3_gru_dims(int* out) {
    using P = LoopParameters::TD3_PARAMETERS;
    out[0] = BATCH; out[1] = SEQ; out[2] = LoopParameters::N_WARMUP_STEPS; out[3] = ENVIRONMENT::Observation::DIM; out[4] = ENVIRONMENT::ACTION_DIM;
    out[5] = LoopParameters::BATCH_SAMPLING_PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS;
    out[6] = P::CRITIC_TRAINING_INTERVAL; out[7] = P::CRITIC_TARGET_UPDATE_INTERVAL; out[8] = P::ACTOR_TRAINING_INTERVAL; out[9] = P::ACTOR_TARGET_UPDATE_INTERVAL;
    out[10] = P::IGNORE_TERMINATION;
}
// layer lists of the actor and of a critic: 4 ints per layer [kind (0 dense, 1 GRU), in, out, activation (the reference's enum value; dense only)];
// returns the number of ints written
int rlt_ref_td3_gru_layers(void* h, int critic, int* out) {
    auto& ac = static_cast<Loop*>(h)->ts.actor_critic;
    std::vector<int> v;
    if (critic) model_dims(ac.critics[0], v); else model_dims(ac.actor, v);
    std::memcpy(out, v.data(), v.size() * sizeof(int));
    return (int)v.size();
}
// [gamma, actor polyak, critic polyak, target noise std, target noise clip, actor adam (alpha, beta_1, beta_2, epsilon, epsilon_sqrt), critic adam (5)]
void rlt_ref_td3_gru_hyperparameters(void* h, float* out) {
    using P = LoopParameters::TD3_PARAMETERS;
    auto& L = *static_cast<Loop*>(h); auto& ac = L.ts.actor_critic;
    out[0] = ac.gamma; out[1] = P::ACTOR_POLYAK; out[2] = P::CRITIC_POLYAK; out[3] = ac.target_next_action_noise_std; out[4] = ac.target_next_action_noise_clip;
    auto put = [&](auto& optimizer, float* o) { auto& p = rlt::get_ref(L.device, optimizer.parameters, 0); o[0] = p.alpha; o[1] = p.beta_1; o[2] = p.beta_2; o[3] = p.epsilon; o[4] = p.epsilon_sqrt; };
    put(ac.actor_optimizer, out + 5); put(ac.critic_optimizers[0], out + 10);
}
// flat: actor, critic 0, critic 1, actor target, critic target 0, critic target 1 (layer after layer: dense [W | b], GRU [W_i | b_i | W_h | b_h | h0])
size_t rlt_ref_td3_gru_parameter_count(void* h) { return all_parameters(*static_cast<Loop*>(h)).size(); }
void rlt_ref_td3_gru_get_parameters(void* h, float* out) { auto v = all_parameters(*static_cast<Loop*>(h)); std::memcpy(out, v.data(), v.size() * sizeof(float)); }
// Adam ages [actor, critic 0, critic 1]
void rlt_ref_td3_gru_get_ages(void* h, uint32_t* out) {
    auto& L = *static_cast<Loop*>(h); auto& ac = L.ts.actor_critic;
    out[0] = (uint32_t)rlt::get(L.device, ac.actor_optimizer.age, 0); out[1] = (uint32_t)rlt::get(L.device, ac.critic_optimizers[0].age, 0);
    out[2] = (uint32_t)rlt::get(L.device, ac.critic_optimizers[1].age, 0);
}
// the batch of the last training step: observations_actions_base [(S+1) x B x 4], rewards / terminated / reset / final_step_mask [S x B],
// next_reset_base / next_final_step_mask_base [(S+1) x B]
void rlt_ref_td3_gru_get_batch(void* h, float* oab, float* rewards, uint8_t* terminated, uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask,
                               uint8_t* next_final_step_mask_base) {
    auto& b = static_cast<Loop*>(h)->ts.critic_batch;
    std::memcpy(oab, b.observations_actions_base._data, sizeof(float) * (SEQ + 1) * BATCH * 4);
    std::memcpy(rewards, b.rewards._data, sizeof(float) * SEQ * BATCH);
    for (TI i = 0; i < SEQ * BATCH; i++) { terminated[i] = b.terminated._data[i]; reset[i] = b.reset._data[i]; final_step_mask[i] = b.final_step_mask._data[i]; }
    for (TI i = 0; i < (SEQ + 1) * BATCH; i++) { next_reset_base[i] = b.next_reset_base._data[i]; next_final_step_mask_base[i] = b.next_final_step_mask_base._data[i]; }
}
// the clamped target-action noise of the last training step [(S+1) x B x 1] and what the critic updates left: target values [S x B], d_output [S x B]
void rlt_ref_td3_gru_get_noise(void* h, float* noise) {
    auto& ts = static_cast<Loop*>(h)->ts;
    std::memcpy(noise, rlt::data(ts.critic_training_buffers.target_next_action_noise), sizeof(float) * (SEQ + 1) * BATCH);
}
void rlt_ref_td3_gru_get_critic_buffers(void* h, float* target_action_value, float* d_output) {
    auto& tb = static_cast<Loop*>(h)->ts.critic_training_buffers;
    std::memcpy(target_action_value, rlt::data(tb.target_action_value), sizeof(float) * SEQ * BATCH);
    std::memcpy(d_output, rlt::data(tb.d_output), sizeof(float) * SEQ * BATCH);
}

}  // extern "C"
