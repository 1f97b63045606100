// Harness around the REAL reference (compiled from /root/reference/include where it lies; nothing of it is copied here): the reference's own
// SAC loop on the Pendulum with its recurrent approximators (rl/algorithms/sac/loop/core/approximators_gru.h: dense -> GRU [-> GRU] [-> dense]
// -> dense [-> sample_and_squash]) on sequence batches: three environments, episodes of 30 steps, 260-row replay rings, sequences of 6 steps
// with the first step included in the targets, batches of 16 sequences. After every loop step it exposes every parameter of the five
// networks, log_alpha, the Adam ages, the batch the step trained on and the two noise tensors it drew, so that tests can pin the CPU
// restatement of train_critic / train_actor on sequence batches (oracle/) against it. The training operations draw nothing themselves
// (the noise is passed in), so the loop's own step() is used as it is.
// RLT_REF_SAC_GRU_LAYERS (3, 4 or 5) selects the depth; built by oracle/Makefile into oracle/_ref/librlt_ref_sac_gru<N>_generic.so.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/gru/operations_generic.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/rl/algorithms/sac/loop/core/config.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#include <rl_tools/rl/utils/evaluation/operations_generic.h>

#include <cstdint>
#include <cstring>
#include <vector>

#ifndef RLT_REF_SAC_GRU_LAYERS
#define RLT_REF_SAC_GRU_LAYERS 4
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

struct LoopParameters : rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT> {
    struct SAC_PARAMETERS : rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM> {
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
    static constexpr TI ACTOR_NUM_LAYERS = RLT_REF_SAC_GRU_LAYERS;
    static constexpr TI ACTOR_HIDDEN_DIM = HIDDEN;
    static constexpr TI CRITIC_NUM_LAYERS = RLT_REF_SAC_GRU_LAYERS;
    static constexpr TI CRITIC_HIDDEN_DIM = HIDDEN;
};
using CONFIG = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LoopParameters, rlt::rl::algorithms::sac::loop::core::ConfigApproximatorsGRU>;
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

// flat parameter export of a sequential model, layer after layer: dense [W | b], GRU [W_i | b_i | W_h | b_h | h0]; the sample_and_squash
// layer's log_alpha is exported separately
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
template <typename L> auto layer_parameters(L& l, std::vector<float>&, int) -> decltype(l.log_alpha, void()) {}
template <typename L> auto layer_dims(L& l, std::vector<int>& out, int) -> decltype(l.weights_hidden, void()) { out.push_back(1); out.push_back(L::SPEC::INPUT_DIM); out.push_back(L::SPEC::HIDDEN_DIM); out.push_back(0); }
template <typename L> auto layer_dims(L& l, std::vector<int>& out, int) -> decltype(l.weights, void()) { out.push_back(0); out.push_back(L::INPUT_DIM); out.push_back(L::OUTPUT_DIM); out.push_back((int)L::SPEC::ACTIVATION_FUNCTION); }
template <typename L> auto layer_dims(L& l, std::vector<int>&, int) -> decltype(l.log_alpha, void()) {}
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
template <typename L> auto layer_gradients(L& l, std::vector<float>&, int) -> decltype(l.log_alpha, void()) {}
template <typename M> void model_gradients(M& m, std::vector<float>& out) {
    layer_gradients(m.content, out, 0);
    if constexpr (!rlt::utils::typing::is_same_v<typename M::NEXT_MODULE, rlt::nn_models::sequential::OutputModule>) model_gradients(m.next_module, out);
}
template <typename M> void model_dims(M& m, std::vector<int>& out) {
    layer_dims(m.content, out, 0);
    if constexpr (!rlt::utils::typing::is_same_v<typename M::NEXT_MODULE, rlt::nn_models::sequential::OutputModule>) model_dims(m.next_module, out);
}
// the policy state of the runner's actor (policy index 1): per GRU layer the hidden state [N_ENVS x H] and the step counters [N_ENVS]
template <typename S> auto layer_state(DEVICE& device, S& s, std::vector<float>& hidden, std::vector<uint32_t>& steps, int) -> decltype(s.step, void()) {
    constexpr size_t H = rlt::get<1>(typename decltype(s.state)::SPEC::SHAPE{});
    const float* p = rlt::data(s.state); hidden.insert(hidden.end(), p, p + N_ENVS * H);
    for (TI i = 0; i < N_ENVS; i++) steps.push_back((uint32_t)rlt::get(device, s.step, i));
}
template <typename S> void layer_state(DEVICE&, S&, std::vector<float>&, std::vector<uint32_t>&, long) {}
template <typename CS> void walk_state(DEVICE& device, CS& cs, std::vector<float>& hidden, std::vector<uint32_t>& steps) {
    layer_state(device, cs.state, hidden, steps, 0);
    if constexpr (!rlt::utils::typing::is_same_v<typename CS::NEXT_CONTENT_STATE, rlt::nn_models::sequential::OutputModule>) walk_state(device, cs.next_content_state, hidden, steps);
}
std::vector<float> all_parameters(Loop& L) {
    auto& ac = L.ts.actor_critic;
    std::vector<float> out;
    model_parameters(ac.actor, out); model_parameters(ac.critics[0], out); model_parameters(ac.critics[1], out);
    model_parameters(ac.critics_target[0], out); model_parameters(ac.critics_target[1], out);
    out.push_back(rlt::get(L.device, rlt::get_last_layer(ac.actor).log_alpha.parameters, 0));
    return out;
}
}  // namespace

extern "C" {

void* rlt_ref_sac_gru_create(uint32_t seed) { return new Loop(seed); }
void rlt_ref_sac_gru_destroy(void* h) { delete static_cast<Loop*>(h); }
void rlt_ref_sac_gru_step(void* h) { auto& L = *static_cast<Loop*>(h); rlt::step(L.device, L.ts); }
uint32_t rlt_ref_sac_gru_step_count(void* h) { return (uint32_t)static_cast<Loop*>(h)->ts.step; }

// [batch, sequence length, n_warmup_steps, observation dim, action dim, include_first_step_in_targets]
void rlt_ref_sac_gru_dims(int* out) {
    out[0] = BATCH; out[1] = SEQ; out[2] = LoopParameters::N_WARMUP_STEPS; out[3] = ENVIRONMENT::Observation::DIM; out[4] = ENVIRONMENT::ACTION_DIM;
    out[5] = LoopParameters::BATCH_SAMPLING_PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS;
}
// layer lists of the actor (without its sample_and_squash layer) and of a critic: 4 ints per layer [kind (0 dense, 1 GRU), in, out, activation
// (the reference's enum value; dense only)]; returns the number of ints written
int rlt_ref_sac_gru_layers(void* h, int critic, int* out) {
    auto& ac = static_cast<Loop*>(h)->ts.actor_critic;
    std::vector<int> v;
    if (critic) model_dims(ac.critics[0], v); else model_dims(ac.actor, v);
    std::memcpy(out, v.data(), v.size() * sizeof(int));
    return (int)v.size();
}
// [gamma, polyak, target entropy, log_std lower, log_std upper, log-probability epsilon, actor adam (alpha, beta_1, beta_2, epsilon, epsilon_sqrt),
//  critic adam (5), alpha adam (5)]
void rlt_ref_sac_gru_hyperparameters(void* h, float* out) {
    using P = LoopParameters::SAC_PARAMETERS;
    auto& L = *static_cast<Loop*>(h); auto& ac = L.ts.actor_critic;
    out[0] = P::GAMMA; out[1] = P::CRITIC_POLYAK; out[2] = P::TARGET_ENTROPY; out[3] = P::LOG_STD_LOWER_BOUND; out[4] = P::LOG_STD_UPPER_BOUND; out[5] = P::LOG_PROBABILITY_EPSILON;
    auto put = [&](auto& optimizer, float* o) { auto& p = rlt::get_ref(L.device, optimizer.parameters, 0); o[0] = p.alpha; o[1] = p.beta_1; o[2] = p.beta_2; o[3] = p.epsilon; o[4] = p.epsilon_sqrt; };
    put(ac.actor_optimizer, out + 6); put(ac.critic_optimizers[0], out + 11); put(ac.alpha_optimizer, out + 16);
}
// flat: actor, critic 0, critic 1, critic target 0, critic target 1 (layer after layer: dense [W | b], GRU [W_i | b_i | W_h | b_h | h0]), log_alpha
size_t rlt_ref_sac_gru_parameter_count(void* h) { return all_parameters(*static_cast<Loop*>(h)).size(); }
void rlt_ref_sac_gru_get_parameters(void* h, float* out) { auto v = all_parameters(*static_cast<Loop*>(h)); std::memcpy(out, v.data(), v.size() * sizeof(float)); }
// Adam ages [actor, critic 0, critic 1, alpha]
void rlt_ref_sac_gru_get_ages(void* h, uint32_t* out) {
    auto& L = *static_cast<Loop*>(h); auto& ac = L.ts.actor_critic;
    out[0] = (uint32_t)rlt::get(L.device, ac.actor_optimizer.age, 0); out[1] = (uint32_t)rlt::get(L.device, ac.critic_optimizers[0].age, 0);
    out[2] = (uint32_t)rlt::get(L.device, ac.critic_optimizers[1].age, 0); out[3] = (uint32_t)rlt::get(L.device, ac.alpha_optimizer.age, 0);
}
// the batch of the last training step: observations_actions_base [(S+1) x B x 4], rewards / terminated / reset / final_step_mask [S x B],
// next_reset_base / next_final_step_mask_base [(S+1) x B]
void rlt_ref_sac_gru_get_batch(void* h, float* oab, float* rewards, uint8_t* terminated, uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask,
                               uint8_t* next_final_step_mask_base) {
    auto& b = static_cast<Loop*>(h)->ts.critic_batch;
    std::memcpy(oab, b.observations_actions_base._data, sizeof(float) * (SEQ + 1) * BATCH * 4);
    std::memcpy(rewards, b.rewards._data, sizeof(float) * SEQ * BATCH);
    for (TI i = 0; i < SEQ * BATCH; i++) { terminated[i] = b.terminated._data[i]; reset[i] = b.reset._data[i]; final_step_mask[i] = b.final_step_mask._data[i]; }
    for (TI i = 0; i < (SEQ + 1) * BATCH; i++) { next_reset_base[i] = b.next_reset_base._data[i]; next_final_step_mask_base[i] = b.next_final_step_mask_base._data[i]; }
}
// what the last training step left behind: the gradients of actor, critic 0, critic 1 (same layout as the parameters, log_alpha's last), and of
// the critic training buffers k = 0, 1 the target values [S x B], d_output [S x B] and both target critics' values [(S+1) x B]
void rlt_ref_sac_gru_get_gradients(void* h, float* out) {
    auto& L = *static_cast<Loop*>(h); auto& ac = L.ts.actor_critic;
    std::vector<float> v;
    model_gradients(ac.actor, v); model_gradients(ac.critics[0], v); model_gradients(ac.critics[1], v);
    v.push_back(rlt::get(L.device, rlt::get_last_layer(ac.actor).log_alpha.gradient, 0));
    std::memcpy(out, v.data(), v.size() * sizeof(float));
}
void rlt_ref_sac_gru_get_critic_buffers(void* h, int k, float* target_action_value, float* d_output, float* next_q_1, float* next_q_2) {
    auto& tb = static_cast<Loop*>(h)->ts.critic_training_buffers[k];
    std::memcpy(target_action_value, rlt::data(tb.target_action_value), sizeof(float) * SEQ * BATCH);
    std::memcpy(d_output, rlt::data(tb.d_output), sizeof(float) * SEQ * BATCH);
    std::memcpy(next_q_1, rlt::data(tb.next_state_action_value_critic_1), sizeof(float) * (SEQ + 1) * BATCH);
    std::memcpy(next_q_2, rlt::data(tb.next_state_action_value_critic_2), sizeof(float) * (SEQ + 1) * BATCH);
}
// One loop step past the warm-up assembled from the reference's own operations in the order of sac::loop::core::step, so that what the runner step draws
// can be written out: before it the engine is copied and the same draws are taken from the copy with the reference's own functions (per environment that
// starts a new episode: parameters, initial state; then one N(0,1) value per environment for the sample_and_squash layer). Returns 1 if the copy then
// equals the engine, i.e. exactly these draws were made. Tests compare everything after this with a second loop advanced with rlt_ref_sac_gru_step.
int rlt_ref_sac_gru_manual_step(void* h, float* initial_states, float* action_noise, uint8_t* reset_flags) {
    auto& L = *static_cast<Loop*>(h);
    auto& device = L.device; auto& ts = L.ts; auto& runner = ts.off_policy_runner;
    using CP = CONFIG::CORE_PARAMETERS; using P = CP::SAC_PARAMETERS;
    if (ts.step < CP::N_WARMUP_STEPS) return -1;
    rlt::set_step(device, device.logger, ts.step);
    RNG copy = ts.rng;
    const bool policy_switch = runner.previous_policy_set && runner.previous_policy != 1;      // the first step after the warm-up truncates every episode
    for (TI e = 0; e < N_ENVS; e++) {
        reset_flags[e] = policy_switch || rlt::get(runner.truncated, 0, e);
        initial_states[2 * e] = initial_states[2 * e + 1] = 0;
        if (reset_flags[e]) {
            auto& env = rlt::get(runner.envs, 0, e);
            auto parameters = rlt::get(runner.env_parameters, 0, e);
            typename ENVIRONMENT::State state;
            if (CONFIG::OFF_POLICY_RUNNER_PARAMETERS::SAMPLE_PARAMETERS) rlt::sample_initial_parameters(device, env, parameters, copy);
            rlt::sample_initial_state(device, env, parameters, state, copy);
            initial_states[2 * e] = state.theta; initial_states[2 * e + 1] = state.theta_dot;
        }
    }
    for (TI e = 0; e < N_ENVS; e++) action_noise[e] = rlt::random::normal_distribution::sample(device.random, 0.0f, 1.0f, copy);
    rlt::step<1>(device, runner, rlt::get_actor(ts), ts.actor_buffers_eval, ts.rng);
    const int same = copy.engine == ts.rng.engine;
    const bool train_critic_flag = ts.step >= CP::N_WARMUP_STEPS_CRITIC && ts.step % P::CRITIC_TRAINING_INTERVAL == 0;
    const bool update_critic_targets_flag = ts.step >= CP::N_WARMUP_STEPS_CRITIC && ts.step % P::CRITIC_TARGET_UPDATE_INTERVAL == 0;
    const bool train_actor_flag = ts.step >= CP::N_WARMUP_STEPS_ACTOR && ts.step % P::ACTOR_TRAINING_INTERVAL == 0;
    static_assert(CP::SHARED_BATCH);
    if (train_critic_flag || train_actor_flag) { rlt::gather_batch(device, runner, ts.critic_batch, ts.rng); rlt::randn(device, ts.action_noise_critic, ts.rng); }
    if (train_critic_flag)
        for (int i = 0; i < 2; i++)
            rlt::train_critic(device, ts.actor_critic, ts.actor_critic.critics[i], ts.critic_batch, ts.actor_critic.critic_optimizers[i], ts.actor_target_buffers[i], ts.critic_buffers[i],
                              ts.critic_target_buffers[i], ts.critic_training_buffers[i], ts.action_noise_critic, ts.rng);
    if (update_critic_targets_flag) rlt::update_critic_targets(device, ts.actor_critic);
    if (train_actor_flag) {
        rlt::randn(device, ts.action_noise_actor, ts.rng);
        rlt::train_actor(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.actor_optimizer, ts.actor_buffers[0], ts.critic_buffers[0], ts.actor_training_buffers, ts.action_noise_actor, ts.rng);
    }
    ts.step++;
    return same;
}
// [n_envs, replay capacity, episode step limit, the actor's auto-reset period (the SEQUENCE_LENGTH of its input shape), number of GRU layers in the actor]
void rlt_ref_sac_gru_runner_dims(void* h, int* out) {
    auto& L = *static_cast<Loop*>(h);
    std::vector<float> hidden; std::vector<uint32_t> steps;
    walk_state(L.device, rlt::get<1>(L.ts.off_policy_runner.policy_states).content_state, hidden, steps);
    out[0] = N_ENVS; out[1] = CAPACITY; out[2] = EPISODE_LIMIT; out[3] = SEQ; out[4] = (int)(steps.size() / N_ENVS);
}
// the runner: states [n_envs x 2], episode_step, episode_return, truncated [n_envs]; the actor's policy state: hidden [GRU layers x n_envs x H] (layer after layer),
// step counters [GRU layers x n_envs]
void rlt_ref_sac_gru_get_runner(void* h, float* states, uint32_t* episode_step, float* episode_return, uint8_t* truncated, float* hidden, uint32_t* steps) {
    auto& L = *static_cast<Loop*>(h); auto& runner = L.ts.off_policy_runner;
    for (TI e = 0; e < N_ENVS; e++) {
        auto& st = rlt::get(runner.states, 0, e);
        states[2 * e] = st.theta; states[2 * e + 1] = st.theta_dot;
        episode_step[e] = (uint32_t)rlt::get(runner.episode_step, 0, e); episode_return[e] = rlt::get(runner.episode_return, 0, e); truncated[e] = rlt::get(runner.truncated, 0, e);
    }
    std::vector<float> hv; std::vector<uint32_t> sv;
    walk_state(L.device, rlt::get<1>(runner.policy_states).content_state, hv, sv);
    std::memcpy(hidden, hv.data(), hv.size() * sizeof(float)); std::memcpy(steps, sv.data(), sv.size() * sizeof(uint32_t));
}
// replay ring of one environment: data [capacity x 10], cursor, full flag, start of the running episode, episode starts
void rlt_ref_sac_gru_get_replay(void* h, int env, float* data, uint32_t* position, uint8_t* full, uint32_t* current_episode_start, uint32_t* episode_start) {
    Loop& L = *static_cast<Loop*>(h);
    auto& rb = rlt::get(L.ts.off_policy_runner.replay_buffers, 0, env);
    using RB = rlt::utils::typing::remove_reference_t<decltype(rb)>;
    std::memcpy(data, rb.data._data, sizeof(float) * RB::CAPACITY * RB::DATA_COLS);
    *position = (uint32_t)rb.position; *full = rb.full; *current_episode_start = (uint32_t)rb.current_episode_start;
    for (TI i = 0; i < RB::CAPACITY; i++) episode_start[i] = (uint32_t)rlt::get(L.device, rb.episode_start, i);
}
// the N(0,1) noise of the last training step: critic [(S+1) x B x 1], actor [S x B x 1]
void rlt_ref_sac_gru_get_noise(void* h, float* noise_critic, float* noise_actor) {
    auto& ts = static_cast<Loop*>(h)->ts;
    std::memcpy(noise_critic, ts.action_noise_critic._data, sizeof(float) * (SEQ + 1) * BATCH);
    std::memcpy(noise_actor, ts.action_noise_actor._data, sizeof(float) * SEQ * BATCH);
}

// rl::utils::evaluation::evaluate (rl/utils/evaluation/operations_generic.h:106-233) of the loop's current recurrent actor in Evaluation mode: 5 episodes of 40
// steps from sampled initial states (the actor restarts its hidden state every 6 steps by itself). The initial states the call will draw are exported by drawing
// them first from a copy of the engine. summary = {returns_mean, returns_std, episode_length_mean, episode_length_std, num_terminated, share_terminated}
void rlt_ref_sac_gru_evaluate(void* h, uint32_t seed, float* initial_states, float* returns, uint32_t* episode_length, float* summary) {
    Loop& L = *static_cast<Loop*>(h);
    constexpr TI N_EPISODES = 5, STEP_LIMIT = 40;
    using SPEC = rlt::rl::utils::evaluation::Specification<TYPE_POLICY, TI, ENVIRONMENT, N_EPISODES, STEP_LIMIT>;
    RNG rng;
    rlt::malloc(L.device, rng);
    rlt::init(L.device, rng, seed);
    ENVIRONMENT env;
    ENVIRONMENT::Parameters parameters;
    rlt::init(L.device, env);
    rlt::initial_parameters(L.device, env, parameters);
    {
        RNG copy = rng;
        for (TI e = 0; e < N_EPISODES; e++) {
            ENVIRONMENT::State state;
            rlt::sample_initial_parameters(L.device, env, parameters, copy);
            rlt::sample_initial_state(L.device, env, parameters, state, copy);
            initial_states[2 * e] = state.theta; initial_states[2 * e + 1] = state.theta_dot;
        }
    }
    rlt::rl::utils::evaluation::Result<SPEC> result;
    rlt::rl::environments::DummyUI ui;
    rlt::Mode<rlt::mode::Evaluation<>> mode;
    rlt::evaluate(L.device, env, ui, L.ts.actor_critic.actor, result, rng, mode);
    for (TI e = 0; e < N_EPISODES; e++) { returns[e] = result.returns[e]; episode_length[e] = (uint32_t)result.episode_length[e]; }
    summary[0] = result.returns_mean; summary[1] = result.returns_std; summary[2] = result.episode_length_mean; summary[3] = result.episode_length_std;
    summary[4] = (float)result.num_terminated; summary[5] = result.share_terminated;
    rlt::free(L.device, rng);
}

}  // extern "C"
