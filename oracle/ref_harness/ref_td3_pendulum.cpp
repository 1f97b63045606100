// Harness around the REAL reference (compiled from /root/reference/include where it lies; nothing of it is copied here): runs the
// reference's own TD3-on-Pendulum loop and exposes, after every loop step, all parameters, the batch the step trained on and the
// clamped target-action noise it drew, so that tests can pin the CPU restatement of the TD3 update (oracle/) against it.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
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

namespace rlt = rl_tools;

namespace {
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;
using TI = typename DEVICE::index_t;
using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;
constexpr TI BATCH = 100;

struct LoopParameters : rlt::rl::algorithms::td3::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT> {
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = STEP_LIMIT;
};
using CONFIG = rlt::rl::algorithms::td3::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LoopParameters>;
using STATE = typename CONFIG::template State<CONFIG>;

struct Loop {
    DEVICE device;
    STATE ts;
    explicit Loop(uint32_t seed) { rlt::malloc(device, ts); rlt::init(device, ts, seed); }
    ~Loop() { rlt::free(device, ts); }
};

template <typename MLP>
size_t mlp_count(MLP& mlp) {
    size_t n = 0;
    auto add = [&](auto& layer) { n += layer.INPUT_DIM * layer.OUTPUT_DIM + layer.OUTPUT_DIM; };
    add(mlp.input_layer);
    for (TI i = 0; i < MLP::NUM_HIDDEN_LAYERS; i++) add(mlp.hidden_layers[i]);
    add(mlp.output_layer);
    return n;
}
template <typename MLP>
float* mlp_get(MLP& mlp, float* out) {
    auto put = [&](auto& layer) {
        size_t nw = layer.INPUT_DIM * layer.OUTPUT_DIM, nb = layer.OUTPUT_DIM;
        std::memcpy(out, layer.weights.parameters._data, nw * sizeof(float)); out += nw;
        std::memcpy(out, layer.biases.parameters._data, nb * sizeof(float)); out += nb;
    };
    put(mlp.input_layer);
    for (TI i = 0; i < MLP::NUM_HIDDEN_LAYERS; i++) put(mlp.hidden_layers[i]);
    put(mlp.output_layer);
    return out;
}
// the networks are sequential models whose first module holds the MLP
template <typename MODEL> auto& mlp_of(MODEL& m) { return m.content; }
}  // namespace

extern "C" {

void* rlt_ref_td3_create(uint32_t seed) { return new Loop(seed); }
void rlt_ref_td3_destroy(void* h) { delete static_cast<Loop*>(h); }
void rlt_ref_td3_step(void* h) { auto& L = *static_cast<Loop*>(h); rlt::step(L.device, L.ts); }

// One loop step assembled here from the reference's own operations, in the order of td3::loop::core::step (valid past the warm-up
// only), so that the N(0,1) draws which the actor's sampling layer takes from the RNG inside train_critic / train_actor can be
// written out: before each of these calls the RNG is copied and the same draws are taken from the copy. Tests compare the
// parameters after this with those of a second loop advanced with rlt_ref_td3_step. noise_* are [batch x 1]; noise_target_z are
// the N(0,1) values behind the N(0, std) draws of target_action_noise (std::normal_distribution scales the same draw);
// flags_out = [critic trained, critic targets updated, actor trained, actor target updated].
void rlt_ref_td3_manual_step(void* h, float* noise_target_z, float* noise_critic_0, float* noise_critic_1, float* noise_actor, int* flags_out) {
    auto& L = *static_cast<Loop*>(h);
    auto& device = L.device; auto& ts = L.ts;
    using CP = CONFIG::CORE_PARAMETERS; using P = CP::TD3_PARAMETERS;
    rlt::set_step(device, device.logger, ts.step);
    rlt::step<1>(device, ts.off_policy_runner, rlt::get_actor(ts), ts.actor_buffers_eval, ts.rng);
    bool train_critic_flag = ts.step >= CP::N_WARMUP_STEPS_CRITIC && ts.step % P::CRITIC_TRAINING_INTERVAL == 0;
    bool update_critic_targets_flag = ts.step >= CP::N_WARMUP_STEPS_CRITIC && ts.step % P::CRITIC_TARGET_UPDATE_INTERVAL == 0;
    bool train_actor_flag = ts.step >= CP::N_WARMUP_STEPS_ACTOR && ts.step % P::ACTOR_TRAINING_INTERVAL == 0;
    bool update_actor_target_flag = ts.step >= CP::N_WARMUP_STEPS_ACTOR && ts.step % P::ACTOR_TARGET_UPDATE_INTERVAL == 0;
    auto draws = [&](float* out) { RNG copy = ts.rng; for (TI i = 0; i < BATCH; i++) out[i] = rlt::random::normal_distribution::sample(device.random, 0.0f, 1.0f, copy); };
    if (train_critic_flag || train_actor_flag) {
        rlt::gather_batch(device, ts.off_policy_runner, ts.critic_batch, ts.rng);
        auto view = rlt::matrix_view(device, ts.critic_training_buffers.target_next_action_noise);
        draws(noise_target_z);
        rlt::target_action_noise(device, ts.actor_critic, view, ts.rng);
    }
    if (train_critic_flag)
        for (int i = 0; i < 2; i++) {
            draws(i == 0 ? noise_critic_0 : noise_critic_1);
            rlt::train_critic(device, ts.actor_critic, ts.actor_critic.critics[i], ts.critic_batch, ts.actor_critic.critic_optimizers[i], ts.actor_buffers[i],
                              ts.actor_target_buffers[i], ts.critic_buffers[i], ts.critic_target_buffers[i], ts.critic_training_buffers, ts.rng);
        }
    if (update_critic_targets_flag) rlt::update_critic_targets(device, ts.actor_critic);
    if (train_actor_flag) {
        draws(noise_actor);
        rlt::train_actor(device, ts.actor_critic, ts.critic_batch, ts.actor_critic.actor_optimizer, ts.actor_buffers[0], ts.critic_buffers[0], ts.actor_training_buffers, ts.rng);
    }
    if (update_actor_target_flag) rlt::update_actor_target(device, ts.actor_critic);
    ts.step++;
    flags_out[0] = train_critic_flag; flags_out[1] = update_critic_targets_flag; flags_out[2] = train_actor_flag; flags_out[3] = update_actor_target_flag;
}
uint32_t rlt_ref_td3_step_count(void* h) { return (uint32_t)static_cast<Loop*>(h)->ts.step; }

// [batch, n_warmup_steps, actor_training_interval, critic_target_update_interval, actor_target_update_interval, hidden]
void rlt_ref_td3_dims(int* out) {
    using P = LoopParameters::TD3_PARAMETERS;
    out[0] = P::CRITIC_BATCH_SIZE; out[1] = LoopParameters::N_WARMUP_STEPS; out[2] = P::ACTOR_TRAINING_INTERVAL; out[3] = P::CRITIC_TARGET_UPDATE_INTERVAL;
    out[4] = P::ACTOR_TARGET_UPDATE_INTERVAL; out[5] = LoopParameters::ACTOR_HIDDEN_DIM;
}
// [gamma, actor_polyak, critic_polyak, noise_std, noise_clip, adam alpha, beta_1, beta_2, epsilon, epsilon_sqrt, sampling-layer std]
void rlt_ref_td3_hyperparameters(void* h, float* out) {
    using P = LoopParameters::TD3_PARAMETERS;
    auto& L = *static_cast<Loop*>(h);
    out[0] = P::GAMMA; out[1] = P::ACTOR_POLYAK; out[2] = P::CRITIC_POLYAK; out[3] = P::TARGET_NEXT_ACTION_NOISE_STD; out[4] = P::TARGET_NEXT_ACTION_NOISE_CLIP;
    auto& p = rlt::get_ref(L.device, L.ts.actor_critic.actor_optimizer.parameters, 0);
    out[5] = p.alpha; out[6] = p.beta_1; out[7] = p.beta_2; out[8] = p.epsilon; out[9] = p.epsilon_sqrt;
    out[10] = L.ts.actor_critic.actor.next_module.content.std;
}
// flat: actor, actor_target, critic 0, critic 1, critic target 0, critic target 1 ([W|b] per layer each)
size_t rlt_ref_td3_parameter_count(void* h) {
    auto& ac = static_cast<Loop*>(h)->ts.actor_critic;
    return 2 * mlp_count(mlp_of(ac.actor)) + 4 * mlp_count(mlp_of(ac.critics[0]));
}
void rlt_ref_td3_get_parameters(void* h, float* out) {
    auto& ac = static_cast<Loop*>(h)->ts.actor_critic;
    out = mlp_get(mlp_of(ac.actor), out); out = mlp_get(mlp_of(ac.actor_target), out);
    out = mlp_get(mlp_of(ac.critics[0]), out); out = mlp_get(mlp_of(ac.critics[1]), out);
    out = mlp_get(mlp_of(ac.critics_target[0]), out); mlp_get(mlp_of(ac.critics_target[1]), out);
}
// Adam ages [actor, critic 0, critic 1]
void rlt_ref_td3_get_ages(void* h, uint32_t* out) {
    auto& L = *static_cast<Loop*>(h); auto& ac = L.ts.actor_critic;
    out[0] = (uint32_t)rlt::get(L.device, ac.actor_optimizer.age, 0); out[1] = (uint32_t)rlt::get(L.device, ac.critic_optimizers[0].age, 0);
    out[2] = (uint32_t)rlt::get(L.device, ac.critic_optimizers[1].age, 0);
}
// the batch of the last training step: observations_actions_base [2 x B x 4], rewards [B], terminated [B], and the masks
void rlt_ref_td3_get_batch(void* h, float* oab, float* rewards, uint8_t* terminated, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    auto& b = static_cast<Loop*>(h)->ts.critic_batch;
    std::memcpy(oab, b.observations_actions_base._data, sizeof(float) * 2 * BATCH * 4);
    std::memcpy(rewards, b.rewards._data, sizeof(float) * BATCH);
    for (TI i = 0; i < BATCH; i++) { terminated[i] = b.terminated._data[i]; final_step_mask[i] = b.final_step_mask._data[i]; }
    for (TI i = 0; i < 2 * BATCH; i++) next_final_step_mask_base[i] = b.next_final_step_mask_base._data[i];
}
// the clamped target-action noise of the last training step [B x 1]
void rlt_ref_td3_get_noise(void* h, float* noise) {
    auto& tb = static_cast<Loop*>(h)->ts.critic_training_buffers;
    std::memcpy(noise, rlt::data(tb.target_next_action_noise), sizeof(float) * BATCH);
}

}  // extern "C"
