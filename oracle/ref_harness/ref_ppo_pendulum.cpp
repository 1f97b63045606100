// Harness around the REAL reference (compiled from /root/reference/include where it lies; nothing of it is copied here): runs
// the reference's own PPO-on-Pendulum loop state in two halves per loop step -- (1) collect + critic evaluation + generalized
// advantage estimation, (2) train -- and exposes the dataset, the parameters and the RNG state in between through a small C API,
// so that tests can pin the CPU restatement of GAE and of the PPO update (oracle/) against it.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/rl/environments/pendulum/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/layers/standardize/operations_generic.h>
#include <rl_tools/nn_models/mlp_unconditional_stddev/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/rl/algorithms/ppo/loop/core/config.h>
#include <rl_tools/rl/algorithms/ppo/loop/core/operations_generic.h>

#include <cstdint>
#include <cstring>
#include <sstream>
#include <string>

namespace rlt = rl_tools;

namespace {
using TYPE_POLICY = rlt::numeric_types::Policy<float>;
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;
using TI = typename DEVICE::index_t;
using PENDULUM_SPEC = rlt::rl::environments::pendulum::Specification<float, TI, rlt::rl::environments::pendulum::DefaultParameters<float>>;
using ENVIRONMENT = rlt::rl::environments::Pendulum<PENDULUM_SPEC>;

struct LoopParameters : rlt::rl::algorithms::ppo::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT> {
    static constexpr TI BATCH_SIZE = 64;
    static constexpr TI ACTOR_HIDDEN_DIM = 32;
    static constexpr TI CRITIC_HIDDEN_DIM = 32;
    static constexpr TI ON_POLICY_RUNNER_STEPS_PER_ENV = 40;
    static constexpr TI N_ENVIRONMENTS = 8;
    static constexpr TI STEP_LIMIT = 1000;
    static constexpr TI EPISODE_STEP_LIMIT = 25;       // several truncations inside one dataset
#ifdef RLT_REF_PPO_NORMALIZE                           // second flavour of this harness: running observation normalisation switched on
    static constexpr bool NORMALIZE_OBSERVATIONS = true;
    static constexpr bool NORMALIZE_OBSERVATIONS_CONTINUOUSLY = true;
#endif
    static constexpr auto ACTOR_ACTIVATION_FUNCTION = rlt::nn::activation_functions::ActivationFunction::TANH;
    using ACTOR_OPTIMIZER_PARAMETERS = rlt::nn::optimizers::adam::DEFAULT_PARAMETERS_PYTORCH<TYPE_POLICY>;
    using CRITIC_OPTIMIZER_PARAMETERS = ACTOR_OPTIMIZER_PARAMETERS;
    struct PPO_PARAMETERS : rlt::rl::algorithms::ppo::DefaultParameters<TYPE_POLICY, TI, BATCH_SIZE> {
        static constexpr TI N_EPOCHS = 3;
        static constexpr float GAMMA = 0.9;
        static constexpr float INITIAL_ACTION_STD = 2.0;
    };
};
using CONFIG = rlt::rl::algorithms::ppo::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LoopParameters>;
using STATE = typename CONFIG::template State<CONFIG>;
using PPO_PARAMETERS = typename CONFIG::PPO_SPEC::PARAMETERS;
using DATASET = typename CONFIG::ON_POLICY_RUNNER_DATASET_TYPE;

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
}  // namespace

extern "C" {

void* rlt_ref_ppo_create(uint32_t seed) { return new Loop(seed); }
void rlt_ref_ppo_destroy(void* h) { delete static_cast<Loop*>(h); }

// The loop step (rl/algorithms/ppo/loop/core/operations_generic.h:89-154) in the pieces it is made of, so that tests can look at the
// state between them; rlt_ref_ppo_step runs the reference's own step() for comparison.
void rlt_ref_ppo_step(void* h) { auto& L = *static_cast<Loop*>(h); rlt::step(L.device, L.ts); }
void rlt_ref_ppo_collect(void* h) {
    auto& L = *static_cast<Loop*>(h);
    rlt::collect(L.device, L.ts.on_policy_runner_dataset, L.ts.on_policy_runner, L.ts.ppo.actor, L.ts.actor_eval_buffers, L.ts.rng);
}
// :106-109 / :115-119: both running normalisers take the dataset just collected, and their statistics go into the standardize layers
void rlt_ref_ppo_update_normalizers(void* h) {
    auto& L = *static_cast<Loop*>(h);
    auto& ts = L.ts; auto& device = L.device;
    rlt::copy(device, device, ts.on_policy_runner_dataset.observations, ts.observations_dense);
    rlt::update(device, ts.observation_normalizer, ts.observations_dense);
    rlt::update(device, ts.observation_privileged_normalizer, ts.on_policy_runner_dataset.all_observations_privileged);
    rlt::set_statistics(device, rlt::get_first_layer(ts.ppo.actor), ts.observation_normalizer.mean, ts.observation_normalizer.std);
    rlt::set_statistics(device, ts.ppo.critic.content, ts.observation_privileged_normalizer.mean, ts.observation_privileged_normalizer.std);
}
// :111 re-initialisation of the runner after the warm-up collect
void rlt_ref_ppo_reinit_runner(void* h) {
    auto& L = *static_cast<Loop*>(h);
    rlt::init(L.device, L.ts.on_policy_runner, L.ts.envs, L.ts.env_parameters, L.ts.ppo.actor, L.ts.rng);
}
// [normalize_observations, normalize_observations_continuously, truncate_on_each_iteration]
void rlt_ref_ppo_flags(int* out) {
    out[0] = LoopParameters::NORMALIZE_OBSERVATIONS; out[1] = LoopParameters::NORMALIZE_OBSERVATIONS_CONTINUOUSLY; out[2] = CONFIG::ON_POLICY_RUNNER_SPEC::TRUNCATE_ON_EACH_ITERATION;
}
// runner state: states [n x 2] (theta, theta_dot), episode_step [n], episode_return [n], truncated [n]
void rlt_ref_ppo_get_runner(void* h, float* states, uint32_t* episode_step, float* episode_return, uint8_t* truncated) {
    auto& L = *static_cast<Loop*>(h); auto& r = L.ts.on_policy_runner;
    for (TI e = 0; e < LoopParameters::N_ENVIRONMENTS; e++) {
        auto& st = rlt::get(r.states, 0, e);
        states[2 * e] = st.theta; states[2 * e + 1] = st.theta_dot;
        episode_step[e] = (uint32_t)rlt::get(r.episode_step, 0, e); episode_return[e] = rlt::get(r.episode_return, 0, e); truncated[e] = rlt::get(r.truncated, 0, e);
    }
}
// running normalisers (observation, privileged observation): mean [obs], std [obs] each, ages [2]
void rlt_ref_ppo_get_normalizers(void* h, float* mean, float* std, float* mean_privileged, float* std_privileged, uint32_t* ages) {
    auto& ts = static_cast<Loop*>(h)->ts;
    constexpr TI D = ENVIRONMENT::Observation::DIM;
    std::memcpy(mean, ts.observation_normalizer.mean._data, sizeof(float) * D); std::memcpy(std, ts.observation_normalizer.std._data, sizeof(float) * D);
    std::memcpy(mean_privileged, ts.observation_privileged_normalizer.mean._data, sizeof(float) * D); std::memcpy(std_privileged, ts.observation_privileged_normalizer.std._data, sizeof(float) * D);
    ages[0] = (uint32_t)ts.observation_normalizer.age; ages[1] = (uint32_t)ts.observation_privileged_normalizer.age;
}
// the standardize layers in front of actor and critic: mean [obs], precision [obs] each
void rlt_ref_ppo_get_standardize(void* h, float* actor_mean, float* actor_precision, float* critic_mean, float* critic_precision) {
    auto& L = *static_cast<Loop*>(h); auto& ts = L.ts;
    constexpr TI D = ENVIRONMENT::Observation::DIM;
    auto& a = rlt::get_first_layer(ts.ppo.actor); auto& c = ts.ppo.critic.content;
    for (TI i = 0; i < D; i++) {
        actor_mean[i] = rlt::get(L.device, a.mean.parameters, i); actor_precision[i] = rlt::get(L.device, a.precision.parameters, i);
        critic_mean[i] = rlt::get(L.device, c.mean.parameters, i); critic_precision[i] = rlt::get(L.device, c.precision.parameters, i);
    }
}
void rlt_ref_ppo_values_and_gae(void* h);
void rlt_ref_ppo_collect_and_gae(void* h) { rlt_ref_ppo_collect(h); rlt_ref_ppo_values_and_gae(h); }
// :122-136 critic on all observations, then the advantage estimate
void rlt_ref_ppo_values_and_gae(void* h) {
    auto& L = *static_cast<Loop*>(h);
    auto& ts = L.ts; auto& device = L.device;
    constexpr TI STEPS = 1, FORWARD_BATCH_SIZE = CONFIG::ON_POLICY_RUNNER_DATASET_SPEC::STEPS_TOTAL_ALL;
    auto obs = rlt::to_tensor(device, ts.on_policy_runner_dataset.all_observations_privileged);
    auto obs_r = rlt::reshape_row_major(device, obs, rlt::tensor::Shape<TI, STEPS, FORWARD_BATCH_SIZE, decltype(obs)::SHAPE::LAST>{});
    auto val = rlt::to_tensor(device, ts.on_policy_runner_dataset.all_values);
    auto val_r = rlt::reshape_row_major(device, val, rlt::tensor::Shape<TI, STEPS, FORWARD_BATCH_SIZE, 1>{});
    auto rst = rlt::to_tensor(device, ts.on_policy_runner_dataset.all_reset);
    auto rst_r = rlt::reshape_row_major(device, rst, rlt::tensor::Shape<TI, STEPS, FORWARD_BATCH_SIZE, 1>{});
    rlt::Mode<rlt::nn::layers::gru::ResetMode<rlt::mode::Rollout<>, rlt::nn::layers::gru::ResetModeSpecification<TI, decltype(rst_r)>>> mode;
    mode.reset_container = rst_r;
    rlt::evaluate(device, ts.ppo.critic, obs_r, val_r, ts.critic_buffers_gae, ts.rng, mode);
    rlt::estimate_generalized_advantages(device, ts.on_policy_runner_dataset, PPO_PARAMETERS{});
}
// second half: the PPO update itself (rl/algorithms/ppo/operations_generic.h:96-330)
void rlt_ref_ppo_train(void* h) {
    auto& L = *static_cast<Loop*>(h);
    auto& ts = L.ts;
    rlt::train(L.device, ts.ppo, ts.on_policy_runner_dataset, ts.actor_optimizer, ts.critic_optimizer, ts.ppo_buffers, ts.actor_buffers, ts.critic_buffers, ts.rng);
    ts.step++;
}

// [n_envs, steps_per_env, data_dim, rows, obs_dim, action_dim, batch, epochs, actor_hidden, critic_hidden, episode_step_limit]
void rlt_ref_ppo_dims(int* out) {
    out[0] = LoopParameters::N_ENVIRONMENTS; out[1] = LoopParameters::ON_POLICY_RUNNER_STEPS_PER_ENV; out[2] = DATASET::DATA_DIM;
    out[3] = DATASET::STEPS_TOTAL + LoopParameters::N_ENVIRONMENTS; out[4] = ENVIRONMENT::Observation::DIM; out[5] = ENVIRONMENT::ACTION_DIM;
    out[6] = LoopParameters::BATCH_SIZE; out[7] = PPO_PARAMETERS::N_EPOCHS; out[8] = LoopParameters::ACTOR_HIDDEN_DIM; out[9] = LoopParameters::CRITIC_HIDDEN_DIM;
    out[10] = LoopParameters::EPISODE_STEP_LIMIT;
}
// [gamma, lambda, epsilon_clip, action_entropy_coefficient, advantage_epsilon, normalize_advantage, learn_action_std, adam alpha, beta_1, beta_2, epsilon, epsilon_sqrt]
void rlt_ref_ppo_hyperparameters(void* h, float* out) {
    auto& ts = static_cast<Loop*>(h)->ts;
    out[0] = PPO_PARAMETERS::GAMMA; out[1] = PPO_PARAMETERS::LAMBDA; out[2] = PPO_PARAMETERS::EPSILON_CLIP; out[3] = PPO_PARAMETERS::ACTION_ENTROPY_COEFFICIENT;
    out[4] = PPO_PARAMETERS::ADVANTAGE_EPSILON; out[5] = PPO_PARAMETERS::NORMALIZE_ADVANTAGE; out[6] = PPO_PARAMETERS::LEARN_ACTION_STD;
    auto& p = rlt::get_ref(static_cast<Loop*>(h)->device, ts.actor_optimizer.parameters, 0);
    out[7] = p.alpha; out[8] = p.beta_1; out[9] = p.beta_2; out[10] = p.epsilon; out[11] = p.epsilon_sqrt;
}
// column of each dataset view inside a dataset row, in this order: all_observations_privileged, observations, actions_mean, actions,
// action_log_probs, rewards, terminated, truncated, all_reset, reset, all_values, values, advantages, target_values
void rlt_ref_ppo_columns(void* h, int* out) {
    auto& d = static_cast<Loop*>(h)->ts.on_policy_runner_dataset;
    const float* base = d.data._data;
    int i = 0;
    out[i++] = (int)(d.all_observations_privileged._data - base); out[i++] = (int)(d.observations._data - base);
    out[i++] = (int)(d.actions_mean._data - base); out[i++] = (int)(d.actions._data - base); out[i++] = (int)(d.action_log_probs._data - base);
    out[i++] = (int)(d.rewards._data - base); out[i++] = (int)(d.terminated._data - base); out[i++] = (int)(d.truncated._data - base);
    out[i++] = (int)(d.all_reset._data - base); out[i++] = (int)(d.reset._data - base); out[i++] = (int)(d.all_values._data - base);
    out[i++] = (int)(d.values._data - base); out[i++] = (int)(d.advantages._data - base); out[i++] = (int)(d.target_values._data - base);
}
void rlt_ref_ppo_get_dataset(void* h, float* out) {
    auto& d = static_cast<Loop*>(h)->ts.on_policy_runner_dataset;
    std::memcpy(out, d.data._data, sizeof(float) * (DATASET::STEPS_TOTAL + LoopParameters::N_ENVIRONMENTS) * DATASET::DATA_DIM);
}
// flat: actor [W|b per layer], actor log_std, critic [W|b per layer]
size_t rlt_ref_ppo_parameter_count(void* h) {
    auto& ts = static_cast<Loop*>(h)->ts;
    return mlp_count(rlt::get_last_layer(ts.ppo.actor)) + ENVIRONMENT::ACTION_DIM + mlp_count(rlt::get_last_layer(ts.ppo.critic));
}
void rlt_ref_ppo_get_parameters(void* h, float* out) {
    auto& ts = static_cast<Loop*>(h)->ts;
    auto& actor = rlt::get_last_layer(ts.ppo.actor);
    out = mlp_get(actor, out);
    std::memcpy(out, actor.log_std.parameters._data, sizeof(float) * ENVIRONMENT::ACTION_DIM); out += ENVIRONMENT::ACTION_DIM;
    mlp_get(rlt::get_last_layer(ts.ppo.critic), out);
}
// the optimisers' step counters (1 before the first update)
void rlt_ref_ppo_get_ages(void* h, uint32_t* out) {
    auto& ts = static_cast<Loop*>(h)->ts;
    auto& device = static_cast<Loop*>(h)->device;
    out[0] = (uint32_t)rlt::get(device, ts.actor_optimizer.age, 0); out[1] = (uint32_t)rlt::get(device, ts.critic_optimizer.age, 0);
}
// textual state of the loop's std::mt19937 (operator<<), NUL terminated; returns the length needed
int rlt_ref_ppo_get_rng_state(void* h, char* buffer, int capacity) {
    std::stringstream ss;
    ss << static_cast<Loop*>(h)->ts.rng.engine;
    const std::string s = ss.str();
    if ((int)s.size() + 1 <= capacity) std::memcpy(buffer, s.c_str(), s.size() + 1);
    return (int)s.size() + 1;
}

}  // extern "C"
