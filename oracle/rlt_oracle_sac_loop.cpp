// CPU restatement of the reference's SAC training loop on Pendulum, including its random-number stream
// (test infrastructure only, see rlt_oracle.h). Reference paths are relative to /root/reference/include/rl_tools/.
//
// The reference's CPU device draws everything from one std::mt19937 seeded with seed+1 through libstdc++'s
// distributions (random/operations_cpu.h:21-47), constructing a fresh distribution object per draw. The same
// calls are made here in the same order, so with the same libstdc++ the streams coincide:
//   init: actor, critic 0, critic 1 weights (rl/algorithms/sac/operations_generic.h:112-131; per dense layer and per
//         output row: bias then the row's weights, nn/layers/dense/operations_generic.h:60-87)
//   step: [reset: theta, theta_dot] -> policy noise -> per sample (env index, offset) -> critic noise -> actor noise
//         (rl/algorithms/sac/loop/core/operations_generic.h:110-155)
#include "rlt_oracle.h"
#include "rlt_oracle_sac_loop.h"

#include <cmath>
#include <cstring>
#include <random>
#include <vector>

namespace {

struct Net {
    std::vector<int> dims;       // in, hidden..., out
    std::vector<int> acts;
    std::vector<float> params, grads, m, v;
    std::vector<std::vector<float>> pre, out;
    std::vector<rlt_dense_layer> layers;
    std::vector<rlt_adam_tensor> adam;
    uint32_t age = 1;
    void build(const std::vector<int>& d, int hidden_act, int batch, bool trainable) {
        dims = d;
        int n = (int)d.size() - 1;
        size_t total = 0;
        for (int l = 0; l < n; l++) total += (size_t)d[l] * d[l + 1] + d[l + 1];
        params.assign(total, 0);
        if (trainable) { grads.assign(total, 0); m.assign(total, 0); v.assign(total, 0); pre.resize(n); out.resize(n); }
        layers.resize(n); adam.clear();
        size_t off = 0;
        for (int l = 0; l < n; l++) {
            rlt_dense_layer& L = layers[l];
            std::memset(&L, 0, sizeof L);
            L.in_dim = d[l]; L.out_dim = d[l + 1]; L.activation = (l == n - 1) ? RLT_ACT_IDENTITY : hidden_act;
            size_t nw = (size_t)d[l] * d[l + 1], nb = d[l + 1];
            L.weights = params.data() + off; L.biases = params.data() + off + nw;
            if (trainable) {
                L.d_weights = grads.data() + off; L.d_biases = grads.data() + off + nw;
                pre[l].assign((size_t)batch * d[l + 1], 0); out[l].assign((size_t)batch * d[l + 1], 0);
                L.pre_activations = pre[l].data(); L.output = out[l].data();
                rlt_adam_tensor tw = {L.weights, L.d_weights, m.data() + off, v.data() + off, nullptr, (uint32_t)nw, 1u};
                rlt_adam_tensor tb = {L.biases, L.d_biases, m.data() + off + nw, v.data() + off + nw, nullptr, (uint32_t)nb, 2u};
                adam.push_back(tw); adam.push_back(tb);
            }
            off += nw + nb;
        }
    }
};

// nn/layers/dense/operations_generic.h:60-87, legacy Kaiming-uniform (layer.h:28-39)
void init_weights(Net& net, std::mt19937& rng) {
    for (auto& L : net.layers) {
        float negative_slope = std::sqrt(5.0f);
        float gain = std::sqrt(2.0f / (1 + negative_slope * negative_slope));
        float fan = (float)L.in_dim;
        float sd = gain / std::sqrt(fan);
        float weight_bound = std::sqrt(3.0f) * sd;
        float bias_bound = 1 / std::sqrt((float)L.in_dim);
        for (int i = 0; i < L.out_dim; i++) {
            L.biases[i] = std::uniform_real_distribution<float>(-bias_bound, bias_bound)(rng);
            for (int j = 0; j < L.in_dim; j++) L.weights[(size_t)i * L.in_dim + j] = std::uniform_real_distribution<float>(-weight_bound, weight_bound)(rng);
        }
    }
}
// random/operations_cpu.h:38-47
inline float normal_sample(std::mt19937& rng) { return (float)std::normal_distribution<float>(0.0f, 1.0f)(rng); }

}  // namespace

struct rlt_oracle_sac_loop {
    rlt_oracle_sac_loop_config cfg;
    std::mt19937 rng;
    Net actor, critics[2], targets[2];
    float log_alpha[4] = {0, 0, 0, 0};  // parameter, gradient, m, v
    uint32_t alpha_age = 1;
    rlt_sac_agent agent;
    rlt_replay_buffer rb;
    rlt_pendulum_runner runner;
    // storage
    std::vector<float> rb_data; std::vector<uint32_t> rb_episode_start;
    uint32_t rb_position = 0, rb_current_episode_start = 0; uint8_t rb_full = 0;
    float state[2] = {0, 0}; uint32_t episode_step = 0; float episode_return = 0; uint8_t truncated = 1;
    std::vector<float> oab, rewards, nsavi, next_q[2], next_lp, target_q, d_out_c[2], savi, d_out_a, d_ci[2], d_aos, d_ao, a_pre, a_lp, a_act;
    std::vector<uint8_t> terminated, m_reset, m_next_reset, m_final, m_next_final;
    std::vector<float> noise_critic, noise_actor;
    std::vector<uint32_t> env_indices, sample_offsets;
    float last_rollout_noise = 0, last_action = 0, last_initial_state[2] = {0, 0};
    uint8_t last_reset = 0;
    uint32_t step = 0;
    bool previous_policy_set = false; int previous_policy = 0;
    float last_critic_loss[2] = {0, 0};
};

extern "C" {

rlt_oracle_sac_loop* rlt_oracle_sac_loop_create(const rlt_oracle_sac_loop_config* c) {
    if (!c || c->batch <= 0 || c->hidden_dim <= 0 || c->replay_capacity <= 0) return nullptr;
    auto* S = new rlt_oracle_sac_loop();
    S->cfg = *c;
    const int B = c->batch, H = c->hidden_dim, OBS = 3, ACT = 1, D = OBS + ACT;
    S->rng = std::mt19937(static_cast<std::mt19937::result_type>(c->seed + 1));     // random/operations_cpu.h:21-24
    S->actor.build({OBS, H, H, 2 * ACT}, RLT_ACT_RELU, B, true);
    for (int k = 0; k < 2; k++) { S->critics[k].build({D, H, H, 1}, RLT_ACT_RELU, B, true); S->targets[k].build({D, H, H, 1}, RLT_ACT_RELU, B, false); }
    // rl/algorithms/sac/operations_generic.h:112-131
    init_weights(S->actor, S->rng);
    S->log_alpha[0] = std::log(0.5f);                                                // sample_and_squash/operations_generic.h:76-80, sac.h:27
    init_weights(S->critics[0], S->rng);
    init_weights(S->critics[1], S->rng);
    for (int k = 0; k < 2; k++) std::copy(S->critics[k].params.begin(), S->critics[k].params.end(), S->targets[k].params.begin());  // :128-129
    // replay buffer + runner (off_policy_runner/operations_generic.h:166-181: truncated initialised to true)
    const int R = 2 * OBS + ACT + 3;
    S->rb_data.assign((size_t)c->replay_capacity * R, 0); S->rb_episode_start.assign(c->replay_capacity, 0);
    S->rb = {S->rb_data.data(), S->rb_episode_start.data(), &S->rb_position, &S->rb_current_episode_start, &S->rb_full, 1, c->replay_capacity, OBS, ACT};
    S->runner = {S->state, &S->episode_step, &S->episode_return, &S->truncated, 1, c->episode_step_limit, {10.0f, 8.0f, 2.0f, 0.05f, 1.0f, 1.0f}};
    // batch + training buffers
    S->oab.assign((size_t)2 * B * D, 0); S->rewards.assign(B, 0); S->terminated.assign(B, 0);
    S->m_reset.assign(B, 0); S->m_next_reset.assign(2 * B, 0); S->m_final.assign(B, 0); S->m_next_final.assign(2 * B, 0);
    S->nsavi.assign((size_t)B * D, 0); S->savi.assign((size_t)B * D, 0);
    for (int k = 0; k < 2; k++) { S->next_q[k].assign(B, 0); S->d_out_c[k].assign(B, 0); S->d_ci[k].assign((size_t)B * D, 0); }
    S->next_lp.assign(B, 0); S->target_q.assign(B, 0); S->d_out_a.assign(B, 0); S->d_aos.assign((size_t)B * ACT, 0); S->d_ao.assign((size_t)B * 2 * ACT, 0);
    S->a_pre.assign((size_t)B * ACT, 0); S->a_lp.assign(B, 0); S->a_act.assign((size_t)B * ACT, 0);
    S->noise_critic.assign((size_t)B * ACT, 0); S->noise_actor.assign((size_t)B * ACT, 0);
    S->env_indices.assign(B, 0); S->sample_offsets.assign(B, 0);
    rlt_sac_agent& A = S->agent;
    std::memset(&A, 0, sizeof A);
    A.batch = B; A.observation_dim = OBS; A.action_dim = ACT; A.n_actor_layers = 3; A.n_critic_layers = 3;
    A.gamma = 0.99f; A.polyak = (float)(1.0 - 0.005);                                 // sac.h:13,19
    A.sas = {-20.0f, 2.0f, 1e-6f, -(float)ACT};                                      // sac.h:25-31
    rlt_adam_parameters ap = {1e-3f, 0.9f, 0.999f, c->adam_epsilon, c->adam_epsilon, 0, 1, 0, 0, 0, 1};   // adam.h:26-48
    A.actor_adam = ap; A.critic_adam = ap; A.alpha_adam = ap;
    A.actor = S->actor.layers.data();
    A.actor_adam_tensors = S->actor.adam.data(); A.n_actor_adam_tensors = (int)S->actor.adam.size();
    for (int k = 0; k < 2; k++) {
        A.critics[k] = S->critics[k].layers.data(); A.critics_target[k] = S->targets[k].layers.data();
        A.critic_adam_tensors[k] = S->critics[k].adam.data(); A.critic_age[k] = &S->critics[k].age;
        A.next_q[k] = S->next_q[k].data(); A.d_output_critic[k] = S->d_out_c[k].data(); A.d_critic_input[k] = S->d_ci[k].data();
    }
    A.n_critic_adam_tensors = (int)S->critics[0].adam.size();
    A.log_alpha = {&S->log_alpha[0], &S->log_alpha[1], &S->log_alpha[2], &S->log_alpha[3], nullptr, 1u, 0u};
    A.actor_age = &S->actor.age; A.alpha_age = &S->alpha_age;
    A.observations_actions_base = S->oab.data(); A.rewards = S->rewards.data(); A.terminated = S->terminated.data();
    A.final_step_mask = S->m_final.data(); A.next_final_step_mask = S->m_next_final.data() + B; A.reset = S->m_reset.data();
    A.next_state_action_value_input = S->nsavi.data(); A.next_log_probabilities = S->next_lp.data(); A.target_action_value = S->target_q.data();
    A.state_action_value_input = S->savi.data(); A.d_output_actor_critics = S->d_out_a.data();
    A.d_actor_output_squashing = S->d_aos.data(); A.d_actor_output = S->d_ao.data();
    A.actor_pre_squashing = S->a_pre.data(); A.actor_log_probabilities = S->a_lp.data(); A.actor_actions = S->a_act.data();
    return S;
}

void rlt_oracle_sac_loop_destroy(rlt_oracle_sac_loop* S) { delete S; }

// rl/algorithms/sac/loop/core/operations_generic.h:110-155
int rlt_oracle_sac_loop_step(rlt_oracle_sac_loop* S) {
    if (!S) return RLT_E_INVALID_ARGUMENT;
    const rlt_oracle_sac_loop_config& c = S->cfg;
    const int B = c.batch;
    int rc;
    // ---- off-policy runner step (rl/components/off_policy_runner/operations_generic.h:216-238)
    int policy = S->step >= (uint32_t)c.n_warmup_steps ? 1 : 0;
    if (S->previous_policy_set && policy != S->previous_policy) S->truncated = 1;                // truncate_all on a policy switch
    float initial_state[2] = {0, 0};
    S->last_reset = S->truncated;
    if (S->truncated) {                                                                          // pendulum/operations_generic.h:58-61
        initial_state[0] = std::uniform_real_distribution<float>(-(float)M_PI, (float)M_PI)(S->rng);
        initial_state[1] = std::uniform_real_distribution<float>(-1.0f, 1.0f)(S->rng);
    }
    S->last_initial_state[0] = initial_state[0]; S->last_initial_state[1] = initial_state[1];
    float action_in = 0, noise = 0;
    if (policy == 0) action_in = std::uniform_real_distribution<float>(-1.0f, 1.0f)(S->rng);     // nn_models/random_uniform/operations_generic.h:28-44
    else noise = normal_sample(S->rng);                                                          // sample_and_squash Rollout mode, operations_generic.h:163-166
    S->last_rollout_noise = noise;
    rlt_sas_parameters sas = S->agent.sas;
    rc = rlt_oracle_pendulum_runner_step(&S->runner, &S->rb, policy == 0 ? 0 : 2, S->actor.layers.data(), 3, &sas, &action_in, &noise, initial_state);
    if (rc) return rc;
    { uint32_t last = S->rb_position == 0 ? (uint32_t)S->cfg.replay_capacity - 1 : S->rb_position - 1; S->last_action = S->rb_data[(size_t)last * 10 + 3]; }
    S->previous_policy = policy; S->previous_policy_set = true;
    // ---- training (loop/core/operations_generic.h:126-151; all intervals are 1, SHARED_BATCH)
    bool train = S->step >= (uint32_t)c.n_warmup_steps;
    if (train) {
        for (int i = 0; i < B; i++) {                                                            // off_policy_runner/operations_generic.h:421-430, :304
            S->env_indices[i] = (uint32_t)std::uniform_int_distribution<size_t>(0, 0)(S->rng);
            size_t eligible = S->rb_full ? (size_t)c.replay_capacity : (size_t)S->rb_position;
            S->sample_offsets[i] = (uint32_t)std::uniform_int_distribution<size_t>(0, eligible - 1)(S->rng);
        }
        rc = rlt_oracle_gather_batch(&S->rb, S->env_indices.data(), S->sample_offsets.data(), 0, c.episode_step_limit, B,
                                     S->oab.data(), S->rewards.data(), S->terminated.data(), S->m_reset.data(), S->m_next_reset.data(),
                                     S->m_final.data(), S->m_next_final.data());
        if (rc) return rc;
        for (auto& x : S->noise_critic) x = normal_sample(S->rng);                               // containers/matrix/operations_generic.h:632-639
        for (int k = 0; k < 2; k++) {
            if ((rc = rlt_oracle_sac_train_critic(&S->agent, k, S->noise_critic.data()))) return rc;
            const float* q = S->critics[k].layers[2].output;                                      // mse::evaluate with the loss weight 0.5 (sac/operations_generic.h:327)
            rlt_oracle_mse_evaluate(q, 1, S->target_q.data(), 1, B, 1, 0.5f, &S->last_critic_loss[k]);
        }
        if ((rc = rlt_oracle_sac_update_critic_targets(&S->agent))) return rc;
        for (auto& x : S->noise_actor) x = normal_sample(S->rng);
        if ((rc = rlt_oracle_sac_train_actor(&S->agent, S->noise_actor.data()))) return rc;
    }
    S->step++;
    return 0;
}

const rlt_sac_agent* rlt_oracle_sac_loop_agent(rlt_oracle_sac_loop* S) { return &S->agent; }
const rlt_replay_buffer* rlt_oracle_sac_loop_replay(rlt_oracle_sac_loop* S) { return &S->rb; }
const rlt_pendulum_runner* rlt_oracle_sac_loop_runner(rlt_oracle_sac_loop* S) { return &S->runner; }
const float* rlt_oracle_sac_loop_noise_critic(rlt_oracle_sac_loop* S) { return S->noise_critic.data(); }
const float* rlt_oracle_sac_loop_noise_actor(rlt_oracle_sac_loop* S) { return S->noise_actor.data(); }
const uint32_t* rlt_oracle_sac_loop_env_indices(rlt_oracle_sac_loop* S) { return S->env_indices.data(); }
const uint32_t* rlt_oracle_sac_loop_sample_offsets(rlt_oracle_sac_loop* S) { return S->sample_offsets.data(); }
uint32_t rlt_oracle_sac_loop_step_count(rlt_oracle_sac_loop* S) { return S->step; }
float rlt_oracle_sac_loop_critic_loss(rlt_oracle_sac_loop* S, int k) { return S->last_critic_loss[k & 1]; }
void rlt_oracle_sac_loop_last_env_step(rlt_oracle_sac_loop* S, float* out6) {
    out6[0] = S->last_reset; out6[1] = S->last_initial_state[0]; out6[2] = S->last_initial_state[1];
    out6[3] = S->last_rollout_noise; out6[4] = S->last_action; out6[5] = S->episode_return;
}
size_t rlt_oracle_sac_loop_parameter_count(rlt_oracle_sac_loop* S) {
    return S->actor.params.size() + 2 * S->critics[0].params.size() + 2 * S->targets[0].params.size() + 1;
}
// flat order: actor, critic 0, critic 1, target 0, target 1, log_alpha ; per network: per layer [weights, biases]
void rlt_oracle_sac_loop_get_parameters(rlt_oracle_sac_loop* S, float* out) {
    size_t o = 0;
    auto put = [&](const std::vector<float>& v) { std::memcpy(out + o, v.data(), sizeof(float) * v.size()); o += v.size(); };
    put(S->actor.params); put(S->critics[0].params); put(S->critics[1].params); put(S->targets[0].params); put(S->targets[1].params);
    out[o] = S->log_alpha[0];
}

}  // extern "C"
