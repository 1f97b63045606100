// CPU restatement of the reference's sequential models with GRU layers and of SAC's train_critic / train_actor on sequence batches
// (test infrastructure only, see rlt_oracle.h). Reference paths are relative to /root/reference/include/rl_tools/.
//
// A sequential model (nn_models/sequential/operations_generic.h) hands the output every layer keeps to the next layer; dense layers see the
// [steps x batch x dim] tensors as steps*batch rows (nn/layers/dense/layer.h:52-54), GRU layers walk the steps. evaluate and forward
// compute the same values (evaluate keeps its intermediates in buffers instead of in the layer), so both are stated as forward here.
#include "rlt_oracle.h"

#include <cmath>
#include <cstring>
#include <vector>

namespace {

// math/operations_generic.h:247-251
inline float fast_tanh_(float x) {
    x = x < -3.0f ? -3.0f : (x > 3.0f ? 3.0f : x);
    float x2 = x * x;
    return x * (27 + x2) / (27 + 9 * x2);
}

int layer_in(const rlt_seq_layer& L) { return L.kind ? L.gru.input_dim : L.dense.in_dim; }
int layer_out(const rlt_seq_layer& L) { return L.kind ? L.gru.hidden_dim : L.dense.out_dim; }
const float* layer_output(const rlt_seq_layer& L) { return L.kind ? L.gru.output : L.dense.output; }

bool layers_ok(const rlt_seq_layer* layers, int n) {
    if (!layers || n <= 0) return false;
    for (int l = 0; l < n; l++) {
        if (layers[l].kind != 0 && layers[l].kind != 1) return false;
        if (l && layer_in(layers[l]) != layer_out(layers[l - 1])) return false;
        if (l + 1 < n && !layer_output(layers[l])) return false;
    }
    return true;
}

int adam_over(const rlt_adam_tensor* t, int n, const rlt_adam_parameters* p, uint32_t* age) { return rlt_oracle_adam_step(t, n, p, age, 0.0f, nullptr); }

}  // namespace

extern "C" {

// nn_models/sequential/operations_generic.h:329-336 (_forward), :277-298 (_evaluate)
int rlt_oracle_seq_forward(const rlt_seq_layer* layers, int n, const float* x, int ldx, const uint8_t* reset, int steps, int batch) {
    if (!layers_ok(layers, n) || !x || steps <= 0 || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    const float* in = x; int ld = ldx, rc;
    for (int l = 0; l < n; l++) {
        const rlt_seq_layer& L = layers[l];
        if (L.kind == 0) {
            if ((rc = rlt_oracle_dense_forward(&L.dense, in, ld, nullptr, 0, steps * batch))) return rc;
        } else {
            if (ld != L.gru.input_dim) return RLT_E_INVALID_ARGUMENT;
            if ((rc = rlt_oracle_gru_forward(&L.gru, in, reset, steps, batch))) return rc;
        }
        in = layer_output(L); ld = layer_out(L);
    }
    return 0;
}

// :369-428: backward (no d_input: the first layer runs `backward`, the others `backward_full`), backward_full, and backward_input, whose inner
// calls (:405-406) drop the mode -- with more than one layer the GRU layers then see no resets (reset_in_backward_input = 0).
int rlt_oracle_seq_backward(const rlt_seq_layer* layers, int n, const float* x, int ldx, float* d_output, float* d_input, const uint8_t* reset, int steps, int batch,
                            int want_w, int reset_in_backward_input) {
    if (!layers_ok(layers, n) || !d_output || steps <= 0 || batch <= 0 || (want_w && !x)) return RLT_E_INVALID_ARGUMENT;
    const int rows = steps * batch;
    const uint8_t* reset_here = (want_w || reset_in_backward_input || n == 1) ? reset : nullptr;
    std::vector<float> tick_tock[2];      // the gradient buffers between the layers (the reference's tick / tock)
    int which = 0;
    float* d_cur = d_output; int rc;
    for (int l = n - 1; l >= 0; l--) {
        const rlt_seq_layer& L = layers[l];
        const float* in = l ? layer_output(layers[l - 1]) : x;
        const int ld_in = l ? layer_out(layers[l - 1]) : ldx;
        float* d_in = nullptr;
        if (l > 0) { tick_tock[which].assign((size_t)rows * layer_in(L), 0.0f); d_in = tick_tock[which].data(); which ^= 1; }
        else d_in = d_input;
        if (L.kind == 0) {
            if (want_w && d_in) rc = rlt_oracle_dense_backward_full(&L.dense, in, ld_in, d_cur, L.dense.out_dim, d_in, L.dense.in_dim, rows);
            else if (want_w) rc = rlt_oracle_dense_backward(&L.dense, in, ld_in, d_cur, L.dense.out_dim, rows);
            else rc = d_in ? rlt_oracle_dense_backward_input(&L.dense, d_cur, L.dense.out_dim, d_in, L.dense.in_dim, rows) : 0;
        } else {
            if (want_w && ld_in != L.gru.input_dim) return RLT_E_INVALID_ARGUMENT;
            rc = rlt_oracle_gru_backward(&L.gru, in, d_cur, d_in, reset_here, steps, batch, want_w);
        }
        if (rc) return rc;
        d_cur = d_in;
    }
    return 0;
}

// :349-354
int rlt_oracle_seq_zero_gradient(const rlt_seq_layer* layers, int n) {
    if (!layers_ok(layers, n)) return RLT_E_INVALID_ARGUMENT;
    for (int l = 0; l < n; l++) {
        if (layers[l].kind == 0) {
            const rlt_dense_layer& D = layers[l].dense;
            if (!D.d_weights || !D.d_biases) return RLT_E_INVALID_ARGUMENT;
            std::memset(D.d_weights, 0, sizeof(float) * D.in_dim * D.out_dim); std::memset(D.d_biases, 0, sizeof(float) * D.out_dim);
        } else {
            const rlt_gru_layer& G = layers[l].gru;
            if (!G.d_weights_input || !G.d_biases_input || !G.d_weights_hidden || !G.d_biases_hidden) return RLT_E_INVALID_ARGUMENT;
            const size_t H = G.hidden_dim, I = G.input_dim;
            std::memset(G.d_weights_input, 0, sizeof(float) * 3 * H * I); std::memset(G.d_biases_input, 0, sizeof(float) * 3 * H);
            std::memset(G.d_weights_hidden, 0, sizeof(float) * 3 * H * H); std::memset(G.d_biases_hidden, 0, sizeof(float) * 3 * H);
        }
    }
    return 0;
}

// reset(model, state, mode): nn_models/sequential/operations_generic.h:35-41 walks the layers; a GRU layer (nn/layers/gru/operations_generic.h:87-120) starts
// the masked rows (all rows without a mask) again from the initial hidden state, step counter 0
int rlt_oracle_seq_reset_state(const rlt_seq_layer* layers, int n, const rlt_seq_state* state, const uint8_t* mask, int batch) {
    if (!layers || n <= 0 || n > RLT_SEQ_MAX_LAYERS || !state || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int l = 0; l < n; l++) {
        if (!layers[l].kind) continue;
        const rlt_gru_layer& G = layers[l].gru;
        if (!state->hidden[l] || !state->step[l]) return RLT_E_INVALID_ARGUMENT;
        for (int b = 0; b < batch; b++)
            if (!mask || mask[b]) { state->step[l][b] = 0; std::memcpy(state->hidden[l] + (size_t)b * G.hidden_dim, G.initial_hidden_state, sizeof(float) * G.hidden_dim); }
    }
    return 0;
}

// evaluate_step: nn_models/sequential/operations_generic.h:303-327 (tick / tock between the layers); dense layers evaluate; a GRU layer
// (nn/layers/gru/operations_generic.h:348-416) runs the arithmetic of one forward step on its state, in the same order of operations
int rlt_oracle_seq_evaluate_step(const rlt_seq_layer* layers, int n, const float* x, int ldx, const rlt_seq_state* state, int auto_reset_period, float* y, int ldy, int batch) {
    if (!layers || n <= 0 || n > RLT_SEQ_MAX_LAYERS || !x || !state || !y || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    std::vector<float> buffers[2];
    const float* in = x; int ld = ldx, which = 0, rc;
    for (int l = 0; l < n; l++) {
        const rlt_seq_layer& L = layers[l];
        const int out_dim = layer_out(L);
        float* out = y; int ldo = ldy;
        if (l + 1 < n) { buffers[which].assign((size_t)batch * out_dim, 0.0f); out = buffers[which].data(); ldo = out_dim; which ^= 1; }
        if (L.kind == 0) {
            if ((rc = rlt_oracle_dense_evaluate(&L.dense, in, ld, out, ldo, batch))) return rc;
        } else {
            const rlt_gru_layer& G = L.gru;
            const int H = G.hidden_dim, I = G.input_dim, H3 = 3 * H;
            float* hidden = state->hidden[l]; uint32_t* step = state->step[l];
            if (!hidden || !step) return RLT_E_INVALID_ARGUMENT;
            for (int b = 0; b < batch; b++)                                  // reset_truncate (:76-86)
                if (auto_reset_period > 0 && step[b] >= (uint32_t)auto_reset_period) { std::memcpy(hidden + (size_t)b * H, G.initial_hidden_state, sizeof(float) * H); step[b] = 0; }
            std::vector<float> post((size_t)batch * H3), npp((size_t)batch * H);
            for (int b = 0; b < batch; b++) {
                const float* hp = hidden + (size_t)b * H; const float* xb = in + (size_t)b * ld;
                float* p = &post[(size_t)b * H3];
                for (int j = 0; j < H3; j++) {                              // W_h h + b_h (:373)
                    float acc = G.biases_hidden[j];
                    for (int k = 0; k < H; k++) acc += hp[k] * G.weights_hidden[(size_t)j * H + k];
                    p[j] = acc;
                }
                for (int j = 0; j < H; j++) { npp[(size_t)b * H + j] = p[2 * H + j]; p[2 * H + j] = 0; }       // :375-376
                for (int j = 0; j < H3; j++) {                              // += W_i x + b_i (:378)
                    float acc = p[j] + G.biases_input[j];
                    for (int k = 0; k < I; k++) acc += xb[k] * G.weights_input[(size_t)j * I + k];
                    p[j] = acc;
                }
                for (int j = 0; j < 2 * H; j++) p[j] = G.fast_tanh ? 0.5f * fast_tanh_(0.5f * p[j]) + 0.5f : 1 / (1 + std::exp(-p[j]));      // :379-387
                for (int j = 0; j < H; j++) p[2 * H + j] += npp[(size_t)b * H + j] * p[j];                                                   // :388
                for (int j = 0; j < H; j++) p[2 * H + j] = G.fast_tanh ? fast_tanh_(p[2 * H + j]) : std::tanh(p[2 * H + j]);                // :389-397
                for (int j = 0; j < H; j++) {
                    float o = 1 - p[H + j];                                  // one_minus (:398)
                    o = o * p[2 * H + j];                                    // multiply (:403)
                    o += p[H + j] * hp[j];                                   // multiply_accumulate with the previous state (:404)
                    out[(size_t)b * ldo + j] = o;
                }
            }
            for (int b = 0; b < batch; b++) {                                // the new state; auto-reset (:405-415)
                std::memcpy(hidden + (size_t)b * H, out + (size_t)b * ldo, sizeof(float) * H);
                uint32_t new_step = step[b] + 1;
                if (auto_reset_period > 0 && new_step >= (uint32_t)auto_reset_period) { new_step = 0; std::memcpy(hidden + (size_t)b * H, G.initial_hidden_state, sizeof(float) * H); }
                step[b] = new_step;
            }
        }
        in = out; ld = ldo;
    }
    return 0;
}

// rl/components/off_policy_runner/operations_generic.h:189-238 with a sequential policy that ends in [mean | log_std]
int rlt_oracle_pendulum_runner_step_recurrent(const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n, const rlt_seq_state* state,
                                              int auto_reset_period, const rlt_sas_parameters* sas, const float* action_noise, const float* initial_states) {
    if (!rn || !rb || !policy || !state || !sas || !action_noise || n <= 0 || layer_out(policy[n - 1]) != 2) return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs;
    std::vector<float> obs((size_t)N * 3), out((size_t)N * 2), actions(N), lp(N);
    int rc;
    if ((rc = rlt_oracle_pendulum_runner_prologue(rn, rb, initial_states, obs.data()))) return rc;
    if ((rc = rlt_oracle_seq_reset_state(policy, n, state, rn->truncated, N))) return rc;                      // :199-202: the flags the prologue acted on
    if ((rc = rlt_oracle_seq_evaluate_step(policy, n, obs.data(), 3, state, auto_reset_period, out.data(), 2, N))) return rc;   // :203-204
    if ((rc = rlt_oracle_sas_forward(sas, out.data(), 2, action_noise, 1, actions.data(), 1, nullptr, 0, lp.data(), N, 1))) return rc;
    return rlt_oracle_pendulum_runner_epilogue(rn, rb, obs.data(), actions.data());
}

// rl/algorithms/sac/operations_generic.h:243-337
int rlt_oracle_sac_sequence_train_critic(const rlt_sac_sequence_agent* A, int ci, const float* action_noise) {
    if (!A || ci < 0 || ci > 1 || !action_noise) return RLT_E_INVALID_ARGUMENT;
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const int first = A->include_first_step_in_targets ? 1 : 0, T = S + first, next_offset = first ? 0 : 1;     // off_policy_runner/operations_generic.h:85-92
    const rlt_seq_layer* critic = A->critics[ci];
    int rc;
    if ((rc = rlt_oracle_seq_zero_gradient(critic, A->n_critic_layers))) return rc;                                // :263
    const float* base_next = K.observations_actions_base + (size_t)next_offset * B * D;
    const uint8_t* next_reset = K.next_reset_base + (size_t)next_offset * B;
    const uint8_t* next_final = K.next_final_step_mask_base + (size_t)next_offset * B;
    // actor on the next observations, external noise, resets from next_reset (:266-273)
    if ((rc = rlt_oracle_seq_forward(A->actor, A->n_actor_layers, base_next, D, next_reset, T, B))) return rc;
    const float* actor_out = A->actor[A->n_actor_layers - 1].kind ? A->actor[A->n_actor_layers - 1].gru.output : A->actor[A->n_actor_layers - 1].dense.output;
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = rlt_oracle_sas_forward(&A->sas, actor_out, 2 * ACT, action_noise, ACT, next_actions, D, nullptr, 0, A->next_log_probabilities, T * B, ACT))) return rc;
    if ((rc = rlt_oracle_mask_copy(base_next + OBS, D, next_actions, D, next_final, 1, T * B, ACT))) return rc;      // :274-277
    for (int i = 0; i < T * B; i++) std::memcpy(A->next_state_action_value_input + (size_t)i * D, base_next + (size_t)i * D, sizeof(float) * OBS);   // :278
    for (int k = 0; k < 2; k++) {                                                                                  // :283-284
        if ((rc = rlt_oracle_seq_forward(A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, next_reset, T, B))) return rc;
        const rlt_seq_layer& last = A->critics_target[k][A->n_critic_layers - 1];
        std::memcpy(A->next_q[k], last.kind ? last.gru.output : last.dense.output, sizeof(float) * T * B);
    }
    // :133-179: the value of the step after (offset B when the first step is included), the log-probability at the same index
    if ((rc = rlt_oracle_sac_target_action_values(A->next_q[0] + first * B, A->next_q[1] + first * B, K.rewards, K.terminated, A->next_log_probabilities,
                                                 A->log_alpha.parameters, A->gamma, 0, A->target_action_value, S * B))) return rc;   // :289
    if ((rc = rlt_oracle_seq_forward(critic, A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B))) return rc;      // :294
    const rlt_seq_layer& out_layer = critic[A->n_critic_layers - 1];
    const float* q = out_layer.kind ? out_layer.gru.output : out_layer.dense.output;
    float loss_weight = 0;                                                                                         // :298-306
    rlt_oracle_cast_reduce_sum_u8(K.final_step_mask, (size_t)S * B, &loss_weight);
    if (!(loss_weight > 0)) return RLT_E_INVALID_ARGUMENT;
    rlt_oracle_scale_f32(&loss_weight, 1, S * B * 0.5f, 1);
    if ((rc = rlt_oracle_mse_gradient(q, 1, A->target_action_value, 1, A->d_output, 1, S * B, 1, 0, &loss_weight))) return rc;       // :312
    rlt_oracle_mask_zero(A->d_output, 1, K.final_step_mask, 1, S * B, 1);                                          // :314-316
    if ((rc = rlt_oracle_seq_backward(critic, A->n_critic_layers, K.observations_actions_base, D, A->d_output, nullptr, K.reset, S, B, 1, 0))) return rc;   // :329
    return adam_over(A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci]);   // :336
}

// polyak update of a sequential model, layer by layer (sac/operations_generic.h:486-527, td3/operations_generic.h:283-316)
static void polyak_seq(const rlt_seq_layer* source, const rlt_seq_layer* target, int n, float polyak) {
    for (int l = 0; l < n; l++) {
        const rlt_seq_layer& s = source[l]; const rlt_seq_layer& t = target[l];
        if (s.kind == 0) {
            rlt_oracle_polyak_update(s.dense.weights, t.dense.weights, (size_t)s.dense.in_dim * s.dense.out_dim, polyak, 0);
            rlt_oracle_polyak_update(s.dense.biases, t.dense.biases, (size_t)s.dense.out_dim, polyak, 0);
        } else {
            const size_t H = s.gru.hidden_dim, I = s.gru.input_dim;
            rlt_oracle_polyak_update(s.gru.weights_input, t.gru.weights_input, 3 * H * I, polyak, 0);
            rlt_oracle_polyak_update(s.gru.biases_input, t.gru.biases_input, 3 * H, polyak, 0);
            rlt_oracle_polyak_update(s.gru.weights_hidden, t.gru.weights_hidden, 3 * H * H, polyak, 0);
            rlt_oracle_polyak_update(s.gru.biases_hidden, t.gru.biases_hidden, 3 * H, polyak, 0);
            rlt_oracle_polyak_update(s.gru.initial_hidden_state, t.gru.initial_hidden_state, H, polyak, 0);
        }
    }
}
// :486-527
int rlt_oracle_sac_sequence_update_critic_targets(const rlt_sac_sequence_agent* A) {
    if (!A) return RLT_E_INVALID_ARGUMENT;
    for (int k = 0; k < 2; k++) polyak_seq(A->critics[k], A->critics_target[k], A->n_critic_layers, A->polyak);
    return 0;
}

// :395-468
int rlt_oracle_sac_sequence_train_actor(const rlt_sac_sequence_agent* A, const float* action_noise) {
    if (!A || !action_noise) return RLT_E_INVALID_ARGUMENT;
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT, R = S * B;
    int rc;
    if ((rc = rlt_oracle_seq_zero_gradient(A->actor, A->n_actor_layers))) return rc;                               // :414
    A->log_alpha.gradient[0] = 0;   // zero_gradient(actor) also clears the sample_and_squash layer's log_alpha gradient
    const float* obs = K.observations_actions_base;
    if ((rc = rlt_oracle_seq_forward(A->actor, A->n_actor_layers, obs, D, K.reset, S, B))) return rc;              // :427
    const rlt_seq_layer& head = A->actor[A->n_actor_layers - 1];
    const float* actor_out = head.kind ? head.gru.output : head.dense.output;
    if ((rc = rlt_oracle_sas_forward(&A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT, A->actor_log_probabilities, R, ACT))) return rc;
    float* sav_actions = A->state_action_value_input + OBS;
    for (int i = 0; i < R; i++) std::memcpy(sav_actions + (size_t)i * D, A->actor_actions + (size_t)i * ACT, sizeof(float) * ACT);
    if ((rc = rlt_oracle_mask_copy(obs + OBS, D, sav_actions, D, K.final_step_mask, 1, R, ACT))) return rc;         // :428-430
    for (int i = 0; i < R; i++) std::memcpy(A->state_action_value_input + (size_t)i * D, obs + (size_t)i * D, sizeof(float) * OBS);   // :431
    for (int k = 0; k < 2; k++)                                                                                    // :432-433
        if ((rc = rlt_oracle_seq_forward(A->critics[k], A->n_critic_layers, A->state_action_value_input, D, K.reset, S, B))) return rc;
    float loss_weight = 0;                                                                                         // :437-453
    rlt_oracle_cast_reduce_sum_u8(K.final_step_mask, (size_t)R, &loss_weight);
    if (!(loss_weight > 0)) return RLT_E_INVALID_ARGUMENT;
    rlt_oracle_scale_f32(&loss_weight, 1, -1.0f, 1);
    for (int i = 0; i < R; i++) A->d_output[i] = loss_weight;
    rlt_oracle_mask_zero(A->d_output, 1, K.final_step_mask, 1, R, 1);
    // :458-459. One d_output serves both critics, and each layer leaves its own d_pre in the buffer it was handed: with an output layer without
    // activation function that is the same values again, so the second call starts from what the first was given.
    for (int k = 0; k < 2; k++)
        if ((rc = rlt_oracle_seq_backward(A->critics[k], A->n_critic_layers, nullptr, 0, A->d_output, A->d_critic_input[k], K.reset, S, B, 0, 0))) return rc;
    const rlt_seq_layer& q1l = A->critics[0][A->n_critic_layers - 1]; const rlt_seq_layer& q2l = A->critics[1][A->n_critic_layers - 1];
    const float* q1 = q1l.kind ? q1l.gru.output : q1l.dense.output; const float* q2 = q2l.kind ? q2l.gru.output : q2l.dense.output;
    if ((rc = rlt_oracle_sac_min_value_d_output(q1, q2, A->d_critic_input[0], A->d_critic_input[1], D, D, ACT, A->d_actor_output_squashing, ACT, R))) return rc;   // :460
    rlt_oracle_mask_zero(A->d_actor_output_squashing, ACT, K.final_step_mask, 1, R, ACT);                          // :461-463
    // :464 backward of the sequential actor: sample_and_squash backward_full under the reset mode, then the layers below it
    if ((rc = rlt_oracle_sas_backward_reset(&A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT, A->d_actor_output_squashing, ACT,
                                            A->d_actor_output, 2 * ACT, A->log_alpha.parameters, &A->log_alpha.gradient[0], K.reset, R, ACT))) return rc;
    if ((rc = rlt_oracle_seq_backward(A->actor, A->n_actor_layers, obs, D, A->d_actor_output, nullptr, K.reset, S, B, 1, 0))) return rc;
    if ((rc = adam_over(A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age))) return rc;   // :465
    return adam_over(&A->log_alpha, 1, &A->alpha_adam, A->alpha_age);                                             // :466
}

// ------------------------------------------------------------------------------------------------ TD3 on sequence batches
static inline const float* seq_out(const rlt_seq_layer* layers, int n) { const rlt_seq_layer& L = layers[n - 1]; return L.kind ? L.gru.output : L.dense.output; }

// rl/algorithms/td3/operations_generic.h:170-235
int rlt_oracle_td3_sequence_train_critic(const rlt_td3_sequence_agent* A, int ci) {
    if (!A || ci < 0 || ci > 1 || !A->target_next_action_noise) return RLT_E_INVALID_ARGUMENT;
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const int first = A->include_first_step_in_targets ? 1 : 0, T = S + first, next_offset = first ? 0 : 1;     // off_policy_runner/operations_generic.h:85-92
    const rlt_seq_layer* critic = A->critics[ci];
    int rc;
    if ((rc = rlt_oracle_seq_zero_gradient(critic, A->n_critic_layers))) return rc;                                // :185
    const float* base_next = K.observations_actions_base + (size_t)next_offset * B * D;
    const uint8_t* next_reset = K.next_reset_base + (size_t)next_offset * B;
    const uint8_t* next_final = K.next_final_step_mask_base + (size_t)next_offset * B;
    // batch.observations_next is a view of OBS columns out of D; the layers here take contiguous rows
    if (!A->actor_input) return RLT_E_INVALID_ARGUMENT;
    for (int i = 0; i < T * B; i++) std::memcpy(A->actor_input + (size_t)i * OBS, base_next + (size_t)i * D, sizeof(float) * OBS);
    if ((rc = rlt_oracle_seq_forward(A->actor_target, A->n_actor_layers, A->actor_input, OBS, next_reset, T, B))) return rc;   // :191
    const float* mean = seq_out(A->actor_target, A->n_actor_layers);
    float* next_actions = A->next_state_action_value_input + OBS;
    for (int i = 0; i < T * B; i++) std::memcpy(next_actions + (size_t)i * D, mean + (size_t)i * ACT, sizeof(float) * ACT);
    if ((rc = rlt_oracle_td3_noisy_next_actions(next_actions, D, A->target_next_action_noise, ACT, T * B, ACT))) return rc;   // :192
    if ((rc = rlt_oracle_mask_copy(base_next + OBS, D, next_actions, D, next_final, 1, T * B, ACT))) return rc;      // :193-195
    for (int i = 0; i < T * B; i++) std::memcpy(A->next_state_action_value_input + (size_t)i * D, base_next + (size_t)i * D, sizeof(float) * OBS);   // :196
    for (int k = 0; k < 2; k++) {                                                                                  // :197-198
        if ((rc = rlt_oracle_seq_forward(A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, next_reset, T, B))) return rc;
        std::memcpy(A->next_q[k], seq_out(A->critics_target[k], A->n_critic_layers), sizeof(float) * T * B);
    }
    if ((rc = rlt_oracle_td3_target_action_values(A->next_q[0] + first * B, A->next_q[1] + first * B, K.rewards, K.terminated, A->gamma, A->ignore_termination,
                                                 A->target_action_value, S * B))) return rc;                      // :200 (:146-169: the value of the step after)
    if ((rc = rlt_oracle_seq_forward(critic, A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B))) return rc;      // :205
    float n_final = 0;                                                                                             // :207-212
    rlt_oracle_cast_reduce_sum_u8(K.final_step_mask, (size_t)S * B, &n_final);
    if (!(n_final > 0)) return RLT_E_INVALID_ARGUMENT;
    float loss_weight = 1.0f; loss_weight *= (float)(S * B) / n_final;
    if ((rc = rlt_oracle_mse_gradient(seq_out(critic, A->n_critic_layers), 1, A->target_action_value, 1, A->d_output, 1, S * B, 1, loss_weight, nullptr))) return rc;   // :217
    rlt_oracle_mask_zero(A->d_output, 1, K.final_step_mask, 1, S * B, 1);                                          // :218-220
    rlt_oracle_mask_zero(A->target_action_value, 1, K.final_step_mask, 1, S * B, 1);                               // :226 (the logging block, in place)
    if ((rc = rlt_oracle_seq_backward(critic, A->n_critic_layers, K.observations_actions_base, D, A->d_output, nullptr, K.reset, S, B, 1, 0))) return rc;   // :233
    return adam_over(A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci]);   // :234
}

// td3/operations_generic.h:236-281
int rlt_oracle_td3_sequence_train_actor(const rlt_td3_sequence_agent* A) {
    if (!A) return RLT_E_INVALID_ARGUMENT;
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT, R = S * B;
    const float* obs = K.observations_actions_base;
    int rc;
    if (!A->actor_input) return RLT_E_INVALID_ARGUMENT;
    for (int i = 0; i < R; i++) std::memcpy(A->actor_input + (size_t)i * OBS, obs + (size_t)i * D, sizeof(float) * OBS);
    if ((rc = rlt_oracle_seq_forward(A->actor, A->n_actor_layers, A->actor_input, OBS, K.reset, S, B))) return rc;   // :255
    const float* actions = seq_out(A->actor, A->n_actor_layers);
    float* sav_actions = A->state_action_value_input + OBS;
    for (int i = 0; i < R; i++) std::memcpy(sav_actions + (size_t)i * D, actions + (size_t)i * ACT, sizeof(float) * ACT);
    if ((rc = rlt_oracle_mask_copy(obs + OBS, D, sav_actions, D, K.final_step_mask, 1, R, ACT))) return rc;         // :256-258
    for (int i = 0; i < R; i++) std::memcpy(A->state_action_value_input + (size_t)i * D, obs + (size_t)i * D, sizeof(float) * OBS);   // :259
    const rlt_seq_layer* critic = A->critics[0];
    if ((rc = rlt_oracle_seq_forward(critic, A->n_critic_layers, A->state_action_value_input, D, K.reset, S, B))) return rc;      // :261
    float n_final = 0;                                                                                             // :262-267
    rlt_oracle_cast_reduce_sum_u8(K.final_step_mask, (size_t)R, &n_final);
    if (!(n_final > 0)) return RLT_E_INVALID_ARGUMENT;
    for (int i = 0; i < R; i++) A->d_output[i] = (float)-1 / n_final;
    rlt_oracle_mask_zero(A->d_output, 1, K.final_step_mask, 1, R, 1);
    if ((rc = rlt_oracle_seq_backward(critic, A->n_critic_layers, nullptr, 0, A->d_output, A->d_critic_input, K.reset, S, B, 0, 0))) return rc;   // :271
    for (int i = 0; i < R; i++) std::memcpy(A->d_actor_output + (size_t)i * ACT, A->d_critic_input + (size_t)i * D + OBS, sizeof(float) * ACT);   // :272
    rlt_oracle_mask_zero(A->d_actor_output, ACT, K.final_step_mask, 1, R, ACT);                                    // :273-275
    if ((rc = rlt_oracle_seq_zero_gradient(A->actor, A->n_actor_layers))) return rc;                               // :277
    if ((rc = rlt_oracle_seq_backward(A->actor, A->n_actor_layers, A->actor_input, OBS, A->d_actor_output, nullptr, K.reset, S, B, 1, 0))) return rc;   // :278
    return adam_over(A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age);               // :280
}

// td3/operations_generic.h:317-325
int rlt_oracle_td3_sequence_update_critic_targets(const rlt_td3_sequence_agent* A) {
    if (!A) return RLT_E_INVALID_ARGUMENT;
    for (int k = 0; k < 2; k++) polyak_seq(A->critics[k], A->critics_target[k], A->n_critic_layers, A->critic_polyak);
    return 0;
}
int rlt_oracle_td3_sequence_update_actor_target(const rlt_td3_sequence_agent* A) {
    if (!A) return RLT_E_INVALID_ARGUMENT;
    polyak_seq(A->actor, A->actor_target, A->n_actor_layers, A->actor_polyak);
    return 0;
}

}  // extern "C"
