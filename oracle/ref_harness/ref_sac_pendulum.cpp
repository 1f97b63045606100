// Harness around the REAL reference (compiled from /root/reference/include where it lies; nothing of it is copied
// here): runs the reference's own SAC-on-Pendulum loop state and exposes its buffers through a small C API so that
// tests can compare the CPU restatement (oracle/) and the HIP path against it.
// Built by oracle/Makefile into oracle/_ref/ in two flavours:
//   librlt_ref_generic.so  generic loops, IEEE arithmetic (-ffp-contract=off, no fast-math)
//   librlt_ref_blas.so     -DRL_TOOLS_BACKEND_ENABLE_OPENBLAS -O3 -ffast-math -march=native (the reference's own flags,
//                          CMakeLists.txt:33), cblas_sgemm resolved at load time by cblas_trampoline.cpp
#ifdef RL_TOOLS_BACKEND_ENABLE_OPENBLAS
#define RL_TOOLS_NN_DISABLE_GENERIC_FORWARD_BACKWARD
#endif
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/operations_cpu_mux.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_generic.h>
#include <rl_tools/rl/environments/pendulum/operations_cpu.h>
#include <rl_tools/nn_models/mlp/operations_generic.h>
#include <rl_tools/nn_models/sequential/operations_generic.h>
#include <rl_tools/nn_models/random_uniform/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <rl_tools/rl/algorithms/sac/loop/core/config.h>
#include <rl_tools/rl/algorithms/sac/loop/core/operations_generic.h>
#include <rl_tools/rl/utils/evaluation/operations_generic.h>

#include <chrono>
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

template <TI BATCH, TI CAPACITY>
struct LoopParameters : rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT> {
    struct SAC_PARAMETERS : rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM> {
        static constexpr TI ACTOR_BATCH_SIZE = BATCH;
        static constexpr TI CRITIC_BATCH_SIZE = BATCH;
    };
    static constexpr TI N_WARMUP_STEPS = BATCH > 100 ? BATCH : 100;   // the config asserts N_WARMUP_STEPS >= batch size
    static constexpr TI N_WARMUP_STEPS_CRITIC = N_WARMUP_STEPS;
    static constexpr TI N_WARMUP_STEPS_ACTOR = N_WARMUP_STEPS;
    static constexpr TI STEP_LIMIT = 10000;
    static constexpr TI REPLAY_BUFFER_CAP = CAPACITY;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 64;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 64;
};

template <TI BATCH, TI CAPACITY = 10000>
struct Loop {
    using CONFIG = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LoopParameters<BATCH, CAPACITY>>;
    using STATE = typename CONFIG::template State<CONFIG>;
    DEVICE device;
    STATE ts;
    explicit Loop(uint32_t seed) {
        rlt::malloc(device, ts);
        rlt::init(device, ts, seed);
    }
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

struct Any {
    int batch;
    Loop<100>* l100 = nullptr;
    Loop<256>* l256 = nullptr;
    Loop<32, 250>* l32 = nullptr;    // small ring: wraps every 250 steps (episodes are 200 steps long)
};
}  // namespace

#define DISPATCH(h, expr) ((h)->batch == 100 ? [&](auto& L) { return expr; }(*(h)->l100) : ((h)->batch == 256 ? [&](auto& L) { return expr; }(*(h)->l256) : [&](auto& L) { return expr; }(*(h)->l32)))

extern "C" {

const char* rlt_ref_flavour(void) {
#ifdef RL_TOOLS_BACKEND_ENABLE_OPENBLAS
    return "blas";
#else
    return "generic";
#endif
}

void* rlt_ref_sac_create(uint32_t seed, int batch) {
    Any* a = new Any{batch};
    if (batch == 100) a->l100 = new Loop<100>(seed);
    else if (batch == 256) a->l256 = new Loop<256>(seed);
    else if (batch == 32) a->l32 = new Loop<32, 250>(seed);
    else { delete a; return nullptr; }
    return a;
}
void rlt_ref_sac_destroy(void* h) { Any* a = (Any*)h; delete a->l100; delete a->l256; delete a->l32; delete a; }
int rlt_ref_sac_warmup_steps(void* h) { return ((Any*)h)->batch == 256 ? 256 : 100; }
int rlt_ref_sac_step(void* h) { Any* a = (Any*)h; return DISPATCH(a, (int)rlt::step(L.device, L.ts)); }
uint32_t rlt_ref_sac_step_count(void* h) { Any* a = (Any*)h; return DISPATCH(a, (uint32_t)L.ts.step); }

size_t rlt_ref_sac_parameter_count(void* h) {
    Any* a = (Any*)h;
    return DISPATCH(a, mlp_count(L.ts.actor_critic.actor.content) + 2 * mlp_count(L.ts.actor_critic.critics[0].content) + 2 * mlp_count(L.ts.actor_critic.critics_target[0].content) + 1);
}
// flat order: actor, critic 0, critic 1, target 0, target 1, log_alpha ; per network per layer [weights, biases]
void rlt_ref_sac_get_parameters(void* h, float* out) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        auto& ac = L.ts.actor_critic;
        float* o = mlp_get(ac.actor.content, out);
        o = mlp_get(ac.critics[0].content, o);
        o = mlp_get(ac.critics[1].content, o);
        o = mlp_get(ac.critics_target[0].content, o);
        o = mlp_get(ac.critics_target[1].content, o);
        *o = rlt::get(L.device, rlt::get_last_layer(ac.actor).log_alpha.parameters, 0);
        return 0;
    }()));
}
// batch of the last gather: observations_actions_base [2 x B x 4], rewards [B], terminated [B]
void rlt_ref_sac_get_batch(void* h, float* oab, float* rewards, uint8_t* terminated) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        auto& b = L.ts.critic_batch;
        const TI B = a->batch;
        std::memcpy(oab, b.observations_actions_base._data, sizeof(float) * 2 * B * 4);
        std::memcpy(rewards, b.rewards._data, sizeof(float) * B);
        for (TI i = 0; i < B; i++) terminated[i] = b.terminated._data[i];
        return 0;
    }()));
}
void rlt_ref_sac_get_masks(void* h, uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        auto& b = L.ts.critic_batch;
        const TI B = a->batch;
        for (TI i = 0; i < B; i++) { reset[i] = b.reset._data[i]; final_step_mask[i] = b.final_step_mask._data[i]; }
        for (TI i = 0; i < 2 * B; i++) { next_reset_base[i] = b.next_reset_base._data[i]; next_final_step_mask_base[i] = b.next_final_step_mask_base._data[i]; }
        return 0;
    }()));
}
void rlt_ref_sac_get_noise(void* h, float* noise_critic, float* noise_actor) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        std::memcpy(noise_critic, L.ts.action_noise_critic._data, sizeof(float) * a->batch);
        std::memcpy(noise_actor, L.ts.action_noise_actor._data, sizeof(float) * a->batch);
        return 0;
    }()));
}
// replay ring of environment 0: data [capacity x 10], cursor, full flag
void rlt_ref_sac_get_replay(void* h, float* data, uint32_t* position, uint8_t* full, uint32_t* episode_start) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        auto& rb = rlt::get(L.ts.off_policy_runner.replay_buffers, 0, 0);
        using RB = rlt::utils::typing::remove_reference_t<decltype(rb)>;
        if (data) std::memcpy(data, rb.data._data, sizeof(float) * RB::CAPACITY * RB::DATA_COLS);   // caller sizes `data` for the ring's capacity
        *position = (uint32_t)rb.position; *full = rb.full;
        if (episode_start) for (TI i = 0; i < RB::CAPACITY; i++) episode_start[i] = (uint32_t)rlt::get(L.device, rb.episode_start, i);
        return 0;
    }()));
}
// training buffers after the last step (for step-by-step comparisons, pattern of tests/src/rl/cuda/rl.cu:230-376)
void rlt_ref_sac_get_critic_buffers(void* h, int critic, float* target_action_value, float* next_q1, float* next_q2, float* next_input, float* d_output) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        auto& tb = L.ts.critic_training_buffers[critic];
        const TI B = a->batch;
        std::memcpy(target_action_value, tb.target_action_value._data, sizeof(float) * B);
        std::memcpy(next_q1, tb.next_state_action_value_critic_1._data, sizeof(float) * B);
        std::memcpy(next_q2, tb.next_state_action_value_critic_2._data, sizeof(float) * B);
        std::memcpy(next_input, tb.next_state_action_value_input._data, sizeof(float) * B * 4);
        std::memcpy(d_output, tb.d_output._data, sizeof(float) * B);
        return 0;
    }()));
}
void rlt_ref_sac_get_actor_buffers(void* h, float* state_action_value_input, float* d_critic_1_input, float* d_critic_2_input, float* d_actor_output_squashing) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        auto& tb = L.ts.actor_training_buffers;
        const TI B = a->batch;
        std::memcpy(state_action_value_input, tb.state_action_value_input._data, sizeof(float) * B * 4);
        std::memcpy(d_critic_1_input, tb.d_critic_1_input._data, sizeof(float) * B * 4);
        std::memcpy(d_critic_2_input, tb.d_critic_2_input._data, sizeof(float) * B * 4);
        std::memcpy(d_actor_output_squashing, tb.d_actor_output_squashing._data, sizeof(float) * B);
        return 0;
    }()));
}
// Times `steps` loop steps (the reference's benchmark: src/rl/environments/pendulum/sac/cpu/training.h:73-93); seconds.
double rlt_ref_sac_time_steps(void* h, int steps) {
    Any* a = (Any*)h;
    auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; i++) DISPATCH(a, (int)rlt::step(L.device, L.ts));
    auto t1 = std::chrono::steady_clock::now();
    return std::chrono::duration<double>(t1 - t0).count();
}

// rl::utils::evaluation::evaluate (rl/utils/evaluation/operations_generic.h:106-233) of the loop's current actor in Evaluation mode: 10 episodes of
// 200 steps from sampled initial states, the configuration of the evaluation loop step (rl/loop/steps/evaluation/config.h:12-24). The initial
// states the call will draw are exported by drawing them first from a copy of the engine.
// summary = {returns_mean, returns_std, episode_length_mean, episode_length_std, num_terminated, share_terminated}
void rlt_ref_sac_evaluate(void* h, uint32_t seed, float* initial_states, float* returns, uint32_t* episode_length, float* summary) {
    Any* a = (Any*)h;
    DISPATCH(a, ([&] {
        constexpr TI N_EPISODES = 10, STEP_LIMIT = 200;
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
        return 0;
    }()));
}

}  // extern "C"
