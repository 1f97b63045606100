// Harness around the REAL reference's gather_batch for sequence batches (compiled from /root/reference/include where it lies; nothing of it is
// copied here): a SAC-on-Pendulum loop with three environments, episodes of 30 steps and replay rings of 260 rows fills the runner's replay
// buffers (they wrap after 260 loop steps; the runner's MAX_EPISODE_LENGTH is the environment's 200, so 60 rows stay eligible once a ring is full); gather_batch (rl/components/off_policy_runner/operations_generic.h:239-430) is then called on that
// runner with batch types of our choosing and an engine of our own, whose text form before the call is exported.
// Built by oracle/Makefile into oracle/_ref/librlt_ref_gather_seq_generic.so.
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
constexpr TI N_ENVS = 3, CAPACITY = 260, EPISODE_LIMIT = 30, BATCH = 64, SEQ = 8;

struct LoopParameters : rlt::rl::algorithms::sac::loop::core::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT> {
    struct SAC_PARAMETERS : rlt::rl::algorithms::sac::DefaultParameters<TYPE_POLICY, TI, ENVIRONMENT::ACTION_DIM> {
        static constexpr TI ACTOR_BATCH_SIZE = 32;
        static constexpr TI CRITIC_BATCH_SIZE = 32;
    };
    static constexpr TI N_ENVIRONMENTS = N_ENVS;
    static constexpr TI N_WARMUP_STEPS = 100;
    static constexpr TI N_WARMUP_STEPS_CRITIC = 100;
    static constexpr TI N_WARMUP_STEPS_ACTOR = 100;
    static constexpr TI STEP_LIMIT = 100000;
    static constexpr TI REPLAY_BUFFER_CAP = CAPACITY;
    static constexpr TI EPISODE_STEP_LIMIT = EPISODE_LIMIT;
    static constexpr TI ACTOR_NUM_LAYERS = 3;
    static constexpr TI ACTOR_HIDDEN_DIM = 16;
    static constexpr TI CRITIC_NUM_LAYERS = 3;
    static constexpr TI CRITIC_HIDDEN_DIM = 16;
};
using CONFIG = rlt::rl::algorithms::sac::loop::core::Config<TYPE_POLICY, TI, RNG, ENVIRONMENT, LoopParameters>;
using STATE = typename CONFIG::template State<CONFIG>;
using RUNNER_SPEC = typename CONFIG::OFF_POLICY_RUNNER_SPEC;

struct Loop {
    DEVICE device;
    STATE ts;
    explicit Loop(uint32_t seed) { rlt::malloc(device, ts); rlt::init(device, ts, seed); }
    ~Loop() { rlt::free(device, ts); }
};

// sampling parameter sets: the defaults for sequences, and the same with both switches off
struct PlainSampling {
    static constexpr bool INCLUDE_FIRST_STEP_IN_TARGETS = true;
    static constexpr bool ALWAYS_SAMPLE_FROM_INITIAL_STATE = false;
    static constexpr bool RANDOM_SEQ_LENGTH = false;
    static constexpr bool ENABLE_NOMINAL_SEQUENCE_LENGTH_PROBABILITY = true;
    static constexpr float NOMINAL_SEQUENCE_LENGTH_PROBABILITY = 0.5;
};
template <TI SEQUENCE_LENGTH, typename SAMPLING>
using BatchOf = rlt::rl::components::off_policy_runner::SequentialBatch<rlt::rl::components::off_policy_runner::SequentialBatchSpecification<RUNNER_SPEC, SEQUENCE_LENGTH, BATCH, SAMPLING>>;
using DefaultSampling8 = rlt::rl::components::off_policy_runner::SequentialBatchParameters<TYPE_POLICY, TI, SEQ>;
using DefaultSampling1 = rlt::rl::components::off_policy_runner::SequentialBatchParameters<TYPE_POLICY, TI, 1>;

template <typename BATCH_TYPE>
int gather(Loop& L, uint32_t seed, char* rng_text, int rng_capacity, float* oab, float* rewards, uint8_t* terminated, uint8_t* reset, uint8_t* next_reset_base,
           uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    constexpr TI S = BATCH_TYPE::SEQUENCE_LENGTHH, PS = BATCH_TYPE::PADDED_SEQUENCE_LENGTH, D = BATCH_TYPE::DATA_DIM;
    BATCH_TYPE batch;
    rlt::malloc(L.device, batch);
    // what gather_batch does not write keeps these values
    for (TI i = 0; i < PS * BATCH * D; i++) batch.observations_actions_base._data[i] = -777.0f;
    for (TI i = 0; i < S * BATCH; i++) { batch.rewards._data[i] = -777.0f; batch.terminated._data[i] = false; batch.reset._data[i] = false; batch.final_step_mask._data[i] = false; }
    for (TI i = 0; i < PS * BATCH; i++) { batch.next_reset_base._data[i] = false; batch.next_final_step_mask_base._data[i] = false; }
    RNG rng;
    rlt::malloc(L.device, rng);
    rlt::init(L.device, rng, seed);
    std::stringstream ss;
    ss << rng.engine;
    const std::string text = ss.str();
    if ((int)text.size() + 1 > rng_capacity) return (int)text.size() + 1;
    std::memcpy(rng_text, text.c_str(), text.size() + 1);
    rlt::gather_batch(L.device, L.ts.off_policy_runner, batch, rng);
    std::memcpy(oab, batch.observations_actions_base._data, sizeof(float) * PS * BATCH * D);
    std::memcpy(rewards, batch.rewards._data, sizeof(float) * S * BATCH);
    for (TI i = 0; i < S * BATCH; i++) { terminated[i] = batch.terminated._data[i]; reset[i] = batch.reset._data[i]; final_step_mask[i] = batch.final_step_mask._data[i]; }
    for (TI i = 0; i < PS * BATCH; i++) { next_reset_base[i] = batch.next_reset_base._data[i]; next_final_step_mask_base[i] = batch.next_final_step_mask_base._data[i]; }
    rlt::free(L.device, rng);
    rlt::free(L.device, batch);
    return 0;
}
}  // namespace

extern "C" {
void* rlt_ref_gather_seq_create(uint32_t seed) { return new Loop(seed); }
void rlt_ref_gather_seq_destroy(void* h) { delete static_cast<Loop*>(h); }
int rlt_ref_gather_seq_step(void* h) { Loop& L = *static_cast<Loop*>(h); return (int)rlt::step(L.device, L.ts); }
// dims = {n_envs, capacity, episode_step_limit (= the runner's MAX_EPISODE_LENGTH), batch, sequence_length, row width of the replay data}
void rlt_ref_gather_seq_dims(int* dims) {
    using RB = rlt::utils::typing::remove_reference_t<decltype(rlt::get(std::declval<STATE&>().off_policy_runner.replay_buffers, 0, 0))>;
    dims[0] = N_ENVS; dims[1] = CAPACITY; dims[2] = RUNNER_SPEC::MAX_EPISODE_LENGTH; dims[3] = BATCH; dims[4] = SEQ; dims[5] = RB::DATA_COLS;
}
// replay ring of one environment: data [capacity x 10], cursor, full flag, episode starts
void rlt_ref_gather_seq_get_replay(void* h, int env, float* data, uint32_t* position, uint8_t* full, uint32_t* episode_start) {
    Loop& L = *static_cast<Loop*>(h);
    auto& rb = rlt::get(L.ts.off_policy_runner.replay_buffers, 0, env);
    using RB = rlt::utils::typing::remove_reference_t<decltype(rb)>;
    std::memcpy(data, rb.data._data, sizeof(float) * RB::CAPACITY * RB::DATA_COLS);
    *position = (uint32_t)rb.position; *full = rb.full;
    for (TI i = 0; i < RB::CAPACITY; i++) episode_start[i] = (uint32_t)rlt::get(L.device, rb.episode_start, i);
}
// variant 0: sequences of 8 with the reference's defaults (start at the episode's first step, random sequence lengths); 1: sequences of 8 with
// both switched off; 2: single steps with the defaults. Returns 0, or the capacity the engine's text form needs.
int rlt_ref_gather_seq_gather(void* h, int variant, uint32_t seed, char* rng_text, int rng_capacity, float* oab, float* rewards, uint8_t* terminated, uint8_t* reset,
                              uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    Loop& L = *static_cast<Loop*>(h);
    if (variant == 0) return gather<BatchOf<SEQ, DefaultSampling8>>(L, seed, rng_text, rng_capacity, oab, rewards, terminated, reset, next_reset_base, final_step_mask, next_final_step_mask_base);
    if (variant == 1) return gather<BatchOf<SEQ, PlainSampling>>(L, seed, rng_text, rng_capacity, oab, rewards, terminated, reset, next_reset_base, final_step_mask, next_final_step_mask_base);
    if (variant == 2) return gather<BatchOf<1, DefaultSampling1>>(L, seed, rng_text, rng_capacity, oab, rewards, terminated, reset, next_reset_base, final_step_mask, next_final_step_mask_base);
    return -1;
}
}
