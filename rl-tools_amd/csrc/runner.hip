// Replay buffer add / gather_batch, batched Pendulum dynamics and the off-policy runner step.
// reference: rl/components/replay_buffer/operations_generic.h:54-78, rl/components/off_policy_runner/operations_generic.h:183-430
//            (CUDA :14-230), operations_generic_per_env.h:8-108, rl/environments/pendulum/operations_generic.h:14-160.
#include "common.h"
#include "pad.h"
#include "rng.h"
#include "pendulum.h"
#include <cstdlib>

namespace {

__global__ __launch_bounds__(256) void pendulum_step_kernel(rlt_pendulum_parameters p, float* __restrict__ states, const float* __restrict__ actions,
                                                            float* __restrict__ observations, float* __restrict__ next_observations, float* __restrict__ rewards, int n) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        Transition t;
        pendulum_transition(p, states[2 * e], states[2 * e + 1], actions[e], t);
        if (observations) { observations[3 * (size_t)e] = t.obs[0]; observations[3 * (size_t)e + 1] = t.obs[1]; observations[3 * (size_t)e + 2] = t.obs[2]; }
        if (next_observations) { next_observations[3 * (size_t)e] = t.next_obs[0]; next_observations[3 * (size_t)e + 1] = t.next_obs[1]; next_observations[3 * (size_t)e + 2] = t.next_obs[2]; }
        if (rewards) rewards[e] = t.reward;
        states[2 * e] = t.theta; states[2 * e + 1] = t.theta_dot;
    }
}

// replay_buffer/operations_generic.h:54-78, thread per environment (each environment owns its ring)
__global__ __launch_bounds__(256) void replay_add_kernel(rlt_replay_buffer rb, const float* __restrict__ obs, const float* __restrict__ actions, const float* __restrict__ rewards,
                                                         const float* __restrict__ next_obs, const uint8_t* __restrict__ terminated, const uint8_t* __restrict__ truncated) {
    const int OBS = rb.observation_dim, ACT = rb.action_dim, R = 2 * OBS + ACT + 3;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rb.n_envs; e += gridDim.x * blockDim.x) {
        uint32_t pos = rb.position[e];
        float* row = rb.data + ((size_t)e * rb.capacity + pos) * R;
        for (int i = 0; i < OBS; i++) { row[i] = obs[(size_t)e * OBS + i]; row[OBS + ACT + 1 + i] = next_obs[(size_t)e * OBS + i]; }
        for (int i = 0; i < ACT; i++) row[OBS + i] = actions[(size_t)e * ACT + i];
        row[OBS + ACT] = rewards[e];
        row[2 * OBS + ACT + 1] = terminated[e] ? 1.0f : 0.0f;
        row[2 * OBS + ACT + 2] = truncated[e] ? 1.0f : 0.0f;
        rb.episode_start[(size_t)e * rb.capacity + pos] = rb.current_episode_start[e];
        pos = (pos + 1) % (uint32_t)rb.capacity;
        rb.position[e] = pos;
        if (truncated[e]) rb.current_episode_start[e] = pos;
        if (pos == 0 && !rb.full[e]) rb.full[e] = 1;
    }
}

// off_policy_runner/operations_generic.h:240-430 for SEQUENCE_LENGTH = 1: 16 lanes cooperate on one sample so that a replay
// row (2*obs+act+3 floats) is read as one contiguous segment and each batch row is written contiguously.
__global__ __launch_bounds__(256) void gather_kernel(rlt_replay_buffer rb, const uint32_t* __restrict__ env_indices, const uint32_t* __restrict__ sample_offsets,
                                                     int deterministic, int max_episode_length, int batch, float* __restrict__ oab, float* __restrict__ rewards,
                                                     uint8_t* __restrict__ terminated, uint8_t* __restrict__ reset, uint8_t* __restrict__ next_reset_base,
                                                     uint8_t* __restrict__ final_step_mask, uint8_t* __restrict__ next_final_step_mask_base, int* __restrict__ error_flag,
                                                     int draw, uint64_t seed, uint64_t stream, uint32_t* __restrict__ drawn_env_indices, uint32_t* __restrict__ drawn_sample_offsets, const uint64_t* __restrict__ stream_offset) {
    const int OBS = rb.observation_dim, ACT = rb.action_dim, R = 2 * OBS + ACT + 3, D = OBS + ACT;
    if (draw) stream += *stream_offset;
    const int sub = threadIdx.x & 15;
    for (int i = (blockIdx.x * blockDim.x + threadIdx.x) >> 4; i < batch; i += (gridDim.x * blockDim.x) >> 4) {
        uint32_t e, offset;
        if (draw) {      // what gather_draw_kernel would have put into the arrays: words 0 and 1 of group i of the call's stream (all 16 lanes compute it)
            const rlt_u32x4 words = rlt_philox(seed, stream, (uint64_t)i);
            e = rlt_uniform_below(words.x, (uint32_t)rb.n_envs);
            const uint32_t eligible = rb.full[e] ? (uint32_t)rb.capacity : rb.position[e];
            offset = eligible ? (uint32_t)(((uint64_t)words.y * eligible) >> 32) : 0u;
            if (sub == 0) { if (drawn_env_indices) drawn_env_indices[i] = e; if (drawn_sample_offsets) drawn_sample_offsets[i] = offset; }
        } else {
            e = deterministic ? 0u : env_indices[i];
            offset = deterministic ? (uint32_t)i : sample_offsets[i];
        }
        if (e >= (uint32_t)rb.n_envs) { if (sub == 0) *error_flag = 1; continue; }
        uint32_t index = rb.full[e] ? (rb.position[e] + (uint32_t)max_episode_length + offset) % (uint32_t)rb.capacity : offset;
        if (index >= (uint32_t)rb.capacity) { if (sub == 0) *error_flag = 1; continue; }
        const float* row = rb.data + ((size_t)e * rb.capacity + index) * R;
        float* step0 = oab + (size_t)i * D; float* step1 = oab + ((size_t)batch + i) * D;
        for (int j = sub; j < R; j += 16) {
            float v = row[j];
            if (j < D) step0[j] = v;                                   // observation and action of padded step 0
            else if (j == D) rewards[i] = v;
            else if (j < D + 1 + OBS) step1[j - D - 1] = v;            // next observation into padded step 1
            else if (j == D + 1 + OBS) terminated[i] = v != 0.0f;
        }
        for (int j = sub; j < ACT; j += 16) step1[OBS + j] = 0.0f;     // next action zeroed
        if (sub == 0) {
            if (reset) reset[i] = 1;
            if (next_reset_base) { next_reset_base[i] = 1; next_reset_base[batch + i] = 1; }
            if (final_step_mask) final_step_mask[i] = 1;
            if (next_final_step_mask_base) { next_final_step_mask_base[i] = 0; next_final_step_mask_base[batch + i] = 1; }
        }
    }
}

// gather_batch_step for sequences (rl/components/off_policy_runner/operations_generic.h:239-418): a wavefront per sample walks its padded steps through one
// ring; the draws come from arrays, the k-th use of a kind by sample b being entry [b][k]. Copies and index arithmetic only.
// The reference's loop is one step after the other because whether a step ends a sequence is read from its own row. Between two ends the rows are consecutive,
// so the wavefront takes a run of up to 64 steps at once: lane l reads the row of step s + l, the first lane whose step ends the sequence (its row's truncated
// flag, the ring's cursor, the last padded step, the drawn length) is found by a vote, the lanes up to it write their steps, and the walk goes on behind it -- one
// trip to memory per run instead of one per step. The bookkeeping between runs is the same on every lane. The four masks are collected in LDS and written once.
constexpr int GATHER_SEQ_MAX_PADDED = 1024;
__global__ __launch_bounds__(256) void gather_sequence_kernel(rlt_replay_buffer rb, rlt_sequence_sampling P, rlt_sequence_draws draws, int max_episode_length, rlt_sequence_batch B,
                                                              int* __restrict__ error_flag) {
    __shared__ uint8_t masks[4][4][GATHER_SEQ_MAX_PADDED];      // per wavefront: final_step, reset, next_final_step, next_reset
    const int OBS = rb.observation_dim, ACT = rb.action_dim, R = 2 * OBS + ACT + 3, D = OBS + ACT, N = B.batch, SEQ = B.sequence_length, PADDED = SEQ + 1;
    const uint32_t CAP = (uint32_t)rb.capacity;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    volatile uint8_t* final_mask = masks[wave][0]; volatile uint8_t* reset_mask = masks[wave][1]; volatile uint8_t* next_final_mask = masks[wave][2]; volatile uint8_t* next_reset_mask = masks[wave][3];
    for (int b = blockIdx.x * 4 + wave; b < N; b += gridDim.x * 4) {
        const uint32_t e = draws.env_indices[b];
        if (e >= (uint32_t)rb.n_envs) { if (lane == 0) *error_flag = 1; continue; }
        const uint32_t position = rb.position[e];
        const bool full = rb.full[e] != 0;
        const uint32_t* offsets = draws.sample_offsets + (size_t)b * PADDED;
        const uint8_t* nominal = draws.nominal + (size_t)b * (PADDED + 1);
        const uint32_t* lengths = draws.lengths + (size_t)b * (PADDED + 1);
        int n_offset = 0, n_length = 0;
        uint32_t sample_index = 0;
        int current_seq_length = SEQ;
        // a length decision (:266-275, :362-371): nominal[k] says whether the full length is taken, lengths[k] is used where it does not
        auto draw_length = [&]() {
            int length = current_seq_length;
            if (P.enable_nominal_sequence_length_probability && nominal[n_length]) length = SEQ;
            else if (SEQ > 1) length = (int)lengths[n_length];
            n_length++;
            return length;
        };
        if (P.random_seq_length) current_seq_length = draw_length();
        int current_seq_step = 0;
        bool previous_step_truncated = false, previous_padding_step = true;
        for (int s = lane; s < PADDED; s += 64) { final_mask[s] = 0; reset_mask[s] = 0; next_final_mask[s] = 0; next_reset_mask[s] = 0; }
        __builtin_amdgcn_wave_barrier();
        if (lane == 0) { reset_mask[0] = 1; next_reset_mask[0] = 1; next_reset_mask[P.include_first_step_in_targets ? 0 : 1] = 1; }
        bool failed = false;
        int s = 0;
        while (s < PADDED) {
            if (previous_step_truncated) {
                previous_step_truncated = false; previous_padding_step = true;
                if (lane == 0) { next_final_mask[s] = 1; if (s < PADDED - 1) reset_mask[s] = 1; }
                s++;
                continue;
            }
            if (previous_padding_step) {
                if (lane == 0) { if (s < PADDED - 1) reset_mask[s] = 1; next_reset_mask[s] = 1; }
                const uint32_t sample_offset = offsets[n_offset++];
                sample_index = full ? (position + (uint32_t)max_episode_length + sample_offset) % CAP : sample_offset;
                if (P.always_sample_from_initial_state && sample_index < CAP) sample_index = rb.episode_start[(size_t)e * CAP + sample_index];
            }
            if (sample_index >= CAP) { failed = true; break; }
            // the run that starts at step s and row sample_index: lane l takes step s + l and the l-th row behind sample_index
            const int step = s + lane;
            const bool in_range = step < PADDED;
            uint32_t index = sample_index + (uint32_t)lane;
            if (full) index %= CAP;
            const bool readable = in_range && index < CAP;
            const float* row = rb.data + ((size_t)e * CAP + (readable ? index : sample_index)) * R;
            bool truncated = row[2 * OBS + ACT + 2] != 0.0f;
            uint32_t next_index = index + 1;
            if (full) next_index %= CAP;
            if (next_index == position) truncated = true;
            if (step == PADDED - 2) truncated = true;
            const bool length_ends = P.random_seq_length && current_seq_step + lane == current_seq_length - 1;
            if (length_ends) truncated = true;
            // a lane past the ring's last written row (not full: index >= CAP) would be an error if the walk reached it; the cursor ends the run before
            const unsigned long long ends = __ballot(in_range && (truncated || !readable));
            const int last = ends ? __ffsll((long long)ends) - 1 : min(63, PADDED - 1 - s);      // the run's last lane
            const bool run_truncated = ends != 0ull;
            if (lane == last && run_truncated && !readable) failed = true;
            if (__ballot(failed)) { failed = true; break; }
            if (lane <= last && in_range) {
                float* out = B.observations_actions_base + ((size_t)step * N + b) * D;
                for (int k = 0; k < D; k++) out[k] = row[k];
                if (step < PADDED - 1) { B.rewards[(size_t)step * N + b] = row[D]; B.terminated[(size_t)step * N + b] = row[2 * OBS + ACT + 1] != 0.0f; }
                if (lane == last && run_truncated && step < PADDED - 1) {
                    final_mask[step] = 1;
                    float* next = B.observations_actions_base + ((size_t)(step + 1) * N + b) * D;
                    for (int k = 0; k < OBS; k++) next[k] = row[D + 1 + k];
                    for (int k = 0; k < ACT; k++) next[OBS + k] = 0.0f;
                }
            }
            // the bookkeeping behind the run's last step, the same on every lane
            const bool last_length_ends = P.random_seq_length && current_seq_step + last == current_seq_length - 1;
            if (P.random_seq_length) {
                if (last_length_ends) current_seq_length = SEQ > 1 ? draw_length() : SEQ;
                current_seq_step = run_truncated ? 0 : current_seq_step + last + 1;
            }
            uint32_t after = sample_index + (uint32_t)last + 1;
            if (full) after %= CAP;
            sample_index = after;
            previous_padding_step = false;
            previous_step_truncated = run_truncated;
            s += last + 1;
        }
        if (failed && lane == 0) *error_flag = 1;
        __builtin_amdgcn_wave_barrier();
        for (int t = lane; t < PADDED; t += 64) {
            if (t < SEQ) { B.final_step_mask[(size_t)t * N + b] = final_mask[t]; B.reset[(size_t)t * N + b] = reset_mask[t]; }
            B.next_final_step_mask_base[(size_t)t * N + b] = next_final_mask[t]; B.next_reset_base[(size_t)t * N + b] = next_reset_mask[t];
        }
        __builtin_amdgcn_wave_barrier();
    }
}

__global__ __launch_bounds__(256) void gather_draw_kernel(rlt_replay_buffer rb, int batch, uint64_t seed, uint64_t stream, uint32_t* __restrict__ env_indices, uint32_t* __restrict__ sample_offsets, const uint64_t* __restrict__ stream_offset) {
    stream += *stream_offset;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch; i += gridDim.x * blockDim.x) {
        const rlt_u32x4 draw = rlt_philox(seed, stream, (uint64_t)i);   // sample i takes words 0 and 1 of group i of the call's stream
        const uint32_t r1 = draw.y;
        uint32_t e = rlt_uniform_below(draw.x, (uint32_t)rb.n_envs);
        uint32_t eligible = rb.full[e] ? (uint32_t)rb.capacity : rb.position[e];
        env_indices[i] = e;
        sample_offsets[i] = eligible ? (uint32_t)(((uint64_t)r1 * eligible) >> 32) : 0u;
    }
}

// The draws of a sequence batch (the arrays of rlt_sequence_draws), on the device: sample b takes the words of groups [b G, (b + 1) G) of the call's
// stream, G = ceil((3 padded + 3) / 4), in the order environment, padded offsets, padded + 1 nominal decisions, padded + 1 lengths.
__global__ __launch_bounds__(256) void gather_sequence_draw_kernel(rlt_replay_buffer rb, rlt_sequence_sampling P, int max_episode_length, int batch, int sequence_length, uint64_t seed,
                                                                   uint64_t stream, uint32_t* __restrict__ env_indices, uint32_t* __restrict__ sample_offsets,
                                                                   uint8_t* __restrict__ nominal, uint32_t* __restrict__ lengths, const uint64_t* __restrict__ stream_offset) {
    stream += *stream_offset;
    const int PADDED = sequence_length + 1, WORDS = 3 * PADDED + 3, G = (WORDS + 3) / 4;
    // a thread per (sample, group of four words); the offsets need the sample's environment, which is word 0 of its first group
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < (size_t)batch * G; t += (size_t)gridDim.x * blockDim.x) {
        const int b = (int)(t / G), g = (int)(t - (size_t)b * G);
        const rlt_u32x4 draw = rlt_philox(seed, stream, (uint64_t)b * G + g);
        const uint32_t first_word = g == 0 ? draw.x : rlt_philox(seed, stream, (uint64_t)b * G).x;
        const uint32_t env = rlt_uniform_below(first_word, (uint32_t)rb.n_envs);
        const uint32_t eligible = rb.full[env] ? (uint32_t)(P.always_sample_from_initial_state ? rb.capacity - max_episode_length : rb.capacity) : rb.position[env];
        const uint32_t words[4] = {draw.x, draw.y, draw.z, draw.w};
        for (int i = 0; i < 4; i++) {
            const int w = 4 * g + i;
            if (w >= WORDS) break;
            if (w == 0) env_indices[b] = env;
            else if (w <= PADDED) sample_offsets[(size_t)b * PADDED + (w - 1)] = eligible ? rlt_uniform_below(words[i], eligible) : 0u;
            else if (w <= 2 * PADDED + 1) nominal[(size_t)b * (PADDED + 1) + (w - PADDED - 1)] = rlt_u01(words[i]) < P.nominal_sequence_length_probability ? 1 : 0;
            else lengths[(size_t)b * (PADDED + 1) + (w - 2 * PADDED - 2)] = sequence_length > 1 ? 1u + rlt_uniform_below(words[i], (uint32_t)(sequence_length - 1)) : 1u;
        }
    }
}

// prologue of the runner step (operations_generic_per_env.h:8-66): reset where truncated, flag the previous replay row, observe
__global__ __launch_bounds__(256) void runner_prologue_kernel(rlt_pendulum_runner rn, rlt_replay_buffer rb, const float* __restrict__ initial_states, uint64_t seed, uint64_t stream,
                                                              float* __restrict__ observations, const uint64_t* __restrict__ stream_offset) {
    stream += *stream_offset;
    const int R = 2 * rb.observation_dim + rb.action_dim + 3;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        if (rn.truncated[e]) {
            float th, thd;
            if (initial_states) { th = initial_states[2 * e]; thd = initial_states[2 * e + 1]; }
            else {
                const float PI = 3.14159265358979323846f;
                const rlt_u32x4 draw = rlt_philox(seed, stream, (uint64_t)e);   // environment e takes words 0 and 1 of group e of the call's stream
                const float u0 = rlt_u01(draw.x), u1 = rlt_u01(draw.y);
                th = -PI + 2.0f * PI * u0; thd = -1.0f + 2.0f * u1;
            }
            rn.states[2 * e] = th; rn.states[2 * e + 1] = thd;
            rn.episode_step[e] = 0; rn.episode_return[e] = 0.0f;
            if (rb.full[e] || rb.position[e] > 0) {
                uint32_t prev = rb.position[e] == 0 ? (uint32_t)rb.capacity - 1 : rb.position[e] - 1;
                rb.data[((size_t)e * rb.capacity + prev) * R + (R - 1)] = 1.0f;
                rb.current_episode_start[e] = rb.position[e];
            }
        }
        float s, c;
        sincosf(rn.states[2 * e], &s, &c);
        observations[3 * (size_t)e] = c; observations[3 * (size_t)e + 1] = s; observations[3 * (size_t)e + 2] = rn.states[2 * e + 1];
    }
}
// epilogue (operations_generic_per_env.h:67-108): env step, reward, next observation, truncation, replay add
__global__ __launch_bounds__(256) void runner_epilogue_kernel(rlt_pendulum_runner rn, rlt_replay_buffer rb, const float* __restrict__ actions) {
    const int R = 10;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        Transition t;
        pendulum_transition(rn.env, rn.states[2 * e], rn.states[2 * e + 1], actions[e], t);
        uint32_t step = rn.episode_step[e] + 1;
        rn.episode_step[e] = step;
        rn.episode_return[e] += t.reward;
        const bool truncated = step == (uint32_t)rn.episode_step_limit;
        rn.truncated[e] = truncated;
        rn.states[2 * e] = t.theta; rn.states[2 * e + 1] = t.theta_dot;
        uint32_t pos = rb.position[e];
        float* row = rb.data + ((size_t)e * rb.capacity + pos) * R;
        row[0] = t.obs[0]; row[1] = t.obs[1]; row[2] = t.obs[2]; row[3] = t.action; row[4] = t.reward;
        row[5] = t.next_obs[0]; row[6] = t.next_obs[1]; row[7] = t.next_obs[2]; row[8] = 0.0f; row[9] = truncated ? 1.0f : 0.0f;
        rb.episode_start[(size_t)e * rb.capacity + pos] = rb.current_episode_start[e];
        pos = (pos + 1) % (uint32_t)rb.capacity;
        rb.position[e] = pos;
        if (truncated) rb.current_episode_start[e] = pos;
        if (pos == 0 && !rb.full[e]) rb.full[e] = 1;
    }
}

// ---- the whole runner step in one launch for 3 -> 64 -> 64 -> {1, 2} actors ---------------------------------------------------
// A wavefront owns tiles of 32 environments, one per lane of its lower half, and keeps the actor in registers (W2 as 64
// matrix-instruction operands; one workgroup per CU stages it through LDS once). Per tile the owning lanes run the prologue for
// their environments and write the observations into the wavefront's corner of LDS; the network then runs on
// v_mfma_f32_16x16x4_f32 as two independent groups of 16 rows: layer 1, the hidden activations through that same corner (no
// workgroup barrier: nothing is shared between wavefronts), layer 2, layer 3 as a 16-lane reduction whose results go back through
// LDS to the lanes that own the rows; these finish with the policy head, the dynamics, the reward and the replay add. Two
// wavefronts share a SIMD so that one's per-environment arithmetic overlaps the other's matrix instructions, which bound the
// kernel: 8,704 flop per environment on the fp32 matrix pipe. Traffic is what the step must move: state in, state and one replay
// row out, all but the replay rows coalesced.
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) float* lptr;
constexpr int FH = 64, FTILE = 32, FAS = FH + 1, FXS = 5;
constexpr int FUSED_LDS_PER_WAVE = 2 * 16 * FAS + FTILE * FXS + FTILE * 2;  // hidden activations of 2 x 16 rows, observations, outputs
constexpr int FWAVES = 8;        // wavefronts per workgroup: two per SIMD, one's scalar work (prologue, dynamics) overlaps the other's matrix instructions

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
template <int CTRL>
__device__ __forceinline__ float dpp(float x) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true)); }
__device__ __forceinline__ float row16_sum(float x) { asm volatile("" : "+v"(x)); /* keeps a producing multiplication out of the first addition: all lanes then hold the same sum */ x += dpp<0xB1>(x); x += dpp<0x4E>(x); x += dpp<0x141>(x); x += dpp<0x140>(x); return x; }

struct FusedRunnerArgs {
    rlt_pendulum_runner rn; rlt_replay_buffer rb;
    const float* w1; const float* b1; const float* w2; const float* b2; const float* w3; const float* b3;
    int act_hidden, act_out, out_dim, policy_kind;
    rlt_sas_parameters sas;
    const float* action_noise; const float* initial_states;
    uint64_t seed, stream;
    const uint64_t* stream_offset;                  // added to both stream numbers
    uint64_t noise_stream; float* drawn_noise;      // action_noise == NULL: element e of the standard-normal stream (seed, noise_stream), also written to drawn_noise if given
};

template <int ACT_H>      // hidden activation, a compile-time constant: it sits inside the unrolled matrix-instruction loops
__global__ __launch_bounds__(64 * FWAVES) void runner_fused_kernel(FusedRunnerArgs A) {
    __shared__ float lds[FWAVES * FUSED_LDS_PER_WAVE + FH * FAS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, kk = lane >> 4;
    const lptr hs = (lptr)lds + wave * FUSED_LDS_PER_WAVE, xs = hs + 2 * 16 * FAS, ys = xs + FTILE * FXS, w2s = (lptr)lds + FWAVES * FUSED_LDS_PER_WAVE;
    // W2 goes through LDS (coalesced rows in, padded rows out), the small tensors straight from memory
    for (int i = threadIdx.x; i < FH * FH; i += 64 * FWAVES) w2s[(i >> 6) * FAS + (i & 63)] = A.w2[i];
    __syncthreads();
    // the actor, as the operands this lane feeds to the matrix instructions (any fixed assignment of the reduction index to the
    // four lane groups is valid as long as both operands agree: group kk takes [16 kk, 16 kk + 16) of a 64-long reduction)
    float w1r[4], b1r[4], w2r[4][16], b2r[4], w3r[2][4];
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        const int n = 16 * nt + r;
        w1r[nt] = kk < 3 ? A.w1[n * 3 + kk] : 0.f; b1r[nt] = A.b1[n]; b2r[nt] = A.b2[n];
#pragma unroll
        for (int q = 0; q < 16; q++) w2r[nt][q] = w2s[n * FAS + kk * 16 + q];
#pragma unroll
        for (int c = 0; c < 2; c++) w3r[c][nt] = c < A.out_dim ? A.w3[c * FH + n] : 0.f;
    }
    const float b3r0 = A.b3[0], b3r1 = A.out_dim > 1 ? A.b3[1] : 0.f;
    const int n_tiles = (A.rn.n_envs + FTILE - 1) / FTILE;
    const int R = 10;
    for (int tile = blockIdx.x * FWAVES + wave; tile < n_tiles; tile += gridDim.x * FWAVES) {
        const int e = tile * FTILE + lane;
        const bool live = lane < FTILE && e < A.rn.n_envs;
        float th = 0.f, thd = 0.f, ep_ret = 0.f, noise = 0.f; uint32_t ep_step = 0, pos = 0, ces = 0; int full = 0;
        if (live) {
            const float2 st = reinterpret_cast<const float2*>(A.rn.states)[e];
            th = st.x; thd = st.y; ep_step = A.rn.episode_step[e]; ep_ret = A.rn.episode_return[e];
            pos = A.rb.position[e]; ces = A.rb.current_episode_start[e]; full = A.rb.full[e];
            if (A.policy_kind == 2) {
                noise = A.action_noise ? A.action_noise[e] : rlt_randn_element(A.seed, A.noise_stream + *A.stream_offset, (uint64_t)e);
                if (A.drawn_noise) A.drawn_noise[e] = noise;
            }
            if (A.rn.truncated[e]) {    // prologue (operations_generic_per_env.h:8-66): reset, flag the previous replay row
                if (A.initial_states) { const float2 ini = reinterpret_cast<const float2*>(A.initial_states)[e]; th = ini.x; thd = ini.y; }
                else {
                    const float PI = 3.14159265358979323846f;
                    const rlt_u32x4 draw = rlt_philox(A.seed, A.stream + *A.stream_offset, (uint64_t)e);
                    const float u0 = rlt_u01(draw.x), u1 = rlt_u01(draw.y);
                    th = -PI + 2.0f * PI * u0; thd = -1.0f + 2.0f * u1;
                }
                ep_step = 0; ep_ret = 0.f;
                if (full || pos > 0) {
                    const uint32_t prev = pos == 0 ? (uint32_t)A.rb.capacity - 1 : pos - 1;
                    A.rb.data[((size_t)e * A.rb.capacity + prev) * R + (R - 1)] = 1.0f;
                    ces = pos;
                }
            }
        }
        if (lane < FTILE) {
            float sn, cs; sincosf(th, &sn, &cs);
            xs[lane * FXS] = cs; xs[lane * FXS + 1] = sn; xs[lane * FXS + 2] = thd; xs[lane * FXS + 3] = 0.f;
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll 1
        for (int m = 0; m < FTILE / 16; m += 2) {       // 2 x 16 environments at a time: two independent chains of matrix instructions in flight
            // layer 1
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const float xa = xs[(16 * (m + h) + r) * FXS + kk];
#pragma unroll
                for (int nt = 0; nt < 4; nt++) {
                    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                    const floatx4 acc = mfma16(xa, w1r[nt], zero);
#pragma unroll
                    for (int v = 0; v < 4; v++) hs[h * 16 * FAS + (4 * kk + v) * FAS + 16 * nt + r] = rlt_act(acc[v] + b1r[nt], ACT_H);
                }
            }
            __builtin_amdgcn_wave_barrier();
            // layer 2, and layer 3 as partial dot products over this lane's hidden units
            float a[2][16];
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int q = 0; q < 16; q++) a[h][q] = hs[h * 16 * FAS + r * FAS + kk * 16 + q];
            float p0[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, p1[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int nt = 0; nt < 4; nt++) {
                floatx4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int q = 0; q < 16; q++) { acc0 = mfma16(a[0][q], w2r[nt][q], acc0); acc1 = mfma16(a[1][q], w2r[nt][q], acc1); }
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float g0 = rlt_act(acc0[v] + b2r[nt], ACT_H), g1 = rlt_act(acc1[v] + b2r[nt], ACT_H);
                    p0[0][v] += g0 * w3r[0][nt]; p1[0][v] += g0 * w3r[1][nt]; p0[1][v] += g1 * w3r[0][nt]; p1[1][v] += g1 * w3r[1][nt];
                }
            }
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float s0 = row16_sum(p0[h][v]), s1 = row16_sum(p1[h][v]);
                    if (r == v) { ys[(16 * (m + h) + 4 * kk + v) * 2] = s0; ys[(16 * (m + h) + 4 * kk + v) * 2 + 1] = s1; }
                }
            __builtin_amdgcn_wave_barrier();
        }
        if (live) {
            const float y0 = ys[lane * 2] + b3r0, y1 = ys[lane * 2 + 1] + b3r1;
            float action;
            if (A.policy_kind == 1) action = rlt_act(y0, A.act_out);
            else {      // sample_and_squash in rollout mode (nn/layers/sample_and_squash/operations_generic.h:149-195)
                const float ls = clampf(rlt_act(y1, A.act_out), A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
                action = tanhf(rlt_act(y0, A.act_out) + noise * expf(ls));
            }
            Transition t;
            pendulum_transition(A.rn.env, th, thd, action, t);     // epilogue (operations_generic_per_env.h:67-108)
            ep_step += 1;
            const bool truncated = ep_step == (uint32_t)A.rn.episode_step_limit;
            A.rn.episode_step[e] = ep_step; A.rn.episode_return[e] = ep_ret + t.reward; A.rn.truncated[e] = truncated;
            reinterpret_cast<float2*>(A.rn.states)[e] = make_float2(t.theta, t.theta_dot);
            float2* row = reinterpret_cast<float2*>(A.rb.data + ((size_t)e * A.rb.capacity + pos) * R);       // rows are 40 bytes: 8-byte aligned
            row[0] = make_float2(t.obs[0], t.obs[1]); row[1] = make_float2(t.obs[2], t.action); row[2] = make_float2(t.reward, t.next_obs[0]);
            row[3] = make_float2(t.next_obs[1], t.next_obs[2]); row[4] = make_float2(0.0f, truncated ? 1.0f : 0.0f);
            A.rb.episode_start[(size_t)e * A.rb.capacity + pos] = ces;
            pos = (pos + 1) % (uint32_t)A.rb.capacity;
            A.rb.position[e] = pos;
            if (truncated) ces = pos;
            A.rb.current_episode_start[e] = ces;
            if (pos == 0 && !full) A.rb.full[e] = 1;
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// ---- on-policy collection (rl/components/on_policy_runner/operations_generic_per_env.h:8-74), one lane per environment ----------
__device__ __forceinline__ float mul_add_rn(float a, float b, float c) {
#pragma clang fp contract(off)
    const float product = a * b;
    return product + c;
}
// prologue of step `step`: reset where truncated (the flag is cleared), observe into the dataset row of this step; with final = 1 only the
// observation after the last step is written
__global__ __launch_bounds__(256) void on_policy_prologue_kernel(rlt_pendulum_runner rn, rlt_on_policy_dataset D, const float* __restrict__ initial_states, int step, int final,
                                                                 int force_truncated) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        const size_t row = (size_t)step * rn.n_envs + e;
        if (!final) {
            bool truncated = rn.truncated[e] != 0 || force_truncated;
            if (step == 0) D.all_reset[(size_t)e * D.ld] = truncated ? 1.0f : 0.0f;      // reset aliases the first rows of all_reset
            if (truncated) {
                rn.truncated[e] = 0; rn.episode_step[e] = 0; rn.episode_return[e] = 0.0f;
                rn.states[2 * e] = initial_states[2 * row]; rn.states[2 * e + 1] = initial_states[2 * row + 1];
            }
        }
        float s, c;
        sincosf(rn.states[2 * e], &s, &c);
        float* o = D.observations + row * D.ld;
        o[0] = c; o[1] = s; o[2] = rn.states[2 * e + 1];
    }
}
// epilogue: sample the action around the actor's mean, its log-probability (random/operations_generic.h:73-81), step, reward, flags
__global__ __launch_bounds__(256) void on_policy_epilogue_kernel(rlt_pendulum_runner rn, rlt_on_policy_dataset D, const float* __restrict__ log_std,
                                                                 const float* __restrict__ action_noise, int step) {
    const float ls = log_std[0], sd = expf(ls);
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < rn.n_envs; e += gridDim.x * blockDim.x) {
        const size_t row = (size_t)step * rn.n_envs + e;
        const float mean = D.actions_mean[row * D.ld];
        const float action = mul_add_rn(action_noise[row], sd, mean);      // z * std + mean, rounded twice as the reference's CPU build does
        const float pre = (action - mean) / sd;
        D.actions[row * D.ld] = action;
        D.action_log_probs[row * D.ld] = (-0.9189385332046727f - ls) - 0.5f * pre * pre;
        Transition t;
        pendulum_transition(rn.env, rn.states[2 * e], rn.states[2 * e + 1], action, t);
        D.terminated[row * D.ld] = 0.0f;
        D.rewards[row * D.ld] = t.reward;
        rn.episode_return[e] += t.reward;
        const uint32_t n = rn.episode_step[e] + 1;
        rn.episode_step[e] = n;
        const bool truncated = rn.episode_step_limit > 0 && n >= (uint32_t)rn.episode_step_limit;
        D.truncated[row * D.ld] = truncated ? 1.0f : 0.0f;
        D.all_reset[(row + rn.n_envs) * D.ld] = truncated ? 1.0f : 0.0f;
        rn.truncated[e] = truncated;
        rn.states[2 * e] = t.theta; rn.states[2 * e + 1] = t.theta_dot;
    }
}

// The whole collection in one launch for 3 -> 64 -> 64 -> 1 actors: the environments do not interact, so a wavefront takes 16 of them through all the
// steps (prologue, standardize, actor on v_mfma_f32_16x16x4_f32 with W2 in registers, epilogue; the same arithmetic as the per-step kernels above), with
// the environment state in the registers of the 16 owning lanes between steps. Bound by the chain of steps_per_env dependent steps per wavefront.
struct CollectArgs {
    rlt_pendulum_runner rn; rlt_on_policy_dataset D;
    const float *w1, *b1, *w2, *b2, *w3, *b3;
    int act_out, force_truncated;
    const float* log_std; const float* standardize_mean; const float* standardize_precision; const float* action_noise; const float* initial_states;
};
constexpr int CWAVES = 4, COLLECT_LDS_PER_WAVE = 16 * FAS + 16 * 4 + 16;
template <int ACT_H>
__global__ __launch_bounds__(64 * CWAVES) void on_policy_collect_kernel(CollectArgs A) {
    __shared__ float lds[CWAVES * COLLECT_LDS_PER_WAVE + FH * FAS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, kk = lane >> 4;
    const lptr hs = (lptr)lds + wave * COLLECT_LDS_PER_WAVE, xs = hs + 16 * FAS, ys = xs + 16 * 4, w2s = (lptr)lds + CWAVES * COLLECT_LDS_PER_WAVE;
    for (int i = threadIdx.x; i < FH * FH; i += 64 * CWAVES) w2s[(i >> 6) * FAS + (i & 63)] = A.w2[i];
    __syncthreads();
    float w1r[4], b1r[4], w2r[4][16], b2r[4], w3r[4];
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        const int n = 16 * nt + r;
        w1r[nt] = kk < 3 ? A.w1[n * 3 + kk] : 0.f; b1r[nt] = A.b1[n]; b2r[nt] = A.b2[n]; w3r[nt] = A.w3[n];
#pragma unroll
        for (int q = 0; q < 16; q++) w2r[nt][q] = w2s[n * FAS + kk * 16 + q];
    }
    const float b3 = A.b3[0], ls = A.log_std[0], sd = expf(ls);
    float sm[3] = {0.f, 0.f, 0.f}, sp[3] = {0.f, 0.f, 0.f};
    if (A.standardize_mean) for (int c = 0; c < 3; c++) { sm[c] = A.standardize_mean[c]; sp[c] = A.standardize_precision[c]; }
    const int N = A.rn.n_envs, S = A.D.steps_per_env, n_tiles = (N + 15) / 16;
    const size_t ld = A.D.ld;
    for (int tile = blockIdx.x * CWAVES + wave; tile < n_tiles; tile += gridDim.x * CWAVES) {
        const int e = tile * 16 + lane;
        const bool live = lane < 16 && e < N;
        float th = 0.f, thd = 0.f, ep_ret = 0.f; uint32_t ep_step = 0; bool trunc = false;
        if (live) { th = A.rn.states[2 * e]; thd = A.rn.states[2 * e + 1]; ep_ret = A.rn.episode_return[e]; ep_step = A.rn.episode_step[e]; trunc = A.rn.truncated[e] != 0; }
        for (int step = 0; step < S; step++) {
            const size_t row = (size_t)step * N + e;
            if (live) {         // prologue (operations_generic_per_env.h:8-35): reset where truncated, observe into the dataset row of this step
                const bool truncated = trunc || (step == 0 && A.force_truncated);
                if (step == 0) A.D.all_reset[(size_t)e * ld] = truncated ? 1.0f : 0.0f;
                if (truncated) { trunc = false; ep_step = 0; ep_ret = 0.0f; th = A.initial_states[2 * row]; thd = A.initial_states[2 * row + 1]; }
                float sn, cs;
                sincosf(th, &sn, &cs);
                float* o = A.D.observations + row * ld;
                o[0] = cs; o[1] = sn; o[2] = thd;
                float x[3] = {cs, sn, thd};
                if (A.standardize_mean) {
#pragma unroll
                    for (int c = 0; c < 3; c++) { x[c] -= sm[c]; if (sp[c] != 0.0f) x[c] *= sp[c]; }
                }
                xs[lane * 4] = x[0]; xs[lane * 4 + 1] = x[1]; xs[lane * 4 + 2] = x[2]; xs[lane * 4 + 3] = 0.f;
            } else if (lane < 16) { xs[lane * 4] = 0.f; xs[lane * 4 + 1] = 0.f; xs[lane * 4 + 2] = 0.f; xs[lane * 4 + 3] = 0.f; }
            __builtin_amdgcn_wave_barrier();
            {   // layer 1
                const float xa = xs[r * 4 + kk];
#pragma unroll
                for (int nt = 0; nt < 4; nt++) {
                    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                    const floatx4 acc = mfma16(xa, w1r[nt], zero);
#pragma unroll
                    for (int v = 0; v < 4; v++) hs[(4 * kk + v) * FAS + 16 * nt + r] = rlt_act(acc[v] + b1r[nt], ACT_H);
                }
            }
            __builtin_amdgcn_wave_barrier();
            {   // layer 2, and layer 3 as partial dot products over this lane's hidden units
                float a[16];
#pragma unroll
                for (int q = 0; q < 16; q++) a[q] = hs[r * FAS + kk * 16 + q];
                float p[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int nt = 0; nt < 4; nt++) {
                    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int q = 0; q < 16; q++) acc = mfma16(a[q], w2r[nt][q], acc);
#pragma unroll
                    for (int v = 0; v < 4; v++) p[v] += rlt_act(acc[v] + b2r[nt], ACT_H) * w3r[nt];
                }
#pragma unroll
                for (int v = 0; v < 4; v++) { const float sum = row16_sum(p[v]); if (r == v) ys[4 * kk + v] = sum; }
            }
            __builtin_amdgcn_wave_barrier();
            if (live) {         // epilogue (:36-74): sample around the mean, log-probability (random/operations_generic.h:73-81), step, reward, flags
                const float mean = rlt_act(ys[lane] + b3, A.act_out);
                const float action = mul_add_rn(A.action_noise[row], sd, mean);
                const float pre = (action - mean) / sd;
                A.D.actions_mean[row * ld] = mean;
                A.D.actions[row * ld] = action;
                A.D.action_log_probs[row * ld] = (-0.9189385332046727f - ls) - 0.5f * pre * pre;
                Transition t;
                pendulum_transition(A.rn.env, th, thd, action, t);
                A.D.terminated[row * ld] = 0.0f;
                A.D.rewards[row * ld] = t.reward;
                ep_ret += t.reward;
                ep_step += 1;
                const bool truncated = A.rn.episode_step_limit > 0 && ep_step >= (uint32_t)A.rn.episode_step_limit;
                A.D.truncated[row * ld] = truncated ? 1.0f : 0.0f;
                A.D.all_reset[(row + N) * ld] = truncated ? 1.0f : 0.0f;
                trunc = truncated;
                th = t.theta; thd = t.theta_dot;
            }
            __builtin_amdgcn_wave_barrier();
        }
        if (live) {             // the observation after the last step, and the runner's state
            float sn, cs;
            sincosf(th, &sn, &cs);
            float* o = A.D.observations + ((size_t)S * N + e) * ld;
            o[0] = cs; o[1] = sn; o[2] = thd;
            A.rn.states[2 * e] = th; A.rn.states[2 * e + 1] = thd; A.rn.episode_return[e] = ep_ret; A.rn.episode_step[e] = ep_step; A.rn.truncated[e] = trunc;
        }
    }
}
// RLT_COLLECT_ONE_LAUNCH=0 keeps the collection on the per-step kernels (tests compare the two paths with each other)
bool evaluate_one_launch_enabled() { const char* v = std::getenv("RLT_EVALUATE_ONE_LAUNCH"); return !(v && v[0] == '0'); }
bool collect_one_launch_enabled() { const char* v = std::getenv("RLT_COLLECT_ONE_LAUNCH"); return !(v && v[0] == '0'); }
bool fused_collect_ok(const rlt_dense_layer* L, int n) {
    return n == 3 && L[0].in_dim == 3 && L[0].out_dim == FH && L[1].in_dim == FH && L[1].out_dim == FH && L[2].in_dim == FH && L[2].out_dim == 1 &&
           L[0].activation == L[1].activation;
}

int grid1(int n) { int b = (n + 255) / 256; return b > 2048 ? 2048 : (b < 1 ? 1 : b); }
// the shapes the one-launch step is built for
bool fused_runner_ok(const rlt_dense_layer* L, int n, int policy_kind, const rlt_replay_buffer* rb, const rlt_pendulum_runner* rn, const float* initial_states) {
    if (policy_kind == 0 || n != 3 || L[0].in_dim != 3 || L[0].out_dim != FH || L[1].in_dim != FH || L[1].out_dim != FH || L[2].in_dim != FH) return false;
    if (L[0].activation != L[1].activation) return false;
    return (((uintptr_t)rb->data | (uintptr_t)rn->states | (uintptr_t)initial_states) & 7) == 0;      // replay rows and states move as 8-byte pairs
}
bool rb_ok(const rlt_replay_buffer* rb) {
    return rb && rb->data && rb->episode_start && rb->position && rb->current_episode_start && rb->full && rb->n_envs > 0 && rb->capacity > 0 &&
           rb->observation_dim > 0 && rb->action_dim > 0;
}


// ---- evaluation episodes (rl/utils/evaluation/operations_generic.h:106-233) ----------------------------------------------------
// One launch runs every step of every episode for actors 3 -> H -> H -> out with H <= 64: a wavefront per episode, lane j holds hidden unit j of both
// hidden layers (its row of W1, its bias, its column of W3 in registers, W2 in LDS), the first layer's activations pass between lanes with
// v_readlane, the output is a wavefront sum; every lane carries a copy of the environment state, and the action that advances it is taken from one
// lane, so that the copies stay identical bit for bit. The chain of step_limit dependent steps bounds the kernel.
struct EvaluateArgs {
    rlt_pendulum_parameters env;
    const float *w1, *b1, *w2, *b2, *w3, *b3;
    const float *std_mean, *std_precision;      // a standardize layer in front of the actor: (observation - mean) * precision; NULL: none
    int H, act1, act2, act_out, policy_kind, step_limit;
    const float* initial_states; float* returns; uint32_t* episode_length;
};
__global__ __launch_bounds__(64) void pendulum_evaluate_kernel(EvaluateArgs A) {
    __shared__ float w2s[64 * 65];
    const int j = threadIdx.x, e = blockIdx.x, H = A.H;
    for (int n = 0; n < H; n++) if (j < H) w2s[n * 65 + j] = A.w2[n * H + j];
    __syncthreads();
    const bool live = j < H;
    const int jc = live ? j : 0;
    const float w10 = A.w1[jc * 3], w11 = A.w1[jc * 3 + 1], w12 = A.w1[jc * 3 + 2], b1 = A.b1[jc], b2 = A.b2[jc], w3 = live ? A.w3[jc] : 0.f, b3 = A.b3[0];
    float m0 = 0.f, m1 = 0.f, m2 = 0.f, p0 = 1.f, p1 = 1.f, p2 = 1.f;
    if (A.std_mean) { m0 = A.std_mean[0]; m1 = A.std_mean[1]; m2 = A.std_mean[2]; p0 = A.std_precision[0]; p1 = A.std_precision[1]; p2 = A.std_precision[2]; }
    float theta = A.initial_states[2 * e], theta_dot = A.initial_states[2 * e + 1], episode_return = 0.f;
    float sn, cs;
    sincosf(theta, &sn, &cs);
    for (int step = 0; step < A.step_limit; step++) {
        const float h1 = live ? rlt_act(b1 + w10 * ((cs - m0) * p0) + w11 * ((sn - m1) * p1) + w12 * ((theta_dot - m2) * p2), A.act1) : 0.f;
        float acc = b2;
        for (int k = 0; k < H; k++) acc += w2s[j * 65 + k] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(h1), k));
        const float h2 = live ? rlt_act(acc, A.act2) : 0.f;
        const float y = rlt_act(rlt_wave_sum(w3 * h2) + b3, A.act_out);
        // Evaluation mode: the action is the output, or the squashed mean of a [mean | log_std] head (sample_and_squash with zero noise).
        // Every lane carries a copy of the episode's state, and lane j's hidden unit is computed from lane j's copy: the copies must stay identical bit
        // for bit, or the network sees a state no single pendulum is in (a trained actor that balances the pendulum then loses it within 100 steps).
        // Taking the action from one lane makes that hold whatever the compiler does with the reduction above.
        const float action_own = A.policy_kind == 2 ? tanhf(y) : y;
        const float action = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(action_own)));
        Transition t;
        pendulum_transition(A.env, theta, theta_dot, action, t);
        theta = t.theta; theta_dot = t.theta_dot; cs = t.next_obs[0]; sn = t.next_obs[1];
        episode_return += t.reward;      // the Pendulum has no terminal states: every step counts (:188-197)
    }
    if (j == 0) { A.returns[e] = episode_return; A.episode_length[e] = (uint32_t)A.step_limit; }
}
// other actor shapes: one step of all episodes per launch around the per-layer network kernels
__global__ __launch_bounds__(256) void evaluate_observe_kernel(const float* __restrict__ states, float* __restrict__ obs, int n, const float* __restrict__ std_mean,
                                                               const float* __restrict__ std_precision) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    float sn, cs; sincosf(states[2 * e], &sn, &cs);
    float o[3] = {cs, sn, states[2 * e + 1]};
    if (std_mean) for (int i = 0; i < 3; i++) o[i] = (o[i] - std_mean[i]) * std_precision[i];
    obs[3 * e] = o[0]; obs[3 * e + 1] = o[1]; obs[3 * e + 2] = o[2];
}
__global__ __launch_bounds__(256) void evaluate_step_kernel(rlt_pendulum_parameters env, float* __restrict__ states, const float* __restrict__ actor_out, int ld_out, int policy_kind,
                                                            float* __restrict__ returns, uint32_t* __restrict__ episode_length, int n) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    const float y = actor_out[(size_t)e * ld_out], action = policy_kind == 2 ? tanhf(y) : y;
    Transition t;
    pendulum_transition(env, states[2 * e], states[2 * e + 1], action, t);
    states[2 * e] = t.theta; states[2 * e + 1] = t.theta_dot;
    returns[e] += t.reward; episode_length[e] += 1;
}
// mean and standard deviation of returns and episode lengths, accumulated in episode order as the reference does (:213-227)
__global__ void evaluate_summary_kernel(const float* __restrict__ returns, const uint32_t* __restrict__ episode_length, int n, float* __restrict__ summary) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    float rm = 0.f, rs = 0.f, lm = 0.f, ls = 0.f;
    for (int e = 0; e < n; e++) { rm += returns[e]; rs += returns[e] * returns[e]; lm += (float)episode_length[e]; ls += (float)(episode_length[e] * episode_length[e]); }
    rm /= (float)n; lm /= (float)n;
    summary[0] = rm; summary[1] = sqrtf(fmaxf(0.f, rs / (float)n - rm * rm));
    summary[2] = lm; summary[3] = sqrtf(fmaxf(0.f, ls / (float)n - lm * lm));
    summary[4] = 0.f; summary[5] = 0.f;       // num_terminated, share_terminated
}
}  // namespace

extern "C" {

int rlt_rocm_replay_add(rlt_rocm_device* device, const rlt_replay_buffer* rb, const float* observations, const float* actions, const float* rewards,
                        const float* next_observations, const uint8_t* terminated, const uint8_t* truncated) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && observations && actions && rewards && next_observations && terminated && truncated);
    hipLaunchKernelGGL(replay_add_kernel, dim3(grid1(rb->n_envs)), dim3(256), 0, device->stream, *rb, observations, actions, rewards, next_observations, terminated, truncated);
    return rlt_launch_status(device);
}

int rlt_rocm_gather_batch(rlt_rocm_device* device, const rlt_replay_buffer* rb, const uint32_t* env_indices, const uint32_t* sample_offsets, int deterministic,
                          int max_episode_length, int batch, float* observations_actions_base, float* rewards, uint8_t* terminated,
                          uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && batch > 0 && observations_actions_base && rewards && terminated && max_episode_length >= 0);
    RLT_REQUIRE(deterministic || (env_indices && sample_offsets));
    int* error_flag = (int*)(device->fault + 1);        // read back by rlt_rocm_check_status
    device->fault_armed = 1;
    hipLaunchKernelGGL(gather_kernel, dim3(grid1(batch * 16)), dim3(256), 0, device->stream, *rb, env_indices, sample_offsets, deterministic, max_episode_length, batch,
                       observations_actions_base, rewards, terminated, reset, next_reset_base, final_step_mask, next_final_step_mask_base, error_flag, 0, (uint64_t)0, (uint64_t)0,
                       (uint32_t*)nullptr, (uint32_t*)nullptr, (const uint64_t*)device->stream_offset);
    return rlt_launch_status(device);
}

int rlt_rocm_gather_batch_drawn(rlt_rocm_device* device, const rlt_replay_buffer* rb, uint64_t seed, uint64_t stream, uint32_t* drawn_env_indices, uint32_t* drawn_sample_offsets,
                                int max_episode_length, int batch, float* observations_actions_base, float* rewards, uint8_t* terminated,
                                uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && batch > 0 && observations_actions_base && rewards && terminated && max_episode_length >= 0);
    int* error_flag = (int*)(device->fault + 1);
    device->fault_armed = 1;
    hipLaunchKernelGGL(gather_kernel, dim3(grid1(batch * 16)), dim3(256), 0, device->stream, *rb, (const uint32_t*)nullptr, (const uint32_t*)nullptr, 0, max_episode_length, batch,
                       observations_actions_base, rewards, terminated, reset, next_reset_base, final_step_mask, next_final_step_mask_base, error_flag, 1, seed, stream,
                       drawn_env_indices, drawn_sample_offsets, (const uint64_t*)device->stream_offset);
    return rlt_launch_status(device);
}

int rlt_rocm_gather_sequence_batch(rlt_rocm_device* device, const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling, const rlt_sequence_draws* draws,
                                   int max_episode_length, const rlt_sequence_batch* B) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && sampling && draws && B && max_episode_length >= 0 && B->batch > 0 && B->sequence_length >= 1);
    RLT_REQUIRE(B->observations_actions_base && B->rewards && B->terminated && B->reset && B->next_reset_base && B->final_step_mask && B->next_final_step_mask_base);
    RLT_REQUIRE(draws->env_indices && draws->sample_offsets && (!sampling->random_seq_length || (draws->nominal && draws->lengths)));
    RLT_REQUIRE(!sampling->always_sample_from_initial_state || rb->capacity > max_episode_length);      // otherwise no row is eligible once a ring is full (:259)
    if (B->sequence_length + 1 > GATHER_SEQ_MAX_PADDED) return RLT_E_UNSUPPORTED;      // the kernel keeps a sample's four masks in LDS
    device->fault_armed = 1;
    hipLaunchKernelGGL(gather_sequence_kernel, dim3(grid1((size_t)B->batch * 64)), dim3(256), 0, device->stream, *rb, *sampling, *draws, max_episode_length, *B, (int*)(device->fault + 1));
    return rlt_launch_status(device);
}

int rlt_rocm_gather_draw(rlt_rocm_device* device, const rlt_replay_buffer* rb, int batch, uint64_t seed, uint64_t stream, uint32_t* env_indices, uint32_t* sample_offsets) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && batch > 0 && env_indices && sample_offsets);
    hipLaunchKernelGGL(gather_draw_kernel, dim3(grid1(batch)), dim3(256), 0, device->stream, *rb, batch, seed, stream, env_indices, sample_offsets, (const uint64_t*)device->stream_offset);
    return rlt_launch_status(device);
}

int rlt_rocm_gather_sequence_draw(rlt_rocm_device* device, const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling, int max_episode_length, int batch, int sequence_length,
                                  uint64_t seed, uint64_t stream, uint32_t* env_indices, uint32_t* sample_offsets, uint8_t* nominal, uint32_t* lengths) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rb_ok(rb) && sampling && batch > 0 && sequence_length >= 1 && max_episode_length >= 0 && env_indices && sample_offsets && nominal && lengths);
    RLT_REQUIRE(!sampling->always_sample_from_initial_state || rb->capacity > max_episode_length);
    hipLaunchKernelGGL(gather_sequence_draw_kernel, dim3(grid1((size_t)batch * ((3 * (sequence_length + 1) + 3 + 3) / 4))), dim3(256), 0, device->stream, *rb, *sampling, max_episode_length, batch, sequence_length, seed, stream,
                       env_indices, sample_offsets, nominal, lengths, (const uint64_t*)device->stream_offset);
    return rlt_launch_status(device);
}

int rlt_rocm_pendulum_step(rlt_rocm_device* device, const rlt_pendulum_parameters* p, float* states, const float* actions, float* observations,
                           float* next_observations, float* rewards, int n_envs) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(p && states && actions && n_envs > 0);
    hipLaunchKernelGGL(pendulum_step_kernel, dim3(grid1(n_envs)), dim3(256), 0, device->stream, *p, states, actions, observations, next_observations, rewards, n_envs);
    return rlt_launch_status(device);
}

static int runner_step(rlt_rocm_device* device, const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, int policy_kind,
                       const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas, const float* actions_in, const float* action_noise,
                       const float* initial_states, uint64_t seed, uint64_t stream, bool draw_noise, uint64_t noise_stream, float* drawn_noise);

int rlt_rocm_pendulum_runner_step(rlt_rocm_device* device, const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, int policy_kind,
                                  const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas, const float* actions_in, const float* action_noise,
                                  const float* initial_states, uint64_t seed, uint64_t stream) {
    return runner_step(device, rn, rb, policy_kind, actor, n_actor_layers, sas, actions_in, action_noise, initial_states, seed, stream, false, 0, nullptr);
}

int rlt_rocm_pendulum_runner_step_drawn(rlt_rocm_device* device, const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, const rlt_dense_layer* actor, int n_actor_layers,
                                        const rlt_sas_parameters* sas, float* drawn_noise, uint64_t seed, uint64_t noise_stream, uint64_t initial_state_stream) {
    return runner_step(device, rn, rb, 2, actor, n_actor_layers, sas, nullptr, nullptr, nullptr, seed, initial_state_stream, true, noise_stream, drawn_noise);
}

static int runner_step(rlt_rocm_device* device, const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, int policy_kind,
                       const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas, const float* actions_in, const float* action_noise,
                       const float* initial_states, uint64_t seed, uint64_t stream, bool draw_noise, uint64_t noise_stream, float* drawn_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rn->states && rn->episode_step && rn->episode_return && rn->truncated && rn->n_envs > 0 && rb_ok(rb));
    RLT_REQUIRE(rn->n_envs == rb->n_envs && rb->observation_dim == 3 && rb->action_dim == 1 && policy_kind >= 0 && policy_kind <= 2);
    RLT_REQUIRE(policy_kind != 0 || actions_in);
    RLT_REQUIRE(policy_kind == 0 || (actor && n_actor_layers >= 1 && actor[0].in_dim == 3 && actor[n_actor_layers - 1].out_dim == (policy_kind == 2 ? 2 : 1)));
    RLT_REQUIRE(policy_kind != 2 || (sas && (action_noise || draw_noise)));
    const int N = rn->n_envs;
    if (draw_noise && !fused_runner_ok(actor, n_actor_layers, policy_kind, rb, rn, initial_states)) {
        // the per-operation launches read the noise from an array: fill it first
        RLT_REQUIRE(drawn_noise);
        const int rc = rlt_rocm_randn_f32(device, drawn_noise, (size_t)N, seed, noise_stream);
        if (rc) return rc;
        action_noise = drawn_noise;
    }
    if (fused_runner_ok(actor, n_actor_layers, policy_kind, rb, rn, initial_states)) {
        FusedRunnerArgs a = {};
        a.rn = *rn; a.rb = *rb;
        a.w1 = actor[0].weights; a.b1 = actor[0].biases; a.w2 = actor[1].weights; a.b2 = actor[1].biases; a.w3 = actor[2].weights; a.b3 = actor[2].biases;
        a.act_hidden = actor[0].activation; a.act_out = actor[2].activation; a.out_dim = actor[2].out_dim; a.policy_kind = policy_kind;
        if (sas) a.sas = *sas;
        a.action_noise = action_noise; a.initial_states = initial_states; a.seed = seed; a.stream = stream;
        a.noise_stream = noise_stream; a.drawn_noise = action_noise ? nullptr : drawn_noise; a.stream_offset = device->stream_offset;
        const int tiles = rlt_div_up(N, FTILE);
        int blocks = rlt_div_up(tiles, FWAVES); if (blocks > device->compute_units) blocks = device->compute_units;
        switch (a.act_hidden) {
            case RLT_ACT_RELU: hipLaunchKernelGGL(runner_fused_kernel<RLT_ACT_RELU>, dim3(blocks), dim3(64 * FWAVES), 0, device->stream, a); break;
            case RLT_ACT_TANH: hipLaunchKernelGGL(runner_fused_kernel<RLT_ACT_TANH>, dim3(blocks), dim3(64 * FWAVES), 0, device->stream, a); break;
            case RLT_ACT_FAST_TANH: hipLaunchKernelGGL(runner_fused_kernel<RLT_ACT_FAST_TANH>, dim3(blocks), dim3(64 * FWAVES), 0, device->stream, a); break;
            case RLT_ACT_GELU: hipLaunchKernelGGL(runner_fused_kernel<RLT_ACT_GELU>, dim3(blocks), dim3(64 * FWAVES), 0, device->stream, a); break;
            case RLT_ACT_SIGMOID: hipLaunchKernelGGL(runner_fused_kernel<RLT_ACT_SIGMOID>, dim3(blocks), dim3(64 * FWAVES), 0, device->stream, a); break;
            default: hipLaunchKernelGGL(runner_fused_kernel<RLT_ACT_IDENTITY>, dim3(blocks), dim3(64 * FWAVES), 0, device->stream, a); break;
        }
        return rlt_launch_status(device);
    }
    // scratch: observations [N x 3], actor output [N x 2], actions [N], log-probs [N], then the MLP workspace
    size_t mlp_ws = policy_kind ? rlt_rocm_mlp_workspace_bytes(actor, n_actor_layers, N) : 0;
    size_t head = (((size_t)N * 7 * sizeof(float)) + 255) & ~(size_t)255;
    void* scratch; int rc = rlt_scratch(device, head + mlp_ws, &scratch); if (rc) return rc;
    float* obs = (float*)scratch; float* actor_out = obs + (size_t)N * 3; float* actions = actor_out + (size_t)N * 2; float* lp = actions + N;
    void* ws = (char*)scratch + head;
    hipLaunchKernelGGL(runner_prologue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *rb, initial_states, seed, stream, obs, (const uint64_t*)device->stream_offset);
    if ((rc = rlt_launch_status(device))) return rc;
    const float* act_ptr = actions;
    if (policy_kind == 0) act_ptr = actions_in;
    else if (policy_kind == 1) { if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, obs, 3, actions, 1, N, ws, mlp_ws))) return rc; }
    else {
        if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, obs, 3, actor_out, 2, N, ws, mlp_ws))) return rc;
        if ((rc = rlt_rocm_sas_forward(device, sas, actor_out, 2, action_noise, 1, actions, 1, nullptr, 0, lp, N, 1))) return rc;
    }
    hipLaunchKernelGGL(runner_epilogue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *rb, act_ptr);
    return rlt_launch_status(device);
}

size_t rlt_rocm_pendulum_runner_step_recurrent_workspace_bytes(const rlt_seq_layer* policy, int n_layers, int n_envs) {
    if (!policy || n_layers < 1 || n_envs < 1) return 0;
    return ((((size_t)n_envs * 7 * sizeof(float)) + 255) & ~(size_t)255) + rlt_rocm_seq_evaluate_step_workspace_bytes(policy, n_layers, n_envs) + 256;
}

// rl/components/off_policy_runner/operations_generic.h:189-238 with a sequential (recurrent) policy ending in [mean | log_std]: prologue, reset of the policy
// state where a new episode starts (the flags the prologue acted on: it leaves `truncated` as it found it), one evaluate_step, sample_and_squash, epilogue
int rlt_rocm_pendulum_runner_step_recurrent(rlt_rocm_device* device, const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n_layers,
                                            const rlt_seq_state* state, int auto_reset_period, const rlt_sas_parameters* sas, const float* action_noise,
                                            const float* initial_states, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rn->states && rn->episode_step && rn->episode_return && rn->truncated && rn->n_envs > 0 && rb_ok(rb));
    RLT_REQUIRE(rn->n_envs == rb->n_envs && rb->observation_dim == 3 && rb->action_dim == 1 && policy && n_layers >= 1 && state && sas && action_noise && initial_states);
    const int N = rn->n_envs;
    const size_t head = (((size_t)N * 7 * sizeof(float)) + 255) & ~(size_t)255;      // observations [N x 3], policy output [N x 2], actions [N], log-probabilities [N]
    const size_t step_ws = rlt_rocm_seq_evaluate_step_workspace_bytes(policy, n_layers, N);
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_pendulum_runner_step_recurrent_workspace_bytes(policy, n_layers, N));
    char* w = reinterpret_cast<char*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    float* obs = (float*)w; float* policy_out = obs + (size_t)N * 3; float* actions = policy_out + (size_t)N * 2; float* lp = actions + N;
    int rc;
    hipLaunchKernelGGL(runner_prologue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *rb, initial_states, (uint64_t)0, (uint64_t)0, obs, (const uint64_t*)device->stream_offset);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_seq_reset_state(device, policy, n_layers, state, rn->truncated, N))) return rc;
    if ((rc = rlt_rocm_seq_evaluate_step(device, policy, n_layers, obs, 3, state, auto_reset_period, policy_out, 2, N, w + head, step_ws))) return rc;
    if ((rc = rlt_rocm_sas_forward(device, sas, policy_out, 2, action_noise, 1, actions, 1, nullptr, 0, lp, N, 1))) return rc;
    hipLaunchKernelGGL(runner_epilogue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *rb, (const float*)actions);
    return rlt_launch_status(device);
}

size_t rlt_rocm_on_policy_collect_workspace_bytes(const rlt_pendulum_runner* rn, const rlt_dense_layer* actor, int n_actor_layers) {
    if (!rn || !actor || n_actor_layers < 1 || rn->n_envs < 1) return 0;
    return (((size_t)rn->n_envs * 3 * sizeof(float) + 255) & ~(size_t)255) + rlt_rocm_mlp_workspace_bytes(actor, n_actor_layers, rn->n_envs) + 256;
}

// rl/components/on_policy_runner/operations_generic.h:105-146: per step prologue, actor, epilogue; then the final observation
int rlt_rocm_on_policy_collect(rlt_rocm_device* device, const rlt_pendulum_runner* rn, const rlt_on_policy_dataset* D, const rlt_dense_layer* actor, int n_actor_layers,
                               const float* log_std, const float* standardize_mean, const float* standardize_precision, const float* action_noise,
                               const float* initial_states, int truncate_on_each_iteration, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(rn && rn->states && rn->episode_step && rn->episode_return && rn->truncated && rn->n_envs > 0 && D && D->steps_per_env > 0 && D->ld >= 3);
    RLT_REQUIRE(D->observations && D->actions_mean && D->actions && D->action_log_probs && D->rewards && D->terminated && D->truncated && D->all_reset);
    RLT_REQUIRE(actor && n_actor_layers >= 1 && actor[0].in_dim == 3 && actor[n_actor_layers - 1].out_dim == 1 && log_std && action_noise && initial_states);
    RLT_REQUIRE((standardize_mean == nullptr) == (standardize_precision == nullptr));
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_on_policy_collect_workspace_bytes(rn, actor, n_actor_layers));
    const int N = rn->n_envs;
    rlt_padded_net padded;
    if (collect_one_launch_enabled() && !fused_collect_ok(actor, n_actor_layers) && rlt_pad_eligible(actor, n_actor_layers)) {
        // hidden widths below 64 run the one-launch kernel on zero-padded copies of the parameters (pad.h)
        void* memory = nullptr;
        int rc = rlt_pad_scratch(device, rlt_pad_floats(actor, false) * sizeof(float), &memory);
        if (rc) return rc;
        if ((rc = rlt_pad_parameters(device, actor, (float*)memory, false, &padded))) return rc;
        if (fused_collect_ok(padded.L, 3)) actor = padded.L;
    }
    if (fused_collect_ok(actor, n_actor_layers) && collect_one_launch_enabled()) {
        CollectArgs a = {};
        a.rn = *rn; a.D = *D;
        a.w1 = actor[0].weights; a.b1 = actor[0].biases; a.w2 = actor[1].weights; a.b2 = actor[1].biases; a.w3 = actor[2].weights; a.b3 = actor[2].biases;
        a.act_out = actor[2].activation; a.force_truncated = truncate_on_each_iteration;
        a.log_std = log_std; a.standardize_mean = standardize_mean; a.standardize_precision = standardize_precision; a.action_noise = action_noise; a.initial_states = initial_states;
        int blocks = rlt_div_up(rlt_div_up(N, 16), CWAVES); if (blocks > device->compute_units) blocks = device->compute_units;
        switch (actor[0].activation) {
            case RLT_ACT_RELU: hipLaunchKernelGGL(on_policy_collect_kernel<RLT_ACT_RELU>, dim3(blocks), dim3(64 * CWAVES), 0, device->stream, a); break;
            case RLT_ACT_TANH: hipLaunchKernelGGL(on_policy_collect_kernel<RLT_ACT_TANH>, dim3(blocks), dim3(64 * CWAVES), 0, device->stream, a); break;
            case RLT_ACT_FAST_TANH: hipLaunchKernelGGL(on_policy_collect_kernel<RLT_ACT_FAST_TANH>, dim3(blocks), dim3(64 * CWAVES), 0, device->stream, a); break;
            case RLT_ACT_GELU: hipLaunchKernelGGL(on_policy_collect_kernel<RLT_ACT_GELU>, dim3(blocks), dim3(64 * CWAVES), 0, device->stream, a); break;
            case RLT_ACT_SIGMOID: hipLaunchKernelGGL(on_policy_collect_kernel<RLT_ACT_SIGMOID>, dim3(blocks), dim3(64 * CWAVES), 0, device->stream, a); break;
            default: hipLaunchKernelGGL(on_policy_collect_kernel<RLT_ACT_IDENTITY>, dim3(blocks), dim3(64 * CWAVES), 0, device->stream, a); break;
        }
        return rlt_launch_status(device);
    }
    float* standardized = reinterpret_cast<float*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    const size_t head = ((size_t)N * 3 * sizeof(float) + 255) & ~(size_t)255;
    void* ws = (char*)standardized + head;
    const size_t ws_bytes = workspace_bytes - (size_t)((char*)ws - (char*)workspace);
    int rc;
    for (int step = 0; step < D->steps_per_env; step++) {
        hipLaunchKernelGGL(on_policy_prologue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *D, initial_states, step, 0, step == 0 && truncate_on_each_iteration);
        if ((rc = rlt_launch_status(device))) return rc;
        const float* obs = D->observations + (size_t)step * N * D->ld; int ldo = D->ld;
        if (standardize_mean) {
            if ((rc = rlt_rocm_standardize_forward(device, standardize_mean, standardize_precision, obs, D->ld, standardized, 3, N, 3))) return rc;
            obs = standardized; ldo = 3;
        }
        if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, obs, ldo, D->actions_mean + (size_t)step * N * D->ld, D->ld, N, ws, ws_bytes))) return rc;
        hipLaunchKernelGGL(on_policy_epilogue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *D, log_std, action_noise, step);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    hipLaunchKernelGGL(on_policy_prologue_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *rn, *D, initial_states, D->steps_per_env, 1, 0);
    return rlt_launch_status(device);
}

// rl::utils::evaluation::evaluate with the Pendulum environment (rl/utils/evaluation/operations_generic.h:106-233)
int rlt_rocm_pendulum_evaluate(rlt_rocm_device* device, const rlt_pendulum_parameters* env, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers,
                               const float* initial_states, int n_episodes, int step_limit, float* returns, uint32_t* episode_length, float* summary) {
    return rlt_rocm_pendulum_evaluate_standardized(device, env, policy_kind, actor, n_actor_layers, nullptr, nullptr, initial_states, n_episodes, step_limit, returns,
                                                   episode_length, summary);
}
// the same with a standardize layer (nn/layers/standardize/operations_generic.h:69-135) in front of the actor, as PPO's actors have it
int rlt_rocm_pendulum_evaluate_standardized(rlt_rocm_device* device, const rlt_pendulum_parameters* env, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers,
                                            const float* observation_mean, const float* observation_precision, const float* initial_states, int n_episodes,
                                            int step_limit, float* returns, uint32_t* episode_length, float* summary) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(env && actor && n_actor_layers >= 1 && initial_states && n_episodes >= 1 && step_limit >= 1 && returns && episode_length && summary);
    RLT_REQUIRE((observation_mean == nullptr) == (observation_precision == nullptr));
    RLT_REQUIRE((policy_kind == 1 || policy_kind == 2) && actor[0].in_dim == 3 && actor[n_actor_layers - 1].out_dim == policy_kind);
    for (int l = 0; l < n_actor_layers; l++) RLT_REQUIRE(actor[l].weights && actor[l].biases && (l == 0 || actor[l].in_dim == actor[l - 1].out_dim));
    const int N = n_episodes;
    int rc;
    if (n_actor_layers == 3 && actor[0].out_dim <= 64 && actor[1].out_dim == actor[0].out_dim && evaluate_one_launch_enabled()) {
        EvaluateArgs a = {};
        a.env = *env;
        a.w1 = actor[0].weights; a.b1 = actor[0].biases; a.w2 = actor[1].weights; a.b2 = actor[1].biases; a.w3 = actor[2].weights; a.b3 = actor[2].biases;
        a.std_mean = observation_mean; a.std_precision = observation_precision;
        a.H = actor[0].out_dim; a.act1 = actor[0].activation; a.act2 = actor[1].activation; a.act_out = actor[2].activation; a.policy_kind = policy_kind; a.step_limit = step_limit;
        a.initial_states = initial_states; a.returns = returns; a.episode_length = episode_length;
        hipLaunchKernelGGL(pendulum_evaluate_kernel, dim3(N), dim3(64), 0, device->stream, a);
        if ((rc = rlt_launch_status(device))) return rc;
    } else {
        // scratch: states [N x 2], observations [N x 3], actor output [N x out], then the network workspace
        const int out_dim = policy_kind;
        const size_t mlp_ws = rlt_rocm_mlp_workspace_bytes(actor, n_actor_layers, N);
        const size_t head = (((size_t)N * (5 + out_dim) * sizeof(float)) + 255) & ~(size_t)255;
        void* scratch;
        if ((rc = rlt_scratch(device, head + mlp_ws, &scratch))) return rc;
        float* states = (float*)scratch; float* obs = states + (size_t)N * 2; float* out = obs + (size_t)N * 3;
        void* ws = (char*)scratch + head;
        RLT_HIP(hipMemcpyAsync(states, initial_states, (size_t)N * 2 * sizeof(float), hipMemcpyDeviceToDevice, device->stream));
        if ((rc = rlt_rocm_fill_f32(device, returns, 1, N, N, 0.0f))) return rc;
        if ((rc = rlt_rocm_fill_f32(device, (float*)episode_length, 1, N, N, 0.0f))) return rc;      // the bit pattern of 0.0f is the integer 0
        for (int step = 0; step < step_limit; step++) {
            hipLaunchKernelGGL(evaluate_observe_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, states, obs, N, observation_mean, observation_precision);
            if ((rc = rlt_launch_status(device))) return rc;
            if ((rc = rlt_rocm_mlp_evaluate(device, actor, n_actor_layers, obs, 3, out, out_dim, N, ws, mlp_ws))) return rc;
            hipLaunchKernelGGL(evaluate_step_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *env, states, out, out_dim, policy_kind, returns, episode_length, N);
            if ((rc = rlt_launch_status(device))) return rc;
        }
    }
    hipLaunchKernelGGL(evaluate_summary_kernel, dim3(1), dim3(64), 0, device->stream, returns, episode_length, N, summary);
    return rlt_launch_status(device);
}

size_t rlt_rocm_pendulum_evaluate_recurrent_workspace_bytes(const rlt_seq_layer* policy, int n_layers, int n_episodes) {
    if (!policy || n_layers < 1 || n_episodes < 1) return 0;
    return ((((size_t)n_episodes * 7 * sizeof(float)) + 255) & ~(size_t)255) + rlt_rocm_seq_evaluate_step_workspace_bytes(policy, n_layers, n_episodes) + 256;
}

// rl::utils::evaluation::evaluate (rl/utils/evaluation/operations_generic.h:106-233) with a sequential (recurrent) policy: the kept state of every episode is reset
// before the first step (:135), every step is one evaluate_step (:163); the policy keeps seeing terminated episodes, only their environment stops
int rlt_rocm_pendulum_evaluate_recurrent(rlt_rocm_device* device, const rlt_pendulum_parameters* env, int policy_kind, const rlt_seq_layer* policy, int n_layers,
                                         const rlt_seq_state* state, int auto_reset_period, const float* initial_states, int n_episodes, int step_limit,
                                         float* returns, uint32_t* episode_length, float* summary, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(env && policy && n_layers >= 1 && state && initial_states && n_episodes >= 1 && step_limit >= 1 && returns && episode_length && summary);
    RLT_REQUIRE((policy_kind == 1 || policy_kind == 2) && auto_reset_period >= 0 && n_layers <= RLT_SEQ_MAX_LAYERS);
    RLT_REQUIRE((policy[0].kind ? policy[0].gru.input_dim : policy[0].dense.in_dim) == 3);
    RLT_REQUIRE((policy[n_layers - 1].kind ? policy[n_layers - 1].gru.hidden_dim : policy[n_layers - 1].dense.out_dim) == policy_kind);
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_pendulum_evaluate_recurrent_workspace_bytes(policy, n_layers, n_episodes));
    const int N = n_episodes;
    const size_t head = (((size_t)N * 7 * sizeof(float)) + 255) & ~(size_t)255;      // states [N x 2], observations [N x 3], policy output [N x kind]
    const size_t step_ws = rlt_rocm_seq_evaluate_step_workspace_bytes(policy, n_layers, N);
    char* w = reinterpret_cast<char*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    float* states = (float*)w; float* obs = states + (size_t)N * 2; float* out = obs + (size_t)N * 3;
    int rc;
    RLT_HIP(hipMemcpyAsync(states, initial_states, (size_t)N * 2 * sizeof(float), hipMemcpyDeviceToDevice, device->stream));
    if ((rc = rlt_rocm_fill_f32(device, returns, 1, N, N, 0.0f))) return rc;
    if ((rc = rlt_rocm_fill_f32(device, (float*)episode_length, 1, N, N, 0.0f))) return rc;      // the bit pattern of 0.0f is the integer 0
    if ((rc = rlt_rocm_seq_reset_state(device, policy, n_layers, state, nullptr, N))) return rc;
    for (int step = 0; step < step_limit; step++) {
        hipLaunchKernelGGL(evaluate_observe_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, states, obs, N, (const float*)nullptr, (const float*)nullptr);
        if ((rc = rlt_launch_status(device))) return rc;
        if ((rc = rlt_rocm_seq_evaluate_step(device, policy, n_layers, obs, 3, state, auto_reset_period, out, policy_kind, N, w + head, step_ws))) return rc;
        hipLaunchKernelGGL(evaluate_step_kernel, dim3(grid1(N)), dim3(256), 0, device->stream, *env, states, out, policy_kind, policy_kind, returns, episode_length, N);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    hipLaunchKernelGGL(evaluate_summary_kernel, dim3(1), dim3(64), 0, device->stream, returns, episode_length, N, summary);
    return rlt_launch_status(device);
}

}  // extern "C"
