// Persistent SAC-on-Pendulum training loop: N reference loop steps in ONE launch.
//
// reference: rl/algorithms/sac/loop/core/operations_generic.h:110-155 (step), the runner step it calls
// (rl/components/off_policy_runner/operations_generic.h:183-238, operations_generic_per_env.h:8-108), gather_batch (:240-430),
// train_critic / update_critic_targets / train_actor (rl/algorithms/sac/operations_generic.h:243-527). The reference's CUDA
// example replays three captured graphs of ~100 tiny launches per step (src/rl/environments/pendulum/sac/cuda/sac.cu:122-164);
// at batch 256 and width 64 a step is 43 MFLOP, so launch latency, not arithmetic, sets its speed.
//
// Here G = batch/16 workgroups stay resident for the whole run. Each owns 16 samples of the batch, keeps nothing but
// activations in LDS, reads weights straight from L2 (each weight is used once per pass by a 16-row tile, so staging buys
// nothing) and contracts with v_mfma_f32_16x16x4_f32. Per loop step:
//   S0  every workgroup redundantly advances the single environment (actor on one observation, dynamics, reward) so that
//       the new transition is known everywhere without a grid barrier; workgroup 0 writes it to the replay ring
//   S1  gather of the workgroup's 16 samples; next actions + log-probabilities from the actor; both target critics;
//       TD target; both critics forward + backward -> per-workgroup partial gradients
//   --- grid barrier ---
//   S2  each workgroup sums a slice of the partial gradients (fixed order), applies Adam and the polyak target update
//   --- grid barrier ---
//   S3  actor forward, both critics forward / backward_input, min-Q routing, sample_and_squash backward, actor backward
//       -> partial gradients
//   --- grid barrier ---
//   S4  Adam on the actor slice and on log_alpha
//   --- grid barrier ---
// Two wave groups of four wavefronts each work on independent networks (critic 0 / critic 1) at the same time.
#include "common.h"

typedef float floatx4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int H = 64;           // hidden width this kernel is built for
constexpr int ROWS = 16;        // samples per workgroup (one MFMA tile of rows)
constexpr int AS = H + 1;       // LDS row stride of activation buffers
constexpr int XS = 17;          // LDS row stride of network inputs (<= 16 columns)
constexpr int THREADS = 512;
constexpr int MAX_G = 64;

struct FusedArgs {
    // parameter / moment / gradient arenas ([W1|b1|W2|b2|W3|b3] each)
    float* actor_p; float* actor_g; float* actor_m; float* actor_v;
    float* critic_p[2]; float* critic_g[2]; float* critic_m[2]; float* critic_v[2];
    float* target_p[2];
    float* log_alpha;   // [4] parameter, gradient, first moment, second moment
    uint32_t* actor_age; uint32_t* critic_age[2]; uint32_t* alpha_age;
    rlt_adam_parameters adam_actor, adam_critic, adam_alpha;
    rlt_sas_parameters sas;
    float gamma, polyak;
    int obs, act, batch, n_steps;
    rlt_pendulum_runner runner;
    rlt_replay_buffer rb;
    float* partial;            // [G][2*n_critic + n_actor + 8]
    unsigned* barrier_counter;
    // optional host-drawn randomness (parity runs); NULL -> counter-based device RNG
    const float* rollout_noise; const float* initial_states; const uint32_t* sample_offsets;
    const float* noise_critic; const float* noise_actor;
    uint64_t seed, step_offset;
    float* out_critic_loss;    // [n_steps][2] optional
    // batch views for inspection (optional): last gathered batch / targets
    float* out_oab; float* out_rewards; uint8_t* out_terminated; float* out_target;
};

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

__device__ __forceinline__ void grid_barrier(unsigned* counter, unsigned target) {
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        while (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < target) __builtin_amdgcn_s_sleep(1);
    }
    __syncthreads();
}

__device__ __forceinline__ uint32_t mix32(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull; x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull; x = (x ^ (x >> 27)) * 0x94D049BB133111EBull; x ^= x >> 31;
    return (uint32_t)(x >> 32);
}
__device__ __forceinline__ float u01(uint32_t x) { return ((x >> 8) + 0.5f) * (1.0f / 16777216.0f); }
// standard normal from a (seed, stream, index) triple: Box-Muller on two hashed uniforms
__device__ __forceinline__ float randn_at(uint64_t seed, uint64_t stream, uint64_t index) {
    uint64_t key = seed ^ (stream * 0xD1B54A32D192ED03ull) ^ (index * 0x9E3779B97F4A7C15ull);
    float u1 = u01(mix32(key)), u2 = u01(mix32(key ^ 0xA5A5A5A5A5A5A5A5ull));
    return sqrtf(-2.0f * logf(u1)) * cosf(6.283185307179586f * u2);
}
__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }

// ---- 16-row tile contractions. Lane l of a wavefront: r = l & 15, kk = l >> 4. An instruction consumes 4 values of the
// reduction index, one per kk; lane group kk is given the contiguous range [kk*NM, (kk+1)*NM) of it (any fixed assignment of
// reduction indices to (instruction, kk) is valid as long as A and B agree), so each lane reads NM consecutive values.
// Result element v of lane l: row 4*kk + v, column r.

// forward: D[s][n0+r] = sum_k in[s][k] * W[n0+r][k]   (in: LDS rows = samples; W: global, row-major [N x K])
template <int NM>
__device__ __forceinline__ floatx4 fwd_tile(const float* in, int in_stride, int K, const float* __restrict__ W, int n0, int N, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = n0 + r;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NM; s++) {
        const int k = kk * NM + s;
        const float a = (k < K) ? in[r * in_stride + k] : 0.f;
        const float b = (k < K && n < N) ? W[n * K + k] : 0.f;
        acc = mfma16(a, b, acc);
    }
    return acc;
}
// the same with the reduction range restricted to [k_begin, k_begin + 4*NM) (split of K across wavefronts)
template <int NM>
__device__ __forceinline__ floatx4 fwd_tile_ksplit(const float* in, int in_stride, int K, int k_begin, const float* __restrict__ W, int N, int lane) {
    const int r = lane & 15, kk = lane >> 4;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NM; s++) {
        const int k = k_begin + kk * NM + s;
        const float a = (k < K) ? in[r * in_stride + k] : 0.f;
        const float b = (k < K && r < N) ? W[r * K + k] : 0.f;
        acc = mfma16(a, b, acc);
    }
    return acc;
}
// d_input: D[s][i0+r] = sum_o dpre[s][o] * W[o][i0+r]   (W: global [O x I])
template <int NM>
__device__ __forceinline__ floatx4 bwdin_tile(const float* dpre, int stride, int O, int o_begin, const float* __restrict__ W, int I, int i0, int lane) {
    const int r = lane & 15, kk = lane >> 4, i = i0 + r;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NM; s++) {
        const int o = o_begin + kk * NM + s;
        const float a = (o < O) ? dpre[r * stride + o] : 0.f;
        const float b = (o < O && i < I) ? W[o * I + i] : 0.f;
        acc = mfma16(a, b, acc);
    }
    return acc;
}
// weight gradient over the 16 samples: D[o0 + 4*kk + v][i0 + r] = sum_s dpre[s][o0+..] * in[s][i0+r]
__device__ __forceinline__ floatx4 wgrad_tile(const float* dpre, int dstride, int O, int o0, const float* in, int istride, int I, int i0, int lane) {
    const int r = lane & 15, kk = lane >> 4;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int smp = kk * 4 + s;
        const float a = (o0 + r < O) ? dpre[smp * dstride + o0 + r] : 0.f;
        const float b = (i0 + r < I) ? in[smp * istride + i0 + r] : 0.f;
        acc = mfma16(a, b, acc);
    }
    return acc;
}

// arena offsets of a 3-layer network in -> H -> H -> out
struct NetLayout {
    int in, out;
    __device__ __host__ int w1() const { return 0; }
    __device__ __host__ int b1() const { return H * in; }
    __device__ __host__ int w2() const { return H * in + H; }
    __device__ __host__ int b2() const { return H * in + H + H * H; }
    __device__ __host__ int w3() const { return H * in + H + H * H + H; }
    __device__ __host__ int b3() const { return H * in + H + H * H + H + out * H; }
    __device__ __host__ int total() const { return H * in + H + H * H + H + out * H + out; }
};

// LDS working set of one wave group (row strides: AS for the H-wide buffers, XS for the <= 16-wide ones)
struct GroupLds {
    float x[ROWS * XS];        // network input rows
    float h1[ROWS * AS];       // relu outputs of layer 1
    float h2[ROWS * AS];       // relu outputs of layer 2
    float dp1[ROWS * AS];      // d_pre of layer 1
    float dp2[ROWS * AS];      // d_pre of layer 2
    float out[ROWS * XS];      // network outputs
    float dout[ROWS * XS];     // gradient at the (identity) output
    float din[ROWS * XS];      // gradient wrt the network input
    float part[4 * ROWS * 16]; // K-split partial tiles
};
// The buffers one pass works on. For a backward_input-only pass h1/h2 may alias dp1/dp2 (every element is read and then
// written by the same lane, and no weight gradient reads the activations afterwards).
struct NetBufs { const float* x; float* h1; float* h2; float* out; float* dp1; float* dp2; const float* dout; float* din; float* part; };
// built member by member: an aggregate of LDS addresses would be folded into a constant initialiser, which LDS symbols cannot be
__device__ __forceinline__ NetBufs make_bufs(const float* x, float* h1, float* h2, float* out, float* dp1, float* dp2, const float* dout, float* din, float* part) {
    NetBufs b;
    b.x = x; b.h1 = h1; b.h2 = h2; b.out = out; b.dp1 = dp1; b.dp2 = dp2; b.dout = dout; b.din = din; b.part = part;
    return b;
}

// Forward of one 3-layer network on 16 rows by the four wavefronts of a group (w = wavefront within the group). Contains
// workgroup barriers: every wavefront of the workgroup calls it the same number of times, `active` gates the work.
__device__ __noinline__ void net_forward(bool active, NetBufs B, const float* __restrict__ P, NetLayout nl, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4;
    if (active) {   // layer 1: in -> H, one 16-column tile per wavefront
        floatx4 acc = fwd_tile<4>(B.x, XS, nl.in, P + nl.w1(), 16 * w, H, lane);
        const float b = P[nl.b1() + 16 * w + r];
#pragma unroll
        for (int v = 0; v < 4; v++) B.h1[(4 * kk + v) * AS + 16 * w + r] = fmaxf(acc[v] + b, 0.f);
    }
    __syncthreads();
    if (active) {   // layer 2: H -> H
        floatx4 acc = fwd_tile<16>(B.h1, AS, H, P + nl.w2(), 16 * w, H, lane);
        const float b = P[nl.b2() + 16 * w + r];
#pragma unroll
        for (int v = 0; v < 4; v++) B.h2[(4 * kk + v) * AS + 16 * w + r] = fmaxf(acc[v] + b, 0.f);
    }
    __syncthreads();
    if (active) {   // layer 3: H -> out (<= 16 columns): the reduction is split over the four wavefronts
        floatx4 acc = fwd_tile_ksplit<4>(B.h2, AS, H, 16 * w, P + nl.w3(), nl.out, lane);
#pragma unroll
        for (int v = 0; v < 4; v++) B.part[(w * ROWS + 4 * kk + v) * 16 + r] = acc[v];
    }
    __syncthreads();
    if (active) {
        const int t = w * 64 + lane, s = t >> 4, c = t & 15;       // 256 lanes of the group: one (row, column) each
        if (c < nl.out) B.out[s * XS + c] = ((B.part[(0 * ROWS + s) * 16 + c] + B.part[(1 * ROWS + s) * 16 + c]) + (B.part[(2 * ROWS + s) * 16 + c] + B.part[(3 * ROWS + s) * 16 + c])) + P[nl.b3() + c];
    }
    __syncthreads();
}

// Backward from B.dout (gradient at the identity output). want_w: weight and bias gradients of the 16 rows into G (arena layout);
// want_din: gradient wrt the input rows into B.din. Same barrier discipline as net_forward.
__device__ __noinline__ void net_backward(bool active, NetBufs B, const float* __restrict__ P, NetLayout nl, float* __restrict__ G, bool want_w, bool want_din, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, t = w * 64 + lane;
    if (active) {
        // layer 3: dW3 = dout^T h2 (out x H, an i-tile per wavefront), db3 = column sums; d_h2 = dout W3 gated by relu'(h2)
        if (want_w) {
            floatx4 acc = wgrad_tile(B.dout, XS, nl.out, 0, B.h2, AS, H, 16 * w, lane);
#pragma unroll
            for (int v = 0; v < 4; v++) if (4 * kk + v < nl.out) G[nl.w3() + (4 * kk + v) * H + 16 * w + r] = acc[v];
            if (t < nl.out) { float s = 0.f; for (int i = 0; i < ROWS; i++) s += B.dout[i * XS + t]; G[nl.b3() + t] = s; }
        }
        floatx4 acc = bwdin_tile<4>(B.dout, XS, nl.out, 0, P + nl.w3(), H, 16 * w, lane);
#pragma unroll
        for (int v = 0; v < 4; v++) { const int idx = (4 * kk + v) * AS + 16 * w + r; B.dp2[idx] = B.h2[idx] > 0.f ? acc[v] : 0.f; }
    }
    __syncthreads();
    if (active) {
        // layer 2: dW2 = dp2^T h1 (wavefront w owns rows [16w,16w+16) and walks the four i-tiles), db2; d_h1 = dp2 W2 gated by relu'(h1)
        if (want_w) {
#pragma unroll
            for (int it = 0; it < 4; it++) {
                floatx4 acc = wgrad_tile(B.dp2, AS, H, 16 * w, B.h1, AS, H, 16 * it, lane);
#pragma unroll
                for (int v = 0; v < 4; v++) G[nl.w2() + (16 * w + 4 * kk + v) * H + 16 * it + r] = acc[v];
            }
            if (lane < 16) { float s = 0.f; for (int i = 0; i < ROWS; i++) s += B.dp2[i * AS + 16 * w + lane]; G[nl.b2() + 16 * w + lane] = s; }
        }
        floatx4 acc = bwdin_tile<16>(B.dp2, AS, H, 0, P + nl.w2(), H, 16 * w, lane);
#pragma unroll
        for (int v = 0; v < 4; v++) { const int idx = (4 * kk + v) * AS + 16 * w + r; B.dp1[idx] = B.h1[idx] > 0.f ? acc[v] : 0.f; }
    }
    __syncthreads();
    if (active) {
        // layer 1: dW1 = dp1^T x (H x in, an o-tile per wavefront), db1; d_in = dp1 W1 with the reduction split over the wavefronts
        if (want_w) {
            floatx4 acc = wgrad_tile(B.dp1, AS, H, 16 * w, B.x, XS, nl.in, 0, lane);
#pragma unroll
            for (int v = 0; v < 4; v++) if (r < nl.in) G[nl.w1() + (16 * w + 4 * kk + v) * nl.in + r] = acc[v];
            if (lane < 16) { float s = 0.f; for (int i = 0; i < ROWS; i++) s += B.dp1[i * AS + 16 * w + lane]; G[nl.b1() + 16 * w + lane] = s; }
        }
        if (want_din) {
            floatx4 acc = bwdin_tile<4>(B.dp1, AS, H, 16 * w, P + nl.w1(), nl.in, 0, lane);
#pragma unroll
            for (int v = 0; v < 4; v++) B.part[(w * ROWS + 4 * kk + v) * 16 + r] = acc[v];
        }
    }
    __syncthreads();
    if (active && want_din) {
        const int s = t >> 4, c = t & 15;
        if (c < nl.in) B.din[s * XS + c] = (B.part[(0 * ROWS + s) * 16 + c] + B.part[(1 * ROWS + s) * 16 + c]) + (B.part[(2 * ROWS + s) * 16 + c] + B.part[(3 * ROWS + s) * 16 + c]);
    }
    __syncthreads();
}

// Adam on one element (nn/optimizers/adam/instance/operations_generic.h:26-72)
__device__ __forceinline__ float adam_element(const rlt_adam_parameters& p, float bc1, float bc2, float g, float& m, float& v, float param) {
    if (p.enable_gradient_clipping) g = clampf(g, -p.gradient_clip_value, p.gradient_clip_value);
    m = p.beta_1 * m + (1.0f - p.beta_1) * g;
    v = p.beta_2 * v + (1.0f - p.beta_2) * g * g;
    const float pre_sqrt = fmaxf(v * bc2, p.epsilon_sqrt);
    return param - p.alpha * bc1 * m / (sqrtf(pre_sqrt) + p.epsilon);
}

struct Shared {
    GroupLds grp[2];
    // single-environment state, replicated in every workgroup
    float th, thd, ep_return; unsigned ep_step; int truncated;
    unsigned rb_pos, rb_ces; int rb_full;
    unsigned new_pos;
    float new_row[16];
    float a1[H]; float a2[H]; float apart[4 * H]; float aout[8];
    float nx[ROWS * XS];          // second set of input rows: [next_obs | next_action] (S1), [obs | new action] (S3)
    float dci[2][ROWS * 4];       // action columns of d_critic_k_input
    // per-sample vectors of the workgroup's 16 rows
    float reward[ROWS]; float notdone[ROWS]; float next_logp[ROWS]; float y[ROWS]; float q[2][ROWS]; float nq[2][ROWS];
    float noise[ROWS * 4]; float act_pre[ROWS * 4]; float act_a[ROWS * 4]; float logp[ROWS]; float red[16];
};

__global__ __launch_bounds__(THREADS) void sac_pendulum_loop_kernel(FusedArgs A) {
    __shared__ Shared S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, grp = wave >> 2, w = wave & 3;
    const int g = blockIdx.x, G = gridDim.x;
    const int OBS = A.obs, ACT = A.act, D = OBS + ACT, B = A.batch;
    const NetLayout NA{OBS, 2 * ACT}, NC{D, 1};
    const int n_a = NA.total(), n_c = NC.total();
    const int n_partial = 2 * n_c + n_a + 8;
    float* const my_partial = A.partial + (size_t)g * n_partial;
    GroupLds& L = S.grp[grp];
    const int R = 2 * OBS + ACT + 3;
    unsigned barrier_index = 0;

    if (tid == 0) {
        S.th = A.runner.states[0]; S.thd = A.runner.states[1]; S.ep_return = A.runner.episode_return[0];
        S.ep_step = A.runner.episode_step[0]; S.truncated = A.runner.truncated[0];
        S.rb_pos = A.rb.position[0]; S.rb_ces = A.rb.current_episode_start[0]; S.rb_full = A.rb.full[0];
    }
    // optimiser ages advance by exactly one per loop step: keep them in registers, write back at the end
    const uint32_t age_actor0 = *A.actor_age, age_c00 = *A.critic_age[0], age_c10 = *A.critic_age[1], age_alpha0 = *A.alpha_age;
    __syncthreads();

    for (int step = 0; step < A.n_steps; step++) {
        const uint64_t gstep = A.step_offset + (uint64_t)step;
        // ================= S0: environment step (identical in every workgroup) =================
        if (tid == 0) {
            if (S.truncated) {   // prologue_per_env: reset, mark the previous row truncated
                if (A.initial_states) { S.th = A.initial_states[2 * step]; S.thd = A.initial_states[2 * step + 1]; }
                else {
                    const float PI = 3.14159265358979323846f;
                    S.th = -PI + 2.0f * PI * u01(mix32(A.seed ^ (gstep * 8 + 1))); S.thd = -1.0f + 2.0f * u01(mix32(A.seed ^ (gstep * 8 + 2)));
                }
                S.ep_step = 0; S.ep_return = 0.f;
                if (S.rb_full || S.rb_pos > 0) {
                    const unsigned prev = S.rb_pos == 0 ? (unsigned)A.rb.capacity - 1 : S.rb_pos - 1;
                    if (g == 0) A.rb.data[(size_t)prev * R + (R - 1)] = 1.0f;
                    S.rb_ces = S.rb_pos;
                }
            }
            float sn, cs; sincosf(S.th, &sn, &cs);
            S.new_row[0] = cs; S.new_row[1] = sn; S.new_row[2] = S.thd;
        }
        __syncthreads();
        // actor on the single observation (vector ALU: one row does not fill a matrix tile)
        if (tid < H) {
            float s = A.actor_p[NA.b1() + tid];
            for (int k = 0; k < OBS; k++) s += A.actor_p[NA.w1() + tid * OBS + k] * S.new_row[k];
            S.a1[tid] = fmaxf(s, 0.f);
        }
        __syncthreads();
        if (tid < 4 * H) {
            const int u = tid & 63, qd = tid >> 6;
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < 16; k++) s += A.actor_p[NA.w2() + u * H + 16 * qd + k] * S.a1[16 * qd + k];
            S.apart[qd * H + u] = s;
        }
        __syncthreads();
        if (tid < H) S.a2[tid] = fmaxf(((S.apart[tid] + S.apart[H + tid]) + (S.apart[2 * H + tid] + S.apart[3 * H + tid])) + A.actor_p[NA.b2() + tid], 0.f);
        __syncthreads();
        if (wave < 2 * ACT) {
            float s = A.actor_p[NA.w3() + wave * H + lane] * S.a2[lane];
            s = rlt_wave_sum(s);
            if (lane == 0) S.aout[wave] = s + A.actor_p[NA.b3() + wave];
        }
        __syncthreads();
        if (tid == 0) {
            // sample_and_squash in rollout mode (one action dimension for Pendulum), dynamics, reward, replay add
            const float mean = S.aout[0], ls = clampf(S.aout[1], A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
            const float eps = A.rollout_noise ? A.rollout_noise[step] : randn_at(A.seed, 3, gstep);
            const float action = tanhf(mean + eps * expf(ls));
            const rlt_pendulum_parameters& p = A.runner.env;
            float u = p.max_torque * clampf(action, -1.f, 1.f);
            u = clampf(u, -p.max_torque, p.max_torque);
            float nthd = S.thd + (3.0f * p.g / (2.0f * p.l) * S.new_row[1] + 3.0f / (p.m * p.l * p.l) * u) * p.dt;
            nthd = clampf(nthd, -p.max_speed, p.max_speed);
            const float nth = S.th + nthd * p.dt;
            const float PI = 3.14159265358979323846f;
            const float a0 = S.th + PI, b0 = 2.0f * PI;
            const float an = (a0 - b0 * floorf(a0 / b0)) - PI;
            const float ur = p.max_torque * action;
            const float reward = -(an * an + 0.1f * S.thd * S.thd + 0.001f * (ur * ur));
            float sn, cs; sincosf(nth, &sn, &cs);
            S.new_row[3] = action; S.new_row[4] = reward; S.new_row[5] = cs; S.new_row[6] = sn; S.new_row[7] = nthd;
            S.ep_step += 1; S.ep_return += reward;
            const int trunc = S.ep_step == (unsigned)A.runner.episode_step_limit;
            S.new_row[8] = 0.f; S.new_row[9] = trunc ? 1.f : 0.f;
            S.truncated = trunc; S.th = nth; S.thd = nthd;
            if (g == 0) {
                float* row = A.rb.data + (size_t)S.rb_pos * R;
                for (int j = 0; j < R; j++) row[j] = S.new_row[j];
                A.rb.episode_start[S.rb_pos] = S.rb_ces;
            }
            S.new_pos = S.rb_pos;
            S.rb_pos = (S.rb_pos + 1) % (unsigned)A.rb.capacity;
            if (trunc) S.rb_ces = S.rb_pos;
            if (S.rb_pos == 0 && !S.rb_full) S.rb_full = 1;
        }
        __syncthreads();
        // ================= S1: gather + critic phase =================
        {
            const unsigned eligible = S.rb_full ? (unsigned)A.rb.capacity : S.rb_pos;
            if (tid < ROWS * 16) {
                const int s = tid >> 4, j = tid & 15;
                const int sample = g * ROWS + s;
                const unsigned off = A.sample_offsets ? A.sample_offsets[(size_t)step * B + sample]
                                                      : (unsigned)(((uint64_t)mix32(A.seed ^ ((gstep * (uint64_t)B + sample) * 8 + 4)) * eligible) >> 32);
                unsigned index = S.rb_full ? (S.rb_pos + (unsigned)A.runner.episode_step_limit + off) % (unsigned)A.rb.capacity : off;
                if (index >= (unsigned)A.rb.capacity) index = 0;     // cannot happen for valid offsets; keeps the access in bounds
                if (j < R) {
                    // the transition added in S0 may not have reached memory from workgroup 0 yet: every workgroup holds its own copy
                    const float v = (index == S.new_pos) ? S.new_row[j] : A.rb.data[(size_t)index * R + j];
                    if (j < D) { S.grp[0].x[s * XS + j] = v; S.grp[1].x[s * XS + j] = v; if (A.out_oab) A.out_oab[(size_t)sample * D + j] = v; }
                    else if (j == D) { S.reward[s] = v; if (A.out_rewards) A.out_rewards[sample] = v; }
                    else if (j < D + 1 + OBS) { S.nx[s * XS + (j - D - 1)] = v; if (A.out_oab) A.out_oab[((size_t)B + sample) * D + (j - D - 1)] = v; }
                    else if (j == D + 1 + OBS) { S.notdone[s] = v != 0.f ? 0.f : 1.f; if (A.out_terminated) A.out_terminated[sample] = v != 0.f; }
                }
                if (j < ACT) {
                    S.noise[s * 4 + j] = A.noise_critic ? A.noise_critic[((size_t)step * B + sample) * ACT + j] : randn_at(A.seed, 5, (gstep * (uint64_t)B + sample) * ACT + j);
                    if (A.out_oab) A.out_oab[((size_t)B + sample) * D + OBS + j] = 0.f;
                }
            }
            __syncthreads();
            // A: group 0 evaluates the actor on the next observations (activations in the dp buffers, free until the backward pass);
            //    group 1 meanwhile runs critic 1's training forward on the current (obs, action)
            {
                const NetBufs actor_next = make_bufs(S.nx, L.dp1, L.dp2, L.out, nullptr, nullptr, nullptr, nullptr, L.part);
                const NetBufs train = make_bufs(L.x, L.h1, L.h2, L.out, L.dp1, L.dp2, L.dout, L.din, L.part);
                net_forward(true, grp == 0 ? actor_next : train, grp == 0 ? A.actor_p : A.critic_p[1], grp == 0 ? NA : NC, w, lane);
            }
            if (grp == 0 && tid < ROWS) {   // sample_and_squash evaluate with the external noise -> next action, its log-probability
                float lp = 0.f;
                for (int a = 0; a < ACT; a++) {
                    const float mean = L.out[tid * XS + a];
                    const float ls = clampf(L.out[tid * XS + ACT + a], A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
                    const float sd = expf(ls), eps = S.noise[tid * 4 + a];
                    const float sample = mean + eps * sd, act = tanhf(sample);
                    const float z = (sample - mean) / sd;
                    lp += (-0.9189385332046727f - ls - 0.5f * z * z) - logf(1.0f - act * act + A.sas.log_probability_epsilon);
                    S.nx[tid * XS + OBS + a] = act;
                }
                S.next_logp[tid] = lp;
            }
            if (grp == 1 && w == 0 && lane < ROWS) S.q[1][lane] = L.out[lane * XS];
            __syncthreads();
            // B: target critic k on [next_obs | next_action] by group k
            {
                const NetBufs tgt = make_bufs(S.nx, L.dp1, L.dp2, L.out, nullptr, nullptr, nullptr, nullptr, L.part);
                net_forward(true, tgt, A.target_p[grp], NC, w, lane);
            }
            if (w == 0 && lane < ROWS) S.nq[grp][lane] = L.out[lane * XS];
            __syncthreads();
            // C: TD target (sac/operations_generic.h:133-179)
            if (tid < ROWS) {
                const float alpha = expf(A.log_alpha[0]);
                const float min_q = fminf(S.nq[0][tid], S.nq[1][tid]) - alpha * S.next_logp[tid];
                S.y[tid] = S.reward[tid] + S.notdone[tid] * A.gamma * min_q;
                if (A.out_target) A.out_target[g * ROWS + tid] = S.y[tid];
            }
            // D: critic 0's training forward by group 0 (critic 1's is already there), then both backward passes
            const NetBufs train = make_bufs(L.x, L.h1, L.h2, L.out, L.dp1, L.dp2, L.dout, L.din, L.part);
            net_forward(grp == 0, train, A.critic_p[0], NC, w, lane);
            if (grp == 0 && w == 0 && lane < ROWS) S.q[0][lane] = L.out[lane * XS];
            __syncthreads();
            if (w == 0 && lane < ROWS) {
                // d_output = (Q - y) * 2/B * loss_weight, loss_weight = B*0.5 / num_final_steps = 0.5 (sac/operations_generic.h:298-312)
                const float diff = S.q[grp][lane] - S.y[lane];
                L.dout[lane * XS] = diff * (2.0f / (float)B) * (((float)B * 0.5f) / (float)B);
            }
            __syncthreads();
            net_backward(true, train, A.critic_p[grp], NC, my_partial + grp * n_c, true, false, w, lane);
            if (A.out_critic_loss && w == 0) {      // sum of squared TD errors of this workgroup's rows
                float d = lane < ROWS ? (S.q[grp][lane] - S.y[lane]) : 0.f;
                d = rlt_wave_sum(d * d);
                if (lane == 0) my_partial[2 * n_c + n_a + 1 + grp] = d;
            }
        }
        grid_barrier(A.barrier_counter, (unsigned)G * (++barrier_index));
        // ================= S2: reduce + Adam + polyak for both critics =================
        {
            const int total = 2 * n_c, chunk = (total + G - 1) / G;
            const int begin = g * chunk, end = min(total, begin + chunk);
            for (int idx = begin + tid; idx < end; idx += THREADS) {
                const int k = idx >= n_c ? 1 : 0, o = idx - k * n_c;
                float gsum = 0.f;
                for (int ww = 0; ww < G; ww++) gsum += A.partial[(size_t)ww * n_partial + idx];
                const uint32_t age = (k ? age_c10 : age_c00) + (uint32_t)step;
                const float bc1 = 1.0f / (1.0f - powf(A.adam_critic.beta_1, (float)age)), bc2 = 1.0f / (1.0f - powf(A.adam_critic.beta_2, (float)age));
                float m = A.critic_m[k][o], v = A.critic_v[k][o];
                const float pnew = adam_element(A.adam_critic, bc1, bc2, gsum, m, v, A.critic_p[k][o]);
                A.critic_g[k][o] = gsum; A.critic_m[k][o] = m; A.critic_v[k][o] = v; A.critic_p[k][o] = pnew;
                A.target_p[k][o] = A.polyak * A.target_p[k][o] + (1.0f - A.polyak) * pnew;
            }
            if (g == 0 && A.out_critic_loss && tid < 2) {
                float s = 0.f;
                for (int ww = 0; ww < G; ww++) s += A.partial[(size_t)ww * n_partial + 2 * n_c + n_a + 1 + tid];
                A.out_critic_loss[(size_t)step * 2 + tid] = s * 0.5f / (float)B;
            }
        }
        grid_barrier(A.barrier_counter, (unsigned)G * (++barrier_index));
        // ================= S3: actor phase =================
        {
            if (tid < ROWS * 4) {
                const int s = tid >> 2, j = tid & 3;
                if (j < ACT) S.noise[s * 4 + j] = A.noise_actor ? A.noise_actor[((size_t)step * B + g * ROWS + s) * ACT + j] : randn_at(A.seed, 6, (gstep * (uint64_t)B + g * ROWS + s) * ACT + j);
            }
            __syncthreads();
            // actor forward on the current observations by group 0 (its x rows are [obs | action]; the actor reads the first OBS columns)
            GroupLds& L0 = S.grp[0];
            const NetBufs actor = make_bufs(L0.x, L0.h1, L0.h2, L0.out, L0.dp1, L0.dp2, L0.dout, L0.din, L0.part);
            net_forward(grp == 0, actor, A.actor_p, NA, w, lane);
            if (grp == 0 && tid < ROWS) {   // sample_and_squash forward: keeps the pre-squashing sample, the action and the log-probability
                float lp = 0.f;
                for (int a = 0; a < ACT; a++) {
                    const float mean = L0.out[tid * XS + a];
                    const float ls = clampf(L0.out[tid * XS + ACT + a], A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
                    const float sd = expf(ls), eps = S.noise[tid * 4 + a];
                    const float sample = mean + eps * sd, act = tanhf(sample);
                    const float z = (sample - mean) / sd;
                    lp += (-0.9189385332046727f - ls - 0.5f * z * z) - logf(1.0f - act * act + A.sas.log_probability_epsilon);
                    S.act_pre[tid * 4 + a] = sample; S.act_a[tid * 4 + a] = act;
                    S.nx[tid * XS + OBS + a] = act;
                }
                S.logp[tid] = lp;
                for (int j = 0; j < OBS; j++) S.nx[tid * XS + j] = L0.x[tid * XS + j];
            }
            __syncthreads();
            // critic k forward + backward_input on [obs | new action] by group k; activations live in the dp buffers so that group 0
            // keeps the actor's h1/h2 for the actor backward
            {
                const NetBufs crit = make_bufs(S.nx, L.dp1, L.dp2, L.din, L.dp1, L.dp2, L.dout, L.din, L.part);
                net_forward(true, crit, A.critic_p[grp], NC, w, lane);
                if (w == 0 && lane < ROWS) { S.q[grp][lane] = L.din[lane * XS]; L.dout[lane * XS] = -1.0f / (float)B; }   // d_output = -1/num_final_steps (:437-453)
                __syncthreads();
                net_backward(true, crit, A.critic_p[grp], NC, nullptr, false, true, w, lane);
                if (w == 0 && lane < ROWS) for (int a = 0; a < ACT; a++) S.dci[grp][lane * 4 + a] = L.din[lane * XS + OBS + a];
                __syncthreads();
            }
            // min-Q routing (sac/operations_generic.h:358-393), sample_and_squash backward (nn/layers/sample_and_squash/operations_generic.h:289-398)
            if (grp == 0 && tid < ROWS) {
                const float alpha = expf(A.log_alpha[0]), alpha_b = alpha / (float)B;
                const int first = S.q[0][tid] < S.q[1][tid] ? 0 : 1;
                float entropy = 0.f;
                for (int a = 0; a < ACT; a++) {
                    const float d_out = S.dci[first][tid * 4 + a];
                    const float action = S.act_a[tid * 4 + a];
                    const float gte = d_out * (1.0f - action * action);
                    const float eps = S.noise[tid * 4 + a];
                    const float ls_raw = L0.out[tid * XS + ACT + a];
                    const float ls = clampf(ls_raw, A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
                    const float sd = expf(ls), mu = L0.out[tid * XS + a], sample = S.act_pre[tid * 4 + a];
                    const float z = (sample - mu) / sd;
                    const float d_mu = gte + alpha_b * ((z / sd) + (-z / sd) + 2.0f * action);
                    float d_ls = sd * (gte * eps) + alpha_b * ((z * z - 1.0f) + (-z / sd) * eps * sd + 2.0f * action * eps * sd);
                    if (ls_raw < A.sas.log_std_lower_bound || ls_raw > A.sas.log_std_upper_bound) d_ls = 0.f;
                    L0.dout[tid * XS + a] = d_mu; L0.dout[tid * XS + ACT + a] = d_ls;
                    const float lp = (-0.9189385332046727f - ls - 0.5f * z * z) - logf(1.0f - action * action + A.sas.log_probability_epsilon);
                    entropy -= lp;
                }
                S.red[tid] = alpha * (entropy - A.sas.target_entropy);
            }
            __syncthreads();
            if (grp == 0 && tid == 0) { float s = 0.f; for (int i = 0; i < ROWS; i++) s += S.red[i]; my_partial[2 * n_c + n_a] = s; }
            net_backward(grp == 0, actor, A.actor_p, NA, my_partial + 2 * n_c, true, false, w, lane);
        }
        grid_barrier(A.barrier_counter, (unsigned)G * (++barrier_index));
        // ================= S4: reduce + Adam for the actor and log_alpha =================
        {
            const int chunk = (n_a + G - 1) / G;
            const int begin = g * chunk, end = min(n_a, begin + chunk);
            const uint32_t age = age_actor0 + (uint32_t)step;
            const float bc1 = 1.0f / (1.0f - powf(A.adam_actor.beta_1, (float)age)), bc2 = 1.0f / (1.0f - powf(A.adam_actor.beta_2, (float)age));
            for (int o = begin + tid; o < end; o += THREADS) {
                float gsum = 0.f;
                for (int ww = 0; ww < G; ww++) gsum += A.partial[(size_t)ww * n_partial + 2 * n_c + o];
                float m = A.actor_m[o], v = A.actor_v[o];
                const float pnew = adam_element(A.adam_actor, bc1, bc2, gsum, m, v, A.actor_p[o]);
                A.actor_g[o] = gsum; A.actor_m[o] = m; A.actor_v[o] = v; A.actor_p[o] = pnew;
            }
            if (g == G - 1 && tid == 0) {   // log_alpha: gradient = mean over the batch of alpha * (entropy - target entropy)
                float gsum = 0.f;
                for (int ww = 0; ww < G; ww++) gsum += A.partial[(size_t)ww * n_partial + 2 * n_c + n_a];
                gsum /= (float)B;
                const uint32_t aage = age_alpha0 + (uint32_t)step;
                const float b1 = 1.0f / (1.0f - powf(A.adam_alpha.beta_1, (float)aage)), b2 = 1.0f / (1.0f - powf(A.adam_alpha.beta_2, (float)aage));
                float m = A.log_alpha[2], v = A.log_alpha[3];
                const float pnew = adam_element(A.adam_alpha, b1, b2, gsum, m, v, A.log_alpha[0]);
                A.log_alpha[1] = gsum; A.log_alpha[2] = m; A.log_alpha[3] = v; A.log_alpha[0] = pnew;
            }
        }
        grid_barrier(A.barrier_counter, (unsigned)G * (++barrier_index));
    }
    if (g == 0 && tid == 0) {
        A.runner.states[0] = S.th; A.runner.states[1] = S.thd; A.runner.episode_return[0] = S.ep_return;
        A.runner.episode_step[0] = S.ep_step; A.runner.truncated[0] = (uint8_t)S.truncated;
        A.rb.position[0] = S.rb_pos; A.rb.current_episode_start[0] = S.rb_ces; A.rb.full[0] = (uint8_t)S.rb_full;
        *A.actor_age = age_actor0 + (uint32_t)A.n_steps; *A.critic_age[0] = age_c00 + (uint32_t)A.n_steps;
        *A.critic_age[1] = age_c10 + (uint32_t)A.n_steps; *A.alpha_age = age_alpha0 + (uint32_t)A.n_steps;
    }
}

bool contiguous_arena(const rlt_dense_layer* L, int n, int in, int out, bool need_grad) {
    if (n != 3 || L[0].in_dim != in || L[0].out_dim != H || L[1].in_dim != H || L[1].out_dim != H || L[2].in_dim != H || L[2].out_dim != out) return false;
    if (L[0].activation != RLT_ACT_RELU || L[1].activation != RLT_ACT_RELU || L[2].activation != RLT_ACT_IDENTITY) return false;
    const float* p = L[0].weights; const float* gq = L[0].d_weights;
    for (int l = 0; l < 3; l++) {
        if (L[l].weights != p) return false; p += (size_t)L[l].in_dim * L[l].out_dim;
        if (L[l].biases != p) return false; p += L[l].out_dim;
        if (need_grad) {
            if (L[l].d_weights != gq) return false; gq += (size_t)L[l].in_dim * L[l].out_dim;
            if (L[l].d_biases != gq) return false; gq += L[l].out_dim;
        }
    }
    return true;
}
bool adam_arena(const rlt_adam_tensor* t, int n, const float* params, size_t total) {
    if (n < 1 || t[0].parameters != params) return false;
    size_t off = 0;
    for (int i = 0; i < n; i++) {
        if (t[i].parameters != params + off || t[i].first_moment != t[0].first_moment + off || t[i].second_moment != t[0].second_moment + off) return false;
        if (t[i].polyak_target) return false;
        off += t[i].count;
    }
    return off == total;
}

}  // namespace

extern "C" int rlt_rocm_sac_pendulum_loop(rlt_rocm_device* device, const rlt_sac_agent* agent, const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb,
                                          int n_steps, uint64_t seed, uint64_t step_offset, const rlt_sac_loop_inputs* inputs, const rlt_sac_loop_outputs* outputs) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent && runner && rb && n_steps > 0);
    const int OBS = agent->observation_dim, ACT = agent->action_dim, B = agent->batch;
    // what the kernel is built for; anything else has to take the per-operation entry points
    if (OBS != 3 || ACT != 1 || B % ROWS != 0 || B / ROWS > MAX_G || B / ROWS > device->compute_units) return RLT_E_UNSUPPORTED;
    if (runner->n_envs != 1 || rb->n_envs != 1 || rb->observation_dim != OBS || rb->action_dim != ACT) return RLT_E_UNSUPPORTED;
    if (agent->final_step_mask || agent->next_final_step_mask || agent->reset) return RLT_E_UNSUPPORTED;   // all-true masks only (SEQUENCE_LENGTH = 1)
    NetLayout NA{OBS, 2 * ACT}, NC{OBS + ACT, 1};
    if (!contiguous_arena(agent->actor, agent->n_actor_layers, OBS, 2 * ACT, true)) return RLT_E_UNSUPPORTED;
    if (!adam_arena(agent->actor_adam_tensors, agent->n_actor_adam_tensors, agent->actor[0].weights, (size_t)NA.total())) return RLT_E_UNSUPPORTED;
    for (int k = 0; k < 2; k++) {
        if (!contiguous_arena(agent->critics[k], agent->n_critic_layers, OBS + ACT, 1, true)) return RLT_E_UNSUPPORTED;
        if (!contiguous_arena(agent->critics_target[k], agent->n_critic_layers, OBS + ACT, 1, false)) return RLT_E_UNSUPPORTED;
        if (!adam_arena(agent->critic_adam_tensors[k], agent->n_critic_adam_tensors, agent->critics[k][0].weights, (size_t)NC.total())) return RLT_E_UNSUPPORTED;
    }
    RLT_REQUIRE(agent->log_alpha.parameters && agent->log_alpha.gradient == agent->log_alpha.parameters + 1 &&
                agent->log_alpha.first_moment == agent->log_alpha.parameters + 2 && agent->log_alpha.second_moment == agent->log_alpha.parameters + 3);
    RLT_REQUIRE(agent->actor_age && agent->critic_age[0] && agent->critic_age[1] && agent->alpha_age);
    RLT_REQUIRE(runner->states && runner->episode_step && runner->episode_return && runner->truncated && rb->data && rb->episode_start && rb->position &&
                rb->current_episode_start && rb->full && rb->capacity > 0);
    const int G = B / ROWS;
    const size_t n_partial = (size_t)2 * NC.total() + NA.total() + 8;
    void* scratch = nullptr;
    int rc = rlt_scratch(device, (size_t)G * n_partial * sizeof(float) + 256, &scratch);
    if (rc) return rc;
    FusedArgs a = {};
    a.actor_p = agent->actor[0].weights; a.actor_g = agent->actor[0].d_weights;
    a.actor_m = agent->actor_adam_tensors[0].first_moment; a.actor_v = agent->actor_adam_tensors[0].second_moment;
    for (int k = 0; k < 2; k++) {
        a.critic_p[k] = agent->critics[k][0].weights; a.critic_g[k] = agent->critics[k][0].d_weights;
        a.critic_m[k] = agent->critic_adam_tensors[k][0].first_moment; a.critic_v[k] = agent->critic_adam_tensors[k][0].second_moment;
        a.target_p[k] = agent->critics_target[k][0].weights; a.critic_age[k] = agent->critic_age[k];
    }
    a.log_alpha = agent->log_alpha.parameters;
    a.actor_age = agent->actor_age; a.alpha_age = agent->alpha_age;
    a.adam_actor = agent->actor_adam; a.adam_critic = agent->critic_adam; a.adam_alpha = agent->alpha_adam;
    a.sas = agent->sas; a.gamma = agent->gamma; a.polyak = agent->polyak;
    a.obs = OBS; a.act = ACT; a.batch = B; a.n_steps = n_steps;
    a.runner = *runner; a.rb = *rb;
    a.barrier_counter = (unsigned*)scratch; a.partial = (float*)((char*)scratch + 256);
    if (inputs) { a.rollout_noise = inputs->rollout_noise; a.initial_states = inputs->initial_states; a.sample_offsets = inputs->sample_offsets;
                  a.noise_critic = inputs->noise_critic; a.noise_actor = inputs->noise_actor; }
    a.seed = seed; a.step_offset = step_offset;
    if (outputs) { a.out_critic_loss = outputs->critic_loss; a.out_oab = outputs->observations_actions_base; a.out_rewards = outputs->rewards;
                   a.out_terminated = outputs->terminated; a.out_target = outputs->target_action_value; }
    RLT_HIP(hipMemsetAsync(scratch, 0, 256, device->stream));
    hipLaunchKernelGGL(sac_pendulum_loop_kernel, dim3(G), dim3(THREADS), 0, device->stream, a);
    return rlt_launch_status(device);
}
