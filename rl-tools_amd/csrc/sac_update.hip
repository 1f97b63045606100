// One launch for the network passes of a SAC critic update, one for those of an actor update, for actors obs -> 64 -> 64 -> 2 act and
// critics obs + act -> 64 -> 64 -> 1 of any observation / action width up to 128 inputs and 8 actions; and the same for TD3 (actors
// obs -> 64 -> 64 -> act with a tanh output and the td3_sampling layer; rl/algorithms/td3/operations_generic.h:170-281), whose updates have
// the same stages with another head, no entropy terms, and the policy gradient through critic 0 only.
// reference: rl/algorithms/sac/operations_generic.h:243-337 (train_critic), :395-468 (train_actor),
//            nn/layers/sample_and_squash/operations_generic.h:148-398, nn_models/mlp/operations_generic.h:128-260.
//
// A workgroup of two teams of four wavefronts takes 16 rows of the batch through every pass of the update:
//   critic update   stage A: actor on the next observations (team 0) | trained critic on the current rows (team 1)
//                   -> squashed sample and its log-probability -> stage B: target critic 0 (team 0) | target critic 1 (team 1)
//                   -> TD target, MSE gradient -> stage C: critic backward (team 1)
//   actor update    stage A: actor forward (team 1) -> squashed sample -> stage B: critic 0 | critic 1 forward and input gradient with
//                   d_output = -1 / batch -> gradient of the smaller value per row -> sample_and_squash backward (entropy term,
//                   log_alpha gradient) -> stage C: actor backward (team 1)
// The update is a chain of small dependent matrix products, so its duration is the length of that chain: independent networks run side
// by side, and the four wavefronts of a team share every link of one network. Wavefront w of a team owns hidden units 16 w .. 16 w + 15:
// in a hidden layer it computes that tile of the 16 x 64 activations from the whole previous layer (which the others read after a
// workgroup barrier), in the output layer it contributes the quarter of the reduction that its units feed (the four partial tiles are
// added in a fixed order), in the backward pass it owns the same units' pre-activation gradients and the rows of dW1, dW2 and columns of
// dW3 that belong to them. The per-row arithmetic between the network passes (sample_and_squash, TD target, loss gradients) is one
// wavefront's work.
// Parameters go from global memory straight into the registers that feed v_mfma_f32_16x16x4_f32 as B operands (each wavefront needs
// only its own units' rows and columns), all requested at the start of the kernel; activations stay in LDS in the instruction's
// operand layouts (lane l = r + 16 kk feeds A[r][kk] and B[kk][r], receives D[4 kk + v][r]). A workgroup writes one block of partial
// sums of the trained network's gradients; the optimiser's launch adds the blocks up in workgroup order (in the order of the small-MLP
// path's reduction kernel, which runs as a launch of its own where the Adam tensors are not the network's gradient buffers), stores the
// sums as the gradients (OVERWRITING them: what zero_gradient followed by backward leaves) and steps.
// Bound: latency (a batch of 256 is sixteen workgroups); the point of this path is two launches per update instead of about twenty.
#include "sac_update.h"
#include "mlp_small.h"
#include "optim.h"
#include "rng.h"
#include "sac_heads.h"

namespace {
typedef float floatx4 __attribute__((ext_vector_type(4)));
constexpr int H = 64, HS = H + 1, TEAM_WAVES = 4, WAVES = 2 * TEAM_WAVES, ROWS = 16, THREADS = 64 * WAVES, MAX_D = 128, MAX_ACT = 8, MAX_OUT = 16, D3S = MAX_OUT + 1, N_EXTRA = 16,
              MISC = 64;
static_assert(H == 16 * TEAM_WAVES, "one 16-unit tile of the hidden layers per wavefront of a team");
enum { MODE_CRITIC = 0, MODE_ACTOR = 1, MODE_TD3_CRITIC = 2, MODE_TD3_ACTOR = 3 };     // SAC's two updates, TD3's two updates

struct Net { const float *W1, *b1, *W2, *b2, *W3, *b3; int in, out, act_h; };      // the output layer has no activation
struct UpdateArgs {
    Net actor, critic[2], target[2];       // critic update: critic[0] is the critic that is trained
    const float* batch_base;               // [2][batch][obs + act]: current rows, then next rows
    const float* rewards; const uint8_t* terminated;
    const float* noise;                    // [batch][act]
    const float* log_alpha;
    rlt_sas_parameters sas;
    float gamma;
    int batch, obs, act;
    float* partial; int count;             // per workgroup: dW1 [64 x in], db1 [64], dW2 [64 x 64], db2 [64], dW3 [out x 64], db3 [out], extra [16]
    // optional outputs (the reference's training buffers)
    float* out_log_probabilities;          // critic update: next_log_probabilities; actor update: actor_log_probabilities
    float* out_target_action_value;        // critic update
    float* out_actions; float* out_pre_squashing;      // actor update, [batch][act]
    // TD3 (rl/algorithms/td3/operations_generic.h:170-281): `actor` is the target actor in the critic update; its output passes tanh and the
    // td3_sampling layer (action = clamp(tanh(output) + sampling_std * noise, -1, 1), nn/layers/td3_sampling/operations_generic.h:75-128)
    float sampling_std; int ignore_termination;
    const float* target_noise;             // critic update: [batch][act], already clamped (target_action_noise), added to the next action before a second clamp
    float* out_pre_clip;                   // actor update: [batch][act], the sampling layer's value before the clamp
    // noise == NULL: element i of the noise is element i of the standard-normal stream (noise_seed, noise_stream), what
    // rlt_rocm_randn_f32 would have put there; out_noise (optional) receives the values
    uint64_t noise_seed, noise_stream; float* out_noise; const uint64_t* stream_offset;      // *stream_offset is added to noise_stream
    // TD3's critic update for both critics (blockIdx.y): the second critic's sampling noise (noise_second, or its stream where the draws are made here), and the
    // smoothing noise clamp(N(0, 1) * target_noise_std, -clip, clip) drawn here where target_noise is NULL and stored to out_target_noise
    const float* noise_second; uint64_t noise_stream_second, target_noise_stream; float target_noise_std, target_noise_clip; float* out_target_noise;
    // every 8th workgroup of an 8 x larger grid works, so that all of them run on one XCD and share its L2 (the device hands out
    // workgroups round robin over the XCDs)
    int packed;
    // the optimiser's step at the end of the launch (optim.h); critic updates: blockIdx.y selects the trained critic (critic[y], tail.opt[y])
    rlt_tail_args tail;
};

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
using namespace rlt_sac;

// hidden activation: a compile-time constant where the kernel is instantiated for it (ACT_H >= 0), else the network's run-time value
template <int ACT_H> __device__ __forceinline__ float act_hidden(float x, int f) { return rlt_act(x, ACT_H >= 0 ? ACT_H : f); }
template <int ACT_H> __device__ __forceinline__ float dact_hidden(float o, int f) { return rlt_dact_from_output(o, ACT_H >= 0 ? ACT_H : f); }

constexpr int YP = ROWS * D3S;      // one partial tile of an output layer
constexpr size_t lds_floats(int nt1c) {
    const int sx = 16 * nt1c + 1;
    // two input tiles, the trained network's h1 and h2, two scratch activations per team, d_pre3 of the trained network and of each
    // team's critic, the output layers' partial tiles of two stages x two teams x four wavefronts, per-row scalars, a tile per
    // wavefront to turn its parameters through
    return (size_t)ROWS * (2 * sx + 6 * HS + 3 * D3S) + (size_t)4 * TEAM_WAVES * YP + MISC + (size_t)WAVES * 16 * (sx > HS ? sx : HS);
}

// A wavefront's share of a network in the registers that feed the matrix cores: the rows of W1 and W2 of its 16 hidden units, and the
// columns of W3 that those units feed. Lane (r, kk) holds the B operand of every step of the reduction: k = 4 s + kk at step s.
// The rows are stored [unit][input], so a lane's operands lie a row apart: they are requested as whole rows (one coalesced request per
// row: 64 lanes, 64 consecutive floats -- requests with a lane per cache line each keep the address unit of the compute unit busy for
// thousands of cycles) and turned through a tile of LDS that belongs to the wavefront.
template <int NT1C> struct ForwardRegs { float w1[4 * NT1C], w2[16], w3[4], b1, b2; };
template <int NT1C> struct RowRegs { float w2[16], w1[16][(NT1C + 3) / 4]; };
template <int NT1C>
__device__ __forceinline__ void request_forward(const Net& N, RowRegs<NT1C>& Q, ForwardRegs<NT1C>& F, int tile, int lane) {
    const int IN = N.in, r = lane & 15, kk = lane >> 4, unit = 16 * tile + r;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        Q.w2[i] = N.W2[(16 * tile + i) * H + lane];
        const float* w1 = N.W1 + (size_t)(16 * tile + i) * IN;
#pragma unroll
        for (int c = 0; c < (NT1C + 3) / 4; c++) { const float v = w1[min(lane + 64 * c, IN - 1)]; Q.w1[i][c] = lane + 64 * c < IN ? v : 0.f; }
    }
    const float* w3 = N.W3 + min(r, N.out - 1) * H + 16 * tile + kk;
#pragma unroll
    for (int q = 0; q < 4; q++) { const float v = w3[4 * q]; F.w3[q] = r < N.out ? v : 0.f; }
    F.b1 = N.b1[unit]; F.b2 = N.b2[unit];
}
template <int SX, int NT1C>
__device__ __forceinline__ void turn_forward(const RowRegs<NT1C>& Q, ForwardRegs<NT1C>& F, lptr stage, int lane) {
    const int r = lane & 15, kk = lane >> 4;
#pragma unroll
    for (int i = 0; i < 16; i++) stage[i * HS + lane] = Q.w2[i];
    wave_sync();
#pragma unroll
    for (int s = 0; s < 16; s++) F.w2[s] = stage[r * HS + 4 * s + kk];
    wave_sync();
#pragma unroll
    for (int i = 0; i < 16; i++)
#pragma unroll
        for (int c = 0; c < (NT1C + 3) / 4; c++)
            if (lane + 64 * c < 16 * NT1C) stage[i * SX + lane + 64 * c] = Q.w1[i][c];
    wave_sync();
#pragma unroll
    for (int j = 0; j < 4 * NT1C; j++) F.w1[j] = stage[r * SX + 4 * j + kk];
    wave_sync();
}
// the same units' columns of W2 and W3 (the transposed products of the backward pass)
struct BackwardRegs { float w2t[16], w3t[4]; };
__device__ __forceinline__ void fetch_backward(const Net& N, BackwardRegs& G, int tile, int r, int kk) {
    const float* w2 = N.W2 + 16 * kk * H + 16 * tile + r;
#pragma unroll
    for (int s = 0; s < 16; s++) G.w2t[s] = w2[s * H];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) { const int o = 4 * ks + kk; const float v = N.W3[min(o, N.out - 1) * H + 16 * tile + r]; G.w3t[ks] = o < N.out ? v : 0.f; }
}

// The three layers on the workgroup's rows by the four wavefronts of a team: this wavefront's tile of h1 and of h2 (after the
// activation) into LDS, then its quarter of the last layer's reduction into yp[tile]. Three workgroup barriers, which every wavefront
// of the workgroup meets, working (on) or not; after the last one output_tile() returns the last layer's sums.
template <int SX, int NT1C, int ACT_H>
__device__ __forceinline__ void forward_wg(bool on, const ForwardRegs<NT1C>& F, int act_h, int NT1, lptr xs, lptr h1s, lptr h2s, lptr yp, int tile, int r, int kk) {
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const int col = 16 * tile + r;
    if (on) {
        floatx4 a0 = zero4, a1 = zero4;
#pragma unroll
        for (int g = 0; g < NT1C; g++)
            if (g < NT1) {
#pragma unroll
                for (int q = 0; q < 4; q += 2) {
                    a0 = mfma16(xs[r * SX + 16 * g + 4 * q + kk], F.w1[4 * g + q], a0);
                    a1 = mfma16(xs[r * SX + 16 * g + 4 * q + 4 + kk], F.w1[4 * g + q + 1], a1);
                }
            }
        const floatx4 acc = a0 + a1;
#pragma unroll
        for (int v = 0; v < 4; v++) h1s[(4 * kk + v) * HS + col] = act_hidden<ACT_H>(acc[v] + F.b1, act_h);
    }
    rlt_lds_barrier();
    if (on) {
        floatx4 a0 = zero4, a1 = zero4;
#pragma unroll
        for (int s = 0; s < 16; s += 2) {
            a0 = mfma16(h1s[r * HS + 4 * s + kk], F.w2[s], a0);
            a1 = mfma16(h1s[r * HS + 4 * s + 4 + kk], F.w2[s + 1], a1);
        }
        const floatx4 acc = a0 + a1;
#pragma unroll
        for (int v = 0; v < 4; v++) h2s[(4 * kk + v) * HS + col] = act_hidden<ACT_H>(acc[v] + F.b2, act_h);
    }
    rlt_lds_barrier();
    if (on) {
        floatx4 a0 = zero4, a1 = zero4;
#pragma unroll
        for (int q = 0; q < 4; q += 2) {
            a0 = mfma16(h2s[r * HS + 16 * tile + 4 * q + kk], F.w3[q], a0);
            a1 = mfma16(h2s[r * HS + 16 * tile + 4 * q + 4 + kk], F.w3[q + 1], a1);
        }
        const floatx4 y = a0 + a1;
#pragma unroll
        for (int v = 0; v < 4; v++) yp[(tile * ROWS + 4 * kk + v) * D3S + r] = y[v];
    }
    rlt_lds_barrier();
}
// the sums of four partial tiles, in a fixed order: element v of lane (r, kk) belongs to row 4 kk + v, column r
__device__ __forceinline__ floatx4 output_tile(lptr yp, int r, int kk) {
    floatx4 y;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const lptr p = yp + (4 * kk + v) * D3S + r;
        y[v] = (p[0] + p[YP]) + (p[2 * YP] + p[3 * YP]);
    }
    return y;
}

// this wavefront's tile of d_pre2 = (d_pre3 W3) f'(h2) into g2s (may be h2s itself); returns the lane's share of its column sum
template <int ACT_H>
__device__ __forceinline__ float backward_layer3(const BackwardRegs& G, int act_h, lptr d3s, lptr h2s, lptr g2s, int tile, int r, int kk) {
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < MAX_OUT / 4; ks++) acc = mfma16(d3s[r * D3S + 4 * ks + kk], G.w3t[ks], acc);      // columns of d_pre3 beyond the output width are zero
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int idx = (4 * kk + v) * HS + 16 * tile + r;
        const float dp = acc[v] * dact_hidden<ACT_H>(h2s[idx], act_h);
        g2s[idx] = dp; sum += dp;
    }
    return sum;
}
// this wavefront's tile of d_pre1 = (d_pre2 W2) f'(h1) into p1s (may be h1s itself); returns the lane's share of its column sum
template <int ACT_H>
__device__ __forceinline__ float backward_layer2(const BackwardRegs& G, int act_h, lptr g2s, lptr h1s, lptr p1s, int tile, int r, int kk) {
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    floatx4 a0 = zero4, a1 = zero4;
#pragma unroll
    for (int s = 0; s < 16; s += 2) {
        a0 = mfma16(g2s[r * HS + 16 * kk + s], G.w2t[s], a0);
        a1 = mfma16(g2s[r * HS + 16 * kk + s + 1], G.w2t[s + 1], a1);
    }
    const floatx4 acc = a0 + a1;
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int idx = (4 * kk + v) * HS + 16 * tile + r;
        const float dp = acc[v] * dact_hidden<ACT_H>(h1s[idx], act_h);
        p1s[idx] = dp; sum += dp;
    }
    return sum;
}

template <int NT1C, int MODE, int ACT_H>
__global__ __launch_bounds__(THREADS) void sac_update_kernel(UpdateArgs A) {
    constexpr bool CRITIC = MODE == 0 || MODE == MODE_TD3_CRITIC, TD3 = MODE == MODE_TD3_CRITIC || MODE == MODE_TD3_ACTOR;
    extern __shared__ float lds_raw[];
    constexpr int SX = 16 * NT1C + 1;
    const int lane = threadIdx.x & 63, r = lane & 15, kk = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), team = wave >> 2, tile = wave & 3;
    const bool scalar_wave = wave == 0;        // the wavefront that does the per-row arithmetic between the network passes
    const bool trainer = team == 1;            // the team that owns the trained network
    const int OBS = A.obs, ACT = A.act, D = OBS + ACT, B = A.batch;
    const lptr xsa = (lptr)lds_raw, xsb = xsa + ROWS * SX, h1s = xsb + ROWS * SX, h2s = h1s + ROWS * HS, tas = h2s + ROWS * HS + team * 2 * ROWS * HS, tbs = tas + ROWS * HS,
               d3s = h2s + 5 * ROWS * HS, d3c = d3s + (1 + team) * ROWS * D3S, yps = d3s + 3 * ROWS * D3S, misc = yps + 4 * TEAM_WAVES * YP,
               stage = misc + MISC + wave * 16 * (SX > HS ? SX : HS);
    const lptr ypa = yps + team * TEAM_WAVES * YP, ypb = yps + (2 + team) * TEAM_WAVES * YP;      // stage A / stage B partial tiles of this team
    if (A.packed && (blockIdx.x & 7)) return;
    const int g = A.packed ? blockIdx.x >> 3 : blockIdx.x, G = A.packed ? gridDim.x >> 3 : gridDim.x;
    const int y = CRITIC ? blockIdx.y : 0;
    const int row0 = g * ROWS;
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    float s3 = 0.f, extra = 0.f;
    const Net trained = CRITIC ? (y ? A.critic[1] : A.critic[0]) : A.actor;      // by value: an index into the kernel's argument would keep all of it in private memory
    const int NT1_D = (D + 15) >> 4, NT1_OBS = (OBS + 15) >> 4;

    // the input tiles (32 threads share a row), then every parameter this wavefront multiplies with in the forward passes, are requested
    // now; the backward pass's after the first forward pass has used its own
    constexpr int XN = (NT1C + 1) / 2;
    float xa[XN], xb[XN];
    {
        const int row = threadIdx.x >> 5, c0 = threadIdx.x & 31;
        const bool rok = row0 + row < B;
        const float* cur = A.batch_base + (size_t)min(row0 + row, B - 1) * D;
        const float* nxt = cur + (size_t)B * D;
#pragma unroll
        for (int j = 0; j < XN; j++) {
            const int c = c0 + 32 * j;
            if (CRITIC) {
                xa[j] = (rok && c < D) ? nxt[min(c, D - 1)] : 0.f;
                xb[j] = (rok && c < D) ? cur[min(c, D - 1)] : 0.f;
            } else {
                xa[j] = (rok && c < OBS) ? cur[min(c, D - 1)] : 0.f;
                xb[j] = 0.f;
            }
        }
    }
    ForwardRegs<NT1C> FA, FB;
    RowRegs<NT1C> QA, QB;
    BackwardRegs GT, GC;
    float wa[4] = {0.f, 0.f, 0.f, 0.f};
    const bool stage_a_on = CRITIC || trainer;
    if (stage_a_on) request_forward<NT1C>(CRITIC && !trainer ? A.actor : trained, QA, FA, tile, lane);
    request_forward<NT1C>(CRITIC ? A.target[team] : A.critic[team], QB, FB, tile, lane);
    {
        const int row = threadIdx.x >> 5, c0 = threadIdx.x & 31;
#pragma unroll
        for (int j = 0; j < XN; j++) {
            const int c = c0 + 32 * j;
            if (c < 16 * NT1C) {
                xsa[row * SX + c] = xa[j];
                if (CRITIC) xsb[row * SX + c] = xb[j];
            }
        }
    }
    float noise[2] = {0.f, 0.f}, target_noise[2] = {0.f, 0.f}, reward[4] = {0.f, 0.f, 0.f, 0.f}, alpha = 0.f, b3_actor = 0.f, b3_q[3] = {0.f, 0.f, 0.f};
    bool terminated[4] = {false, false, false, false};
    if (scalar_wave) {
        if (!TD3) alpha = expf(*A.log_alpha);
        if (MODE == MODE_TD3_CRITIC) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                if (kk + 4 * j < ACT && row0 + r < B) {
                    const size_t i = (size_t)(row0 + r) * ACT + kk + 4 * j;
                    if (A.target_noise) target_noise[j] = A.target_noise[i];
                    else {
                        const float scaled = rlt_randn_element(A.noise_seed, A.target_noise_stream + *A.stream_offset, i) * A.target_noise_std + 0.0f;
                        target_noise[j] = clampf(scaled, -A.target_noise_clip, A.target_noise_clip);
                        if (y == 0) A.out_target_noise[i] = target_noise[j];
                    }
                }
            }
        }
        b3_actor = r < A.actor.out ? A.actor.b3[min(r, A.actor.out - 1)] : 0.f;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if (kk + 4 * j < ACT && row0 + r < B) {
                const size_t i = (size_t)(row0 + r) * ACT + kk + 4 * j;
                const bool second = MODE == MODE_TD3_CRITIC && y;      // TD3's critics each take their own sampling noise
                const float* const given = second ? A.noise_second : A.noise;
                noise[j] = given ? given[i] : rlt_randn_element(A.noise_seed, (second ? A.noise_stream_second : A.noise_stream) + *A.stream_offset, i);
                if (A.out_noise && y == 0) A.out_noise[i] = noise[j];
            }
        }
        if (CRITIC) {
#pragma unroll
            for (int v = 0; v < 4; v++) { const int row = min(row0 + 4 * kk + v, B - 1); reward[v] = A.rewards[row]; terminated[v] = A.terminated[row] != 0; }
            b3_q[0] = A.target[0].b3[0]; b3_q[1] = A.target[1].b3[0]; b3_q[2] = trained.b3[0];
        }
    }
    HeadItem item[2];
    const bool row_ok = row0 + r < B;
    if (stage_a_on) turn_forward<SX, NT1C>(QA, FA, stage, lane);
    rlt_lds_barrier();      // the input tiles are in place

    // stage A: the actor (critic update: on the next observations, by team 0, while team 1 takes the trained critic through the current
    // rows; actor update: on the observations, by the team that will train it), then its squashed sample into the action columns
    if (CRITIC) forward_wg<SX, NT1C, ACT_H>(true, FA, trainer ? trained.act_h : A.actor.act_h, trainer ? NT1_D : NT1_OBS, trainer ? xsb : xsa, trainer ? h1s : tas, trainer ? h2s : tbs, ypa, tile, r, kk);
    else forward_wg<SX, NT1C, ACT_H>(trainer, FA, A.actor.act_h, NT1_OBS, xsa, h1s, h2s, ypa, tile, r, kk);
    turn_forward<SX, NT1C>(QB, FB, stage, lane);
    if (trainer) fetch_backward(trained, GT, tile, r, kk);
    if (!CRITIC) {
        fetch_backward(A.critic[team], GC, tile, r, kk);
        // the action columns of this wavefront's rows of W1: B operand of d_pre1 W1
#pragma unroll
        for (int q = 0; q < 4; q++) { const float v = A.critic[team].W1[(size_t)(16 * tile + 4 * q + kk) * D + OBS + min(r, ACT - 1)]; wa[q] = r < ACT ? v : 0.f; }
    }
    if (scalar_wave) {
        const floatx4 y = output_tile(CRITIC ? yps : yps + TEAM_WAVES * YP, r, kk);
#pragma unroll
        for (int v = 0; v < 4; v++) d3s[(4 * kk + v) * D3S + r] = r < A.actor.out ? y[v] + b3_actor : 0.f;
        wave_sync();
        float log_prob = 0.f;
        if (TD3) td3_head_forward(A.obs, A.act, A.sampling_std, d3s, D3S, xsa, SX, noise, target_noise, CRITIC, r, kk, item);
        else log_prob = head_forward(A.sas, A.obs, A.act, d3s, D3S, xsa, SX, noise, r, kk, item);
        if (TD3) {
            if (!CRITIC && row_ok && A.out_pre_clip) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    if (kk + 4 * j < ACT) A.out_pre_clip[(size_t)(row0 + r) * ACT + kk + 4 * j] = item[j].sample;
            }
        } else if (CRITIC) {
            if (kk == 0) {
                misc[r] = log_prob;
                if (A.out_log_probabilities && row_ok) A.out_log_probabilities[row0 + r] = log_prob;
            }
        } else if (row_ok) {
            if (kk == 0 && A.out_log_probabilities) A.out_log_probabilities[row0 + r] = log_prob;
#pragma unroll
            for (int j = 0; j < 2; j++)
                if (kk + 4 * j < ACT) {
                    if (A.out_actions) A.out_actions[(size_t)(row0 + r) * ACT + kk + 4 * j] = item[j].action;
                    if (A.out_pre_squashing) A.out_pre_squashing[(size_t)(row0 + r) * ACT + kk + 4 * j] = item[j].sample;
                }
        }
    }
    rlt_lds_barrier();      // the action columns are in place

    // stage B: each team takes one of the two (target) critics through [observation | sampled action]
    forward_wg<SX, NT1C, ACT_H>(true, FB, CRITIC ? A.target[team].act_h : A.critic[team].act_h, NT1_D, xsa, tas, tbs, ypb, tile, r, kk);
    if (CRITIC) {
        if (scalar_wave) {
            // TD target of rows 4 kk + v (meaningful in the lanes r == 0, which hold output 0), MSE gradient at the critic's pre-activation
            const floatx4 y0 = output_tile(yps + 2 * TEAM_WAVES * YP, r, kk), y1 = output_tile(yps + 3 * TEAM_WAVES * YP, r, kk), yc = output_tile(yps + TEAM_WAVES * YP, r, kk);
            // loss weight batch * 0.5 / n with n = batch rows (no masks), times the MSE gradient's 2 / batch (rl/algorithms/sac/operations_generic.h:298-316)
            // (TD3: loss weight batch / n, rl/algorithms/td3/operations_generic.h:200-212)
            const float loss_weight = TD3 ? (float)B / (float)B : (1.0f / (float)B) * ((float)B * 0.5f);
            const float constant = 2.0f / (float)B * loss_weight;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float q_min = fminf(y0[v] + b3_q[0], y1[v] + b3_q[1]);
                const float min_q = TD3 ? q_min : q_min - alpha * misc[4 * kk + v];
                const float future = (terminated[v] && !(TD3 && A.ignore_termination)) ? 0.0f : A.gamma * min_q;
                const float y_target = reward[v] + future;
                const bool ok = r == 0 && row0 + 4 * kk + v < B;
                // (SAC's critics share their targets; TD3's are formed with each critic's own sampling noise: the last critic's stay, as after two calls)
                if (A.out_target_action_value && ok && (!TD3 || y == (int)gridDim.y - 1)) A.out_target_action_value[row0 + 4 * kk + v] = y_target;
                const float q = yc[v] + b3_q[2];
                const float diff = q - y_target;
                const float dp = ok ? diff * constant : 0.f;
                if (ok) extra += diff * diff;
                s3 += dp;
                d3s[(4 * kk + v) * D3S + r] = dp;
            }
        }
        rlt_lds_barrier();      // d_pre3 is in place
    } else {
        // value and the gradient of -value / batch with respect to the action, each team for its critic
        const float loss_weight = (1.0f / (float)B) * -1.0f;       // rl/algorithms/sac/operations_generic.h:437-453 with n = batch rows
        const Net& C = A.critic[team];
        if (tile == 0) {
            const floatx4 y = output_tile(ypb, r, kk);
            const float b3 = C.b3[0];
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float q = y[v] + b3;
                if (r == 0) misc[16 * team + 4 * kk + v] = q;
                d3c[(4 * kk + v) * D3S + r] = (r == 0 && row0 + 4 * kk + v < B) ? loss_weight : 0.f;
            }
        }
        rlt_lds_barrier();
        backward_layer3<ACT_H>(GC, C.act_h, d3c, tbs, tbs, tile, r, kk);
        rlt_lds_barrier();
        backward_layer2<ACT_H>(GC, C.act_h, tbs, tas, tas, tile, r, kk);
        wave_sync();
        {   // d value / d action = the action columns of d_pre1 W1: this wavefront's units' share of the reduction (stage A's partial tiles are free to hold it)
            floatx4 acc = zero4;
#pragma unroll
            for (int q = 0; q < 4; q++) acc = mfma16(tas[r * HS + 16 * tile + 4 * q + kk], wa[q], acc);
#pragma unroll
            for (int v = 0; v < 4; v++) ypa[(tile * ROWS + 4 * kk + v) * D3S + r] = acc[v];
        }
        rlt_lds_barrier();
        if (scalar_wave) {
            // sample_and_squash backward (nn/layers/sample_and_squash/operations_generic.h:262-398) on the gradient of the smaller value;
            // TD3: the gradient through critic 0 (both teams ran it), the td3_sampling layer's backward (zero where the sample was clamped,
            // nn/layers/td3_sampling/operations_generic.h:139-163) and the derivative of the actor's tanh output
            const bool first = TD3 || misc[r] < misc[16 + r];
            const lptr da = yps + (first ? 0 : 1) * TEAM_WAVES * YP + r * D3S;
#pragma unroll
            for (int v = 0; v < 4; v++) d3s[(4 * kk + v) * D3S + r] = 0.f;
            wave_sync();
            const float alpha_over_b = alpha / (float)B;
            float entropy = 0.f;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int a = kk + 4 * j;
                if (a < ACT) {
                    const HeadItem& I = item[j];
                    const float d_out = (da[a] + da[YP + a]) + (da[2 * YP + a] + da[3 * YP + a]);
                    if (TD3) {
                        const float d_mean = (I.sample < -1.0f || I.sample > 1.0f) ? 0.0f : d_out;
                        if (row_ok) d3s[r * D3S + a] = d_mean * (1.0f - I.mean * I.mean);
                        continue;
                    }
                    const float g = d_out * (1.0f - I.action * I.action);
                    const float log_std = clampf(I.log_std_raw, A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
                    const float sd = expf(log_std);
                    const float z = (I.sample - I.mean) / sd;
                    const float dlp_dmean = z / sd, dlp_dsample = -z / sd, dlp_dlogstd = z * z - 1.0f;
                    const float d_mu = g + alpha_over_b * (dlp_dmean + dlp_dsample + 2.0f * I.action);
                    float d_ls = sd * (g * I.noise) + alpha_over_b * (dlp_dlogstd + dlp_dsample * I.noise * sd + 2.0f * I.action * I.noise * sd);
                    if (I.log_std_raw < A.sas.log_std_lower_bound || I.log_std_raw > A.sas.log_std_upper_bound) d_ls = 0.0f;
                    if (row_ok) {
                        d3s[r * D3S + a] = d_mu;
                        d3s[r * D3S + ACT + a] = d_ls;
                    }
                    entropy -= normal_log_prob(I.mean, log_std, sd, I.sample) - logf(1.0f - I.action * I.action + A.sas.log_probability_epsilon);
                }
            }
            entropy = groups_sum(entropy);
            // d log_alpha: sum over the rows of alpha (entropy - target entropy), divided by the batch size by the reduction
            const float per_row = (kk == 0 && row_ok) ? alpha * (entropy - A.sas.target_entropy) : 0.f;
            const float tile_sum = row16_sum(per_row);
            if (lane == 0) extra += tile_sum;
            wave_sync();
#pragma unroll
            for (int v = 0; v < 4; v++) s3 += d3s[(4 * kk + v) * D3S + r];
        }
        rlt_lds_barrier();      // d_pre3 is in place
    }

    // stage C: backward pass of the trained network with its weight gradients over the workgroup's 16 rows, by its team; h1, h2: its
    // hidden activations, d3: the gradient at its last pre-activation; the team's ta receives d_pre2, tb receives d_pre1
    float* dst = A.partial + ((size_t)y * G + g) * A.count;
    const int IN = trained.in, OUT = trained.out, NT1 = (IN + 15) >> 4;
    const int o_b1 = H * IN, o_w2 = o_b1 + H, o_b2 = o_w2 + H * H, o_w3 = o_b2 + H, o_b3 = o_w3 + OUT * H, o_ex = o_b3 + OUT;
    const lptr xt = CRITIC ? xsb : xsa;
    floatx4 aW1[NT1C], aW2[4], aW3 = zero4;
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int nt = 0; nt < NT1C; nt++) aW1[nt] = zero4;
#pragma unroll
    for (int nt = 0; nt < 4; nt++) aW2[nt] = zero4;
    if (trainer) {
#pragma unroll
        for (int ks = 0; ks < ROWS / 4; ks++) aW3 = mfma16(d3s[(4 * ks + kk) * D3S + r], h2s[(4 * ks + kk) * HS + 16 * tile + r], aW3);
        s2 = backward_layer3<ACT_H>(GT, trained.act_h, d3s, h2s, tas, tile, r, kk);
    }
    rlt_lds_barrier();      // every wavefront's tile of d_pre2 is in place
    if (trainer) {
#pragma unroll
        for (int ks = 0; ks < ROWS / 4; ks++) {
            const float a = tas[(4 * ks + kk) * HS + 16 * tile + r];
#pragma unroll
            for (int nt = 0; nt < 4; nt++) aW2[nt] = mfma16(a, h1s[(4 * ks + kk) * HS + 16 * nt + r], aW2[nt]);
        }
        s1 = backward_layer2<ACT_H>(GT, trained.act_h, tas, h1s, tbs, tile, r, kk);
        wave_sync();            // dW1's rows are this wavefront's own tile of d_pre1
#pragma unroll
        for (int ks = 0; ks < ROWS / 4; ks++) {
            const float a = tbs[(4 * ks + kk) * HS + 16 * tile + r];
#pragma unroll
            for (int nt = 0; nt < NT1C; nt++)
                if (nt < NT1) aW1[nt] = mfma16(a, xt[(4 * ks + kk) * SX + 16 * nt + r], aW1[nt]);
        }
        // the workgroup's block of partial sums, straight from the registers that own them
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int m = 16 * tile + 4 * kk + v;
#pragma unroll
            for (int nt = 0; nt < NT1C; nt++)
                if (nt < NT1 && 16 * nt + r < IN) dst[m * IN + 16 * nt + r] = aW1[nt][v];
#pragma unroll
            for (int nt = 0; nt < 4; nt++) dst[o_w2 + m * H + 16 * nt + r] = aW2[nt][v];
            if (4 * kk + v < OUT) dst[o_w3 + (4 * kk + v) * H + 16 * tile + r] = aW3[v];
        }
        s1 = groups_sum(s1); s2 = groups_sum(s2);
        if (kk == 0) { dst[o_b1 + 16 * tile + r] = s1; dst[o_b2 + 16 * tile + r] = s2; }
    }
    if (scalar_wave) {
        s3 = groups_sum(s3); extra = groups_sum(extra);
        if (kk == 0) {
            if (r < OUT) dst[o_b3 + r] = s3;
            dst[o_ex + r] = extra;
        }
    }
    if (!A.tail.enabled) return;
    // the kernel's arguments as they lie in its argument segment (the struct is the only explicit argument), so that the optimiser's
    // part, a function of its own, indexes them there
    rlt_optimiser_tail<THREADS>(&((const RLT_CONSTANT UpdateArgs*)__builtin_amdgcn_kernarg_segment_ptr())->tail, y, g, G, (__attribute__((address_space(3))) int*)(misc + 48));
}

// soft update of up to 16 tensors in one launch (utils/polyak/operations_generic.h:11-27): workgroup b serves tensor b % n
constexpr int MAX_POLYAK = 16;
struct PolyakList { const float* source[MAX_POLYAK]; float* target[MAX_POLYAK]; uint32_t count[MAX_POLYAK]; int n; float polyak; };
__global__ __launch_bounds__(256) void polyak_list_kernel(PolyakList P) {
    const int t = blockIdx.x % P.n, part = blockIdx.x / P.n, parts = gridDim.x / P.n;
    const float* __restrict__ s = P.source[t]; float* __restrict__ d = P.target[t];
    for (uint32_t i = part * 256 + threadIdx.x; i < P.count[t]; i += parts * 256) d[i] = rlt_polyak_value(P.polyak, d[i], s[i]);
}

bool hidden_ok(int a) { return a == RLT_ACT_RELU || a == RLT_ACT_TANH || a == RLT_ACT_FAST_TANH || a == RLT_ACT_SIGMOID; }
bool net_ok(const rlt_dense_layer* L, int n, int in, int out, int out_activation = RLT_ACT_IDENTITY) {
    if (!L || n != 3) return false;
    for (int l = 0; l < 3; l++) if (!L[l].weights || !L[l].biases) return false;
    return L[0].in_dim == in && L[0].out_dim == H && L[1].in_dim == H && L[1].out_dim == H && L[2].in_dim == H && L[2].out_dim == out &&
           L[0].activation == L[1].activation && hidden_ok(L[0].activation) && L[2].activation == out_activation;
}
Net net_of(const rlt_dense_layer* L) {
    return {L[0].weights, L[0].biases, L[1].weights, L[1].biases, L[2].weights, L[2].biases, L[0].in_dim, L[2].out_dim, L[0].activation};
}
int tile_bucket(int d) { return d <= 32 ? 2 : MAX_D / 16; }

// Where each Adam tensor's gradient lies in a block of partial sums [dW1 | db1 | dW2 | db2 | dW3 | db3 | extra]: a tensor may span
// several of the network's six gradient buffers where those follow each other in memory. False unless the tensors cover the six
// buffers exactly, at most 12 of them: then the optimiser's launch can read the blocks itself.
bool map_gradients(const rlt_dense_layer* L, const rlt_adam_tensor* T, int n, uint32_t* offsets, int* first_segment = nullptr, int* n_segments = nullptr) {
    if (!T || n < 1 || n > 12) return false;
    const float* seg[6] = {L[0].d_weights, L[0].d_biases, L[1].d_weights, L[1].d_biases, L[2].d_weights, L[2].d_biases};
    const uint32_t size[6] = {(uint32_t)(H * L[0].in_dim), H, H * H, H, (uint32_t)(L[2].out_dim * H), (uint32_t)L[2].out_dim};
    uint32_t off[6], covered = 0;
    for (int k = 0, o = 0; k < 6; o += size[k], k++) off[k] = o;
    for (int i = 0; i < n; i++) {
        int s = 0;
        while (s < 6 && seg[s] != T[i].gradient) s++;
        if (s == 6 || T[i].polyak_target) return false;
        uint32_t cnt = 0; int k = s;
        for (; k < 6 && cnt < T[i].count && seg[k] == seg[s] + cnt; k++) {
            if (covered & (1u << k)) return false;
            covered |= 1u << k; cnt += size[k];
        }
        if (cnt != T[i].count) return false;
        offsets[i] = off[s];
        if (first_segment) first_segment[i] = s;
        if (n_segments) n_segments[i] = k - s;
    }
    return covered == 63u;
}
// where the segments [first, first + count) of a network's parameters lie, if they follow each other in memory (NULL otherwise)
float* parameter_segments(const rlt_dense_layer* L, int first, int count) {
    float* seg[6] = {L[0].weights, L[0].biases, L[1].weights, L[1].biases, L[2].weights, L[2].biases};
    const uint32_t size[6] = {(uint32_t)(H * L[0].in_dim), H, H * H, H, (uint32_t)(L[2].out_dim * H), (uint32_t)L[2].out_dim};
    uint32_t cnt = 0;
    for (int k = first; k < first + count; k++) { if (seg[k] != seg[first] + cnt) return nullptr; cnt += size[k]; }
    return seg[first];
}

// The optimiser of one trained network of the launch; `soft_target` (optional): the network that follows the trained one by the soft update
struct Optimiser {
    const rlt_dense_layer* trained; const rlt_adam_tensor* tensors; int n_tensors; const rlt_adam_parameters* parameters; uint32_t* age;
    const rlt_adam_tensor* second; const rlt_adam_parameters* second_parameters; uint32_t* second_age; float second_scale;
    const rlt_dense_layer* soft_target;
};

// The optimisers as the kernel's own last step: possible where the Adam tensors are the networks' gradient buffers (and the targets'
// parameters are laid out as the trained networks' are) and the grid is small enough to wait for itself.
bool configure_tail(rlt_rocm_device* device, UpdateArgs& a, const Optimiser* opts, int n_opts, int groups, float polyak) {
    if (!device->update_tail || n_opts < 1 || n_opts > 2 || n_opts * groups > RLT_TAIL_MAX_WORKGROUPS) return false;
    rlt_tail_args& T = a.tail;
    for (int k = 0; k < n_opts; k++) {
        const Optimiser& O = opts[k];
        uint32_t offsets[12]; int first[12], count[12];
        if (!map_gradients(O.trained, O.tensors, O.n_tensors, offsets, first, count)) return false;
        if (O.second && (O.second->polyak_target || n_opts != 1 || !O.second->parameters || !O.second->gradient || !O.second->first_moment || !O.second->second_moment)) return false;
        if (!rlt_tail_optimizer_fill(T.opt[k], O.tensors, O.n_tensors, offsets, nullptr, O.parameters, O.age)) return false;
        if (O.soft_target)
            for (int i = 0; i < O.n_tensors; i++) {
                // the tensor's parameters must be the trained network's own segments, so that the target's segments correspond element by element
                if (parameter_segments(O.trained, first[i], count[i]) != O.tensors[i].parameters) return false;
                if (!(T.opt[k].t[i].polyak_target = parameter_segments(O.soft_target, first[i], count[i]))) return false;
            }
        if (O.second) { T.has_second = 1; T.second_offset = a.count - N_EXTRA; T.second = *O.second; T.second_p = *O.second_parameters; T.second_age = O.second_age; T.second_scale = O.second_scale; }
    }
    void* counters = nullptr;
    if (rlt_counters(device, &counters)) return false;
    T.tickets = (uint32_t*)counters + RLT_TICKET_TAIL;
    T.fault = device->fault; T.max_poll = device->wait_limit;
    T.polyak = polyak;
    T.partial = a.partial; T.count = a.count; T.same_xcd = a.packed;
    T.enabled = 1;
    return true;
}

// the workgroups' blocks of partial sums -> gradients -> Adam step(s), as launches after the update kernel: one where the optimiser can
// read the blocks itself, else the reduction kernel and then the optimiser. `second` (optional): an optimiser for one scalar whose
// gradient is extra[0] * second_scale.
int reduce_and_step(rlt_rocm_device* device, const UpdateArgs& a, const float* partial, int groups, const Optimiser& O) {
    uint32_t offsets[12];
    if (map_gradients(O.trained, O.tensors, O.n_tensors, offsets) && (!O.second || !O.second->polyak_target)) {
        float scales[12];
        for (int i = 0; i < 12; i++) scales[i] = 1.0f;
        const rlt_adam_source source = {partial, groups, a.count, offsets, scales};
        if (!O.second) return rlt_adam_step_from_partials(device, O.tensors, O.n_tensors, O.parameters, O.age, &source);
        const uint32_t second_offset = (uint32_t)(a.count - N_EXTRA);
        const rlt_adam_source second_source = {partial, groups, a.count, &second_offset, &O.second_scale};
        return rlt_adam_step_pair(device, O.tensors, O.n_tensors, O.parameters, O.age, O.second, 1, O.second_parameters, O.second_age, &source, &second_source);
    }
    int rc = rlt_mlp3s_reduce(device, O.trained, partial, groups, 1, O.second ? O.second->gradient : nullptr, O.second ? 1 : 0, O.second_scale, 0.0f);
    if (rc) return rc;
    if (O.second && O.n_tensors <= 12) return rlt_adam_step_pair(device, O.tensors, O.n_tensors, O.parameters, O.age, O.second, 1, O.second_parameters, O.second_age);
    if ((rc = rlt_rocm_adam_step(device, O.tensors, O.n_tensors, O.parameters, O.age, 0.0f, nullptr))) return rc;
    return O.second ? rlt_rocm_adam_step(device, O.second, 1, O.second_parameters, O.second_age, 0.0f, nullptr) : 0;
}

// One launch for `n_opts` trained networks (2: both critics of a critic update, one per blockIdx.y) and their optimisers; where the
// optimiser cannot be the kernel's last step it follows as launches of its own.
template <int MODE>
int launch_update(rlt_rocm_device* device, UpdateArgs& a, int groups, const Optimiser* opts, int n_opts, float polyak = 0.0f) {
    const rlt_dense_layer* trained = opts[0].trained;
    const int bucket = tile_bucket(a.obs + a.act);
    const size_t lds_bytes = lds_floats(bucket) * sizeof(float);
    a.count = rlt_mlp3s_partial_count(trained[0].in_dim, trained[2].out_dim);
    void* scratch = nullptr;
    int rc = rlt_scratch(device, (size_t)n_opts * groups * a.count * sizeof(float), &scratch);
    if (rc) return rc;
    a.partial = (float*)scratch;
    a.stream_offset = device->stream_offset;
    // up to 32 workgroups (one per compute unit of an XCD) are placed on one XCD where the device hands out workgroups round robin
    a.packed = device->update_one_xcd && device->xcd_stride == 8 && n_opts * groups <= 32 ? 1 : 0;
    const bool tail = configure_tail(device, a, opts, n_opts, groups, polyak);
    if (tail) device->fault_armed = 1;
    const dim3 grid(a.packed ? 8 * groups : groups, n_opts);
#define RLT_LAUNCH_UPDATE(NT, ACT)                                                                                                                              \
    do {                                                                                                                                                        \
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(sac_update_kernel<NT, MODE, ACT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes)); \
        hipLaunchKernelGGL((sac_update_kernel<NT, MODE, ACT>), grid, dim3(THREADS), lds_bytes, device->stream, a);                                            \
    } while (0)
    // ReLU (the reference's default for SAC) and tanh are compiled in; any other hidden activation, or networks that differ in it, take
    // the variant that looks it up per network
    int act = a.actor.act_h;
    for (int k = 0; k < 2; k++) if (a.critic[k].act_h != act || a.target[k].act_h != act) act = -1;
    if (bucket == 2) {
        if (act == RLT_ACT_RELU) RLT_LAUNCH_UPDATE(2, RLT_ACT_RELU); else if (act == RLT_ACT_TANH) RLT_LAUNCH_UPDATE(2, RLT_ACT_TANH); else RLT_LAUNCH_UPDATE(2, -1);
    } else {
        if (act == RLT_ACT_RELU) RLT_LAUNCH_UPDATE(MAX_D / 16, RLT_ACT_RELU); else if (act == RLT_ACT_TANH) RLT_LAUNCH_UPDATE(MAX_D / 16, RLT_ACT_TANH); else RLT_LAUNCH_UPDATE(MAX_D / 16, -1);
    }
#undef RLT_LAUNCH_UPDATE
    if ((rc = rlt_launch_status(device))) return rc;
    if (tail) return 0;
    for (int k = 0; k < n_opts; k++)
        if ((rc = reduce_and_step(device, a, a.partial + (size_t)k * groups * a.count, groups, opts[k]))) return rc;
    return 0;
}

void set_noise(UpdateArgs& a, const rlt_update_noise& N) { a.noise = N.values; a.noise_seed = N.seed; a.noise_stream = N.stream; a.out_noise = N.values ? nullptr : N.drawn; }
}  // namespace

bool rlt_sac_update_supported(const rlt_rocm_device* device, const rlt_sac_agent* A) {
    const int OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    if (OBS < 1 || ACT < 1 || ACT > MAX_ACT || D > MAX_D || A->batch < 1) return false;
    if (A->final_step_mask || A->next_final_step_mask || A->reset) return false;       // the masked variants count rows over the whole batch first
    if (!net_ok(A->actor, A->n_actor_layers, OBS, 2 * ACT)) return false;
    for (int k = 0; k < 2; k++)
        if (!net_ok(A->critics[k], A->n_critic_layers, D, 1) || !net_ok(A->critics_target[k], A->n_critic_layers, D, 1)) return false;
    return lds_floats(tile_bucket(D)) * sizeof(float) <= (size_t)device->lds_bytes;
}

static void sac_critic_args(UpdateArgs& a, const rlt_sac_agent* A) {
    a.actor = net_of(A->actor);
    for (int k = 0; k < 2; k++) a.target[k] = net_of(A->critics_target[k]);
    a.batch_base = A->observations_actions_base; a.rewards = A->rewards; a.terminated = A->terminated; a.log_alpha = A->log_alpha.parameters;
    a.sas = A->sas; a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_log_probabilities = A->next_log_probabilities; a.out_target_action_value = A->target_action_value;
}

int rlt_sac_update_critic(rlt_rocm_device* device, const rlt_sac_agent* A, int ci, const rlt_update_noise& noise) {
    if (!rlt_sac_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[ci][l].d_weights && A->critics[ci][l].d_biases);
    UpdateArgs a = {};
    sac_critic_args(a, A);
    a.critic[0] = net_of(A->critics[ci]); a.critic[1] = a.critic[0];
    set_noise(a, noise);
    const Optimiser O = {A->critics[ci], A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], nullptr, nullptr, nullptr, 0.0f, nullptr};
    return launch_update<MODE_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), &O, 1);
}

// both critics' updates on the same batch and noise in one launch (they do not depend on each other: each reads the actor, both target
// critics and itself), and after them, if asked for, the soft update of both targets by whichever workgroup finishes last
int rlt_sac_update_critics(rlt_rocm_device* device, const rlt_sac_agent* A, const rlt_update_noise& noise, bool update_targets) {
    if (!rlt_sac_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int k = 0; k < 2; k++) for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[k][l].d_weights && A->critics[k][l].d_biases);
    UpdateArgs a = {};
    sac_critic_args(a, A);
    for (int k = 0; k < 2; k++) a.critic[k] = net_of(A->critics[k]);
    set_noise(a, noise);
    const Optimiser O[2] = {{A->critics[0], A->critic_adam_tensors[0], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[0], nullptr, nullptr, nullptr, 0.0f, update_targets ? A->critics_target[0] : nullptr},
                            {A->critics[1], A->critic_adam_tensors[1], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[1], nullptr, nullptr, nullptr, 0.0f, update_targets ? A->critics_target[1] : nullptr}};
    const int rc = launch_update<MODE_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), O, 2, A->polyak);
    if (rc || !update_targets || a.tail.enabled) return rc;
    return rlt_rocm_sac_update_critic_targets(device, A);      // the optimisers ran as launches of their own: so does the soft update
}

int rlt_sac_update_actor(rlt_rocm_device* device, const rlt_sac_agent* A, const rlt_update_noise& noise) {
    if (!rlt_sac_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->actor[l].d_weights && A->actor[l].d_biases);
    RLT_REQUIRE(A->log_alpha.gradient);
    UpdateArgs a = {};
    a.actor = net_of(A->actor);
    for (int k = 0; k < 2; k++) { a.critic[k] = net_of(A->critics[k]); a.target[k] = a.critic[k]; }
    a.batch_base = A->observations_actions_base; a.log_alpha = A->log_alpha.parameters;
    set_noise(a, noise);
    a.sas = A->sas; a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_log_probabilities = A->actor_log_probabilities; a.out_actions = A->actor_actions; a.out_pre_squashing = A->actor_pre_squashing;
    const Optimiser O = {A->actor, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, &A->log_alpha, &A->alpha_adam, A->alpha_age, 1.0f / (float)A->batch, nullptr};
    return launch_update<MODE_ACTOR>(device, a, rlt_div_up(A->batch, ROWS), &O, 1);
}

// ---- TD3: the same kernel with the td3_sampling head (rl/algorithms/td3/operations_generic.h:170-281)

bool rlt_td3_update_supported(const rlt_rocm_device* device, const rlt_td3_agent* A) {
    const int OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    if (OBS < 1 || ACT < 1 || ACT > MAX_ACT || D > MAX_D || A->batch < 1) return false;
    if (A->final_step_mask || A->next_final_step_mask) return false;       // the masked variants count rows over the whole batch first
    if (!net_ok(A->actor, A->n_actor_layers, OBS, ACT, RLT_ACT_TANH) || !net_ok(A->actor_target, A->n_actor_layers, OBS, ACT, RLT_ACT_TANH)) return false;
    for (int k = 0; k < 2; k++)
        if (!net_ok(A->critics[k], A->n_critic_layers, D, 1) || !net_ok(A->critics_target[k], A->n_critic_layers, D, 1)) return false;
    return lds_floats(tile_bucket(D)) * sizeof(float) <= (size_t)device->lds_bytes;
}

int rlt_td3_update_critic(rlt_rocm_device* device, const rlt_td3_agent* A, int ci, const float* sampling_noise) {
    if (!rlt_td3_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[ci][l].d_weights && A->critics[ci][l].d_biases);
    RLT_REQUIRE(A->target_next_action_noise && sampling_noise);
    UpdateArgs a = {};
    a.actor = net_of(A->actor_target); a.critic[0] = net_of(A->critics[ci]); a.critic[1] = a.critic[0];
    for (int k = 0; k < 2; k++) a.target[k] = net_of(A->critics_target[k]);
    a.batch_base = A->observations_actions_base; a.rewards = A->rewards; a.terminated = A->terminated; a.noise = sampling_noise; a.target_noise = A->target_next_action_noise;
    a.sampling_std = A->sampling_std; a.ignore_termination = A->ignore_termination;
    a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_target_action_value = A->target_action_value;
    const Optimiser O = {A->critics[ci], A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], nullptr, nullptr, nullptr, 0.0f, nullptr};
    return launch_update<MODE_TD3_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), &O, 1);
}

// both critics on the agent's batch in one launch (blockIdx.y selects the critic), each with its own sampling noise; draws != NULL: the two sampling noises and the
// smoothing noise are drawn inside the launch; update_targets: the targets' soft update afterwards (by the launch's last workgroup where the optimisers run there)
int rlt_td3_update_critics(rlt_rocm_device* device, const rlt_td3_agent* A, const float* sampling_noise_first, const float* sampling_noise_second, const rlt_td3_critic_draws* draws, bool update_targets) {
    if (!rlt_td3_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int k = 0; k < 2; k++) for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[k][l].d_weights && A->critics[k][l].d_biases);
    RLT_REQUIRE(A->target_next_action_noise && (draws || (sampling_noise_first && sampling_noise_second)));
    UpdateArgs a = {};
    a.actor = net_of(A->actor_target);
    for (int k = 0; k < 2; k++) { a.critic[k] = net_of(A->critics[k]); a.target[k] = net_of(A->critics_target[k]); }
    a.batch_base = A->observations_actions_base; a.rewards = A->rewards; a.terminated = A->terminated;
    if (draws) {
        a.noise_seed = draws->seed; a.noise_stream = draws->sampling_stream[0]; a.noise_stream_second = draws->sampling_stream[1]; a.target_noise_stream = draws->target_noise_stream;
        a.target_noise_std = draws->target_noise_std; a.target_noise_clip = draws->target_noise_clip; a.out_target_noise = A->target_next_action_noise;
    } else { a.noise = sampling_noise_first; a.noise_second = sampling_noise_second; a.target_noise = A->target_next_action_noise; }
    a.sampling_std = A->sampling_std; a.ignore_termination = A->ignore_termination;
    a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_target_action_value = A->target_action_value;
    Optimiser O[2];
    for (int k = 0; k < 2; k++)
        O[k] = {A->critics[k], A->critic_adam_tensors[k], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[k], nullptr, nullptr, nullptr, 0.0f, update_targets ? A->critics_target[k] : nullptr};
    const int rc = launch_update<MODE_TD3_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), O, 2, A->critic_polyak);
    if (rc || !update_targets || a.tail.enabled) return rc;
    return rlt_rocm_td3_update_critic_targets(device, A);      // the optimisers ran as launches of their own: so does the soft update
}

int rlt_td3_update_actor(rlt_rocm_device* device, const rlt_td3_agent* A, const float* sampling_noise, uint64_t seed, uint64_t stream) {
    if (!rlt_td3_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->actor[l].d_weights && A->actor[l].d_biases);
    UpdateArgs a = {};
    a.actor = net_of(A->actor);
    for (int k = 0; k < 2; k++) { a.critic[k] = net_of(A->critics[0]); a.target[k] = a.critic[k]; }       // the policy gradient goes through critic 0 (:260)
    a.batch_base = A->observations_actions_base; a.noise = sampling_noise; a.noise_seed = seed; a.noise_stream = stream;      // sampling_noise NULL: drawn from (seed, stream)
    a.sampling_std = A->sampling_std;
    a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_pre_clip = A->actor_pre_clip;
    const Optimiser O = {A->actor, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, nullptr, nullptr, nullptr, 0.0f, nullptr};
    return launch_update<MODE_TD3_ACTOR>(device, a, rlt_div_up(A->batch, ROWS), &O, 1);
}

int rlt_sac_polyak_list(rlt_rocm_device* device, const float* const* sources, float* const* targets, const uint32_t* counts, int n, float polyak) {
    for (int base = 0; base < n; base += MAX_POLYAK) {
        PolyakList P = {};
        P.n = n - base < MAX_POLYAK ? n - base : MAX_POLYAK; P.polyak = polyak;
        uint32_t largest = 0;
        for (int i = 0; i < P.n; i++) { P.source[i] = sources[base + i]; P.target[i] = targets[base + i]; P.count[i] = counts[base + i]; largest = counts[base + i] > largest ? counts[base + i] : largest; }
        const int parts = (int)((largest + 2047) / 2048);
        hipLaunchKernelGGL(polyak_list_kernel, dim3(P.n * (parts < 1 ? 1 : parts)), dim3(256), 0, device->stream, P);
        int rc = rlt_launch_status(device);
        if (rc) return rc;
    }
    return 0;
}

extern "C" int rlt_rocm_polyak_update_list(rlt_rocm_device* device, const float* const* sources, float* const* targets, const uint32_t* counts, int n_tensors, float polyak) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(sources && targets && counts && n_tensors >= 0);
    for (int i = 0; i < n_tensors; i++) RLT_REQUIRE(sources[i] && targets[i]);
    return rlt_sac_polyak_list(device, sources, targets, counts, n_tensors, polyak);
}
