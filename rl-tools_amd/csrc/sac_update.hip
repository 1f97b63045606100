// One launch for the network passes of a SAC critic update, one for those of an actor update, for actors obs -> 64 -> 64 -> 2 act and
// critics obs + act -> 64 -> 64 -> 1 of any observation / action width up to 128 inputs and 8 actions.
// reference: rl/algorithms/sac/operations_generic.h:243-337 (train_critic), :395-468 (train_actor),
//            nn/layers/sample_and_squash/operations_generic.h:148-398, nn_models/mlp/operations_generic.h:128-260.
//
// A workgroup of four wavefronts takes 64 rows of the batch, each wavefront its own 16 rows, through every pass of the update:
//   critic update   actor on the next observations -> squashed sample and its log-probability -> both target critics -> TD target ->
//                   critic forward, MSE gradient, backward
//   actor update    actor forward -> squashed sample -> both critics forward and input gradient with d_output = -1 / batch -> gradient of
//                   the smaller value per row -> sample_and_squash backward (entropy term, log_alpha gradient) -> actor backward
// The networks take turns in one LDS region for the weights (staged by the whole workgroup between two barriers); activations stay in
// LDS in the operand layouts of v_mfma_f32_16x16x4_f32 (lane l = r + 16 kk feeds A[r][kk] and B[kk][r], receives D[4 kk + v][r]). The
// weight gradients of the trained network are reductions over the workgroup's 64 rows, split by output columns across the wavefronts
// (wavefront w owns rows 16 w .. 16 w + 15 of dW1 and dW2 and 16 columns of dW3), so every accumulator tile lives in one wavefront's
// registers; a workgroup writes one block of partial sums, which the reduction kernel of the small-MLP path adds up in workgroup order
// (OVERWRITING the gradients: what zero_gradient followed by backward leaves). The Adam step is the library's usual launch.
// Bound: latency (a batch of 256 is four workgroups); the point of this path is three launches per update instead of about twenty.
#include "sac_update.h"
#include "mlp_small.h"
#include "optim.h"

namespace {
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) float* lptr;
constexpr int H = 64, HS = H + 1, WAVES = 4, ROWS = 16 * WAVES, THREADS = 64 * WAVES, MAX_D = 128, MAX_ACT = 8, MAX_OUT = 16, D3S = MAX_OUT + 1, N_EXTRA = 16,
              N_SUMS = 2 * H + MAX_OUT + N_EXTRA, MISC = 16, N_BIAS = 2 * H + MAX_OUT;
enum { MODE_CRITIC = 0, MODE_ACTOR = 1 };

struct Net { const float *W1, *b1, *W2, *b2, *W3, *b3; int in, out, act_h, act3; };
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
};

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
template <int CTRL>
__device__ __forceinline__ float dpp(float x) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true)); }
// sum over the 16 lanes of a row (r = 0..15), every lane of the row receives it
__device__ __forceinline__ float row16_sum(float x) { asm volatile("" : "+v"(x)); x += dpp<0xB1>(x); x += dpp<0x4E>(x); x += dpp<0x141>(x); x += dpp<0x140>(x); return x; }
// sum over the four lane groups (lanes r, r + 16, r + 32, r + 48), in a fixed order
__device__ __forceinline__ float groups_sum(float v) { asm volatile("" : "+v"(v)); v += __shfl_xor(v, 16, 64); v += __shfl_xor(v, 32, 64); return v; }
// lanes of one wavefront exchange data through LDS: the hardware executes a wavefront's LDS instructions in order, the fences keep
// the compiler from moving them across
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }
__device__ __forceinline__ float normal_log_prob(float mean, float log_std, float sd, float value) {
    const float z = (value - mean) / sd;
    return -0.9189385332046727f - log_std - 0.5f * z * z;
}

// hidden activation: a compile-time constant where the kernel is instantiated for it (ACT_H >= 0), else the network's run-time value
template <int ACT_H> __device__ __forceinline__ float act_hidden(float x, int f) { return rlt_act(x, ACT_H >= 0 ? ACT_H : f); }
template <int ACT_H> __device__ __forceinline__ float dact_hidden(float o, int f) { return rlt_dact_from_output(o, ACT_H >= 0 ? ACT_H : f); }

constexpr size_t lds_floats(int nt1c) {
    const int sx = 16 * nt1c + 1;
    return (size_t)H * sx + H * HS + MAX_OUT * HS + N_BIAS + (size_t)ROWS * (sx + 4 * HS + D3S) + WAVES * MISC;
}

// The workgroup replaces the network in LDS in two halves, so that the loads travel while the previous network is still at work:
// fetch_net requests this thread's share of the parameters into registers, commit_net waits for every wavefront to be done with the
// previous network, stores them and meets again. W1 rows are padded to SX with zeros beyond the input width (so the padded reduction
// steps and columns that hold something else add nothing), W3 rows and biases beyond the output width are zero.
struct NetRegs { float v1[H / WAVES][2], v2[H * H / THREADS], v3[MAX_OUT * H / THREADS], bias; };
__device__ __forceinline__ void fetch_net(const Net& N, NetRegs& R, int wave, int lane) {
    const int IN = N.in, OUT = N.out, t = threadIdx.x;
#pragma unroll
    for (int j = 0; j < H / WAVES; j++) {
        const float* src = N.W1 + (size_t)(wave * (H / WAVES) + j) * IN;
        R.v1[j][0] = src[min(lane, IN - 1)];
        R.v1[j][1] = IN > 64 ? src[min(64 + lane, IN - 1)] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < H * H / THREADS; u++) R.v2[u] = N.W2[u * THREADS + t];
#pragma unroll
    for (int u = 0; u < MAX_OUT * H / THREADS; u++) R.v3[u] = N.W3[min(u * THREADS + t, OUT * H - 1)];
    R.bias = t < H ? N.b1[t] : t < 2 * H ? N.b2[t - H] : N.b3[min(t - 2 * H, OUT - 1)];
}
template <int SX>
__device__ __forceinline__ void commit_net(const NetRegs& R, int IN, int OUT, lptr w1s, lptr w2s, lptr w3s, lptr bs, int wave, int lane) {
    rlt_lds_barrier();      // nobody reads the previous network any more
#pragma unroll
    for (int j = 0; j < H / WAVES; j++) {
        const lptr dst = w1s + (wave * (H / WAVES) + j) * SX;
        if (lane < SX) dst[lane] = lane < IN ? R.v1[j][0] : 0.f;
        if (64 + lane < SX) dst[64 + lane] = 64 + lane < IN ? R.v1[j][1] : 0.f;
        if (lane == 0 && SX > 128) dst[128] = 0.f;
    }
#pragma unroll
    for (int u = 0; u < H * H / THREADS; u++) { const int i = u * THREADS + threadIdx.x; w2s[(i >> 6) * HS + (i & 63)] = R.v2[u]; }
#pragma unroll
    for (int u = 0; u < MAX_OUT * H / THREADS; u++) { const int i = u * THREADS + threadIdx.x; w3s[(i >> 6) * HS + (i & 63)] = (i >> 6) < OUT ? R.v3[u] : 0.f; }
    if (threadIdx.x < N_BIAS) bs[threadIdx.x] = (int)threadIdx.x < 2 * H + OUT ? R.bias : 0.f;
    rlt_lds_barrier();
}

// the wavefront's 16 rows of a [batch x ld] array for its input tile: columns [0, valid), zero beyond them and beyond the batch; requested
// into registers, stored later
struct RowRegs { float va[16], vb[16]; };
__device__ __forceinline__ void request_rows(RowRegs& X, const float* base, int ld, int row0, int batch, int valid, int lane) {
#pragma unroll
    for (int row = 0; row < 16; row++) {
        const bool rok = row0 + row < batch;
        const float* src = base + (size_t)min(row0 + row, batch - 1) * ld;
        X.va[row] = (rok && lane < valid) ? src[lane] : 0.f;
        X.vb[row] = (rok && 64 + lane < valid) ? src[64 + lane] : 0.f;
    }
}
template <int SX, int NT1C>
__device__ __forceinline__ void store_rows(const RowRegs& X, lptr xs, int lane) {
#pragma unroll
    for (int row = 0; row < 16; row++) {
        if (lane < 16 * NT1C) xs[row * SX + lane] = X.va[row];
        if (64 + lane < 16 * NT1C) xs[row * SX + 64 + lane] = X.vb[row];
    }
}

// the three layers on the wavefront's rows; h1 and h2 (after the activation) stay in LDS; returns the last layer's sums before bias and
// activation: element v of lane (r, kk) belongs to row 4 kk + v, output r
template <int SX, int ACT_H>
__device__ __forceinline__ floatx4 forward16(const Net& N, lptr w1s, lptr w2s, lptr w3s, lptr bs, lptr xs, lptr h1s, lptr h2s, int r, int kk) {
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const int NT1 = (N.in + 15) >> 4;
    floatx4 acc[4] = {zero4, zero4, zero4, zero4};
    for (int g = 0; g < NT1; g++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float a = xs[r * SX + 16 * g + 4 * q + kk];
#pragma unroll
            for (int nt = 0; nt < 4; nt++) acc[nt] = mfma16(a, w1s[(16 * nt + r) * SX + 16 * g + 4 * q + kk], acc[nt]);
        }
    }
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        const float b = bs[16 * nt + r];
#pragma unroll
        for (int v = 0; v < 4; v++) h1s[(4 * kk + v) * HS + 16 * nt + r] = act_hidden<ACT_H>(acc[nt][v] + b, N.act_h);
    }
    wave_sync();
#pragma unroll
    for (int nt = 0; nt < 4; nt++) acc[nt] = zero4;
#pragma unroll
    for (int s = 0; s < 16; s++) {
        const float a = h1s[r * HS + 16 * kk + s];
#pragma unroll
        for (int nt = 0; nt < 4; nt++) acc[nt] = mfma16(a, w2s[(16 * nt + r) * HS + 16 * kk + s], acc[nt]);
    }
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        const float b = bs[H + 16 * nt + r];
#pragma unroll
        for (int v = 0; v < 4; v++) h2s[(4 * kk + v) * HS + 16 * nt + r] = act_hidden<ACT_H>(acc[nt][v] + b, N.act_h);
    }
    wave_sync();
    floatx4 y0 = zero4, y1 = zero4;
#pragma unroll
    for (int s = 0; s < 16; s += 2) {
        y0 = mfma16(h2s[r * HS + 16 * kk + s], w3s[r * HS + 16 * kk + s], y0);
        y1 = mfma16(h2s[r * HS + 16 * kk + s + 1], w3s[r * HS + 16 * kk + s + 1], y1);
    }
    return y0 + y1;
}

// d_pre2 = (d_pre3 W3) f'(h2) into g2s (may be h2s itself), accumulating its column sums
template <int ACT_H>
__device__ __forceinline__ void backward_layer3(const Net& N, lptr w3s, lptr d3s, lptr h2s, lptr g2s, float (&s2)[4], int r, int kk) {
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    floatx4 acc[4] = {zero4, zero4, zero4, zero4};
#pragma unroll
    for (int ks = 0; ks < MAX_OUT / 4; ks++) {      // columns of d_pre3 and rows of W3 beyond the output width are zero
        const float a = d3s[r * D3S + 4 * ks + kk];
#pragma unroll
        for (int nt = 0; nt < 4; nt++) acc[nt] = mfma16(a, w3s[(4 * ks + kk) * HS + 16 * nt + r], acc[nt]);
    }
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int idx = (4 * kk + v) * HS + 16 * nt + r;
            const float dp = acc[nt][v] * dact_hidden<ACT_H>(h2s[idx], N.act_h);
            g2s[idx] = dp; s2[nt] += dp;
        }
}
// d_pre1 = (d_pre2 W2) f'(h1) into p1s (may be h1s itself), accumulating its column sums
template <int ACT_H>
__device__ __forceinline__ void backward_layer2(const Net& N, lptr w2s, lptr g2s, lptr h1s, lptr p1s, float (&s1)[4], int r, int kk) {
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    floatx4 acc[4] = {zero4, zero4, zero4, zero4};
#pragma unroll
    for (int s = 0; s < 16; s++) {
        const float a = g2s[r * HS + 16 * kk + s];
#pragma unroll
        for (int nt = 0; nt < 4; nt++) acc[nt] = mfma16(a, w2s[(16 * kk + s) * HS + 16 * nt + r], acc[nt]);
    }
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int idx = (4 * kk + v) * HS + 16 * nt + r;
            const float dp = acc[nt][v] * dact_hidden<ACT_H>(h1s[idx], N.act_h);
            p1s[idx] = dp; s1[nt] += dp;
        }
}

// sample_and_squash forward for the items of a lane: row r of the wavefront's tile, actions kk and kk + 4
struct HeadItem { float mean, log_std_raw, noise, sample, action; };
__device__ __forceinline__ float head_forward(const UpdateArgs& A, lptr d3s, lptr xs, int SX, const float (&noise)[2], int r, int kk, HeadItem (&item)[2]) {
    float log_prob = 0.f;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int a = kk + 4 * j;
        HeadItem& I = item[j];
        I = {0.f, 0.f, 0.f, 0.f, 0.f};
        if (a < A.act) {
            I.mean = d3s[r * D3S + a];
            I.log_std_raw = d3s[r * D3S + A.act + a];
            const float log_std = clampf(I.log_std_raw, A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
            const float sd = expf(log_std);
            I.noise = noise[j];
            I.sample = I.mean + I.noise * sd;
            I.action = tanhf(I.sample);
            xs[r * SX + A.obs + a] = I.action;
            log_prob += normal_log_prob(I.mean, log_std, sd, I.sample) - logf(1.0f - I.action * I.action + A.sas.log_probability_epsilon);
        }
    }
    return groups_sum(log_prob);
}

template <int NT1C, int MODE, int ACT_H>
__global__ __launch_bounds__(THREADS) void sac_update_kernel(UpdateArgs A) {
    extern __shared__ float lds_raw[];
    constexpr int SX = 16 * NT1C + 1;
    const int lane = threadIdx.x & 63, r = lane & 15, kk = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int OBS = A.obs, ACT = A.act, D = OBS + ACT, B = A.batch;
    const lptr w1s = (lptr)lds_raw, w2s = w1s + H * SX, w3s = w2s + H * HS, bs = w3s + MAX_OUT * HS;
    const lptr xs_all = bs + N_BIAS, h1_all = xs_all + ROWS * SX, h2_all = h1_all + ROWS * HS, ta_all = h2_all + ROWS * HS, tb_all = ta_all + ROWS * HS,
               d3_all = tb_all + ROWS * HS, misc_all = d3_all + ROWS * D3S;
    const lptr xs = xs_all + 16 * wave * SX, h1s = h1_all + 16 * wave * HS, h2s = h2_all + 16 * wave * HS, tas = ta_all + 16 * wave * HS, tbs = tb_all + 16 * wave * HS,
               d3s = d3_all + 16 * wave * D3S, misc = misc_all + wave * MISC;
    const int row0 = blockIdx.x * ROWS + 16 * wave;
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    float s1[4] = {0.f, 0.f, 0.f, 0.f}, s2[4] = {0.f, 0.f, 0.f, 0.f}, s3 = 0.f, extra = 0.f, unused[4] = {0.f, 0.f, 0.f, 0.f};
    const Net& trained = MODE == MODE_CRITIC ? A.critic[0] : A.actor;
    // every global load is requested one stage ahead of its use: the next network's parameters while the current one computes
    NetRegs R;
    RowRegs X;
    fetch_net(A.actor, R, wave, lane);
    request_rows(X, MODE == MODE_CRITIC ? A.batch_base + (size_t)B * D : A.batch_base, D, row0, B, MODE == MODE_CRITIC ? D : OBS, lane);
    const float alpha = expf(*A.log_alpha);
    float noise[2];
#pragma unroll
    for (int j = 0; j < 2; j++) noise[j] = (kk + 4 * j < ACT && row0 + r < B) ? A.noise[(size_t)(row0 + r) * ACT + kk + 4 * j] : 0.f;
    HeadItem item[2];

    if (MODE == MODE_CRITIC) {
        float reward[4]; bool terminated[4];
#pragma unroll
        for (int v = 0; v < 4; v++) { const int row = min(row0 + 4 * kk + v, B - 1); reward[v] = A.rewards[row]; terminated[v] = A.terminated[row] != 0; }
        // the actor on the next observations, its squashed sample into the action columns of the tile
        store_rows<SX, NT1C>(X, xs, lane);
        commit_net<SX>(R, A.actor.in, A.actor.out, w1s, w2s, w3s, bs, wave, lane);
        fetch_net(A.target[0], R, wave, lane);
        {
            const floatx4 y = forward16<SX, ACT_H>(A.actor, w1s, w2s, w3s, bs, xs, tas, tbs, r, kk);
            const float b3 = bs[2 * H + r];
#pragma unroll
            for (int v = 0; v < 4; v++) d3s[(4 * kk + v) * D3S + r] = r < A.actor.out ? rlt_act(y[v] + b3, A.actor.act3) : 0.f;
        }
        wave_sync();
        const float next_log_prob = head_forward(A, d3s, xs, SX, noise, r, kk, item);
        if (kk == 0) {
            misc[r] = next_log_prob;
            if (A.out_log_probabilities && row0 + r < B) A.out_log_probabilities[row0 + r] = next_log_prob;
        }
        wave_sync();
        // both target critics on [next observation | sampled action]
        float q_min[4];
#pragma unroll
        for (int k = 0; k < 2; k++) {
            commit_net<SX>(R, A.target[k].in, A.target[k].out, w1s, w2s, w3s, bs, wave, lane);
            if (k == 0) fetch_net(A.target[1], R, wave, lane);
            else { fetch_net(trained, R, wave, lane); request_rows(X, A.batch_base, D, row0, B, D, lane); }
            const floatx4 y = forward16<SX, ACT_H>(A.target[k], w1s, w2s, w3s, bs, xs, tas, tbs, r, kk);
            const float b3 = bs[2 * H];
#pragma unroll
            for (int v = 0; v < 4; v++) { const float q = rlt_act(y[v] + b3, A.target[k].act3); q_min[v] = k ? fminf(q_min[v], q) : q; }
        }
        // TD target of rows 4 kk + v (meaningful in the lanes r == 0, which hold output 0)
        float y_target[4];
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float min_q = q_min[v] - alpha * misc[4 * kk + v];
            const float future = terminated[v] ? 0.0f : A.gamma * min_q;
            y_target[v] = reward[v] + future;
            if (A.out_target_action_value && r == 0 && row0 + 4 * kk + v < B) A.out_target_action_value[row0 + 4 * kk + v] = y_target[v];
        }
        // the critic on the current rows, MSE gradient at its pre-activation
        wave_sync();
        store_rows<SX, NT1C>(X, xs, lane);
        commit_net<SX>(R, trained.in, trained.out, w1s, w2s, w3s, bs, wave, lane);
        const floatx4 y = forward16<SX, ACT_H>(trained, w1s, w2s, w3s, bs, xs, h1s, h2s, r, kk);
        const float b3 = bs[2 * H];
        // loss weight batch * 0.5 / n with n = batch rows (no masks), times the MSE gradient's 2 / batch (rl/algorithms/sac/operations_generic.h:298-316)
        const float loss_weight = (1.0f / (float)B) * ((float)B * 0.5f);
        const float constant = 2.0f / (float)B * loss_weight;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const bool ok = r == 0 && row0 + 4 * kk + v < B;
            const float q = rlt_act(y[v] + b3, trained.act3);
            const float diff = q - y_target[v];
            const float dp = ok ? diff * constant * rlt_dact_from_output(q, trained.act3) : 0.f;
            if (ok) extra += diff * diff;
            s3 += dp;
            d3s[(4 * kk + v) * D3S + r] = dp;
        }
    } else {
        // actor forward on the observations (its hidden activations are kept for the backward pass), squashed sample into the action columns
        store_rows<SX, NT1C>(X, xs, lane);
        commit_net<SX>(R, A.actor.in, A.actor.out, w1s, w2s, w3s, bs, wave, lane);
        fetch_net(A.critic[0], R, wave, lane);
        {
            const floatx4 y = forward16<SX, ACT_H>(A.actor, w1s, w2s, w3s, bs, xs, h1s, h2s, r, kk);
            const float b3 = bs[2 * H + r];
#pragma unroll
            for (int v = 0; v < 4; v++) d3s[(4 * kk + v) * D3S + r] = r < A.actor.out ? rlt_act(y[v] + b3, A.actor.act3) : 0.f;
        }
        wave_sync();
        const float log_prob = head_forward(A, d3s, xs, SX, noise, r, kk, item);
        const bool row_ok = row0 + r < B;
        if (row_ok) {
            if (kk == 0 && A.out_log_probabilities) A.out_log_probabilities[row0 + r] = log_prob;
#pragma unroll
            for (int j = 0; j < 2; j++)
                if (kk + 4 * j < ACT) {
                    if (A.out_actions) A.out_actions[(size_t)(row0 + r) * ACT + kk + 4 * j] = item[j].action;
                    if (A.out_pre_squashing) A.out_pre_squashing[(size_t)(row0 + r) * ACT + kk + 4 * j] = item[j].sample;
                }
        }
        wave_sync();
        // both critics on [observation | sampled action]: value and the gradient of -value / batch with respect to the action
        const float loss_weight = (1.0f / (float)B) * -1.0f;       // rl/algorithms/sac/operations_generic.h:437-453 with n = batch rows
        float q_row[2], d_action[2][2];
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const Net& C = A.critic[k];
            commit_net<SX>(R, C.in, C.out, w1s, w2s, w3s, bs, wave, lane);
            fetch_net(k == 0 ? A.critic[1] : A.actor, R, wave, lane);
            const floatx4 y = forward16<SX, ACT_H>(C, w1s, w2s, w3s, bs, xs, tas, tbs, r, kk);
            const float b3 = bs[2 * H];
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float q = rlt_act(y[v] + b3, C.act3);
                if (r == 0) misc[4 * kk + v] = q;
                d3s[(4 * kk + v) * D3S + r] = (r == 0 && row0 + 4 * kk + v < B) ? loss_weight * rlt_dact_from_output(q, C.act3) : 0.f;
            }
            wave_sync();
            backward_layer3<ACT_H>(C, w3s, d3s, tbs, tbs, unused, r, kk);
            wave_sync();
            backward_layer2<ACT_H>(C, w2s, tbs, tas, tas, unused, r, kk);
            wave_sync();
            q_row[k] = misc[r];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                float dot = 0.f;
                if (kk + 4 * j < ACT)
                    for (int n = 0; n < H; n++) dot += tas[r * HS + n] * w1s[n * SX + OBS + kk + 4 * j];
                d_action[k][j] = dot;
            }
            wave_sync();
        }
        // sample_and_squash backward (nn/layers/sample_and_squash/operations_generic.h:262-398) on the gradient of the smaller value
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
                const float d_out = q_row[0] < q_row[1] ? d_action[0][j] : d_action[1][j];
                const float g = d_out * (1.0f - I.action * I.action);
                const float log_std = clampf(I.log_std_raw, A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
                const float sd = expf(log_std);
                const float z = (I.sample - I.mean) / sd;
                const float dlp_dmean = z / sd, dlp_dsample = -z / sd, dlp_dlogstd = z * z - 1.0f;
                const float d_mu = g + alpha_over_b * (dlp_dmean + dlp_dsample + 2.0f * I.action);
                float d_ls = sd * (g * I.noise) + alpha_over_b * (dlp_dlogstd + dlp_dsample * I.noise * sd + 2.0f * I.action * I.noise * sd);
                if (I.log_std_raw < A.sas.log_std_lower_bound || I.log_std_raw > A.sas.log_std_upper_bound) d_ls = 0.0f;
                if (row_ok) {
                    d3s[r * D3S + a] = d_mu * rlt_dact_from_output(I.mean, A.actor.act3);
                    d3s[r * D3S + ACT + a] = d_ls * rlt_dact_from_output(I.log_std_raw, A.actor.act3);
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
        commit_net<SX>(R, A.actor.in, A.actor.out, w1s, w2s, w3s, bs, wave, lane);
    }

    // backward pass of the trained network with its weight gradients over the workgroup's 64 rows; h1, h2: its hidden activations,
    // d3: the gradient at its last pre-activation; ta receives d_pre2, h2 is replaced by d_pre1
    floatx4 aW1[NT1C], aW2[4], aW3a = zero4, aW3b = zero4;
#pragma unroll
    for (int nt = 0; nt < NT1C; nt++) aW1[nt] = zero4;
#pragma unroll
    for (int nt = 0; nt < 4; nt++) aW2[nt] = zero4;
    rlt_lds_barrier();      // every wavefront's h2 and d_pre3 are in place
#pragma unroll
    for (int ks = 0; ks < ROWS / 4; ks++) {
        const float a = d3_all[(4 * ks + kk) * D3S + r], b = h2_all[(4 * ks + kk) * HS + 16 * wave + r];
        if (ks & 1) aW3b = mfma16(a, b, aW3b); else aW3a = mfma16(a, b, aW3a);
    }
    backward_layer3<ACT_H>(trained, w3s, d3s, h2s, tas, s2, r, kk);
    rlt_lds_barrier();      // every wavefront's d_pre2 is in place, and nobody reads h2 any more
#pragma unroll
    for (int ks = 0; ks < ROWS / 4; ks++) {
        const float a = ta_all[(4 * ks + kk) * HS + 16 * wave + r];
#pragma unroll
        for (int nt = 0; nt < 4; nt++) aW2[nt] = mfma16(a, h1_all[(4 * ks + kk) * HS + 16 * nt + r], aW2[nt]);
    }
    backward_layer2<ACT_H>(trained, w2s, tas, h1s, h2s, s1, r, kk);
    rlt_lds_barrier();      // every wavefront's d_pre1 is in place
#pragma unroll 4
    for (int ks = 0; ks < ROWS / 4; ks++) {
        const float a = h2_all[(4 * ks + kk) * HS + 16 * wave + r];
#pragma unroll
        for (int nt = 0; nt < NT1C; nt++) aW1[nt] = mfma16(a, xs_all[(4 * ks + kk) * SX + 16 * nt + r], aW1[nt]);
    }
    rlt_lds_barrier();      // the weights may be overwritten

    // the workgroup's block of partial sums: weight gradients straight from the registers that own them, ...
    const int IN = trained.in, OUT = trained.out, NT1 = (IN + 15) >> 4;
    float* dst = A.partial + (size_t)blockIdx.x * A.count;
    const int o_b1 = H * IN, o_w2 = o_b1 + H, o_b2 = o_w2 + H * H, o_w3 = o_b2 + H, o_b3 = o_w3 + OUT * H, o_ex = o_b3 + OUT;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int m = 16 * wave + 4 * kk + v;
#pragma unroll
        for (int nt = 0; nt < NT1C; nt++)
            if (nt < NT1 && 16 * nt + r < IN) dst[m * IN + 16 * nt + r] = aW1[nt][v];
#pragma unroll
        for (int nt = 0; nt < 4; nt++) dst[o_w2 + m * H + 16 * nt + r] = aW2[nt][v];
        if (4 * kk + v < OUT) dst[o_w3 + (4 * kk + v) * H + 16 * wave + r] = aW3a[v] + aW3b[v];
    }
    // ... the bias gradients and the extra sum, which every wavefront holds for its own rows, summed in wavefront order through LDS
    const lptr sums = (lptr)lds_raw;        // [WAVES][N_SUMS]
#pragma unroll
    for (int nt = 0; nt < 4; nt++) { s1[nt] = groups_sum(s1[nt]); s2[nt] = groups_sum(s2[nt]); }
    s3 = groups_sum(s3); extra = groups_sum(extra);
    if (kk == 0) {
#pragma unroll
        for (int nt = 0; nt < 4; nt++) { sums[wave * N_SUMS + 16 * nt + r] = s1[nt]; sums[wave * N_SUMS + H + 16 * nt + r] = s2[nt]; }
        sums[wave * N_SUMS + 2 * H + r] = s3; sums[wave * N_SUMS + 2 * H + MAX_OUT + r] = extra;
    }
    rlt_lds_barrier();
    if (threadIdx.x < N_SUMS) {
        const int i = threadIdx.x;
        const float total = (sums[i] + sums[N_SUMS + i]) + (sums[2 * N_SUMS + i] + sums[3 * N_SUMS + i]);
        if (i < H) dst[o_b1 + i] = total;
        else if (i < 2 * H) dst[o_b2 + i - H] = total;
        else if (i < 2 * H + MAX_OUT) { if (i - 2 * H < OUT) dst[o_b3 + i - 2 * H] = total; }
        else dst[o_ex + i - 2 * H - MAX_OUT] = total;
    }
}

// soft update of up to 16 tensors in one launch (utils/polyak/operations_generic.h:11-27): workgroup b serves tensor b % n
constexpr int MAX_POLYAK = 16;
struct PolyakList { const float* source[MAX_POLYAK]; float* target[MAX_POLYAK]; uint32_t count[MAX_POLYAK]; int n; float polyak; };
__global__ __launch_bounds__(256) void polyak_list_kernel(PolyakList P) {
    const int t = blockIdx.x % P.n, part = blockIdx.x / P.n, parts = gridDim.x / P.n;
    const float* __restrict__ s = P.source[t]; float* __restrict__ d = P.target[t];
    for (uint32_t i = part * 256 + threadIdx.x; i < P.count[t]; i += parts * 256) d[i] = P.polyak * d[i] + (1.0f - P.polyak) * s[i];
}

bool hidden_ok(int a) { return a == RLT_ACT_RELU || a == RLT_ACT_TANH || a == RLT_ACT_FAST_TANH || a == RLT_ACT_SIGMOID; }
bool out_ok(int a) { return a != RLT_ACT_GELU; }
bool net_ok(const rlt_dense_layer* L, int n, int in, int out) {
    if (!L || n != 3) return false;
    for (int l = 0; l < 3; l++) if (!L[l].weights || !L[l].biases) return false;
    return L[0].in_dim == in && L[0].out_dim == H && L[1].in_dim == H && L[1].out_dim == H && L[2].in_dim == H && L[2].out_dim == out &&
           L[0].activation == L[1].activation && hidden_ok(L[0].activation) && out_ok(L[2].activation);
}
Net net_of(const rlt_dense_layer* L) {
    return {L[0].weights, L[0].biases, L[1].weights, L[1].biases, L[2].weights, L[2].biases, L[0].in_dim, L[2].out_dim, L[0].activation, L[2].activation};
}
int tile_bucket(int d) { return d <= 32 ? 2 : MAX_D / 16; }

template <int MODE>
int launch_update(rlt_rocm_device* device, UpdateArgs& a, int groups, const rlt_dense_layer* trained, float* extra, float extra_scale) {
    const int bucket = tile_bucket(a.obs + a.act);
    const size_t lds_bytes = lds_floats(bucket) * sizeof(float);
    a.count = rlt_mlp3s_partial_count(trained[0].in_dim, trained[2].out_dim);
    void* scratch = nullptr;
    int rc = rlt_scratch(device, (size_t)groups * a.count * sizeof(float), &scratch);
    if (rc) return rc;
    a.partial = (float*)scratch;
#define RLT_LAUNCH_UPDATE(NT, ACT)                                                                                                                              \
    do {                                                                                                                                                        \
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(sac_update_kernel<NT, MODE, ACT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes)); \
        hipLaunchKernelGGL((sac_update_kernel<NT, MODE, ACT>), dim3(groups), dim3(THREADS), lds_bytes, device->stream, a);                                    \
    } while (0)
    // ReLU (the reference's default for SAC) and tanh are compiled in; any other hidden activation takes the variant that looks it up
    const int act = a.actor.act_h == a.critic[0].act_h && a.actor.act_h == a.target[0].act_h ? a.actor.act_h : -1;
    if (bucket == 2) {
        if (act == RLT_ACT_RELU) RLT_LAUNCH_UPDATE(2, RLT_ACT_RELU); else if (act == RLT_ACT_TANH) RLT_LAUNCH_UPDATE(2, RLT_ACT_TANH); else RLT_LAUNCH_UPDATE(2, -1);
    } else {
        if (act == RLT_ACT_RELU) RLT_LAUNCH_UPDATE(MAX_D / 16, RLT_ACT_RELU); else if (act == RLT_ACT_TANH) RLT_LAUNCH_UPDATE(MAX_D / 16, RLT_ACT_TANH); else RLT_LAUNCH_UPDATE(MAX_D / 16, -1);
    }
#undef RLT_LAUNCH_UPDATE
    if ((rc = rlt_launch_status(device))) return rc;
    return rlt_mlp3s_reduce(device, trained, a.partial, groups, 1, extra, extra ? 1 : 0, extra_scale, 0.0f);
}
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

int rlt_sac_update_critic(rlt_rocm_device* device, const rlt_sac_agent* A, int ci, const float* action_noise) {
    if (!rlt_sac_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[ci][l].d_weights && A->critics[ci][l].d_biases);
    UpdateArgs a = {};
    a.actor = net_of(A->actor); a.critic[0] = net_of(A->critics[ci]); a.critic[1] = a.critic[0];
    for (int k = 0; k < 2; k++) a.target[k] = net_of(A->critics_target[k]);
    a.batch_base = A->observations_actions_base; a.rewards = A->rewards; a.terminated = A->terminated; a.noise = action_noise; a.log_alpha = A->log_alpha.parameters;
    a.sas = A->sas; a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_log_probabilities = A->next_log_probabilities; a.out_target_action_value = A->target_action_value;
    int rc = launch_update<MODE_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), A->critics[ci], nullptr, 0.0f);
    if (rc) return rc;
    return rlt_rocm_adam_step(device, A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], 0.0f, nullptr);
}

int rlt_sac_update_actor(rlt_rocm_device* device, const rlt_sac_agent* A, const float* action_noise) {
    if (!rlt_sac_update_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->actor[l].d_weights && A->actor[l].d_biases);
    RLT_REQUIRE(A->log_alpha.gradient);
    UpdateArgs a = {};
    a.actor = net_of(A->actor);
    for (int k = 0; k < 2; k++) { a.critic[k] = net_of(A->critics[k]); a.target[k] = a.critic[k]; }
    a.batch_base = A->observations_actions_base; a.noise = action_noise; a.log_alpha = A->log_alpha.parameters;
    a.sas = A->sas; a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_log_probabilities = A->actor_log_probabilities; a.out_actions = A->actor_actions; a.out_pre_squashing = A->actor_pre_squashing;
    int rc = launch_update<MODE_ACTOR>(device, a, rlt_div_up(A->batch, ROWS), A->actor, A->log_alpha.gradient, 1.0f / (float)A->batch);
    if (rc) return rc;
    if (A->n_actor_adam_tensors <= 12)
        return rlt_adam_step_pair(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, &A->log_alpha, 1, &A->alpha_adam, A->alpha_age);
    if ((rc = rlt_rocm_adam_step(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, 0.0f, nullptr))) return rc;
    return rlt_rocm_adam_step(device, &A->log_alpha, 1, &A->alpha_adam, A->alpha_age, 0.0f, nullptr);
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
