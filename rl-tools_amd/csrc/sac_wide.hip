// One launch for the network passes of a SAC critic update, one for those of an actor update, for three-layer networks of any hidden width
// up to 256 (the zoo's agents are 256 wide: src/rl/zoo/acrobot-swingup-v0/sac.h, ant-v4): actors obs -> h -> h -> 2 act, critics
// obs + act -> h -> h -> 1, at most 128 critic inputs and 8 actions.
// reference: rl/algorithms/sac/operations_generic.h:243-337 (train_critic), :395-468 (train_actor),
//            nn/layers/sample_and_squash/operations_generic.h:148-398, nn_models/mlp/operations_generic.h:128-260.
//
// A workgroup of sixteen wavefronts takes 16 rows of the batch through every pass of the update, one network after the other:
//   critic update   actor on the next observations -> squashed sample and its log-probability -> target critic 0, target critic 1 on
//                   [next observation | sample] -> TD target -> trained critic forward on the current rows -> MSE gradient -> backward
//   actor update    actor forward -> squashed sample -> critic 0, then critic 1: forward and the gradient of -value / batch with respect
//                   to the action -> gradient of the smaller value per row -> sample_and_squash backward (entropy term, log_alpha
//                   gradient) -> actor backward
// The same kernel runs TD3's two updates (rl/algorithms/td3/operations_generic.h:170-281; actors obs -> h -> h -> act with a tanh output followed by the
// td3_sampling layer): the critic update with the target actor, the smoothing noise on the next action and no entropy term, the actor update through critic 0 only.
// Wavefront w owns hidden units 16 w .. 16 w + 15 of every layer: it computes that tile of the 16 x h activations from the whole previous
// layer (LDS, behind a workgroup barrier), contributes the units' share of the output layer's reduction (the partial tiles are added in
// wavefront order), and in the backward pass owns the same units' pre-activation gradients and their rows of dW1, dW2 and columns of dW3.
// Weights are read from memory (L2) straight into the B operands of v_mfma_f32_16x16x4_f32 when a layer needs them, the second
// layer's first half a layer ahead; hidden widths that are no multiple of 16 are completed with zero operands. The reduction index of a
// 16-deep chunk is dealt to the four lane groups as k = 16 j + 4 g + i for the i-th of four instructions, so that activations (LDS) and
// weights (memory) are both read 16 bytes at a time.
// A workgroup writes one block of partial sums of the trained network's gradients [dW1 | db1 | dW2 | db2 | dW3 | db3 | extra]; the
// optimiser's launch adds the blocks up over the whole chip (one compute unit draws about 4 GB/s from memory and 20 GB/s from L2 with loads
// of this kind: read by the update's own sixteen workgroups, the 4.4 MB of blocks at width 256 took 70 us; spread over all compute units, 10).
// Bound: per workgroup, a 16 x 256 x 256 layer is 2.1 MFLOP = 3.4 us of one compute unit's matrix pipeline, and an update has six or seven
// of them; a batch of 256 is sixteen workgroups (thirty-two where both critics share the launch).
#include "sac_update.h"
#include "optim.h"
#include "rng.h"
#include "sac_heads.h"

namespace {
using namespace rlt_sac;
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) floatx4* lptr4;
constexpr int ROWS = 16, MAX_H = 256, WAVES = MAX_H / 16, THREADS = 64 * WAVES, S = MAX_H + 4, MAX_D = 128, SXS = MAX_D + 4, MAX_ACT = 8, MAX_OUT = 16, D3S = MAX_OUT + 1,
              N_EXTRA = 16, MISC = 64, YP = ROWS * D3S;
enum { MODE_CRITIC = 0, MODE_ACTOR = 1, MODE_TD3_CRITIC = 2, MODE_TD3_ACTOR = 3 };      // SAC's two updates, TD3's two updates

// W2f / W2b: copies of the second layer's weights in the order the wavefronts consume them (wide_prepare_kernel): 16 bytes per lane, a wavefront's load 1 KB in a row
struct WNet { const float *W1, *b1, *W2, *b2, *W3, *b3; int in, hid, out, act_h, vec1, vec2, vec3; const float *W2f, *W2b; };      // vecN: the rows of WN can be read 16 bytes at a time
struct WideArgs {
    WNet actor, critic[2], target[2];
    const float* batch_base;               // [2][batch][obs + act]: current rows, then next rows
    const float* rewards; const uint8_t* terminated;
    const float* noise;                    // [batch][act], or NULL: drawn from (noise_seed, noise_stream + *stream_offset)
    uint64_t noise_seed, noise_stream; float* out_noise; const uint64_t* stream_offset;
    // TD3's critic update with its draws made here (noise, noise_second and target_noise NULL): the second critic's sampling noise and the smoothing noise
    // clamp(N(0, 1) * target_noise_std, -clip, clip) on streams of their own, the latter stored to out_target_noise
    uint64_t noise_stream_second, target_noise_stream; float target_noise_std, target_noise_clip; float* out_target_noise;
    const float* log_alpha;
    rlt_sas_parameters sas;
    float gamma;
    int batch, obs, act;
    float* partial; int count;             // per workgroup and trained network: count floats (the optimiser's launch adds the blocks up)
    float* out_log_probabilities; float* out_target_action_value; float* out_actions; float* out_pre_squashing;
    // TD3 (rl/algorithms/td3/operations_generic.h:170-281): `actor` is the target actor in the critic update and has `act` outputs; they pass tanh and the
    // td3_sampling layer (sac_heads.h); the critic update adds target_noise [batch][act] (already clamped) to the next action; the actor update goes through critic[0] only
    float sampling_std; int ignore_termination; const float* target_noise; float* out_pre_clip;
    const float* noise_second;             // TD3 critic update of both critics in one launch: the sampling noise of the second (blockIdx.y = 1), each critic's targets being formed with its own
    int packed;                            // every 8th workgroup of an 8 x larger grid works: all of them on one XCD
};

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
template <int ACT_H> __device__ __forceinline__ float act_hidden(float x, int f) { return rlt_act(x, ACT_H >= 0 ? ACT_H : f); }
template <int ACT_H> __device__ __forceinline__ float dact_hidden(float o, int f) { return rlt_dact_from_output(o, ACT_H >= 0 ? ACT_H : f); }

// B operands of one layer for this lane's output column n: W[n][16 j + 4 g ... + 3] for chunks j0 <= j < j0 + JN; zero beyond the layer's shape
template <int JN>
__device__ __forceinline__ void load_rows(const float* __restrict__ W, int K, int N, bool vec, int n, int g, int j0, floatx4 (&b)[JN]) {
    const bool n_ok = n < N;
    const float* row = W + (size_t)(n_ok ? n : 0) * K;
#pragma unroll
    for (int j = 0; j < JN; j++) {
        const int k = 16 * (j0 + j) + 4 * g;
        floatx4 v = {0.f, 0.f, 0.f, 0.f};
        if (n_ok && k < K) {
            if (vec) v = *reinterpret_cast<const floatx4*>(row + k);      // K is a multiple of 4 here
            else { v[0] = row[k]; if (k + 1 < K) v[1] = row[k + 1]; if (k + 2 < K) v[2] = row[k + 2]; if (k + 3 < K) v[3] = row[k + 3]; }
        }
        b[j] = v;
    }
}
// The same operands from a copy laid out in consumption order: [wavefront's 16 units][16-deep chunk j][lane][4] -- lane (c, g) finds W[16 w + c][16 j + 4 g ... + 3]
// (forward copy) or W[16 j + 4 g ... + 3][16 w + c] (backward copy), zero beyond the layer's shape, and a wavefront's load is 1 KB of consecutive addresses. Straight from
// W a lane's 16 bytes lie a row (1 KB) apart from its neighbour's: 64 lines per load, which the compute unit's address pipeline takes 64 cycles for.
template <int JN>
__device__ __forceinline__ void load_swizzled(const float* __restrict__ copy, int tiles, int wave, int lane, int j0, floatx4 (&b)[JN]) {
#pragma unroll
    for (int j = 0; j < JN; j++) {
        floatx4 v = {0.f, 0.f, 0.f, 0.f};
        if (j0 + j < tiles) v = *reinterpret_cast<const floatx4*>(copy + ((size_t)(wave * tiles + j0 + j) * 64 + lane) * 4);
        b[j] = v;
    }
}
// acc += in[rows][16 (j0 + j) + ...] * b[j], the workgroup's 16 rows against this lane's column
template <int JN>
__device__ __forceinline__ void chunks(floatx4& a0, floatx4& a1, lptr in, int stride, int c, int g, int j0, int steps, const floatx4 (&b)[JN]) {
#pragma unroll
    for (int j = 0; j < JN; j++) {
        if (j0 + j < steps) {
            const floatx4 a = *(lptr4)(in + c * stride + 16 * (j0 + j) + 4 * g);
            a0 = mfma16(a[0], b[j][0], a0); a1 = mfma16(a[1], b[j][1], a1);
            a0 = mfma16(a[2], b[j][2], a0); a1 = mfma16(a[3], b[j][3], a1);
        }
    }
}

// profiling builds (-DRLT_WIDE_PROFILE): thread 0 of workgroup 0 notes the constant-rate clock at the stage boundaries, rlt_sac_wide_ticks copies the notes out
#ifdef RLT_WIDE_PROFILE
__device__ unsigned long long rlt_wide_ticks[2][32];
#define RLT_TICK(i) do { if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) rlt_wide_ticks[MODE & 1][i] = wall_clock64(); } while (0)
#else
#define RLT_TICK(i) do {} while (0)
#endif

// A wavefront's weight operands of one network: its 16 units' rows of W1 and W2 (the B operands of layers 1 and 2), row c of W3 for its 16 units, its lane's biases
template <int NT1C>
struct Operands { floatx4 w1[NT1C], w2a[8], w2b[8], w3; float b1, b2; };
__device__ __forceinline__ floatx4 load_w3(const WNet& N, int wave, int c, int g) {
    floatx4 w3 = {0.f, 0.f, 0.f, 0.f};
    if (c < N.out) {      // row c of W3 (c < out), this wavefront's 16 units
        const int k = 16 * wave + 4 * g;
        const float* row = N.W3 + (size_t)c * N.hid;
        if (N.vec3 && k + 3 < N.hid) w3 = *reinterpret_cast<const floatx4*>(row + k);
        else { if (k < N.hid) w3[0] = row[k]; if (k + 1 < N.hid) w3[1] = row[k + 1]; if (k + 2 < N.hid) w3[2] = row[k + 2]; if (k + 3 < N.hid) w3[3] = row[k + 3]; }
    }
    return w3;
}
// everything of network N that forward3 reads from memory, requested at once (few first-layer operands leave room for the whole second layer; otherwise its second
// half is requested after the first layer has run)
template <int NT1C>
__device__ __forceinline__ void load_operands(const WNet& N, int wave, int c, int g, Operands<NT1C>& W) {
    const int n = 16 * wave + c;
    if (wave < ((N.hid + 15) >> 4)) {
        load_rows<NT1C>(N.W1, N.in, N.hid, N.vec1, n, g, 0, W.w1);
        const int tiles = (N.hid + 15) >> 4, lane = c + 16 * g;
        load_swizzled<8>(N.W2f, tiles, wave, lane, 0, W.w2a);
        if (NT1C <= 2) load_swizzled<8>(N.W2f, tiles, wave, lane, 8, W.w2b);
        W.b1 = n < N.hid ? N.b1[n] : 0.f; W.b2 = n < N.hid ? N.b2[n] : 0.f;
        W.w3 = load_w3(N, wave, c, g);
    }
}

// The three layers of network N on the workgroup's rows x [16][xstride]: this wavefront's tile of h1 and h2 (after the activation) into
// LDS, then its units' share of the output layer's reduction into yp[wave]. Three workgroup barriers, which every wavefront meets; after
// the last one output_tile() returns the output layer's sums (without the bias).
// The operands W are in registers (or on their way) when the call starts. With PREFETCH each group of them is requested again for network `next` as soon as this
// network has used it, so that the next forward3 finds its operands loaded: a wavefront's weights are 16 KB per layer from L2, a compute unit's 256 KB, which
// took as long as the layers' arithmetic when they were requested at the start of each pass.
// First layers of more than two chunks fill too many registers for that: then only the second layer's first half (and the small operands) are requested ahead, the
// first layer's own operands at the start of the pass (W1_READY = false) and the second half after the first layer, as before.
template <int ACT_H, int NT1C, bool PREFETCH, bool W1_READY>
__device__ __forceinline__ void forward3(const WNet& N, Operands<NT1C>& W, const WNet& next, lptr x, int xstride, lptr h1, lptr h2, lptr yp, int wave, int c, int g, int tick = -1) {
#ifdef RLT_WIDE_PROFILE
#define FT(i) do { if (tick >= 0 && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) rlt_wide_ticks[0][tick + i] = wall_clock64(); } while (0)
#else
#define FT(i) do {} while (0)
#endif
    const int HID = N.hid, n = 16 * wave + c, tiles = (HID + 15) >> 4;
    const bool on = wave < tiles, n_ok = n < HID;
    const int n_next = 16 * wave + c;
    const bool next_on = PREFETCH && wave < ((next.hid + 15) >> 4);
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    if (on) {
        if (!W1_READY) load_rows<NT1C>(N.W1, N.in, HID, N.vec1, n, g, 0, W.w1);
        floatx4 a0 = zero4, a1 = zero4;
        FT(0);
        chunks<NT1C>(a0, a1, x, xstride, c, g, 0, (N.in + 15) >> 4, W.w1);
        FT(1);
        const floatx4 acc = a0 + a1;
#pragma unroll
        for (int v = 0; v < 4; v++) h1[(4 * g + v) * S + n] = n_ok ? act_hidden<ACT_H>(acc[v] + W.b1, N.act_h) : 0.f;
        if (NT1C > 2) load_swizzled<8>(N.W2f, tiles, wave, c + 16 * g, 8, W.w2b);
    }
    if (next_on) {
        if (NT1C <= 2) load_rows<NT1C>(next.W1, next.in, next.hid, next.vec1, n_next, g, 0, W.w1);
        W.b1 = n_next < next.hid ? next.b1[n_next] : 0.f;
    }
    FT(2);
    rlt_lds_barrier();
    FT(3);
    {
        floatx4 a0 = zero4, a1 = zero4;
        if (on) chunks<8>(a0, a1, h1, S, c, g, 0, tiles, W.w2a);
        if (next_on) load_swizzled<8>(next.W2f, (next.hid + 15) >> 4, wave, c + 16 * g, 0, W.w2a);
        FT(4);
        if (on) chunks<8>(a0, a1, h1, S, c, g, 8, tiles, W.w2b);
        if (next_on && NT1C <= 2) load_swizzled<8>(next.W2f, (next.hid + 15) >> 4, wave, c + 16 * g, 8, W.w2b);
        FT(5);
        if (on) {
            const floatx4 acc = a0 + a1;
#pragma unroll
            for (int v = 0; v < 4; v++) h2[(4 * g + v) * S + n] = n_ok ? act_hidden<ACT_H>(acc[v] + W.b2, N.act_h) : 0.f;
        }
        if (next_on) W.b2 = n_next < next.hid ? next.b2[n_next] : 0.f;
    }
    FT(6);
    rlt_lds_barrier();
    FT(7);
    if (on) {
        const floatx4 a = *(lptr4)(h2 + c * S + 16 * wave + 4 * g);
        floatx4 y = zero4;
        y = mfma16(a[0], W.w3[0], y); y = mfma16(a[1], W.w3[1], y); y = mfma16(a[2], W.w3[2], y); y = mfma16(a[3], W.w3[3], y);
#pragma unroll
        for (int v = 0; v < 4; v++) yp[(wave * ROWS + 4 * g + v) * D3S + c] = y[v];
    }
    if (next_on) W.w3 = load_w3(next, wave, c, g);
    rlt_lds_barrier();
}
// The same three layers for a pass that requests its own operands when it starts (the actor update: its passes are separated by the head and the critics' backward
// passes, which need the registers)
// KEEP: the hidden layers' pre-activations and outputs are also stored to memory, rows [row0, row0 + 16) of [batch x hid] arrays (forward() of a network keeps them)
struct KeepArgs { float* pre[2]; float* out[2]; int row0, batch; };
template <int ACT_H, int NT1C, bool KEEP = false>
__device__ __forceinline__ void forward3_own_loads(const WNet& N, lptr x, int xstride, lptr h1, lptr h2, lptr yp, int wave, int c, int g, const KeepArgs* keep = nullptr) {
    const int HID = N.hid, n = 16 * wave + c, tiles = (HID + 15) >> 4;
    const bool on = wave < tiles, n_ok = n < HID;
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    floatx4 w2a[8], w2b[8], w3 = zero4;
    float b1 = 0.f, b2 = 0.f;
    if (on) {
        floatx4 w1[NT1C];
        load_rows<NT1C>(N.W1, N.in, HID, N.vec1, n, g, 0, w1);
        load_swizzled<8>(N.W2f, tiles, wave, c + 16 * g, 0, w2a);      // on their way while the first layer runs
        if (NT1C <= 2) load_swizzled<8>(N.W2f, tiles, wave, c + 16 * g, 8, w2b);      // few first-layer operands: room for the whole second layer at once
        if (n_ok) { b1 = N.b1[n]; b2 = N.b2[n]; }
        // the output layer's operands: row c of W3 (c < out), this wavefront's 16 units
        if (c < N.out) {
            const int k = 16 * wave + 4 * g;
            const float* row = N.W3 + (size_t)c * HID;
            if (N.vec3 && k + 3 < HID) w3 = *reinterpret_cast<const floatx4*>(row + k);
            else { if (k < HID) w3[0] = row[k]; if (k + 1 < HID) w3[1] = row[k + 1]; if (k + 2 < HID) w3[2] = row[k + 2]; if (k + 3 < HID) w3[3] = row[k + 3]; }
        }
        floatx4 a0 = zero4, a1 = zero4;
        chunks<NT1C>(a0, a1, x, xstride, c, g, 0, (N.in + 15) >> 4, w1);
        const floatx4 acc = a0 + a1;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float pre = acc[v] + b1, o = act_hidden<ACT_H>(pre, N.act_h);
            h1[(4 * g + v) * S + n] = n_ok ? o : 0.f;
            if (KEEP && n_ok && keep->row0 + 4 * g + v < keep->batch) {
                const size_t at = (size_t)(keep->row0 + 4 * g + v) * HID + n;
                if (keep->pre[0]) keep->pre[0][at] = pre;
                if (keep->out[0]) keep->out[0][at] = o;
            }
        }
        if (NT1C > 2) load_swizzled<8>(N.W2f, tiles, wave, c + 16 * g, 8, w2b);
    }
    rlt_lds_barrier();
    if (on) {
        floatx4 a0 = zero4, a1 = zero4;
        chunks<8>(a0, a1, h1, S, c, g, 0, tiles, w2a);
        chunks<8>(a0, a1, h1, S, c, g, 8, tiles, w2b);
        const floatx4 acc = a0 + a1;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float pre = acc[v] + b2, o = act_hidden<ACT_H>(pre, N.act_h);
            h2[(4 * g + v) * S + n] = n_ok ? o : 0.f;
            if (KEEP && n_ok && keep->row0 + 4 * g + v < keep->batch) {
                const size_t at = (size_t)(keep->row0 + 4 * g + v) * HID + n;
                if (keep->pre[1]) keep->pre[1][at] = pre;
                if (keep->out[1]) keep->out[1][at] = o;
            }
        }
    }
    rlt_lds_barrier();
    if (on) {
        const floatx4 a = *(lptr4)(h2 + c * S + 16 * wave + 4 * g);
        floatx4 y = zero4;
        y = mfma16(a[0], w3[0], y); y = mfma16(a[1], w3[1], y); y = mfma16(a[2], w3[2], y); y = mfma16(a[3], w3[3], y);
#pragma unroll
        for (int v = 0; v < 4; v++) yp[(wave * ROWS + 4 * g + v) * D3S + c] = y[v];
    }
    rlt_lds_barrier();
}
// the sums of the partial tiles, in wavefront order: element v of lane (c, g) belongs to row 4 g + v, column c
__device__ __forceinline__ floatx4 output_tile(lptr yp, int tiles, int c, int g) {
    floatx4 y = {0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < tiles; w++)
#pragma unroll
        for (int v = 0; v < 4; v++) y[v] += yp[(w * ROWS + 4 * g + v) * D3S + c];
    return y;
}

// this wavefront's tile of d_pre2 = (d_pre3 W3) f'(h2) into g2 (may be h2 itself); returns the lane's share of its unit's column sum
template <int ACT_H>
__device__ __forceinline__ float backward_layer3(const WNet& N, lptr d3, lptr h2, lptr g2, int wave, int c, int g) {
    const int n = 16 * wave + c;
    const bool n_ok = n < N.hid;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < MAX_OUT / 4; ks++) {
        const int o = 4 * ks + g;
        const float w = (o < N.out && n_ok) ? N.W3[(size_t)o * N.hid + n] : 0.f;
        acc = mfma16(d3[c * D3S + 4 * ks + g], w, acc);      // columns of d_pre3 beyond the output width are zero
    }
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int idx = (4 * g + v) * S + n;
        const float dp = n_ok ? acc[v] * dact_hidden<ACT_H>(h2[idx], N.act_h) : 0.f;
        g2[idx] = dp; sum += dp;
    }
    return sum;
}
// this wavefront's tile of d_pre1 = (d_pre2 W2) f'(h1) into p1 (may be h1 itself); returns the lane's share of its unit's column sum
template <int ACT_H>
__device__ __forceinline__ float backward_layer2(const WNet& N, lptr g2, lptr h1, lptr p1, int wave, int c, int g) {
    const int HID = N.hid, n = 16 * wave + c, tiles = (HID + 15) >> 4;
    const bool n_ok = n < HID;
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    floatx4 a0 = zero4, a1 = zero4;
#pragma unroll 1
    for (int j0 = 0; j0 < tiles; j0 += 4) {
        floatx4 b[4];
        load_swizzled<4>(N.W2b, tiles, wave, c + 16 * g, j0, b);      // W2[16 j + 4 g + i][n]
        chunks<4>(a0, a1, g2, S, c, g, j0, tiles, b);
    }
    const floatx4 acc = a0 + a1;
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int idx = (4 * g + v) * S + n;
        const float dp = n_ok ? acc[v] * dact_hidden<ACT_H>(h1[idx], N.act_h) : 0.f;
        p1[idx] = dp; sum += dp;
    }
    return sum;
}

// The copies of the second layers' weights that load_swizzled reads, made anew before every update (the optimisers change the weights between them): thread t of
// block (x, job) writes the 16 bytes of lane t % 64 of one (wavefront, chunk) pair. Forward copies read 16 consecutive bytes of a row of W2, backward copies four
// values a row apart (the 16 lanes of a group read 64 consecutive bytes each time).
constexpr int PREP_JOBS = 8;
struct PrepArgs { const float* W2[PREP_JOBS]; float* dst[PREP_JOBS]; int hid[PREP_JOBS]; int backward[PREP_JOBS]; };
__global__ __launch_bounds__(256) void wide_prepare_kernel(PrepArgs P) {
    const int job = blockIdx.y, HID = P.hid[job], tiles = (HID + 15) >> 4;
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= tiles * tiles * 64) return;
    const int lane = t & 63, pair = t >> 6, w = pair / tiles, j = pair - w * tiles, c = lane & 15, g = lane >> 4;
    const int n = 16 * w + c, k = 16 * j + 4 * g;
    const float* W = P.W2[job];
    floatx4 v = {0.f, 0.f, 0.f, 0.f};
    if (n < HID) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (k + i < HID) v[i] = P.backward[job] ? W[(size_t)(k + i) * HID + n] : W[(size_t)n * HID + k + i];
    }
    *reinterpret_cast<floatx4*>(P.dst[job] + (size_t)t * 4) = v;
}

template <int MODE, int ACT_H, int NT1C>
__global__ __launch_bounds__(THREADS) void sac_wide_kernel(WideArgs A) {
    constexpr bool CRITIC = MODE == MODE_CRITIC || MODE == MODE_TD3_CRITIC, TD3 = MODE == MODE_TD3_CRITIC || MODE == MODE_TD3_ACTOR;
    extern __shared__ __attribute__((aligned(16))) float lds_wide[];
    if (A.packed && (blockIdx.x & 7)) return;
    const int gi = A.packed ? blockIdx.x >> 3 : blockIdx.x, G = A.packed ? gridDim.x >> 3 : gridDim.x;
    const int y = CRITIC ? blockIdx.y : 0;
    const int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool scalar_wave = wave == 0;
    const int OBS = A.obs, ACT = A.act, D = OBS + ACT, B = A.batch;
    const lptr xa = (lptr)lds_wide, xb = xa + ROWS * SXS, h1 = xb + ROWS * SXS, h2 = h1 + ROWS * S, ta = h2 + ROWS * S, tb = ta + ROWS * S,
               d3 = tb + ROWS * S, d3c = d3 + ROWS * D3S, da = d3c + ROWS * D3S, yp = da + 2 * ROWS * D3S, misc = yp + WAVES * YP;
    const int row0 = gi * ROWS;
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const WNet trained = CRITIC ? (y ? A.critic[1] : A.critic[0]) : A.actor;      // by value: an index into the kernel's argument would keep all of it in private memory
    const int HID = trained.hid, tiles = (HID + 15) >> 4;
    const bool on = wave < tiles;

    // the input tiles: xa = next rows (critic update) or current rows (actor update; the actor reads its observation columns), xb = current rows
    for (int e = threadIdx.x; e < ROWS * SXS; e += THREADS) {
        const int r = e / SXS, k = e % SXS;
        const bool ok = row0 + r < B && k < D;
        const float* cur = A.batch_base + (size_t)min(row0 + r, B - 1) * D + min(k, D - 1);
        if (CRITIC) { xa[e] = ok ? cur[(size_t)B * D] : 0.f; xb[e] = ok ? cur[0] : 0.f; }
        else xa[e] = (ok && k < OBS) ? cur[0] : 0.f;
    }
    float noise[2] = {0.f, 0.f}, target_noise[2] = {0.f, 0.f}, reward[4] = {0.f, 0.f, 0.f, 0.f}, alpha = 0.f, s3 = 0.f, extra = 0.f;
    bool terminated[4] = {false, false, false, false};
    if (scalar_wave) {
        if (!TD3) alpha = expf(*A.log_alpha);
        if (MODE == MODE_TD3_CRITIC) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                if (g + 4 * j < ACT && row0 + c < B) {
                    const size_t i = (size_t)(row0 + c) * ACT + g + 4 * j;
                    if (A.target_noise) target_noise[j] = A.target_noise[i];
                    else {
                        const float scaled = rlt_randn_element(A.noise_seed, A.target_noise_stream + *A.stream_offset, i) * A.target_noise_std + 0.0f;
                        target_noise[j] = clampf(scaled, -A.target_noise_clip, A.target_noise_clip);
                        if (y == 0) A.out_target_noise[i] = target_noise[j];
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if (g + 4 * j < ACT && row0 + c < B) {
                const size_t i = (size_t)(row0 + c) * ACT + g + 4 * j;
                const float* const given = (MODE == MODE_TD3_CRITIC && y) ? A.noise_second : A.noise;
                noise[j] = given ? given[i] : rlt_randn_element(A.noise_seed, ((MODE == MODE_TD3_CRITIC && y) ? A.noise_stream_second : A.noise_stream) + *A.stream_offset, i);
                if (A.out_noise && y == 0) A.out_noise[i] = noise[j];
            }
        }
        if (CRITIC) {
#pragma unroll
            for (int v = 0; v < 4; v++) { const int row = min(row0 + 4 * g + v, B - 1); reward[v] = A.rewards[row]; terminated[v] = A.terminated[row] != 0; }
        }
    }
    HeadItem item[2];
    const bool row_ok = row0 + c < B;
    Operands<NT1C> W;
    if (CRITIC) load_operands<NT1C>(A.actor, wave, c, g, W);      // on their way while the input tiles are written
    RLT_TICK(0);
    rlt_lds_barrier();      // the input tiles are in place
    RLT_TICK(1);

    // the actor (critic update: on the next observations; actor update: on the observations, activations kept for its backward pass)
    if (CRITIC) forward3<ACT_H, NT1C, true, true>(A.actor, W, A.target[0], xa, SXS, ta, tb, yp, wave, c, g);
    else forward3_own_loads<ACT_H, NT1C>(A.actor, xa, SXS, h1, h2, yp, wave, c, g);
    RLT_TICK(2);
    if (scalar_wave) {
        const floatx4 out = output_tile(yp, (A.actor.hid + 15) >> 4, c, g);
        const float b3 = c < A.actor.out ? A.actor.b3[c] : 0.f;
#pragma unroll
        for (int v = 0; v < 4; v++) d3[(4 * g + v) * D3S + c] = c < A.actor.out ? out[v] + b3 : 0.f;
        wave_sync();
        float log_prob = 0.f;
        if (TD3) td3_head_forward(OBS, ACT, A.sampling_std, d3, D3S, xa, SXS, noise, target_noise, CRITIC, c, g, item);
        else log_prob = head_forward(A.sas, OBS, ACT, d3, D3S, xa, SXS, noise, c, g, item);
        if (TD3) {
            if (!CRITIC && row_ok && A.out_pre_clip) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    if (g + 4 * j < ACT) A.out_pre_clip[(size_t)(row0 + c) * ACT + g + 4 * j] = item[j].sample;
            }
        } else if (g == 0) {
            if (CRITIC) misc[c] = log_prob;
            if (A.out_log_probabilities && row_ok) A.out_log_probabilities[row0 + c] = log_prob;
        }
        if (!TD3 && !CRITIC && row_ok) {
#pragma unroll
            for (int j = 0; j < 2; j++)
                if (g + 4 * j < ACT) {
                    if (A.out_actions) A.out_actions[(size_t)(row0 + c) * ACT + g + 4 * j] = item[j].action;
                    if (A.out_pre_squashing) A.out_pre_squashing[(size_t)(row0 + c) * ACT + g + 4 * j] = item[j].sample;
                }
        }
    }
    rlt_lds_barrier();      // the action columns of xa are in place
    RLT_TICK(3);

    if (CRITIC) {
        // both target critics on [next observation | sampled action], then the trained critic on the current rows
        floatx4 q_next[2];
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const WNet T = k ? A.target[1] : A.target[0];
            const WNet after = k ? trained : A.target[1];
            forward3<ACT_H, NT1C, true, NT1C <= 2>(T, W, after, xa, SXS, ta, tb, yp, wave, c, g, k == 0 && CRITIC ? 20 : -1);
            RLT_TICK(4 + k);
            if (scalar_wave) { q_next[k] = output_tile(yp, (T.hid + 15) >> 4, c, g); const float b3 = T.b3[0]; for (int v = 0; v < 4; v++) q_next[k][v] += b3; }
        }
        forward3<ACT_H, NT1C, false, NT1C <= 2>(trained, W, trained, xb, SXS, h1, h2, yp, wave, c, g);
        RLT_TICK(6);
        if (scalar_wave) {
            // TD target of rows 4 g + v (meaningful in the lanes c == 0, which hold output 0), MSE gradient at the critic's pre-activation:
            // loss weight batch * 0.5 / n with n = batch rows (no masks), times the MSE gradient's 2 / batch (rl/algorithms/sac/operations_generic.h:298-316)
            const floatx4 yc = output_tile(yp, tiles, c, g);
            const float b3 = trained.b3[0];
            // (TD3: loss weight batch / n, rl/algorithms/td3/operations_generic.h:200-212)
            const float loss_weight = TD3 ? (float)B / (float)B : (1.0f / (float)B) * ((float)B * 0.5f);
            const float constant = 2.0f / (float)B * loss_weight;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float q_min = fminf(q_next[0][v], q_next[1][v]);
                const float min_q = TD3 ? q_min : q_min - alpha * misc[4 * g + v];
                const float future = (terminated[v] && !(TD3 && A.ignore_termination)) ? 0.0f : A.gamma * min_q;
                const float y_target = reward[v] + future;
                const bool ok = c == 0 && row0 + 4 * g + v < B;
                // (SAC's critics share their targets; TD3's are formed with each critic's own sampling noise: the last critic's stay, as after two calls)
                if (A.out_target_action_value && ok && y == (TD3 ? (int)gridDim.y - 1 : 0)) A.out_target_action_value[row0 + 4 * g + v] = y_target;
                const float diff = (yc[v] + b3) - y_target;
                const float dp = ok ? diff * constant : 0.f;
                if (ok) extra += diff * diff;
                s3 += dp;
                d3[(4 * g + v) * D3S + c] = dp;
            }
        }
        rlt_lds_barrier();      // d_pre3 is in place
        RLT_TICK(7);
    } else {
        // each critic (TD3: critic 0 only, rl/algorithms/td3/operations_generic.h:260): value on [observation | sampled action], then the gradient of -value / batch
        // with respect to the action
        const float loss_weight = (1.0f / (float)B) * -1.0f;       // rl/algorithms/sac/operations_generic.h:437-453 with n = batch rows
#pragma unroll 1
        for (int k = 0; k < (TD3 ? 1 : 2); k++) {
            const WNet C = k ? A.critic[1] : A.critic[0];
            const int ctiles = (C.hid + 15) >> 4;
            forward3_own_loads<ACT_H, NT1C>(C, xa, SXS, ta, tb, yp, wave, c, g);
            RLT_TICK(4 + 4 * k);
            if (scalar_wave) {
                const floatx4 out = output_tile(yp, ctiles, c, g);
                const float b3 = C.b3[0];
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    if (c == 0) misc[16 * k + 4 * g + v] = out[v] + b3;
                    d3c[(4 * g + v) * D3S + c] = (c == 0 && row0 + 4 * g + v < B) ? loss_weight : 0.f;
                }
            }
            rlt_lds_barrier();
            if (wave < ctiles) backward_layer3<ACT_H>(C, d3c, tb, tb, wave, c, g);
            rlt_lds_barrier();
            RLT_TICK(5 + 4 * k);
            if (wave < ctiles) {
                backward_layer2<ACT_H>(C, tb, ta, ta, wave, c, g);
                wave_sync();
                // d value / d action = the action columns of d_pre1 W1: this wavefront's units' share of the reduction
                floatx4 acc = zero4;
                const floatx4 a = *(lptr4)(ta + c * S + 16 * wave + 4 * g);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int unit = 16 * wave + 4 * g + i;
                    const float w = (c < ACT && unit < C.hid) ? C.W1[(size_t)unit * D + OBS + c] : 0.f;
                    acc = mfma16(a[i], w, acc);
                }
#pragma unroll
                for (int v = 0; v < 4; v++) yp[(wave * ROWS + 4 * g + v) * D3S + c] = acc[v];
            }
            rlt_lds_barrier();
            RLT_TICK(6 + 4 * k);
            if (scalar_wave) {
                const floatx4 out = output_tile(yp, ctiles, c, g);
#pragma unroll
                for (int v = 0; v < 4; v++) da[(k * ROWS + 4 * g + v) * D3S + c] = out[v];
            }
        }
        if (scalar_wave) {
            // sample_and_squash backward on the gradient of the smaller value; TD3: the td3_sampling layer's backward (zero where the sample was clamped,
            // nn/layers/td3_sampling/operations_generic.h:139-163) and the derivative of the actor's tanh output
            wave_sync();
            const lptr dak = da + ((TD3 || misc[c] < misc[16 + c]) ? 0 : 1) * ROWS * D3S + c * D3S;
#pragma unroll
            for (int v = 0; v < 4; v++) d3[(4 * g + v) * D3S + c] = 0.f;
            wave_sync();
            const float alpha_over_b = alpha / (float)B;
            float entropy = 0.f;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int a = g + 4 * j;
                if (a < ACT) {
                    if (TD3) {
                        const float d_mean = (item[j].sample < -1.0f || item[j].sample > 1.0f) ? 0.0f : dak[a];
                        if (row_ok) d3[c * D3S + a] = d_mean * (1.0f - item[j].mean * item[j].mean);
                        continue;
                    }
                    float d_mu, d_ls;
                    head_backward(A.sas, item[j], dak[a], alpha_over_b, d_mu, d_ls, entropy);
                    if (row_ok) { d3[c * D3S + a] = d_mu; d3[c * D3S + ACT + a] = d_ls; }
                }
            }
            entropy = groups_sum(entropy);
            // d log_alpha: sum over the rows of alpha (entropy - target entropy), divided by the batch size by the reduction
            const float per_row = (g == 0 && row_ok) ? alpha * (entropy - A.sas.target_entropy) : 0.f;
            const float tile_sum = row16_sum(per_row);
            if (lane == 0) extra += tile_sum;
            wave_sync();
#pragma unroll
            for (int v = 0; v < 4; v++) s3 += d3[(4 * g + v) * D3S + c];
        }
        rlt_lds_barrier();      // d_pre3 is in place
        RLT_TICK(12);
    }

    // backward pass of the trained network with its weight gradients over the workgroup's 16 rows; h1, h2: its hidden activations,
    // d3: the gradient at its last pre-activation; ta receives d_pre2, tb receives d_pre1
    float* dst = A.partial + ((size_t)y * G + gi) * A.count;
    const int IN = trained.in, OUT = trained.out, NT1 = (IN + 15) >> 4;
    const int o_b1 = HID * IN, o_w2 = o_b1 + HID, o_b2 = o_w2 + HID * HID, o_w3 = o_b2 + HID, o_b3 = o_w3 + OUT * HID, o_ex = o_b3 + OUT;
    const lptr xt = CRITIC ? xb : xa;
    const int n = 16 * wave + c;
    const bool n_ok = n < HID;
    float s2 = 0.f;
    if (on) {
        floatx4 aW3 = zero4;
#pragma unroll
        for (int ks = 0; ks < ROWS / 4; ks++) aW3 = mfma16(d3[(4 * ks + g) * D3S + c], h2[(4 * ks + g) * S + n], aW3);
#pragma unroll
        for (int v = 0; v < 4; v++)
            if (4 * g + v < OUT && n_ok) dst[o_w3 + (4 * g + v) * HID + n] = aW3[v];
        s2 = backward_layer3<ACT_H>(trained, d3, h2, ta, wave, c, g);
    }
    rlt_lds_barrier();      // every wavefront's tile of d_pre2 is in place
    RLT_TICK(13);
    if (on) {
        {   // dW2: this wavefront's units' rows
            float a[4];
#pragma unroll
            for (int ks = 0; ks < 4; ks++) a[ks] = ta[(4 * ks + g) * S + n];
#pragma unroll 4
            for (int nt = 0; nt < tiles; nt++) {
                floatx4 acc = zero4;
#pragma unroll
                for (int ks = 0; ks < 4; ks++) acc = mfma16(a[ks], h1[(4 * ks + g) * S + 16 * nt + c], acc);
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int m = 16 * wave + 4 * g + v;
                    if (m < HID && 16 * nt + c < HID) dst[o_w2 + (size_t)m * HID + 16 * nt + c] = acc[v];
                }
            }
        }
        RLT_TICK(14);
        float s1 = backward_layer2<ACT_H>(trained, ta, h1, tb, wave, c, g);
        RLT_TICK(15);
        wave_sync();            // dW1's rows are this wavefront's own tile of d_pre1
        {
            float a[4];
#pragma unroll
            for (int ks = 0; ks < 4; ks++) a[ks] = tb[(4 * ks + g) * S + n];
#pragma unroll 2
            for (int nt = 0; nt < NT1; nt++) {
                floatx4 acc = zero4;
#pragma unroll
                for (int ks = 0; ks < 4; ks++) acc = mfma16(a[ks], xt[(4 * ks + g) * SXS + 16 * nt + c], acc);
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int m = 16 * wave + 4 * g + v;
                    if (m < HID && 16 * nt + c < IN) dst[(size_t)m * IN + 16 * nt + c] = acc[v];
                }
            }
        }
        s1 = groups_sum(s1); s2 = groups_sum(s2);
        if (g == 0 && n_ok) { dst[o_b1 + n] = s1; dst[o_b2 + n] = s2; }
    }
    if (scalar_wave) {
        s3 = groups_sum(s3); extra = groups_sum(extra);
        if (g == 0) {
            if (c < OUT) dst[o_b3 + c] = s3;
            dst[o_ex + c] = extra;
        }
    }
    RLT_TICK(16);
}

constexpr size_t LDS_FLOATS = (size_t)2 * ROWS * SXS + 4 * ROWS * S + 4 * ROWS * D3S + WAVES * YP + MISC;

// ---- Forward and backward pass of one three-layer network over a few thousand rows at most, on the same machinery (nn_models/mlp/operations_generic.h:103-204: forward, the
// loss gradient given or formed from a target as the MSE's, backward with weight gradients): a workgroup takes 16 rows through the three layers and back, the activations
// never leave LDS, and writes one block of partial sums [dW1 | db1 | dW2 | db2 | dW3 | db3]; mlp_wide_reduce_kernel adds the blocks up in workgroup order onto the layers'
// gradients. Where a batch is too small to fill the chip with the 64-row tiles of the one-pass kernel for large batches (mlp_fused.hip: 4,096 rows are 64 tiles for 256
// compute units, and a tile takes its 74 us whatever the batch), sixteen-row tiles are a launch of 256 workgroups.
struct MlpWideArgs {
    WNet net;
    const float* x; int ldx; float* y; int ldy;
    const float* d_output; int ldd; const float* target; int ldt; float mse_scale;
    int batch;
    float* partial; int count;
    const float* out1; const float* out2;      // MLP_BACKWARD: the outputs of layers 1 and 2 that a forward() left in memory, [batch x hid] each; d_output is then the gradient at the last pre-activations
    float* keep_pre[3]; float* keep_out[3]; int act3;      // MLP_FORWARD: every layer's pre-activations and outputs as forward() keeps them (each may be NULL); the last layer's activation
};
enum { MLP_FORWARD_BACKWARD = 0, MLP_BACKWARD = 1, MLP_FORWARD = 2 };
template <int ACT_H, int NT1C, int PASS>
__global__ __launch_bounds__(THREADS) void mlp_wide_kernel(MlpWideArgs A) {
    constexpr bool BACKWARD_ONLY = PASS == MLP_BACKWARD;
    extern __shared__ __attribute__((aligned(16))) float lds_wide[];
    const int gi = blockIdx.x;
    const int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const lptr xa = (lptr)lds_wide, h1 = xa + 2 * ROWS * SXS, h2 = h1 + ROWS * S, ta = h2 + ROWS * S, tb = ta + ROWS * S, d3 = tb + ROWS * S, yp = d3 + 4 * ROWS * D3S;
    const WNet N = A.net;
    const int B = A.batch, IN = N.in, HID = N.hid, OUT = N.out, tiles = (HID + 15) >> 4, row0 = gi * ROWS;
    const bool on = wave < tiles;
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    for (int e = threadIdx.x; e < ROWS * SXS; e += THREADS) {
        const int r = e / SXS, k = e % SXS;
        xa[e] = (row0 + r < B && k < IN) ? A.x[(size_t)(row0 + r) * A.ldx + k] : 0.f;
    }
    if (BACKWARD_ONLY) {
        // the hidden activations come back from memory (zero beyond the batch and beyond the width, up to the multiple of 16 that the tiles run to)
        const int HP = 16 * tiles;
        for (int e = threadIdx.x; e < ROWS * HP; e += THREADS) {
            const int r = e / HP, k = e - r * HP;
            const bool ok = row0 + r < B && k < HID;
            h1[r * S + k] = ok ? A.out1[(size_t)(row0 + r) * HID + k] : 0.f;
            h2[r * S + k] = ok ? A.out2[(size_t)(row0 + r) * HID + k] : 0.f;
        }
    }
    rlt_lds_barrier();
    if (PASS == MLP_FORWARD) {
        const KeepArgs keep = {{A.keep_pre[0], A.keep_pre[1]}, {A.keep_out[0], A.keep_out[1]}, row0, B};
        forward3_own_loads<ACT_H, NT1C, true>(N, xa, SXS, h1, h2, yp, wave, c, g, &keep);
        if (wave == 0) {
            const floatx4 out = output_tile(yp, tiles, c, g);
            const float b3 = c < OUT ? N.b3[c] : 0.f;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = row0 + 4 * g + v;
                if (c < OUT && row < B) {
                    const float pre = out[v] + b3;
                    if (A.keep_pre[2]) A.keep_pre[2][(size_t)row * OUT + c] = pre;
                    const float o = rlt_act(pre, A.act3);
                    if (A.keep_out[2]) A.keep_out[2][(size_t)row * OUT + c] = o;
                    if (A.y) A.y[(size_t)row * A.ldy + c] = o;
                }
            }
        }
        return;
    }
    if (PASS == MLP_FORWARD_BACKWARD) forward3_own_loads<ACT_H, NT1C>(N, xa, SXS, h1, h2, yp, wave, c, g);
    float s3 = 0.f;
    if (BACKWARD_ONLY) {
        if (wave == 0) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = row0 + 4 * g + v;
                const float d = (c < OUT && row < B) ? A.d_output[(size_t)row * A.ldd + c] : 0.f;
                d3[(4 * g + v) * D3S + c] = d;
                s3 += d;
            }
        }
    } else if (wave == 0) {
        // lane (c, g): output column c of rows 4 g + v; the gradient at the output (the last layer has no activation): given, or the MSE's against the target
        const floatx4 out = output_tile(yp, tiles, c, g);
        const float b3 = c < OUT ? N.b3[c] : 0.f;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = row0 + 4 * g + v;
            const bool ok = c < OUT && row < B;
            const float yv = out[v] + b3;
            if (ok && A.y) A.y[(size_t)row * A.ldy + c] = yv;
            float d = 0.f;
            if (ok) d = A.target ? (yv - A.target[(size_t)row * A.ldt + c]) * A.mse_scale : A.d_output[(size_t)row * A.ldd + c];
            d3[(4 * g + v) * D3S + c] = d;
            s3 += d;
        }
    }
    rlt_lds_barrier();      // d_pre3 is in place
    // backward pass with the weight gradients over the workgroup's 16 rows: ta receives d_pre2, tb receives d_pre1
    float* dst = A.partial + (size_t)gi * A.count;
    const int NT1 = (IN + 15) >> 4;
    const int o_b1 = HID * IN, o_w2 = o_b1 + HID, o_b2 = o_w2 + HID * HID, o_w3 = o_b2 + HID, o_b3 = o_w3 + OUT * HID;
    const int n = 16 * wave + c;
    const bool n_ok = n < HID;
    float s2 = 0.f;
    if (on) {
        floatx4 aW3 = zero4;
#pragma unroll
        for (int ks = 0; ks < ROWS / 4; ks++) aW3 = mfma16(d3[(4 * ks + g) * D3S + c], h2[(4 * ks + g) * S + n], aW3);
#pragma unroll
        for (int v = 0; v < 4; v++)
            if (4 * g + v < OUT && n_ok) dst[o_w3 + (4 * g + v) * HID + n] = aW3[v];
        s2 = backward_layer3<ACT_H>(N, d3, h2, ta, wave, c, g);
    }
    rlt_lds_barrier();      // every wavefront's tile of d_pre2 is in place
    if (on) {
        {   // dW2: this wavefront's units' rows
            float a[4];
#pragma unroll
            for (int ks = 0; ks < 4; ks++) a[ks] = ta[(4 * ks + g) * S + n];
#pragma unroll 4
            for (int nt = 0; nt < tiles; nt++) {
                floatx4 acc = zero4;
#pragma unroll
                for (int ks = 0; ks < 4; ks++) acc = mfma16(a[ks], h1[(4 * ks + g) * S + 16 * nt + c], acc);
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int m = 16 * wave + 4 * g + v;
                    if (m < HID && 16 * nt + c < HID) dst[o_w2 + (size_t)m * HID + 16 * nt + c] = acc[v];
                }
            }
        }
        float s1 = backward_layer2<ACT_H>(N, ta, h1, tb, wave, c, g);
        wave_sync();            // dW1's rows are this wavefront's own tile of d_pre1
        {
            float a[4];
#pragma unroll
            for (int ks = 0; ks < 4; ks++) a[ks] = tb[(4 * ks + g) * S + n];
#pragma unroll 2
            for (int nt = 0; nt < NT1; nt++) {
                floatx4 acc = zero4;
#pragma unroll
                for (int ks = 0; ks < 4; ks++) acc = mfma16(a[ks], xa[(4 * ks + g) * SXS + 16 * nt + c], acc);
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int m = 16 * wave + 4 * g + v;
                    if (m < HID && 16 * nt + c < IN) dst[(size_t)m * IN + 16 * nt + c] = acc[v];
                }
            }
        }
        s1 = groups_sum(s1); s2 = groups_sum(s2);
        if (g == 0 && n_ok) { dst[o_b1 + n] = s1; dst[o_b2 + n] = s2; }
    }
    if (wave == 0) {
        s3 = groups_sum(s3);
        if (g == 0 && c < OUT) dst[o_b3 + c] = s3;
    }
}
// gradient[e] += the sum over the workgroups' blocks of element e, in workgroup order; thread = one element, sixteen blocks' loads in flight
struct WideReduceArgs { const float* partial; int blocks, count, total; float* dst[6]; int end[6]; };
__global__ __launch_bounds__(256) void mlp_wide_reduce_kernel(WideReduceArgs R) {
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= R.total) return;
    float sum = 0.f;
    for (int b0 = 0; b0 < R.blocks; b0 += 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; u++) v[u] = b0 + u < R.blocks ? R.partial[(size_t)(b0 + u) * R.count + e] : 0.f;
#pragma unroll
        for (int u = 0; u < 16; u++) sum += v[u];
    }
    int k = 0, begin = 0;
#pragma unroll
    for (int q = 0; q < 5; q++) if (e >= R.end[q]) { k = q + 1; begin = R.end[q]; }
    float* const dst = k == 0 ? R.dst[0] : k == 1 ? R.dst[1] : k == 2 ? R.dst[2] : k == 3 ? R.dst[3] : k == 4 ? R.dst[4] : R.dst[5];
    dst[e - begin] += sum;
}

bool hidden_ok(int a) { return a == RLT_ACT_RELU || a == RLT_ACT_TANH || a == RLT_ACT_FAST_TANH || a == RLT_ACT_SIGMOID; }
bool net_ok(const rlt_dense_layer* L, int n, int in, int out, int& hid, int last_activation = RLT_ACT_IDENTITY) {
    if (!L || n != 3) return false;
    for (int l = 0; l < 3; l++) if (!L[l].weights || !L[l].biases) return false;
    if (hid == 0) hid = L[0].out_dim;
    return hid >= 1 && hid <= MAX_H && L[0].in_dim == in && L[0].out_dim == hid && L[1].in_dim == hid && L[1].out_dim == hid && L[2].in_dim == hid && L[2].out_dim == out &&
           L[0].activation == L[1].activation && hidden_ok(L[0].activation) && L[2].activation == last_activation;
}
bool aligned16(const float* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
WNet net_of(const rlt_dense_layer* L) {
    const int in = L[0].in_dim, hid = L[0].out_dim;
    return {L[0].weights, L[0].biases, L[1].weights, L[1].biases, L[2].weights, L[2].biases, in, hid, L[2].out_dim, L[0].activation,
            in % 4 == 0 && aligned16(L[0].weights), hid % 4 == 0 && aligned16(L[1].weights), hid % 4 == 0 && aligned16(L[2].weights)};
}
int partial_count(int in, int hid, int out) { return hid * in + hid + hid * hid + hid + out * hid + out + N_EXTRA; }

// where each Adam tensor's gradient lies in a block of partial sums (a tensor may span several of the network's six gradient buffers
// where those follow each other in memory); false unless the tensors cover the six buffers exactly
bool map_gradients(const rlt_dense_layer* L, const rlt_adam_tensor* T, int n, uint32_t* offsets, int* first_segment, int* n_segments) {
    if (!T || n < 1 || n > RLT_TAIL_TENSORS) return false;
    const int hid = L[0].out_dim;
    const float* seg[6] = {L[0].d_weights, L[0].d_biases, L[1].d_weights, L[1].d_biases, L[2].d_weights, L[2].d_biases};
    const uint32_t size[6] = {(uint32_t)(hid * L[0].in_dim), (uint32_t)hid, (uint32_t)(hid * hid), (uint32_t)hid, (uint32_t)(L[2].out_dim * hid), (uint32_t)L[2].out_dim};
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
        offsets[i] = off[s]; first_segment[i] = s; n_segments[i] = k - s;
    }
    return covered == 63u;
}
float* parameter_segments(const rlt_dense_layer* L, int first, int count) {
    const int hid = L[0].out_dim;
    float* seg[6] = {L[0].weights, L[0].biases, L[1].weights, L[1].biases, L[2].weights, L[2].biases};
    const uint32_t size[6] = {(uint32_t)(hid * L[0].in_dim), (uint32_t)hid, (uint32_t)(hid * hid), (uint32_t)hid, (uint32_t)(L[2].out_dim * hid), (uint32_t)L[2].out_dim};
    uint32_t cnt = 0;
    for (int k = first; k < first + count; k++) { if (seg[k] != seg[first] + cnt) return nullptr; cnt += size[k]; }
    return seg[first];
}

struct Optimiser {
    const rlt_dense_layer* trained; const rlt_adam_tensor* tensors; int n_tensors; const rlt_adam_parameters* parameters; uint32_t* age;
    const rlt_adam_tensor* second; const rlt_adam_parameters* second_parameters; uint32_t* second_age; float second_scale;
    const rlt_dense_layer* soft_target;
};

// The optimisers' steps, as one launch after the update kernel that adds up the workgroups' blocks itself (16 blocks of 68 k floats at
// width 256: read through one compute unit each, as the update kernel's own last step, that costs 70 us; spread over the chip 10): both
// critics' optimisers share it, and a tensor's soft update of its target rides along where the layouts correspond.
struct Step { rlt_adam_tensor tensors[RLT_TAIL_TENSORS]; uint32_t offsets[RLT_TAIL_TENSORS]; float scales[RLT_TAIL_TENSORS]; bool targets_fused; };
bool describe_step(const Optimiser& O, Step& S) {
    int first[RLT_TAIL_TENSORS], count[RLT_TAIL_TENSORS];
    if (!map_gradients(O.trained, O.tensors, O.n_tensors, S.offsets, first, count)) return false;
    S.targets_fused = O.soft_target != nullptr;
    for (int i = 0; i < O.n_tensors; i++) {
        S.tensors[i] = O.tensors[i]; S.scales[i] = 1.0f;
        if (O.soft_target && (parameter_segments(O.trained, first[i], count[i]) != O.tensors[i].parameters || !(S.tensors[i].polyak_target = parameter_segments(O.soft_target, first[i], count[i])))) S.targets_fused = false;
    }
    if (!S.targets_fused) for (int i = 0; i < O.n_tensors; i++) S.tensors[i].polyak_target = nullptr;
    return true;
}

// false: the agent's Adam tensors are not its networks' gradient buffers; the caller takes the per-operation path
bool steps_describable(const Optimiser* opts, int n_opts) {
    Step S;
    for (int k = 0; k < n_opts; k++) {
        if (!describe_step(opts[k], S)) return false;
        if (opts[k].second && (opts[k].second->polyak_target || !opts[k].second->parameters || !opts[k].second->gradient || !opts[k].second->first_moment || !opts[k].second->second_moment)) return false;
    }
    return true;
}

template <int MODE>
int launch_wide(rlt_rocm_device* device, WideArgs& a, int groups, const Optimiser* opts, int n_opts, float polyak, bool* targets_done) {
    const rlt_dense_layer* trained = opts[0].trained;
    if (!steps_describable(opts, n_opts)) return RLT_E_UNSUPPORTED;
    const int exact_count = partial_count(trained[0].in_dim, trained[0].out_dim, trained[2].out_dim);
    a.count = (exact_count + 63) & ~63;      // blocks start on 256-byte boundaries: the optimisers' launch reads them 16 bytes per lane
    // the copies of the second layers' weights: forward copies of every network that runs forward, backward copies of those whose second layer is also walked backwards
    WNet* forward_nets[5]; WNet* backward_nets[3];
    int n_forward = 0, n_backward = 0;
    forward_nets[n_forward++] = &a.actor;
    for (int k = 0; k < 2; k++) forward_nets[n_forward++] = &a.critic[k];
    constexpr bool CRITIC_UPDATE = MODE == MODE_CRITIC || MODE == MODE_TD3_CRITIC;
    if (CRITIC_UPDATE) for (int k = 0; k < 2; k++) forward_nets[n_forward++] = &a.target[k];
    for (int k = 0; k < 2; k++) backward_nets[n_backward++] = &a.critic[k];
    if (!CRITIC_UPDATE) backward_nets[n_backward++] = &a.actor;
    const size_t copy_floats = (size_t)256 * WAVES * WAVES;      // [16 wavefronts][16 chunks][64 lanes][4] at width 256
    const size_t partial_bytes = ((size_t)n_opts * groups * a.count * sizeof(float) + 255) & ~(size_t)255;
    void* scratch = nullptr;
    int rc = rlt_scratch(device, partial_bytes + (size_t)PREP_JOBS * copy_floats * sizeof(float), &scratch);
    if (rc) return rc;
    a.partial = (float*)scratch;
    {
        PrepArgs P = {};
        float* copies = (float*)((char*)scratch + partial_bytes);
        int jobs = 0, max_tiles = 1;
        auto job = [&](WNet* net, bool backward) {
            for (int q = 0; q < jobs; q++)      // networks given twice (one critic trained alone) share a copy
                if (P.W2[q] == net->W2 && P.backward[q] == (backward ? 1 : 0)) { (backward ? net->W2b : net->W2f) = P.dst[q]; return; }
            P.W2[jobs] = net->W2; P.dst[jobs] = copies + (size_t)jobs * copy_floats; P.hid[jobs] = net->hid; P.backward[jobs] = backward ? 1 : 0;
            (backward ? net->W2b : net->W2f) = P.dst[jobs];
            const int tiles = (net->hid + 15) >> 4;
            if (tiles > max_tiles) max_tiles = tiles;
            jobs++;
        };
        for (int q = 0; q < n_forward; q++) job(forward_nets[q], false);
        for (int q = 0; q < n_backward; q++) job(backward_nets[q], true);
        hipLaunchKernelGGL(wide_prepare_kernel, dim3(rlt_div_up(max_tiles * max_tiles * 64, 256), jobs), dim3(256), 0, device->stream, P);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    a.stream_offset = device->stream_offset;
    a.packed = device->update_one_xcd && device->xcd_stride == 8 && n_opts * groups <= 32 ? 1 : 0;
    const size_t lds_bytes = LDS_FLOATS * sizeof(float);
    const dim3 grid(a.packed ? 8 * groups : groups, n_opts);
#define RLT_LAUNCH_WIDE(ACT, NT)                                                                                                                          \
    do {                                                                                                                                                  \
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(sac_wide_kernel<MODE, ACT, NT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes)); \
        hipLaunchKernelGGL((sac_wide_kernel<MODE, ACT, NT>), grid, dim3(THREADS), lds_bytes, device->stream, a);                                          \
    } while (0)
    int act = a.actor.act_h;
    for (int k = 0; k < 2; k++) if (a.critic[k].act_h != act || a.target[k].act_h != act) act = -1;
    // first layers of at most 32 inputs (two 16-deep chunks) leave registers for all of a pass's weights at once
    if (a.obs + a.act <= 32) {
        if (act == RLT_ACT_RELU) RLT_LAUNCH_WIDE(RLT_ACT_RELU, 2); else if (act == RLT_ACT_FAST_TANH) RLT_LAUNCH_WIDE(RLT_ACT_FAST_TANH, 2); else RLT_LAUNCH_WIDE(-1, 2);
    } else {
        if (act == RLT_ACT_RELU) RLT_LAUNCH_WIDE(RLT_ACT_RELU, MAX_D / 16); else if (act == RLT_ACT_FAST_TANH) RLT_LAUNCH_WIDE(RLT_ACT_FAST_TANH, MAX_D / 16); else RLT_LAUNCH_WIDE(-1, MAX_D / 16);
    }
#undef RLT_LAUNCH_WIDE
    if ((rc = rlt_launch_status(device))) return rc;
    Step S[2];
    rlt_adam_source source[2];
    for (int k = 0; k < n_opts; k++) {
        describe_step(opts[k], S[k]);
        source[k] = {a.partial + (size_t)k * groups * a.count, groups, a.count, S[k].offsets, S[k].scales};
    }
    if (targets_done) *targets_done = n_opts == 2 && S[0].targets_fused && S[1].targets_fused;
    if (targets_done && !*targets_done) for (int k = 0; k < n_opts; k++) for (int i = 0; i < opts[k].n_tensors; i++) S[k].tensors[i].polyak_target = nullptr;
    if (n_opts == 2)
        return rlt_adam_step_pair(device, S[0].tensors, opts[0].n_tensors, opts[0].parameters, opts[0].age, S[1].tensors, opts[1].n_tensors, opts[1].parameters, opts[1].age, &source[0], &source[1], polyak);
    if (opts[0].second) {
        const uint32_t second_offset = (uint32_t)(exact_count - N_EXTRA);
        const rlt_adam_source second_source = {a.partial, groups, a.count, &second_offset, &opts[0].second_scale};
        return rlt_adam_step_pair(device, S[0].tensors, opts[0].n_tensors, opts[0].parameters, opts[0].age, opts[0].second, 1, opts[0].second_parameters, opts[0].second_age, &source[0], &second_source);
    }
    return rlt_adam_step_from_partials(device, S[0].tensors, opts[0].n_tensors, opts[0].parameters, opts[0].age, &source[0]);
}

void set_noise(WideArgs& a, const rlt_update_noise& N) { a.noise = N.values; a.noise_seed = N.seed; a.noise_stream = N.stream; a.out_noise = N.values ? nullptr : N.drawn; }
void common_args(WideArgs& a, const rlt_sac_agent* A) {
    a.actor = net_of(A->actor);
    for (int k = 0; k < 2; k++) { a.critic[k] = net_of(A->critics[k]); a.target[k] = net_of(A->critics_target[k]); }
    a.batch_base = A->observations_actions_base; a.rewards = A->rewards; a.terminated = A->terminated; a.log_alpha = A->log_alpha.parameters;
    a.sas = A->sas; a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
}
}  // namespace

bool rlt_sac_wide_supported(const rlt_rocm_device* device, const rlt_sac_agent* A) {
    const int OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    if (OBS < 1 || ACT < 1 || ACT > MAX_ACT || D > MAX_D || A->batch < 1) return false;
    if (A->final_step_mask || A->next_final_step_mask || A->reset) return false;
    if (A->batch > 2048) return false;      // larger batches are the per-layer kernels' ground
    int hid_a = 0, hid_c = 0;
    if (!net_ok(A->actor, A->n_actor_layers, OBS, 2 * ACT, hid_a)) return false;
    for (int k = 0; k < 2; k++)
        if (!net_ok(A->critics[k], A->n_critic_layers, D, 1, hid_c) || !net_ok(A->critics_target[k], A->n_critic_layers, D, 1, hid_c)) return false;
    return LDS_FLOATS * sizeof(float) <= (size_t)device->lds_bytes;
}

int rlt_sac_wide_update_critics(rlt_rocm_device* device, const rlt_sac_agent* A, int first, int count, const rlt_update_noise& noise, bool update_targets) {
    if (!rlt_sac_wide_supported(device, A)) return RLT_E_UNSUPPORTED;
    RLT_REQUIRE(first >= 0 && count >= 1 && first + count <= 2 && (!update_targets || count == 2));
    for (int k = first; k < first + count; k++) for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[k][l].d_weights && A->critics[k][l].d_biases);
    WideArgs a = {};
    common_args(a, A);
    if (count == 1) { a.critic[0] = net_of(A->critics[first]); a.critic[1] = a.critic[0]; }
    set_noise(a, noise);
    a.out_log_probabilities = A->next_log_probabilities; a.out_target_action_value = A->target_action_value;
    Optimiser O[2];
    for (int k = 0; k < count; k++)
        O[k] = {A->critics[first + k], A->critic_adam_tensors[first + k], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[first + k], nullptr, nullptr, nullptr, 0.0f,
                update_targets ? A->critics_target[first + k] : nullptr};
    bool targets_done = false;
    const int rc = launch_wide<MODE_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), O, count, A->polyak, &targets_done);
    if (rc || !update_targets || targets_done) return rc;
    return rlt_rocm_sac_update_critic_targets(device, A);
}

int rlt_sac_wide_update_actor(rlt_rocm_device* device, const rlt_sac_agent* A, const rlt_update_noise& noise) {
    if (!rlt_sac_wide_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->actor[l].d_weights && A->actor[l].d_biases);
    RLT_REQUIRE(A->log_alpha.gradient);
    WideArgs a = {};
    common_args(a, A);
    set_noise(a, noise);
    a.out_log_probabilities = A->actor_log_probabilities; a.out_actions = A->actor_actions; a.out_pre_squashing = A->actor_pre_squashing;
    const Optimiser O = {A->actor, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, &A->log_alpha, &A->alpha_adam, A->alpha_age, 1.0f / (float)A->batch, nullptr};
    return launch_wide<MODE_ACTOR>(device, a, rlt_div_up(A->batch, ROWS), &O, 1, 0.0f, nullptr);
}

// ---- TD3: the same kernel with the td3_sampling head (rl/algorithms/td3/operations_generic.h:170-281)

bool rlt_td3_wide_supported(const rlt_rocm_device* device, const rlt_td3_agent* A) {
    const int OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    if (OBS < 1 || ACT < 1 || ACT > MAX_ACT || D > MAX_D || A->batch < 1 || A->batch > 2048) return false;
    if (A->final_step_mask || A->next_final_step_mask) return false;
    int hid_a = 0, hid_c = 0;
    if (!net_ok(A->actor, A->n_actor_layers, OBS, ACT, hid_a, RLT_ACT_TANH) || !net_ok(A->actor_target, A->n_actor_layers, OBS, ACT, hid_a, RLT_ACT_TANH)) return false;
    for (int k = 0; k < 2; k++)
        if (!net_ok(A->critics[k], A->n_critic_layers, D, 1, hid_c) || !net_ok(A->critics_target[k], A->n_critic_layers, D, 1, hid_c)) return false;
    return LDS_FLOATS * sizeof(float) <= (size_t)device->lds_bytes;
}

int rlt_td3_wide_update_critic(rlt_rocm_device* device, const rlt_td3_agent* A, int ci, const float* sampling_noise) {
    if (!rlt_td3_wide_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[ci][l].d_weights && A->critics[ci][l].d_biases);
    RLT_REQUIRE(A->target_next_action_noise && sampling_noise);
    WideArgs a = {};
    a.actor = net_of(A->actor_target); a.critic[0] = net_of(A->critics[ci]); a.critic[1] = a.critic[0];
    for (int k = 0; k < 2; k++) a.target[k] = net_of(A->critics_target[k]);
    a.batch_base = A->observations_actions_base; a.rewards = A->rewards; a.terminated = A->terminated; a.noise = sampling_noise; a.target_noise = A->target_next_action_noise;
    a.sampling_std = A->sampling_std; a.ignore_termination = A->ignore_termination;
    a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_target_action_value = A->target_action_value;
    const Optimiser O = {A->critics[ci], A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], nullptr, nullptr, nullptr, 0.0f, nullptr};
    return launch_wide<MODE_TD3_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), &O, 1, 0.0f, nullptr);
}

// both critics on the agent's batch in one launch (blockIdx.y selects the critic), each with its own sampling noise for the target actor's td3_sampling layer:
// what rlt_td3_wide_update_critic for critic 0 and then for critic 1 leave, bit for bit
int rlt_td3_wide_update_critics(rlt_rocm_device* device, const rlt_td3_agent* A, const float* sampling_noise_first, const float* sampling_noise_second, const rlt_td3_critic_draws* draws, bool update_targets) {
    if (!rlt_td3_wide_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int k = 0; k < 2; k++) for (int l = 0; l < 3; l++) RLT_REQUIRE(A->critics[k][l].d_weights && A->critics[k][l].d_biases);
    RLT_REQUIRE(A->target_next_action_noise && (draws || (sampling_noise_first && sampling_noise_second)));
    WideArgs a = {};
    a.actor = net_of(A->actor_target);
    for (int k = 0; k < 2; k++) { a.critic[k] = net_of(A->critics[k]); a.target[k] = net_of(A->critics_target[k]); }
    a.batch_base = A->observations_actions_base; a.rewards = A->rewards; a.terminated = A->terminated;
    if (draws) {        // the three noise tensors are drawn by the kernel; the smoothing noise is left in the agent's buffer as target_action_noise leaves it
        a.noise_seed = draws->seed; a.noise_stream = draws->sampling_stream[0]; a.noise_stream_second = draws->sampling_stream[1]; a.target_noise_stream = draws->target_noise_stream;
        a.target_noise_std = draws->target_noise_std; a.target_noise_clip = draws->target_noise_clip; a.out_target_noise = A->target_next_action_noise;
    } else { a.noise = sampling_noise_first; a.noise_second = sampling_noise_second; a.target_noise = A->target_next_action_noise; }
    a.sampling_std = A->sampling_std; a.ignore_termination = A->ignore_termination;
    a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_target_action_value = A->target_action_value;
    Optimiser O[2];
    for (int k = 0; k < 2; k++)
        O[k] = {A->critics[k], A->critic_adam_tensors[k], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[k], nullptr, nullptr, nullptr, 0.0f, update_targets ? A->critics_target[k] : nullptr};
    bool targets_done = false;      // the targets' soft update rides along in the optimisers' launch where the tensors correspond
    const int rc = launch_wide<MODE_TD3_CRITIC>(device, a, rlt_div_up(A->batch, ROWS), O, 2, A->critic_polyak, &targets_done);
    if (rc || !update_targets || targets_done) return rc;
    return rlt_rocm_td3_update_critic_targets(device, A);
}

int rlt_td3_wide_update_actor(rlt_rocm_device* device, const rlt_td3_agent* A, const float* sampling_noise, uint64_t seed, uint64_t stream) {
    if (!rlt_td3_wide_supported(device, A)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) RLT_REQUIRE(A->actor[l].d_weights && A->actor[l].d_biases);
    WideArgs a = {};
    a.actor = net_of(A->actor);
    for (int k = 0; k < 2; k++) { a.critic[k] = net_of(A->critics[0]); a.target[k] = a.critic[k]; }       // the policy gradient goes through critic 0 (:260)
    a.batch_base = A->observations_actions_base; a.noise = sampling_noise; a.noise_seed = seed; a.noise_stream = stream;      // sampling_noise NULL: drawn from (seed, stream)
    a.sampling_std = A->sampling_std;
    a.gamma = A->gamma; a.batch = A->batch; a.obs = A->observation_dim; a.act = A->action_dim;
    a.out_pre_clip = A->actor_pre_clip;
    const Optimiser O = {A->actor, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, nullptr, nullptr, nullptr, 0.0f, nullptr};
    return launch_wide<MODE_TD3_ACTOR>(device, a, rlt_div_up(A->batch, ROWS), &O, 1, 0.0f, nullptr);
}


// ---- forward + backward of a three-layer network on sixteen-row tiles (see mlp_wide_kernel), or the backward pass alone from the outputs that a forward() left in
// the layers; RLT_E_UNSUPPORTED: the caller takes another path
static int mlp_wide_launch(rlt_rocm_device* device, const rlt_dense_layer* L, int n_layers, const float* x, int ldx, float* y, int ldy,
                           const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch, int pass) {
    const bool backward_only = pass == MLP_BACKWARD, forward_only = pass == MLP_FORWARD;
    if (n_layers != 3 || batch < 1 || batch > RLT_MLP_WIDE_MAX_BATCH || L[0].in_dim < 1 || L[0].in_dim > MAX_D || L[2].out_dim < 1 || L[2].out_dim > MAX_OUT) return RLT_E_UNSUPPORTED;
    int hid = 0;
    // the backward pass alone is handed the gradient at the last pre-activations: the last layer's activation plays no part in it
    // (forward() applies the last layer's activation per element when it stores the outputs)
    if (!net_ok(L, 3, L[0].in_dim, L[2].out_dim, hid, pass == MLP_FORWARD_BACKWARD ? RLT_ACT_IDENTITY : L[2].activation)) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) if (!forward_only && (!L[l].d_weights || !L[l].d_biases)) return RLT_E_UNSUPPORTED;
    if (backward_only && (!L[0].output || !L[1].output)) return RLT_E_UNSUPPORTED;
    if (LDS_FLOATS * sizeof(float) > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    MlpWideArgs a = {};
    a.net = net_of(L);
    a.x = x; a.ldx = ldx; a.y = y; a.ldy = ldy; a.d_output = d_output; a.ldd = ldd; a.target = target; a.ldt = ldt; a.mse_scale = mse_scale; a.batch = batch;
    a.out1 = L[0].output; a.out2 = L[1].output;
    if (forward_only) for (int l = 0; l < 3; l++) { a.keep_pre[l] = L[l].pre_activations; a.keep_out[l] = L[l].output; }
    a.act3 = L[2].activation;
    const int IN = L[0].in_dim, OUT = L[2].out_dim, groups = rlt_div_up(batch, ROWS);
    const int exact = hid * IN + hid + hid * hid + hid + OUT * hid + OUT;
    a.count = (exact + 63) & ~63;
    const size_t copy_floats = (size_t)256 * WAVES * WAVES;
    const size_t partial_bytes = forward_only ? 0 : ((size_t)groups * a.count * sizeof(float) + 255) & ~(size_t)255;
    void* scratch = nullptr;
    int rc = 0;
    if (!forward_only) {
        if ((rc = rlt_scratch(device, partial_bytes, &scratch))) return rc;
        a.partial = (float*)scratch;
    }
    // the weight copies have a buffer of their own: forward() and evaluate() have never touched the handle's scratch buffer at these batch sizes, and callers hold data there across them
    if (device->copy_scratch_bytes < 2 * copy_floats * sizeof(float)) {
        if (device->capturing) return RLT_E_CAPTURING;
        if (device->copy_scratch) RLT_HIP(hipFree(device->copy_scratch));
        device->copy_scratch = nullptr; device->copy_scratch_bytes = 0;
        RLT_HIP(hipMalloc(&device->copy_scratch, 2 * copy_floats * sizeof(float)));
        device->copy_scratch_bytes = 2 * copy_floats * sizeof(float);
    }
    {
        // the second layer's weights in the order the wavefronts consume them: the copy for d_pre2 W2, and for the forward pass the one for h1 W2^T
        PrepArgs P = {};
        float* copies = (float*)device->copy_scratch;
        const int jobs = pass == MLP_FORWARD_BACKWARD ? 2 : 1;
        for (int q = 0; q < jobs; q++) { P.W2[q] = a.net.W2; P.dst[q] = copies + (size_t)q * copy_floats; P.hid[q] = hid; P.backward[q] = (q == 0 && !forward_only) ? 1 : 0; }
        a.net.W2b = forward_only ? nullptr : P.dst[0]; a.net.W2f = forward_only ? P.dst[0] : (backward_only ? nullptr : P.dst[1]);
        const int tiles = (hid + 15) >> 4;
        hipLaunchKernelGGL(wide_prepare_kernel, dim3(rlt_div_up(tiles * tiles * 64, 256), jobs), dim3(256), 0, device->stream, P);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    const size_t lds_bytes = LDS_FLOATS * sizeof(float);
#define RLT_LAUNCH_MLP_WIDE(ACT, NT, BWD)                                                                                                                   \
    do {                                                                                                                                                    \
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(mlp_wide_kernel<ACT, NT, BWD>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes)); \
        hipLaunchKernelGGL((mlp_wide_kernel<ACT, NT, BWD>), dim3(groups), dim3(THREADS), lds_bytes, device->stream, a);                                    \
    } while (0)
    const bool relu = a.net.act_h == RLT_ACT_RELU;
#define RLT_LAUNCH_MLP_WIDE_PASS(P)                                                                                                       \
    do {                                                                                                                                  \
        if (IN <= 32) { if (relu) RLT_LAUNCH_MLP_WIDE(RLT_ACT_RELU, 2, P); else RLT_LAUNCH_MLP_WIDE(-1, 2, P); }                          \
        else { if (relu) RLT_LAUNCH_MLP_WIDE(RLT_ACT_RELU, MAX_D / 16, P); else RLT_LAUNCH_MLP_WIDE(-1, MAX_D / 16, P); }                  \
    } while (0)
    if (backward_only) RLT_LAUNCH_MLP_WIDE_PASS(MLP_BACKWARD); else if (forward_only) RLT_LAUNCH_MLP_WIDE_PASS(MLP_FORWARD); else RLT_LAUNCH_MLP_WIDE_PASS(MLP_FORWARD_BACKWARD);
#undef RLT_LAUNCH_MLP_WIDE_PASS
#undef RLT_LAUNCH_MLP_WIDE
    if ((rc = rlt_launch_status(device))) return rc;
    if (forward_only) return 0;
    WideReduceArgs R = {};
    R.partial = a.partial; R.blocks = groups; R.count = a.count; R.total = exact;
    float* const dst[6] = {L[0].d_weights, L[0].d_biases, L[1].d_weights, L[1].d_biases, L[2].d_weights, L[2].d_biases};
    const int size[6] = {hid * IN, hid, hid * hid, hid, OUT * hid, OUT};
    for (int k = 0, end = 0; k < 6; k++) { end += size[k]; R.dst[k] = dst[k]; R.end[k] = end; }
    hipLaunchKernelGGL(mlp_wide_reduce_kernel, dim3(rlt_div_up(exact, 256)), dim3(256), 0, device->stream, R);
    return rlt_launch_status(device);
}
int rlt_mlp_wide_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* L, int n_layers, const float* x, int ldx, float* y, int ldy,
                                  const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch) {
    return mlp_wide_launch(device, L, n_layers, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch, MLP_FORWARD_BACKWARD);
}
int rlt_mlp_wide_backward(rlt_rocm_device* device, const rlt_dense_layer* L, int n_layers, const float* x, int ldx, const float* d_pre_last, int ldd, int batch) {
    return mlp_wide_launch(device, L, n_layers, x, ldx, nullptr, 0, d_pre_last, ldd, nullptr, 0, 0.0f, batch, MLP_BACKWARD);
}
int rlt_mlp_wide_forward(rlt_rocm_device* device, const rlt_dense_layer* L, int n_layers, const float* x, int ldx, float* y, int ldy, int batch, bool keep) {
    if (keep) return mlp_wide_launch(device, L, n_layers, x, ldx, y, ldy, nullptr, 0, nullptr, 0, 0.0f, batch, MLP_FORWARD);
    rlt_dense_layer plain[3];      // evaluate(): nothing is kept
    if (n_layers != 3) return RLT_E_UNSUPPORTED;
    for (int l = 0; l < 3; l++) { plain[l] = L[l]; plain[l].pre_activations = nullptr; plain[l].output = nullptr; }
    return mlp_wide_launch(device, plain, n_layers, x, ldx, y, ldy, nullptr, 0, nullptr, 0, 0.0f, batch, MLP_FORWARD);
}

#ifdef RLT_WIDE_PROFILE
extern "C" int rlt_sac_wide_ticks(unsigned long long* out) { return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(rlt_wide_ticks), sizeof(unsigned long long) * 64); }
#endif
