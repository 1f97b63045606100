// Single-pass forward + backward of a 3-layer MLP in -> 64 -> 64 -> out for the narrow networks of PPO, TD3 and SAC
// (nn_models/mlp/operations_generic.h:128-181 forward, :183-260 backward; nn/layers/dense/operations_generic.h:98-260).
//
// A workgroup of four wavefronts takes 64 batch rows per round. The work is split two ways:
//   by rows      each wavefront runs its own 16 rows through the three layers, the loss and the input-gradient products
//                  h1 = f(x W1^T + b1), h2 = f(h1 W2^T + b2), y = g(h2 W3^T + b3), d_pre3 from the caller's d_output / an MSE target / PPO's
//                  clipped surrogate, d_pre2 = (d_pre3 W3) f'(h2), d_pre1 = (d_pre2 W2) f'(h1)
//   by columns   for the weight gradients dW3 += d_pre3^T h2, dW2 += d_pre2^T h1, dW1 += d_pre1^T x the reduction runs over all 64 rows of the
//                  round, and wavefront w owns the 16 output rows 16 w .. 16 w + 15 of dW1 and dW2 and 16 columns of dW3
// so every accumulator tile of a weight gradient lives in exactly one wavefront's registers for the whole kernel (8 + 4 + 1 tiles), no sums
// are exchanged between wavefronts, and a workgroup writes one block of partial sums at the end, which a second kernel adds to the layers'
// gradients in workgroup order: the result does not depend on scheduling. Activations and gradients of the round sit in LDS in the layouts
// v_mfma_f32_16x16x4_f32 wants (lane l = r + 16 kk feeds A[r][kk] and B[kk][r] and receives D[4 kk + v][r], v = 0..3); the weights are staged
// once per workgroup in LDS (padded rows, read as both W and W^T). Four workgroup barriers per round order the two kinds of phase.
// Bound: the fp32 matrix pipe, 2 (in + 64 + out) 64 flop per row forward and twice that backward less the input gradient of layer 1.
#include "mlp_small.h"
#include "optim.h"
#include "xcd_reduce.h"

namespace {
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) float* lptr;
constexpr int H = 64, HS = H + 1, WAVES = 4, ROWS = 16 * WAVES, THREADS = 64 * WAVES, MAX_IN = 128, MAX_OUT = 16, MAX_NT1 = MAX_IN / 16, D3S = MAX_OUT + 1,
              N_EXTRA = 16, N_SUMS = 2 * H + MAX_OUT + N_EXTRA;
enum { LOSS_GIVEN = 0, LOSS_MSE = 1, LOSS_PPO = 2 };

struct SmallArgs {
    const float* x; int ldx, batch, in, out, act3;
    const uint32_t* rows;           // optional: batch row b reads row rows[b] of x, d_output / target / actions / log_probs / advantages (y is written at row b)
    const float *W1, *b1, *W2, *b2, *W3, *b3;
    float* y; int ldy;
    int loss;
    const float* d_output; int ldd;
    const float* target; int ldt; float mse_scale;
    const float* log_std; const float* actions; int ld_actions; const float* log_probs; int ld_lp; const float* advantages; int ld_adv; const float* stats;
    float epsilon_clip, advantage_epsilon; int normalize_advantage;
    float* partial; int count;      // per workgroup: dW1 [64 x in], db1 [64], dW2 [64 x 64], db2 [64], dW3 [out x 64], db3 [out], extra [16]
    float* d_input; int ld_di;      // optional: gradient with respect to x, written at row b
    const float* std_mean; const float* std_precision;      // optional standardize layer in front: the network reads (x - mean) * precision (the factor where it is not 0)
};

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
template <int CTRL>
__device__ __forceinline__ float dpp(float x) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true)); }
__device__ __forceinline__ float row16_sum(float x) { asm volatile("" : "+v"(x)); /* keeps a producing multiplication out of the first addition: all lanes then hold the same sum */ x += dpp<0xB1>(x); x += dpp<0x4E>(x); x += dpp<0x141>(x); x += dpp<0x140>(x); return x; }
// lanes of one wavefront exchange data through LDS: the hardware executes a wavefront's LDS instructions in order, the fences keep
// the compiler from moving them across
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// sum over the four lane groups (lanes r, r + 16, r + 32, r + 48), in a fixed order
__device__ __forceinline__ float groups_sum(float v) { asm volatile("" : "+v"(v)); v += __shfl_xor(v, 16, 64); v += __shfl_xor(v, 32, 64); return v; }

// LDS: W1 [64][SX], W2 [64][HS], W3 [16][HS], then per round x [64][SX], h1 [64][HS], h2 [64][HS], g2 [64][HS], d3 [64][D3S]; SX = 16 nt1c + 1
constexpr size_t lds_floats(int nt1c) {
    const int sx = 16 * nt1c + 1;
    return (size_t)H * sx + H * HS + MAX_OUT * HS + (size_t)ROWS * (sx + 3 * HS + D3S);
}

// global loads of one tile of 16 rows, issued together: the inputs (lane = column, up to two columns per lane) and what the loss needs of the
// rows this lane will hold after the forward pass (rows 4 kk + v, column r); columns beyond the extent are clamped here and masked later.
// `vrows`: the rows' indices, requested a round earlier so that nothing waits for them here.
struct TileRegs { float xa[16], xb[16], in0[4], in1[4], in2[4]; };
__device__ __forceinline__ void request_tile(const SmallArgs& A, uint32_t vrows, int lane, TileRegs& T) {
    const int r = lane & 15, kk = lane >> 4;
    const int c0 = min(lane, A.in - 1), c1 = min(64 + lane, A.in - 1), c = min(r, A.out - 1);
#pragma unroll
    for (int row = 0; row < 16; row++) {
        const float* src = A.x + (size_t)(uint32_t)__builtin_amdgcn_readlane((int)vrows, row) * A.ldx;      // wavefront-uniform: scalar address arithmetic
        T.xa[row] = src[c0];
        T.xb[row] = A.in > 64 ? src[c1] : 0.f;
    }
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const size_t row = (size_t)(uint32_t)__shfl((int)vrows, 4 * kk + v, 64);
        T.in0[v] = T.in1[v] = T.in2[v] = 0.f;
        if (A.loss == LOSS_GIVEN) T.in0[v] = A.d_output[row * A.ldd + c];
        else if (A.loss == LOSS_MSE) T.in0[v] = A.target[row * A.ldt + c];
        else { T.in0[v] = A.actions[row * A.ld_actions + c]; T.in1[v] = A.advantages[row * A.ld_adv]; T.in2[v] = A.log_probs[row * A.ld_lp]; }
    }
}


// profiling builds (-DRLT_SMALL_PROFILE): thread 0 of workgroup 0 notes the constant-rate clock at the stage boundaries, rlt_mlp3s_ticks copies the notes out
#ifdef RLT_SMALL_PROFILE
__device__ unsigned long long rlt_small_ticks[32];
__device__ unsigned long long rlt_small_spans[512][2];
#define RLT_TICK(i) do { if (blockIdx.x == 0 && threadIdx.x == 0) rlt_small_ticks[i] = wall_clock64(); } while (0)
#else
#define RLT_TICK(i) do {} while (0)
#endif

// ACT_H: hidden activation; NT1C: number of 16-column tiles of dW1 the code is unrolled for (>= the NT1 the input width needs; the surplus
// tiles multiply zero columns and are never stored). Both are compile-time constants: a matrix instruction under a run-time
// condition makes the compiler carry both versions of its accumulator.
// One launch can carry two networks (PPO's actor and critic on the same minibatch): workgroups [0, groups0) work on A0, the rest on A1.
// LAYERS = 2: the network is in -> 64 -> out; layer 2, its weight gradient and its input gradient drop out, the output layer reads h1, and the
// gradient at layer 1's pre-activations is formed directly from the output layer's.
// xr (optional): the blocks of partial sums are added up per XCD inside the launch (xcd_reduce.h); network j's eight blocks of sums then lie at xsum[j]
struct SmallLaunch { SmallArgs a0, a1; int groups0; rlt_xcd_reduce_args xr; float* xsum[2]; };
template <int ACT_H, int NT1C, int LAYERS>
__global__ __launch_bounds__(THREADS) void mlp3s_kernel(SmallLaunch K) {
    RLT_TICK(0);
#ifdef RLT_SMALL_PROFILE
    if (threadIdx.x == 0) rlt_small_spans[blockIdx.x][0] = wall_clock64();
#endif
    extern __shared__ float lds_raw[];
    const int groups0 = K.groups0;
    const bool second = (int)blockIdx.x >= groups0;
    const SmallArgs& A = second ? K.a1 : K.a0;
    const int block = second ? blockIdx.x - groups0 : blockIdx.x, n_blocks = second ? gridDim.x - groups0 : groups0;
    const int lane = threadIdx.x & 63, r = lane & 15, kk = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // wavefront-uniform: addresses derived from it are computed on the scalar unit
    const int IN = A.in, OUT = A.out, NT1 = (IN + 15) >> 4;
    constexpr int SX = 16 * NT1C + 1;        // row stride of the input tile and of W1 in LDS: a constant, so that LDS offsets fold into the instructions
    const lptr w1s = (lptr)lds_raw, w2s = w1s + H * SX, w3s = w2s + H * HS;
    const lptr xs_all = w3s + MAX_OUT * HS, h1s_all = xs_all + ROWS * SX, h2s_all = h1s_all + ROWS * HS, g2s_all = h2s_all + ROWS * HS, d3s_all = g2s_all + ROWS * HS;
    const lptr xs = xs_all + 16 * wave * SX, h1s = h1s_all + 16 * wave * HS, h2s = h2s_all + 16 * wave * HS, g2s = g2s_all + 16 * wave * HS, d3s = d3s_all + 16 * wave * D3S;
    const int n_tiles = (A.batch + 15) >> 4, n_rounds = (n_tiles + WAVES - 1) / WAVES;
    // lane l: the row of the input arrays that row (l & 15) of this wavefront's tile of round `round` reads; a tile beyond the batch is clamped here and masked later
    auto rows_of = [&](int round) -> uint32_t {
        const int b = min(min(round * WAVES + wave, n_tiles - 1) * 16 + (lane & 15), A.batch - 1);
        return A.rows ? A.rows[b] : (uint32_t)b;
    };
    // The launch's critical path starts with two dependent trips to memory (the row indices, then the rows): the index loads go out first, the
    // weights' and constants' loads follow while the indices travel, then the first tile's loads, and the weights are stored to LDS while those
    // travel.
    uint32_t rows_next = rows_of(block), rows_after = rows_next;
    if (block + n_blocks < n_rounds) rows_after = rows_of(block + n_blocks);
    TileRegs T;
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const int xgroup = (second ? RLT_XCD_GROUPS : 0) + (block & 7);      // with the XCD-level sums: this workgroup's group (network, XCD)
    uint32_t xepoch = 0;
    if (K.xr.enabled) xepoch = rlt_xcd_epoch(K.xr, xgroup);
    float v1[H / WAVES][2], v2[H * H / THREADS], v3[MAX_OUT * H / THREADS];
#pragma unroll
    for (int j = 0; j < H / WAVES; j++) {
        const float* src = A.W1 + (size_t)(wave * (H / WAVES) + j) * IN;
        v1[j][0] = src[min(lane, IN - 1)];
        v1[j][1] = IN > 64 ? src[min(64 + lane, IN - 1)] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < H * H / THREADS; u++) v2[u] = LAYERS == 3 ? A.W2[u * THREADS + threadIdx.x] : 0.f;
#pragma unroll
    for (int u = 0; u < MAX_OUT * H / THREADS; u++) v3[u] = A.W3[min(u * THREADS + (int)threadIdx.x, OUT * H - 1)];
    float b1r[4], b2r[4];
#pragma unroll
    for (int nt = 0; nt < 4; nt++) { b1r[nt] = A.b1[16 * nt + r]; b2r[nt] = LAYERS == 3 ? A.b2[16 * nt + r] : 0.f; }
    const float b3r = A.b3[min(r, OUT - 1)];
    float ls = 0.f, adv_mean = 0.f, adv_std = 0.f;
    if (A.loss == LOSS_PPO) {
        ls = A.log_std[min(r, OUT - 1)];
        if (A.normalize_advantage) { adv_mean = A.stats[0]; adv_std = A.stats[1]; }
    }
    // the standardize layer's constants for this lane's columns (nn/layers/standardize/operations_generic.h:68-86); without one: x - 0 times 1
    float sm0 = 0.f, sp0 = 1.f, sm1 = 0.f, sp1 = 1.f;
    if (A.std_mean) {
        sm0 = A.std_mean[min(lane, IN - 1)]; sp0 = A.std_precision[min(lane, IN - 1)];
        if (IN > 64) { sm1 = A.std_mean[min(64 + lane, IN - 1)]; sp1 = A.std_precision[min(64 + lane, IN - 1)]; }
        sp0 = sp0 != 0.f ? sp0 : 1.f; sp1 = sp1 != 0.f ? sp1 : 1.f;
    }
    __builtin_amdgcn_sched_barrier(0);      // the loads above are issued before the first wait for the row indices
    request_tile(A, rows_next, lane, T);
    RLT_TICK(1);
    // weights into LDS, rows padded to SX (zero beyond the input width, so the padded reduction steps add nothing)
    {
#pragma unroll
        for (int j = 0; j < H / WAVES; j++) {
            const lptr dst = w1s + (wave * (H / WAVES) + j) * SX;
            if (lane < SX) dst[lane] = lane < IN ? v1[j][0] : 0.f;
            if (64 + lane < SX) dst[64 + lane] = 64 + lane < IN ? v1[j][1] : 0.f;
            if (lane == 0 && SX > 128) dst[128] = 0.f;
        }
#pragma unroll
        for (int u = 0; u < H * H / THREADS; u++) { const int i = u * THREADS + threadIdx.x; w2s[(i >> 6) * HS + (i & 63)] = v2[u]; }
#pragma unroll
        for (int u = 0; u < MAX_OUT * H / THREADS; u++) { const int i = u * THREADS + threadIdx.x; w3s[(i >> 6) * HS + (i & 63)] = (i >> 6) < OUT ? v3[u] : 0.f; }
    }
    RLT_TICK(2);
    const float sd = expf(ls);
    rlt_lds_barrier();

    RLT_TICK(3);
    // this wavefront's share of the weight gradients: rows 16 wave + 4 kk + v of dW1 (columns 16 nt + r) and of dW2, columns 16 wave + r of dW3 (rows 4 kk + v)
    floatx4 aW1[NT1C], aW2[4], aW3a = zero4, aW3b = zero4;
#pragma unroll
    for (int nt = 0; nt < NT1C; nt++) aW1[nt] = zero4;
#pragma unroll
    for (int nt = 0; nt < 4; nt++) aW2[nt] = zero4;
    float s1[4] = {0.f, 0.f, 0.f, 0.f}, s2[4] = {0.f, 0.f, 0.f, 0.f}, s3 = 0.f, gls = 0.f;      // bias gradients and the extra sums (PPO: log_std gradient; MSE: squared error) over this wavefront's rows

    for (int round = block; round < n_rounds; round += n_blocks) {
        const int tile = round * WAVES + wave, row0 = tile * 16;
        // inputs of the tile into LDS, zero beyond the batch and beyond the input width
#pragma unroll
        for (int row = 0; row < 16; row++) {
            const bool rok = row0 + row < A.batch;
            if (lane < 16 * NT1C) xs[row * SX + lane] = (rok && lane < IN) ? (T.xa[row] - sm0) * sp0 : 0.f;
            if (64 + lane < 16 * NT1C) xs[row * SX + 64 + lane] = (rok && 64 + lane < IN) ? (T.xb[row] - sm1) * sp1 : 0.f;
        }
    RLT_TICK(4);
        float in0[4], in1[4], in2[4];
#pragma unroll
        for (int v = 0; v < 4; v++) { in0[v] = T.in0[v]; in1[v] = T.in1[v]; in2[v] = T.in2[v]; }
        wave_sync();
        // the next round's loads travel while this one is computed, with row indices requested a round earlier
        if (round + n_blocks < n_rounds) {
            rows_next = rows_after;
            if (round + 2 * n_blocks < n_rounds) rows_after = rows_of(round + 2 * n_blocks);
            request_tile(A, rows_next, lane, T);
        }

    RLT_TICK(5);
        // layer 1: groups of four reduction steps, the operands of the next group requested before this group's matrix instructions. Lane
        // group kk supplies input column 32 (g / 2) + 4 (g % 2) + q + koff with koff = 0, 16, 8, 24: the two lane groups that the LDS serves
        // together read columns 16 apart, that is different banks (rows are an odd number of floats apart)
        floatx4 acc[4] = {zero4, zero4, zero4, zero4};
        {
            const int koff = 16 * (kk & 1) + 8 * (kk >> 1), n_groups = 2 * ((IN + 31) >> 5);
            float a_c[4], b_c[4][4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                a_c[q] = xs[r * SX + koff + q];
#pragma unroll
                for (int nt = 0; nt < 4; nt++) b_c[q][nt] = w1s[(16 * nt + r) * SX + koff + q];
            }
            for (int g = 0; g < n_groups; g++) {
                const int gn = min(g + 1, n_groups - 1), kn = 32 * (gn >> 1) + 4 * (gn & 1) + koff;
                float a_n[4], b_n[4][4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    a_n[q] = xs[r * SX + kn + q];
#pragma unroll
                    for (int nt = 0; nt < 4; nt++) b_n[q][nt] = w1s[(16 * nt + r) * SX + kn + q];
                }
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int nt = 0; nt < 4; nt++) acc[nt] = mfma16(a_c[q], b_c[q][nt], acc[nt]);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    a_c[q] = a_n[q];
#pragma unroll
                    for (int nt = 0; nt < 4; nt++) b_c[q][nt] = b_n[q][nt];
                }
            }
        }
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
            for (int v = 0; v < 4; v++) h1s[(4 * kk + v) * HS + 16 * nt + r] = rlt_act(acc[nt][v] + b1r[nt], ACT_H);
        wave_sync();

    RLT_TICK(6);
        // layer 2
        if (LAYERS == 3) {
#pragma unroll
            for (int nt = 0; nt < 4; nt++) acc[nt] = zero4;
#pragma unroll
            for (int s = 0; s < 16; s++) {
                const float a = h1s[r * HS + 16 * kk + s];
#pragma unroll
                for (int nt = 0; nt < 4; nt++) acc[nt] = mfma16(a, w2s[(16 * nt + r) * HS + 16 * kk + s], acc[nt]);
            }
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int v = 0; v < 4; v++) h2s[(4 * kk + v) * HS + 16 * nt + r] = rlt_act(acc[nt][v] + b2r[nt], ACT_H);
            wave_sync();
        }
        const lptr hls = LAYERS == 3 ? h2s : h1s, hls_all = LAYERS == 3 ? h2s_all : h1s_all;      // the last hidden layer's activations

    RLT_TICK(7);
        // layer 3 (two chains of matrix instructions) and the gradient at its pre-activations
        floatx4 y0 = zero4, y1 = zero4;
#pragma unroll
        for (int s = 0; s < 16; s += 2) {
            y0 = mfma16(hls[r * HS + 16 * kk + s], w3s[r * HS + 16 * kk + s], y0);
            y1 = mfma16(hls[r * HS + 16 * kk + s + 1], w3s[r * HS + 16 * kk + s + 1], y1);
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = row0 + 4 * kk + v;
            const bool ok = row < A.batch && r < OUT;
            const float yv = rlt_act((y0[v] + y1[v]) + b3r, A.act3);
            if (A.y && ok) A.y[(size_t)row * A.ldy + r] = yv;
            float d = 0.f;
            if (A.loss == LOSS_GIVEN) d = in0[v];
            else if (A.loss == LOSS_MSE) { const float diff = yv - in0[v]; d = diff * A.mse_scale; if (ok) gls += diff * diff; }    // gls: the column's summed squared error
            else {
                // per sample (rl/algorithms/ppo/operations_generic.h:205-269): log-probability of the rollout action under the current
                // policy (random/operations_generic.h:73-96), ratio, clipping, d loss / d mean and the surrogate part of d loss / d log_std
                const float value = in0[v];
                const float pre = (value - yv) / sd;
                const float lp = row16_sum(ok ? (-0.9189385332046727f - ls) - 0.5f * pre * pre : 0.f);
                float advantage = in1[v];
                if (A.normalize_advantage) advantage = (advantage - adv_mean) / (adv_std + A.advantage_epsilon);
                const float ratio = expf(lp - in2[v]);
                const float clipped_ratio = fminf(fmaxf(ratio, 1.0f - A.epsilon_clip), 1.0f + A.epsilon_clip);
                const bool clipped = ratio != clipped_ratio;
                const bool ratio_min_switch = ratio * advantage - clipped_ratio * advantage <= 0.0f;
                const float d_surrogate_d_ratio = ratio_min_switch ? advantage : (clipped ? 0.0f : advantage);
                const float d_loss_d_lp = (-1.0f / (float)A.batch) * d_surrogate_d_ratio * ratio;
                if (ok) { d = d_loss_d_lp * (pre / sd); gls += d_loss_d_lp * (pre * pre - 1.0f); }
            }
            const float dp = ok ? d * rlt_dact_from_output(yv, A.act3) : 0.f;
            s3 += dp;
            d3s[(4 * kk + v) * D3S + r] = dp;
        }
    RLT_TICK(8);
        rlt_lds_barrier();      // every wavefront's last hidden activations and d_pre3 are in place

        // dW3 (columns 16 wave + r) += d_pre3^T h over the 64 rows, two chains; in the weight gradients' reductions lane group kk supplies rows
        // 16 kk + ks (wavefront kk's tile), so that the lane groups served together read different LDS banks
        {
            float a_c = d3s_all[16 * kk * D3S + r], b_c = hls_all[16 * kk * HS + 16 * wave + r];
#pragma unroll
            for (int ks = 0; ks < ROWS / 4; ks++) {
                const int kn = min(ks + 1, ROWS / 4 - 1);
                const float a_n = d3s_all[(16 * kk + kn) * D3S + r], b_n = hls_all[(16 * kk + kn) * HS + 16 * wave + r];
                if (ks & 1) aW3b = mfma16(a_c, b_c, aW3b); else aW3a = mfma16(a_c, b_c, aW3a);
                a_c = a_n; b_c = b_n;
            }
        }
    RLT_TICK(9);
        // d_pre2 = (d_pre3 W3) f'(h2) for the wavefront's own rows, into g2
#pragma unroll
        for (int nt = 0; nt < 4; nt++) acc[nt] = zero4;
#pragma unroll
        for (int ks = 0; ks < MAX_OUT / 4; ks++) {      // columns of d_pre3 and rows of W3 beyond `out` are zero
            const float a = d3s[r * D3S + 4 * ks + kk];
#pragma unroll
            for (int nt = 0; nt < 4; nt++) acc[nt] = mfma16(a, w3s[(4 * ks + kk) * HS + 16 * nt + r], acc[nt]);
        }
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int idx = (4 * kk + v) * HS + 16 * nt + r;
                const float dp = acc[nt][v] * rlt_dact_from_output(hls[idx], ACT_H);
                if (LAYERS == 3) { g2s[idx] = dp; s2[nt] += dp; }
                else { h2s[idx] = dp; s1[nt] += dp; }       // two layers: this is already the gradient at layer 1's pre-activations, kept where dW1 reads it
            }
    RLT_TICK(10);
        rlt_lds_barrier();      // every wavefront's d_pre2 is in place, and nobody reads h2 any more
        if (LAYERS == 3) {

        // dW2 (rows 16 wave + ..) += d_pre2^T h1 over the 64 rows
        {
            float a_c = g2s_all[16 * kk * HS + 16 * wave + r], b_c[4];
#pragma unroll
            for (int nt = 0; nt < 4; nt++) b_c[nt] = h1s_all[16 * kk * HS + 16 * nt + r];
#pragma unroll
            for (int ks = 0; ks < ROWS / 4; ks++) {
                const int kn = min(ks + 1, ROWS / 4 - 1);
                float a_n = g2s_all[(16 * kk + kn) * HS + 16 * wave + r], b_n[4];
#pragma unroll
                for (int nt = 0; nt < 4; nt++) b_n[nt] = h1s_all[(16 * kk + kn) * HS + 16 * nt + r];
#pragma unroll
                for (int nt = 0; nt < 4; nt++) aW2[nt] = mfma16(a_c, b_c[nt], aW2[nt]);
                a_c = a_n;
#pragma unroll
                for (int nt = 0; nt < 4; nt++) b_c[nt] = b_n[nt];
            }
        }
    RLT_TICK(11);
        // d_pre1 = (d_pre2 W2) f'(h1) for the wavefront's own rows, into the place of h2
#pragma unroll
        for (int nt = 0; nt < 4; nt++) acc[nt] = zero4;
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
                const float dp = acc[nt][v] * rlt_dact_from_output(h1s[idx], ACT_H);
                h2s[idx] = dp; s1[nt] += dp;
            }
    RLT_TICK(12);
        rlt_lds_barrier();      // every wavefront's d_pre1 is in place
        }

        // gradient with respect to the input, for the wavefront's own rows: d_x = d_pre1 W1, one tile of 16 input columns at a time
        if (A.d_input) {
            for (int nt = 0; nt < NT1; nt++) {
                floatx4 dx = zero4;
#pragma unroll
                for (int s = 0; s < 16; s++) dx = mfma16(h2s[r * HS + 16 * kk + s], w1s[(16 * kk + s) * SX + 16 * nt + r], dx);
#pragma unroll
                for (int v = 0; v < 4; v++)
                    if (row0 + 4 * kk + v < A.batch && 16 * nt + r < IN) A.d_input[(size_t)(row0 + 4 * kk + v) * A.ld_di + 16 * nt + r] = dx[v];
            }
        }

    RLT_TICK(13);
        // dW1 (rows 16 wave + ..) += d_pre1^T x over the 64 rows
        {
            float a_c = h2s_all[16 * kk * HS + 16 * wave + r], b_c[NT1C];
#pragma unroll
            for (int nt = 0; nt < NT1C; nt++) b_c[nt] = xs_all[16 * kk * SX + 16 * nt + r];
#pragma unroll 4
            for (int ks = 0; ks < ROWS / 4; ks++) {
                const int kn = min(ks + 1, ROWS / 4 - 1);
                float a_n = h2s_all[(16 * kk + kn) * HS + 16 * wave + r], b_n[NT1C];
#pragma unroll
                for (int nt = 0; nt < NT1C; nt++) b_n[nt] = xs_all[(16 * kk + kn) * SX + 16 * nt + r];
#pragma unroll
                for (int nt = 0; nt < NT1C; nt++) aW1[nt] = mfma16(a_c, b_c[nt], aW1[nt]);
                a_c = a_n;
#pragma unroll
                for (int nt = 0; nt < NT1C; nt++) b_c[nt] = b_n[nt];
            }
        }
    RLT_TICK(14);
        rlt_lds_barrier();      // the round's tiles may be overwritten
    }

    RLT_TICK(15);
    // the workgroup's block of partial sums: weight gradients straight from the registers that own them, ...
    float* dst = A.partial + (size_t)block * A.count;
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
    RLT_TICK(16);
    // ... the bias and log_std gradients, which every wavefront holds for its own rows, summed in wavefront order through LDS
    const lptr sums = (lptr)lds_raw;        // [WAVES][N_SUMS]; the weights are no longer needed
#pragma unroll
    for (int nt = 0; nt < 4; nt++) { s1[nt] = groups_sum(s1[nt]); s2[nt] = groups_sum(s2[nt]); }
    s3 = groups_sum(s3); gls = groups_sum(gls);
    if (kk == 0) {
#pragma unroll
        for (int nt = 0; nt < 4; nt++) { sums[wave * N_SUMS + 16 * nt + r] = s1[nt]; sums[wave * N_SUMS + H + 16 * nt + r] = s2[nt]; }
        sums[wave * N_SUMS + 2 * H + r] = s3; sums[wave * N_SUMS + 2 * H + MAX_OUT + r] = gls;
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
    RLT_TICK(17);
    if (K.xr.enabled)       // the block joins those of the workgroups on this XCD: eight blocks of sums per network leave the launch
        rlt_xcd_group_reduce<THREADS>(K.xr, xgroup, block >> 3, n_blocks >> 3, xepoch, A.partial + (size_t)(block & 7) * A.count, A.count,
                                      (second ? K.xsum[1] : K.xsum[0]) + (size_t)(block & 7) * A.count, (__attribute__((address_space(3))) int*)((lptr)lds_raw + 4 * N_SUMS));
    RLT_TICK(18);
#ifdef RLT_SMALL_PROFILE
    __builtin_amdgcn_s_waitcnt(0);
    if (threadIdx.x == 0) rlt_small_spans[blockIdx.x][1] = wall_clock64();
#endif
}

// where the elements of a block of partial sums go; overwrite: gradient = sum instead of gradient += sum (for a caller that would zero the gradient first)
struct SmallTargets { float* dW1; float* db1; float* dW2; float* db2; float* dW3; float* db3; float* extra; int in, out, n_extra; float extra_scale, extra_offset; int overwrite;
                      const float* partial; int groups, count, blocks; };
// gradient[e] (+)= sum over the workgroups' partial values, in workgroup order: a block of 256 threads handles 64 elements, four threads
// per element each sum a quarter of the workgroups and are combined in a fixed order. Blocks [0, T0.blocks) serve T0, the rest T1.
__global__ __launch_bounds__(256) void mlp3s_reduce_kernel(SmallTargets T0, SmallTargets T1) {
    __shared__ float part[4][64];
    const bool second = (int)blockIdx.x >= T0.blocks;
    const SmallTargets& T = second ? T1 : T0;
    const int el = threadIdx.x & 63, qtr = threadIdx.x >> 6, e = (second ? blockIdx.x - T0.blocks : blockIdx.x) * 64 + el, count = T.count, groups = T.groups;
    const int ec = e < count ? e : count - 1;
    const int per = (groups + 3) / 4, g0 = qtr * per, g1 = min(groups, g0 + per);
    const float* __restrict__ partial = T.partial;
    float s = 0.f;
    for (int gb = g0; gb < g1; gb += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = partial[(size_t)min(gb + u, g1 - 1) * count + ec];
#pragma unroll
        for (int u = 0; u < 8; u++) s += (gb + u < g1) ? v[u] : 0.f;
    }
    part[qtr][el] = s;
    __syncthreads();
    if (qtr != 0 || e >= count) return;
    float total = (part[0][el] + part[1][el]) + (part[2][el] + part[3][el]);
    float* slot = nullptr;
    int i = e, n = H * T.in;
    if (i < n) slot = T.dW1 + i;
    else if ((i -= n) < H) slot = T.db1 + i;
    else if ((i -= H) < H * H) slot = T.dW2 ? T.dW2 + i : nullptr;      // a two-layer network has no middle layer: its block entries are skipped
    else if ((i -= H * H) < H) slot = T.db2 ? T.db2 + i : nullptr;
    else if ((i -= H) < T.out * H) slot = T.dW3 + i;
    else if ((i -= T.out * H) < T.out) slot = T.db3 + i;
    else if ((i -= T.out) < T.n_extra && T.extra) { slot = T.extra + i; total = total * T.extra_scale + T.extra_offset; }
    if (slot) *slot = T.overwrite ? total : *slot + total;
}

bool hidden_act_ok(int a) { return a == RLT_ACT_RELU || a == RLT_ACT_TANH || a == RLT_ACT_FAST_TANH; }
bool out_act_ok(int a) { return a == RLT_ACT_IDENTITY || a == RLT_ACT_RELU || a == RLT_ACT_TANH || a == RLT_ACT_FAST_TANH || a == RLT_ACT_SIGMOID; }

struct SmallJob { const rlt_dense_layer* L; int n_layers; SmallArgs a; float* extra; int n_extra; float extra_scale, extra_offset; int overwrite; };

bool shape_ok(const rlt_dense_layer* L, int n) {
    if (L && n == 2)
        return L[0].in_dim >= 1 && L[0].in_dim <= MAX_IN && L[0].out_dim == H && L[1].in_dim == H && L[1].out_dim >= 1 && L[1].out_dim <= MAX_OUT &&
               hidden_act_ok(L[0].activation) && out_act_ok(L[1].activation);
    return L && n == 3 && L[0].in_dim >= 1 && L[0].in_dim <= MAX_IN && L[0].out_dim == H && L[1].in_dim == H && L[1].out_dim == H && L[2].in_dim == H &&
           L[2].out_dim >= 1 && L[2].out_dim <= MAX_OUT && L[0].activation == L[1].activation && hidden_act_ok(L[0].activation) && out_act_ok(L[2].activation);
}
int tile_bucket(int in) { return in <= 32 ? 2 : in <= 64 ? 4 : MAX_NT1; }

// Where each tensor of an optimiser lies in the job's block of partial sums [dW1 | db1 | dW2 | db2 | dW3 | db3 | extra]: a tensor may span
// several of the six gradient buffers where those follow each other in memory; the job's extra values (a gradient with its own scale
// and offset) must be a tensor of their own. False unless the tensors cover all of these exactly once: then the optimiser's launch
// can add the blocks up itself.
bool map_step(const SmallJob& job, const rlt_mlp3s_step& S, bool extra_is_gradient, uint32_t* offsets, float* scales, float* adds) {
    if (!S.tensors || S.n < 1 || S.n > 12 || job.n_layers != 3) return false;
    const rlt_dense_layer* L = job.L;
    const float* seg[6] = {L[0].d_weights, L[0].d_biases, L[1].d_weights, L[1].d_biases, L[2].d_weights, L[2].d_biases};
    const uint32_t size[6] = {(uint32_t)(H * L[0].in_dim), H, H * H, H, (uint32_t)(L[2].out_dim * H), (uint32_t)L[2].out_dim};
    uint32_t off[6], covered = 0;
    for (int k = 0, o = 0; k < 6; o += size[k], k++) off[k] = o;
    bool extra_covered = false;
    for (int i = 0; i < S.n; i++) {
        const rlt_adam_tensor& T = S.tensors[i];
        if (T.polyak_target) return false;
        if (extra_is_gradient && job.extra && T.gradient == job.extra) {
            if (extra_covered || T.count != (uint32_t)job.n_extra) return false;
            extra_covered = true;
            offsets[i] = (uint32_t)(job.a.count - N_EXTRA); scales[i] = job.extra_scale; adds[i] = job.extra_offset;
            continue;
        }
        int s = 0;
        while (s < 6 && seg[s] != T.gradient) s++;
        if (s == 6) return false;
        uint32_t cnt = 0;
        for (int k = s; k < 6 && cnt < T.count && seg[k] == seg[s] + cnt; k++) {
            if (covered & (1u << k)) return false;
            covered |= 1u << k; cnt += size[k];
        }
        if (cnt != T.count) return false;
        offsets[i] = off[s]; scales[i] = 1.0f; adds[i] = 0.0f;
    }
    return covered == 63u && extra_covered == (extra_is_gradient && job.extra != nullptr);
}

// one or two networks in one launch; two only if they share the hidden activation and the input-width bucket. `steps` (optional, one per
// job): the optimisers' steps follow in one launch that reads the blocks of partial sums itself (a gradient's extra values only for job 0;
// job 1's single extra value is an output); *stepped tells whether they did, else the gradients were formed and the caller steps.
int launch(rlt_rocm_device* device, SmallJob* jobs, int n_jobs, const rlt_mlp3s_step* steps = nullptr, bool* stepped = nullptr) {
    if (stepped) *stepped = false;
    int groups[2] = {0, 0};
    size_t offset[2] = {0, 0}, total = 0;
    for (int j = 0; j < n_jobs; j++) {
        const rlt_dense_layer* L = jobs[j].L; SmallArgs& a = jobs[j].a;
        const int n = jobs[j].n_layers, last = n - 1;
        RLT_REQUIRE((n == 2 || n == 3) && n == jobs[0].n_layers);
        for (int l = 0; l < n; l++) RLT_REQUIRE(L[l].weights && L[l].biases && L[l].d_weights && L[l].d_biases);
        a.in = L[0].in_dim; a.out = L[last].out_dim; a.act3 = L[last].activation;
        a.W1 = L[0].weights; a.b1 = L[0].biases; a.W2 = n == 3 ? L[1].weights : nullptr; a.b2 = n == 3 ? L[1].biases : nullptr; a.W3 = L[last].weights; a.b3 = L[last].biases;
        a.count = H * a.in + H + H * H + H + a.out * H + a.out + N_EXTRA;
        const int rounds = (a.batch + ROWS - 1) / ROWS, share = device->compute_units / n_jobs;
        groups[j] = rounds < share ? rounds : share;
        offset[j] = total; total += ((size_t)groups[j] * a.count + 63) & ~(size_t)63;
    }
    const int bucket = tile_bucket(jobs[0].a.in), act = jobs[0].L[0].activation;
    if (n_jobs == 2 && (tile_bucket(jobs[1].a.in) != bucket || jobs[1].L[0].activation != act)) return RLT_E_UNSUPPORTED;
    const size_t lds_bytes = lds_floats(bucket) * sizeof(float);
    if (lds_bytes > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    // the optimisers' steps follow in one launch that adds the blocks of partial sums up itself, where the tensors allow
    uint32_t offsets[2][12]; float scales[2][12], adds[2][12];
    const bool steps_mapped = steps && n_jobs == 2 && jobs[0].overwrite && jobs[1].overwrite && (!jobs[1].extra || jobs[1].n_extra == 1) &&
                              map_step(jobs[0], steps[0], true, offsets[0], scales[0], adds[0]) && map_step(jobs[1], steps[1], false, offsets[1], scales[1], adds[1]);
    SmallLaunch K = {};
    // sums per XCD inside the launch: where workgroup i runs on XCD i % 8, every network's workgroups are a multiple of 8 (at most 32 per XCD)
    // and the grid is resident as a whole
    bool xcd_sums = device->update_tail && device->xcd_stride == 8 && groups[0] + groups[n_jobs - 1] * (n_jobs - 1) <= device->compute_units;
    size_t xsum_offset[2] = {0, 0};
    for (int j = 0; j < n_jobs; j++) {
        xcd_sums = xcd_sums && groups[j] % RLT_XCD_GROUPS == 0 && groups[j] >= 2 * RLT_XCD_GROUPS && groups[j] <= RLT_XCD_GROUPS * RLT_XCD_MAX_MEMBERS;
        xsum_offset[j] = total; total += ((size_t)RLT_XCD_GROUPS * jobs[j].a.count + 63) & ~(size_t)63;
    }
    void* scratch = nullptr;
    int rc = rlt_scratch(device, total * sizeof(float), &scratch);
    if (rc) return rc;
    for (int j = 0; j < n_jobs; j++) jobs[j].a.partial = (float*)scratch + offset[j];
    if (xcd_sums) {
        void* counters = nullptr;
        if ((rc = rlt_counters(device, &counters))) return rc;
        K.xr.enabled = 1; K.xr.max_poll = device->wait_limit; K.xr.words = (uint32_t*)counters + RLT_XCD_WORDS_OFFSET; K.xr.fault = device->fault;
        for (int j = 0; j < n_jobs; j++) K.xsum[j] = (float*)scratch + xsum_offset[j];
        device->fault_armed = 1;
    }
    K.a0 = jobs[0].a; K.a1 = jobs[n_jobs - 1].a; K.groups0 = groups[0];
    const int grid = groups[0] + (n_jobs == 2 ? groups[1] : 0);
    const bool two_layers = jobs[0].n_layers == 2;
#define RLT_LAUNCH_SMALL_AS(ACT, NT, LAYERS)                                                                                                                    \
    do {                                                                                                                                                        \
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(mlp3s_kernel<ACT, NT, LAYERS>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes)); \
        hipLaunchKernelGGL((mlp3s_kernel<ACT, NT, LAYERS>), dim3(grid), dim3(THREADS), lds_bytes, device->stream, K);                                         \
    } while (0)
#define RLT_LAUNCH_SMALL(ACT, NT)                                                                                                                               \
    do {                                                                                                                                                        \
        if (two_layers) RLT_LAUNCH_SMALL_AS(ACT, NT, 2); else RLT_LAUNCH_SMALL_AS(ACT, NT, 3);                                                                  \
    } while (0)
    switch (act) {
        case RLT_ACT_RELU: if (bucket == 2) RLT_LAUNCH_SMALL(RLT_ACT_RELU, 2); else if (bucket == 4) RLT_LAUNCH_SMALL(RLT_ACT_RELU, 4); else RLT_LAUNCH_SMALL(RLT_ACT_RELU, MAX_NT1); break;
        case RLT_ACT_TANH: if (bucket == 2) RLT_LAUNCH_SMALL(RLT_ACT_TANH, 2); else if (bucket == 4) RLT_LAUNCH_SMALL(RLT_ACT_TANH, 4); else RLT_LAUNCH_SMALL(RLT_ACT_TANH, MAX_NT1); break;
        default: if (bucket == 2) RLT_LAUNCH_SMALL(RLT_ACT_FAST_TANH, 2); else if (bucket == 4) RLT_LAUNCH_SMALL(RLT_ACT_FAST_TANH, 4); else RLT_LAUNCH_SMALL(RLT_ACT_FAST_TANH, MAX_NT1); break;
    }
#undef RLT_LAUNCH_SMALL
#undef RLT_LAUNCH_SMALL_AS
    if ((rc = rlt_launch_status(device))) return rc;
    const float* sums[2]; int n_sums[2];      // what is left to add up: the workgroups' blocks, or one block per XCD
    for (int j = 0; j < n_jobs; j++) { sums[j] = xcd_sums ? K.xsum[j] : jobs[j].a.partial; n_sums[j] = xcd_sums ? RLT_XCD_GROUPS : groups[j]; }
    if (steps_mapped) {
        rlt_adam_source src[2] = {};
        for (int j = 0; j < 2; j++) { src[j].partial = sums[j]; src[j].groups = n_sums[j]; src[j].block_stride = jobs[j].a.count; src[j].offsets = offsets[j]; src[j].scales = scales[j]; src[j].adds = adds[j]; }
        if (jobs[1].extra) { src[1].extra_out = jobs[1].extra; src[1].extra_offset = (uint32_t)(jobs[1].a.count - N_EXTRA); src[1].extra_scale = jobs[1].extra_scale; }
        if (stepped) *stepped = true;
        return rlt_adam_step_pair(device, steps[0].tensors, steps[0].n, steps[0].parameters, steps[0].age, steps[1].tensors, steps[1].n, steps[1].parameters, steps[1].age, &src[0], &src[1]);
    }
    SmallTargets T[2] = {};
    int blocks = 0;
    for (int j = 0; j < n_jobs; j++) {
        const rlt_dense_layer* L = jobs[j].L; const SmallArgs& a = jobs[j].a;
        const int count = jobs[j].extra ? a.count : a.count - N_EXTRA;      // the extra slots sit at the end of a block
        const int last = jobs[j].n_layers - 1;
        T[j] = {L[0].d_weights, L[0].d_biases, last == 2 ? L[1].d_weights : nullptr, last == 2 ? L[1].d_biases : nullptr, L[last].d_weights, L[last].d_biases, jobs[j].extra, a.in, a.out, jobs[j].n_extra,
                jobs[j].extra_scale, jobs[j].extra_offset, jobs[j].overwrite, sums[j], n_sums[j], a.count, (count + 63) / 64};
        blocks += T[j].blocks;
    }
    if (n_jobs == 1) T[1] = T[0];
    hipLaunchKernelGGL(mlp3s_reduce_kernel, dim3(blocks), dim3(256), 0, device->stream, T[0], T[1]);
    return rlt_launch_status(device);
}

SmallJob plain_job(const rlt_dense_layer* L, int n_layers, const float* x, int ldx, float* y, int ldy, const float* d_output, int ldd, const float* target, int ldt, float mse_scale,
                   int batch, int overwrite, const uint32_t* rows, float* d_input = nullptr, int ld_di = 0) {
    SmallJob job = {};
    job.L = L; job.n_layers = n_layers; job.overwrite = overwrite; job.a.d_input = d_input; job.a.ld_di = ld_di;
    SmallArgs& a = job.a;
    a.rows = rows; a.x = x; a.ldx = ldx; a.batch = batch; a.y = y; a.ldy = ldy;
    a.loss = target ? LOSS_MSE : LOSS_GIVEN; a.d_output = d_output; a.ldd = ldd; a.target = target; a.ldt = ldt; a.mse_scale = mse_scale;
    return job;
}
SmallJob ppo_actor_job(const rlt_dense_layer* L, const float* x, int ldx, float* means, int ld_means, const float* log_std, const float* actions, int ld_actions,
                       const float* log_probs, int ld_lp, const float* advantages, int ld_adv, const float* stats, const rlt_ppo_parameters* P, float* d_log_std,
                       float log_std_gradient_offset, int batch, int overwrite, const uint32_t* rows) {
    SmallJob job = {};
    job.L = L; job.n_layers = 3; job.overwrite = overwrite; job.extra = d_log_std; job.n_extra = L[2].out_dim; job.extra_scale = 1.0f; job.extra_offset = log_std_gradient_offset;
    SmallArgs& a = job.a;
    a.rows = rows; a.x = x; a.ldx = ldx; a.batch = batch; a.y = means; a.ldy = ld_means;
    a.loss = LOSS_PPO; a.log_std = log_std; a.actions = actions; a.ld_actions = ld_actions; a.log_probs = log_probs; a.ld_lp = ld_lp;
    a.advantages = advantages; a.ld_adv = ld_adv; a.stats = stats;
    a.epsilon_clip = P->epsilon_clip; a.advantage_epsilon = P->advantage_epsilon; a.normalize_advantage = P->normalize_advantage;
    return job;
}
}  // namespace

bool rlt_mlp3s_supported(const rlt_dense_layer* L, int n) { return shape_ok(L, n); }

int rlt_mlp3s_partial_count(int in_dim, int out_dim) { return H * in_dim + H + H * H + H + out_dim * H + out_dim + N_EXTRA; }

int rlt_mlp3s_reduce(rlt_rocm_device* device, const rlt_dense_layer* L, const float* partial, int groups, int overwrite, float* extra, int n_extra, float extra_scale,
                     float extra_offset) {
    for (int l = 0; l < 3; l++) RLT_REQUIRE(L[l].d_weights && L[l].d_biases);
    const int in = L[0].in_dim, out = L[2].out_dim, count = rlt_mlp3s_partial_count(in, out);
    SmallTargets T = {L[0].d_weights, L[0].d_biases, L[1].d_weights, L[1].d_biases, L[2].d_weights, L[2].d_biases, extra, in, out, n_extra, extra_scale, extra_offset, overwrite,
                      partial, groups, count, ((extra ? count : count - N_EXTRA) + 63) / 64};
    hipLaunchKernelGGL(mlp3s_reduce_kernel, dim3(T.blocks), dim3(256), 0, device->stream, T, T);
    return rlt_launch_status(device);
}

int rlt_mlp3s_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* L, int n, const float* x, int ldx, float* y, int ldy, const float* d_output, int ldd,
                               const float* target, int ldt, float mse_scale, int batch, float* d_input, int ldi) {
    if (!shape_ok(L, n)) return RLT_E_UNSUPPORTED;
    SmallJob job = plain_job(L, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch, 0, nullptr, d_input, ldi);
    return launch(device, &job, 1);
}

int rlt_mlp3s_ppo_actor(rlt_rocm_device* device, const rlt_dense_layer* L, int n, const float* x, int ldx, float* means, int ld_means, const float* log_std,
                        const float* actions, int ld_actions, const float* log_probs, int ld_lp, const float* advantages, int ld_adv, const float* stats,
                        const rlt_ppo_parameters* P, float* d_log_std, float log_std_gradient_offset, int batch) {
    if (!shape_ok(L, n) || n != 3) return RLT_E_UNSUPPORTED;
    SmallJob job = ppo_actor_job(L, x, ldx, means, ld_means, log_std, actions, ld_actions, log_probs, ld_lp, advantages, ld_adv, stats, P, d_log_std,
                                 log_std_gradient_offset, batch, 0, nullptr);
    return launch(device, &job, 1);
}

bool rlt_mlp3s_pair_supported(const rlt_dense_layer* a, int n_a, const rlt_dense_layer* b, int n_b) {
    return n_a == 3 && n_b == 3 && shape_ok(a, n_a) && shape_ok(b, n_b) && a[0].activation == b[0].activation && tile_bucket(a[0].in_dim) == tile_bucket(b[0].in_dim);
}

int rlt_mlp3s_ppo_actor_critic(rlt_rocm_device* device, const rlt_dense_layer* actor, int n_actor, const float* x, float* means, int ld_means,
                               const float* log_std, const float* actions, const float* log_probs, const float* advantages,
                               const float* stats, const rlt_ppo_parameters* P, float* d_log_std, float log_std_gradient_offset,
                               const rlt_dense_layer* critic, int n_critic, const float* x_critic, float* values, int ld_values,
                               const float* target_values, float mse_scale, float* out_critic_loss, int ld, const uint32_t* rows, int batch,
                               const float* actor_std_mean, const float* actor_std_precision, const float* critic_std_mean, const float* critic_std_precision,
                               const rlt_mlp3s_step* steps, bool* stepped) {
    if (!rlt_mlp3s_pair_supported(actor, n_actor, critic, n_critic) || (out_critic_loss && critic[2].out_dim != 1)) return RLT_E_UNSUPPORTED;
    SmallJob jobs[2] = {ppo_actor_job(actor, x, ld, means, ld_means, log_std, actions, ld, log_probs, ld, advantages, ld, stats, P, d_log_std,
                                      log_std_gradient_offset, batch, 1, rows),
                        plain_job(critic, 3, x_critic, ld, values, ld_values, nullptr, 0, target_values, ld, mse_scale, batch, 1, rows)};
    if (out_critic_loss) { jobs[1].extra = out_critic_loss; jobs[1].n_extra = 1; jobs[1].extra_scale = 1.0f / (float)batch; jobs[1].extra_offset = 0.0f; }
    jobs[0].a.std_mean = actor_std_mean; jobs[0].a.std_precision = actor_std_mean ? actor_std_precision : nullptr;
    jobs[1].a.std_mean = critic_std_mean; jobs[1].a.std_precision = critic_std_mean ? critic_std_precision : nullptr;
    return launch(device, jobs, 2, steps, stepped);
}

#ifdef RLT_SMALL_PROFILE
extern "C" int rlt_mlp3s_spans(unsigned long long* out) { return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(rlt_small_spans), sizeof(unsigned long long) * 1024); }
extern "C" int rlt_mlp3s_ticks(unsigned long long* out) { return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(rlt_small_ticks), sizeof(unsigned long long) * 32); }
#endif
