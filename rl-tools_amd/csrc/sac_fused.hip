// Persistent SAC-on-Pendulum training loop: N reference loop steps in ONE launch.
//
// reference: rl/algorithms/sac/loop/core/operations_generic.h:110-155 (step), the runner step it calls
// (rl/components/off_policy_runner/operations_generic.h:183-238, operations_generic_per_env.h:8-108), gather_batch (:240-430),
// train_critic / update_critic_targets / train_actor (rl/algorithms/sac/operations_generic.h:243-527). The reference's CUDA
// example replays three captured graphs of ~100 tiny launches per step (src/rl/environments/pendulum/sac/cuda/sac.cu:122-164);
// at batch 256 and width 64 a step is 43 MFLOP, so launch latency, not arithmetic, sets its speed.
//
// Here G = batch/16 workgroups stay resident for the whole run. Each owns 16 samples of the batch and keeps a copy of all
// five networks (actor, two critics, two target critics) in LDS next to its activations; the 64x64 contractions run on
// v_mfma_f32_16x16x4_f32, the layers with <= 4 inputs or <= 2 outputs on one matrix instruction or on the vector ALU.
// Observation (3) and action (1) widths and the hidden width (64) are compile-time constants, so every LDS address is an
// immediate offset. Per loop step:
//   S0  wavefront 0 of every workgroup redundantly advances the single environment (actor on one observation, dynamics,
//       reward) so that the new transition is known everywhere without a grid barrier; workgroup 0 writes it to the replay
//       ring. The replay rows of this step's batch were requested from memory before S0 and arrive while it runs.
//   S1  next actions + log-probabilities from the actor; both target critics; TD target; both critics forward + backward
//       -> per-workgroup partial gradients
//   S2  each workgroup sums a slice of the partial gradients (fixed order), applies Adam and the polyak target update;
//       then every workgroup reloads the critics and targets into LDS
//   S3  actor forward, both critics forward / backward_input, min-Q routing, sample_and_squash backward, actor backward
//       -> partial gradients
//   S4  Adam on the actor slice and on log_alpha; then every workgroup reloads the actor
// Two wave groups of four wavefronts each work on independent networks (critic 0 / critic 1) at the same time.
//
// The workgroups exchange partial gradients (S1 -> S2, S3 -> S4) and updated parameters (S2 -> S3, S4 -> next step) through
// memory with one word per workgroup and exchange instead of grid barriers with agent-scope release / acquire (which write back
// and invalidate the whole L2 of the XCD and cost 3.2 us one way for 8 KB between two CUs, against 1.6 us for this): a
// workgroup waits until its own stores have completed (s_waitcnt), sets its word, and the consumers, once all words are set,
// load the data past their CU's vector cache. Up to 32 workgroups are placed on ONE XCD (every 8th workgroup of an 8x larger
// grid; the others exit at once): there plain stores land in the L2 that all of them share, and non-temporal loads, which
// never allocate in the vector cache, read it. Larger grids spread over the XCDs, store through to memory and load with agent
// scope. Any address that another workgroup may have rewritten is read in one of these two ways everywhere in the kernel.
// No slot is overwritten before its consumer has read it: a workgroup rewrites its partial gradients of a phase only after
// every consumer has announced the parameters it made from them, and a consumer rewrites parameters only after every workgroup
// has announced its next partial gradients, which they write after having read the old parameters.
// The target critics are not exchanged at all: every workgroup applies the polyak update to its own LDS copy, with the same
// arithmetic on the same bits as the owner of the element applies to the arena in memory.
#include "common.h"
#include "rng.h"
#include <cstdio>
#include <cstdlib>
#include <cstring>

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) float* lptr;      // LDS address (32 bit): keeps every access a ds_* instruction

extern __shared__ __attribute__((aligned(16))) float rlt_sac_lds[];

namespace {

constexpr int OBS = 3, ACT = 1, D = OBS + ACT;
constexpr int H = 64;           // hidden width this kernel is built for
constexpr int ROWS = 16;        // samples per workgroup (one MFMA tile of rows)
constexpr int AS = H + 1;       // LDS row stride of activation buffers
constexpr int XS = 17;          // LDS row stride of network inputs
constexpr int THREADS = 512;
constexpr int MAX_G = 64;
constexpr int R = 2 * OBS + ACT + 3;    // floats per replay row
constexpr int MAX_PACKED_G = 32;        // workgroups that fit on one XCD (32 CUs) with one workgroup per CU

// A 3-layer network IN -> H -> H -> OUT: offsets in its flat arena [W1|b1|W2|b2|W3|b3] and in the workgroup's LDS copy. The
// LDS rows are padded to odd strides so that the 16 rows a tile reads side by side fall into different banks; W1 rows are
// 5 wide with zeros beyond IN, so that the one matrix instruction of layer 1 can always read 4 columns.
template <int IN_, int OUT_>
struct Net {
    static constexpr int IN = IN_, OUT = OUT_;
    static constexpr int w1 = 0, b1 = H * IN, w2 = b1 + H, b2 = w2 + H * H, w3 = b2 + H, b3 = w3 + OUT * H, total = b3 + OUT;
    static constexpr int LD1 = 5, LD2 = H + 1;
    static constexpr int lw1 = 0, lb1 = H * LD1, lw2 = lb1 + H, lb2 = lw2 + H * LD2, lw3 = lb2 + H, lb3 = lw3 + OUT * LD2;
    static constexpr int ltotal = (lb3 + OUT + 3) & ~3;
    static constexpr int per_thread = (total + THREADS - 1) / THREADS;
    static_assert(IN <= 4 && OUT <= 2, "layer 1 is one 4-deep matrix instruction; layer 3 is done on the vector ALU");
    // arena index -> offset in the LDS copy
    static __device__ __forceinline__ int slot(int idx) {
        if (idx < b1) return lw1 + (idx / IN) * LD1 + idx % IN;
        if (idx < w2) return lb1 + idx - b1;
        if (idx < b2) { const int j = idx - w2; return lw2 + (j >> 6) * LD2 + (j & 63); }
        if (idx < w3) return lb2 + idx - b2;
        if (idx < b3) { const int j = idx - w3; return lw3 + (j >> 6) * LD2 + (j & 63); }
        return lb3 + idx - b3;
    }
};
using NA = Net<OBS, 2 * ACT>;
using NC = Net<D, 1>;
constexpr int N_PARTIAL = 2 * NC::total + NA::total + 8;   // per workgroup: critic 0, critic 1, actor gradients; alpha gradient; 2 loss sums

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
    int batch, n_steps, lds_floats;
    rlt_pendulum_runner runner;
    rlt_replay_buffer rb;
    float* partial;            // [G + 1][N_PARTIAL], row G stays zero
    unsigned* fault;           // set when a workgroup gave up waiting
    unsigned max_poll;         // polls after which a waiting workgroup gives up: bounded wait for another workgroup's data (about a second by default), then the run is abandoned
    unsigned* xcd_mask;        // bit x set: some workgroup of this launch ran on XCD x
    unsigned* ready;           // [4][64] per exchange kind and workgroup: the sequence number of the last completed exchange
    // optional host-drawn randomness (parity runs); NULL -> counter-based device RNG
    const float* rollout_noise; const float* initial_states; const uint32_t* sample_offsets;
    const float* noise_critic; const float* noise_actor;
    uint64_t seed, step_offset;
    float* out_critic_loss;    // [n_steps][2] optional
    // batch views for inspection (optional): last gathered batch / targets
    float* out_oab; float* out_rewards; uint8_t* out_terminated; float* out_target;
    unsigned long long* phase_ticks;   // [16] optional: constant-rate clock ticks workgroup 0 spent in each phase, summed over the steps
    unsigned long long* stage_ticks;   // [48] optional: the same clock between the barrier-separated stages of the critic and actor phases (thread 0)
    // optional: the draws every step used (host-drawn or the kernel's own), so that a run can be replayed elsewhere
    float* drawn_rollout; float* drawn_initial; uint32_t* drawn_offsets; float* drawn_noise_c; float* drawn_noise_a;
};

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

template <int CTRL>
__device__ __forceinline__ float dpp(float x) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true)); }
// sum over each row of 16 lanes, result in all 16 (quad swaps, then mirror within 8, then within 16)
__device__ __forceinline__ float row16_sum(float x) {
    asm volatile("" : "+v"(x));      // keeps a producing multiplication out of the first addition: all lanes of the row then hold the same sum bit for bit
    x += dpp<0xB1>(x); x += dpp<0x4E>(x); x += dpp<0x141>(x); x += dpp<0x140>(x);
    return x;
}
// sum over the four rows of a wavefront (lanes l, l^16, l^32, l^48), result in all
__device__ __forceinline__ float kk_sum(float x) { asm volatile("" : "+v"(x)); x += __shfl_xor(x, 16, 64); x += __shfl_xor(x, 32, 64); return x; }

// ---- exchange between workgroups
// loads of data that another workgroup may have rewritten: never from this CU's vector cache
template <bool PACKED>
__device__ __forceinline__ float get_shared(const float* p) {
    if (PACKED) return __builtin_nontemporal_load(p);                                   // never allocates in the vector cache; reads the XCD's L2
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);            // past the vector cache, coherent across XCDs
}
template <bool PACKED>
__device__ __forceinline__ void put_shared(float* p, float v) {
    if (PACKED) *p = v;                                                                 // lands in the XCD's L2, which every consumer reads
    else __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);          // written through to memory
}
// the target update, in one place so that the owner of an element and every workgroup's LDS copy compute the same bits
__device__ __forceinline__ float polyak_step(float polyak, float target, float source) { return __builtin_fmaf(polyak, target, (1.0f - polyak) * source); }
// after a failed wait: tell every workgroup (they look at this word while they wait) and this workgroup (it leaves the step loop)
__device__ __forceinline__ void give_up(unsigned* fault, __attribute__((address_space(3))) int* abort_flag) {
    __hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *abort_flag = 1;
}
// true while waiting may go on: not too long yet, and no workgroup has given up
__device__ __forceinline__ bool keep_waiting(unsigned& tries, const unsigned* fault, unsigned max_poll) {
    __builtin_amdgcn_s_sleep(1);      // a waiting wavefront should not keep the memory system busy
    ++tries;
    if (tries >= max_poll) return false;
    if ((tries & 63u) == 0u && __hip_atomic_load(fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return false;
    return true;
}
// One word per workgroup and exchange kind holds the sequence number of the last exchange the workgroup has completed its stores
// for. announce: wait for this wavefront's stores (and loads) to complete, meet the other wavefronts, set the word.
constexpr int READY_STRIDE = 64;     // words per exchange kind (MAX_G)
enum { READY_CRITIC_GRADIENTS = 0, READY_CRITIC_PARAMETERS = 1, READY_ACTOR_GRADIENTS = 2, READY_ACTOR_PARAMETERS = 3 };
template <bool PACKED>
__device__ __forceinline__ void announce(unsigned* ready, int kind, int g, unsigned tag) {
    __builtin_amdgcn_s_waitcnt(0);
    rlt_lds_barrier();
    if (threadIdx.x == 0) {
        if (PACKED) ready[kind * READY_STRIDE + g] = tag;
        else __hip_atomic_store(ready + kind * READY_STRIDE + g, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
// wavefront 0 waits for all G words, the others wait for it at the workgroup barrier
__device__ __forceinline__ void await(const unsigned* ready, int kind, int G, unsigned tag, const unsigned* fault, __attribute__((address_space(3))) int* abort_flag, unsigned max_poll) {
    if (threadIdx.x < 64) {
        const unsigned* p = ready + kind * READY_STRIDE + min((int)threadIdx.x, G - 1);
        unsigned tries = 0;
        while (__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < tag) if (!keep_waiting(tries, fault, max_poll)) { give_up(const_cast<unsigned*>(fault), abort_flag); break; }
    }
    rlt_lds_barrier();
}

// The kernel's own draws (taken when the caller passes no host-drawn array): Philox groups (rng.h) of these streams under the
// launch's seed; the index is the global step (step_offset + step), times the batch size plus the sample where a draw is per sample.
enum { STREAM_INITIAL_STATE = 1, STREAM_ROLLOUT_NOISE = 3, STREAM_GATHER = 4, STREAM_NOISE_CRITIC = 5, STREAM_NOISE_ACTOR = 6 };
// standard normal from one group: Box-Muller on its first two words
__device__ __forceinline__ float randn_at(uint64_t seed, uint64_t stream, uint64_t index) {
    const rlt_u32x4 r = rlt_philox(seed, stream, index);
    return sqrtf(-2.0f * logf(rlt_u01(r.x))) * cosf(6.283185307179586f * rlt_u01(r.y));
}
__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }

// ---- passes over one network on the workgroup's 16 rows, by the four wavefronts of a wave group (w = wavefront within the
// group). Lane l of a wavefront: r = l & 15, kk = l >> 4; wavefront w owns the hidden units n = 16 w + r. A matrix instruction
// consumes 4 values of the reduction index, one per kk; lane group kk is given the contiguous range [16 kk, 16 kk + 16) of a
// 64-long reduction (any fixed assignment is valid as long as both operands agree). Result element v of lane l belongs to row
// 4 kk + v and column r of the tile. The stage functions contain no barrier; the caller separates them with __syncthreads().

// The weights a stage needs are loaded from the LDS copy into registers by a load_* function that the caller places BEFORE the
// barrier the stage waits behind (weights do not depend on the previous stage), so that after the barrier only activations are read.
struct Fwd1W { float w, b; };
struct Fwd2W { float b[16], bias, w3[2]; };
struct Bwd1W { float w3[2]; };
struct Bwd2W { float b[16], wa; };
template <class N>
__device__ __forceinline__ Fwd1W load_fwd1(lptr P, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    Fwd1W f; f.w = P[N::lw1 + n * N::LD1 + kk]; f.b = P[N::lb1 + n];
    return f;
}
template <class N>
__device__ __forceinline__ Fwd2W load_fwd2(lptr P, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    Fwd2W f;
#pragma unroll
    for (int s = 0; s < 16; s++) f.b[s] = P[N::lw2 + n * N::LD2 + kk * 16 + s];
    f.bias = P[N::lb2 + n];
#pragma unroll
    for (int c = 0; c < 2; c++) f.w3[c] = c < N::OUT ? P[N::lw3 + c * N::LD2 + n] : 0.f;
    return f;
}
template <class N>
__device__ __forceinline__ Bwd1W load_bwd1(lptr P, int w, int lane) {
    const int n = 16 * w + (lane & 15);
    Bwd1W f;
#pragma unroll
    for (int c = 0; c < 2; c++) f.w3[c] = c < N::OUT ? P[N::lw3 + c * N::LD2 + n] : 0.f;
    return f;
}
template <class N>
__device__ __forceinline__ Bwd2W load_bwd2(lptr P, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    Bwd2W f;
#pragma unroll
    for (int s = 0; s < 16; s++) f.b[s] = P[N::lw2 + (kk * 16 + s) * N::LD2 + n];
    f.wa = P[N::lw1 + n * N::LD1 + OBS];
    return f;
}

// layer 1: h1 = relu(x W1^T + b1)
__device__ __forceinline__ void forward_stage1(lptr x, lptr h1, const Fwd1W& f, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    const floatx4 acc = mfma16(x[r * XS + kk], f.w, zero);
#pragma unroll
    for (int v = 0; v < 4; v++) h1[(4 * kk + v) * AS + n] = fmaxf(acc[v] + f.b, 0.f);
}
// layer 2: h2 = relu(h1 W2^T + b2); layer 3 as per-wavefront partial dot products: part[(c*4 + w)*ROWS + row] = sum over the
// wavefront's 16 hidden units of h2[row][n] W3[c][n]
template <int OUT>
__device__ __forceinline__ void forward_stage2(lptr h1, lptr h2, lptr part, const Fwd2W& f, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    float a[16];
#pragma unroll
    for (int s = 0; s < 16; s++) a[s] = h1[r * AS + kk * 16 + s];
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 16; s++) acc = mfma16(a[s], f.b[s], acc);
    float hv[4];
#pragma unroll
    for (int v = 0; v < 4; v++) { hv[v] = fmaxf(acc[v] + f.bias, 0.f); h2[(4 * kk + v) * AS + n] = hv[v]; }
#pragma unroll
    for (int c = 0; c < OUT; c++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float t = row16_sum(hv[v] * f.w3[c]);
            if (r == 0) part[(c * 4 + w) * ROWS + 4 * kk + v] = t;
        }
    }
}
// output c of row `row` once the partial dot products are visible
template <class N>
__device__ __forceinline__ float net_output(lptr part, lptr P, int row, int c) {
    return ((part[(c * 4 + 0) * ROWS + row] + part[(c * 4 + 1) * ROWS + row]) + (part[(c * 4 + 2) * ROWS + row] + part[(c * 4 + 3) * ROWS + row])) + P[N::lb3 + c];
}

// backward, layer 3 and the gate of layer 2: dp2 = (dout W3) * relu'(h2); with WANT_W also dW3, db3, db2 of the 16 rows into the
// gradient arena Gd. dout is [ROWS][2] (gradient at the identity output).
template <class N, bool WANT_W, bool PK>
__device__ __forceinline__ void backward_stage1(lptr h2, lptr dp2, lptr dout, const Bwd1W& f, float* __restrict__ Gd, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    float wsum[N::OUT];
#pragma unroll
    for (int c = 0; c < N::OUT; c++) wsum[c] = 0.f;
    float dsum = 0.f;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int row = 4 * kk + v;
        const float hv = h2[row * AS + n];
        float g = 0.f;
#pragma unroll
        for (int c = 0; c < N::OUT; c++) { const float dc = dout[row * 2 + c]; g += dc * f.w3[c]; wsum[c] += dc * hv; }
        const float d = hv > 0.f ? g : 0.f;
        dp2[row * AS + n] = d;
        dsum += d;
    }
    if (WANT_W) {
#pragma unroll
        for (int c = 0; c < N::OUT; c++) { const float s = kk_sum(wsum[c]); if (kk == 0) put_shared<PK>(Gd + N::w3 + c * H + n, s); }
        const float s = kk_sum(dsum);
        if (kk == 0) put_shared<PK>(Gd + N::b2 + n, s);
        if (w == 0 && lane < N::OUT) { float t = 0.f; for (int i = 0; i < ROWS; i++) t += dout[i * 2 + lane]; put_shared<PK>(Gd + N::b3 + lane, t); }
    }
}
// backward, layer 2 weight gradient: dW2 = dp2^T h1, wavefront w owns rows [16w, 16w+16) of it
template <class N, bool PK>
__device__ __forceinline__ void backward_w2(lptr h1, lptr dp2, float* __restrict__ Gd, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    float a[4];
#pragma unroll
    for (int s = 0; s < 4; s++) a[s] = dp2[(4 * kk + s) * AS + n];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; s++) acc = mfma16(a[s], h1[(4 * kk + s) * AS + 16 * it + r], acc);
#pragma unroll
        for (int v = 0; v < 4; v++) put_shared<PK>(Gd + N::w2 + (16 * w + 4 * kk + v) * H + 16 * it + r, acc[v]);
    }
}
// backward, layer 1: d_h1 = dp2 W2 gated by relu'(h1) stays in registers and yields, with WANT_W, db1 and dW1 (vector ALU, IN <= 4
// columns) and, with WANT_DACT, the per-wavefront partial of the gradient wrt the action input column: part[w*ROWS + row]
template <class N, bool WANT_W, bool WANT_DACT, bool PK>
__device__ __forceinline__ void backward_l1(lptr x, lptr h1, lptr dp2, lptr part, const Bwd2W& f, float* __restrict__ Gd, int w, int lane) {
    const int r = lane & 15, kk = lane >> 4, n = 16 * w + r;
    float a[16];
#pragma unroll
    for (int s = 0; s < 16; s++) a[s] = dp2[r * AS + kk * 16 + s];
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 16; s++) acc = mfma16(a[s], f.b[s], acc);
    float d[4];
#pragma unroll
    for (int v = 0; v < 4; v++) d[v] = h1[(4 * kk + v) * AS + n] > 0.f ? acc[v] : 0.f;
    if (WANT_W) {
        const float s = kk_sum((d[0] + d[1]) + (d[2] + d[3]));
        if (kk == 0) put_shared<PK>(Gd + N::b1 + n, s);
#pragma unroll
        for (int i = 0; i < N::IN; i++) {
            float t = 0.f;
#pragma unroll
            for (int v = 0; v < 4; v++) t += d[v] * x[(4 * kk + v) * XS + i];
            t = kk_sum(t);
            if (kk == 0) put_shared<PK>(Gd + N::w1 + n * N::IN + i, t);
        }
    }
    if (WANT_DACT) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float t = row16_sum(d[v] * f.wa);
            if (r == 0) part[w * ROWS + 4 * kk + v] = t;
        }
    }
}

// copy of network parameters from the global arena into the padded LDS layout, in two halves: all loads are issued before the
// first store, so the whole copy costs about one memory round trip, and work that does not need the new values can run between
template <class N, int COUNT, bool PK>
__device__ __forceinline__ void load_nets(float (&v)[COUNT][N::per_thread], const float* const (&src)[COUNT], int tid) {
#pragma unroll
    for (int k = 0; k < COUNT; k++)
#pragma unroll
        for (int u = 0; u < N::per_thread; u++) { const int idx = tid + u * THREADS; v[k][u] = get_shared<PK>(src[k] + (idx < N::total ? idx : N::total - 1)); /* unconditional: a clamped duplicate load instead of a branch */ }
}
template <class N, int COUNT>
__device__ __forceinline__ void store_nets(lptr const (&dst)[COUNT], const float (&v)[COUNT][N::per_thread], int tid) {
#pragma unroll
    for (int u = 0; u < N::per_thread; u++) {
        const int idx = tid + u * THREADS;
        if (idx < N::total) {
            const int slot = N::slot(idx);
#pragma unroll
            for (int k = 0; k < COUNT; k++) dst[k][slot] = v[k][u];
        }
    }
}
// target networks in LDS: target = polyak * target + (1 - polyak) * source, source being freshly loaded parameters
template <class N, int COUNT>
__device__ __forceinline__ void polyak_nets(lptr const (&dst)[COUNT], const float (&v)[COUNT][N::per_thread], float polyak, int tid) {
#pragma unroll
    for (int u = 0; u < N::per_thread; u++) {
        const int idx = tid + u * THREADS;
        if (idx < N::total) {
            const int slot = N::slot(idx);
#pragma unroll
            for (int k = 0; k < COUNT; k++) dst[k][slot] = polyak_step(polyak, dst[k][slot], v[k][u]);
        }
    }
}
template <class N, int COUNT, bool PK>
__device__ __forceinline__ void cache_nets(lptr const (&dst)[COUNT], const float* const (&src)[COUNT], int tid) {
    float v[COUNT][N::per_thread];
    load_nets<N, COUNT, PK>(v, src, tid);
    store_nets<N, COUNT>(dst, v, tid);
}

// Adam on one element (nn/optimizers/adam/instance/operations_generic.h:26-72)
__device__ __forceinline__ float adam_element(const rlt_adam_parameters& p, float bc1, float bc2, float g, float& m, float& v, float param) {
    if (p.enable_gradient_clipping) g = clampf(g, -p.gradient_clip_value, p.gradient_clip_value);
    m = p.beta_1 * m + (1.0f - p.beta_1) * g;
    v = p.beta_2 * v + (1.0f - p.beta_2) * g * g;
    const float pre_sqrt = fmaxf(v * bc2, p.epsilon_sqrt);
    return param - p.alpha * bc1 * m / (sqrtf(pre_sqrt) + p.epsilon);
}

// sum over the workgroups' partial values of one or two gradient elements, in workgroup order; the loads of 16 workgroups are in
// flight together
template <int E, bool PK>
__device__ __forceinline__ void sum_partials(const float* __restrict__ partial, const int (&idx)[E], int G, float (&sum)[E]) {
#pragma unroll
    for (int e = 0; e < E; e++) sum[e] = 0.f;
    for (int w0 = 0; w0 < G; w0 += 16) {
        float pv[E][16];
#pragma unroll
        for (int e = 0; e < E; e++)
#pragma unroll
            for (int u = 0; u < 16; u++) pv[e][u] = get_shared<PK>(partial + (size_t)min(w0 + u, G) * N_PARTIAL + idx[e]);   // row G is all zeros: no select, no branch
        __builtin_amdgcn_sched_barrier(0);    // all loads are issued before the first add waits for one
#pragma unroll
        for (int e = 0; e < E; e++)
#pragma unroll
            for (int u = 0; u < 16; u++) sum[e] += pv[e][u];
    }
}

// LDS working set of one wave group
struct GroupLds {
    float a1[ROWS * AS], a2[ROWS * AS];   // activations kept for a backward pass with weight gradients
    float e1[ROWS * AS], e2[ROWS * AS];   // activations of evaluate-only and backward_input-only passes
    float dp2[ROWS * AS];                 // d_pre of layer 2
    float part[2 * 4 * ROWS];             // per-wavefront partial dot products
    float dout[ROWS * 2];                 // gradient at the network output
};
struct Shared {
    GroupLds grp[2];
    float actor_h1[ROWS * AS], actor_h2[ROWS * AS];   // the actor's activations on the batch observations, kept for its backward pass
    float actor_dout[ROWS * 2];
    float x[ROWS * XS];           // [obs | action] rows of the batch
    float nx[ROWS * XS];          // [next_obs | next_action] (S1), [obs | new action] (S3)
    float dout_actor_critic[ROWS * 2];   // -1/batch: the gradient the actor loss puts on both critics' outputs
    float new_row[16];            // the transition added this step
    unsigned long long ticks[16]; // per-phase clock ticks of this workgroup (profiling aid), flushed at the end
    unsigned long long sticks[48]; // per-stage clock ticks (profiling aid)
    int abort;                    // a wait for another workgroup failed: leave the step loop
    float alpha;                  // exp(log_alpha) of this step
    float rollout_eps[2];         // exploration noise of this step and the next (indexed by step parity)
    float bc[8];                  // Adam bias corrections of this step: actor, critic 0, critic 1, alpha
    float reward[ROWS], notdone[ROWS], next_logp[ROWS], y[ROWS], q[2][ROWS];
    float noise_c[ROWS], noise_a[ROWS], mean[ROWS], ls_raw[ROWS], act_pre[ROWS], act_a[ROWS];
};
typedef __attribute__((address_space(3))) Shared* sptr;

template <bool PACKED>
__global__ __launch_bounds__(THREADS) void sac_pendulum_loop_kernel(FusedArgs A) {
    if (PACKED && (blockIdx.x & 7)) return;      // only every 8th workgroup works: they share one XCD
    const sptr S = (sptr)rlt_sac_lds;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), grp = wave >> 2, w = wave & 3;
    const int g = PACKED ? blockIdx.x >> 3 : blockIdx.x, G = PACKED ? gridDim.x >> 3 : gridDim.x;
    const int B = A.batch;
    float* const my_partial = A.partial + (size_t)g * N_PARTIAL;
    if (threadIdx.x == 0) atomicOr(A.xcd_mask, 1u << (__builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xf));
    // LDS copies of all five networks, refreshed after the grid barrier that follows each optimiser phase
    const lptr w_actor = (lptr)rlt_sac_lds + ((sizeof(Shared) / 4 + 3) & ~3);
    const lptr w_critic0 = w_actor + NA::ltotal, w_critic1 = w_critic0 + NC::ltotal, w_target0 = w_critic1 + NC::ltotal, w_target1 = w_target0 + NC::ltotal;
    const lptr w_critic = grp == 0 ? w_critic0 : w_critic1, w_target = grp == 0 ? w_target0 : w_target1;
    // the wave group's buffers
    const lptr La1 = &S->grp[grp].a1[0], La2 = &S->grp[grp].a2[0], Le1 = &S->grp[grp].e1[0], Le2 = &S->grp[grp].e2[0];
    const lptr Ldp2 = &S->grp[grp].dp2[0], Lpart = &S->grp[grp].part[0], Ldout = &S->grp[grp].dout[0];
    const lptr part0 = &S->grp[0].part[0], part1 = &S->grp[1].part[0];
    const lptr Sx = &S->x[0], Snx = &S->nx[0], Ah1 = &S->actor_h1[0], Ah2 = &S->actor_h2[0];

    // padding columns and input buffers are read by matrix instructions against zero weights: they must hold finite values
    for (int i = tid; i < A.lds_floats; i += THREADS) ((lptr)rlt_sac_lds)[i] = 0.f;
    __syncthreads();
    {
        const lptr dst_a[1] = {w_actor}; const float* const src_a[1] = {A.actor_p};
        cache_nets<NA, 1, PACKED>(dst_a, src_a, tid);
        const lptr dst_c[4] = {w_critic0, w_critic1, w_target0, w_target1}; const float* const src_c[4] = {A.critic_p[0], A.critic_p[1], A.target_p[0], A.target_p[1]};
        cache_nets<NC, 4, PACKED>(dst_c, src_c, tid);
    }
    if (tid < ROWS) { S->dout_actor_critic[2 * tid] = -1.0f / (float)B; S->dout_actor_critic[2 * tid + 1] = 0.f; }   // d_output = -1/num_final_steps (sac/operations_generic.h:437-453)

    // single-environment state: every lane of every wavefront 0 carries it (uniform); replay cursor: every thread
    float th = A.runner.states[0], thd = A.runner.states[1], ep_return = A.runner.episode_return[0];
    unsigned ep_step = A.runner.episode_step[0]; int truncated = A.runner.truncated[0];
    unsigned rb_pos = A.rb.position[0], rb_ces = A.rb.current_episode_start[0]; int rb_full = A.rb.full[0];
    const unsigned cap = (unsigned)A.rb.capacity;
    // optimiser ages advance by exactly one per loop step: keep them in registers, write back at the end
    const uint32_t age_actor0 = *A.actor_age, age_c00 = *A.critic_age[0], age_c10 = *A.critic_age[1], age_alpha0 = *A.alpha_age;
    __syncthreads();

    if (tid == 0) {
        const float eps0 = A.rollout_noise ? A.rollout_noise[0] : randn_at(A.seed, STREAM_ROLLOUT_NOISE, A.step_offset);
        S->rollout_eps[0] = eps0;
        if (g == 0 && A.drawn_rollout) A.drawn_rollout[0] = eps0;
    }
    __syncthreads();
    unsigned long long t_prev = A.phase_ticks ? wall_clock64() : 0ull;
    const unsigned long long shader_clock_begin = A.phase_ticks ? clock64() : 0ull;
    auto tick = [&](int phase) {
        if (A.phase_ticks && g == 0 && threadIdx.x == 0) { const unsigned long long t = wall_clock64(); S->ticks[phase] += t - t_prev; t_prev = t; }
    };
    // finer clock for the stage profile: stage_begin() restarts it, stage(i) adds the time since the last call to slot i
    unsigned long long s_prev = 0ull;
    auto stage_begin = [&]() { if (A.stage_ticks && g == 0 && threadIdx.x == 0) s_prev = wall_clock64(); };
    auto stage = [&](int i) {
        if (A.stage_ticks && g == 0 && threadIdx.x == 0) { const unsigned long long t = wall_clock64(); S->sticks[i] += t - s_prev; s_prev = t; }
    };
    const int lane_invariant = lane, wave_base = wave << 6;
    for (int step = 0; step < A.n_steps; step++) {
        // Everything per-lane below derives from a lane index the optimiser cannot see through: otherwise it hoists hundreds of
        // per-lane addresses out of this loop and spills them.
        int lane = lane_invariant;
        asm volatile("" : "+v"(lane));
        const int tid = wave_base | lane;
        const uint64_t gstep = A.step_offset + (uint64_t)step;
        const unsigned seq = (unsigned)step + 1u;    // sequence number of this step's exchanges
        // ---- replay cursor after this step's add (replay_buffer add: position advances, full latches when it wraps)
        const unsigned new_pos = rb_pos; const int full_before = rb_full;
        rb_pos = rb_pos + 1 == cap ? 0u : rb_pos + 1;
        if (rb_pos == 0) rb_full = 1;
        // ---- request this step's batch rows and noise now; they are consumed after the environment step
        float gathered = 0.f; bool is_new = false; float noise_reg = 0.f;
        if (tid < ROWS * 16) {
            const int s = tid >> 4, j = tid & 15, sample = g * ROWS + s;
            const unsigned eligible = rb_full ? cap : rb_pos;
            const unsigned off = A.sample_offsets ? A.sample_offsets[(size_t)step * B + sample]
                                                  : rlt_uniform_below(rlt_philox(A.seed, STREAM_GATHER, gstep * (uint64_t)B + sample).x, eligible);
            if (j == 0 && A.drawn_offsets) A.drawn_offsets[(size_t)step * B + sample] = off;
            unsigned index = off;
            if (rb_full) { index = rb_pos + (unsigned)A.runner.episode_step_limit + off; index = index % cap; }
            if (index >= cap) index = 0;     // cannot happen for valid offsets; keeps the access in bounds
            is_new = index == new_pos;       // the row added in S0 may not have reached memory from workgroup 0: every workgroup holds its own copy
            if (j < R) gathered = get_shared<PACKED>(A.rb.data + (size_t)index * R + j);   // written by workgroup 0 in an earlier step
        } else if (tid < ROWS * 16 + 2 * ROWS) {
            const int s = tid & 15, sample = g * ROWS + s; const bool actor_phase = tid >= ROWS * 16 + ROWS;
            const float* src = actor_phase ? A.noise_actor : A.noise_critic;
            noise_reg = src ? src[(size_t)step * B + sample] : randn_at(A.seed, actor_phase ? STREAM_NOISE_ACTOR : STREAM_NOISE_CRITIC, gstep * (uint64_t)B + sample);
            float* const drawn = actor_phase ? A.drawn_noise_a : A.drawn_noise_c;
            if (drawn) drawn[(size_t)step * B + sample] = noise_reg;
        }
        // ================= S0: environment step (wavefront 0, identical in every workgroup) =================
        if (wave == 0) {
            if (truncated) {   // prologue_per_env: reset, mark the previous row truncated
                if (A.initial_states) { th = A.initial_states[2 * step]; thd = A.initial_states[2 * step + 1]; }
                else {
                    const float PI = 3.14159265358979323846f;
                    const rlt_u32x4 draw = rlt_philox(A.seed, STREAM_INITIAL_STATE, gstep);
                    th = -PI + 2.0f * PI * rlt_u01(draw.x); thd = -1.0f + 2.0f * rlt_u01(draw.y);
                }
                if (g == 0 && lane == 0 && A.drawn_initial) { A.drawn_initial[2 * step] = th; A.drawn_initial[2 * step + 1] = thd; }
                ep_step = 0; ep_return = 0.f;
                if (full_before || new_pos > 0) {
                    const unsigned prev = new_pos == 0 ? cap - 1 : new_pos - 1;
                    if (g == 0 && lane == 0) put_shared<PACKED>(A.rb.data + (size_t)prev * R + (R - 1), 1.0f);
                    rb_ces = new_pos;
                }
            }
            const float eps = S->rollout_eps[step & 1];
            float sn0, cs0; sincosf(th, &sn0, &cs0);
            // actor on the single observation: lane u owns hidden unit u; layer 2 reads layer 1 across lanes
            const float h1 = fmaxf(((w_actor[NA::lb1 + lane] + w_actor[NA::lw1 + lane * NA::LD1] * cs0) + w_actor[NA::lw1 + lane * NA::LD1 + 1] * sn0) + w_actor[NA::lw1 + lane * NA::LD1 + 2] * thd, 0.f);
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int k = 0; k < H; k += 2) {
                s0 += w_actor[NA::lw2 + lane * NA::LD2 + k] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(h1), k));
                s1 += w_actor[NA::lw2 + lane * NA::LD2 + k + 1] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(h1), k + 1));
            }
            const float h2 = fmaxf((s0 + s1) + w_actor[NA::lb2 + lane], 0.f);
            const float mean = kk_sum(row16_sum(w_actor[NA::lw3 + lane] * h2)) + w_actor[NA::lb3];
            const float ls_raw = kk_sum(row16_sum(w_actor[NA::lw3 + NA::LD2 + lane] * h2)) + w_actor[NA::lb3 + 1];
            // sample_and_squash in rollout mode (one action dimension), dynamics, reward, replay add
            const float ls = clampf(ls_raw, A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
            // every lane of this wavefront carries the environment's state and feeds its own hidden unit from its own copy: the action comes from one lane, so
            // that the copies stay identical bit for bit
            const float action = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(tanhf(mean + eps * expf(ls)))));
            const rlt_pendulum_parameters& p = A.runner.env;
            float u = p.max_torque * clampf(action, -1.f, 1.f);
            u = clampf(u, -p.max_torque, p.max_torque);
            float nthd = thd + (3.0f * p.g / (2.0f * p.l) * sn0 + 3.0f / (p.m * p.l * p.l) * u) * p.dt;
            nthd = clampf(nthd, -p.max_speed, p.max_speed);
            const float nth = th + nthd * p.dt;
            const float PI = 3.14159265358979323846f;
            const float a0 = th + PI, b0 = 2.0f * PI;
            const float an = (a0 - b0 * floorf(a0 / b0)) - PI;
            const float ur = p.max_torque * action;
            const float reward = -(an * an + 0.1f * thd * thd + 0.001f * (ur * ur));
            float sn1, cs1; sincosf(nth, &sn1, &cs1);
            ep_step += 1; ep_return += reward;
            const int trunc = ep_step == (unsigned)A.runner.episode_step_limit;
            float rowv = cs0;
            rowv = lane == 1 ? sn0 : rowv; rowv = lane == 2 ? thd : rowv; rowv = lane == 3 ? action : rowv; rowv = lane == 4 ? reward : rowv;
            rowv = lane == 5 ? cs1 : rowv; rowv = lane == 6 ? sn1 : rowv; rowv = lane == 7 ? nthd : rowv; rowv = lane == 8 ? 0.f : rowv;
            rowv = lane == 9 ? (trunc ? 1.f : 0.f) : rowv;
            if (lane < R) {
                S->new_row[lane] = rowv;
                if (g == 0) put_shared<PACKED>(A.rb.data + (size_t)new_pos * R + lane, rowv);
            }
            if (g == 0 && lane == 0) A.rb.episode_start[new_pos] = rb_ces;
            truncated = trunc; th = nth; thd = nthd;
            if (trunc) rb_ces = rb_pos;
        } else if (wave == 2) {
            // off the critical path: entropy coefficient of this step, exploration noise of the next one
            if (lane == 0) {
                S->alpha = expf(get_shared<PACKED>(A.log_alpha));      // rewritten by the last workgroup in the previous step's S4
            }
            if (lane == 1 && step + 1 < A.n_steps) {
                const float eps1 = A.rollout_noise ? A.rollout_noise[step + 1] : randn_at(A.seed, STREAM_ROLLOUT_NOISE, gstep + 1);
                S->rollout_eps[(step + 1) & 1] = eps1;
                if (g == 0 && A.drawn_rollout) A.drawn_rollout[step + 1] = eps1;
            }
        } else if (wave == 1 && lane < 4) {
            // bias corrections 1/(1 - beta^age) of this step (adam/operations_generic.h:43-66)
            const rlt_adam_parameters& p = lane == 0 ? A.adam_actor : (lane == 3 ? A.adam_alpha : A.adam_critic);
            const uint32_t age0 = lane == 0 ? age_actor0 : lane == 1 ? age_c00 : lane == 2 ? age_c10 : age_alpha0;
            const float age = (float)(age0 + (uint32_t)step);
            S->bc[2 * lane] = 1.0f / (1.0f - powf(p.beta_1, age)); S->bc[2 * lane + 1] = 1.0f / (1.0f - powf(p.beta_2, age));
        }
        // the gathered values land in LDS (other wavefronts do this while wavefront 0 steps the environment, except for the new row)
        rlt_lds_barrier();
        tick(0);
        if (S->abort) break;      // uniform: every write to it is separated from this read by a workgroup barrier on both sides
        // ================= S1: critic phase =================
        if (tid < ROWS * 16) {
            const int s = tid >> 4, j = tid & 15, sample = g * ROWS + s;
            if (j < R) {
                const float v = is_new ? S->new_row[j] : gathered;
                if (j < D) { Sx[s * XS + j] = v; if (A.out_oab) A.out_oab[(size_t)sample * D + j] = v; }
                else if (j == D) { S->reward[s] = v; if (A.out_rewards) A.out_rewards[sample] = v; }
                else if (j < D + 1 + OBS) { Snx[s * XS + (j - D - 1)] = v; if (A.out_oab) A.out_oab[((size_t)B + sample) * D + (j - D - 1)] = v; }
                else if (j == D + 1 + OBS) { S->notdone[s] = v != 0.f ? 0.f : 1.f; if (A.out_terminated) A.out_terminated[sample] = v != 0.f; }
            }
            if (j == 0 && A.out_oab) A.out_oab[((size_t)B + sample) * D + OBS] = 0.f;
        } else if (tid < ROWS * 16 + ROWS) S->noise_c[tid & 15] = noise_reg;
        else if (tid < ROWS * 16 + 2 * ROWS) S->noise_a[tid & 15] = noise_reg;
        rlt_lds_barrier();
        tick(11);
        stage_begin();
        // A: group 0 evaluates the actor on the next observations; group 1 meanwhile runs critic 1's training forward
        {
            Fwd1W f1; Fwd2W f2;
            if (grp == 0) { f1 = load_fwd1<NA>(w_actor, w, lane); f2 = load_fwd2<NA>(w_actor, w, lane); }
            else { f1 = load_fwd1<NC>(w_critic1, w, lane); f2 = load_fwd2<NC>(w_critic1, w, lane); }
            forward_stage1(grp == 0 ? Snx : Sx, grp == 0 ? Le1 : La1, f1, w, lane);
            stage(0);
            rlt_lds_barrier();
            stage(1);
            if (grp == 0) forward_stage2<2>(Le1, Le2, Lpart, f2, w, lane); else forward_stage2<1>(La1, La2, Lpart, f2, w, lane);
        }
        const Fwd1W t1 = load_fwd1<NC>(w_target, w, lane); const Fwd2W t2 = load_fwd2<NC>(w_target, w, lane);
        stage(2);
        rlt_lds_barrier();
        stage(3);
        if (wave == 0 && lane < ROWS) {   // sample_and_squash evaluate with the external noise -> next action, its log-probability
            const float mean = net_output<NA>(part0, w_actor, lane, 0);
            const float ls = clampf(net_output<NA>(part0, w_actor, lane, 1), A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
            const float sd = expf(ls), eps = S->noise_c[lane];
            const float sample = mean + eps * sd, act = tanhf(sample);
            const float z = (sample - mean) / sd;
            S->next_logp[lane] = (-0.9189385332046727f - ls - 0.5f * z * z) - logf(1.0f - act * act + A.sas.log_probability_epsilon);
            Snx[lane * XS + OBS] = act;
        }
        if (wave == 4 && lane < ROWS) S->q[1][lane] = net_output<NC>(part1, w_critic1, lane, 0);
        stage(4);
        rlt_lds_barrier();
        tick(12);
        stage(5);
        // B: target critic k on [next_obs | next_action] by group k
        forward_stage1(Snx, Le1, t1, w, lane);
        stage(6);
        rlt_lds_barrier();
        stage(7);
        forward_stage2<1>(Le1, Le2, Lpart, t2, w, lane);
        // D (weights): group 0 runs critic 0's training forward (critic 1's is already there), group 1 the actor on the batch
        // observations, whose result the actor phase needs (x rows are [obs | action]; the actor's weights for the action column are zero)
        Fwd1W d1; Fwd2W d2;
        if (grp == 0) { d1 = load_fwd1<NC>(w_critic0, w, lane); d2 = load_fwd2<NC>(w_critic0, w, lane); }
        else { d1 = load_fwd1<NA>(w_actor, w, lane); d2 = load_fwd2<NA>(w_actor, w, lane); }
        stage(8);
        rlt_lds_barrier();
        tick(13);
        stage(9);
        // C: TD target (sac/operations_generic.h:133-179)
        if (wave == 0 && lane < ROWS) {
            const float alpha = S->alpha;
            const float min_q = fminf(net_output<NC>(part0, w_target0, lane, 0), net_output<NC>(part1, w_target1, lane, 0)) - alpha * S->next_logp[lane];
            const float y = S->reward[lane] + S->notdone[lane] * A.gamma * min_q;
            S->y[lane] = y;
            if (A.out_target) A.out_target[g * ROWS + lane] = y;
        }
        // D
        forward_stage1(Sx, grp == 0 ? La1 : Ah1, d1, w, lane);
        stage(10);
        rlt_lds_barrier();
        stage(11);
        if (grp == 0) forward_stage2<1>(La1, La2, Lpart, d2, w, lane); else forward_stage2<2>(Ah1, Ah2, Lpart, d2, w, lane);
        const Bwd1W cb1 = load_bwd1<NC>(w_critic, w, lane); const Bwd2W cb2 = load_bwd2<NC>(w_critic, w, lane);
        stage(12);
        rlt_lds_barrier();
        tick(14);
        stage(13);
        if (w == 0 && lane < ROWS) {
            // d_output = (Q - y) * 2/B * loss_weight, loss_weight = B*0.5 / num_final_steps = 0.5 (sac/operations_generic.h:298-312)
            float q;
            if (grp == 0) { q = net_output<NC>(part0, w_critic0, lane, 0); S->q[0][lane] = q; } else q = S->q[1][lane];
            Ldout[lane * 2] = (q - S->y[lane]) * (2.0f / (float)B) * (((float)B * 0.5f) / (float)B);
        }
        if (wave == 5 && lane < ROWS) {   // sample_and_squash forward of the actor phase: keeps the pre-squashing sample and the action
            const float mean = net_output<NA>(part1, w_actor, lane, 0), ls_raw = net_output<NA>(part1, w_actor, lane, 1);
            const float ls = clampf(ls_raw, A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
            const float sample = mean + S->noise_a[lane] * expf(ls), act = tanhf(sample);
            S->mean[lane] = mean; S->ls_raw[lane] = ls_raw; S->act_pre[lane] = sample; S->act_a[lane] = act;
#pragma unroll
            for (int j = 0; j < OBS; j++) Snx[lane * XS + j] = Sx[lane * XS + j];   // [obs | new action] rows for the critics of the actor phase
            Snx[lane * XS + OBS] = act;
        }
        stage(14);
        rlt_lds_barrier();
        stage(15);
        backward_stage1<NC, true, PACKED>(La2, Ldp2, Ldout, cb1, my_partial + grp * NC::total, w, lane);
        stage(16);
        rlt_lds_barrier();
        stage(17);
        backward_w2<NC, PACKED>(La1, Ldp2, my_partial + grp * NC::total, w, lane);
        backward_l1<NC, true, false, PACKED>(Sx, La1, Ldp2, Lpart, cb2, my_partial + grp * NC::total, w, lane);
        if (A.out_critic_loss && w == 0) {      // sum of squared TD errors of this workgroup's rows
            float d = lane < ROWS ? (S->q[grp][lane] - S->y[lane]) : 0.f;
            d = kk_sum(row16_sum(d * d));
            if (lane == 0) put_shared<PACKED>(my_partial + 2 * NC::total + NA::total + 1 + grp, d);
        }
        stage(18);
        tick(1);
        announce<PACKED>(A.ready, READY_CRITIC_GRADIENTS, g, seq);
        tick(2);
        // ================= S2: reduce + Adam + polyak for both critics =================
        await(A.ready, READY_CRITIC_GRADIENTS, G, seq, A.fault, &S->abort, A.max_poll);
        {
            constexpr int total = 2 * NC::total;
            const int chunk = (total + G - 1) / G;
            const int begin = g * chunk, end = min(total, begin + chunk);
            for (int base = begin; base < end; base += 2 * THREADS) {
                bool ok[2]; int o[2], kq[2], idc[2]; float gsum[2], m[2], v[2], p[2], t[2];
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const int idx = base + tid + e * THREADS;
                    ok[e] = idx < end; idc[e] = ok[e] ? idx : begin;
                    kq[e] = idc[e] >= NC::total ? 1 : 0; o[e] = idc[e] - kq[e] * NC::total;
                    m[e] = (kq[e] ? A.critic_m[1] : A.critic_m[0])[o[e]]; v[e] = (kq[e] ? A.critic_v[1] : A.critic_v[0])[o[e]];
                    p[e] = get_shared<PACKED>((kq[e] ? A.critic_p[1] : A.critic_p[0]) + o[e]); t[e] = (kq[e] ? A.target_p[1] : A.target_p[0])[o[e]];
                }
                sum_partials<2, PACKED>(A.partial, idc, G, gsum);
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    if (ok[e]) {
                        const float pnew = adam_element(A.adam_critic, S->bc[2 + 2 * kq[e]], S->bc[3 + 2 * kq[e]], gsum[e], m[e], v[e], p[e]);
                        put_shared<PACKED>((kq[e] ? A.critic_p[1] : A.critic_p[0]) + o[e], pnew);      // what the other workgroups wait for first
                        (kq[e] ? A.critic_g[1] : A.critic_g[0])[o[e]] = gsum[e]; (kq[e] ? A.critic_m[1] : A.critic_m[0])[o[e]] = m[e];
                        (kq[e] ? A.critic_v[1] : A.critic_v[0])[o[e]] = v[e];
                        (kq[e] ? A.target_p[1] : A.target_p[0])[o[e]] = polyak_step(A.polyak, t[e], pnew);
                    }
                }
            }
            if (g == 0 && A.out_critic_loss && tid < 2) {
                const int idx[1] = {2 * NC::total + NA::total + 1 + tid}; float s[1];
                sum_partials<1, PACKED>(A.partial, idx, G, s);
                A.out_critic_loss[(size_t)step * 2 + tid] = s[0] * 0.5f / (float)B;
            }
        }
        tick(3);
        announce<PACKED>(A.ready, READY_CRITIC_PARAMETERS, g, seq);
        await(A.ready, READY_CRITIC_PARAMETERS, G, seq, A.fault, &S->abort, A.max_poll);
        tick(4);
        // both critics are needed now; the target critics, read next in the following step's critic phase, follow from them later in this step
        float fresh[2][NC::per_thread];
        {
            const float* const src_c[2] = {A.critic_p[0], A.critic_p[1]};
            load_nets<NC, 2, PACKED>(fresh, src_c, tid);
            const lptr dst_c[2] = {w_critic0, w_critic1};
            store_nets<NC, 2>(dst_c, fresh, tid);
        }
        rlt_lds_barrier();
        tick(5);
        stage_begin();
        // ================= S3: actor phase =================
        // (the actor's forward on the batch observations and its sample_and_squash forward were done in the critic phase)
        // critic k forward + backward_input on [obs | new action] by group k
        {
            const Fwd1W f1 = load_fwd1<NC>(w_critic, w, lane); const Fwd2W f2 = load_fwd2<NC>(w_critic, w, lane);
            forward_stage1(Snx, Le1, f1, w, lane);
            stage(20);
            rlt_lds_barrier();
            stage(21);
            forward_stage2<1>(Le1, Le2, Lpart, f2, w, lane);
        }
        {
            const Bwd1W b1 = load_bwd1<NC>(w_critic, w, lane); const Bwd2W b2 = load_bwd2<NC>(w_critic, w, lane);
            stage(22);
            rlt_lds_barrier();
            stage(23);
            if (w == 0 && lane < ROWS) S->q[grp][lane] = net_output<NC>(Lpart, w_critic, lane, 0);
            backward_stage1<NC, false, PACKED>(Le2, Ldp2, &S->dout_actor_critic[0], b1, nullptr, w, lane);
            stage(24);
            rlt_lds_barrier();
            stage(25);
            backward_l1<NC, false, true, PACKED>(Snx, Le1, Ldp2, Lpart, b2, nullptr, w, lane);
        }
        const Bwd1W ab1 = load_bwd1<NA>(w_actor, w, lane); const Bwd2W ab2 = load_bwd2<NA>(w_actor, w, lane);
        stage(26);
        rlt_lds_barrier();
        stage(27);
        // min-Q routing (sac/operations_generic.h:358-393), sample_and_squash backward (nn/layers/sample_and_squash/operations_generic.h:289-398)
        if (wave == 0) {
            float alpha_term = 0.f;
            if (lane < ROWS) {
                const float alpha = S->alpha, alpha_b = alpha / (float)B;
                const lptr pk = S->q[0][lane] < S->q[1][lane] ? part0 : part1;
                const float d_out = (pk[0 * ROWS + lane] + pk[1 * ROWS + lane]) + (pk[2 * ROWS + lane] + pk[3 * ROWS + lane]);
                const float action = S->act_a[lane];
                const float gte = d_out * (1.0f - action * action);
                const float eps = S->noise_a[lane];
                const float ls_raw = S->ls_raw[lane];
                const float ls = clampf(ls_raw, A.sas.log_std_lower_bound, A.sas.log_std_upper_bound);
                const float sd = expf(ls), mu = S->mean[lane], sample = S->act_pre[lane];
                const float z = (sample - mu) / sd;
                const float d_mu = gte + alpha_b * ((z / sd) + (-z / sd) + 2.0f * action);
                float d_ls = sd * (gte * eps) + alpha_b * ((z * z - 1.0f) + (-z / sd) * eps * sd + 2.0f * action * eps * sd);
                if (ls_raw < A.sas.log_std_lower_bound || ls_raw > A.sas.log_std_upper_bound) d_ls = 0.f;
                S->actor_dout[lane * 2] = d_mu; S->actor_dout[lane * 2 + 1] = d_ls;
                const float lp = (-0.9189385332046727f - ls - 0.5f * z * z) - logf(1.0f - action * action + A.sas.log_probability_epsilon);
                alpha_term = alpha * (-lp - A.sas.target_entropy);
            }
            alpha_term = row16_sum(alpha_term);
            if (lane == 0) put_shared<PACKED>(my_partial + 2 * NC::total + NA::total, alpha_term);
        }
        stage(28);
        rlt_lds_barrier();
        stage(29);
        // actor backward: layer 3 and the layer-2 gate by group 0, then the layer-2 weight gradient by group 0 and layer 1 by group 1
        const lptr dp2a = &S->grp[0].dp2[0];
        if (grp == 0) backward_stage1<NA, true, PACKED>(Ah2, dp2a, &S->actor_dout[0], ab1, my_partial + 2 * NC::total, w, lane);
        stage(30);
        rlt_lds_barrier();
        stage(31);
        if (grp == 0) backward_w2<NA, PACKED>(Ah1, dp2a, my_partial + 2 * NC::total, w, lane);
        else backward_l1<NA, true, false, PACKED>(Sx, Ah1, dp2a, Lpart, ab2, my_partial + 2 * NC::total, w, lane);
        stage(32);
        tick(6);
        announce<PACKED>(A.ready, READY_ACTOR_GRADIENTS, g, seq);
        {   // the target critics' soft update on the LDS copies, while the other workgroups' gradients arrive (read next after several barriers)
            const lptr dst_t[2] = {w_target0, w_target1};
            polyak_nets<NC, 2>(dst_t, fresh, A.polyak, tid);
        }
        await(A.ready, READY_ACTOR_GRADIENTS, G, seq, A.fault, &S->abort, A.max_poll);
        tick(7);
        // ================= S4: reduce + Adam for the actor and log_alpha =================
        {
            const int chunk = (NA::total + G - 1) / G;
            const int begin = g * chunk, end = min(NA::total, begin + chunk);
            for (int base = begin; base < end; base += THREADS) {
                const bool ok = base + tid < end;
                const int o = ok ? base + tid : begin;      // idle lanes redo the first element and drop the result: no branch around the loads
                float m = A.actor_m[o], v = A.actor_v[o]; const float p = get_shared<PACKED>(A.actor_p + o);
                const int idx[1] = {2 * NC::total + o}; float gs[1];
                sum_partials<1, PACKED>(A.partial, idx, G, gs);
                const float pnew = adam_element(A.adam_actor, S->bc[0], S->bc[1], gs[0], m, v, p);
                if (ok) { put_shared<PACKED>(A.actor_p + o, pnew); A.actor_g[o] = gs[0]; A.actor_m[o] = m; A.actor_v[o] = v; }
            }
            if (g == G - 1 && tid == THREADS - 1) {   // log_alpha: gradient = mean over the batch of alpha * (entropy - target entropy)
                const int idx[1] = {2 * NC::total + NA::total}; float gs[1];
                sum_partials<1, PACKED>(A.partial, idx, G, gs);
                const float gsum = gs[0] / (float)B;
                // gradient and moments share the parameter's cache line, which every workgroup reads: all four go the shared way
                float m = get_shared<PACKED>(A.log_alpha + 2), v = get_shared<PACKED>(A.log_alpha + 3);
                const float pnew = adam_element(A.adam_alpha, S->bc[6], S->bc[7], gsum, m, v, get_shared<PACKED>(A.log_alpha));
                put_shared<PACKED>(A.log_alpha + 1, gsum); put_shared<PACKED>(A.log_alpha + 2, m); put_shared<PACKED>(A.log_alpha + 3, v); put_shared<PACKED>(A.log_alpha, pnew);
            }
        }
        tick(8);
        announce<PACKED>(A.ready, READY_ACTOR_PARAMETERS, g, seq);
        await(A.ready, READY_ACTOR_PARAMETERS, G, seq, A.fault, &S->abort, A.max_poll);
        tick(9);
        {
            const lptr dst_a[1] = {w_actor}; const float* const src_a[1] = {A.actor_p};
            cache_nets<NA, 1, PACKED>(dst_a, src_a, tid);
        }
        rlt_lds_barrier();
        tick(10);
    }
    if (A.phase_ticks && g == 0 && tid == 0) {
        S->ticks[15] = clock64() - shader_clock_begin;     // shader clock cycles of the whole run: with the sum of the others it gives the clock rate
        for (int i = 0; i < 16; i++) A.phase_ticks[i] += S->ticks[i];
    }
    if (A.stage_ticks && g == 0 && tid == 0)
        for (int i = 0; i < 48; i++) A.stage_ticks[i] += S->sticks[i];
    // the placement on one XCD is what makes plain stores visible to the other workgroups: a run that was placed otherwise is void
    if (PACKED && g == 0 && tid == 0) {
        const unsigned mask = __hip_atomic_load(A.xcd_mask, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (mask & (mask - 1)) __hip_atomic_store(A.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (g == 0 && tid == 0) {
        A.runner.states[0] = th; A.runner.states[1] = thd; A.runner.episode_return[0] = ep_return;
        A.runner.episode_step[0] = ep_step; A.runner.truncated[0] = (uint8_t)truncated;
        A.rb.position[0] = rb_pos; A.rb.current_episode_start[0] = rb_ces; A.rb.full[0] = (uint8_t)rb_full;
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
    const int B = agent->batch;
    // what the kernel is built for; anything else has to take the per-operation entry points
    if (agent->observation_dim != OBS || agent->action_dim != ACT || B % ROWS != 0 || B / ROWS > MAX_G || B / ROWS > device->compute_units) return RLT_E_UNSUPPORTED;
    if (runner->n_envs != 1 || rb->n_envs != 1 || rb->observation_dim != OBS || rb->action_dim != ACT) return RLT_E_UNSUPPORTED;
    if (agent->final_step_mask || agent->next_final_step_mask || agent->reset) return RLT_E_UNSUPPORTED;   // all-true masks only (SEQUENCE_LENGTH = 1)
    if (!contiguous_arena(agent->actor, agent->n_actor_layers, OBS, 2 * ACT, true)) return RLT_E_UNSUPPORTED;
    if (!adam_arena(agent->actor_adam_tensors, agent->n_actor_adam_tensors, agent->actor[0].weights, (size_t)NA::total)) return RLT_E_UNSUPPORTED;
    for (int k = 0; k < 2; k++) {
        if (!contiguous_arena(agent->critics[k], agent->n_critic_layers, OBS + ACT, 1, true)) return RLT_E_UNSUPPORTED;
        if (!contiguous_arena(agent->critics_target[k], agent->n_critic_layers, OBS + ACT, 1, false)) return RLT_E_UNSUPPORTED;
        if (!adam_arena(agent->critic_adam_tensors[k], agent->n_critic_adam_tensors, agent->critics[k][0].weights, (size_t)NC::total)) return RLT_E_UNSUPPORTED;
    }
    RLT_REQUIRE(agent->log_alpha.parameters && agent->log_alpha.gradient == agent->log_alpha.parameters + 1 &&
                agent->log_alpha.first_moment == agent->log_alpha.parameters + 2 && agent->log_alpha.second_moment == agent->log_alpha.parameters + 3);
    RLT_REQUIRE(agent->actor_age && agent->critic_age[0] && agent->critic_age[1] && agent->alpha_age);
    RLT_REQUIRE(runner->states && runner->episode_step && runner->episode_return && runner->truncated && rb->data && rb->episode_start && rb->position &&
                rb->current_episode_start && rb->full && rb->capacity > 0);
    const int G = B / ROWS;
    const size_t n_partial = (size_t)N_PARTIAL;
    void* scratch = nullptr;
    const size_t scratch_bytes = 2048 + (size_t)(G + 1) * n_partial * sizeof(float);
    int rc = rlt_scratch(device, scratch_bytes, &scratch);
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
    a.batch = B; a.n_steps = n_steps;
    a.runner = *runner; a.rb = *rb;
    a.xcd_mask = (unsigned*)scratch; a.ready = (unsigned*)((char*)scratch + 256); a.partial = (float*)((char*)scratch + 2048);
    a.fault = device->fault; a.max_poll = device->wait_limit;
    if (inputs) { a.rollout_noise = inputs->rollout_noise; a.initial_states = inputs->initial_states; a.sample_offsets = inputs->sample_offsets;
                  a.noise_critic = inputs->noise_critic; a.noise_actor = inputs->noise_actor; }
    a.seed = seed; a.step_offset = step_offset;
    if (outputs) { a.out_critic_loss = outputs->critic_loss; a.out_oab = outputs->observations_actions_base; a.out_rewards = outputs->rewards;
                   a.out_terminated = outputs->terminated; a.out_target = outputs->target_action_value; a.phase_ticks = (unsigned long long*)outputs->phase_ticks; a.stage_ticks = (unsigned long long*)outputs->stage_ticks;
                   a.drawn_rollout = outputs->drawn_rollout_noise; a.drawn_initial = outputs->drawn_initial_states; a.drawn_offsets = outputs->drawn_sample_offsets;
                   a.drawn_noise_c = outputs->drawn_noise_critic; a.drawn_noise_a = outputs->drawn_noise_actor; }
    const size_t lds_floats = ((sizeof(Shared) / 4 + 3) & ~(size_t)3) + (size_t)(NA::ltotal + 4 * NC::ltotal);
    const size_t lds_bytes = lds_floats * sizeof(float);
    a.lds_floats = (int)lds_floats;
    if (lds_bytes > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    // sequence numbers restart with every launch; the zero row of the partial sums
    RLT_HIP(hipMemsetAsync(scratch, 0, 2048, device->stream));
    RLT_HIP(hipMemsetAsync((char*)scratch + 2048 + (size_t)G * n_partial * sizeof(float), 0, n_partial * sizeof(float), device->stream));
    device->fault_armed = 1;
    // one XCD holds 32 CUs: up to that many workgroups are placed on one XCD if the device hands out workgroups round robin
    // RLT_SAC_LOOP_PLACEMENT=spread keeps the workgroups spread over the XCDs (the path larger batches take), for tests and comparisons
    const char* placement = std::getenv("RLT_SAC_LOOP_PLACEMENT");
    const bool spread = placement && std::strcmp(placement, "spread") == 0;
    if (std::getenv("RLT_ROCM_VERBOSE")) std::fprintf(stderr, "rlt_rocm_sac_pendulum_loop: %d workgroups, xcd stride %d, %s\n", G, device->xcd_stride,
                                                      (G <= MAX_PACKED_G && device->xcd_stride == 8 && !spread) ? "on one XCD" : "spread");
    if (G <= MAX_PACKED_G && device->xcd_stride == 8 && !spread) {
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(sac_pendulum_loop_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        hipLaunchKernelGGL(sac_pendulum_loop_kernel<true>, dim3(8 * G), dim3(THREADS), lds_bytes, device->stream, a);
    } else {
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(sac_pendulum_loop_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        hipLaunchKernelGGL(sac_pendulum_loop_kernel<false>, dim3(G), dim3(THREADS), lds_bytes, device->stream, a);
    }
    return rlt_launch_status(device);
}
