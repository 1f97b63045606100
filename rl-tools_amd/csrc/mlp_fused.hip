// Forward + backward of a 3-layer MLP  in -> 256 -> 256 -> out  in ONE pass over the batch: activations never leave the chip.
//
// reference: forward(mlp) / backward(mlp) nn_models/mlp/operations_generic.h:103-204, built from the dense layer's forward,
// backward_input and weight-gradient contractions (nn/layers/dense/operations_generic.h:122-271). The reference (and the
// per-layer path of this library) materialises every layer's activations in memory: at batch 65,536 and width 256 that is
// ~0.4 GB of HBM traffic per call for 27.5 GFLOP, and eleven launches.
//
// Here one persistent workgroup per compute unit (4 wavefronts, one per SIMD, up to 512 registers each) walks over tiles of 64
// batch rows. Per tile, in LDS: h1 and h2 (64 x 256 each, row stride 257), the input rows (64 x 33) and the output gradient
// (64 x 17). Per tile, on v_mfma_f32_32x32x2_f32 unless noted:
//   P1  h1 = act(x W1^T + b1)                       K = in
//   P2  h2 = act(h1 W2^T + b2)                      K = 256, W2 read from L2 in a pre-swizzled layout, one dwordx4 per 4 k-steps
//   P3  y = act(h2 W3^T + b3), d_pre3               16x16x4, wavefront w owns rows [16w, 16w+16)
//   P4  dW3 += d_pre3^T h2                          16x16x4
//   P5  d_pre2 = (d_pre3 W3) * act'(h2)  in place of h2
//   P6  dW2 += d_pre2^T h1 ; d_h1 = d_pre2 W2       K = 64 rows / K = 256
//   P7  d_pre1 = d_h1 * act'(h1)  in place of h1
//   P8  dW1 += d_pre1^T x
// The weight-gradient accumulators (256 + 32 + 16 registers per lane) live in registers for the whole launch; at the end every
// workgroup writes its partial gradients and a second kernel sums them in a fixed order into the layers' gradients (beta = 1).
// act' is taken from the layer output, which relu / tanh / fast_tanh / sigmoid / identity allow.
//
// The reference's own call pattern is forward(), then (after the caller has formed the loss gradient) backward(). The same kernel
// serves it in two more modes: FORWARD runs P1-P3 and writes every layer's pre-activations and outputs, as forward() must;
// BACKWARD reads the outputs of layers 1 and 2 back into LDS and runs P4-P8 on the gradient it is given.
#include "common.h"
#include "mlp_fused.h"

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) float* lptr;

extern __shared__ __attribute__((aligned(16))) float rlt_mlp3_lds[];

namespace {

constexpr int HID = 256;     // hidden width the kernel is built for
constexpr int BM = 64;       // batch rows per tile
constexpr int HS = HID + 1;  // LDS row stride of h1 / h2: odd, so that 32 rows read side by side fall into 32 banks
constexpr int XSP = 33;      // LDS row stride of the input rows (in <= 32, zero padded)
constexpr int DS = 17;       // LDS row stride of the output-gradient rows (out <= 16, zero padded)
constexpr int THREADS = 256;
constexpr int MAX_WORKGROUPS = 256;
constexpr int LDS_FLOATS = 2 * BM * HS + BM * XSP + BM * DS + 16 * HS;   // h1, h2, input rows, output-gradient rows, W3 (zero padded to 16 rows)

// swizzled weight copies (floats), built once per call by mlp3_prepare_kernel
constexpr size_t W2F_FLOATS = 65536, W2B_FLOATS = 65536, W1S_FLOATS = 8 * 16 * 64;
constexpr size_t PREP_FLOATS = W2F_FLOATS + W2B_FLOATS + W1S_FLOATS;

enum { MODE_FUSED = 0, MODE_FORWARD = 1, MODE_BACKWARD = 2 };

struct Mlp3Args {
    const float* x; int ldx; float* y; int ldy; const float* d_output; int ldd; const float* target; int ldt; float mse_scale;
    float* act_pre[3]; float* act_out[3];      // FORWARD: written (each may be NULL); BACKWARD: act_out[0], act_out[1] are read
    int batch, in, out, act1, act2, act3, n_tiles;
    const float* b1; const float* b2; const float* b3;
    const float* w2f; const float* w2b; const float* w1s; const float* W3;
    float* partial;      // [workgroups][count rounded up to a multiple of 64]
};

__device__ __forceinline__ floatx16 mfma32(float a, float b, floatx16 c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
// row of element v of a 32x32 result tile held by a lane with hi = lane >> 5
__device__ __forceinline__ int row32(int v, int hi) { return 8 * (v >> 2) + 4 * hi + (v & 3); }

// activation and its derivative from the output, with the kind as a compile-time constant: the epilogues dispatch once per phase
// instead of once per element
template <int ACT> __device__ __forceinline__ float act_c(float x) { return rlt_act(x, ACT); }
template <int ACT> __device__ __forceinline__ float dact_c(float o) { return rlt_dact_from_output(o, ACT); }
template <int ACT> struct ActKind { static constexpr int value = ACT; };
template <class F>
__device__ __forceinline__ void act_dispatch(int kind, F&& body) {
    switch (kind) {
        case RLT_ACT_RELU: body(ActKind<RLT_ACT_RELU>{}); break;
        case RLT_ACT_TANH: body(ActKind<RLT_ACT_TANH>{}); break;
        case RLT_ACT_FAST_TANH: body(ActKind<RLT_ACT_FAST_TANH>{}); break;
        case RLT_ACT_SIGMOID: body(ActKind<RLT_ACT_SIGMOID>{}); break;
        default: body(ActKind<RLT_ACT_IDENTITY>{}); break;
    }
}

// k-step count as a compile-time constant (rounded up to a multiple of 4; the padding steps multiply zeros): straight-line code whose
// LDS reads are all issued before the first matrix instruction waits
template <int N> struct StepCount { static constexpr int value = N; };
template <class F>
__device__ __forceinline__ void steps_dispatch(int steps, F&& body) {
    if (steps <= 4) body(StepCount<4>{});
    else if (steps <= 8) body(StepCount<8>{});
    else if (steps <= 12) body(StepCount<12>{});
    else body(StepCount<16>{});
}

// Operand layouts of the matrix instructions (lane l):
//   32x32x2: A[row l%32][k l/32], B[k l/32][col l%32], result v -> row 8(v/4) + 4(l/32) + v%4, col l%32
//   16x16x4: A[row l%16][k l/16], B[k l/16][col l%16], result v -> row 4(l/16) + v, col l%16
// w2f[nt][g][l][t] = W2[32nt + l%32][2(4g+t) + l/32]    B operand of h1 W2^T   for column tile nt, k-step 4g+t
// w2b[it][g][l][t] = W2[2(4g+t) + l/32][32it + l%32]    B operand of d_pre2 W2 for column tile it
// w1s[nt][j][l]    = W1[32nt + l%32][2j + l/32]         (0 beyond in)
// W3 (out x 256) is small enough to sit in LDS for the whole launch (rows padded to 16 with zeros).
__global__ void mlp3_prepare_kernel(const float* __restrict__ W1, const float* __restrict__ W2, int in, float* __restrict__ prep) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    float* w2f = prep; float* w2b = w2f + W2F_FLOATS; float* w1s = w2b + W2B_FLOATS;
    if (idx < 65536) {
        const int t = idx & 3, l = (idx >> 2) & 63, g = (idx >> 8) & 31, tile = idx >> 13;
        const int k = 2 * (4 * g + t) + (l >> 5), c = 32 * tile + (l & 31);
        w2f[idx] = W2[c * HID + k];
        w2b[idx] = W2[k * HID + c];
    }
    if (idx < (int)W1S_FLOATS) {
        const int l = idx & 63, j = (idx >> 6) & 15, nt = idx >> 10;
        const int k = 2 * j + (l >> 5), n = 32 * nt + (l & 31);
        w1s[idx] = k < in ? W1[n * in + k] : 0.f;
    }
}

// 64 x 64 block of  A[64 x 256] (LDS, row stride HS) times a pre-swizzled 256 x 256 weight: wavefront w owns column tiles 2w, 2w+1.
// The LDS operands of k-step s+1 and the weight group two ahead are requested before the matrix instructions of step s are issued.
__device__ __forceinline__ void contract_256(lptr a, const float* __restrict__ wsw, int w, int lane, floatx16 (&acc)[2][2]) {
    const int c32 = lane & 31, hi = lane >> 5;
    const floatx4* b0p = reinterpret_cast<const floatx4*>(wsw) + (size_t)(2 * w) * 32 * 64 + lane;
    const floatx4* b1p = b0p + 32 * 64;
    const lptr a0 = a + c32 * HS + hi, a1 = a0 + 32 * HS;
    floatx4 b0 = b0p[0], b1 = b1p[0];
    floatx4 n0 = b0p[64], n1 = b1p[64];
    float x0 = a0[0], x1 = a1[0];
#pragma unroll       // fully unrolled: the rotation of the prefetch registers becomes renaming instead of copies that wait for the loads
    for (int g = 0; g < 32; g++) {
        const int gp = g + 2 < 32 ? g + 2 : 31;      // two groups ahead; the last iterations re-read the final group
        const floatx4 p0 = b0p[gp * 64], p1 = b1p[gp * 64];
        __builtin_amdgcn_sched_barrier(0);      // the requests above are not to be moved down to their first use
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int next = 4 * g + t + 1 < 128 ? 4 * g + t + 1 : 127;
            const float y0 = a0[2 * next], y1 = a1[2 * next];
            acc[0][0] = mfma32(x0, b0[t], acc[0][0]);
            acc[0][1] = mfma32(x0, b1[t], acc[0][1]);
            acc[1][0] = mfma32(x1, b0[t], acc[1][0]);
            acc[1][1] = mfma32(x1, b1[t], acc[1][1]);
            x0 = y0; x1 = y1;
        }
        b0 = n0; b1 = n1; n0 = p0; n1 = p1;
    }
}

template <int MODE>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void mlp3_fused_kernel(Mlp3Args A) {
    const lptr h1 = (lptr)rlt_mlp3_lds, h2 = h1 + BM * HS, xs = h2 + BM * HS, dp3 = xs + BM * XSP, w3l = dp3 + BM * DS;
    const int lane_invariant = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nk1 = (A.in + 1) >> 1, nk3 = (A.out + 1) >> 1;
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
    floatx16 aW2[2][8], aW1[2];
    floatx4 aW3[4];
#pragma unroll
    for (int a = 0; a < 2; a++) { aW1[a] = zero16;
#pragma unroll
        for (int b = 0; b < 8; b++) aW2[a][b] = zero16; }
#pragma unroll
    for (int t = 0; t < 4; t++) aW3[t] = zero4;
    float db1 = 0.f, db2 = 0.f, db3 = 0.f;
    const float bias1[2] = {A.b1[32 * (2 * w) + (lane_invariant & 31)], A.b1[32 * (2 * w + 1) + (lane_invariant & 31)]};
    const float bias2[2] = {A.b2[32 * (2 * w) + (lane_invariant & 31)], A.b2[32 * (2 * w + 1) + (lane_invariant & 31)]};
    const float bias3 = (lane_invariant & 15) < A.out ? A.b3[lane_invariant & 15] : 0.f;

#ifdef RLT_MLP3_PROFILE      // build-time profiling aid: shader clock cycles workgroup 0 spends in each phase, printed at the end
    unsigned long long phase_cycles[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, t_prev = clock64();
#define RLT_TICK(i) { const unsigned long long t_now = clock64(); phase_cycles[i] += t_now - t_prev; t_prev = t_now; }
#else
#define RLT_TICK(i)
#endif
    // W3 into LDS once (rows beyond out stay zero)
    for (int idx = threadIdx.x; idx < 16 * HS; idx += THREADS) { const int n = idx / HS, k = idx - n * HS; w3l[idx] = (n < A.out && k < HID) ? A.W3[n * HID + k] : 0.f; }
    // input rows and upstream gradient (or target) rows of a tile travel through registers: requested a whole tile ahead
    // four threads per row: thread t covers columns (t & 3) + 4u of row t >> 2
    constexpr int NX = 8, ND = 4;
    float vx[NX], vd[ND];
    const float* dsrc = MODE == MODE_FORWARD ? A.x : (A.target ? A.target : A.d_output); const int ldsrc = A.target ? A.ldt : A.ldd;
    auto request_tile = [&](int tile, int tid) {
        const int row = tid >> 2, c0 = tid & 3, grow = tile * BM + row;
        const bool row_ok = grow < A.batch;
        const float* xr = A.x + (size_t)(row_ok ? grow : 0) * A.ldx;
        const float* dr = dsrc + (size_t)(row_ok ? grow : 0) * ldsrc;
#pragma unroll
        for (int u = 0; u < NX; u++) { const int c = c0 + 4 * u; const bool ok = row_ok && c < A.in; const float v = xr[ok ? c : 0]; vx[u] = ok ? v : 0.f; }
        if (MODE != MODE_FORWARD) {
#pragma unroll
            for (int u = 0; u < ND; u++) { const int c = c0 + 4 * u; const bool ok = row_ok && c < A.out; const float v = dr[ok ? c : 0]; vd[u] = ok ? v : 0.f; }
        }
    };
    request_tile(blockIdx.x, threadIdx.x);
    int lane = lane_invariant;
    for (int tile = blockIdx.x; tile < A.n_tiles; tile += gridDim.x) {
        // per-lane addresses derive from a lane index the optimiser cannot see through, or it hoists them all out of this loop and spills them
        asm volatile("" : "+v"(lane));
        const int tid = (w << 6) | lane, c32 = lane & 31, hi = lane >> 5, r16 = lane & 15, q = lane >> 4;
        const int r0 = tile * BM;
        // ---- P0: this tile's rows into LDS (zero padded), the next tile's requested; layer-1 weight fragments requested
#pragma unroll
        for (int u = 0; u < NX; u++) xs[(tid >> 2) * XSP + (tid & 3) + 4 * u] = vx[u];
        if (MODE != MODE_FORWARD) {
#pragma unroll
            for (int u = 0; u < ND; u++) dp3[(tid >> 2) * DS + (tid & 3) + 4 * u] = vd[u];
        }
        float wf[2][16];
        if (MODE != MODE_BACKWARD) {
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int j = 0; j < 16; j++) wf[a][j] = A.w1s[((2 * w + a) * 16 + j) * 64 + lane];
        }
        if (MODE == MODE_BACKWARD) {
            // the outputs of layers 1 and 2 of this tile, as forward() left them in memory, into LDS (rows beyond the batch as zeros)
#pragma unroll 1
            for (int half = 0; half < 2; half++) {
                const float* src = A.act_out[half]; const lptr dst = half ? h2 : h1;
#pragma unroll
                for (int i0 = 0; i0 < 16; i0 += 8) {
                    floatx4 v[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const int idx = tid + THREADS * (i0 + i), row = idx >> 6, grow = r0 + row;
                        v[i] = reinterpret_cast<const floatx4*>(src + (size_t)(grow < A.batch ? grow : 0) * HID)[idx & 63];
                    }
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const int idx = tid + THREADS * (i0 + i), row = idx >> 6, c4 = (idx & 63) * 4;
                        const bool ok = r0 + row < A.batch;
#pragma unroll
                        for (int e = 0; e < 4; e++) dst[row * HS + c4 + e] = ok ? v[i][e] : 0.f;
                    }
                }
            }
        }
        if (tile + (int)gridDim.x < A.n_tiles) request_tile(tile + gridDim.x, tid);
        rlt_lds_barrier();
        RLT_TICK(0)
        // ---- P1: h1 = act(x W1^T + b1); wavefront w owns columns [64w, 64w+64)
        if (MODE != MODE_BACKWARD) {
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const int nt = 2 * w + a;
            floatx16 acc[2] = {zero16, zero16};
            steps_dispatch(nk1, [&](auto steps) { constexpr int NK = decltype(steps)::value;
                float xa[2][NK];
#pragma unroll
                for (int j = 0; j < NK; j++) { xa[0][j] = xs[c32 * XSP + 2 * j + hi]; xa[1][j] = xs[(32 + c32) * XSP + 2 * j + hi]; }
#pragma unroll
                for (int j = 0; j < NK; j++) { acc[0] = mfma32(xa[0][j], wf[a][j], acc[0]); acc[1] = mfma32(xa[1][j], wf[a][j], acc[1]); }
            });
            act_dispatch(A.act1, [&](auto kind) { constexpr int ACT = decltype(kind)::value;
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const float pre = acc[mt][v] + bias1[a], o = act_c<ACT>(pre);
                    h1[(32 * mt + row32(v, hi)) * HS + 32 * nt + c32] = o;
                    if (MODE == MODE_FORWARD) {
                        const int grow = r0 + 32 * mt + row32(v, hi);
                        if (grow < A.batch) { if (A.act_pre[0]) A.act_pre[0][(size_t)grow * HID + 32 * nt + c32] = pre; if (A.act_out[0]) A.act_out[0][(size_t)grow * HID + 32 * nt + c32] = o; }
                    }
                }
            });
        }
        rlt_lds_barrier();
        }
        RLT_TICK(1)
        // ---- P2: h2 = act(h1 W2^T + b2)
        if (MODE != MODE_BACKWARD) {
            floatx16 acc[2][2] = {{zero16, zero16}, {zero16, zero16}};
            contract_256(h1, A.w2f, w, lane, acc);
            act_dispatch(A.act2, [&](auto kind) { constexpr int ACT = decltype(kind)::value;
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const float pre = acc[mt][a][v] + bias2[a], o = act_c<ACT>(pre);
                        h2[(32 * mt + row32(v, hi)) * HS + 32 * (2 * w + a) + c32] = o;
                        if (MODE == MODE_FORWARD) {
                            const int grow = r0 + 32 * mt + row32(v, hi);
                            if (grow < A.batch) { if (A.act_pre[1]) A.act_pre[1][(size_t)grow * HID + 32 * (2 * w + a) + c32] = pre; if (A.act_out[1]) A.act_out[1][(size_t)grow * HID + 32 * (2 * w + a) + c32] = o; }
                        }
                    }
            });
            rlt_lds_barrier();
        }
        RLT_TICK(2)
        // ---- P3: y = act(h2 W3^T + b3) for rows [16w, 16w+16) (lane group q takes the reduction range [64q, 64q+64)), then d_pre3
        // (BACKWARD is handed d_pre3 itself: the caller has applied the output activation's derivative, as dense backward does in place)
        if (MODE != MODE_BACKWARD) {
            floatx4 acc = zero4, acc2 = zero4;
            const lptr wp = w3l + r16 * HS + 64 * q;
            const lptr ap = h2 + (16 * w + r16) * HS + 64 * q;
#pragma unroll 16
            for (int u = 0; u < 64; u += 2) {
                acc = mfma16(ap[u], wp[u], acc);
                acc2 = mfma16(ap[u + 1], wp[u + 1], acc2);
            }
            acc += acc2;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * w + 4 * q + v, grow = r0 + row;
                const bool ok = r16 < A.out && grow < A.batch;
                const float pre = acc[v] + bias3, yv = rlt_act(pre, A.act3);
                if (ok && A.y) A.y[(size_t)grow * A.ldy + r16] = yv;
                if (MODE == MODE_FORWARD) {
                    if (ok && A.act_pre[2]) A.act_pre[2][(size_t)grow * A.out + r16] = pre;
                } else {
                    const float raw = dp3[row * DS + r16];
                    float d = A.target ? (yv - raw) * A.mse_scale : raw;
                    d *= rlt_dact_from_output(yv, A.act3);
                    dp3[row * DS + r16] = ok ? d : 0.f;
                }
            }
            rlt_lds_barrier();
        }
        RLT_TICK(3)
        if (MODE == MODE_FORWARD) continue;
        // ---- P4: dW3 += d_pre3^T h2 (rows = outputs, wavefront w owns columns [64w, 64w+64)); db3
#pragma unroll 8
        for (int j = 0; j < 16; j++) {
            const float a = dp3[(4 * j + q) * DS + r16];
#pragma unroll
            for (int t = 0; t < 4; t++) aW3[t] = mfma16(a, h2[(4 * j + q) * HS + 64 * w + 16 * t + r16], aW3[t]);
        }
        if (tid < 16) {
            float s = 0.f;
#pragma unroll 1
            for (int rb = 0; rb < BM; rb += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = dp3[(rb + u) * DS + tid];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 8; u++) s += v[u];
            }
            db3 += s;
        }
        rlt_lds_barrier();
        RLT_TICK(4)
        // ---- P5: d_pre2 = (d_pre3 W3) * act'(h2), in place of h2
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const int nt = 2 * w + a;
            floatx16 acc[2] = {zero16, zero16};
            steps_dispatch(nk3, [&](auto steps) { constexpr int NK = decltype(steps)::value < 8 ? decltype(steps)::value : 8;
                float da[2][NK], wb[NK];
#pragma unroll
                for (int j = 0; j < NK; j++) { wb[j] = w3l[(2 * j + hi) * HS + 32 * nt + c32]; da[0][j] = dp3[c32 * DS + 2 * j + hi]; da[1][j] = dp3[(32 + c32) * DS + 2 * j + hi]; }
#pragma unroll
                for (int j = 0; j < NK; j++) { acc[0] = mfma32(da[0][j], wb[j], acc[0]); acc[1] = mfma32(da[1][j], wb[j], acc[1]); }
            });
            act_dispatch(A.act2, [&](auto kind) { constexpr int ACT = decltype(kind)::value;
#pragma unroll
            for (int mt = 0; mt < 2; mt++) {
#pragma unroll
                for (int vb = 0; vb < 16; vb += 8) {
                    float hv[8];
#pragma unroll
                    for (int v = 0; v < 8; v++) hv[v] = h2[(32 * mt + row32(vb + v, hi)) * HS + 32 * nt + c32];
#pragma unroll
                    for (int v = 0; v < 8; v++) h2[(32 * mt + row32(vb + v, hi)) * HS + 32 * nt + c32] = acc[mt][vb + v] * dact_c<ACT>(hv[v]);
                }
            }
            });
        }
        rlt_lds_barrier();
        RLT_TICK(5)
        // ---- P6: dW2 += d_pre2^T h1 (wavefront w owns row tiles 2w, 2w+1 of it); db2; d_h1 = d_pre2 W2
        {
            const lptr dbase = h2 + hi * HS + c32 + 32 * (2 * w), hbase = h1 + hi * HS + c32;
            float a0 = dbase[0], a1 = dbase[32], bv[8];
#pragma unroll
            for (int b = 0; b < 8; b++) bv[b] = hbase[32 * b];
#pragma unroll 2
            for (int k = 0; k < BM / 2; k++) {
                const int kn = k + 1 < BM / 2 ? k + 1 : k;       // operands of the next row pair, requested before this pair's matrix instructions
                const float na0 = dbase[2 * kn * HS], na1 = dbase[2 * kn * HS + 32];
                float nb[8];
#pragma unroll
                for (int b = 0; b < 8; b++) nb[b] = hbase[2 * kn * HS + 32 * b];
#pragma unroll
                for (int b = 0; b < 8; b++) {
                    aW2[0][b] = mfma32(a0, bv[b], aW2[0][b]);
                    aW2[1][b] = mfma32(a1, bv[b], aW2[1][b]);
                }
                a0 = na0; a1 = na1;
#pragma unroll
                for (int b = 0; b < 8; b++) bv[b] = nb[b];
            }
        }
        {
            float s = 0.f;
#pragma unroll 1
            for (int rb = 0; rb < BM; rb += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = h2[(rb + u) * HS + tid];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 8; u++) s += v[u];
            }
            db2 += s;
        }
        {
            floatx16 acc[2][2] = {{zero16, zero16}, {zero16, zero16}};
            contract_256(h2, A.w2b, w, lane, acc);
            rlt_lds_barrier();      // every wavefront is done reading h1
            RLT_TICK(6)
            // ---- P7: d_pre1 = d_h1 * act'(h1), in place of h1
            act_dispatch(A.act1, [&](auto kind) { constexpr int ACT = decltype(kind)::value;
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int a = 0; a < 2; a++) {
#pragma unroll
                    for (int vb = 0; vb < 16; vb += 8) {
                        float hv[8];
#pragma unroll
                        for (int v = 0; v < 8; v++) hv[v] = h1[(32 * mt + row32(vb + v, hi)) * HS + 32 * (2 * w + a) + c32];
#pragma unroll
                        for (int v = 0; v < 8; v++) h1[(32 * mt + row32(vb + v, hi)) * HS + 32 * (2 * w + a) + c32] = acc[mt][a][vb + v] * dact_c<ACT>(hv[v]);
                    }
                }
            });
        }
        rlt_lds_barrier();
        RLT_TICK(7)
        // ---- P8: dW1 += d_pre1^T x ; db1
#pragma unroll 8
        for (int k = 0; k < BM / 2; k++) {
            const float bv = xs[(2 * k + hi) * XSP + c32];
            const lptr dr = h1 + (2 * k + hi) * HS + c32;
            aW1[0] = mfma32(dr[32 * (2 * w)], bv, aW1[0]);
            aW1[1] = mfma32(dr[32 * (2 * w + 1)], bv, aW1[1]);
        }
        {
            float s = 0.f;
#pragma unroll 1
            for (int rb = 0; rb < BM; rb += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = h1[(rb + u) * HS + tid];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 8; u++) s += v[u];
            }
            db1 += s;
        }
        rlt_lds_barrier();
        RLT_TICK(8)
    }
    if (MODE == MODE_FORWARD) return;
    // ---- this workgroup's partial gradients: [dW1 | db1 | dW2 | db2 | dW3 | db3]
    const int tid = threadIdx.x, c32 = lane & 31, hi = lane >> 5, r16 = lane & 15, q = lane >> 4;
    const int count = HID * A.in + HID + HID * HID + HID + A.out * HID + A.out;
    float* P = A.partial + (size_t)blockIdx.x * ((count + 63) & ~63);      // blocks start on 256-byte boundaries: a wavefront's 256-byte load or store touches two 128-byte lines, not three
    float* pW1 = P; float* pb1 = pW1 + HID * A.in; float* pW2 = pb1 + HID; float* pb2 = pW2 + HID * HID; float* pW3 = pb2 + HID; float* pb3 = pW3 + A.out * HID;
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int o = 32 * (2 * w + a) + row32(v, hi);
            if (c32 < A.in) pW1[o * A.in + c32] = aW1[a][v];
#pragma unroll
            for (int b = 0; b < 8; b++) pW2[o * HID + 32 * b + c32] = aW2[a][b][v];
        }
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int v = 0; v < 4; v++) { const int o = 4 * q + v; if (o < A.out) pW3[o * HID + 64 * w + 16 * t + r16] = aW3[t][v]; }
    pb1[tid] = db1; pb2[tid] = db2;
    if (tid < A.out) pb3[tid] = db3;
#ifdef RLT_MLP3_PROFILE
    RLT_TICK(9)
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        printf("mlp3 phase cycles: load %llu | L1 %llu | L2 %llu | L3 %llu | dW3 %llu | dpre2 %llu | dW2+dh1 %llu | gate1 %llu | dW1 %llu | store %llu\n", phase_cycles[0], phase_cycles[1],
               phase_cycles[2], phase_cycles[3], phase_cycles[4], phase_cycles[5], phase_cycles[6], phase_cycles[7], phase_cycles[8], phase_cycles[9]);
    }
#endif
}

// destination of gradient element e (same order as a workgroup's partial block)
struct GradTargets { float* dW1; float* db1; float* dW2; float* db2; float* dW3; float* db3; int in, out; };
__device__ __forceinline__ float* grad_slot(const GradTargets& T, int e) {
    int n = HID * T.in; if (e < n) return T.dW1 + e; e -= n;
    if (e < HID) return T.db1 + e; e -= HID;
    if (e < HID * HID) return T.dW2 + e; e -= HID * HID;
    if (e < HID) return T.db2 + e; e -= HID;
    n = T.out * HID; if (e < n) return T.dW3 + e; e -= n;
    return T.db3 + e;
}
// gradient[e] += sum over the workgroups' partial values, in workgroup order. A block of 256 threads handles 64 elements; four
// threads per element each sum a quarter of the workgroups, 16 loads in flight at a time, and are combined in a fixed order.
__global__ __launch_bounds__(256) void mlp3_reduce_kernel(const float* __restrict__ partial, int groups, int count, GradTargets T) {
    const size_t stride = (size_t)((count + 63) & ~63);
    __shared__ float part[4][64];
    const int el = threadIdx.x & 63, qtr = threadIdx.x >> 6, e = blockIdx.x * 64 + el;
    const int ec = e < count ? e : count - 1;
    const int per = (groups + 3) / 4, g0 = qtr * per, g1 = min(groups, g0 + per);
    float s = 0.f;
    for (int gb = g0; gb < g1; gb += 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; u++) v[u] = partial[(size_t)min(gb + u, g1 - 1) * stride + ec];
#pragma unroll
        for (int u = 0; u < 16; u++) s += (gb + u < g1) ? v[u] : 0.f;
    }
    part[qtr][el] = s;
    __syncthreads();
    if (qtr == 0 && e < count) { float* dst = grad_slot(T, e); *dst += (part[0][el] + part[1][el]) + (part[2][el] + part[3][el]); }
}

bool act_ok(int a) { return a == RLT_ACT_IDENTITY || a == RLT_ACT_RELU || a == RLT_ACT_TANH || a == RLT_ACT_FAST_TANH || a == RLT_ACT_SIGMOID; }
bool shape_ok(const rlt_dense_layer* L, int n) {
    return n == 3 && L[0].in_dim >= 1 && L[0].in_dim <= 32 && L[0].out_dim == HID && L[1].in_dim == HID && L[1].out_dim == HID && L[2].in_dim == HID &&
           L[2].out_dim >= 1 && L[2].out_dim <= 16 && act_ok(L[0].activation) && act_ok(L[1].activation) && act_ok(L[2].activation);
}
int workgroups_for(int batch) { const int tiles = (batch + BM - 1) / BM; return tiles < MAX_WORKGROUPS ? tiles : MAX_WORKGROUPS; }
size_t gradient_count(const rlt_dense_layer* L) { return (size_t)HID * L[0].in_dim + HID + (size_t)HID * HID + HID + (size_t)L[2].out_dim * HID + L[2].out_dim; }

}  // namespace

size_t rlt_mlp3_fused_workspace_bytes(const rlt_dense_layer* layers, int n_layers, int batch) {
    if (!shape_ok(layers, n_layers) || batch < 1) return 0;
    return (PREP_FLOATS + (size_t)workgroups_for(batch) * ((gradient_count(layers) + 63) & ~(size_t)63)) * sizeof(float) + 256;
}

namespace {

Mlp3Args base_args(const rlt_dense_layer* L, const float* x, int ldx, int batch, float* prep) {
    Mlp3Args a = {};
    a.x = x; a.ldx = ldx; a.batch = batch; a.in = L[0].in_dim; a.out = L[2].out_dim;
    a.act1 = L[0].activation; a.act2 = L[1].activation; a.act3 = L[2].activation;
    a.n_tiles = (batch + BM - 1) / BM;
    a.b1 = L[0].biases; a.b2 = L[1].biases; a.b3 = L[2].biases;
    a.w2f = prep; a.w2b = a.w2f + W2F_FLOATS; a.w1s = a.w2b + W2B_FLOATS; a.W3 = L[2].weights;
    a.partial = prep + PREP_FLOATS;
    return a;
}
template <int MODE>
int launch_mode(rlt_rocm_device* device, const Mlp3Args& a, int groups) {
    const size_t lds_bytes = (size_t)LDS_FLOATS * sizeof(float);
    RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(mlp3_fused_kernel<MODE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    hipLaunchKernelGGL(mlp3_fused_kernel<MODE>, dim3(groups), dim3(THREADS), lds_bytes, device->stream, a);
    return rlt_launch_status(device);
}
int reduce_partials(rlt_rocm_device* device, const rlt_dense_layer* L, const Mlp3Args& a, int groups) {
    const int count = (int)gradient_count(L);
    GradTargets T = {L[0].d_weights, L[0].d_biases, L[1].d_weights, L[1].d_biases, L[2].d_weights, L[2].d_biases, L[0].in_dim, L[2].out_dim};
    hipLaunchKernelGGL(mlp3_reduce_kernel, dim3((count + 63) / 64), dim3(256), 0, device->stream, a.partial, groups, count, T);
    return rlt_launch_status(device);
}

}  // namespace

int rlt_mlp3_fused_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* L, int n, const float* x, int ldx, float* y, int ldy,
                                    const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch,
                                    void* workspace, size_t workspace_bytes) {
    if (!shape_ok(L, n)) return RLT_E_UNSUPPORTED;
    if (workspace_bytes < rlt_mlp3_fused_workspace_bytes(L, n, batch)) return RLT_E_UNSUPPORTED;
    if ((size_t)LDS_FLOATS * sizeof(float) > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    float* prep = reinterpret_cast<float*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    hipLaunchKernelGGL(mlp3_prepare_kernel, dim3(65536 / 256), dim3(256), 0, device->stream, L[0].weights, L[1].weights, L[0].in_dim, prep);
    int rc = rlt_launch_status(device);
    if (rc) return rc;
    Mlp3Args a = base_args(L, x, ldx, batch, prep);
    a.y = y; a.ldy = ldy; a.d_output = d_output; a.ldd = ldd; a.target = target; a.ldt = ldt; a.mse_scale = mse_scale;
    const int groups = workgroups_for(batch);
    if ((rc = launch_mode<MODE_FUSED>(device, a, groups))) return rc;
    return reduce_partials(device, L, a, groups);
}

// forward(mlp): every layer's pre-activations and outputs are written; the swizzled weight copies live in the device handle's scratch
int rlt_mlp3_fused_forward(rlt_rocm_device* device, const rlt_dense_layer* L, int n, const float* x, int ldx, int batch) {
    if (!shape_ok(L, n)) return RLT_E_UNSUPPORTED;
    if ((size_t)LDS_FLOATS * sizeof(float) > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    if ((((uintptr_t)L[0].output | (uintptr_t)L[1].output) & 15) != 0) return RLT_E_UNSUPPORTED;
    void* scratch = nullptr;
    int rc = rlt_scratch(device, PREP_FLOATS * sizeof(float) + 256, &scratch);
    if (rc) return rc;
    float* prep = reinterpret_cast<float*>(((uintptr_t)scratch + 255) & ~(uintptr_t)255);
    hipLaunchKernelGGL(mlp3_prepare_kernel, dim3(65536 / 256), dim3(256), 0, device->stream, L[0].weights, L[1].weights, L[0].in_dim, prep);
    if ((rc = rlt_launch_status(device))) return rc;
    Mlp3Args a = base_args(L, x, ldx, batch, prep);
    for (int l = 0; l < 3; l++) { a.act_pre[l] = L[l].pre_activations; a.act_out[l] = L[l].output; }
    a.y = L[2].output; a.ldy = L[2].out_dim;
    return launch_mode<MODE_FORWARD>(device, a, workgroups_for(batch));
}

// backward(mlp) with weight gradients and no input gradient; d_pre_last is the gradient at the last layer's pre-activations
int rlt_mlp3_fused_backward(rlt_rocm_device* device, const rlt_dense_layer* L, int n, const float* x, int ldx, const float* d_pre_last, int ldd, int batch,
                            void* workspace, size_t workspace_bytes) {
    if (!shape_ok(L, n) || !L[0].output || !L[1].output) return RLT_E_UNSUPPORTED;
    if (workspace_bytes < rlt_mlp3_fused_workspace_bytes(L, n, batch)) return RLT_E_UNSUPPORTED;
    if ((size_t)LDS_FLOATS * sizeof(float) > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    if ((((uintptr_t)L[0].output | (uintptr_t)L[1].output) & 15) != 0) return RLT_E_UNSUPPORTED;      // the activations are read back 16 bytes at a time
    float* prep = reinterpret_cast<float*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    hipLaunchKernelGGL(mlp3_prepare_kernel, dim3(65536 / 256), dim3(256), 0, device->stream, L[0].weights, L[1].weights, L[0].in_dim, prep);
    int rc = rlt_launch_status(device);
    if (rc) return rc;
    Mlp3Args a = base_args(L, x, ldx, batch, prep);
    a.d_output = d_pre_last; a.ldd = ldd;
    a.act_out[0] = L[0].output; a.act_out[1] = L[1].output;
    const int groups = workgroups_for(batch);
    if ((rc = launch_mode<MODE_BACKWARD>(device, a, groups))) return rc;
    return reduce_partials(device, L, a, groups);
}
