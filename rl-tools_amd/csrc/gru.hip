// GRU layer: forward with kept intermediates and backward through time.
// reference: nn/layers/gru/operations_generic.h:231-341 (evaluate / forward), :594-795 (_backward per step, from the last step to the
// first). The reference walks the sequence on the host and issues a handful of small tensor operations per step.
//
// Here the work is split by what depends on time:
//   * W_i x + b_i for ALL steps is one contraction over sequence*batch rows (gemm.hip), written straight into post_activation;
//   * the recurrence runs in ONE launch: batch rows are independent, so no grid-wide synchronisation is needed. At hidden width 64 a
//     wavefront owns one row for the whole sequence with W_h in its registers; at other widths a workgroup owns a few rows and keeps W_h
//     and its rows' hidden state in LDS;
//   * backward does the same in reverse and stores, per step, the gradient at the gate pre-activations (one copy as the input path sees
//     it, one as the hidden path sees it, which differs in the n gate by the factor r) and the previous hidden state; the weight
//     gradients and d_input are then three contractions over sequence*batch rows.
#include "common.h"
#include "gemm.h"

namespace {

constexpr int GRU_THREADS = 256;

struct GruArgs {
    rlt_gru_layer L;
    const float* input; const uint8_t* reset;
    float* d_output; float* buffer_input; float* buffer_hidden; float* h_previous; float* db_hn_partial;
    int S, B, rows_per_group;
};

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
// the gate functions; fast = the rational approximations of math/operations_generic.h:247-255 (a wavefront-uniform switch)
__device__ __forceinline__ float gate_sigmoid(float x, int fast) { return fast ? 0.5f * rlt_fast_tanh(0.5f * x) + 0.5f : sigmoidf_(x); }
__device__ __forceinline__ float gate_tanh(float x, int fast) { return fast ? rlt_fast_tanh(x) : tanhf(x); }

// post_activation holds W_i x + b_i on entry. Thread (row, j): hidden unit j of one batch row.
__global__ __launch_bounds__(GRU_THREADS) void gru_forward_kernel(GruArgs A) {
    extern __shared__ float lds[];
    const int H = A.L.hidden_dim, H3 = 3 * H, R = A.rows_per_group;
    float* wt = lds;                 // W_h transposed: wt[k * 3H + j]
    float* hs = wt + (size_t)H3 * H; // hidden state of the workgroup's rows
    for (int i = threadIdx.x; i < H3 * H; i += blockDim.x) { const int j = i / H, k = i - j * H; wt[k * H3 + j] = A.L.weights_hidden[i]; }
    const int row = threadIdx.x / H, j = threadIdx.x - row * H, b = blockIdx.x * R + row;
    const bool active = row < R && b < A.B;
    const float bhr = active ? A.L.biases_hidden[j] : 0.f, bhz = active ? A.L.biases_hidden[H + j] : 0.f, bhn = active ? A.L.biases_hidden[2 * H + j] : 0.f;
    const float h0 = active ? A.L.initial_hidden_state[j] : 0.f;
    float h = h0;
    for (int t = 0; t < A.S; t++) {
        if (active) {
            if (t == 0 || (A.reset && A.reset[(size_t)t * A.B + b])) h = h0;
            hs[row * H + j] = h;
        }
        __syncthreads();
        if (active) {
            float ar = bhr, az = bhz, an = bhn;
            const float* hr = hs + row * H;
            for (int k = 0; k < H; k++) { const float hk = hr[k]; const float* w = wt + k * H3; ar += hk * w[j]; az += hk * w[H + j]; an += hk * w[2 * H + j]; }
            float* post = A.L.post_activation + ((size_t)t * A.B + b) * H3;
            const float r = gate_sigmoid(post[j] + ar, A.L.fast_tanh), z = gate_sigmoid(post[H + j] + az, A.L.fast_tanh);
            const float n = gate_tanh(post[2 * H + j] + an * r, A.L.fast_tanh);
            post[j] = r; post[H + j] = z; post[2 * H + j] = n;
            A.L.n_pre_pre_activation[((size_t)t * A.B + b) * H + j] = an;
            h = (1.0f - z) * n + z * h;
            A.L.output[((size_t)t * A.B + b) * H + j] = h;
        }
        __syncthreads();
    }
}

// Reverse pass. Thread (row, j). d_output is accumulated into in place as in the reference.
__global__ __launch_bounds__(GRU_THREADS) void gru_backward_kernel(GruArgs A) {
    extern __shared__ float lds[];
    const int H = A.L.hidden_dim, H3 = 3 * H, R = A.rows_per_group;
    float* w = lds;                          // W_h row-major: w[j * H + k]
    float* bs = w + (size_t)H3 * H;          // hidden-path gate gradients of the workgroup's rows: bs[row * 3H + j]
    for (int i = threadIdx.x; i < H3 * H; i += blockDim.x) w[i] = A.L.weights_hidden[i];
    const int row = threadIdx.x / H, j = threadIdx.x - row * H, b = blockIdx.x * R + row;
    const bool active = row < R && b < A.B;
    const float h0 = active ? A.L.initial_hidden_state[j] : 0.f;
    float carry = 0.f;       // gradient arriving at this step's hidden state from the step after it
    float db_hn = 0.f;
    __syncthreads();
    for (int t = A.S - 1; t >= 0; t--) {
        bool from_initial = true;
        if (active) {
            const size_t at = (size_t)t * A.B + b;
            from_initial = t == 0 || (A.reset && A.reset[at]);
            const float* post = A.L.post_activation + at * H3;
            const float r = post[j], z = post[H + j], n = post[2 * H + j];
            const float hp = from_initial ? h0 : A.L.output[((size_t)(t - 1) * A.B + b) * H + j];
            const float dh = A.d_output[at * H + j] + carry;
            A.d_output[at * H + j] = dh;
            const float gz = dh * (hp - n) * z * (1.0f - z);
            const float gn = dh * (1.0f - z) * (1.0f - n * n);
            const float gr = gn * A.L.n_pre_pre_activation[at * H + j] * r * (1.0f - r);
            float* bi = A.buffer_input + at * H3; float* bh = A.buffer_hidden + at * H3;
            bi[j] = gr; bi[H + j] = gz; bi[2 * H + j] = gn;
            bh[j] = gr; bh[H + j] = gz; bh[2 * H + j] = gn * r;
            A.h_previous[at * H + j] = hp;
            bs[row * H3 + j] = gr; bs[row * H3 + H + j] = gz; bs[row * H3 + 2 * H + j] = gn * r;
            // the reference drops reset samples (t > 0) from the b_hn gradient (their buffer rows are zeroed before that sum, :716-749)
            if (!(t > 0 && from_initial)) db_hn += gn * r;
            carry = from_initial ? 0.f : dh * z;
        }
        __syncthreads();
        if (active && !from_initial) {
            float acc = 0.f;
            const float* br = bs + row * H3;
            for (int jj = 0; jj < H3; jj++) acc += br[jj] * w[jj * H + j];       // d h_prev[j] += sum over gates of buffer * W_h[., j]
            carry += acc;
        }
        __syncthreads();
    }
    if (active && A.db_hn_partial) A.db_hn_partial[(size_t)b * H + j] = db_hn;
}

// ---- hidden widths 64, 32 and 16: W_h in registers, no LDS, no barrier -------------------------------------------------------
// A wavefront carries 64 / H batch rows; lane (row, j) owns hidden unit j of its row and keeps rows j, H + j, 2H + j of W_h (3H values) in
// registers for the whole sequence. The previous hidden state reaches the lanes of its row through H lane reads per step at H = 64, where the
// wavefront is one row, and through a 64-float slot of LDS private to the wavefront below that (one write, H / 4 broadcast reads of four
// values); a step needs no workgroup barrier, and the wavefronts of a workgroup are independent (they only share the launch). The step's inputs W_i x + b_i
// are requested one step ahead.
__device__ __forceinline__ float lane_read(float x, int k) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), k)); }
// lanes of one wavefront exchange data through LDS: the hardware executes a wavefront's LDS instructions in order, the fences keep the
// compiler from moving them across
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int H, bool FAST>
__global__ __launch_bounds__(GRU_THREADS) void gru_forward_reg_kernel(GruArgs A) {
    constexpr int G = 64 / H;                               // batch rows per wavefront
    __shared__ __align__(16) float exchange[GRU_THREADS / 64][1][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, u = lane & (H - 1), row_base = lane & ~(H - 1);
    const int b = (blockIdx.x * (GRU_THREADS / 64) + wave) * G + lane / H;
    if (b >= A.B) return;                                   // the lanes of whole rows leave; lane reads stay within a row; no barrier follows
    float wr[H], wz[H], wn[H];
    {
        const float4* r4 = reinterpret_cast<const float4*>(A.L.weights_hidden + (size_t)u * H);
        const float4* z4 = reinterpret_cast<const float4*>(A.L.weights_hidden + (size_t)(H + u) * H);
        const float4* n4 = reinterpret_cast<const float4*>(A.L.weights_hidden + (size_t)(2 * H + u) * H);
#pragma unroll
        for (int q = 0; q < H / 4; q++) {
            const float4 a = r4[q], c = z4[q], d = n4[q];
            wr[4 * q] = a.x; wr[4 * q + 1] = a.y; wr[4 * q + 2] = a.z; wr[4 * q + 3] = a.w;
            wz[4 * q] = c.x; wz[4 * q + 1] = c.y; wz[4 * q + 2] = c.z; wz[4 * q + 3] = c.w;
            wn[4 * q] = d.x; wn[4 * q + 1] = d.y; wn[4 * q + 2] = d.z; wn[4 * q + 3] = d.w;
        }
    }
    const float bhr = A.L.biases_hidden[u], bhz = A.L.biases_hidden[H + u], bhn = A.L.biases_hidden[2 * H + u];
    const float h0 = A.L.initial_hidden_state[u];
    float h = h0;
    const size_t stride = (size_t)A.B * 3 * H;
    float* post = A.L.post_activation + (size_t)b * 3 * H;
    float xr = post[u], xz = post[H + u], xn = post[2 * H + u];
    int rs = A.reset ? A.reset[b] : 0;
    // The inputs of later steps are requested D steps ahead and wait in a queue of D - 1 entries. Consecutive steps lie 12 H B bytes apart, on
    // other pages; two steps of distance pay at widths 16 and 32 (85 -> 59 us for 101 steps at 32), at 64 one step measures faster (60 against 67 us).
    constexpr int D = H == 64 ? 1 : 2, Q = D > 1 ? D - 1 : 1;
    float qr[Q], qz[Q], qn[Q]; int qs[Q];
#pragma unroll
    for (int d = 0; d < D - 1; d++) {
        const int tq = d + 1 < A.S ? d + 1 : A.S - 1;
        const float* pq = A.L.post_activation + (size_t)tq * stride + (size_t)b * 3 * H;
        qr[d] = pq[u]; qz[d] = pq[H + u]; qn[d] = pq[2 * H + u]; qs[d] = A.reset ? A.reset[(size_t)tq * A.B + b] : 0;
    }
    for (int t = 0; t < A.S; t++) {
        // (the last steps request the last one again: no branch around the loads)
        const int tn = t + D < A.S ? t + D : A.S - 1;
        const float* pn = A.L.post_activation + (size_t)tn * stride + (size_t)b * 3 * H;
        const float fr = pn[u], fz = pn[H + u], fn = pn[2 * H + u];
        const int fs = A.reset ? A.reset[(size_t)tn * A.B + b] : 0;
        if (t == 0 || rs) h = h0;
        float ar = bhr, az = bhz, an = bhn;
        if (H == 64) {       // measured: 64 scalar lane reads beat the LDS slot here (60 against 67 us for 64 steps), in the reverse pass they lose (103 against 64 us)
#pragma unroll
            for (int k = 0; k < H; k++) { const float hk = lane_read(h, k); ar += hk * wr[k]; az += hk * wz[k]; an += hk * wn[k]; }
        } else {
            float* xw = &exchange[wave][0][0];
            xw[lane] = h;
            wave_sync();
#pragma unroll
            for (int k = 0; k < H; k += 4) {
                const float4 hv = *reinterpret_cast<const float4*>(xw + row_base + k);
                ar += hv.x * wr[k]; az += hv.x * wz[k]; an += hv.x * wn[k];
                ar += hv.y * wr[k + 1]; az += hv.y * wz[k + 1]; an += hv.y * wn[k + 1];
                ar += hv.z * wr[k + 2]; az += hv.z * wz[k + 2]; an += hv.z * wn[k + 2];
                ar += hv.w * wr[k + 3]; az += hv.w * wz[k + 3]; an += hv.w * wn[k + 3];
            }
            wave_sync();
        }
        const float r = gate_sigmoid(xr + ar, FAST), z = gate_sigmoid(xz + az, FAST);
        const float n = gate_tanh(xn + an * r, FAST);
        float* po = A.L.post_activation + (size_t)t * stride + (size_t)b * 3 * H;
        po[u] = r; po[H + u] = z; po[2 * H + u] = n;
        const size_t at = ((size_t)t * A.B + b) * H + u;
        A.L.n_pre_pre_activation[at] = an;
        h = (1.0f - z) * n + z * h;
        A.L.output[at] = h;
        if (D == 1) { xr = fr; xz = fz; xn = fn; rs = fs; }
        else {
            xr = qr[0]; xz = qz[0]; xn = qn[0]; rs = qs[0];
#pragma unroll
            for (int d = 0; d + 1 < D - 1; d++) { qr[d] = qr[d + 1]; qz[d] = qz[d + 1]; qn[d] = qn[d + 1]; qs[d] = qs[d + 1]; }
            qr[Q - 1] = fr; qz[Q - 1] = fz; qn[Q - 1] = fn; qs[Q - 1] = fs;
        }
    }
}

// Reverse pass at these widths: lane (row, k) keeps column k of W_h (the 3H weights that multiply the gate gradients on the way to
// d h_prev[k]); the gate gradients of the row's H units reach its lanes through three 64-float slots of LDS private to the wavefront.
template <int H>
__global__ __launch_bounds__(GRU_THREADS) void gru_backward_reg_kernel(GruArgs A) {
    constexpr int G = 64 / H;
    __shared__ __align__(16) float exchange[GRU_THREADS / 64][3][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, u = lane & (H - 1), row_base = lane & ~(H - 1);
    const int b = (blockIdx.x * (GRU_THREADS / 64) + wave) * G + lane / H;
    if (b >= A.B) return;
    float cr[H], cz[H], cn[H];
#pragma unroll
    for (int j = 0; j < H; j++) {
        cr[j] = A.L.weights_hidden[(size_t)j * H + u]; cz[j] = A.L.weights_hidden[(size_t)(H + j) * H + u]; cn[j] = A.L.weights_hidden[(size_t)(2 * H + j) * H + u];
    }
    const float h0 = A.L.initial_hidden_state[u];
    float carry = 0.f, db_hn = 0.f;
    // a step's saved values are requested two steps ahead (consecutive steps lie on different pages); steps before the first read the first again
    struct Saved { float r, z, n, npp, dy, hp; int rs; };
    auto request = [&](int t) {
        const size_t a = (size_t)(t > 0 ? t : 0) * A.B + b;
        Saved v;
        v.r = A.L.post_activation[a * 3 * H + u]; v.z = A.L.post_activation[a * 3 * H + H + u]; v.n = A.L.post_activation[a * 3 * H + 2 * H + u];
        v.npp = A.L.n_pre_pre_activation[a * H + u]; v.dy = A.d_output[a * H + u];
        v.hp = A.L.output[((size_t)(t > 1 ? t - 1 : 0) * A.B + b) * H + u];
        v.rs = A.reset ? A.reset[a] : 0;
        return v;
    };
    Saved cur = request(A.S - 1), nxt = request(A.S - 2);
    for (int t = A.S - 1; t >= 0; t--) {
        const size_t at = (size_t)t * A.B + b;
        const Saved far = request(t - 2);
        const float r = cur.r, z = cur.z, n = cur.n, npp = cur.npp, dy = cur.dy, hp_raw = cur.hp;
        const int rs = cur.rs;
        const bool from_initial = t == 0 || rs;
        const float hp = from_initial ? h0 : hp_raw;
        const float dh = dy + carry;
        A.d_output[at * H + u] = dh;
        const float gz = dh * (hp - n) * z * (1.0f - z);
        const float gn = dh * (1.0f - z) * (1.0f - n * n);
        const float gr = gn * npp * r * (1.0f - r);
        const float gnr = gn * r;
        float* bi = A.buffer_input + at * 3 * H; float* bh = A.buffer_hidden + at * 3 * H;
        bi[u] = gr; bi[H + u] = gz; bi[2 * H + u] = gn;
        bh[u] = gr; bh[H + u] = gz; bh[2 * H + u] = gnr;
        A.h_previous[at * H + u] = hp;
        // the reference drops reset samples (t > 0) from the b_hn gradient (their buffer rows are zeroed before that sum, :716-749)
        if (!(t > 0 && from_initial)) db_hn += gnr;
        // the rows of one wavefront restart at different steps: every lane forms the sum, a restarting row drops it
        float a0 = dh * z, a1 = 0.f, a2 = 0.f;
        {
            float* xw = &exchange[wave][0][0];
            xw[lane] = gr; xw[64 + lane] = gz; xw[128 + lane] = gnr;
            wave_sync();
#pragma unroll
            for (int j = 0; j < H; j += 4) {
                const float4 vr = *reinterpret_cast<const float4*>(xw + row_base + j), vz = *reinterpret_cast<const float4*>(xw + 64 + row_base + j),
                             vn = *reinterpret_cast<const float4*>(xw + 128 + row_base + j);
                a0 += vr.x * cr[j]; a1 += vz.x * cz[j]; a2 += vn.x * cn[j];
                a0 += vr.y * cr[j + 1]; a1 += vz.y * cz[j + 1]; a2 += vn.y * cn[j + 1];
                a0 += vr.z * cr[j + 2]; a1 += vz.z * cz[j + 2]; a2 += vn.z * cn[j + 2];
                a0 += vr.w * cr[j + 3]; a1 += vz.w * cz[j + 3]; a2 += vn.w * cn[j + 3];
            }
            wave_sync();
        }
        carry = from_initial ? 0.f : a0 + (a1 + a2);
        cur = nxt; nxt = far;
    }
    if (A.db_hn_partial) A.db_hn_partial[(size_t)b * H + u] = db_hn;
}

// ---- hidden width 64: the recurrence on the matrix cores -------------------------------------------------------------------------
// A workgroup of four wavefronts carries FOUR batch rows through the sequence; W_h stays in registers as the B operand of
// v_mfma_f32_4x4x1_16b_f32 (16 blocks of a 4 x 1 by 1 x 4 product: lane 4 blk + i supplies A[i], lane 4 blk + j supplies B[j], register i of
// lane 4 blk + j receives D[i][j]; with the broadcast control set to 16 blocks every block takes its A from the block the instruction names,
// so one register of previous hidden states feeds 16 reduction steps). The four rows are the A side (i = row), a block is one hidden unit and
// its four columns are that unit's r, z and n gates (the fourth is idle): 64 instructions of 8 cycles replace the 192 multiply-adds and 64
// lane reads per lane of the vector version, and a step takes about half its time at any batch size (the chain of dependent steps, not the
// arithmetic, bounds both).
// The gates at this width on the hardware's exponential and reciprocal (v_exp_f32, v_rcp_f32: 1 ulp each; absolute error of a gate below 3e-7, an order
// below the tolerance the layer is held to): the library routines cost 500 cycles of every step's 1,900, these 300.
__device__ __forceinline__ float hw_sigmoid(float x) { return __frcp_rn(1.0f + __expf(-x)); }
__device__ __forceinline__ float hw_tanh(float x) { return 1.0f - 2.0f * __frcp_rn(__expf(2.0f * x) + 1.0f); }
typedef float gru_floatx4 __attribute__((ext_vector_type(4)));
constexpr int GM_ROWS = 4;
template <int ABID> __device__ __forceinline__ gru_floatx4 mfma4(float a, float b, gru_floatx4 c) { return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 4, ABID, 0); }
// 16 reduction steps: A register `a` holds, in block blk, the four rows' values of reduction index base + blk
__device__ __forceinline__ void mfma4_16(float a, const float* w, gru_floatx4& c0, gru_floatx4& c1, gru_floatx4& c2, gru_floatx4& c3) {
    c0 = mfma4<0>(a, w[0], c0); c1 = mfma4<1>(a, w[1], c1); c2 = mfma4<2>(a, w[2], c2); c3 = mfma4<3>(a, w[3], c3);
    c0 = mfma4<4>(a, w[4], c0); c1 = mfma4<5>(a, w[5], c1); c2 = mfma4<6>(a, w[6], c2); c3 = mfma4<7>(a, w[7], c3);
    c0 = mfma4<8>(a, w[8], c0); c1 = mfma4<9>(a, w[9], c1); c2 = mfma4<10>(a, w[10], c2); c3 = mfma4<11>(a, w[11], c3);
    c0 = mfma4<12>(a, w[12], c0); c1 = mfma4<13>(a, w[13], c1); c2 = mfma4<14>(a, w[14], c2); c3 = mfma4<15>(a, w[15], c3);
}

// Wavefront w owns hidden units 16 w ... 16 w + 15. hs (two copies, by the parity of the step) holds the previous hidden state of the four rows,
// unit-major: hs[unit * 4 + row]. One workgroup barrier per step; the pre-activations pass from the matrix layout (lane = unit, gate; register =
// row) to the lane that finishes (row, unit) through a slot of LDS private to the wavefront.
template <bool FAST>
__global__ __launch_bounds__(256) void gru_forward_mfma_kernel(GruArgs A) {
    constexpr int H = 64;
    __shared__ __align__(16) float hs[2][H * GM_ROWS];
    __shared__ __align__(16) float xw[4][GM_ROWS * 64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, blk = lane >> 2, j = lane & 3;
    // B operand: column j of block blk = gate j of unit 16 w + blk, one register per reduction index
    float wb[H];
    {
        const float4* src = reinterpret_cast<const float4*>(A.L.weights_hidden + ((size_t)(j < 3 ? j : 0) * H + 16 * w + blk) * H);
#pragma unroll
        for (int q = 0; q < H / 4; q++) {
            const float4 v = src[q];
            wb[4 * q] = j < 3 ? v.x : 0.f; wb[4 * q + 1] = j < 3 ? v.y : 0.f; wb[4 * q + 2] = j < 3 ? v.z : 0.f; wb[4 * q + 3] = j < 3 ? v.w : 0.f;
        }
    }
    // the lane that finishes (row, unit)
    const int row_local = lane >> 4, u = 16 * w + (lane & 15);
    const int b_raw = blockIdx.x * GM_ROWS + row_local;
    const bool live = b_raw < A.B;
    const int b = live ? b_raw : A.B - 1;      // rows beyond the batch read the last row and store nothing
    const float bhr = A.L.biases_hidden[u], bhz = A.L.biases_hidden[H + u], bhn = A.L.biases_hidden[2 * H + u];
    const float h0 = A.L.initial_hidden_state[u];
    const size_t stride = (size_t)A.B * 3 * H;
    // The inputs W_i x + b_i (and the reset flag) of step t + D are requested during step t and wait in a queue: consecutive steps lie 12 H B bytes
    // apart, and a load takes longer than a step.
    constexpr int D = 4;
    struct In { float r, z, n; int rs; };
    auto request = [&](int t) {
        const int tc = t < A.S ? t : A.S - 1;       // the last steps request the last one again: no branch around the loads
        const float* p = A.L.post_activation + (size_t)tc * stride + (size_t)b * 3 * H;
        In v; v.r = p[u]; v.z = p[H + u]; v.n = p[2 * H + u]; v.rs = A.reset ? A.reset[(size_t)tc * A.B + b] : 0;
        return v;
    };
    In q[D];
#pragma unroll
    for (int d = 0; d < D; d++) q[d] = request(d);
    float h = h0;
    hs[0][u * GM_ROWS + row_local] = h;
    for (int t = 0; t < A.S; t++) {
        rlt_lds_barrier();
        const float* hp = hs[t & 1];
        const float a0 = hp[lane], a1 = hp[64 + lane], a2 = hp[128 + lane], a3 = hp[192 + lane];
        const In far = request(t + D);
        gru_floatx4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = c0, c2 = c0, c3 = c0;
        mfma4_16(a0, wb, c0, c1, c2, c3); mfma4_16(a1, wb + 16, c0, c1, c2, c3); mfma4_16(a2, wb + 32, c0, c1, c2, c3); mfma4_16(a3, wb + 48, c0, c1, c2, c3);
        const gru_floatx4 c = (c0 + c1) + (c2 + c3);
        float* x = xw[w];
        x[lane] = c[0]; x[64 + lane] = c[1]; x[128 + lane] = c[2]; x[192 + lane] = c[3];      // x[(row * 16 + unit) * 4 + gate]
        wave_sync();
        const float4 pre = *reinterpret_cast<const float4*>(x + 4 * lane);
        wave_sync();
        const float ar = bhr + pre.x, az = bhz + pre.y, an = bhn + pre.z;
        const float r = FAST ? gate_sigmoid(q[0].r + ar, 1) : hw_sigmoid(q[0].r + ar), z = FAST ? gate_sigmoid(q[0].z + az, 1) : hw_sigmoid(q[0].z + az);
        const float n = FAST ? gate_tanh(q[0].n + an * r, 1) : hw_tanh(q[0].n + an * r);
        h = (1.0f - z) * n + z * h;
        if (live) {
            float* po = A.L.post_activation + (size_t)t * stride + (size_t)b * 3 * H;
            po[u] = r; po[H + u] = z; po[2 * H + u] = n;
            const size_t at = ((size_t)t * A.B + b) * H + u;
            A.L.n_pre_pre_activation[at] = an;
            A.L.output[at] = h;
        }
        if (t + 1 < A.S && q[1].rs) h = h0;       // the next step starts an episode
        hs[(t + 1) & 1][u * GM_ROWS + row_local] = h;
#pragma unroll
        for (int d = 0; d + 1 < D; d++) q[d] = q[d + 1];
        q[D - 1] = far;
    }
}

// Reverse pass. The gate gradients of the four rows are the A side, the reduction runs over the 192 (gate, unit) pairs -- a quarter per
// wavefront, whose B operands are rows 48 w ... 48 w + 47 of W_h (lane = column: coalesced) -- and the four partial sums of d h_prev meet in
// LDS. Thread (w, lane) finishes (row w, unit lane): its loads and stores are whole rows. Two workgroup barriers per step.
__global__ __launch_bounds__(256) void gru_backward_mfma_kernel(GruArgs A) {
    constexpr int H = 64, GS = 3 * H + 16;      // row stride of the gate gradients in LDS: rows 16 banks apart
    __shared__ float gs[GM_ROWS * GS];
    __shared__ float part[4][GM_ROWS * 64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, blk = lane >> 2, i = lane & 3;
    float wb[48];
#pragma unroll
    for (int k = 0; k < 48; k++) wb[k] = A.L.weights_hidden[(size_t)(48 * w + k) * H + lane];
    const int b_raw = blockIdx.x * GM_ROWS + w;
    const bool live = b_raw < A.B;
    const int b = live ? b_raw : A.B - 1;
    const int u = lane;
    const float h0 = A.L.initial_hidden_state[u];
    float carry = 0.f, db_hn = 0.f;
    struct Saved { float r, z, n, npp, dy, hp; int rs; };
    auto request = [&](int t) {
        const size_t a = (size_t)(t > 0 ? t : 0) * A.B + b;
        Saved v;
        v.r = A.L.post_activation[a * 3 * H + u]; v.z = A.L.post_activation[a * 3 * H + H + u]; v.n = A.L.post_activation[a * 3 * H + 2 * H + u];
        v.npp = A.L.n_pre_pre_activation[a * H + u]; v.dy = A.d_output[a * H + u];
        v.hp = A.L.output[((size_t)(t > 1 ? t - 1 : 0) * A.B + b) * H + u];
        v.rs = A.reset ? A.reset[a] : 0;
        return v;
    };
    // a step's saved values are requested D steps ahead (a load takes longer than a step); steps before the first read the first again
    constexpr int D = 3;
    Saved q[D];
#pragma unroll
    for (int d = 0; d < D; d++) q[d] = request(A.S - 1 - d);
    for (int t = A.S - 1; t >= 0; t--) {
        const size_t at = (size_t)t * A.B + b;
        const Saved far = request(t - D);
        const Saved cur = q[0];
        const bool from_initial = t == 0 || cur.rs;
        const float hp = from_initial ? h0 : cur.hp;
        const float dh = cur.dy + carry;
        const float gz = dh * (hp - cur.n) * cur.z * (1.0f - cur.z);
        const float gn = dh * (1.0f - cur.z) * (1.0f - cur.n * cur.n);
        const float gr = gn * cur.npp * cur.r * (1.0f - cur.r);
        const float gnr = gn * cur.r;
        if (live) {
            A.d_output[at * H + u] = dh;
            float* bi = A.buffer_input + at * 3 * H; float* bh = A.buffer_hidden + at * 3 * H;
            bi[u] = gr; bi[H + u] = gz; bi[2 * H + u] = gn;
            bh[u] = gr; bh[H + u] = gz; bh[2 * H + u] = gnr;
            A.h_previous[at * H + u] = hp;
        }
        // the reference drops reset samples (t > 0) from the b_hn gradient (their buffer rows are zeroed before that sum, :716-749)
        if (!(t > 0 && from_initial)) db_hn += gnr;
        gs[w * GS + u] = gr; gs[w * GS + H + u] = gz; gs[w * GS + 2 * H + u] = gnr;
        rlt_lds_barrier();
        const float* ga = gs + i * GS + 48 * w + blk;
        const float a0 = ga[0], a1 = ga[16], a2 = ga[32];
        gru_floatx4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = c0, c2 = c0, c3 = c0;
        mfma4_16(a0, wb, c0, c1, c2, c3); mfma4_16(a1, wb + 16, c0, c1, c2, c3); mfma4_16(a2, wb + 32, c0, c1, c2, c3);
        const gru_floatx4 c = (c0 + c1) + (c2 + c3);
        float* pw = part[w];
        pw[lane] = c[0]; pw[64 + lane] = c[1]; pw[128 + lane] = c[2]; pw[192 + lane] = c[3];      // part[w][row * 64 + column]
        rlt_lds_barrier();
        const float sum = (part[0][w * 64 + u] + part[1][w * 64 + u]) + (part[2][w * 64 + u] + part[3][w * 64 + u]);
        carry = from_initial ? 0.f : dh * cur.z + sum;
#pragma unroll
        for (int d = 0; d + 1 < D; d++) q[d] = q[d + 1];
        q[D - 1] = far;
    }
    if (live && A.db_hn_partial) A.db_hn_partial[(size_t)b * H + u] = db_hn;
}

// db_h[n part] += sum over batch rows of the per-row sums, db_h[r, z parts] = db_i[r, z parts] (the reference copies, :679-681).
// One workgroup per hidden unit.
__global__ __launch_bounds__(256) void gru_bias_hidden_kernel(const float* __restrict__ partial, int B, int H, const float* __restrict__ db_i, float* __restrict__ db_h) {
    __shared__ float part[4];
    const int j = blockIdx.x;
    float s = 0.f;
    for (int b = threadIdx.x; b < B; b += blockDim.x) s += partial[(size_t)b * H + j];
    s = rlt_wave_sum(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) { db_h[2 * H + j] += (part[0] + part[1]) + (part[2] + part[3]); db_h[j] = db_i[j]; db_h[H + j] = db_i[H + j]; }
}

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
bool layer_ok(const rlt_gru_layer* L) {
    return L && L->weights_input && L->biases_input && L->weights_hidden && L->biases_hidden && L->initial_hidden_state && L->post_activation &&
           L->n_pre_pre_activation && L->output && L->input_dim >= 1 && L->hidden_dim >= 1 && L->hidden_dim <= GRU_THREADS;
}
int rows_per_group(int H) { return GRU_THREADS / H; }
size_t lds_bytes(int H, bool backward) { return ((size_t)3 * H * H + (size_t)rows_per_group(H) * (backward ? 3 * H : H)) * sizeof(float); }

}  // namespace

extern "C" {

size_t rlt_rocm_gru_workspace_bytes(const rlt_gru_layer* L, int S, int B) {
    if (!L || S < 1 || B < 1 || L->hidden_dim < 1) return 0;
    const size_t rows = (size_t)S * B, H = (size_t)L->hidden_dim;
    return align256(rows * 3 * H * sizeof(float)) * 2 + align256(rows * H * sizeof(float)) + align256((size_t)B * H * sizeof(float)) + 256;
}

int rlt_rocm_gru_forward(rlt_rocm_device* device, const rlt_gru_layer* L, const float* input, const uint8_t* reset, int S, int B, void* workspace, size_t workspace_bytes) {
    (void)workspace; (void)workspace_bytes;
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_ok(L) && input && S > 0 && B > 0);
    const int H = L->hidden_dim;
    if (lds_bytes(H, false) > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    // W_i x + b_i for every step at once, into post_activation
    int rc = rlt_gemm_forward(device, input, L->input_dim, L->weights_input, L->biases_input, RLT_ACT_IDENTITY, nullptr, nullptr, L->post_activation, 3 * H, S * B, L->input_dim, 3 * H);
    if (rc) return rc;
    GruArgs a = {}; a.L = *L; a.input = input; a.reset = reset; a.S = S; a.B = B; a.rows_per_group = rows_per_group(H);
    if (H == 64 || H == 32 || H == 16) {
        const dim3 grid(rlt_div_up(B, GRU_THREADS / H)), block(GRU_THREADS);      // GRU_THREADS / 64 wavefronts of 64 / H rows
        const bool fast = L->fast_tanh != 0;      // a template parameter: as a run-time switch inside the step it cost 10% at width 64
        if (H == 64) {
            const dim3 grid4(rlt_div_up(B, GM_ROWS));
            if (fast) hipLaunchKernelGGL(gru_forward_mfma_kernel<true>, grid4, block, 0, device->stream, a); else hipLaunchKernelGGL(gru_forward_mfma_kernel<false>, grid4, block, 0, device->stream, a);
        }
        else if (H == 32) { if (fast) hipLaunchKernelGGL((gru_forward_reg_kernel<32, true>), grid, block, 0, device->stream, a); else hipLaunchKernelGGL((gru_forward_reg_kernel<32, false>), grid, block, 0, device->stream, a); }
        else { if (fast) hipLaunchKernelGGL((gru_forward_reg_kernel<16, true>), grid, block, 0, device->stream, a); else hipLaunchKernelGGL((gru_forward_reg_kernel<16, false>), grid, block, 0, device->stream, a); }
        return rlt_launch_status(device);
    }
    const size_t lds = lds_bytes(H, false);
    RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gru_forward_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(gru_forward_kernel, dim3(rlt_div_up(B, a.rows_per_group)), dim3(GRU_THREADS), lds, device->stream, a);
    return rlt_launch_status(device);
}

int rlt_rocm_gru_backward(rlt_rocm_device* device, const rlt_gru_layer* L, const float* input, float* d_output, float* d_input, const uint8_t* reset, int S, int B,
                          int want_weight_gradients, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_ok(L) && d_output && S > 0 && B > 0 && (input || !want_weight_gradients));
    RLT_REQUIRE(!want_weight_gradients || (L->d_weights_input && L->d_biases_input && L->d_weights_hidden && L->d_biases_hidden));
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_gru_workspace_bytes(L, S, B));
    const int H = L->hidden_dim, I = L->input_dim, rows = S * B;
    if (lds_bytes(H, true) > (size_t)device->lds_bytes) return RLT_E_UNSUPPORTED;
    char* w = reinterpret_cast<char*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    float* buffer_input = (float*)w; w += align256((size_t)rows * 3 * H * sizeof(float));
    float* buffer_hidden = (float*)w; w += align256((size_t)rows * 3 * H * sizeof(float));
    float* h_previous = (float*)w; w += align256((size_t)rows * H * sizeof(float));
    float* db_hn_partial = (float*)w;
    GruArgs a = {}; a.L = *L; a.input = input; a.reset = reset; a.d_output = d_output; a.buffer_input = buffer_input; a.buffer_hidden = buffer_hidden;
    a.h_previous = h_previous; a.db_hn_partial = want_weight_gradients ? db_hn_partial : nullptr; a.S = S; a.B = B; a.rows_per_group = rows_per_group(H);
    if (H == 64 || H == 32 || H == 16) {
        const dim3 grid(rlt_div_up(B, GRU_THREADS / H)), block(GRU_THREADS);
        if (H == 64) hipLaunchKernelGGL(gru_backward_mfma_kernel, dim3(rlt_div_up(B, GM_ROWS)), block, 0, device->stream, a);
        else if (H == 32) hipLaunchKernelGGL(gru_backward_reg_kernel<32>, grid, block, 0, device->stream, a);
        else hipLaunchKernelGGL(gru_backward_reg_kernel<16>, grid, block, 0, device->stream, a);
    } else {
        const size_t lds = lds_bytes(H, true);
        RLT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gru_backward_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(gru_backward_kernel, dim3(rlt_div_up(B, a.rows_per_group)), dim3(GRU_THREADS), lds, device->stream, a);
    }
    int rc = rlt_launch_status(device);
    if (rc) return rc;
    if (want_weight_gradients) {
        if ((rc = rlt_gemm_wgrad(device, buffer_input, 3 * H, input, I, L->d_weights_input, L->d_biases_input, rows, I, 3 * H, false, true))) return rc;       // :677-678
        if ((rc = rlt_gemm_wgrad(device, buffer_hidden, 3 * H, h_previous, H, L->d_weights_hidden, nullptr, rows, H, 3 * H, false, true))) return rc;         // :693-742
        hipLaunchKernelGGL(gru_bias_hidden_kernel, dim3(H), dim3(256), 0, device->stream, (const float*)db_hn_partial, B, H, (const float*)L->d_biases_input, L->d_biases_hidden);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    if (d_input) rc = rlt_gemm_backward_input(device, buffer_input, 3 * H, L->weights_input, d_input, I, nullptr, 0, 0, rows, I, 3 * H);           // :688
    return rc;
}

}  // extern "C"
