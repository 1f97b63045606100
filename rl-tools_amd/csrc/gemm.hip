// fp32 MFMA tile kernels for the three contractions of a dense layer
// (reference: nn/layers/dense/operations_cpu_blas.h:36-218 -- one sgemm each for forward, d_input and d_weights,
//  with the bias broadcast, activation, activation derivative and bias-gradient loops around them; here those loops
//  are the kernels' epilogues / side sums).
//
//   mode 0  forward        C[b][o] = act( sum_i x[b][i] W[o][i] + bias[o] )           A, B both K-contiguous
//   mode 1  d_input        C[b][i] = sum_o d_pre[b][o] W[o][i]   (* act'(pre_prev))   A K-contiguous, B N-contiguous
//   mode 2  d_weights      C[o][i] += sum_b d_pre[b][o] x[b][i], d_bias[o] += sum_b   A M-contiguous, B N-contiguous,
//                                                                                      batch split over blockIdx.z
//
// A workgroup is 4 wavefronts (256 lanes) arranged WAVES_M x WAVES_N; each wavefront owns TM x TN tiles of 32x32 and
// issues v_mfma_f32_32x32x2_f32. Operand tiles are staged through LDS k-major ([BK][rows+PAD]) so that the 32 lanes of
// a half-wavefront read 32 consecutive words (no bank conflicts) and the two halves read consecutive k.
#include "common.h"
#include "gemm.h"
#include <mutex>

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int BK = 16;
constexpr int PAD = 4;
constexpr int THREADS = 256;

struct GemmParams {
    const float* A; int lda;
    const float* B; int ldb;
    int M, N, K;
    int k_per_split;
    int vecA, vecB;
    // mode 0
    const float* bias; int act; float* pre; float* out; float* y; int ldy;
    // mode 1
    float* C; int ldc; const float* dact_pre; int dact_kind; int dact_from_output;
    // mode 2
    float* dW; float* dbias; float* ws; int splits;
};

// a KB-deep operand tile of R rows in registers: R * KB / 4 quads over the workgroup's lanes
template <int R, int KB = BK>
struct TileRegs { float4 v[(R * KB / 4 + THREADS - 1) / THREADS]; };

// source rows are contiguous along k: tile element (row r, k) = src[(row0+r)*ld + k0+k]
template <int R, int KB = BK>
__device__ __forceinline__ void gload_kcontig(TileRegs<R, KB>& t, const float* __restrict__ src, int ld, int row0, int nrows,
                                              int k0, int kend, int vec, int tid) {
    constexpr int QUADS = R * KB / 4, NQ = (QUADS + THREADS - 1) / THREADS, QPK = KB / 4;
#pragma unroll
    for (int i = 0; i < NQ; i++) {
        int q = tid + i * THREADS;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (q < QUADS) {
            int row = q / QPK, kq = (q % QPK) * 4;
            int gr = row0 + row, gk = k0 + kq;
            if (gr < nrows && gk < kend) {
                const float* p = src + (size_t)gr * ld + gk;
                if (vec == 4 && gk + 3 < kend) v = *reinterpret_cast<const float4*>(p);
                else if (vec == 2 && gk + 3 < kend) {       // rows that are only 8-byte aligned (an even leading dimension that is no multiple of 4)
                    const float2 lo = *reinterpret_cast<const float2*>(p), hi = *reinterpret_cast<const float2*>(p + 2);
                    v = make_float4(lo.x, lo.y, hi.x, hi.y);
                } else {
                    v.x = p[0];
                    if (gk + 1 < kend) v.y = p[1];
                    if (gk + 2 < kend) v.z = p[2];
                    if (gk + 3 < kend) v.w = p[3];
                }
            }
        }
        t.v[i] = v;
    }
}
template <int R, int KB = BK, int P = PAD>
__device__ __forceinline__ void sstore_kcontig(const TileRegs<R, KB>& t, float* s, int tid) {
    constexpr int QUADS = R * KB / 4, NQ = (QUADS + THREADS - 1) / THREADS, QPK = KB / 4;
#pragma unroll
    for (int i = 0; i < NQ; i++) {
        int q = tid + i * THREADS;
        if (q < QUADS) {
            int row = q / QPK, kq = (q % QPK) * 4;
            s[(kq + 0) * (R + P) + row] = t.v[i].x;
            s[(kq + 1) * (R + P) + row] = t.v[i].y;
            s[(kq + 2) * (R + P) + row] = t.v[i].z;
            s[(kq + 3) * (R + P) + row] = t.v[i].w;
        }
    }
}
// source rows are k, contiguous along the tile's m/n: tile element (k, c) = src[(k0+k)*ld + col0+c]
template <int R, int KB = BK>
__device__ __forceinline__ void gload_mncontig(TileRegs<R, KB>& t, const float* __restrict__ src, int ld, int col0, int ncols,
                                               int k0, int kend, int vec, int tid) {
    constexpr int QUADS = R * KB / 4, NQ = (QUADS + THREADS - 1) / THREADS;
    constexpr int QPR = R / 4;  // quads per k-row
#pragma unroll
    for (int i = 0; i < NQ; i++) {
        int q = tid + i * THREADS;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (q < QUADS) {
            int k = q / QPR, c4 = (q % QPR) * 4;
            int gk = k0 + k, gc = col0 + c4;
            if (gk < kend && gc < ncols) {
                const float* p = src + (size_t)gk * ld + gc;
                if (vec == 4 && gc + 3 < ncols) v = *reinterpret_cast<const float4*>(p);
                else if (vec == 2 && gc + 3 < ncols) {
                    const float2 lo = *reinterpret_cast<const float2*>(p), hi = *reinterpret_cast<const float2*>(p + 2);
                    v = make_float4(lo.x, lo.y, hi.x, hi.y);
                } else {
                    v.x = p[0];
                    if (gc + 1 < ncols) v.y = p[1];
                    if (gc + 2 < ncols) v.z = p[2];
                    if (gc + 3 < ncols) v.w = p[3];
                }
            }
        }
        t.v[i] = v;
    }
}
template <int R, int KB = BK, int P = PAD>
__device__ __forceinline__ void sstore_mncontig(const TileRegs<R, KB>& t, float* s, int tid) {
    constexpr int QUADS = R * KB / 4, NQ = (QUADS + THREADS - 1) / THREADS;
    constexpr int QPR = R / 4;
#pragma unroll
    for (int i = 0; i < NQ; i++) {
        int q = tid + i * THREADS;
        if (q < QUADS) {
            int k = q / QPR, c4 = (q % QPR) * 4;
            *reinterpret_cast<float4*>(&s[k * (R + P) + c4]) = t.v[i];
        }
    }
}

template <int MODE, int WAVES_M, int WAVES_N, int TM, int TN>
__global__ __launch_bounds__(THREADS) void gemm_kernel(GemmParams p) {
    static_assert(WAVES_M * WAVES_N == 4, "four wavefronts per workgroup");
    constexpr int BM = WAVES_M * TM * 32;
    constexpr int BN = WAVES_N * TN * 32;
    constexpr int KB = BK;
    __shared__ __attribute__((aligned(16))) float sA[2][KB * (BM + PAD)];
    __shared__ __attribute__((aligned(16))) float sB[2][KB * (BN + PAD)];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    int ks = 0, ke = p.K;
    if (MODE == 2) { ks = blockIdx.z * p.k_per_split; ke = min(p.K, ks + p.k_per_split); }
    const int nk = (ke - ks + KB - 1) / KB;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    TileRegs<BM, KB> ra;
    TileRegs<BN, KB> rb;
    auto gload = [&](int k0) {
        if (MODE == 2) gload_mncontig<BM, KB>(ra, p.A, p.lda, m0, p.M, k0, ke, p.vecA, tid);
        else gload_kcontig<BM, KB>(ra, p.A, p.lda, m0, p.M, k0, ke, p.vecA, tid);
        if (MODE == 0) gload_kcontig<BN, KB>(rb, p.B, p.ldb, n0, p.N, k0, ke, p.vecB, tid);
        else gload_mncontig<BN, KB>(rb, p.B, p.ldb, n0, p.N, k0, ke, p.vecB, tid);
    };
    auto sstore = [&](int buf) {
        if (MODE == 2) sstore_mncontig<BM, KB>(ra, sA[buf], tid); else sstore_kcontig<BM, KB>(ra, sA[buf], tid);
        if (MODE == 0) sstore_kcontig<BN, KB>(rb, sB[buf], tid); else sstore_mncontig<BN, KB>(rb, sB[buf], tid);
    };

    const bool bias_block = (MODE == 2) && (blockIdx.x == 0) && (p.dbias != nullptr);
    float bsum = 0.0f;

    if (nk > 0) { gload(ks); sstore(0); }
    __syncthreads();
    for (int t = 0; t < nk; t++) {
        const int cur = t & 1;
        if (t + 1 < nk) gload(ks + (t + 1) * KB);
        const float* a_base = sA[cur] + (lane >> 5) * (BM + PAD) + wm * (TM * 32) + (lane & 31);
        const float* b_base = sB[cur] + (lane >> 5) * (BN + PAD) + wn * (TN * 32) + (lane & 31);
#pragma unroll
        for (int kk = 0; kk < KB / 2; kk++) {
            float a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = a_base[kk * 2 * (BM + PAD) + i * 32];
#pragma unroll
            for (int j = 0; j < TN; j++) b[j] = b_base[kk * 2 * (BN + PAD) + j * 32];
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (bias_block && tid < BM) {
#pragma unroll
            for (int k = 0; k < KB; k++) bsum += sA[cur][k * (BM + PAD) + tid];
        }
        if (t + 1 < nk) sstore(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue. Accumulator element v of lane l in a 32x32 tile: row = 8*(v/4) + 4*(l/32) + v%4, col = l%32.
    // What a tile reads from memory (the bias of its column, the activation-derivative operands or the gradient so far of its 16 elements) is
    // requested before its first store: a read issued between the stores waits for every store before it, one memory round trip per element.
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = n0 + wn * (TN * 32) + j * 32 + (lane & 31);
            const int row_base = m0 + wm * (TM * 32) + i * 32 + 4 * (lane >> 5);
            const bool col_ok = col < p.N;
            float bias_c = 0.0f;
            if (MODE == 0 && p.bias && col_ok) bias_c = p.bias[col];
            float operand[16];
            const bool want_operand = MODE == 1 ? p.dact_pre != nullptr : (MODE == 2 && p.splits == 1);
            if (MODE != 0 && want_operand) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int row = row_base + 8 * (v >> 2) + (v & 3);
                    const float* src = MODE == 1 ? p.dact_pre : p.dW;
                    operand[v] = (row < p.M && col_ok) ? src[(size_t)row * p.N + col] : 0.0f;
                }
            }
            // everything that depends on those reads is computed before the first store too (a use of a loaded value further down, in a block of its own,
            // would again wait for all memory operations before it)
            float val[16];
#pragma unroll
            for (int v = 0; v < 16; v++) {
                val[v] = acc[i][j][v];
                if (MODE == 0) val[v] += bias_c;
                else if (MODE == 1) { if (p.dact_pre) val[v] *= p.dact_from_output ? rlt_dact_from_output(operand[v], p.dact_kind) : rlt_dact(operand[v], p.dact_kind); }
                else if (p.splits == 1) val[v] = operand[v] + val[v];
                asm volatile("" : "+v"(val[v]));      // the value is final here: the compiler would otherwise sink the arithmetic into the store's block
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = row_base + 8 * (v >> 2) + (v & 3);
                if (row < p.M && col_ok) {
                    if (MODE == 0) {
                        if (p.pre) p.pre[(size_t)row * p.N + col] = val[v];
                        float o = rlt_act(val[v], p.act);
                        if (p.out) p.out[(size_t)row * p.N + col] = o;
                        if (p.y) p.y[(size_t)row * p.ldy + col] = o;
                    } else if (MODE == 1) {
                        p.C[(size_t)row * p.ldc + col] = val[v];
                    } else {
                        if (p.splits == 1) p.dW[(size_t)row * p.N + col] = val[v];
                        else p.ws[(size_t)blockIdx.z * ((size_t)p.M * p.N + p.M) + (size_t)row * p.N + col] = val[v];
                    }
                }
            }
        }
    }
    if (bias_block && tid < BM && m0 + tid < p.M) {
        if (p.splits == 1) p.dbias[m0 + tid] += bsum;
        else p.ws[(size_t)blockIdx.z * ((size_t)p.M * p.N + p.M) + (size_t)p.M * p.N + m0 + tid] = bsum;
    }
}

// dW += sum_s ws[s][0:MN], dbias += sum_s ws[s][MN:MN+M]. A workgroup owns 64 consecutive outputs; its four wavefronts each sum
// a quarter of the splits (every read is a 256-byte row segment) and the four partials are combined in a fixed order.
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(float* __restrict__ dW, float* __restrict__ dbias, const float* __restrict__ ws,
                                                           int mn, int m, int splits) {
    __shared__ float partial[4][64];
    const int total = mn + (dbias ? m : 0);
    const size_t stride = (size_t)mn + m;
    const int e = blockIdx.x * 64 + (threadIdx.x & 63), g = threadIdx.x >> 6;
    float s = 0.0f;
    if (e < total)
        for (int k0 = g; k0 < splits; k0 += 32) {      // eight loads in flight, added in the order of the splits
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) { const int k = k0 + 4 * u; v[u] = k < splits ? ws[(size_t)k * stride + e] : 0.0f; }
#pragma unroll
            for (int u = 0; u < 8; u++) s += v[u];
        }
    partial[g][threadIdx.x & 63] = s;
    __syncthreads();
    if (g == 0 && e < total) {
        float r = (partial[0][threadIdx.x] + partial[1][threadIdx.x]) + (partial[2][threadIdx.x] + partial[3][threadIdx.x]);
        if (e < mn) dW[e] += r; else dbias[e - mn] += r;
    }
}

// ---- weight gradients of narrow layers over long batches ----------------------------------------------------------------------------
// dW [M x N] with M <= 192, N <= 16 NT (a GRU's 3H x I and 3H x H at hidden width 64) over tens of thousands of rows: the tiled kernel above
// cuts such a matrix into 64 x 64 tiles and every operand row is fetched by three workgroups, each with a short reduction of its own. Here a
// workgroup keeps the WHOLE gradient in accumulators (wavefront w: rows 48 w ... 48 w + 47 of dW as 3 x NT tiles of v_mfma_f32_16x16x4_f32) and
// walks its share of the batch 16 rows at a time: both operands are read from memory exactly once, staged through LDS (double buffered, the
// next 16 rows requested before the current ones are multiplied, one barrier per 16 rows). The bias gradient is summed on the side from the
// registers the d_pre rows pass through. A workgroup writes one block of partial sums in the layout wgrad_reduce_kernel adds up.
typedef float wide_floatx4 __attribute__((ext_vector_type(4)));
constexpr int WIDE_M = 192, WIDE_KT = 16, WIDE_GS = WIDE_M + 16;
struct WideArgs { const float* G; int ldg; const float* X; int ldx; int M, N, K, rows_per_group; float* ws; int want_bias; };
template <int NT, int PF>
__global__ __launch_bounds__(THREADS) void wgrad_wide_kernel(WideArgs a) {
    constexpr int XS = 16 * NT + 16;                        // both strides are 16 mod 32: the four k-rows a wavefront reads fall on two sets of banks
    constexpr int GQ = WIDE_KT * WIDE_M / 4 / THREADS;      // float4 of d_pre per thread and 16 rows (3)
    constexpr int XQ = (WIDE_KT * 8 * NT + THREADS - 1) / THREADS;      // float2 of x per thread and 16 rows
    __shared__ __align__(16) float gs[2][WIDE_KT * WIDE_GS];
    __shared__ __align__(16) float xs[2][WIDE_KT * XS];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r = lane & 15, kk = lane >> 4;
    const int k_begin = blockIdx.x * a.rows_per_group, k_end = min(a.K, k_begin + a.rows_per_group);
    // 16 rows of both operands as they travel from memory to LDS. A load under load takes longer than the matrix work on 16 rows, so PF such
    // tiles are on their way at any time (with one, the kernel ran at the rate of one tile per memory latency: 2 TB/s over the whole device).
    struct Tile { float4 g[GQ]; float2 x[XQ]; };
    float4 bsum[GQ];
#pragma unroll
    for (int q = 0; q < GQ; q++) bsum[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    auto request = [&](int k0) {
        Tile t;
#pragma unroll
        for (int q = 0; q < GQ; q++) {
            const int idx = tid + THREADS * q, row = idx / (WIDE_M / 4), col = 4 * (idx % (WIDE_M / 4));
            t.g[q] = (k0 + row < k_end && col < a.M) ? *reinterpret_cast<const float4*>(a.G + (size_t)(k0 + row) * a.ldg + col) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int q = 0; q < XQ; q++) {
            const int idx = tid + THREADS * q, row = idx / (8 * NT), col = 2 * (idx % (8 * NT));
            t.x[q] = (idx < WIDE_KT * 8 * NT && k0 + row < k_end && col < a.N) ? *reinterpret_cast<const float2*>(a.X + (size_t)(k0 + row) * a.ldx + col) : make_float2(0.f, 0.f);
        }
        return t;
    };
    auto stage = [&](const Tile& t, int buf) {
#pragma unroll
        for (int q = 0; q < GQ; q++) {
            const int idx = tid + THREADS * q, row = idx / (WIDE_M / 4), col = 4 * (idx % (WIDE_M / 4));
            *reinterpret_cast<float4*>(&gs[buf][row * WIDE_GS + col]) = t.g[q];
            bsum[q].x += t.g[q].x; bsum[q].y += t.g[q].y; bsum[q].z += t.g[q].z; bsum[q].w += t.g[q].w;
        }
#pragma unroll
        for (int q = 0; q < XQ; q++) {
            const int idx = tid + THREADS * q, row = idx / (8 * NT), col = 2 * (idx % (8 * NT));
            if (idx < WIDE_KT * 8 * NT) *reinterpret_cast<float2*>(&xs[buf][row * XS + col]) = t.x[q];
        }
    };
    wide_floatx4 acc[3][NT];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = wide_floatx4{0.f, 0.f, 0.f, 0.f};
    Tile queue[PF];
    {
        const Tile first = request(k_begin);
#pragma unroll
        for (int d = 0; d < PF; d++) queue[d] = request(k_begin + (d + 1) * WIDE_KT);
        stage(first, 0);
    }
    __syncthreads();
    int buf = 0;
    for (int k0 = k_begin; k0 < k_end; k0 += WIDE_KT) {
        const Tile far = request(k0 + (PF + 1) * WIDE_KT);
        __builtin_amdgcn_sched_barrier(0);      // the requests go out first, and nothing that waits for them moves above the matrix work
        const float* g = gs[buf] + kk * WIDE_GS + 48 * w + r;
        const float* x = xs[buf] + kk * XS + r;
#pragma unroll
        for (int s4 = 0; s4 < WIDE_KT / 4; s4++) {
            float av[3], bv[NT];
#pragma unroll
            for (int i = 0; i < 3; i++) av[i] = g[4 * s4 * WIDE_GS + 16 * i];
#pragma unroll
            for (int j = 0; j < NT; j++) bv[j] = x[4 * s4 * XS + 16 * j];
#pragma unroll
            for (int i = 0; i < 3; i++)
#pragma unroll
                for (int j = 0; j < NT; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (k0 + WIDE_KT < k_end) stage(queue[0], buf ^ 1);
        rlt_lds_barrier();
        buf ^= 1;
#pragma unroll
        for (int d = 0; d + 1 < PF; d++) queue[d] = queue[d + 1];
        queue[PF - 1] = far;
    }
    // element v of lane (r, kk) of tile (i, j): dW[48 w + 16 i + 4 kk + v][16 j + r]
    float* out = a.ws + (size_t)blockIdx.x * ((size_t)a.M * a.N + a.M);
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int m = 48 * w + 16 * i + 4 * kk + v;
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const int n = 16 * j + r;
                if (m < a.M && n < a.N) out[(size_t)m * a.N + n] = acc[i][j][v];
            }
        }
    if (a.want_bias) {      // 16 row slots of column sums meet in LDS and are added in the order of the slots
        float* bs = gs[0];
#pragma unroll
        for (int q = 0; q < GQ; q++) {
            const int idx = tid + THREADS * q, row = idx / (WIDE_M / 4), col = 4 * (idx % (WIDE_M / 4));
            *reinterpret_cast<float4*>(&bs[row * WIDE_GS + col]) = bsum[q];
        }
        __syncthreads();
        if (tid < a.M) {
            float sum = 0.f;
#pragma unroll
            for (int row = 0; row < WIDE_KT; row++) sum += bs[row * WIDE_GS + tid];
            out[(size_t)a.M * a.N + tid] = sum;
        }
    }
}

// ---- the same contractions on tiles of 16x16 per wavefront -----------------------------------------------------------------------
// A problem whose 64x64 tiles number fewer than the compute units (a batch of a few hundred rows through layers a few hundred wide) leaves most of the chip
// idle while each of its workgroups works through hundreds of dependent 32x32x2 multiplies. Here a wavefront owns one 16x16 tile (v_mfma_f32_16x16x4_f32,
// a quarter of the multiply time per unit of k) and a workgroup WAVES_M x WAVES_N of them (32x32, or 64x16 / 16x64 for one narrow side): four times the
// workgroups, each with a quarter of the chain. 64 rows of k per step through one LDS buffer, LDS reads of eight multiplies in flight at a time.
// Operand A/B lane layout of the instruction: lane l holds A[row l % 16][k l / 16] and B[k l / 16][col l % 16]; accumulator element v of lane l is
// C[row 4 * (l / 16) + v][col l % 16].
template <int MODE, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(THREADS) void gemm_small_kernel(GemmParams p) {
    static_assert(WAVES_M * WAVES_N == 4, "four wavefronts per workgroup");
    constexpr int KB = 64, BM = WAVES_M * 16, BN = WAVES_N * 16;
    constexpr int PA = (48 - BM % 32) % 32, PB = (48 - BN % 32) % 32;      // k-rows 16 banks apart: the four k of a multiply's operand read fall on disjoint halves in pairs
    __shared__ __attribute__((aligned(16))) float sA[KB * (BM + PA)];
    __shared__ __attribute__((aligned(16))) float sB[KB * (BN + PB)];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    int ks = 0, ke = p.K;
    if (MODE == 2) { ks = blockIdx.z * p.k_per_split; ke = min(p.K, ks + p.k_per_split); }
    const int nk = (ke - ks + KB - 1) / KB;
    wide_floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    TileRegs<BM, KB> ra;
    TileRegs<BN, KB> rb;
    auto gload = [&](int k0) {
        if (MODE == 2) gload_mncontig<BM, KB>(ra, p.A, p.lda, m0, p.M, k0, ke, p.vecA, tid);
        else gload_kcontig<BM, KB>(ra, p.A, p.lda, m0, p.M, k0, ke, p.vecA, tid);
        if (MODE == 0) gload_kcontig<BN, KB>(rb, p.B, p.ldb, n0, p.N, k0, ke, p.vecB, tid);
        else gload_mncontig<BN, KB>(rb, p.B, p.ldb, n0, p.N, k0, ke, p.vecB, tid);
    };
    auto sstore = [&]() {
        if (MODE == 2) sstore_mncontig<BM, KB, PA>(ra, sA, tid); else sstore_kcontig<BM, KB, PA>(ra, sA, tid);
        if (MODE == 0) sstore_kcontig<BN, KB, PB>(rb, sB, tid); else sstore_mncontig<BN, KB, PB>(rb, sB, tid);
    };
    const bool bias_block = (MODE == 2) && (blockIdx.x == 0) && (p.dbias != nullptr);
    float bsum = 0.0f;
    if (nk > 0) { gload(ks); sstore(); }
    __syncthreads();
    for (int t = 0; t < nk; t++) {
        if (t + 1 < nk) gload(ks + (t + 1) * KB);
        const float* a_base = sA + (lane >> 4) * (BM + PA) + wm * 16 + (lane & 15);
        const float* b_base = sB + (lane >> 4) * (BN + PB) + wn * 16 + (lane & 15);
#pragma unroll
        for (int kk0 = 0; kk0 < KB / 4; kk0 += 8) {
            float a[8], b[8];
#pragma unroll
            for (int c = 0; c < 8; c++) { a[c] = a_base[(kk0 + c) * 4 * (BM + PA)]; b[c] = b_base[(kk0 + c) * 4 * (BN + PB)]; }
            __builtin_amdgcn_sched_barrier(0);      // keeps the eight pairs of reads ahead of the multiplies
#pragma unroll
            for (int c = 0; c < 8; c++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[c], b[c], acc, 0, 0, 0);
        }
        if (bias_block && tid < BM) {
#pragma unroll
            for (int k = 0; k < KB; k++) bsum += sA[k * (BM + PA) + tid];
        }
        __syncthreads();      // every wavefront has read this step's tile
        if (t + 1 < nk) sstore();
        __syncthreads();
    }
    // epilogue: what the tile reads from memory is requested, and everything that depends on it computed, before the first store (see gemm_kernel)
    const int col = n0 + wn * 16 + (lane & 15), row_base = m0 + wm * 16 + 4 * (lane >> 4);
    const bool col_ok = col < p.N;
    float bias_c = 0.0f;
    if (MODE == 0 && p.bias && col_ok) bias_c = p.bias[col];
    float operand[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const bool want_operand = MODE == 1 ? p.dact_pre != nullptr : (MODE == 2 && p.splits == 1);
    if (MODE != 0 && want_operand) {
        const float* src = MODE == 1 ? p.dact_pre : p.dW;
#pragma unroll
        for (int v = 0; v < 4; v++) operand[v] = (row_base + v < p.M && col_ok) ? src[(size_t)(row_base + v) * p.N + col] : 0.0f;
    }
    float val[4];
#pragma unroll
    for (int v = 0; v < 4; v++) {
        val[v] = acc[v];
        if (MODE == 0) val[v] += bias_c;
        else if (MODE == 1) { if (p.dact_pre) val[v] *= p.dact_from_output ? rlt_dact_from_output(operand[v], p.dact_kind) : rlt_dact(operand[v], p.dact_kind); }
        else if (p.splits == 1) val[v] = operand[v] + val[v];
        asm volatile("" : "+v"(val[v]));
    }
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int row = row_base + v;
        if (row < p.M && col_ok) {
            if (MODE == 0) {
                if (p.pre) p.pre[(size_t)row * p.N + col] = val[v];
                const float o = rlt_act(val[v], p.act);
                if (p.out) p.out[(size_t)row * p.N + col] = o;
                if (p.y) p.y[(size_t)row * p.ldy + col] = o;
            } else if (MODE == 1) {
                p.C[(size_t)row * p.ldc + col] = val[v];
            } else {
                if (p.splits == 1) p.dW[(size_t)row * p.N + col] = val[v];
                else p.ws[(size_t)blockIdx.z * ((size_t)p.M * p.N + p.M) + (size_t)row * p.N + col] = val[v];
            }
        }
    }
    if (bias_block && tid < BM && m0 + tid < p.M) {
        if (p.splits == 1) p.dbias[m0 + tid] += bsum;
        else p.ws[(size_t)blockIdx.z * ((size_t)p.M * p.N + p.M) + (size_t)p.M * p.N + m0 + tid] = bsum;
    }
}

// d_pre = act'(pre) * d_output (nn/layers/dense/operations_cpu_blas.h:119-141); dst may alias src
__global__ __launch_bounds__(256) void dpre_kernel(const float* src, int lds, float* dst, int ldd, const float* __restrict__ pre, int rows, int cols, int act, int from_output) {
    const size_t total = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        int r = (int)(i / cols), c = (int)(i % cols);
        dst[(size_t)r * ldd + c] = (from_output ? rlt_dact_from_output(pre[i], act) : rlt_dact(pre[i], act)) * src[(size_t)r * lds + c];
    }
}

// widest vector a row-contiguous operand can be loaded with: 4 floats (16-byte aligned base, leading dimension a multiple of 4), 2, or 1
inline int vector_width(const void* p, int ld) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    if ((a & 15u) == 0 && ld % 4 == 0) return 4;
    if ((a & 7u) == 0 && ld % 2 == 0) return 2;
    return 1;
}

// Tile shape by problem shape. One side narrow: 128x32 / 32x128. Small problems: 64x64. Otherwise, measured on 65,536-row batches at widths 146-256:
// the forward and input-gradient contractions (reduction over a layer width, i.e. a few k-steps per tile) run fastest on 128x64 tiles, which keep
// more workgroups resident to hide the short reduction's prologue and epilogue; the weight-gradient contraction (reduction over the batch) on
// 128x128 tiles unless those overhang the matrix by more than 15 % over 64x64 tiles (192 x 146 weights: 65,536 against 36,864 padded elements).
enum TileShape { TILE_128x32, TILE_32x128, TILE_64x64, TILE_128x128, TILE_128x64 };
void tile_dims(TileShape shape, int& bm, int& bn) {
    switch (shape) {
        case TILE_128x32: bm = 128; bn = 32; break;
        case TILE_32x128: bm = 32; bn = 128; break;
        case TILE_64x64: bm = 64; bn = 64; break;
        case TILE_128x64: bm = 128; bn = 64; break;
        default: bm = 128; bn = 128; break;
    }
}
long long padded_area(int M, int N, TileShape shape) {
    int bm, bn;
    tile_dims(shape, bm, bn);
    return (long long)rlt_div_up(M, bm) * bm * rlt_div_up(N, bn) * bn;
}
TileShape pick_tile(int M, int N, int mode) {
    if (N <= 32) return TILE_128x32;
    if (M <= 32) return TILE_32x128;
    if (M <= 64 || N <= 64 || (long long)M * N < 128ll * 128) return TILE_64x64;
    if (mode != 2) return TILE_128x64;
    return 100 * padded_area(M, N, TILE_128x128) <= 115 * padded_area(M, N, TILE_64x64) ? TILE_128x128 : TILE_64x64;
}

// The tile shape a contraction runs with. A grid of large tiles that leaves compute units idle runs faster as 64x64 tiles (the forward and
// input-gradient contractions do not split k to fill the chip); the weight gradient over a short batch (k_total rows) has few rows to split and
// takes 64x64 tiles as well.
constexpr int SHORT_BATCH = 2048;
TileShape plan_tile(const rlt_rocm_device* device, int M, int N, int mode, int k_total) {
    TileShape shape = pick_tile(M, N, mode);
    int bm, bn;
    tile_dims(shape, bm, bn);
    if (mode != 2 && bm >= 128 && bn >= 64 && rlt_div_up(N, bn) * rlt_div_up(M, bm) < device->compute_units) shape = TILE_64x64;
    if (mode == 2 && shape == TILE_128x128 && k_total <= SHORT_BATCH) shape = TILE_64x64;
    return shape;
}

template <int MODE>
int launch(rlt_rocm_device* device, const GemmParams& p, int splits) {
    dim3 block(THREADS);
    const TileShape shape = plan_tile(device, p.M, p.N, MODE, p.K);
    int bm, bn;
    tile_dims(shape, bm, bn);
    const dim3 grid(rlt_div_up(p.N, bn), rlt_div_up(p.M, bm), splits);
    // workgroups for at most a quarter of the compute units and a reduction of some length: four times the workgroups on 16x16 tiles per wavefront (gemm_small_kernel);
    // measured at 4,096 x 146 -> 192 (192 workgroups of 64x64): 13.7 us as it is, 15.5 us on 768 small ones
    const bool few = 4ll * grid.x * grid.y * grid.z <= device->compute_units && p.k_per_split >= 64 && shape != TILE_128x64 && shape != TILE_128x128;
    if (few) {
        if (p.N <= 16) hipLaunchKernelGGL((gemm_small_kernel<MODE, 4, 1>), dim3(rlt_div_up(p.N, 16), rlt_div_up(p.M, 64), splits), block, 0, device->stream, p);
        else if (p.M <= 16) hipLaunchKernelGGL((gemm_small_kernel<MODE, 1, 4>), dim3(rlt_div_up(p.N, 64), rlt_div_up(p.M, 16), splits), block, 0, device->stream, p);
        else hipLaunchKernelGGL((gemm_small_kernel<MODE, 2, 2>), dim3(rlt_div_up(p.N, 32), rlt_div_up(p.M, 32), splits), block, 0, device->stream, p);
        return rlt_launch_status(device);
    }
    switch (shape) {
        case TILE_128x32: hipLaunchKernelGGL((gemm_kernel<MODE, 4, 1, 1, 1>), grid, block, 0, device->stream, p); break;
        case TILE_32x128: hipLaunchKernelGGL((gemm_kernel<MODE, 1, 4, 1, 1>), grid, block, 0, device->stream, p); break;
        case TILE_64x64: hipLaunchKernelGGL((gemm_kernel<MODE, 2, 2, 1, 1>), grid, block, 0, device->stream, p); break;
        case TILE_128x64: hipLaunchKernelGGL((gemm_kernel<MODE, 2, 2, 2, 1>), grid, block, 0, device->stream, p); break;
        default: hipLaunchKernelGGL((gemm_kernel<MODE, 2, 2, 2, 2>), grid, block, 0, device->stream, p); break;
    }
    return rlt_launch_status(device);
}

}  // namespace

int rlt_gemm_forward(rlt_rocm_device* device, const float* x, int ldx, const float* W, const float* bias, int act,
                     float* pre, float* out, float* y, int ldy, int batch, int in_dim, int out_dim) {
    if (rlt_div_up(batch, 32) > 65535) return RLT_E_UNSUPPORTED;
    GemmParams p = {};
    p.A = x; p.lda = ldx; p.B = W; p.ldb = in_dim; p.M = batch; p.N = out_dim; p.K = in_dim; p.k_per_split = in_dim;
    p.vecA = vector_width(x, ldx); p.vecB = vector_width(W, in_dim);
    p.bias = bias; p.act = act; p.pre = pre; p.out = out; p.y = y; p.ldy = ldy; p.splits = 1;
    return launch<0>(device, p, 1);
}

int rlt_gemm_backward_input(rlt_rocm_device* device, const float* d_pre, int ldd, const float* W, float* d_in, int ldi,
                            const float* dact_pre, int dact_kind, int dact_from_output, int batch, int in_dim, int out_dim) {
    if (rlt_div_up(batch, 32) > 65535) return RLT_E_UNSUPPORTED;
    GemmParams p = {};
    p.A = d_pre; p.lda = ldd; p.B = W; p.ldb = in_dim; p.M = batch; p.N = in_dim; p.K = out_dim; p.k_per_split = out_dim;
    p.vecA = vector_width(d_pre, ldd); p.vecB = vector_width(W, in_dim);
    p.C = d_in; p.ldc = ldi; p.dact_pre = dact_pre; p.dact_kind = dact_kind; p.dact_from_output = dact_from_output; p.splits = 1;
    return launch<1>(device, p, 1);
}

// How the weight-gradient contraction splits the batch so that the grid fills the chip: about 2 workgroups per compute unit, at least
// 256 rows per split (64 for small gradients). Each split writes one block of out_dim * in_dim + out_dim partial sums.
static void wgrad_split(const rlt_rocm_device* device, int batch, int in_dim, int out_dim, int& splits, int& kps) {
    int bm, bn;
    tile_dims(plan_tile(device, out_dim, in_dim, 2, batch), bm, bn);
    int tiles = rlt_div_up(out_dim, bm) * rlt_div_up(in_dim, bn);
    splits = (2 * device->compute_units + tiles - 1) / tiles;
    // at least 256 rows per split; for small gradients (up to 96 x 64: the layers of width 16 and 32) 64 rows, i.e. 4 k-steps: a short batch is bound by the chain
    // of k-steps in one workgroup, and such partial sums cost little
    int max_splits = rlt_div_up(batch, (long long)in_dim * out_dim <= 96 * 64 ? 64 : 256);
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    kps = rlt_div_up(rlt_div_up(batch, splits), BK) * BK;
    splits = rlt_div_up(batch, kps);
}

// ---- partial sums without an allocation ------------------------------------------------------------------------------------
// Callers that must not allocate (code under HIP graph capture, tight serving loops) get their split-batch partial sums from this
// array instead of the handle's grow-only workspace. It is part of the library's device image: every GPU the library runs on holds
// its own copy, at its own address, from the first use of the library on that GPU to the end of the process. In host code the
// array's NAME is only a handle for hipGetSymbolAddress; what kernels and copies receive is the address looked up below.
static __device__ __align__(256) float scratch[RLT_STATIC_SCRATCH_BYTES / sizeof(float)];
namespace {
constexpr int MAX_HIP_DEVICES = 64;
float* scratch_address[MAX_HIP_DEVICES];      // per HIP device: where that GPU keeps its copy of `scratch`
std::mutex scratch_mutex;
}
int rlt_gemm_static_scratch_setup(rlt_rocm_device* device) {
    const int index = device->hip_device;
    if (index < 0 || index >= MAX_HIP_DEVICES) return RLT_E_UNSUPPORTED;
    std::lock_guard<std::mutex> guard(scratch_mutex);
    if (scratch_address[index]) return 0;
    int current = -1;
    RLT_HIP(hipGetDevice(&current));
    if (current != index) RLT_HIP(hipSetDevice(index));
    void* address = nullptr;
    const hipError_t e = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (current != index) (void)hipSetDevice(current);
    if (e != hipSuccess || !address) { device->sticky_error = (int)(e != hipSuccess ? e : hipErrorInvalidSymbol); return device->sticky_error; }
    scratch_address[index] = (float*)address;
    return 0;
}

int rlt_gemm_wgrad(rlt_rocm_device* device, const float* d_pre, int ldd, const float* x, int ldx, float* dW, float* dbias,
                   int batch, int in_dim, int out_dim, bool static_scratch, bool narrow_long) {
    GemmParams p = {};
    p.A = d_pre; p.lda = ldd; p.B = x; p.ldb = ldx; p.M = out_dim; p.N = in_dim; p.K = batch;
    p.vecA = vector_width(d_pre, ldd); p.vecB = vector_width(x, ldx);
    p.dW = dW; p.dbias = dbias;
    // narrow layer, long batch: one workgroup per share of the batch holds the whole gradient (wgrad_wide_kernel)
    if (narrow_long && !static_scratch && out_dim <= WIDE_M && out_dim % 4 == 0 && in_dim > 64 && in_dim <= 160 && in_dim % 2 == 0 && batch >= 16384 && ldd % 4 == 0 && ldx % 2 == 0 &&
        (reinterpret_cast<uintptr_t>(d_pre) & 15u) == 0 && (reinterpret_cast<uintptr_t>(x) & 7u) == 0) {
        const int groups = device->compute_units < batch / 64 ? device->compute_units : batch / 64;
        const int rows_per_group = rlt_div_up(rlt_div_up(batch, groups), WIDE_KT) * WIDE_KT, used = rlt_div_up(batch, rows_per_group);
        void* ws = nullptr;
        int rc = rlt_scratch(device, (size_t)used * ((size_t)out_dim * in_dim + out_dim) * sizeof(float), &ws);
        if (rc) return rc;
        WideArgs a = {d_pre, ldd, x, ldx, out_dim, in_dim, batch, rows_per_group, (float*)ws, 1};
        hipLaunchKernelGGL((wgrad_wide_kernel<10, 2>), dim3(used), dim3(THREADS), 0, device->stream, a);
        if ((rc = rlt_launch_status(device))) return rc;
        const int mn = out_dim * in_dim;
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(rlt_div_up(mn + out_dim, 64)), dim3(256), 0, device->stream, dW, dbias, (const float*)ws, mn, out_dim, used);
        return rlt_launch_status(device);
    }
    int splits, kps;
    wgrad_split(device, batch, in_dim, out_dim, splits, kps);
    p.k_per_split = kps; p.splits = splits;
    if (splits > 1) {
        const size_t floats = (size_t)splits * ((size_t)out_dim * in_dim + out_dim);
        if (static_scratch) {
            if (floats * sizeof(float) > (size_t)RLT_STATIC_SCRATCH_BYTES) return RLT_E_WORKSPACE_TOO_SMALL;
            const int index = device->hip_device;
            if (index < 0 || index >= MAX_HIP_DEVICES || !scratch_address[index]) return RLT_E_NOT_INITIALISED;
            p.ws = scratch_address[index];        // every partial the reduction reads is written by this call's contraction first: nothing to clear
        } else {
            void* ws = nullptr;
            int rc = rlt_scratch(device, floats * sizeof(float), &ws);
            if (rc) return rc;
            p.ws = (float*)ws;
        }
    }
    int rc = launch<2>(device, p, splits);
    if (rc) return rc;
    if (splits > 1) {
        int mn = out_dim * in_dim;
        int blocks = rlt_div_up(mn + out_dim, 64);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(blocks), dim3(256), 0, device->stream, dW, dbias, p.ws, mn, out_dim, splits);
        return rlt_launch_status(device);
    }
    return 0;
}

int rlt_dpre(rlt_rocm_device* device, const float* src, int lds, float* dst, int ldd, const float* pre, int rows, int cols, int act, int from_output) {
    if (act == RLT_ACT_IDENTITY && src == dst) return 0;
    size_t total = (size_t)rows * cols;
    int blocks = (int)((total + 255) / 256); if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(dpre_kernel, dim3(blocks), dim3(256), 0, device->stream, src, lds, dst, ldd, pre, rows, cols, act, from_output);
    return rlt_launch_status(device);
}

// backward(dense) for callers that cannot allocate: the same launches as rlt_rocm_dense_backward (act'(pre) * d_output in place, then the
// split-batch contraction and its fixed-order reduction), with the partial sums in the library's fixed device array.
extern "C" int rlt_rocm_dense_backward_static(rlt_rocm_device* device, const rlt_dense_layer* L, const float* x, int ldx, float* d_output, int ldd, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(L && L->weights && L->biases && L->in_dim > 0 && L->out_dim > 0 && L->activation >= RLT_ACT_IDENTITY && L->activation <= RLT_ACT_SIGMOID);
    RLT_REQUIRE(L->pre_activations && L->d_weights && L->d_biases && x && d_output && batch > 0 && ldd >= L->out_dim && ldx >= L->in_dim);
    {   // refuse before anything is launched
        int splits, kps;
        wgrad_split(device, batch, L->in_dim, L->out_dim, splits, kps);
        if (splits > 1 && (size_t)splits * ((size_t)L->out_dim * L->in_dim + L->out_dim) * sizeof(float) > (size_t)RLT_STATIC_SCRATCH_BYTES) return RLT_E_WORKSPACE_TOO_SMALL;
    }
    int rc = rlt_dpre(device, d_output, ldd, d_output, ldd, L->pre_activations, batch, L->out_dim, L->activation, 0);
    if (rc) return rc;
    return rlt_gemm_wgrad(device, d_output, ldd, x, ldx, L->d_weights, L->d_biases, batch, L->in_dim, L->out_dim, true);
}
