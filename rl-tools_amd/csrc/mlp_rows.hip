// The forward pass of a whole MLP over a batch of a few hundred rows in one launch
// (reference: nn_models/mlp/operations_generic.h:77-130 evaluate / forward, one sgemm per layer in nn/layers/dense/operations_cpu_blas.h:36-80).
//
// At such a batch a layer is a handful of tiles: per-layer launches leave most of the chip idle and pay a launch, a cold start and a trip through
// memory for the activations per layer (measured at batch 256, widths 256: 6.5 + 10.6 + 10.1 us for the three layers of a critic). Here a workgroup of
// sixteen wavefronts takes 16 rows through all layers: the activations stay in LDS, wavefront w owns the output columns 16 w ... 16 w + 15 of every layer
// and reads that tile's rows of W from memory straight into the B operands of v_mfma_f32_16x16x4_f32, all of them at once and a layer ahead: the next
// layer's weights are requested before this layer's results are written, so their way from memory overlaps the epilogue and the barrier.
// Operand lane layout of the instruction: lane l = 16 g + c holds A[row c][k g] and B[k g][col c]; the four k of one instruction may be any four as long as
// both operands agree, so lane group g takes k = 16 j + 4 g + i for the i-th of four consecutive instructions: one 16-byte read per operand per four
// instructions. Accumulator element v of lane l is C[row 4 g + v][col c].
// Two networks of one shape on the same rows (a pair of critics) share a launch: blockIdx.y selects the network.
#include "mlp_rows.h"
#include <cstdlib>

typedef float rows_floatx4 __attribute__((ext_vector_type(4)));

namespace {
constexpr int ROWS = 16, MAX_WIDTH = 256, MAX_LAYERS = 8, STRIDE = MAX_WIDTH + 4, WAVES = MAX_WIDTH / 16;
struct RowsLayer { const float* W; const float* b; float* pre; float* out; int in_dim, out_dim, act, vec; };
struct RowsArgs { RowsLayer L[MAX_LAYERS]; int n; const float* x; int ldx; float* y; int ldy; int batch; };
struct RowsPair { RowsArgs net[2]; };      // blockIdx.y selects the network: two networks of one shape on one batch (SAC's and TD3's pairs of critics) share a launch

// what a lane needs of a layer: its column's row of W as B operands (lane group g: k = 16 j + 4 g ... + 3 of every 16), zero beyond the layer's shape, and its bias
struct RowsWeights { float4 b[MAX_WIDTH / 16]; float bias; };
__device__ __forceinline__ void load_weights(const RowsLayer& L, int n, int g, RowsWeights& w) {
    const int K = L.in_dim, steps = (K + 15) >> 4;
    const bool n_ok = n < L.out_dim;
    const float* w_row = L.W + (size_t)(n_ok ? n : 0) * K;
    if (L.vec) {
#pragma unroll
        for (int j = 0; j < MAX_WIDTH / 16; j++) {
            w.b[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (j < steps && n_ok && 16 * j + 4 * g < K) w.b[j] = *reinterpret_cast<const float4*>(w_row + 16 * j + 4 * g);      // K is a multiple of 4 here
        }
    } else {
#pragma unroll
        for (int j = 0; j < MAX_WIDTH / 16; j++) {
            w.b[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (j < steps && n_ok) {
                const int k = 16 * j + 4 * g;
                if (k + 0 < K) w.b[j].x = w_row[k + 0];
                if (k + 1 < K) w.b[j].y = w_row[k + 1];
                if (k + 2 < K) w.b[j].z = w_row[k + 2];
                if (k + 3 < K) w.b[j].w = w_row[k + 3];
            }
        }
    }
    w.bias = n_ok ? L.b[n] : 0.0f;
}

__global__ __launch_bounds__(WAVES * 64) void mlp_rows_kernel(RowsPair P) {
    const RowsArgs& A = P.net[blockIdx.y];
    __shared__ __attribute__((aligned(16))) float act[2][ROWS * STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, c = lane & 15;
    const int row0 = blockIdx.x * ROWS;
    const int n = wave * 16 + c;      // this lane's output column in every layer: wavefront w owns columns 16 w ... 16 w + 15
    RowsWeights w;
    load_weights(A.L[0], n, g, w);      // requested before the input rows: the weights do not depend on them
    {   // the input rows, zero beyond the batch and beyond the input width (up to the next multiple of 16, which the first layer's reduction runs to)
        const int K = A.L[0].in_dim, K16 = (K + 15) & ~15;
        for (int e = tid; e < ROWS * K16; e += WAVES * 64) {
            const int r = e / K16, k = e % K16;
            act[0][r * STRIDE + k] = (row0 + r < A.batch && k < K) ? A.x[(size_t)(row0 + r) * A.ldx + k] : 0.0f;
        }
    }
    __syncthreads();
    for (int l = 0; l < A.n; l++) {
        const RowsLayer& L = A.L[l];
        const float* in = act[l & 1];
        float* next = act[(l + 1) & 1];
        const int N = L.out_dim, steps = (L.in_dim + 15) >> 4, tiles = (N + 15) >> 4;
        const bool last = l + 1 == A.n;
        rows_floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        if (wave < tiles) {      // the same for a whole wavefront
            const float* a_row = in + c * STRIDE + 4 * g;
#pragma unroll
            for (int j = 0; j < MAX_WIDTH / 16; j++) {
                if (j < steps) {
                    const float4 a = *reinterpret_cast<const float4*>(a_row + 16 * j);
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, w.b[j].x, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, w.b[j].y, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, w.b[j].z, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, w.b[j].w, acc, 0, 0, 0);
                }
            }
        }
        const float bias = w.bias;
        if (!last) load_weights(A.L[l + 1], n, g, w);      // on their way while this layer's results are written and the workgroup meets
        if (wave < tiles) {
            const bool n_ok = n < N;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int r = 4 * g + v, row = row0 + r;
                const float pre = acc[v] + bias;
                const float o = rlt_act(pre, L.act);
                if (!last) next[r * STRIDE + n] = n_ok ? o : 0.0f;      // columns up to the next multiple of 16 are part of the next layer's reduction
                if (n_ok && row < A.batch) {
                    if (L.pre) L.pre[(size_t)row * N + n] = pre;
                    if (L.out) L.out[(size_t)row * N + n] = o;
                    if (last && A.y) A.y[(size_t)row * A.ldy + n] = o;
                }
            }
        }
        __syncthreads();
    }
}
}  // namespace

bool rlt_mlp_rows_enabled() { const char* v = std::getenv("RLT_MLP_ROWS"); return !(v && v[0] == '0'); }

static int describe_rows(const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy, int batch, bool keep, RowsArgs& a) {
    if (n_layers < 1 || n_layers > MAX_LAYERS || batch < 1 || batch > RLT_MLP_ROWS_MAX_BATCH) return RLT_E_UNSUPPORTED;
    a = RowsArgs{};
    for (int l = 0; l < n_layers; l++) {
        const rlt_dense_layer& L = layers[l];
        if (L.in_dim > MAX_WIDTH || L.out_dim > MAX_WIDTH) return RLT_E_UNSUPPORTED;
        const bool vec = L.in_dim % 4 == 0 && (reinterpret_cast<uintptr_t>(L.weights) & 15u) == 0;
        a.L[l] = RowsLayer{L.weights, L.biases, keep ? L.pre_activations : nullptr, keep ? L.output : nullptr, L.in_dim, L.out_dim, L.activation, vec ? 1 : 0};
    }
    a.n = n_layers; a.x = x; a.ldx = ldx; a.y = y; a.ldy = ldy; a.batch = batch;
    return 0;
}

int rlt_mlp_rows_forward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy, int batch, bool keep) {
    RowsPair p = {};
    const int rc = describe_rows(layers, n_layers, x, ldx, y, ldy, batch, keep, p.net[0]);
    if (rc) return rc;
    hipLaunchKernelGGL(mlp_rows_kernel, dim3(rlt_div_up(batch, ROWS), 1), dim3(WAVES * 64), 0, device->stream, p);
    return rlt_launch_status(device);
}

int rlt_mlp_rows_forward_pair(rlt_rocm_device* device, const rlt_dense_layer* first, const rlt_dense_layer* second, int n_layers, const float* x, int ldx,
                              float* y_first, float* y_second, int ldy, int batch, bool keep) {
    RowsPair p = {};
    int rc = describe_rows(first, n_layers, x, ldx, y_first, ldy, batch, keep, p.net[0]);
    if (rc) return rc;
    if ((rc = describe_rows(second, n_layers, x, ldx, y_second, ldy, batch, keep, p.net[1]))) return rc;
    hipLaunchKernelGGL(mlp_rows_kernel, dim3(rlt_div_up(batch, ROWS), 2), dim3(WAVES * 64), 0, device->stream, p);
    return rlt_launch_status(device);
}

int rlt_mlp_forward_pair(rlt_rocm_device* device, const rlt_dense_layer* first, const rlt_dense_layer* second, int n_layers, const float* x, int ldx, float* y_first,
                         float* y_second, int ldy, int batch, bool keep, void* ws, size_t ws_bytes) {
    if (n_layers > 1 && batch < 1024 && rlt_mlp_rows_enabled()) {      // from 1,024 rows forward() has a single-pass kernel of its own
        const int rc = rlt_mlp_rows_forward_pair(device, first, second, n_layers, x, ldx, y_first, y_second, ldy, batch, keep);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    const rlt_dense_layer* nets[2] = {first, second};
    float* ys[2] = {y_first, y_second};
    for (int k = 0; k < 2; k++) {
        const int rc = keep ? rlt_rocm_mlp_forward(device, nets[k], n_layers, x, ldx, batch) : rlt_rocm_mlp_evaluate(device, nets[k], n_layers, x, ldx, ys[k], ldy, batch, ws, ws_bytes);
        if (rc) return rc;
    }
    return 0;
}
