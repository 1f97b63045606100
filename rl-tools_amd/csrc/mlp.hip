// dense layer and MLP entry points of the C ABI, built on the contraction kernels of gemm.hip
// (reference: nn/layers/dense/operations_cpu_blas.h:36-228, nn_models/mlp/operations_generic.h:77-204).
#include "common.h"
#include <cstdlib>
#include "gemm.h"
#include "mlp_fused.h"
#include "mlp_small.h"
#include "mlp_rows.h"
#include "sac_update.h"

namespace {

bool layer_ok(const rlt_dense_layer* L) {
    return L && L->weights && L->biases && L->in_dim > 0 && L->out_dim > 0 && L->activation >= 0 && L->activation <= RLT_ACT_SIGMOID;
}
int max_dim(const rlt_dense_layer* layers, int n) {
    int m = 1;
    for (int i = 0; i < n; i++) { if (layers[i].out_dim > m) m = layers[i].out_dim; if (layers[i].in_dim > m) m = layers[i].in_dim; }
    return m;
}
size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }
// below this batch the single-pass kernels (one 64-row tile per workgroup, plus the weight swizzle) do not pay against the per-layer kernels
constexpr int FUSED_MIN_BATCH = 1024;
// a few hundred rows through layers at most 256 wide: all layers in one launch (mlp_rows.hip)
bool rows_enabled() { return rlt_mlp_rows_enabled(); }
// RLT_MLP_SINGLE_PASS=0 keeps forward() / backward() on the per-layer kernels (tests compare the two paths with each other)
bool single_pass_enabled() { const char* v = std::getenv("RLT_MLP_SINGLE_PASS"); return !(v && v[0] == '0'); }
// RLT_MLP_WIDE=0 keeps forward + backward calls of a few thousand rows off the sixteen-row-tile kernel (tests and measurements compare the paths)
bool wide_enabled() { const char* v = std::getenv("RLT_MLP_WIDE"); return !(v && v[0] == '0'); }
bool chain_ok(const rlt_dense_layer* layers, int n) {
    if (!layers || n < 1) return false;
    for (int i = 0; i < n; i++) { if (!layer_ok(&layers[i])) return false; if (i > 0 && layers[i].in_dim != layers[i - 1].out_dim) return false; }
    return true;
}

__global__ __launch_bounds__(256) void zero_kernel(float* __restrict__ a, size_t na, float* __restrict__ b, size_t nb) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < na + nb; i += (size_t)gridDim.x * blockDim.x) {
        if (i < na) a[i] = 0.0f; else b[i - na] = 0.0f;
    }
}
// up to 16 separate runs of floats cleared by one launch (a network whose gradient tensors are allocations of their own, as the reference's containers are)
constexpr int ZERO_RUNS = 16;
struct ZeroRuns { float* begin[ZERO_RUNS]; size_t prefix[ZERO_RUNS + 1]; int n; };
__global__ __launch_bounds__(256) void zero_runs_kernel(ZeroRuns z) {
    const size_t total = z.prefix[z.n];
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        int r = 0;
#pragma unroll
        for (int k = 1; k < ZERO_RUNS; k++) r += (k < z.n && i >= z.prefix[k]) ? 1 : 0;
        z.begin[r][i - z.prefix[r]] = 0.0f;
    }
}
// d = (y - target) * scale  (nn/loss_functions/mse/operations_generic.h:41-56 with scale = 2/(rows*cols)*w)
__global__ __launch_bounds__(256) void mse_d_kernel(const float* __restrict__ y, int ldy, const float* __restrict__ t, int ldt, float* __restrict__ d, int ldd,
                                                    int rows, int cols, float scale) {
    const size_t total = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i / cols, c = i % cols;
        d[r * ldd + c] = (y[r * ldy + c] - t[r * ldt + c]) * scale;
    }
}

}  // namespace

// zeroes a list of tensors: tensors laid out back to back (the flat arena [dW0 | db0 | dW1 | db1 | ...]) form one run, tensors that are allocations of their own a run
// each; up to 16 runs per launch
int rlt_zero_tensors(rlt_rocm_device* device, float* const* begins, const size_t* counts, int n) {
    ZeroRuns z = {};
    auto flush = [&]() -> int {
        if (z.n == 0) return 0;
        const size_t total = z.prefix[z.n];
        int blocks = (int)((total + 255) / 256); if (blocks > 1024) blocks = 1024;
        if (z.n == 1) hipLaunchKernelGGL(zero_kernel, dim3(blocks), dim3(256), 0, device->stream, z.begin[0], total, z.begin[0], (size_t)0);
        else hipLaunchKernelGGL(zero_runs_kernel, dim3(blocks), dim3(256), 0, device->stream, z);
        z = ZeroRuns{};
        return rlt_launch_status(device);
    };
    for (int i = 0; i < n; i++) {
        if (!begins[i]) return RLT_E_INVALID_ARGUMENT;
        if (counts[i] == 0) continue;
        if (z.n > 0 && z.begin[z.n - 1] + (z.prefix[z.n] - z.prefix[z.n - 1]) == begins[i]) { z.prefix[z.n] += counts[i]; continue; }      // continues the last run
        if (z.n == ZERO_RUNS) { const int rc = flush(); if (rc) return rc; }
        z.begin[z.n] = begins[i]; z.prefix[z.n + 1] = z.prefix[z.n] + counts[i]; z.n++;
    }
    return flush();
}

extern "C" {

int rlt_rocm_dense_evaluate(rlt_rocm_device* device, const rlt_dense_layer* L, const float* x, int ldx, float* y, int ldy, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_ok(L) && x && y && batch > 0 && ldx >= L->in_dim && ldy >= L->out_dim);
    return rlt_gemm_forward(device, x, ldx, L->weights, L->biases, L->activation, nullptr, nullptr, y, ldy, batch, L->in_dim, L->out_dim);
}
int rlt_rocm_dense_forward(rlt_rocm_device* device, const rlt_dense_layer* L, const float* x, int ldx, float* y, int ldy, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_ok(L) && L->pre_activations && x && batch > 0 && ldx >= L->in_dim && (!y || ldy >= L->out_dim));
    return rlt_gemm_forward(device, x, ldx, L->weights, L->biases, L->activation, L->pre_activations, L->output, y, ldy, batch, L->in_dim, L->out_dim);
}
int rlt_rocm_dense_backward_input(rlt_rocm_device* device, const rlt_dense_layer* L, float* d_output, int ldd, float* d_input, int ldi, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_ok(L) && L->pre_activations && d_output && d_input && batch > 0 && ldd >= L->out_dim && ldi >= L->in_dim);
    int rc = rlt_dpre(device, d_output, ldd, d_output, ldd, L->pre_activations, batch, L->out_dim, L->activation, 0);
    if (rc) return rc;
    return rlt_gemm_backward_input(device, d_output, ldd, L->weights, d_input, ldi, nullptr, 0, 0, batch, L->in_dim, L->out_dim);
}
int rlt_rocm_dense_backward(rlt_rocm_device* device, const rlt_dense_layer* L, const float* x, int ldx, float* d_output, int ldd, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_ok(L) && L->pre_activations && L->d_weights && L->d_biases && x && d_output && batch > 0 && ldd >= L->out_dim && ldx >= L->in_dim);
    int rc = rlt_dpre(device, d_output, ldd, d_output, ldd, L->pre_activations, batch, L->out_dim, L->activation, 0);
    if (rc) return rc;
    return rlt_gemm_wgrad(device, d_output, ldd, x, ldx, L->d_weights, L->d_biases, batch, L->in_dim, L->out_dim);
}
int rlt_rocm_dense_backward_full(rlt_rocm_device* device, const rlt_dense_layer* L, const float* x, int ldx, float* d_output, int ldd,
                                 float* d_input, int ldi, int batch) {
    int rc = rlt_rocm_dense_backward(device, L, x, ldx, d_output, ldd, batch);
    if (rc) return rc;
    RLT_REQUIRE(d_input && ldi >= L->in_dim);
    return rlt_gemm_backward_input(device, d_output, ldd, L->weights, d_input, ldi, nullptr, 0, 0, batch, L->in_dim, L->out_dim);
}

size_t rlt_rocm_mlp_workspace_bytes(const rlt_dense_layer* layers, int n_layers, int batch) {
    if (!layers || n_layers < 1 || batch < 1) return 0;
    size_t per_row = 0;
    for (int i = 0; i < n_layers; i++) per_row += 2 * (size_t)layers[i].out_dim;   // private pre/out of forward_backward
    per_row += 3 * (size_t)max_dim(layers, n_layers);                                // tick, tock, upstream gradient copy
    const size_t per_layer = align_up(per_row * (size_t)batch * sizeof(float)) + 4 * 256;
    const size_t fused = rlt_mlp3_fused_workspace_bytes(layers, n_layers, batch);
    return per_layer > fused ? per_layer : fused;
}

int rlt_rocm_mlp_evaluate(rlt_rocm_device* device, const rlt_dense_layer* layers, int n, const float* x, int ldx, float* y, int ldy, int batch,
                          void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(chain_ok(layers, n) && x && y && batch > 0 && ldx >= layers[0].in_dim && ldy >= layers[n - 1].out_dim);
    const size_t buf = align_up((size_t)batch * max_dim(layers, n) * sizeof(float));
    RLT_REQUIRE(n == 1 || (workspace && workspace_bytes >= 2 * buf));
    if (n == 3 && batch <= RLT_MLP_WIDE_MAX_BATCH && layers[0].out_dim > 64 && single_pass_enabled() && wide_enabled()) {      // as forward(): the same kernel, the same bits
        const int rc = rlt_mlp_wide_forward(device, layers, n, x, ldx, y, ldy, batch, false);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    if (n > 1 && batch <= RLT_MLP_ROWS_MAX_BATCH && rows_enabled()) {
        const int rc = rlt_mlp_rows_forward(device, layers, n, x, ldx, y, ldy, batch, false);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    float* tick = (float*)workspace; float* tock = (float*)((char*)workspace + buf);
    const float* in = x; int ldin = ldx;
    for (int l = 0; l < n; l++) {
        float* out = (l == n - 1) ? y : ((l % 2 == 0) ? tick : tock);
        int ldo = (l == n - 1) ? ldy : layers[l].out_dim;
        int rc = rlt_gemm_forward(device, in, ldin, layers[l].weights, layers[l].biases, layers[l].activation, nullptr, nullptr, out, ldo, batch, layers[l].in_dim, layers[l].out_dim);
        if (rc) return rc;
        in = out; ldin = ldo;
    }
    return 0;
}

int rlt_rocm_mlp_forward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n, const float* x, int ldx, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(chain_ok(layers, n) && x && batch > 0 && ldx >= layers[0].in_dim);
    for (int l = 0; l < n; l++) RLT_REQUIRE(layers[l].pre_activations && layers[l].output);
    if (n == 3 && batch <= RLT_MLP_WIDE_MAX_BATCH && layers[0].out_dim > 64 && single_pass_enabled() && wide_enabled()) {
        // hidden widths beyond 64 over a few thousand rows at most: sixteen-row tiles with the second layer's weights read from a copy in consumption order
        // (narrower networks' weights are few enough for the few-rows kernel below to read them as they lie)
        const int rc = rlt_mlp_wide_forward(device, layers, n, x, ldx, nullptr, 0, batch, true);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    if (n > 1 && batch <= RLT_MLP_ROWS_MAX_BATCH && batch < FUSED_MIN_BATCH && rows_enabled()) {
        const int rc = rlt_mlp_rows_forward(device, layers, n, x, ldx, nullptr, 0, batch, true);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    if (batch >= FUSED_MIN_BATCH && single_pass_enabled()) {       // in -> 256 -> 256 -> out: one pass that keeps the hidden activations on chip on their way to the next layer
        const int rc = rlt_mlp3_fused_forward(device, layers, n, x, ldx, batch);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    const float* in = x; int ldin = ldx;
    for (int l = 0; l < n; l++) {
        int rc = rlt_gemm_forward(device, in, ldin, layers[l].weights, layers[l].biases, layers[l].activation, layers[l].pre_activations, layers[l].output,
                                  nullptr, 0, batch, layers[l].in_dim, layers[l].out_dim);
        if (rc) return rc;
        in = layers[l].output; ldin = layers[l].out_dim;
    }
    return 0;
}

// Shared by mlp_backward and mlp_forward_backward. d_pre_last: [batch x out] holding the LAST layer's d_pre already.
// With from_output set, a layer's `pre_activations` may be NULL and the activation derivative is taken from its `output`.
static int mlp_backward_from_dpre(rlt_rocm_device* device, const rlt_dense_layer* layers, int n, const float* x, int ldx,
                                  float* d_pre_last, int ldd, float* d_input, int ldi, int batch, int want_w, float* tick, float* tock,
                                  bool from_output = false) {
    float* d_pre = d_pre_last; int ld_pre = ldd;
    for (int l = n - 1; l >= 0; l--) {
        const rlt_dense_layer& L = layers[l];
        const float* in = (l == 0) ? x : layers[l - 1].output; int ldin = (l == 0) ? ldx : layers[l - 1].out_dim;
        if (want_w) {
            int rc = rlt_gemm_wgrad(device, d_pre, ld_pre, in, ldin, L.d_weights, L.d_biases, batch, L.in_dim, L.out_dim);
            if (rc) return rc;
        }
        if (l > 0) {
            // d_input of this layer becomes d_pre of the layer below: the activation derivative is applied in the epilogue
            float* d_in = ((n - 1 - l) % 2 == 0) ? tick : tock;
            const bool fo = from_output && layers[l - 1].pre_activations == nullptr;
            int rc = rlt_gemm_backward_input(device, d_pre, ld_pre, L.weights, d_in, L.in_dim, fo ? layers[l - 1].output : layers[l - 1].pre_activations,
                                             layers[l - 1].activation, fo ? 1 : 0, batch, L.in_dim, L.out_dim);
            if (rc) return rc;
            d_pre = d_in; ld_pre = L.in_dim;
        } else if (d_input) {
            int rc = rlt_gemm_backward_input(device, d_pre, ld_pre, L.weights, d_input, ldi, nullptr, 0, 0, batch, L.in_dim, L.out_dim);
            if (rc) return rc;
        }
    }
    return 0;
}

int rlt_rocm_mlp_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n, const float* x, int ldx, float* d_output, int ldd,
                          float* d_input, int ldi, int batch, int want_w, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(chain_ok(layers, n) && d_output && batch > 0 && ldd >= layers[n - 1].out_dim);
    RLT_REQUIRE(!want_w || (x && ldx >= layers[0].in_dim));
    RLT_REQUIRE(want_w || d_input);
    RLT_REQUIRE(!d_input || ldi >= layers[0].in_dim);
    for (int l = 0; l < n; l++) {
        RLT_REQUIRE(layers[l].pre_activations);
        if (want_w) RLT_REQUIRE(layers[l].d_weights && layers[l].d_biases && (l == n - 1 || layers[l].output));
    }
    const size_t buf = align_up((size_t)batch * max_dim(layers, n) * sizeof(float));
    RLT_REQUIRE(n == 1 || (workspace && workspace_bytes >= 2 * buf));
    float* tick = (float*)workspace; float* tock = (float*)((char*)workspace + buf);
    const rlt_dense_layer& last = layers[n - 1];
    int rc = rlt_dpre(device, d_output, ldd, d_output, ldd, last.pre_activations, batch, last.out_dim, last.activation, 0);
    if (rc) return rc;
    if (want_w && !d_input && batch <= RLT_MLP_WIDE_MAX_BATCH && single_pass_enabled() && wide_enabled()) {      // a few thousand rows at most: sixteen-row tiles
        rc = rlt_mlp_wide_backward(device, layers, n, x, ldx, d_output, ldd, batch);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    if (want_w && !d_input && batch >= FUSED_MIN_BATCH && single_pass_enabled()) {
        rc = rlt_mlp3_fused_backward(device, layers, n, x, ldx, d_output, ldd, batch, workspace, workspace_bytes);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    return mlp_backward_from_dpre(device, layers, n, x, ldx, d_output, ldd, d_input, ldi, batch, want_w, tick, tock);
}

int rlt_rocm_mlp_zero_gradient(rlt_rocm_device* device, const rlt_dense_layer* layers, int n) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layers && n >= 1 && n <= 64);
    float* begins[128]; size_t counts[128];
    for (int l = 0; l < n; l++) {
        RLT_REQUIRE(layers[l].d_weights && layers[l].d_biases && layers[l].in_dim > 0 && layers[l].out_dim > 0);
        begins[2 * l] = layers[l].d_weights; counts[2 * l] = (size_t)layers[l].in_dim * layers[l].out_dim;
        begins[2 * l + 1] = layers[l].d_biases; counts[2 * l + 1] = (size_t)layers[l].out_dim;
    }
    return rlt_zero_tensors(device, begins, counts, 2 * n);
}

}  // extern "C"
static int forward_backward_impl(rlt_rocm_device* device, const rlt_dense_layer* layers, int n, const float* x, int ldx, float* y, int ldy,
                                  const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch,
                                  void* workspace, size_t workspace_bytes, float* d_input, int ldi) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(chain_ok(layers, n) && x && batch > 0 && ldx >= layers[0].in_dim && (d_output || target));
    const int O = layers[n - 1].out_dim;
    RLT_REQUIRE((!y || ldy >= O) && (!d_output || ldd >= O) && (!target || ldt >= O) && (!d_input || ldi >= layers[0].in_dim));
    for (int l = 0; l < n; l++) RLT_REQUIRE(layers[l].d_weights && layers[l].d_biases);
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_mlp_workspace_bytes(layers, n, batch));
    if (!d_input && batch > RLT_MLP_WIDE_MAX_BATCH) {
        // one pass over the batch with on-chip activations where the network has the shape that kernel is built for
        const int rc = rlt_mlp3_fused_forward_backward(device, layers, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch, workspace, workspace_bytes);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    if (single_pass_enabled()) {
        int rc = rlt_mlp3s_forward_backward(device, layers, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch, d_input, ldi);
        if (rc != RLT_E_UNSUPPORTED) return rc;
        // a few thousand rows at most, hidden widths up to 256: sixteen-row tiles, one workgroup each (the 64-row tiles of the kernel above leave most of the chip idle there)
        if (!d_input && wide_enabled()) {
            rc = rlt_mlp_wide_forward_backward(device, layers, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch);
            if (rc != RLT_E_UNSUPPORTED) return rc;
        }
    }
    if (!d_input && batch >= FUSED_MIN_BATCH) {
        const int rc = rlt_mlp3_fused_forward_backward(device, layers, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch, workspace, workspace_bytes);
        if (rc != RLT_E_UNSUPPORTED) return rc;
    }
    // carve private activation storage out of the workspace
    rlt_dense_layer priv[16];
    RLT_REQUIRE(n <= 16);
    char* w = (char*)workspace;
    const size_t buf = align_up((size_t)batch * max_dim(layers, n) * sizeof(float));
    float* tick = (float*)w; w += buf; float* tock = (float*)w; w += buf; float* dlast = (float*)w; w += buf;
    const bool few_rows = n > 1 && batch <= RLT_MLP_ROWS_MAX_BATCH && rows_enabled();      // all layers' forward passes in one launch, which writes both buffers of a layer
    for (int l = 0; l < n; l++) {
        priv[l] = layers[l];
        // the activation derivative is recovered from the output wherever the activation allows it, so only GELU layers keep both
        priv[l].pre_activations = nullptr;
        if (few_rows || layers[l].activation == RLT_ACT_GELU) { priv[l].pre_activations = (float*)w; w += (size_t)batch * layers[l].out_dim * sizeof(float); }
        priv[l].output = (float*)w; w += (size_t)batch * layers[l].out_dim * sizeof(float);
    }
    bool forwarded = false;
    if (few_rows) {
        const int rc = rlt_mlp_rows_forward(device, priv, n, x, ldx, y, ldy, batch, true);
        if (rc && rc != RLT_E_UNSUPPORTED) return rc;
        forwarded = rc == 0;
    }
    const float* in = x; int ldin = ldx;
    for (int l = 0; l < n && !forwarded; l++) {
        int rc = rlt_gemm_forward(device, in, ldin, priv[l].weights, priv[l].biases, priv[l].activation, priv[l].pre_activations, priv[l].output,
                                  (l == n - 1) ? y : nullptr, ldy, batch, priv[l].in_dim, priv[l].out_dim);
        if (rc) return rc;
        in = priv[l].output; ldin = priv[l].out_dim;
    }
    const rlt_dense_layer& last = priv[n - 1];
    int rc;
    if (target) {
        size_t total = (size_t)batch * O; int blocks = (int)((total + 255) / 256); if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(mse_d_kernel, dim3(blocks), dim3(256), 0, device->stream, last.output, O, target, ldt, dlast, O, batch, O, mse_scale);
        if ((rc = rlt_launch_status(device))) return rc;
        const bool fo = last.pre_activations == nullptr;
        if ((rc = rlt_dpre(device, dlast, O, dlast, O, fo ? last.output : last.pre_activations, batch, O, last.activation, fo))) return rc;
    } else {
        const bool fo = last.pre_activations == nullptr;
        if ((rc = rlt_dpre(device, d_output, ldd, dlast, O, fo ? last.output : last.pre_activations, batch, O, last.activation, fo))) return rc;
    }
    return mlp_backward_from_dpre(device, priv, n, x, ldx, dlast, O, d_input, ldi, batch, 1, tick, tock, true);
}

extern "C" {
int rlt_rocm_mlp_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n, const float* x, int ldx, float* y, int ldy,
                                  const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch, void* workspace, size_t workspace_bytes) {
    return forward_backward_impl(device, layers, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch, workspace, workspace_bytes, nullptr, 0);
}
int rlt_rocm_mlp_forward_backward_input(rlt_rocm_device* device, const rlt_dense_layer* layers, int n, const float* x, int ldx, float* y, int ldy,
                                        const float* d_output, int ldd, const float* target, int ldt, float mse_scale, float* d_input, int ldi, int batch,
                                        void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(d_input);
    return forward_backward_impl(device, layers, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, batch, workspace, workspace_bytes, d_input, ldi);
}

}  // extern "C"
