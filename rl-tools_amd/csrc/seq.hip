// Sequential models of dense and GRU layers (the reference's recurrent approximators, rl/algorithms/sac/loop/core/approximators_gru.h:13-74):
// forward / backward / zero_gradient assembled from the dense and GRU entry points of this library.
// reference: nn_models/sequential/operations_generic.h:277-428.
#include "common.h"
#include "gemm.h"
#include "mlp_rows.h"
#include <algorithm>

namespace {

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
inline int layer_in(const rlt_seq_layer& L) { return L.kind ? L.gru.input_dim : L.dense.in_dim; }
inline int layer_out(const rlt_seq_layer& L) { return L.kind ? L.gru.hidden_dim : L.dense.out_dim; }
inline const float* layer_output(const rlt_seq_layer& L) { return L.kind ? L.gru.output : L.dense.output; }

bool layers_ok(const rlt_seq_layer* layers, int n) {
    if (!layers || n <= 0) return false;
    for (int l = 0; l < n; l++) {
        if (layers[l].kind != 0 && layers[l].kind != 1) return false;
        if (layer_in(layers[l]) <= 0 || layer_out(layers[l]) <= 0) return false;
        if (l && layer_in(layers[l]) != layer_out(layers[l - 1])) return false;
        if (!layer_output(layers[l])) return false;
        if (layers[l].kind == 0 && !layers[l].dense.pre_activations) return false;
    }
    return true;
}

// the two gradient buffers between the layers (the reference's tick / tock), then the GRU layers' workspace
struct Workspace { float* tick_tock[2]; void* gru; size_t gru_bytes; };
size_t max_width(const rlt_seq_layer* layers, int n) { size_t m = 1; for (int l = 1; l < n; l++) m = std::max(m, (size_t)layer_in(layers[l])); return m; }
size_t gru_bytes(const rlt_seq_layer* layers, int n, int steps, int batch) {
    size_t m = 0;
    for (int l = 0; l < n; l++) if (layers[l].kind) m = std::max(m, rlt_rocm_gru_workspace_bytes(&layers[l].gru, steps, batch));
    return m;
}
bool carve(const rlt_seq_layer* layers, int n, int steps, int batch, void* workspace, size_t bytes, Workspace* W) {
    const size_t need = rlt_rocm_seq_workspace_bytes(layers, n, steps, batch);
    if (need && (!workspace || bytes < need)) return false;
    char* w = reinterpret_cast<char*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    const size_t one = align256((size_t)steps * batch * max_width(layers, n) * sizeof(float));
    W->tick_tock[0] = (float*)w; W->tick_tock[1] = (float*)(w + one);
    W->gru = w + 2 * one; W->gru_bytes = gru_bytes(layers, n, steps, batch);
    return true;
}

// ---- rollout state of the GRU layers (nn/layers/gru/layer.h State) ---------------------------------------------------------------
__global__ __launch_bounds__(256) void seq_reset_state_kernel(float* __restrict__ hidden, uint32_t* __restrict__ step, const float* __restrict__ h0,
                                                              const uint8_t* __restrict__ mask, int batch, int H) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * H; i += gridDim.x * blockDim.x) {
        const int b = i / H, j = i - b * H;
        if (mask && !mask[b]) continue;
        hidden[i] = h0[j];
        if (j == 0) step[b] = 0;
    }
}
__device__ __forceinline__ float fast_tanh_gate(float x) { return rlt_fast_tanh(x); }
// One GRU step on the kept state: thread (row, unit). `post` holds W_i x + b_i of the step; the new hidden state goes to `out` (the state itself
// is advanced by the commit kernel, after every thread has read the old one).
__global__ __launch_bounds__(256) void gru_state_step_kernel(rlt_gru_layer L, const float* __restrict__ post, const float* __restrict__ hidden, const uint32_t* __restrict__ step,
                                                             int period, float* __restrict__ out, int ldo, int batch) {
    const int H = L.hidden_dim;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * H; i += gridDim.x * blockDim.x) {
        const int b = i / H, j = i - b * H;
        const bool restart = period > 0 && step[b] >= (uint32_t)period;                 // reset_truncate (nn/layers/gru/operations_generic.h:76-86)
        const float* hp = restart ? L.initial_hidden_state : hidden + (size_t)b * H;
        float ar = L.biases_hidden[j], az = L.biases_hidden[H + j], an = L.biases_hidden[2 * H + j];
        const float* wr = L.weights_hidden + (size_t)j * H; const float* wz = wr + (size_t)H * H; const float* wn = wz + (size_t)H * H;
        for (int k = 0; k < H; k++) { const float hk = hp[k]; ar += hk * wr[k]; az += hk * wz[k]; an += hk * wn[k]; }
        const float* p = post + (size_t)b * 3 * H;
        const float xr = p[j] + ar, xz = p[H + j] + az;
        const float r = L.fast_tanh ? 0.5f * fast_tanh_gate(0.5f * xr) + 0.5f : 1.0f / (1.0f + expf(-xr));
        const float z = L.fast_tanh ? 0.5f * fast_tanh_gate(0.5f * xz) + 0.5f : 1.0f / (1.0f + expf(-xz));
        const float xn = p[2 * H + j] + an * r;
        const float n = L.fast_tanh ? fast_tanh_gate(xn) : tanhf(xn);
        out[(size_t)b * ldo + j] = (1.0f - z) * n + z * hp[j];
    }
}
// the new state; a row that has run `period` steps starts again from the initial hidden state (:405-415). The step counters are read here and
// advanced by the launch after this one (gru_state_count_kernel), so that no thread reads a counter another one has already advanced.
__device__ __forceinline__ uint32_t next_step(uint32_t old, int period) { return ((period > 0 && old >= (uint32_t)period) ? 0u : old) + 1u; }
__global__ __launch_bounds__(256) void gru_state_commit_kernel(const float* __restrict__ out, int ldo, const float* __restrict__ h0, float* __restrict__ hidden,
                                                               const uint32_t* __restrict__ step, int period, int batch, int H) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * H; i += gridDim.x * blockDim.x) {
        const int b = i / H, j = i - b * H;
        const bool restart = period > 0 && next_step(step[b], period) >= (uint32_t)period;
        hidden[i] = restart ? h0[j] : out[(size_t)b * ldo + j];
    }
}
__global__ __launch_bounds__(256) void gru_state_count_kernel(uint32_t* __restrict__ step, int period, int batch) {
    for (int b = blockIdx.x * blockDim.x + threadIdx.x; b < batch; b += gridDim.x * blockDim.x) {
        const uint32_t next = next_step(step[b], period);
        step[b] = (period > 0 && next >= (uint32_t)period) ? 0u : next;
    }
}
inline int grid_for_elements(size_t n) { size_t b = (n + 255) / 256; return (int)(b > 2048 ? 2048 : (b < 1 ? 1 : b)); }

}  // namespace

extern "C" {

size_t rlt_rocm_seq_workspace_bytes(const rlt_seq_layer* layers, int n, int steps, int batch) {
    if (!layers || n <= 0 || steps <= 0 || batch <= 0) return 0;
    return 2 * align256((size_t)steps * batch * max_width(layers, n) * sizeof(float)) + gru_bytes(layers, n, steps, batch) + 256;
}

int rlt_rocm_seq_forward(rlt_rocm_device* device, const rlt_seq_layer* layers, int n, const float* x, int ldx, const uint8_t* reset, int steps, int batch,
                         void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layers_ok(layers, n) && x && steps > 0 && batch > 0 && ldx >= layer_in(layers[0]));
    Workspace W;
    RLT_REQUIRE(carve(layers, n, steps, batch, workspace, workspace_bytes, &W));
    const float* in = x; int ld = ldx, rc;
    for (int l = 0; l < n; l++) {
        const rlt_seq_layer& L = layers[l];
        if (L.kind == 0) {
            if ((rc = rlt_rocm_dense_forward(device, &L.dense, in, ld, nullptr, 0, steps * batch))) return rc;
        } else {
            RLT_REQUIRE(ld == L.gru.input_dim);
            if ((rc = rlt_rocm_gru_forward(device, &L.gru, in, reset, steps, batch, W.gru, W.gru_bytes))) return rc;
        }
        in = layer_output(L); ld = layer_out(L);
    }
    return 0;
}

int rlt_rocm_seq_backward(rlt_rocm_device* device, const rlt_seq_layer* layers, int n, const float* x, int ldx, float* d_output, float* d_input, const uint8_t* reset,
                          int steps, int batch, int want_w, int reset_in_backward_input, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layers_ok(layers, n) && d_output && steps > 0 && batch > 0 && (!want_w || (x && ldx >= layer_in(layers[0]))));
    Workspace W;
    RLT_REQUIRE(carve(layers, n, steps, batch, workspace, workspace_bytes, &W));
    const int rows = steps * batch;
    // backward and backward_full hand the mode to every layer; backward_input hands it on only when the model has a single layer
    const uint8_t* reset_here = (want_w || reset_in_backward_input || n == 1) ? reset : nullptr;
    float* d_cur = d_output; int which = 0, rc;
    for (int l = n - 1; l >= 0; l--) {
        const rlt_seq_layer& L = layers[l];
        const float* in = l ? layer_output(layers[l - 1]) : x;
        const int ld_in = l ? layer_out(layers[l - 1]) : ldx;
        float* d_in = d_input;
        if (l > 0) { d_in = W.tick_tock[which]; which ^= 1; }
        if (L.kind == 0) {
            if (want_w && d_in) rc = rlt_rocm_dense_backward_full(device, &L.dense, in, ld_in, d_cur, L.dense.out_dim, d_in, L.dense.in_dim, rows);
            else if (want_w) rc = rlt_rocm_dense_backward(device, &L.dense, in, ld_in, d_cur, L.dense.out_dim, rows);
            else rc = d_in ? rlt_rocm_dense_backward_input(device, &L.dense, d_cur, L.dense.out_dim, d_in, L.dense.in_dim, rows) : 0;
        } else {
            RLT_REQUIRE(!want_w || ld_in == L.gru.input_dim);
            rc = rlt_rocm_gru_backward(device, &L.gru, in, d_cur, d_in, reset_here, steps, batch, want_w, W.gru, W.gru_bytes);
        }
        if (rc) return rc;
        d_cur = d_in;
    }
    return 0;
}

int rlt_rocm_seq_reset_state(rlt_rocm_device* device, const rlt_seq_layer* layers, int n, const rlt_seq_state* state, const uint8_t* mask, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layers && n > 0 && n <= RLT_SEQ_MAX_LAYERS && state && batch > 0);
    for (int l = 0; l < n; l++) {
        if (!layers[l].kind) continue;
        const rlt_gru_layer& G = layers[l].gru;
        RLT_REQUIRE(state->hidden[l] && state->step[l] && G.initial_hidden_state && G.hidden_dim > 0);
        hipLaunchKernelGGL(seq_reset_state_kernel, dim3(grid_for_elements((size_t)batch * G.hidden_dim)), dim3(256), 0, device->stream, state->hidden[l], state->step[l],
                           (const float*)G.initial_hidden_state, mask, batch, G.hidden_dim);
        int rc = rlt_launch_status(device);
        if (rc) return rc;
    }
    return 0;
}

// two buffers of batch x (widest layer output) between the layers, one of batch x 3H for the GRU input projections
size_t rlt_rocm_seq_evaluate_step_workspace_bytes(const rlt_seq_layer* layers, int n, int batch) {
    if (!layers || n <= 0 || batch <= 0) return 0;
    size_t width = 1, h3 = 1;
    for (int l = 0; l < n; l++) { width = std::max(width, (size_t)layer_out(layers[l])); if (layers[l].kind) h3 = std::max(h3, (size_t)3 * layers[l].gru.hidden_dim); }
    return 2 * align256((size_t)batch * width * sizeof(float)) + align256((size_t)batch * h3 * sizeof(float)) + 256;
}

int rlt_rocm_seq_evaluate_step(rlt_rocm_device* device, const rlt_seq_layer* layers, int n, const float* x, int ldx, const rlt_seq_state* state, int period,
                               float* y, int ldy, int batch, void* workspace, size_t workspace_bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layers && n > 0 && n <= RLT_SEQ_MAX_LAYERS && x && state && y && batch > 0 && period >= 0);
    RLT_REQUIRE(ldx >= layer_in(layers[0]) && ldy >= layer_out(layers[n - 1]));
    for (int l = 1; l < n; l++) RLT_REQUIRE(layer_in(layers[l]) == layer_out(layers[l - 1]));
    RLT_REQUIRE(workspace && workspace_bytes >= rlt_rocm_seq_evaluate_step_workspace_bytes(layers, n, batch));
    bool dense_only = true;
    for (int l = 0; l < n; l++) dense_only = dense_only && layers[l].kind == 0;
    if (dense_only && n > 1 && batch <= RLT_MLP_ROWS_MAX_BATCH && rlt_mlp_rows_enabled()) {      // a policy without recurrent layers: all layers in one launch
        rlt_dense_layer dense[RLT_SEQ_MAX_LAYERS];
        for (int l = 0; l < n; l++) dense[l] = layers[l].dense;
        const int fused = rlt_mlp_rows_forward(device, dense, n, x, ldx, y, ldy, batch, false);
        if (fused != RLT_E_UNSUPPORTED) return fused;
    }
    size_t width = 1;
    for (int l = 0; l < n; l++) width = std::max(width, (size_t)layer_out(layers[l]));
    char* w = reinterpret_cast<char*>(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    const size_t one = align256((size_t)batch * width * sizeof(float));
    float* buffers[2] = {(float*)w, (float*)(w + one)};
    float* post = (float*)(w + 2 * one);
    const float* in = x; int ld = ldx, which = 0, rc;
    for (int l = 0; l < n; l++) {
        const rlt_seq_layer& L = layers[l];
        const int out_dim = layer_out(L);
        float* out = y; int ldo = ldy;
        if (l + 1 < n) { out = buffers[which]; ldo = out_dim; which ^= 1; }
        if (L.kind == 0) {
            if ((rc = rlt_rocm_dense_evaluate(device, &L.dense, in, ld, out, ldo, batch))) return rc;
        } else {
            const rlt_gru_layer& G = L.gru;
            RLT_REQUIRE(state->hidden[l] && state->step[l] && G.weights_input && G.biases_input && G.weights_hidden && G.biases_hidden && G.initial_hidden_state);
            const int H = G.hidden_dim;
            if ((rc = rlt_gemm_forward(device, in, ld, G.weights_input, G.biases_input, RLT_ACT_IDENTITY, nullptr, nullptr, post, 3 * H, batch, G.input_dim, 3 * H))) return rc;
            const dim3 grid(grid_for_elements((size_t)batch * H));
            hipLaunchKernelGGL(gru_state_step_kernel, grid, dim3(256), 0, device->stream, G, (const float*)post, (const float*)state->hidden[l], (const uint32_t*)state->step[l],
                               period, out, ldo, batch);
            if ((rc = rlt_launch_status(device))) return rc;
            hipLaunchKernelGGL(gru_state_commit_kernel, grid, dim3(256), 0, device->stream, (const float*)out, ldo, (const float*)G.initial_hidden_state, state->hidden[l],
                               (const uint32_t*)state->step[l], period, batch, H);
            if ((rc = rlt_launch_status(device))) return rc;
            hipLaunchKernelGGL(gru_state_count_kernel, dim3(grid_for_elements(batch)), dim3(256), 0, device->stream, state->step[l], period, batch);
            if ((rc = rlt_launch_status(device))) return rc;
        }
        in = out; ld = ldo;
    }
    return 0;
}

int rlt_rocm_seq_zero_gradient(rlt_rocm_device* device, const rlt_seq_layer* layers, int n) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layers && n > 0 && n <= RLT_SEQ_MAX_LAYERS);
    float* begins[4 * RLT_SEQ_MAX_LAYERS]; size_t counts[4 * RLT_SEQ_MAX_LAYERS];
    int m = 0;
    auto add = [&](float* p, size_t count) { begins[m] = p; counts[m++] = count; };
    for (int l = 0; l < n; l++) {
        if (layers[l].kind == 0) {
            const rlt_dense_layer& D = layers[l].dense;
            add(D.d_weights, (size_t)D.in_dim * D.out_dim); add(D.d_biases, D.out_dim);
        } else {
            const rlt_gru_layer& G = layers[l].gru;
            const size_t H = G.hidden_dim, I = G.input_dim;
            add(G.d_weights_input, 3 * H * I); add(G.d_biases_input, 3 * H); add(G.d_weights_hidden, 3 * H * H); add(G.d_biases_hidden, 3 * H);
        }
    }
    return rlt_zero_tensors(device, begins, counts, m);      // all of the network's gradient tensors in one launch (two beyond sixteen separate allocations)
}

}  // extern "C"
