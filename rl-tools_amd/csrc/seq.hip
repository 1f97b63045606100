// Sequential models of dense and GRU layers (the reference's recurrent approximators, rl/algorithms/sac/loop/core/approximators_gru.h:13-74):
// forward / backward / zero_gradient assembled from the dense and GRU entry points of this library.
// reference: nn_models/sequential/operations_generic.h:277-428.
#include "common.h"
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

int rlt_rocm_seq_zero_gradient(rlt_rocm_device* device, const rlt_seq_layer* layers, int n) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layers && n > 0);
    int rc;
    auto zero = [&](float* p, size_t count) { return p ? rlt_rocm_fill_f32(device, p, 1, (int)count, (int)count, 0.0f) : RLT_E_INVALID_ARGUMENT; };
    for (int l = 0; l < n; l++) {
        if (layers[l].kind == 0) {
            const rlt_dense_layer& D = layers[l].dense;
            if ((rc = zero(D.d_weights, (size_t)D.in_dim * D.out_dim)) || (rc = zero(D.d_biases, D.out_dim))) return rc;
        } else {
            const rlt_gru_layer& G = layers[l].gru;
            const size_t H = G.hidden_dim, I = G.input_dim;
            if ((rc = zero(G.d_weights_input, 3 * H * I)) || (rc = zero(G.d_biases_input, 3 * H)) || (rc = zero(G.d_weights_hidden, 3 * H * H)) || (rc = zero(G.d_biases_hidden, 3 * H))) return rc;
        }
    }
    return 0;
}

}  // extern "C"
