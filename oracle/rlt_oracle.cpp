// CPU restatement of the reference algorithms (test infrastructure only, see rlt_oracle.h).
// Reference paths are relative to /root/reference/include/rl_tools/.
#include "rlt_oracle.h"

#include <cmath>
#include <algorithm>
#include <string>
#include <random>
#include <sstream>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <dlfcn.h>
#include <vector>

namespace {

bool g_f64_accumulate = false;

// ---- optional CBLAS provider (the reference's CPU_BLAS device calls cblas_sgemm, devices/cpu_openblas.h:9-27)
enum { ORC_ROW_MAJOR = 101, ORC_NO_TRANS = 111, ORC_TRANS = 112 };
typedef void (*sgemm_fn)(int, int, int, int, int, int, float, const float*, int, const float*, int, float, float*, int);
sgemm_fn g_sgemm = nullptr;
char g_cblas_name[512] = "loops";

inline float dotf(const float* a, int sa, const float* b, int sb, int n, float init) {
    if (g_f64_accumulate) {
        double acc = init;
        for (int i = 0; i < n; i++) acc += (double)a[(size_t)i * sa] * (double)b[(size_t)i * sb];
        return (float)acc;
    }
    float acc = init;
    for (int i = 0; i < n; i++) acc += a[(size_t)i * sa] * b[(size_t)i * sb];
    return acc;
}

// math/operations_generic.h:247-251
inline float fast_tanh(float x) {
    x = x < -3.0f ? -3.0f : (x > 3.0f ? 3.0f : x);
    float x2 = x * x;
    return x * (27 + x2) / (27 + 9 * x2);
}

// random/operations_generic.h:72-105
inline float normal_log_prob(float mean, float log_std, float value) {
    // the reference writes the literals -0.5 and 0.5 as doubles, so the last term and the final subtraction are
    // evaluated in double and rounded once on return
    float neg_log_sqrt_pi = (float)(-0.5 * std::log(2 * (float)M_PI));
    float diff = value - mean;
    float sd = std::exp(log_std);
    float pre_square = diff / sd;
    return (float)((neg_log_sqrt_pi - log_std) - 0.5 * pre_square * pre_square);
}
inline float normal_d_log_prob_d_mean(float mean, float log_std, float value) {
    float diff = value - mean;
    float sd = std::exp(log_std);
    float pre_square = diff / sd;
    return pre_square / sd;
}
inline float normal_d_log_prob_d_log_std(float mean, float log_std, float value) {
    float diff = value - mean;
    float sd = std::exp(log_std);
    float pre_square = diff / sd;
    return -1 + pre_square * pre_square;
}
inline float normal_d_log_prob_d_sample(float mean, float log_std, float value) {
    float diff = value - mean;
    float sd = std::exp(log_std);
    float pre_square = diff / sd;
    return -pre_square / sd;
}
inline float clampf(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }

}  // namespace

extern "C" {

void rlt_oracle_set_f64_accumulate(int enabled) { g_f64_accumulate = enabled != 0; }

int rlt_oracle_use_cblas(const char* library_path) {
    if (!library_path) { g_sgemm = nullptr; std::snprintf(g_cblas_name, sizeof g_cblas_name, "loops"); return 0; }
    void* h = dlopen(library_path, RTLD_NOW | RTLD_LOCAL);
    if (!h) return 1;
    void* f = dlsym(h, "cblas_sgemm");
    if (!f) f = dlsym(h, "scipy_cblas_sgemm");
    if (!f) return 2;
    // single thread, as the reference's OpenBLAS device demands (devices/cpu_openblas.h:31-47)
    typedef void (*set_threads_fn)(int);
    const char* setters[] = {"openblas_set_num_threads", "scipy_openblas_set_num_threads", "MKL_Set_Num_Threads"};
    for (const char* s : setters) { if (void* st = dlsym(h, s)) { ((set_threads_fn)st)(1); break; } }
    g_sgemm = (sgemm_fn)f;
    std::snprintf(g_cblas_name, sizeof g_cblas_name, "%s", library_path);
    return 0;
}
const char* rlt_oracle_cblas_name(void) { return g_cblas_name; }

// nn/activation_functions.h:25-55
float rlt_oracle_activation(float x, int f) {
    switch (f) {
        case RLT_ACT_IDENTITY: return x;
        case RLT_ACT_RELU: return x > 0 ? x : 0;
        case RLT_ACT_GELU: { const float a = (float)(M_2_SQRTPI * M_SQRT1_2 * 0.5); return 0.5f * (x + x * std::tanh(a * (0.044715f * x * x * x + x))); }
        case RLT_ACT_TANH: return std::tanh(x);
        case RLT_ACT_FAST_TANH: return fast_tanh(x);
        case RLT_ACT_SIGMOID: return 1.0f / (1.0f + std::exp(-x));
    }
    return 0;
}
// nn/activation_functions.h:57-90
float rlt_oracle_d_activation(float x, int f) {
    switch (f) {
        case RLT_ACT_IDENTITY: return 1;
        case RLT_ACT_RELU: return x > 0 ? 1 : 0;
        case RLT_ACT_GELU: {
            const float a = (float)(M_2_SQRTPI * M_SQRT1_2 * 0.5); const float b = 0.044715f;
            float t = std::tanh(a * (b * x * x * x + x));
            return 0.5f * (1 + t) + 0.5f * x * (1 - t * t) * a * (3 * b * x * x + 1);
        }
        case RLT_ACT_TANH: { float a = std::tanh(x); return 1 - a * a; }
        case RLT_ACT_FAST_TANH: { float a = fast_tanh(x); return 1 - a * a; }
        case RLT_ACT_SIGMOID: { float s = rlt_oracle_activation(x, RLT_ACT_SIGMOID); return s * (1 - s); }
    }
    return 0;
}

// nn/layers/dense/operations_generic.h:95-138 (loops) / operations_cpu_blas.h:36-116 (bias broadcast, sgemm beta=1,
// copy to pre_activations, activation loop)
static int dense_forward_impl(const rlt_dense_layer* L, const float* x, int ldx, float* y, int ldy, int batch, bool store) {
    if (!L || !x || batch <= 0 || L->in_dim <= 0 || L->out_dim <= 0 || ldx < L->in_dim) return RLT_E_INVALID_ARGUMENT;
    if (y && ldy < L->out_dim) return RLT_E_INVALID_ARGUMENT;
    const int I = L->in_dim, O = L->out_dim;
    std::vector<float> tmp;
    float* acc = nullptr; int lda = O;
    if (g_sgemm) {
        tmp.resize((size_t)batch * O);
        acc = tmp.data();
        for (int b = 0; b < batch; b++) for (int o = 0; o < O; o++) acc[(size_t)b * O + o] = L->biases[o];
        g_sgemm(ORC_ROW_MAJOR, ORC_NO_TRANS, ORC_TRANS, batch, O, I, 1.0f, x, ldx, L->weights, I, 1.0f, acc, lda);
    }
    for (int b = 0; b < batch; b++) {
        for (int o = 0; o < O; o++) {
            float pre = acc ? acc[(size_t)b * O + o] : dotf(L->weights + (size_t)o * I, 1, x + (size_t)b * ldx, 1, I, L->biases[o]);
            float out = rlt_oracle_activation(pre, L->activation);
            if (store && L->pre_activations) L->pre_activations[(size_t)b * O + o] = pre;
            if (store && L->output) L->output[(size_t)b * O + o] = out;
            if (y) y[(size_t)b * ldy + o] = out;
        }
    }
    return 0;
}
int rlt_oracle_dense_evaluate(const rlt_dense_layer* L, const float* x, int ldx, float* y, int ldy, int batch) {
    if (!y) return RLT_E_INVALID_ARGUMENT;
    return dense_forward_impl(L, x, ldx, y, ldy, batch, false);
}
int rlt_oracle_dense_forward(const rlt_dense_layer* L, const float* x, int ldx, float* y, int ldy, int batch) {
    if (!L || !L->pre_activations) return RLT_E_INVALID_ARGUMENT;
    return dense_forward_impl(L, x, ldx, y, ldy, batch, true);
}

// operations_cpu_blas.h:119-141 backward_pre_activations (in place) ; with_bias: the fused loop of :165-171
static void d_pre_inplace(const rlt_dense_layer* L, float* d_output, int ldd, int batch, bool with_bias) {
    const int O = L->out_dim;
    for (int b = 0; b < batch; b++) {
        for (int o = 0; o < O; o++) {
            float d_pre = rlt_oracle_d_activation(L->pre_activations[(size_t)b * O + o], L->activation) * d_output[(size_t)b * ldd + o];
            if (with_bias) L->d_biases[o] += d_pre;
            d_output[(size_t)b * ldd + o] = d_pre;
        }
    }
}
// operations_cpu_blas.h:188-218 : d_input = d_pre W (beta = 0)
static void d_input_from_d_pre(const rlt_dense_layer* L, const float* d_pre, int ldd, float* d_input, int ldi, int batch) {
    const int I = L->in_dim, O = L->out_dim;
    if (g_sgemm) { g_sgemm(ORC_ROW_MAJOR, ORC_NO_TRANS, ORC_NO_TRANS, batch, I, O, 1.0f, d_pre, ldd, L->weights, I, 0.0f, d_input, ldi); return; }
    for (int b = 0; b < batch; b++)
        for (int i = 0; i < I; i++)
            d_input[(size_t)b * ldi + i] = dotf(d_pre + (size_t)b * ldd, 1, L->weights + i, I, O, 0.0f);
}
// operations_cpu_blas.h:173-185 : d_weights += d_pre^T x (beta = 1)
static void d_weights_accumulate(const rlt_dense_layer* L, const float* x, int ldx, const float* d_pre, int ldd, int batch) {
    const int I = L->in_dim, O = L->out_dim;
    if (g_sgemm) { g_sgemm(ORC_ROW_MAJOR, ORC_TRANS, ORC_NO_TRANS, O, I, batch, 1.0f, d_pre, ldd, x, ldx, 1.0f, L->d_weights, I); return; }
    for (int o = 0; o < O; o++)
        for (int i = 0; i < I; i++)
            L->d_weights[(size_t)o * I + i] = dotf(d_pre + o, ldd, x + i, ldx, batch, L->d_weights[(size_t)o * I + i]);
}
int rlt_oracle_dense_backward_input(const rlt_dense_layer* L, float* d_output, int ldd, float* d_input, int ldi, int batch) {
    if (!L || !L->pre_activations || !d_output || !d_input || batch <= 0 || ldd < L->out_dim || ldi < L->in_dim) return RLT_E_INVALID_ARGUMENT;
    d_pre_inplace(L, d_output, ldd, batch, false);
    d_input_from_d_pre(L, d_output, ldd, d_input, ldi, batch);
    return 0;
}
int rlt_oracle_dense_backward(const rlt_dense_layer* L, const float* x, int ldx, float* d_output, int ldd, int batch) {
    if (!L || !L->pre_activations || !L->d_weights || !L->d_biases || !x || !d_output || batch <= 0 || ldd < L->out_dim || ldx < L->in_dim) return RLT_E_INVALID_ARGUMENT;
    d_pre_inplace(L, d_output, ldd, batch, true);
    d_weights_accumulate(L, x, ldx, d_output, ldd, batch);
    return 0;
}
int rlt_oracle_dense_backward_full(const rlt_dense_layer* L, const float* x, int ldx, float* d_output, int ldd, float* d_input, int ldi, int batch) {
    int rc = rlt_oracle_dense_backward(L, x, ldx, d_output, ldd, batch);
    if (rc) return rc;
    if (!d_input || ldi < L->in_dim) return RLT_E_INVALID_ARGUMENT;
    d_input_from_d_pre(L, d_output, ldd, d_input, ldi, batch);
    return 0;
}

static int max_hidden(const rlt_dense_layer* layers, int n) { int m = 1; for (int i = 0; i + 1 < n; i++) if (layers[i].out_dim > m) m = layers[i].out_dim; return m; }

// nn_models/mlp/operations_generic.h:77-102
int rlt_oracle_mlp_evaluate(const rlt_dense_layer* layers, int n, const float* x, int ldx, float* y, int ldy, int batch) {
    if (!layers || n < 1 || !x || !y || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    int H = max_hidden(layers, n);
    std::vector<float> tick((size_t)batch * H), tock((size_t)batch * H);
    const float* in = x; int ldin = ldx;
    for (int l = 0; l < n; l++) {
        float* out = (l == n - 1) ? y : ((l % 2 == 0) ? tick.data() : tock.data());
        int ldo = (l == n - 1) ? ldy : layers[l].out_dim;
        int rc = rlt_oracle_dense_evaluate(&layers[l], in, ldin, out, ldo, batch);
        if (rc) return rc;
        in = out; ldin = ldo;
    }
    return 0;
}
// nn_models/mlp/operations_generic.h:103-114
int rlt_oracle_mlp_forward(const rlt_dense_layer* layers, int n, const float* x, int ldx, int batch) {
    if (!layers || n < 1 || !x || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    const float* in = x; int ldin = ldx;
    for (int l = 0; l < n; l++) {
        if (!layers[l].output) return RLT_E_INVALID_ARGUMENT;
        int rc = rlt_oracle_dense_forward(&layers[l], in, ldin, nullptr, 0, batch);
        if (rc) return rc;
        in = layers[l].output; ldin = layers[l].out_dim;
    }
    return 0;
}
// nn_models/mlp/operations_generic.h:126-204: output and hidden layers backward_full (or backward_input), the input layer
// only produces d_input when asked for (backward_full / backward_input)
int rlt_oracle_mlp_backward(const rlt_dense_layer* layers, int n, const float* x, int ldx, float* d_output, int ldd,
                            float* d_input, int ldi, int batch, int want_w) {
    if (!layers || n < 1 || !d_output || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    if (want_w && !x) return RLT_E_INVALID_ARGUMENT;
    int H = max_hidden(layers, n);
    std::vector<float> tick((size_t)batch * H), tock((size_t)batch * H);
    float* d_out = d_output; int ld_out = ldd;
    for (int l = n - 1; l >= 0; l--) {
        const float* in = (l == 0) ? x : layers[l - 1].output; int ldin = (l == 0) ? ldx : layers[l - 1].out_dim;
        float* d_in; int ld_in;
        if (l == 0) { d_in = d_input; ld_in = ldi; }
        else { d_in = ((n - 1 - l) % 2 == 0) ? tick.data() : tock.data(); ld_in = layers[l].in_dim; }
        int rc;
        if (want_w) {
            if (l > 0 && !in) return RLT_E_INVALID_ARGUMENT;
            rc = d_in ? rlt_oracle_dense_backward_full(&layers[l], in, ldin, d_out, ld_out, d_in, ld_in, batch)
                      : rlt_oracle_dense_backward(&layers[l], in, ldin, d_out, ld_out, batch);
        } else {
            if (!d_in) return RLT_E_INVALID_ARGUMENT;
            rc = rlt_oracle_dense_backward_input(&layers[l], d_out, ld_out, d_in, ld_in, batch);
        }
        if (rc) return rc;
        d_out = d_in; ld_out = ld_in;
    }
    return 0;
}
// nn_models/mlp/operations_generic.h:117-124
int rlt_oracle_mlp_zero_gradient(const rlt_dense_layer* layers, int n) {
    for (int l = 0; l < n; l++) {
        if (!layers[l].d_weights || !layers[l].d_biases) return RLT_E_INVALID_ARGUMENT;
        std::memset(layers[l].d_weights, 0, sizeof(float) * (size_t)layers[l].in_dim * layers[l].out_dim);
        std::memset(layers[l].d_biases, 0, sizeof(float) * (size_t)layers[l].out_dim);
    }
    return 0;
}
// forward (mlp :103-114) + optional mse::gradient (mse/operations_generic.h:41-56) + backward (mlp :180-204),
// with private activation storage so the caller's layers are left untouched.
int rlt_oracle_mlp_forward_backward(const rlt_dense_layer* layers, int n, const float* x, int ldx, float* y, int ldy,
                                    const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch) {
    return rlt_oracle_mlp_forward_backward_input(layers, n, x, ldx, y, ldy, d_output, ldd, target, ldt, mse_scale, nullptr, 0, batch);
}
// forward, loss gradient, backward_full (nn_models/mlp/operations_generic.h:128-260) with private activation storage
int rlt_oracle_mlp_forward_backward_input(const rlt_dense_layer* layers, int n, const float* x, int ldx, float* y, int ldy,
                                          const float* d_output, int ldd, const float* target, int ldt, float mse_scale, float* d_input, int ldi, int batch) {
    if (!layers || n < 1 || !x || batch <= 0 || (!d_output && !target)) return RLT_E_INVALID_ARGUMENT;
    std::vector<rlt_dense_layer> priv(layers, layers + n);
    std::vector<std::vector<float>> pre(n), out(n);
    for (int l = 0; l < n; l++) {
        pre[l].resize((size_t)batch * layers[l].out_dim); out[l].resize((size_t)batch * layers[l].out_dim);
        priv[l].pre_activations = pre[l].data(); priv[l].output = out[l].data();
    }
    int rc = rlt_oracle_mlp_forward(priv.data(), n, x, ldx, batch);
    if (rc) return rc;
    const int O = layers[n - 1].out_dim;
    std::vector<float> d((size_t)batch * O);
    for (int b = 0; b < batch; b++)
        for (int o = 0; o < O; o++) {
            float yv = out[n - 1][(size_t)b * O + o];
            if (y) y[(size_t)b * ldy + o] = yv;
            d[(size_t)b * O + o] = target ? (yv - target[(size_t)b * ldt + o]) * mse_scale : d_output[(size_t)b * ldd + o];
        }
    return rlt_oracle_mlp_backward(priv.data(), n, x, ldx, d.data(), O, d_input, ldi, batch, 1);
}

// nn/optimizers/adam/operations_generic.h:49-66 (_step: bias corrections from age, then age++) and
// instance/operations_generic.h:26-72 (moments via utils/polyak, then gradient_descent)
int rlt_oracle_adam_step(const rlt_adam_tensor* tensors, int n_tensors, const rlt_adam_parameters* p, uint32_t* age,
                         float polyak, float* out_sq_norm) {
    if (!tensors || n_tensors < 0 || !p || !age) return RLT_E_INVALID_ARGUMENT;
    float bc1 = 1 / (1 - std::pow(p->beta_1, (float)*age));
    float bc2 = 1 / (1 - std::pow(p->beta_2, (float)*age));
    *age += 1;
    double sq = 0;
    for (int t = 0; t < n_tensors; t++) {
        const rlt_adam_tensor& T = tensors[t];
        if (!T.parameters || !T.gradient || !T.first_moment || !T.second_moment) return RLT_E_INVALID_ARGUMENT;
        for (uint32_t i = 0; i < T.count; i++) {
            float g = T.gradient[i];
            sq += (double)g * g;
            if (p->enable_gradient_clipping) g = clampf(g, -p->gradient_clip_value, p->gradient_clip_value);
            float m = p->beta_1 * T.first_moment[i] + (1 - p->beta_1) * g;          // utils/polyak/operations_generic.h:11-24
            float v = p->beta_2 * T.second_moment[i] + (1 - p->beta_2) * g * g;     // :27-41
            T.first_moment[i] = m; T.second_moment[i] = v;
            float pre_sqrt = v * bc2;
            pre_sqrt = pre_sqrt > p->epsilon_sqrt ? pre_sqrt : p->epsilon_sqrt;
            float update = p->alpha * bc1 * m / (std::sqrt(pre_sqrt) + p->epsilon);
            if ((T.flags & 2u) && p->enable_bias_lr_factor) update *= p->bias_lr_factor;
            if ((T.flags & 1u) && p->enable_weight_decay) update += T.parameters[i] * p->weight_decay / 2;
            float value = T.parameters[i] - update;
            T.parameters[i] = value;
            if (T.polyak_target) T.polyak_target[i] = polyak * T.polyak_target[i] + (1 - polyak) * value;
        }
    }
    if (out_sq_norm) *out_sq_norm = (float)sq;
    return 0;
}
// adam/operations_generic.h:43-47 + instance/operations_generic.h:65-69
int rlt_oracle_adam_reset(const rlt_adam_tensor* tensors, int n_tensors, uint32_t* age) {
    if (!tensors || !age) return RLT_E_INVALID_ARGUMENT;
    *age = 1;
    for (int t = 0; t < n_tensors; t++) {
        std::memset(tensors[t].first_moment, 0, sizeof(float) * tensors[t].count);
        std::memset(tensors[t].second_moment, 0, sizeof(float) * tensors[t].count);
    }
    return 0;
}
// utils/polyak/operations_generic.h:11-43
int rlt_oracle_polyak_update(const float* source, float* target, size_t count, float polyak, int squared) {
    if (!source || !target) return RLT_E_INVALID_ARGUMENT;
    for (size_t i = 0; i < count; i++) {
        float s = source[i];
        target[i] = squared ? polyak * target[i] + (1 - polyak) * s * s : polyak * target[i] + (1 - polyak) * s;
    }
    return 0;
}

// nn/loss_functions/mse/operations_generic.h:41-56,73-87
int rlt_oracle_mse_gradient(const float* a, int lda, const float* b, int ldb, float* d_a, int ldda, int rows, int cols,
                            float loss_weight, const float* loss_weight_ptr) {
    if (!a || !b || !d_a || rows <= 0 || cols <= 0) return RLT_E_INVALID_ARGUMENT;
    float w = loss_weight_ptr ? *loss_weight_ptr : loss_weight;
    float constant = (float)2 / ((float)rows * cols) * w;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            float diff = a[(size_t)r * lda + c] - b[(size_t)r * ldb + c];
            d_a[(size_t)r * ldda + c] = diff * constant;
        }
    return 0;
}
// mse/operations_generic.h:9-21
int rlt_oracle_mse_evaluate(const float* a, int lda, const float* b, int ldb, int rows, int cols, float loss_weight, float* out_loss) {
    if (!a || !b || !out_loss || rows <= 0 || cols <= 0) return RLT_E_INVALID_ARGUMENT;
    float acc = 0;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            float diff = a[(size_t)r * lda + c] - b[(size_t)r * ldb + c];
            acc += diff * diff;
        }
    *out_loss = acc * loss_weight / (rows * cols);
    return 0;
}

// nn/layers/sample_and_squash/operations_generic.h:148-261
int rlt_oracle_sas_forward(const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                           float* actions, int lda, float* pre_squashing, int ldp, float* log_probabilities, int batch, int dim) {
    if (!p || !input || !actions || !log_probabilities || batch <= 0 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < batch; r++) {
        float log_prob = 0;
        for (int c = 0; c < dim; c++) {
            float mean = input[(size_t)r * ldin + c];
            float log_std = input[(size_t)r * ldin + dim + c];
            float log_std_clipped = clampf(log_std, p->log_std_lower_bound, p->log_std_upper_bound);
            float sd = std::exp(log_std_clipped);
            float eps = noise ? noise[(size_t)r * ldn + c] : 0.0f;
            float sample = noise ? mean + eps * sd : mean;
            if (pre_squashing) pre_squashing[(size_t)r * ldp + c] = sample;
            float squashed = std::tanh(sample);
            actions[(size_t)r * lda + c] = squashed;
            float one_minus_square_plus_eps = (1 - squashed * squashed + p->log_probability_epsilon);
            log_prob += normal_log_prob(mean, log_std_clipped, sample) - std::log(one_minus_square_plus_eps);
        }
        log_probabilities[r] = log_prob;
    }
    return 0;
}
// nn/layers/sample_and_squash/operations_generic.h:289-398
static int sas_backward_impl(const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                            const float* actions, int lda, const float* pre_squashing, int ldp,
                            const float* d_output, int lddo, float* d_input, int lddi,
                            const float* log_alpha, float* d_log_alpha, int batch, int dim, float divisor) {
    if (!p || !input || !noise || !actions || !pre_squashing || !d_output || !d_input || !log_alpha || batch <= 0 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    float alpha = std::exp(*log_alpha);
    float d_log_alpha_sum = 0;
    for (int b = 0; b < batch; b++) {
        float entropy = 0;
        for (int a = 0; a < dim; a++) {
            float action = actions[(size_t)b * lda + a];
            float d_output_value = d_output[(size_t)b * lddo + a];
            float d_tanh_pre_activation = d_output_value * (1 - action * action);
            float d_mu = d_tanh_pre_activation;
            float eps = noise[(size_t)b * ldn + a];
            float d_std = d_tanh_pre_activation * eps;
            float log_std_pre_clamp = input[(size_t)b * ldin + dim + a];
            float log_std_clamped = clampf(log_std_pre_clamp, p->log_std_lower_bound, p->log_std_upper_bound);
            float sd = std::exp(log_std_clamped);
            float d_log_std_clamped = sd * d_std;
            float mu = input[(size_t)b * ldin + a];
            float action_sample = pre_squashing[(size_t)b * ldp + a];
            float dlp_dmean = normal_d_log_prob_d_mean(mu, log_std_clamped, action_sample);
            float dlp_dsample = normal_d_log_prob_d_sample(mu, log_std_clamped, action_sample);
            d_mu += alpha / batch * (dlp_dmean + dlp_dsample + 2 * action);
            float dlp_dlogstd = normal_d_log_prob_d_log_std(mu, log_std_clamped, action_sample);
            d_log_std_clamped += alpha / batch * (dlp_dlogstd + dlp_dsample * eps * sd + 2 * action * eps * sd);
            float d_log_std = (log_std_pre_clamp < p->log_std_lower_bound || log_std_pre_clamp > p->log_std_upper_bound) ? 0 : d_log_std_clamped;
            d_input[(size_t)b * lddi + a] = d_mu;
            d_input[(size_t)b * lddi + dim + a] = d_log_std;
            float one_minus_action_square_plus_eps = (1 - action * action + p->log_probability_epsilon);
            float action_log_prob = normal_log_prob(mu, log_std_clamped, action_sample) - std::log(one_minus_action_square_plus_eps);
            entropy += -action_log_prob;
        }
        float d_alpha = entropy - p->target_entropy;
        d_log_alpha_sum += alpha * d_alpha;
    }
    if (d_log_alpha) *d_log_alpha += d_log_alpha_sum / divisor;
    return 0;
}
int rlt_oracle_sas_backward(const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                            const float* actions, int lda, const float* pre_squashing, int ldp,
                            const float* d_output, int lddo, float* d_input, int lddi,
                            const float* log_alpha, float* d_log_alpha, int batch, int dim) {
    return sas_backward_impl(p, input, ldin, noise, ldn, actions, lda, pre_squashing, ldp, d_output, lddo, d_input, lddi, log_alpha, d_log_alpha, batch, dim, (float)batch);
}
// the same under a ResetMode (:390-394): the sum over the rows is divided by the number of set reset flags (an integer count) instead of the row count
int rlt_oracle_sas_backward_reset(const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                                  const float* actions, int lda, const float* pre_squashing, int ldp,
                                  const float* d_output, int lddo, float* d_input, int lddi,
                                  const float* log_alpha, float* d_log_alpha, const uint8_t* reset, int batch, int dim) {
    if (!reset) return RLT_E_INVALID_ARGUMENT;
    size_t n = 0;
    for (int i = 0; i < batch; i++) n += reset[i] != 0;
    return sas_backward_impl(p, input, ldin, noise, ldn, actions, lda, pre_squashing, ldp, d_output, lddo, d_input, lddi, log_alpha, d_log_alpha, batch, dim, (float)n);
}

// rl/algorithms/sac/operations_generic.h:133-179
int rlt_oracle_sac_target_action_values(const float* q1, const float* q2, const float* rewards, const uint8_t* terminated,
                                        const float* next_log_probs, const float* log_alpha, float gamma, int ignore_termination,
                                        float* target, int batch) {
    if (!q1 || !q2 || !rewards || !terminated || !next_log_probs || !log_alpha || !target || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    float alpha = std::exp(*log_alpha);
    for (int i = 0; i < batch; i++) {
        float min_q = q1[i] < q2[i] ? q1[i] : q2[i];
        float entropy_bonus = -alpha * next_log_probs[i];
        min_q += entropy_bonus;
        float future_value = (ignore_termination || !terminated[i]) ? gamma * min_q : 0;
        target[i] = rewards[i] + future_value;
    }
    return 0;
}
// rl/algorithms/sac/operations_generic.h:358-393
int rlt_oracle_sac_min_value_d_output(const float* q1, const float* q2, const float* d1, const float* d2, int ld, int critic_input_dim,
                                      int action_dim, float* d_actor_output, int ldo, int batch) {
    if (!q1 || !q2 || !d1 || !d2 || !d_actor_output || batch <= 0 || action_dim <= 0 || critic_input_dim < action_dim) return RLT_E_INVALID_ARGUMENT;
    for (int b = 0; b < batch; b++) {
        bool first = q1[b] < q2[b];
        for (int a = 0; a < action_dim; a++) {
            size_t src = (size_t)b * ld + critic_input_dim - action_dim + a;
            d_actor_output[(size_t)b * ldo + a] = first ? d1[src] : d2[src];
        }
    }
    return 0;
}
// rl/algorithms/sac/operations_generic.h:181-209
int rlt_oracle_mask_copy(const float* source, int lds, float* target, int ldt, const uint8_t* mask, int invert, int rows, int cols) {
    if (!source || !target || !mask) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < rows; r++) {
        bool m = mask[r] != 0; if (invert) m = !m;
        if (m) for (int c = 0; c < cols; c++) target[(size_t)r * ldt + c] = source[(size_t)r * lds + c];
    }
    return 0;
}
// rl/algorithms/sac/operations_generic.h:210-234
int rlt_oracle_mask_zero(float* gradient, int ld, const uint8_t* mask, int invert, int rows, int cols) {
    if (!gradient || !mask) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < rows; r++) {
        bool m = mask[r] != 0; if (invert) m = !m;
        if (m) for (int c = 0; c < cols; c++) gradient[(size_t)r * ld + c] = 0;
    }
    return 0;
}
// containers/tensor/operations_generic.h:433-445
int rlt_oracle_scale_f32(float* x, size_t count, float s, int reciprocal) {
    if (!x) return RLT_E_INVALID_ARGUMENT;
    for (size_t i = 0; i < count; i++) x[i] = reciprocal ? (1.0f / x[i]) * s : x[i] * s;   // containers/tensor/operations_generic.h:437-443: the reciprocal first, then the scale
    return 0;
}
// containers/tensor/operations_generic.h:928-985 (CastSum)
int rlt_oracle_cast_reduce_sum_u8(const uint8_t* mask, size_t count, float* out_sum) {
    if (!mask || !out_sum) return RLT_E_INVALID_ARGUMENT;
    float acc = 0;
    for (size_t i = 0; i < count; i++) acc += (float)(mask[i] != 0);
    *out_sum = acc;
    return 0;
}

// --------------------------------------------------------------------------------------------- SAC update steps
static int adam_over(const rlt_adam_tensor* t, int n, const rlt_adam_parameters* p, uint32_t* age) {
    return rlt_oracle_adam_step(t, n, p, age, 0.0f, nullptr);
}

// rl/algorithms/sac/operations_generic.h:243-337 with SEQUENCE_LENGTH = 1
int rlt_oracle_sac_train_critic(const rlt_sac_agent* A, int ci, const float* action_noise) {
    if (!A || ci < 0 || ci > 1 || !action_noise) return RLT_E_INVALID_ARGUMENT;
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const rlt_dense_layer* critic = A->critics[ci];
    int rc;
    if ((rc = rlt_oracle_mlp_zero_gradient(critic, A->n_critic_layers))) return rc;                           // :263
    const float* obs_next = A->observations_actions_base + (size_t)B * D;                                   // padded step 1
    // actor evaluate on next observations with external noise (:266-273): MLP then sample_and_squash
    std::vector<float> actor_out((size_t)B * 2 * ACT);
    if ((rc = rlt_oracle_mlp_evaluate(A->actor, A->n_actor_layers, obs_next, D, actor_out.data(), 2 * ACT, B))) return rc;
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = rlt_oracle_sas_forward(&A->sas, actor_out.data(), 2 * ACT, action_noise, ACT, next_actions, D, nullptr, 0, A->next_log_probabilities, B, ACT))) return rc;
    if (A->next_final_step_mask)                                                                            // :274-277
        if ((rc = rlt_oracle_mask_copy(obs_next + OBS, D, next_actions, D, A->next_final_step_mask, 1, B, ACT))) return rc;
    for (int b = 0; b < B; b++) std::memcpy(A->next_state_action_value_input + (size_t)b * D, obs_next + (size_t)b * D, sizeof(float) * OBS); // :278
    for (int k = 0; k < 2; k++)                                                                             // :283-284
        if ((rc = rlt_oracle_mlp_evaluate(A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, A->next_q[k], 1, B))) return rc;
    if ((rc = rlt_oracle_sac_target_action_values(A->next_q[0], A->next_q[1], A->rewards, A->terminated, A->next_log_probabilities,
                                                 A->log_alpha.parameters, A->gamma, 0, A->target_action_value, B))) return rc;      // :289
    if ((rc = rlt_oracle_mlp_forward(critic, A->n_critic_layers, A->observations_actions_base, D, B))) return rc;                  // :294
    const float* q = critic[A->n_critic_layers - 1].output;
    // :298-306 loss_weight = (SEQ*B*0.5) / num_final_steps
    float loss_weight = 0;
    if (A->final_step_mask) rlt_oracle_cast_reduce_sum_u8(A->final_step_mask, B, &loss_weight); else loss_weight = (float)B;
    rlt_oracle_scale_f32(&loss_weight, 1, 1 * B * 0.5f, 1);
    float* d_out = A->d_output_critic[ci];
    if ((rc = rlt_oracle_mse_gradient(q, 1, A->target_action_value, 1, d_out, 1, B, 1, 0, &loss_weight))) return rc;                 // :312
    if (A->final_step_mask) rlt_oracle_mask_zero(d_out, 1, A->final_step_mask, 1, B, 1);                                          // :314-316
    std::vector<float> scratch;
    if ((rc = rlt_oracle_mlp_backward(critic, A->n_critic_layers, A->observations_actions_base, D, d_out, 1, nullptr, 0, B, 1))) return rc; // :329
    return adam_over(A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci]);                  // :336
}

// rl/algorithms/sac/operations_generic.h:488-527
int rlt_oracle_sac_update_critic_targets(const rlt_sac_agent* A) {
    if (!A) return RLT_E_INVALID_ARGUMENT;
    for (int k = 0; k < 2; k++)
        for (int l = 0; l < A->n_critic_layers; l++) {
            const rlt_dense_layer& s = A->critics[k][l]; const rlt_dense_layer& t = A->critics_target[k][l];
            rlt_oracle_polyak_update(s.weights, t.weights, (size_t)s.in_dim * s.out_dim, A->polyak, 0);
            rlt_oracle_polyak_update(s.biases, t.biases, (size_t)s.out_dim, A->polyak, 0);
        }
    return 0;
}

// rl/algorithms/sac/operations_generic.h:395-468 with SEQUENCE_LENGTH = 1
int rlt_oracle_sac_train_actor(const rlt_sac_agent* A, const float* action_noise) {
    if (!A || !action_noise) return RLT_E_INVALID_ARGUMENT;
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    int rc;
    if ((rc = rlt_oracle_mlp_zero_gradient(A->actor, A->n_actor_layers))) return rc;                          // :414
    A->log_alpha.gradient[0] = 0;   // zero_gradient(actor) also clears the sample_and_squash layer's log_alpha gradient
    const float* obs = A->observations_actions_base;
    if ((rc = rlt_oracle_mlp_forward(A->actor, A->n_actor_layers, obs, D, B))) return rc;                     // :427 (MLP part)
    const float* actor_out = A->actor[A->n_actor_layers - 1].output;
    if ((rc = rlt_oracle_sas_forward(&A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT,
                                     A->actor_log_probabilities, B, ACT))) return rc;
    float* sav_actions = A->state_action_value_input + OBS;
    for (int b = 0; b < B; b++) std::memcpy(sav_actions + (size_t)b * D, A->actor_actions + (size_t)b * ACT, sizeof(float) * ACT);
    if (A->final_step_mask)                                                                                 // :428-430
        if ((rc = rlt_oracle_mask_copy(obs + OBS, D, sav_actions, D, A->final_step_mask, 1, B, ACT))) return rc;
    for (int b = 0; b < B; b++) std::memcpy(A->state_action_value_input + (size_t)b * D, obs + (size_t)b * D, sizeof(float) * OBS); // :431
    for (int k = 0; k < 2; k++)                                                                             // :432-433
        if ((rc = rlt_oracle_mlp_forward(A->critics[k], A->n_critic_layers, A->state_action_value_input, D, B))) return rc;
    // :437-453 d_output = -1/num_final_steps on final steps
    float loss_weight = 0;
    if (A->final_step_mask) rlt_oracle_cast_reduce_sum_u8(A->final_step_mask, B, &loss_weight); else loss_weight = (float)B;
    rlt_oracle_scale_f32(&loss_weight, 1, -1.0f, 1);
    std::vector<float> d_out((size_t)B);
    for (int k = 0; k < 2; k++) {                                                                           // :458-459
        for (int b = 0; b < B; b++) d_out[b] = loss_weight;
        if (A->final_step_mask) rlt_oracle_mask_zero(d_out.data(), 1, A->final_step_mask, 1, B, 1);
        // NOTE the reference reuses ONE d_output tensor for both critics and the first backward_input overwrites it with
        // d_pre of critic 0's output layer; that layer's activation is IDENTITY, so d_pre == d_output and the second call
        // sees the same values.
        if ((rc = rlt_oracle_mlp_backward(A->critics[k], A->n_critic_layers, nullptr, 0, d_out.data(), 1, A->d_critic_input[k], D, B, 0))) return rc;
    }
    std::memcpy(A->d_output_actor_critics, d_out.data(), sizeof(float) * B);
    const float* q1 = A->critics[0][A->n_critic_layers - 1].output; const float* q2 = A->critics[1][A->n_critic_layers - 1].output;
    if ((rc = rlt_oracle_sac_min_value_d_output(q1, q2, A->d_critic_input[0], A->d_critic_input[1], D, D, ACT, A->d_actor_output_squashing, ACT, B))) return rc; // :460
    if (A->final_step_mask) rlt_oracle_mask_zero(A->d_actor_output_squashing, ACT, A->final_step_mask, 1, B, ACT);           // :461-463
    // sequential backward: sample_and_squash backward_full (divides d_log_alpha by num_resets = sum(reset)), then MLP backward (:464)
    if (A->reset) rc = rlt_oracle_sas_backward_reset(&A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT,
                                                     A->d_actor_output_squashing, ACT, A->d_actor_output, 2 * ACT, A->log_alpha.parameters, &A->log_alpha.gradient[0], A->reset, B, ACT);
    else rc = rlt_oracle_sas_backward(&A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT,
                                      A->d_actor_output_squashing, ACT, A->d_actor_output, 2 * ACT, A->log_alpha.parameters, &A->log_alpha.gradient[0], B, ACT);
    if (rc) return rc;
    if ((rc = rlt_oracle_mlp_backward(A->actor, A->n_actor_layers, obs, D, A->d_actor_output, 2 * ACT, nullptr, 0, B, 1))) return rc;
    if ((rc = adam_over(A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age))) return rc;                // :465
    return adam_over(&A->log_alpha, 1, &A->alpha_adam, A->alpha_age);                                                           // :466
}

// ------------------------------------------------------------------------------ replay buffer, gather, Pendulum
static inline int rb_row_dim(const rlt_replay_buffer* rb) { return 2 * rb->observation_dim + rb->action_dim + 3; }

// rl/components/replay_buffer/operations_generic.h:54-78, one transition per environment
int rlt_oracle_replay_add(const rlt_replay_buffer* rb, const float* obs, const float* actions, const float* rewards,
                          const float* next_obs, const uint8_t* terminated, const uint8_t* truncated) {
    if (!rb || !rb->data || !obs || !actions || !rewards || !next_obs || !terminated || !truncated) return RLT_E_INVALID_ARGUMENT;
    const int OBS = rb->observation_dim, ACT = rb->action_dim, R = rb_row_dim(rb);
    for (int e = 0; e < rb->n_envs; e++) {
        uint32_t pos = rb->position[e];
        float* row = rb->data + ((size_t)e * rb->capacity + pos) * R;
        for (int i = 0; i < OBS; i++) { row[i] = obs[(size_t)e * OBS + i]; row[OBS + ACT + 1 + i] = next_obs[(size_t)e * OBS + i]; }
        for (int i = 0; i < ACT; i++) row[OBS + i] = actions[(size_t)e * ACT + i];
        row[OBS + ACT] = rewards[e];
        row[2 * OBS + ACT + 1] = terminated[e] ? 1.0f : 0.0f;
        row[2 * OBS + ACT + 2] = truncated[e] ? 1.0f : 0.0f;
        rb->episode_start[(size_t)e * rb->capacity + pos] = rb->current_episode_start[e];
        pos = (pos + 1) % (uint32_t)rb->capacity;
        rb->position[e] = pos;
        if (truncated[e]) rb->current_episode_start[e] = pos;
        if (pos == 0 && !rb->full[e]) rb->full[e] = 1;
    }
    return 0;
}

// rl/components/off_policy_runner/operations_generic.h:240-430 with SEQUENCE_LENGTH = 1 (PADDED = 2), no
// ALWAYS_SAMPLE_FROM_INITIAL_STATE, no RANDOM_SEQ_LENGTH (off_policy_runner.h:79-87 for SEQUENCE_LENGTH == 1)
int rlt_oracle_gather_batch(const rlt_replay_buffer* rb, const uint32_t* env_indices, const uint32_t* sample_offsets, int deterministic,
                            int max_episode_length, int batch, float* oab, float* rewards, uint8_t* terminated,
                            uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base) {
    if (!rb || !rb->data || batch <= 0 || !oab || !rewards || !terminated) return RLT_E_INVALID_ARGUMENT;
    if (!deterministic && (!env_indices || !sample_offsets)) return RLT_E_INVALID_ARGUMENT;
    const int OBS = rb->observation_dim, ACT = rb->action_dim, R = rb_row_dim(rb), D = OBS + ACT;
    for (int i = 0; i < batch; i++) {
        uint32_t e = deterministic ? 0u : env_indices[i];
        if (e >= (uint32_t)rb->n_envs) return RLT_E_INVALID_ARGUMENT;
        uint32_t offset = deterministic ? (uint32_t)i : sample_offsets[i];
        uint32_t index = rb->full[e] ? (rb->position[e] + (uint32_t)max_episode_length + offset) % (uint32_t)rb->capacity : offset;   // :305-311
        if (index >= (uint32_t)rb->capacity) return RLT_E_INVALID_ARGUMENT;
        const float* row = rb->data + ((size_t)e * rb->capacity + index) * R;
        float* step0 = oab + (size_t)i * D; float* step1 = oab + ((size_t)batch + i) * D;
        for (int k = 0; k < OBS; k++) step0[k] = row[k];                       // :322-327
        for (int k = 0; k < ACT; k++) step0[OBS + k] = row[OBS + k];           // :338-343
        rewards[i] = row[OBS + ACT];                                           // :346
        terminated[i] = row[2 * OBS + ACT + 1] != 0.0f;                        // :347
        // seq_step 0 == PADDED-2 forces truncated (:357-359): next observation into padded step 1, next action zeroed (:392-412)
        for (int k = 0; k < OBS; k++) step1[k] = row[OBS + ACT + 1 + k];
        for (int k = 0; k < ACT; k++) step1[OBS + k] = 0;
        if (reset) reset[i] = 1;                                               // :283,298
        if (next_reset_base) { next_reset_base[i] = 1; next_reset_base[batch + i] = 1; }   // :284,300 (step 0) and :285 via the offset-1 view (step 1)
        if (final_step_mask) final_step_mask[i] = 1;                           // :389-391
        if (next_final_step_mask_base) { next_final_step_mask_base[i] = 0; next_final_step_mask_base[batch + i] = 1; } // :279-280,291
    }
    return 0;
}

// gather_batch_step for sequences (rl/components/off_policy_runner/operations_generic.h:239-418), one sample. DRAWS supplies the randomness:
// offset(max) = uniform_int(0, max), nominal() = uniform_real(0, 1) < probability, length() = uniform_int(1, sequence_length - 1).
extern "C++" {
template <typename DRAWS>
static int gather_sequence_sample(const rlt_replay_buffer* rb, uint32_t e, const rlt_sequence_sampling* P, int max_episode_length, const rlt_sequence_batch* B, int b, DRAWS& draws) {
    const int OBS = rb->observation_dim, ACT = rb->action_dim, R = rb_row_dim(rb), D = OBS + ACT, N = B->batch, SEQ = B->sequence_length, PADDED = SEQ + 1;
    const uint32_t CAP = (uint32_t)rb->capacity, position = rb->position[e];
    const bool full = rb->full[e] != 0;
    const uint32_t eligible = full ? (P->always_sample_from_initial_state ? CAP - (uint32_t)max_episode_length : CAP) : position;      // :259
    if (eligible == 0) return RLT_E_INVALID_ARGUMENT;
    const uint32_t sample_index_max = eligible - 1;
    uint32_t sample_index = 0;
    int current_seq_length = SEQ;
    auto draw_length = [&]() {       // :266-275 and :362-371
        if (P->enable_nominal_sequence_length_probability && draws.nominal()) return SEQ;
        return SEQ > 1 ? (int)draws.length() : current_seq_length;
    };
    if (P->random_seq_length) current_seq_length = draw_length();
    int current_seq_step = 0;
    bool previous_step_truncated = false, previous_padding_step = true;
    for (int s = 0; s < SEQ; s++) { B->final_step_mask[(size_t)s * N + b] = 0; B->reset[(size_t)s * N + b] = 0; }            // :279-287
    for (int s = 0; s < PADDED; s++) { B->next_final_step_mask_base[(size_t)s * N + b] = 0; B->next_reset_base[(size_t)s * N + b] = 0; }
    B->reset[b] = 1; B->next_reset_base[b] = 1;
    B->next_reset_base[(size_t)(P->include_first_step_in_targets ? 0 : 1) * N + b] = 1;           // batch.next_reset is a view from step 0 or 1 (:85-92,286)
    for (int s = 0; s < PADDED; s++) {
        if (previous_step_truncated) {                                                                                       // :289-298
            previous_step_truncated = false; previous_padding_step = true;
            B->next_final_step_mask_base[(size_t)s * N + b] = 1;
            if (s < PADDED - 1) B->reset[(size_t)s * N + b] = 1;
            continue;
        }
        if (previous_padding_step) {                                                                                         // :299-318
            if (s < PADDED - 1) B->reset[(size_t)s * N + b] = 1;
            B->next_reset_base[(size_t)s * N + b] = 1;
            const uint32_t sample_offset = draws.offset(sample_index_max);
            sample_index = full ? (position + (uint32_t)max_episode_length + sample_offset) % CAP : sample_offset;
            if (P->always_sample_from_initial_state) sample_index = rb->episode_start[(size_t)e * CAP + sample_index];
        }
        if (sample_index >= CAP) return RLT_E_INVALID_ARGUMENT;
        const float* row = rb->data + ((size_t)e * CAP + sample_index) * R;
        float* step = B->observations_actions_base + ((size_t)s * N + b) * D;
        for (int k = 0; k < OBS; k++) step[k] = row[k];                                                                      // :321-326
        for (int k = 0; k < ACT; k++) step[OBS + k] = row[OBS + k];                                                          // :336-341
        if (s < PADDED - 1) { B->rewards[(size_t)s * N + b] = row[OBS + ACT]; B->terminated[(size_t)s * N + b] = row[2 * OBS + ACT + 1] != 0.0f; }   // :343-346
        bool truncated = row[2 * OBS + ACT + 2] != 0.0f;                                                                     // :348
        uint32_t next_sample_index = sample_index + 1;
        if (full) next_sample_index %= CAP;
        if (next_sample_index == position) truncated = true;                                                                 // :354-356
        if (s == PADDED - 2) truncated = true;                                                                               // :357-359
        if (P->random_seq_length) {                                                                                          // :360-383
            if (current_seq_step == current_seq_length - 1) {
                truncated = true;
                current_seq_length = SEQ > 1 ? draw_length() : SEQ;
            }
            current_seq_step = truncated ? 0 : current_seq_step + 1;
        }
        if (truncated && s < PADDED - 1) {                                                                                   // :388-413
            B->final_step_mask[(size_t)s * N + b] = 1;
            float* next = B->observations_actions_base + ((size_t)(s + 1) * N + b) * D;
            for (int k = 0; k < OBS; k++) next[k] = row[OBS + ACT + 1 + k];
            for (int k = 0; k < ACT; k++) next[OBS + k] = 0;
        }
        sample_index = next_sample_index;
        previous_padding_step = false;
        previous_step_truncated = truncated;
    }
    return 0;
}
struct ArrayDraws {
    const rlt_sequence_draws* d; int b, padded, n_offset = 0, n_length = 0;
    uint32_t offset(uint32_t) { return d->sample_offsets[(size_t)b * padded + n_offset++]; }
    bool nominal() { return d->nominal[(size_t)b * (padded + 1) + n_length] != 0; }        // the length decision's index advances once per decision:
    uint32_t length() { return d->lengths[(size_t)b * (padded + 1) + n_length]; }
};
struct EngineDraws {
    std::mt19937* engine; const rlt_sequence_sampling* P; int sequence_length, b, padded, n_offset = 0, n_length = 0;
    uint32_t* offsets; uint8_t* nominals; uint32_t* lengths;
    uint32_t offset(uint32_t max) { const uint32_t v = (uint32_t)std::uniform_int_distribution<size_t>(0, max)(*engine); offsets[(size_t)b * padded + n_offset++] = v; return v; }
    bool nominal() { const bool v = std::uniform_real_distribution<double>(0.0, 1.0)(*engine) < P->nominal_sequence_length_probability; nominals[(size_t)b * (padded + 1) + n_length] = v; return v; }
    uint32_t length() { const uint32_t v = (uint32_t)std::uniform_int_distribution<size_t>(1, (size_t)sequence_length - 1)(*engine); lengths[(size_t)b * (padded + 1) + n_length] = v; return v; }
};
}  // extern "C++"
static bool sequence_arguments_ok(const rlt_replay_buffer* rb, const rlt_sequence_sampling* P, const rlt_sequence_batch* B) {
    return rb && rb->data && rb->episode_start && P && B && B->batch > 0 && B->sequence_length >= 1 && B->observations_actions_base && B->rewards && B->terminated && B->reset &&
           B->next_reset_base && B->final_step_mask && B->next_final_step_mask_base;
}
int rlt_oracle_gather_sequence_batch(const rlt_replay_buffer* rb, const rlt_sequence_sampling* P, const rlt_sequence_draws* draws, int max_episode_length,
                                     const rlt_sequence_batch* B) {
    if (!sequence_arguments_ok(rb, P, B) || !draws || !draws->env_indices || !draws->sample_offsets || (P->random_seq_length && (!draws->nominal || !draws->lengths))) return RLT_E_INVALID_ARGUMENT;
    for (int b = 0; b < B->batch; b++) {
        const uint32_t e = draws->env_indices[b];
        if (e >= (uint32_t)rb->n_envs) return RLT_E_INVALID_ARGUMENT;
        // a length decision consumes nominal[k] and, where that is 0, lengths[k]: one index for both
        struct Fed : ArrayDraws { bool nominal() { const bool v = ArrayDraws::nominal(); if (v) n_length++; return v; } uint32_t length() { const uint32_t v = ArrayDraws::length(); n_length++; return v; } };
        Fed fed; fed.d = draws; fed.b = b; fed.padded = B->sequence_length + 1;
        const int rc = gather_sequence_sample(rb, e, P, max_episode_length, B, b, fed);
        if (rc) return rc;
    }
    return 0;
}
// The same with the draws made here, in the reference's order, on the std::mt19937 given in its text form (updated on return); the draws are
// written out in the layout rlt_sequence_draws has, so that feeding them back reproduces the batch. env_indices is drawn too (:426).
int rlt_oracle_gather_sequence_batch_with_rng(const rlt_replay_buffer* rb, const rlt_sequence_sampling* P, int max_episode_length, const rlt_sequence_batch* B,
                                              char* rng_state, int rng_capacity, uint32_t* env_indices, uint32_t* sample_offsets, uint8_t* nominal, uint32_t* lengths) {
    if (!sequence_arguments_ok(rb, P, B) || !rng_state || !env_indices || !sample_offsets || !nominal || !lengths) return RLT_E_INVALID_ARGUMENT;
    std::mt19937 engine;
    { std::istringstream in(rng_state); in >> engine; if (in.fail()) return RLT_E_INVALID_ARGUMENT; }
    const int padded = B->sequence_length + 1;
    std::memset(sample_offsets, 0, sizeof(uint32_t) * (size_t)B->batch * padded);
    std::memset(nominal, 0, (size_t)B->batch * (padded + 1)); std::memset(lengths, 0, sizeof(uint32_t) * (size_t)B->batch * (padded + 1));
    for (int b = 0; b < B->batch; b++) {
        const uint32_t e = (uint32_t)std::uniform_int_distribution<size_t>(0, (size_t)rb->n_envs - 1)(engine);
        env_indices[b] = e;
        struct Drawn : EngineDraws { bool nominal() { const bool v = EngineDraws::nominal(); if (v) n_length++; return v; } uint32_t length() { const uint32_t v = EngineDraws::length(); n_length++; return v; } };
        Drawn drawn; drawn.engine = &engine; drawn.P = P; drawn.sequence_length = B->sequence_length; drawn.b = b; drawn.padded = padded;
        drawn.offsets = sample_offsets; drawn.nominals = nominal; drawn.lengths = lengths;
        const int rc = gather_sequence_sample(rb, e, P, max_episode_length, B, b, drawn);
        if (rc) return rc;
    }
    std::ostringstream out; out << engine;
    const std::string text = out.str();
    if ((int)text.size() + 1 > rng_capacity) return RLT_E_INVALID_ARGUMENT;
    std::memcpy(rng_state, text.c_str(), text.size() + 1);
    return 0;
}

// rl/environments/pendulum/operations_generic.h: angle_normalize, step :79-101, reward :131-139, observe :142-160.
// The literals 3.0, 0.1, 0.001 in the reference are doubles, so those sub-expressions evaluate in double (kept here).
static inline float angle_normalize(float x) { // pendulum/operations_generic.h f_mod_python + angle_normalize
    const float PI = (float)M_PI;
    float a = x + PI, b = 2 * PI;
    float m = a - b * std::floor(a / b);
    return m - PI;
}
static inline void pendulum_observe(float theta, float theta_dot, float* o) { o[0] = std::cos(theta); o[1] = std::sin(theta); o[2] = theta_dot; }
static inline void pendulum_dynamics(const rlt_pendulum_parameters* p, float theta, float theta_dot, float action, float* n_theta, float* n_theta_dot, float* reward) {
    float u_normalised = clampf(action, -1.0f, 1.0f);
    float u = p->max_torque * u_normalised;
    u = clampf(u, -p->max_torque, p->max_torque);
    float newthdot = (float)(theta_dot + (3 * p->g / (2 * p->l) * std::sin(theta) + 3.0 / (p->m * p->l * p->l) * u) * p->dt);
    newthdot = clampf(newthdot, -p->max_speed, p->max_speed);
    *n_theta = theta + newthdot * p->dt;
    *n_theta_dot = newthdot;
    float angle_norm = angle_normalize(theta);
    float ur = p->max_torque * action;    // reward uses the un-clamped action
    float costs = (float)(angle_norm * angle_norm + 0.1 * theta_dot * theta_dot + 0.001 * (ur * ur));
    *reward = -costs;
}
// rl/environments/acrobot/operations_generic.h:56-117 (dsdt, rk4), :118-144 (step), :145-171 (reward), :173-193 (observe, terminated).
// The reference writes these with T = float but with double literals (2.0, 6.0, 1.0, 0.02) and with unqualified cos / sin in dsdt and
// terminated, which resolve to the double functions; the sub-expressions they touch are evaluated in double and rounded once on assignment.
// The expressions below are typed so that the same promotions happen (bit-identical to the compiled reference on random states).
static void acrobot_dsdt(const rlt_acrobot_parameters* P, const float state[4], float action, float d_state[4]) {
    const float m1 = P->link_mass_1, m2 = P->link_mass_2, l1 = P->link_length_1, lc1 = P->link_com_pos_1, lc2 = P->link_com_pos_2, I1 = P->link_moi, I2 = P->link_moi;
    const float g = 9.8;
    const float PI = (float)M_PI;
    const float theta1 = state[0], theta2 = state[1], dtheta1 = state[2], dtheta2 = state[3];
    auto c = [](double x) { return std::cos(x); };
    auto sn = [](double x) { return std::sin(x); };
    const float d1 = m1 * lc1 * lc1 + m2 * (l1 * l1 + lc2 * lc2 + 2 * l1 * lc2 * c(theta2)) + I1 + I2;
    const float d2 = m2 * (lc2 * lc2 + l1 * lc2 * c(theta2)) + I2;
    const float phi2 = m2 * lc2 * g * c(theta1 + theta2 - PI / 2.0);
    const float phi1 = -m2 * l1 * lc2 * dtheta2 * dtheta2 * sn(theta2) - 2 * m2 * l1 * lc2 * dtheta2 * dtheta1 * sn(theta2) + (m1 * lc1 + m2 * l1) * g * c(theta1 - PI / 2) + phi2;
    const float ddtheta2 = (action + d2 / d1 * phi1 - m2 * l1 * lc2 * dtheta1 * dtheta1 * sn(theta2) - phi2) / (m2 * lc2 * lc2 + I2 - d2 * d2 / d1);
    const float ddtheta1 = -(d2 * ddtheta2 + phi1) / d1;
    d_state[0] = dtheta1; d_state[1] = dtheta2; d_state[2] = ddtheta1; d_state[3] = ddtheta2;
}
static void acrobot_rk4(const rlt_acrobot_parameters* P, const float state[4], float action, float next_state[4], float dt) {
    float k1[4], k2[4], k3[4], k4[4], y1[4], y2[4], y3[4];
    const float dt2 = dt / 2.0;
    acrobot_dsdt(P, state, action, k1);
    for (int i = 0; i < 4; i++) y1[i] = state[i] + dt2 * k1[i];
    acrobot_dsdt(P, y1, action, k2);
    for (int i = 0; i < 4; i++) y2[i] = state[i] + dt2 * k2[i];
    acrobot_dsdt(P, y2, action, k3);
    for (int i = 0; i < 4; i++) y3[i] = state[i] + dt * k3[i];
    acrobot_dsdt(P, y3, action, k4);
    for (int i = 0; i < 4; i++) next_state[i] = state[i] + dt / 6.0 * (k1[i] + 2 * k2[i] + 2 * k3[i] + k4[i]);
}
int rlt_oracle_acrobot_step(const rlt_acrobot_parameters* P, int swingup, float* states, const float* actions, float* observations, float* next_observations,
                            float* rewards, uint8_t* terminated, int n_envs) {
    if (!P || !states || !actions || n_envs <= 0) return RLT_E_INVALID_ARGUMENT;
    const float PI = (float)M_PI;
    for (int e = 0; e < n_envs; e++) {
        float* s = states + 4 * (size_t)e;
        float next[4];
        if (observations) { float* o = observations + 6 * (size_t)e; o[0] = std::cos(s[0]); o[1] = std::sin(s[0]); o[2] = std::cos(s[1]); o[3] = std::sin(s[1]); o[4] = s[2]; o[5] = s[3]; }
        const float action_clamped = clampf(actions[e], -1.0f, 1.0f);
        const float action_scaled = (action_clamped + 1.0) / 2.0 * (P->max_torque - (P->min_torque)) + (P->min_torque);
        acrobot_rk4(P, s, action_scaled, next, P->dt);
        next[0] = angle_normalize(next[0]); next[1] = angle_normalize(next[1]);
        next[2] = clampf(next[2], -P->max_vel_1, P->max_vel_1); next[3] = clampf(next[3], -P->max_vel_2, P->max_vel_2);
        if (rewards) {
            if (!swingup) rewards[e] = -1;
            else {
                const float a_angle_cost = std::fabs(angle_normalize(next[0] - PI)), b_angle_cost = std::fabs(angle_normalize(next[1]));
                rewards[e] = (-a_angle_cost - b_angle_cost) / 100 * P->dt / 0.02;
            }
        }
        if (terminated) terminated[e] = swingup ? 0 : ((-std::cos((double)next[0]) - std::cos((double)(next[1] + next[0]))) > 1.0);
        if (next_observations) { float* o = next_observations + 6 * (size_t)e; o[0] = std::cos(next[0]); o[1] = std::sin(next[0]); o[2] = std::cos(next[1]); o[3] = std::sin(next[1]); o[4] = next[2]; o[5] = next[3]; }
        for (int i = 0; i < 4; i++) s[i] = next[i];
    }
    return 0;
}

// rl/environments/car/operations_generic.h:80-84 (terminated), :99-127 (step), :128-135 (reward), :143-155 (observe). T = float; the tire
// force goes through an unqualified atan (the double function) and the reward through the double literal 0.1, kept as the C++ expression has them.
static void car_dynamics(const rlt_car_parameters& p, const float* s, const float* action, float* n) {      // step, :99-127
    const float mu = s[2], vx = s[3], vy = s[4], omega = s[5];
    const float throttle_break = clampf(action[0], -1.0f, 1.0f), delta = clampf(action[1], -1.0f, 1.0f);
    const float alpha_f = std::atan2((vy + p.lf * omega), vx) - delta;
    const float alpha_r = std::atan2((vy - p.lr * omega), vx);
    const float FnF = p.lr / (p.lf + p.lr) * p.m * p.g;
    const float FnR = p.lf / (p.lf + p.lr) * p.m * p.g;
    const float FyF = vx > p.vt || vy > p.vt ? FnF * p.tf_D * std::sin(p.tf_C * std::atan((double)(p.tf_B * (-alpha_f)))) : 0;
    const float FyR = vx > p.vt || vy > p.vt ? FnR * p.tr_D * std::sin(p.tr_C * std::atan((double)(p.tr_B * (-alpha_r)))) : 0;
    const float Fx = p.cm * throttle_break - p.cr0 - p.cr2 * vx * vx;
    for (int i = 0; i < 6; i++) n[i] = s[i];
    n[0] += p.dt * (std::cos(mu) * vx - std::sin(mu) * vy);
    n[1] += p.dt * (std::sin(mu) * vx + std::cos(mu) * vy);
    n[2] += p.dt * (omega);
    n[3] += p.dt * (1 / p.m * (Fx - FyF * std::sin(delta)) + omega * vy);
    n[4] += p.dt * (1 / p.m * (FyF * std::cos(delta) + FyR) - omega * vx);
    n[5] += p.dt * (1 / p.I * (FyF * p.lf * std::cos(delta) - FyR * p.lr));
}
int rlt_oracle_car_step(const rlt_car_parameters* P, float* states, const float* actions, float* observations, float* next_observations, float* rewards,
                        uint8_t* terminated, int n_envs) {
    if (!P || !states || !actions || n_envs <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int e = 0; e < n_envs; e++) {
        float* s = states + 6 * (size_t)e;
        const float x = s[0], y = s[1], mu = s[2];
        if (observations) for (int i = 0; i < 6; i++) observations[6 * (size_t)e + i] = s[i];
        float n[6];
        car_dynamics(*P, s, actions + 2 * (size_t)e, n);
        if (rewards) {
            const float angle_norm = angle_normalize(mu);
            const float cost = 0.1 * angle_norm * angle_norm + x * x + y * y;
            rewards[e] = std::exp(-5 * cost);
        }
        if (terminated) terminated[e] = n[0] > 1.0 || n[0] < -1.0 || n[1] > 1.0 || n[1] < -1.0;
        if (next_observations) for (int i = 0; i < 6; i++) next_observations[6 * (size_t)e + i] = n[i];
        for (int i = 0; i < 6; i++) s[i] = n[i];
    }
    return 0;
}
// CarTrack: terminated :85-98, reward :136-141, observe :156-190 (T = float, TI = size_t; the double literal 2.0 makes the cell coordinates go through
// double). Cells outside the bitmap count as not drivable; the reference's observe would read past its array there.
struct CarTrackMap { const uint8_t* track; int height, width; float scale; };
static bool car_track_cell(const CarTrackMap& M, float x_coord, float y_coord) {
    if (!(x_coord > 0 && x_coord < M.width && y_coord > 0 && y_coord < M.height)) return false;
    return M.track[(size_t)y_coord * M.width + (size_t)x_coord] != 0;
}
static void car_track_observe(const CarTrackMap& M, const float* s, float* o) {
    for (int i = 0; i < 6; i++) o[i] = s[i];
    const float PI = (float)M_PI;
    const int NUM_STEPS = 50;
    const float step_size = M.scale / 2;
    const float directions[3] = {(float)(-20 / 180.0 * PI), 0, (float)(20 / 180.0 * PI)};
    for (int d = 0; d < 3; d++) {
        const float direction_x = std::cos(s[2] + directions[d]) * step_size, direction_y = std::sin(s[2] + directions[d]) * step_size;
        float distance = NUM_STEPS * step_size;
        for (size_t step_i = 0; step_i < (size_t)NUM_STEPS; step_i++) {
            const float x_coord = (+s[0] + direction_x * step_i + M.scale * (size_t)M.width / 2.0) / ((float)M.scale);
            const float y_coord = (-s[1] - direction_y * step_i + M.scale * (size_t)M.height / 2.0) / ((float)M.scale);
            if (!car_track_cell(M, x_coord, y_coord)) { distance = step_i * step_size; break; }
        }
        o[6 + d] = distance / (NUM_STEPS * step_size);
    }
}
int rlt_oracle_car_track_step(const rlt_car_parameters* P, const uint8_t* track, int height, int width, float track_scale, float* states, const float* actions,
                              float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n_envs) {
    if (!P || !track || height < 1 || width < 1 || !(track_scale > 0) || !states || !actions || n_envs <= 0) return RLT_E_INVALID_ARGUMENT;
    const CarTrackMap M = {track, height, width, track_scale};
    for (int e = 0; e < n_envs; e++) {
        float* s = states + 6 * (size_t)e;
        if (observations) car_track_observe(M, s, observations + 9 * (size_t)e);
        float n[6];
        car_dynamics(*P, s, actions + 2 * (size_t)e, n);
        if (rewards) rewards[e] = s[3];
        if (terminated) {
            const float x_coord = (n[0] + M.scale * (size_t)width / 2.0) / ((float)M.scale), y_coord = (-n[1] + M.scale * (size_t)height / 2.0) / ((float)M.scale);
            terminated[e] = !car_track_cell(M, x_coord, y_coord);
        }
        if (next_observations) car_track_observe(M, n, next_observations + 9 * (size_t)e);
        for (int i = 0; i < 6; i++) s[i] = n[i];
    }
    return 0;
}

int rlt_oracle_pendulum_step(const rlt_pendulum_parameters* p, float* states, const float* actions, float* observations,
                             float* next_observations, float* rewards, int n_envs) {
    if (!p || !states || !actions || n_envs <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int e = 0; e < n_envs; e++) {
        float th = states[2 * e], thd = states[2 * e + 1], nth, nthd, r;
        if (observations) pendulum_observe(th, thd, observations + 3 * (size_t)e);
        pendulum_dynamics(p, th, thd, actions[e], &nth, &nthd, &r);
        if (next_observations) pendulum_observe(nth, nthd, next_observations + 3 * (size_t)e);
        if (rewards) rewards[e] = r;
        states[2 * e] = nth; states[2 * e + 1] = nthd;
    }
    return 0;
}

// prologue of the off-policy runner step (operations_generic_per_env.h:8-66): reset where truncated, mark the previous replay row truncated, observe
int rlt_oracle_pendulum_runner_prologue(const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, const float* initial_states, float* observations) {
    if (!rn || !rb || !observations || rn->n_envs != rb->n_envs || rb->observation_dim != 3 || rb->action_dim != 1) return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs, R = rb_row_dim(rb);
    for (int e = 0; e < N; e++) {
        if (rn->truncated[e]) {
            if (!initial_states) return RLT_E_INVALID_ARGUMENT;
            rn->states[2 * e] = initial_states[2 * e]; rn->states[2 * e + 1] = initial_states[2 * e + 1];
            rn->episode_step[e] = 0; rn->episode_return[e] = 0;
            if (rb->full[e] || rb->position[e] > 0) {
                uint32_t prev = rb->position[e] == 0 ? (uint32_t)rb->capacity - 1 : rb->position[e] - 1;
                rb->data[((size_t)e * rb->capacity + prev) * R + (R - 1)] = 1.0f;
                rb->current_episode_start[e] = rb->position[e];
            }
        }
        pendulum_observe(rn->states[2 * e], rn->states[2 * e + 1], observations + 3 * (size_t)e);
    }
    return 0;
}
// epilogue (operations_generic_per_env.h:67-108): step, reward, next observation, counters, truncation, replay add
int rlt_oracle_pendulum_runner_epilogue(const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, const float* observations, const float* actions) {
    if (!rn || !rb || !observations || !actions || rn->n_envs != rb->n_envs) return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs;
    std::vector<float> next_obs((size_t)N * 3), rewards(N);
    std::vector<uint8_t> term(N, 0), trunc(N, 0);
    for (int e = 0; e < N; e++) {
        float nth, nthd, r;
        pendulum_dynamics(&rn->env, rn->states[2 * e], rn->states[2 * e + 1], actions[e], &nth, &nthd, &r);
        pendulum_observe(nth, nthd, &next_obs[3 * (size_t)e]);
        rewards[e] = r;
        rn->episode_step[e] += 1; rn->episode_return[e] += r;
        trunc[e] = rn->episode_step[e] == (uint32_t)rn->episode_step_limit;
        rn->truncated[e] = trunc[e];
        rn->states[2 * e] = nth; rn->states[2 * e + 1] = nthd;
    }
    return rlt_oracle_replay_add(rb, observations, actions, rewards.data(), next_obs.data(), term.data(), trunc.data());
}

// off_policy_runner/operations_generic.h:183-238 + operations_generic_per_env.h:8-108 for Pendulum
int rlt_oracle_pendulum_runner_step(const rlt_pendulum_runner* rn, const rlt_replay_buffer* rb, int policy_kind,
                                    const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas,
                                    const float* actions_in, const float* action_noise, const float* initial_states) {
    if (!rn || !rb || rn->n_envs != rb->n_envs || rb->observation_dim != 3 || rb->action_dim != 1) return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs;
    std::vector<float> obs((size_t)N * 3), actions(N);
    int rc = rlt_oracle_pendulum_runner_prologue(rn, rb, initial_states, obs.data());
    if (rc) return rc;
    // interlude (:190-206): policy evaluate_step in Rollout mode
    if (policy_kind == 0) { if (!actions_in) return RLT_E_INVALID_ARGUMENT; for (int e = 0; e < N; e++) actions[e] = actions_in[e]; }
    else if (policy_kind == 1) { rc = rlt_oracle_mlp_evaluate(actor, n_actor_layers, obs.data(), 3, actions.data(), 1, N); }
    else if (policy_kind == 2) {
        std::vector<float> out((size_t)N * 2), lp(N);
        rc = rlt_oracle_mlp_evaluate(actor, n_actor_layers, obs.data(), 3, out.data(), 2, N);
        if (!rc) rc = rlt_oracle_sas_forward(sas, out.data(), 2, action_noise, 1, actions.data(), 1, nullptr, 0, lp.data(), N, 1);
    } else return RLT_E_INVALID_ARGUMENT;
    if (rc) return rc;
    return rlt_oracle_pendulum_runner_epilogue(rn, rb, obs.data(), actions.data());
}

// The Tensor elementwise operations (containers/tensor/operations_generic.h:365-481 functors, :573-760 operations) on 2-D views
static inline float fast_tanh_elementwise(float x) { x = std::min(std::max(x, -3.0f), 3.0f); const float x2 = x * x; return x * (27.0f + x2) / (27.0f + 9.0f * x2); }   // math/operations_generic.h:247-251
int rlt_oracle_unary_f32(int operation, float parameter, const float* src, int ld_src, float* dst, int ld_dst, int rows, int cols) {
    if (!src || !dst || rows <= 0 || cols <= 0 || operation < RLT_UNARY_NEGATE || operation > RLT_UNARY_SCALE_RECIPROCAL) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            const float a = src[(size_t)r * ld_src + c];
            float v = a;
            switch (operation) {
                case RLT_UNARY_NEGATE: v = -a; break;
                case RLT_UNARY_ABS: v = std::fabs(a); break;
                case RLT_UNARY_CONSTANT: v = parameter; break;
                case RLT_UNARY_SIGMOID: v = a < -20 ? 0.0f : (a > 20 ? 1.0f : 1 / (1 + std::exp(-a))); break;       // :395-400
                case RLT_UNARY_FAST_SIGMOID: v = 0.5f * fast_tanh_elementwise(0.5f * a) + 0.5f; break;                  // math/operations_generic.h:252-255
                case RLT_UNARY_EXP: v = std::exp(a); break;
                case RLT_UNARY_TANH: v = std::tanh(a); break;
                case RLT_UNARY_FAST_TANH: v = fast_tanh_elementwise(a); break;
                case RLT_UNARY_ONE_MINUS: v = 1 - a; break;
                case RLT_UNARY_SCALE: v = a * parameter; break;
                case RLT_UNARY_SCALE_RECIPROCAL: v = 1.0f / a * parameter; break;                                       // :436-441
            }
            dst[(size_t)r * ld_dst + c] = v;
        }
    return 0;
}
int rlt_oracle_binary_f32(int operation, const float* a, int lda, const float* b, int ldb, float* dst, int ld_dst, int rows, int cols) {
    if (!a || !b || !dst || rows <= 0 || cols <= 0 || operation < RLT_BINARY_ADD || operation > RLT_BINARY_DIVIDE) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            const float x = a[(size_t)r * lda + c], y = b[(size_t)r * ldb + c];
            dst[(size_t)r * ld_dst + c] = operation == RLT_BINARY_ADD ? x + y : operation == RLT_BINARY_SUBTRACT ? x - y : operation == RLT_BINARY_MULTIPLY ? x * y : x / y;
        }
    return 0;
}
int rlt_oracle_multiply_accumulate_f32(const float* a, int lda, const float* b, int ldb, const float* accumulator, int ldc, float* dst, int ld_dst, int rows, int cols) {
    if (!a || !b || !accumulator || !dst || rows <= 0 || cols <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            volatile float product = a[(size_t)r * lda + c] * b[(size_t)r * ldb + c];      // rounded before the addition
            dst[(size_t)r * ld_dst + c] = accumulator[(size_t)r * ldc + c] + product;
        }
    return 0;
}
int rlt_oracle_reduce_abs_max_f32(const float* x, size_t count, float* out_max) {
    if (!x || !out_max) return RLT_E_INVALID_ARGUMENT;
    float m = 0;
    for (size_t i = 0; i < count; i++) m = std::max(m, std::fabs(x[i]));
    *out_max = m;
    return 0;
}

// step<POLICY>(device, runner, policy, ...) for any of the environments restated here: rl/components/off_policy_runner/operations_generic.h:183-238 over
// prologue_per_env / epilogue_per_env (operations_generic_per_env.h:8-108). The environment-independent part (reset bookkeeping, counters,
// truncated = terminated or step limit, replay add) is the Pendulum runner's, which the seeded SAC loop pins against the reference; the
// environments' own step / reward / observe / terminated are the functions above, pinned one by one.
static int env_dims_of(int kind, int* state, int* obs, int* act) {
    switch (kind) {
        case RLT_ENV_PENDULUM: *state = 2; *obs = 3; *act = 1; return 0;
        case RLT_ENV_ACROBOT: case RLT_ENV_ACROBOT_SWINGUP: *state = 4; *obs = 6; *act = 1; return 0;
        case RLT_ENV_CAR: *state = 6; *obs = 6; *act = 2; return 0;
        case RLT_ENV_PENDULUM_POSITION: *state = 3; *obs = 2; *act = 1; return 0;
        default: return RLT_E_INVALID_ARGUMENT;
    }
}
static int env_step_of(const rlt_env_runner* rn, float* states, const float* actions, float* observations, float* next_observations, float* rewards, uint8_t* terminated) {
    const int N = rn->n_envs;
    switch (rn->env_kind) {
        case RLT_ENV_PENDULUM: {
            if (terminated) for (int e = 0; e < N; e++) terminated[e] = 0;
            return rlt_oracle_pendulum_step(&rn->pendulum, states, actions, observations, next_observations, rewards, N);
        }
        case RLT_ENV_PENDULUM_POSITION: {
            // rl/environments/pendulum/pendulum.h:117-124: the Pendulum's dynamics and reward (the step above on the first two state entries), the observation's
            // first two entries (operations_generic.h:168-181 with zero observation noise), and the action remembered in the state (:102-108)
            std::vector<float> s2((size_t)N * 2), o3((size_t)N * 3), n3((size_t)N * 3);
            for (int e = 0; e < N; e++) { s2[2 * e] = states[3 * e]; s2[2 * e + 1] = states[3 * e + 1]; }
            const int rc = rlt_oracle_pendulum_step(&rn->pendulum, s2.data(), actions, o3.data(), n3.data(), rewards, N);
            if (rc) return rc;
            for (int e = 0; e < N; e++) {
                states[3 * e] = s2[2 * e]; states[3 * e + 1] = s2[2 * e + 1]; states[3 * e + 2] = actions[e];
                if (observations) { observations[2 * e] = o3[3 * e]; observations[2 * e + 1] = o3[3 * e + 1]; }
                if (next_observations) { next_observations[2 * e] = n3[3 * e]; next_observations[2 * e + 1] = n3[3 * e + 1]; }
                if (terminated) terminated[e] = 0;
            }
            return 0;
        }
        case RLT_ENV_CAR: return rlt_oracle_car_step(&rn->car, states, actions, observations, next_observations, rewards, terminated, N);
        default: return rlt_oracle_acrobot_step(&rn->acrobot, rn->env_kind == RLT_ENV_ACROBOT_SWINGUP, states, actions, observations, next_observations, rewards, terminated, N);
    }
}
int rlt_oracle_env_runner_step(const rlt_env_runner* rn, const rlt_replay_buffer* rb, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers,
                               const rlt_sas_parameters* sas, const float* actions_in, const float* action_noise, const float* initial_states) {
    int SD, OBS, ACT;
    if (!rn || !rb || !initial_states || env_dims_of(rn->env_kind, &SD, &OBS, &ACT) || rn->n_envs != rb->n_envs || rb->observation_dim != OBS || rb->action_dim != ACT)
        return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs, R = rb_row_dim(rb);
    // prologue
    for (int e = 0; e < N; e++)
        if (rn->truncated[e]) {
            for (int i = 0; i < SD; i++) rn->states[(size_t)e * SD + i] = initial_states[(size_t)e * SD + i];
            rn->episode_step[e] = 0; rn->episode_return[e] = 0;
            if (rb->full[e] || rb->position[e] > 0) {
                const uint32_t prev = rb->position[e] == 0 ? (uint32_t)rb->capacity - 1 : rb->position[e] - 1;
                rb->data[((size_t)e * rb->capacity + prev) * R + (R - 1)] = 1.0f;
                rb->current_episode_start[e] = rb->position[e];
            }
        }
    {   // observe: the environment's own step function on a copy of the states yields the observation of the state it was given
        std::vector<float> scratch_states(rn->states, rn->states + (size_t)N * SD), zero_actions((size_t)N * ACT, 0.0f);
        int rc = env_step_of(rn, scratch_states.data(), zero_actions.data(), rn->observations, nullptr, nullptr, nullptr);
        if (rc) return rc;
    }
    // interlude
    int rc = 0;
    if (policy_kind == 0) { if (!actions_in) return RLT_E_INVALID_ARGUMENT; for (size_t i = 0; i < (size_t)N * ACT; i++) rn->actions[i] = actions_in[i]; }
    else if (policy_kind == 1) rc = rlt_oracle_mlp_evaluate(actor, n_actor_layers, rn->observations, OBS, rn->actions, ACT, N);
    else if (policy_kind == 2) {
        std::vector<float> out((size_t)N * 2 * ACT), lp(N);
        rc = rlt_oracle_mlp_evaluate(actor, n_actor_layers, rn->observations, OBS, out.data(), 2 * ACT, N);
        if (!rc) rc = rlt_oracle_sas_forward(sas, out.data(), 2 * ACT, action_noise, ACT, rn->actions, ACT, nullptr, 0, lp.data(), N, ACT);
    } else return RLT_E_INVALID_ARGUMENT;
    if (rc) return rc;
    // epilogue
    if ((rc = env_step_of(rn, rn->states, rn->actions, nullptr, rn->next_observations, rn->rewards, rn->terminated))) return rc;
    std::vector<uint8_t> trunc(N, 0);
    for (int e = 0; e < N; e++) {
        rn->episode_step[e] += 1; rn->episode_return[e] += rn->rewards[e];
        trunc[e] = rn->terminated[e] || rn->episode_step[e] == (uint32_t)rn->episode_step_limit;
        rn->truncated[e] = trunc[e];
    }
    return rlt_oracle_replay_add(rb, rn->observations, rn->actions, rn->rewards, rn->next_observations, rn->terminated, trunc.data());
}

// rl::utils::evaluation::evaluate (rl/utils/evaluation/operations_generic.h:106-233) with the Pendulum environment: n_episodes environments from the
// given initial states (what sample_initial_state drew, :139-142), step_limit steps of observe -> policy in Evaluation mode -> step -> reward;
// an episode stops counting once it has terminated (:188-197; Pendulum never terminates, pendulum/operations_generic.h:161-164). The statistics
// are accumulated in float in episode order (:213-227).
//   policy_kind 1: the actor's output is the action;  2: the actor's output is [mean | log_std] and the action is tanh(mean), which is what
//   sample_and_squash yields in Evaluation mode (noise = 0, nn/layers/sample_and_squash/operations_generic.h:149-195)
//   summary = {returns_mean, returns_std, episode_length_mean, episode_length_std, num_terminated, share_terminated}
// the same runner step with a sequential policy and its rollout state (rl/components/off_policy_runner/operations_generic.h:189-206: reset of the policy state
// under the truncated mask after the prologue, evaluate_step in Rollout mode) and the policy's last layer: 1 none, 2 sample_and_squash, 3 td3_sampling
int rlt_oracle_env_runner_step_sequential(const rlt_env_runner* rn, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n_policy_layers,
                                          const rlt_seq_state* policy_state, int auto_reset_period, int head_kind, const rlt_sas_parameters* sas, float exploration_noise_std,
                                          const float* action_noise, const float* initial_states) {
    int SD, OBS, ACT;
    if (!rn || !rb || !policy || !initial_states || env_dims_of(rn->env_kind, &SD, &OBS, &ACT) || rn->n_envs != rb->n_envs || rb->observation_dim != OBS || rb->action_dim != ACT)
        return RLT_E_INVALID_ARGUMENT;
    if (head_kind < 1 || head_kind > 3 || (head_kind != 1 && !action_noise) || (head_kind == 2 && !sas)) return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs, R = rb_row_dim(rb);
    for (int e = 0; e < N; e++)
        if (rn->truncated[e]) {
            for (int i = 0; i < SD; i++) rn->states[(size_t)e * SD + i] = initial_states[(size_t)e * SD + i];
            rn->episode_step[e] = 0; rn->episode_return[e] = 0;
            if (rb->full[e] || rb->position[e] > 0) {
                const uint32_t prev = rb->position[e] == 0 ? (uint32_t)rb->capacity - 1 : rb->position[e] - 1;
                rb->data[((size_t)e * rb->capacity + prev) * R + (R - 1)] = 1.0f;
                rb->current_episode_start[e] = rb->position[e];
            }
        }
    int rc;
    {
        std::vector<float> scratch_states(rn->states, rn->states + (size_t)N * SD), zero_actions((size_t)N * ACT, 0.0f);
        if ((rc = env_step_of(rn, scratch_states.data(), zero_actions.data(), rn->observations, nullptr, nullptr, nullptr))) return rc;
    }
    const rlt_seq_state no_state = {};
    if (policy_state && (rc = rlt_oracle_seq_reset_state(policy, n_policy_layers, policy_state, rn->truncated, N))) return rc;
    const int out_dim = (head_kind == 2 ? 2 : 1) * ACT;
    std::vector<float> out((size_t)N * out_dim), lp(N);
    if ((rc = rlt_oracle_seq_evaluate_step(policy, n_policy_layers, rn->observations, OBS, policy_state ? policy_state : &no_state, auto_reset_period, out.data(), out_dim, N))) return rc;
    if (head_kind == 1) std::copy(out.begin(), out.end(), rn->actions);
    else if (head_kind == 2) rc = rlt_oracle_sas_forward(sas, out.data(), 2 * ACT, action_noise, ACT, rn->actions, ACT, nullptr, 0, lp.data(), N, ACT);
    else rc = rlt_oracle_td3_sampling_forward(out.data(), ACT, action_noise, ACT, exploration_noise_std, nullptr, 0, rn->actions, ACT, N, ACT);
    if (rc) return rc;
    if ((rc = env_step_of(rn, rn->states, rn->actions, nullptr, rn->next_observations, rn->rewards, rn->terminated))) return rc;
    std::vector<uint8_t> trunc(N, 0);
    for (int e = 0; e < N; e++) {
        rn->episode_step[e] += 1; rn->episode_return[e] += rn->rewards[e];
        trunc[e] = rn->terminated[e] || rn->episode_step[e] == (uint32_t)rn->episode_step_limit;
        rn->truncated[e] = trunc[e];
    }
    return rlt_oracle_replay_add(rb, rn->observations, rn->actions, rn->rewards, rn->next_observations, rn->terminated, trunc.data());
}

// collect for any of the environments restated here and any sequential policy: rl/components/on_policy_runner/operations_generic.h:105-146 over
// operations_generic_per_env.h:8-74 (see on_policy_collect_impl further down for the Pendulum / MLP case, which the reference's PPO loop pins)
int rlt_oracle_env_on_policy_collect(const rlt_env_runner* rn, const rlt_on_policy_dataset* D, const rlt_seq_layer* policy, int n_policy_layers,
                                     const rlt_seq_state* policy_state, int auto_reset_period, const float* log_std, const float* st_mean, const float* st_precision,
                                     const float* action_noise, const float* initial_states, int truncate_on_each_iteration) {
    int SD, OBS, ACT;
    if (!rn || !D || !policy || n_policy_layers < 1 || !log_std || !action_noise || !initial_states || env_dims_of(rn->env_kind, &SD, &OBS, &ACT)) return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs, S = D->steps_per_env, ld = D->ld;
    const rlt_seq_state no_state = {};
    const rlt_seq_state* step_state = policy_state ? policy_state : &no_state;
    if (truncate_on_each_iteration) for (int e = 0; e < N; e++) rn->truncated[e] = 1;                                           // :112-114
    for (int e = 0; e < N; e++) D->all_reset[(size_t)e * ld] = rn->truncated[e];                                                  // :115-117
    std::vector<float> standardized((size_t)N * OBS), packed_obs((size_t)N * OBS), scratch_states((size_t)N * SD), zero_actions((size_t)N * ACT, 0.0f);
    auto observe_into = [&](float* rows) {      // the environment's own step function on a copy of the states yields the observation of the state it was given
        std::copy(rn->states, rn->states + (size_t)N * SD, scratch_states.begin());
        int rc = env_step_of(rn, scratch_states.data(), zero_actions.data(), packed_obs.data(), nullptr, nullptr, nullptr);
        for (int e = 0; e < N && !rc; e++) for (int i = 0; i < OBS; i++) rows[(size_t)e * ld + i] = packed_obs[(size_t)e * OBS + i];
        return rc;
    };
    int rc;
    for (int step = 0; step < S; step++) {
        float* obs = D->observations + (size_t)step * N * ld;
        float* means = D->actions_mean + (size_t)step * N * ld;
        float* actions = D->actions + (size_t)step * N * ld;
        if (policy_state && (rc = rlt_oracle_seq_reset_state(policy, n_policy_layers, policy_state, rn->truncated, N))) return rc;     // :127-130, before the prologue clears the flags
        for (int e = 0; e < N; e++)                                                                                            // prologue, per_env :8-35
            if (rn->truncated[e]) {
                rn->truncated[e] = 0; rn->episode_step[e] = 0; rn->episode_return[e] = 0;
                for (int i = 0; i < SD; i++) rn->states[(size_t)e * SD + i] = initial_states[((size_t)step * N + e) * SD + i];
            }
        if ((rc = observe_into(obs))) return rc;
        if (st_mean) {
            if ((rc = rlt_oracle_standardize_forward(st_mean, st_precision, obs, ld, standardized.data(), OBS, N, OBS))) return rc;
            if ((rc = rlt_oracle_seq_evaluate_step(policy, n_policy_layers, standardized.data(), OBS, step_state, auto_reset_period, means, ld, N))) return rc;
        } else if ((rc = rlt_oracle_seq_evaluate_step(policy, n_policy_layers, obs, ld, step_state, auto_reset_period, means, ld, N))) return rc;
        for (int e = 0; e < N; e++) {                                                                                          // epilogue, per_env :37-58
            const size_t pos = (size_t)step * N + e;
            float log_prob = 0;
            for (int a = 0; a < ACT; a++) {
                const float mean = means[(size_t)e * ld + a];
                const float noisy = action_noise[pos * ACT + a] * std::exp(log_std[a]) + mean;
                log_prob += normal_log_prob(mean, log_std[a], noisy);
                actions[(size_t)e * ld + a] = noisy;
                rn->actions[(size_t)e * ACT + a] = noisy;
            }
            D->action_log_probs[pos * ld] = log_prob;
        }
        if ((rc = env_step_of(rn, rn->states, rn->actions, nullptr, nullptr, rn->rewards, rn->terminated))) return rc;
        for (int e = 0; e < N; e++) {                                                                                          // :59-74
            const size_t pos = (size_t)step * N + e;
            D->terminated[pos * ld] = rn->terminated[e] ? 1.0f : 0.0f;
            rn->episode_return[e] += rn->rewards[e];
            D->rewards[pos * ld] = rn->rewards[e];
            rn->episode_step[e] += 1;
            const bool truncated = rn->terminated[e] || (rn->episode_step_limit > 0 && rn->episode_step[e] >= (uint32_t)rn->episode_step_limit);
            D->truncated[pos * ld] = truncated;
            D->all_reset[(pos + N) * ld] = truncated;
            rn->truncated[e] = truncated;
        }
    }
    return observe_into(D->observations + (size_t)S * N * ld);                                                                   // :137-144
}

}  // extern "C"
template <typename POLICY>
static int pendulum_evaluate_impl(const rlt_pendulum_parameters* env, int policy_kind, POLICY&& policy, const float* initial_states,
                                  int n_episodes, int step_limit, float* returns, uint32_t* episode_length, float* summary) {
    const int N = n_episodes, out_dim = policy_kind;
    std::vector<float> states(initial_states, initial_states + 2 * (size_t)N), obs((size_t)N * 3), out((size_t)N * out_dim);
    std::vector<uint8_t> terminated(N, 0);
    uint32_t num_terminated = 0;
    for (int e = 0; e < N; e++) { returns[e] = 0; episode_length[e] = 0; }
    for (int step = 0; step < step_limit; step++) {
        for (int e = 0; e < N; e++) pendulum_observe(states[2 * e], states[2 * e + 1], &obs[3 * (size_t)e]);
        const int rc = policy(obs.data(), out.data());
        if (rc) return rc;
        for (int e = 0; e < N; e++) {
            if (step > 0 && terminated[e]) continue;
            const float action = policy_kind == 1 ? out[e] : std::tanh(out[2 * (size_t)e]);
            float nth, nthd, r;
            pendulum_dynamics(env, states[2 * e], states[2 * e + 1], action, &nth, &nthd, &r);
            const bool terminated_flag = false;      // the Pendulum has no terminal states
            if (!terminated[e]) { returns[e] += r; episode_length[e] += 1; num_terminated += terminated_flag ? 1 : 0; }
            terminated[e] = terminated_flag || terminated[e];
            states[2 * e] = nth; states[2 * e + 1] = nthd;
        }
    }
    float rm = 0, rs = 0, lm = 0, ls = 0;
    for (int e = 0; e < N; e++) { rm += returns[e]; rs += returns[e] * returns[e]; lm += (float)episode_length[e]; ls += (float)(episode_length[e] * episode_length[e]); }
    rm /= N; lm /= N;
    summary[0] = rm; summary[1] = std::sqrt(std::max(0.0f, rs / N - rm * rm));
    summary[2] = lm; summary[3] = std::sqrt(std::max(0.0f, ls / N - lm * lm));
    summary[4] = (float)num_terminated; summary[5] = num_terminated / (float)N;
    return 0;
}
extern "C" {

int rlt_oracle_pendulum_evaluate(const rlt_pendulum_parameters* env, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers, const float* initial_states,
                                 int n_episodes, int step_limit, float* returns, uint32_t* episode_length, float* summary) {
    if (!env || !actor || n_actor_layers < 1 || !initial_states || n_episodes < 1 || step_limit < 1 || !returns || !episode_length || !summary) return RLT_E_INVALID_ARGUMENT;
    if (policy_kind != 1 && policy_kind != 2) return RLT_E_INVALID_ARGUMENT;
    if (actor[0].in_dim != 3 || actor[n_actor_layers - 1].out_dim != policy_kind) return RLT_E_INVALID_ARGUMENT;
    return pendulum_evaluate_impl(env, policy_kind, [&](const float* obs, float* out) { return rlt_oracle_mlp_evaluate(actor, n_actor_layers, obs, 3, out, policy_kind, n_episodes); },
                                  initial_states, n_episodes, step_limit, returns, episode_length, summary);
}

// with a standardize layer in front of the actor (nn/layers/standardize/operations_generic.h:69-135: output = (input - mean) * precision)
int rlt_oracle_pendulum_evaluate_standardized(const rlt_pendulum_parameters* env, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers, const float* observation_mean,
                                              const float* observation_precision, const float* initial_states, int n_episodes, int step_limit, float* returns,
                                              uint32_t* episode_length, float* summary) {
    if (!env || !actor || n_actor_layers < 1 || !initial_states || n_episodes < 1 || step_limit < 1 || !returns || !episode_length || !summary) return RLT_E_INVALID_ARGUMENT;
    if (policy_kind != 1 && policy_kind != 2) return RLT_E_INVALID_ARGUMENT;
    if (actor[0].in_dim != 3 || actor[n_actor_layers - 1].out_dim != policy_kind || !observation_mean || !observation_precision) return RLT_E_INVALID_ARGUMENT;
    std::vector<float> standardized((size_t)n_episodes * 3);
    return pendulum_evaluate_impl(env, policy_kind, [&](const float* obs, float* out) {
        for (int e = 0; e < n_episodes; e++)
            for (int i = 0; i < 3; i++) standardized[(size_t)e * 3 + i] = (obs[(size_t)e * 3 + i] - observation_mean[i]) * observation_precision[i];
        return rlt_oracle_mlp_evaluate(actor, n_actor_layers, standardized.data(), 3, out, policy_kind, n_episodes); },
                                  initial_states, n_episodes, step_limit, returns, episode_length, summary);
}

// The same evaluation with a sequential (recurrent) policy: its kept state is reset for every episode before the first step (:135) and every step goes through
// evaluate_step (:163), whose GRU layers restart their hidden state by themselves every auto_reset_period steps (nn/layers/gru/operations_generic.h:406-413;
// 0: never). Terminated episodes keep being fed to the policy (:155-163), only their environment stops (:166-170).
int rlt_oracle_pendulum_evaluate_recurrent(const rlt_pendulum_parameters* env, int policy_kind, const rlt_seq_layer* policy, int n_layers, const rlt_seq_state* state,
                                           int auto_reset_period, const float* initial_states, int n_episodes, int step_limit, float* returns, uint32_t* episode_length,
                                           float* summary) {
    if (!env || !policy || n_layers < 1 || !state || !initial_states || n_episodes < 1 || step_limit < 1 || !returns || !episode_length || !summary) return RLT_E_INVALID_ARGUMENT;
    if (policy_kind != 1 && policy_kind != 2) return RLT_E_INVALID_ARGUMENT;
    const int rc = rlt_oracle_seq_reset_state(policy, n_layers, state, nullptr, n_episodes);
    if (rc) return rc;
    return pendulum_evaluate_impl(env, policy_kind, [&](const float* obs, float* out) {
        return rlt_oracle_seq_evaluate_step(policy, n_layers, obs, 3, state, auto_reset_period, out, policy_kind, n_episodes); },
                                  initial_states, n_episodes, step_limit, returns, episode_length, summary);
}

// rl::utils::evaluation::evaluate over any of the environments restated here (rl/utils/evaluation/operations_generic.h:113-233): the loop of
// pendulum_evaluate_impl with the environment's own step / reward / terminated (pinned one by one above) and the terminated bookkeeping that the Pendulum
// never reaches: an episode that has terminated is skipped from then on, its state stays (:166-170), the step that terminates it still counts (:187-192).
int rlt_oracle_env_evaluate(const rlt_env_runner* env, int policy_kind, const rlt_seq_layer* policy, int n_layers, const rlt_seq_state* state, int auto_reset_period,
                            const float* observation_mean, const float* observation_precision, const float* initial_states, int n_episodes, int step_limit, float* returns,
                            uint32_t* episode_length, float* summary) {
    int SD, OBS, ACT;
    if (!env || !policy || n_layers < 1 || !initial_states || n_episodes < 1 || step_limit < 1 || !returns || !episode_length || !summary) return RLT_E_INVALID_ARGUMENT;
    if ((policy_kind != 1 && policy_kind != 2) || env_dims_of(env->env_kind, &SD, &OBS, &ACT) || (observation_mean == nullptr) != (observation_precision == nullptr))
        return RLT_E_INVALID_ARGUMENT;
    const int N = n_episodes, out_dim = policy_kind * ACT;
    int rc;
    const rlt_seq_state no_state = {};
    if (state && (rc = rlt_oracle_seq_reset_state(policy, n_layers, state, nullptr, N))) return rc;
    std::vector<float> states(initial_states, initial_states + (size_t)N * SD), obs((size_t)N * OBS), out((size_t)N * out_dim), action(ACT);
    std::vector<uint8_t> terminated(N, 0);
    uint32_t num_terminated = 0;
    rlt_env_runner all = *env; all.n_envs = N;
    rlt_env_runner one = *env; one.n_envs = 1;
    for (int e = 0; e < N; e++) { returns[e] = 0; episode_length[e] = 0; }
    for (int step = 0; step < step_limit; step++) {
        {   // observe: the environment's own step function on a copy of the states yields the observation of the state it was given
            std::vector<float> scratch_states(states), zero_actions((size_t)N * ACT, 0.0f);
            if ((rc = env_step_of(&all, scratch_states.data(), zero_actions.data(), obs.data(), nullptr, nullptr, nullptr))) return rc;
        }
        if (observation_mean)
            for (int e = 0; e < N; e++)
                for (int i = 0; i < OBS; i++) obs[(size_t)e * OBS + i] = (obs[(size_t)e * OBS + i] - observation_mean[i]) * observation_precision[i];
        if ((rc = rlt_oracle_seq_evaluate_step(policy, n_layers, obs.data(), OBS, state ? state : &no_state, auto_reset_period, out.data(), out_dim, N))) return rc;
        for (int e = 0; e < N; e++) {
            if (step > 0 && terminated[e]) continue;
            for (int a = 0; a < ACT; a++) action[a] = policy_kind == 1 ? out[(size_t)e * out_dim + a] : std::tanh(out[(size_t)e * out_dim + a]);
            float r; uint8_t t;
            if ((rc = env_step_of(&one, &states[(size_t)e * SD], action.data(), nullptr, nullptr, &r, &t))) return rc;
            if (!terminated[e]) { returns[e] += r; episode_length[e] += 1; num_terminated += t ? 1 : 0; }
            terminated[e] = t || terminated[e];
        }
    }
    float rm = 0, rs = 0, lm = 0, ls = 0;
    for (int e = 0; e < N; e++) { rm += returns[e]; rs += returns[e] * returns[e]; lm += (float)episode_length[e]; ls += (float)(episode_length[e] * episode_length[e]); }
    rm /= N; lm /= N;
    summary[0] = rm; summary[1] = std::sqrt(std::max(0.0f, rs / N - rm * rm));
    summary[2] = lm; summary[3] = std::sqrt(std::max(0.0f, ls / N - lm * lm));
    summary[4] = (float)num_terminated; summary[5] = num_terminated / (float)N;
    return 0;
}

// rl/algorithms/ppo/operations_generic.h:60-95
int rlt_oracle_ppo_gae(const float* rewards, const float* terminated, const float* truncated, const float* all_values,
                       float* advantages, float* target_values, int ld, int n_envs, int steps, float gamma, float lambda,
                       int ignore_termination) {
    if (!rewards || !terminated || !truncated || !all_values || !advantages || !target_values || ld < 1 || n_envs <= 0 || steps <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int env = 0; env < n_envs; env++) {
        float previous_value = all_values[((size_t)steps * n_envs + env) * ld];
        float previous_advantage = 0;
        for (int sf = 0; sf < steps; sf++) {
            int sb = steps - 1 - sf;
            size_t pos = ((size_t)sb * n_envs + env) * ld;
            bool term = terminated[pos] != 0.0f, trunc = truncated[pos] != 0.0f;
            float current_step_value = all_values[pos];
            bool terminated_actual = term && !ignore_termination;
            float next_step_value = terminated_actual ? 0 : previous_value;
            float td_error = rewards[pos] + gamma * next_step_value - current_step_value;
            if (trunc) { if (!term) td_error = 0; previous_advantage = 0; }
            float advantage = lambda * gamma * previous_advantage + td_error;
            advantages[pos] = advantage;
            target_values[pos] = advantage + current_step_value;
            previous_advantage = advantage;
            previous_value = current_step_value;
        }
    }
    return 0;
}

// rl/algorithms/ppo/operations_generic.h:170-269 with ADAPTIVE_LEARNING_RATE off; operation order and float/double promotion as there
int rlt_oracle_ppo_surrogate_gradient(const float* action_means, int ld_means, const float* log_std, const float* actions, int ld_actions,
                                      const float* action_log_probs, int ld_log_probs, const float* advantages, int ld_advantages,
                                      const rlt_ppo_parameters* P, float* d_action_means, int ld_d, float* d_log_std, int batch, int action_dim) {
    if (!action_means || !log_std || !actions || !action_log_probs || !advantages || !P || !d_action_means || batch <= 0 || action_dim <= 0) return RLT_E_INVALID_ARGUMENT;
    if (P->learn_action_std && !d_log_std) return RLT_E_INVALID_ARGUMENT;
    const size_t BATCH_SIZE = (size_t)batch;
    float advantage_mean = 0, advantage_std = 0;
    if (P->normalize_advantage) {                                                                       // :170-180
        for (int b = 0; b < batch; b++) {
            float advantage = advantages[(size_t)b * ld_advantages];
            advantage_mean += advantage;
            advantage_std += advantage * advantage;
        }
        advantage_mean /= BATCH_SIZE;
        advantage_std /= BATCH_SIZE;
        advantage_std = std::sqrt(std::max((float)0, advantage_std - advantage_mean * advantage_mean));
    }
    std::vector<float> d_lp_d_ls((size_t)action_dim);
    for (int b = 0; b < batch; b++) {                                                                   // :205-269
        float action_log_prob = 0;
        for (int a = 0; a < action_dim; a++) {
            float current_action = action_means[(size_t)b * ld_means + a];
            float rollout_action = actions[(size_t)b * ld_actions + a];
            float current_action_log_std = log_std[a];
            action_log_prob += normal_log_prob(current_action, current_action_log_std, rollout_action);
            d_action_means[(size_t)b * ld_d + a] = normal_d_log_prob_d_mean(current_action, current_action_log_std, rollout_action);
            if (P->learn_action_std) {
                float d_entropy_loss_d_current_action_log_std = -(float)1 / BATCH_SIZE * P->action_entropy_coefficient;
                d_log_std[a] += d_entropy_loss_d_current_action_log_std;
                float diff = rollout_action - current_action;                                           // random/operations_generic.h:90-97
                float sd = std::exp(current_action_log_std);
                float pre_square = diff / sd;
                d_lp_d_ls[a] = -1 + pre_square * pre_square;
            }
        }
        float rollout_action_log_prob = action_log_probs[(size_t)b * ld_log_probs];
        float advantage = advantages[(size_t)b * ld_advantages];
        if (P->normalize_advantage) advantage = (advantage - advantage_mean) / (advantage_std + P->advantage_epsilon);
        float log_ratio = action_log_prob - rollout_action_log_prob;
        float ratio = std::exp(log_ratio);
        float clipped_ratio = std::clamp(ratio, 1 - P->epsilon_clip, 1 + P->epsilon_clip);
        bool clipped = ratio != clipped_ratio;
        float normal_advantage = ratio * advantage;
        float clipped_advantage = clipped_ratio * advantage;
        float slippage = 0.0;
        bool ratio_min_switch = normal_advantage - clipped_advantage <= slippage;
        float d_loss_d_pessimistic_surrogate = -(float)1 / BATCH_SIZE;
        float d_pessimistic_surrogate_d_normal_advantage = ratio_min_switch ? 1 : 0;
        float d_pessimistic_surrogate_d_clipped_advantage = ratio_min_switch ? 0 : 1;
        float d_normal_advantage_d_ratio = advantage;
        float d_clipped_advantage_d_clipped_ratio = advantage;
        float d_clipped_ratio_d_ratio = clipped ? 0 : 1;
        float d_pessimistic_surrogate_d_ratio = d_pessimistic_surrogate_d_normal_advantage * d_normal_advantage_d_ratio +
                                                d_pessimistic_surrogate_d_clipped_advantage * d_clipped_advantage_d_clipped_ratio * d_clipped_ratio_d_ratio;
        float d_loss_d_ratio = d_loss_d_pessimistic_surrogate * d_pessimistic_surrogate_d_ratio;
        float d_ratio_d_action_log_prob = ratio;
        float d_loss_d_action_log_prob = d_loss_d_ratio * d_ratio_d_action_log_prob;
        for (int a = 0; a < action_dim; a++) {
            d_action_means[(size_t)b * ld_d + a] *= d_loss_d_action_log_prob;
            if (P->learn_action_std) d_log_std[a] += d_loss_d_action_log_prob * d_lp_d_ls[a];
        }
    }
    return 0;
}

// body of the batch loop, rl/algorithms/ppo/operations_generic.h:156-318
int rlt_oracle_ppo_train_minibatch(const rlt_ppo_agent* A, const rlt_ppo_parameters* P, const float* observations, const float* observations_privileged,
                                   const float* actions, const float* action_log_probs, const float* advantages, const float* target_values, int ld,
                                   const uint32_t* row_indices, float* out_critic_loss) {
    if (!A || !P || !observations || !observations_privileged || !actions || !action_log_probs || !advantages || !target_values || ld < 1) return RLT_E_INVALID_ARGUMENT;
    const int B = A->batch, O = A->observation_dim, OP = A->observation_privileged_dim, AD = A->action_dim;
    std::vector<float> obs((size_t)B * O), obsp((size_t)B * OP), act((size_t)B * AD), lp(B), adv(B), tgt(B), d_act((size_t)B * AD), d_crit(B);
    for (int b = 0; b < B; b++) {
        const size_t row = row_indices ? row_indices[b] : (size_t)b;
        std::memcpy(&obs[(size_t)b * O], observations + row * ld, sizeof(float) * O);
        std::memcpy(&obsp[(size_t)b * OP], observations_privileged + row * ld, sizeof(float) * OP);
        std::memcpy(&act[(size_t)b * AD], actions + row * ld, sizeof(float) * AD);
        lp[b] = action_log_probs[row * ld]; adv[b] = advantages[row * ld]; tgt[b] = target_values[row * ld];
    }
    // the optional standardize layers in front of the networks (nn/layers/standardize/operations_generic.h:68-86; no trainable parameters,
    // and the first layer's input gradient is not formed, so only the forward pass sees them)
    if (A->actor_standardize_mean)
        for (int b = 0; b < B; b++)
            for (int c = 0; c < O; c++) {
                float v = obs[(size_t)b * O + c] - A->actor_standardize_mean[c];
                if (A->actor_standardize_precision[c] != 0) v *= A->actor_standardize_precision[c];
                obs[(size_t)b * O + c] = v;
            }
    if (A->critic_standardize_mean)
        for (int b = 0; b < B; b++)
            for (int c = 0; c < OP; c++) {
                float v = obsp[(size_t)b * OP + c] - A->critic_standardize_mean[c];
                if (A->critic_standardize_precision[c] != 0) v *= A->critic_standardize_precision[c];
                obsp[(size_t)b * OP + c] = v;
            }
    int rc;
    if ((rc = rlt_oracle_mlp_zero_gradient(A->critic, A->n_critic_layers))) return rc;                   // :158
    if ((rc = rlt_oracle_mlp_zero_gradient(A->actor, A->n_actor_layers))) return rc;                     // :159 (clears the log_std gradient too)
    if (A->d_log_std) for (int a = 0; a < AD; a++) A->d_log_std[a] = 0;
    if ((rc = rlt_oracle_mlp_forward(A->actor, A->n_actor_layers, obs.data(), O, B))) return rc;          // :203
    const float* means = A->actor[A->n_actor_layers - 1].output;
    if ((rc = rlt_oracle_ppo_surrogate_gradient(means, AD, A->log_std, act.data(), AD, lp.data(), 1, adv.data(), 1, P, d_act.data(), AD, A->d_log_std, B, AD))) return rc;
    if ((rc = rlt_oracle_mlp_backward(A->actor, A->n_actor_layers, obs.data(), O, d_act.data(), AD, nullptr, 0, B, 1))) return rc;   // :285
    if ((rc = rlt_oracle_mlp_forward(A->critic, A->n_critic_layers, obsp.data(), OP, B))) return rc;     // :291
    const float* values = A->critic[A->n_critic_layers - 1].output;
    float loss_weight = 0.5f;
    if ((rc = rlt_oracle_mse_gradient(values, 1, tgt.data(), 1, d_crit.data(), 1, B, 1, 0, &loss_weight))) return rc;                // :295
    if (out_critic_loss) if ((rc = rlt_oracle_mse_evaluate(values, 1, tgt.data(), 1, B, 1, 1.0f, out_critic_loss))) return rc;       // :303
    if ((rc = rlt_oracle_mlp_backward(A->critic, A->n_critic_layers, obsp.data(), OP, d_crit.data(), 1, nullptr, 0, B, 1))) return rc; // :298
    if ((rc = adam_over(A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age))) return rc;                   // :305
    return adam_over(A->critic_adam_tensors, A->n_critic_adam_tensors, &A->critic_adam, A->critic_age);                              // :306
}

// One epoch of train(): the batch loop rl/algorithms/ppo/operations_generic.h:156-318 over the rows the epoch's shuffle (:126-155) put in place,
// given here as a permutation; minibatch i takes entries [i * batch, (i + 1) * batch).
int rlt_oracle_ppo_train_epoch(const rlt_ppo_agent* A, const rlt_ppo_parameters* P, const float* observations, const float* observations_privileged,
                               const float* actions, const float* action_log_probs, const float* advantages, const float* target_values, int ld,
                               const uint32_t* row_indices, int n_minibatches, float* out_critic_losses) {
    if (!A || !row_indices || n_minibatches < 1) return RLT_E_INVALID_ARGUMENT;
    for (int i = 0; i < n_minibatches; i++) {
        const int rc = rlt_oracle_ppo_train_minibatch(A, P, observations, observations_privileged, actions, action_log_probs, advantages, target_values, ld,
                                                      row_indices + (size_t)i * A->batch, out_critic_losses ? out_critic_losses + i : nullptr);
        if (rc) return rc;
    }
    return 0;
}

// The in-place dataset shuffle of train() (rl/algorithms/ppo/operations_generic.h:126-155) restated on a row-index array: for
// each epoch, for i in [0, n): j = uniform_int(i, n-1) (std::uniform_int_distribution on the loop's std::mt19937, as
// random/operations_cpu.h:26-29 does), swap(rows i, j). rng_state is the engine's text form (operator<<) and is advanced in place;
// permutations receives [epochs][n]: the original row index that sits at each position while that epoch's minibatches are taken.
int rlt_oracle_ppo_shuffle(char* rng_state, int rng_state_capacity, int n, int epochs, uint32_t* permutations) {
    if (!rng_state || n <= 0 || epochs <= 0 || !permutations) return RLT_E_INVALID_ARGUMENT;
    std::mt19937 engine;
    { std::istringstream in(rng_state); in >> engine; if (in.fail()) return RLT_E_INVALID_ARGUMENT; }
    std::vector<uint32_t> perm((size_t)n);
    for (int i = 0; i < n; i++) perm[i] = (uint32_t)i;
    for (int e = 0; e < epochs; e++) {
        for (size_t i = 0; i < (size_t)n; i++) {
            size_t j = std::uniform_int_distribution<size_t>(i, (size_t)n - 1)(engine);
            std::swap(perm[i], perm[j]);
        }
        std::memcpy(permutations + (size_t)e * n, perm.data(), sizeof(uint32_t) * n);
    }
    std::ostringstream out; out << engine;
    const std::string s = out.str();
    if ((int)s.size() + 1 > rng_state_capacity) return RLT_E_INVALID_ARGUMENT;
    std::memcpy(rng_state, s.c_str(), s.size() + 1);
    return 0;
}

// nn/layers/gru/operations_generic.h:231-341 (evaluate with multi-step intermediates = forward), loop order as there
int rlt_oracle_gru_forward(const rlt_gru_layer* L, const float* input, const uint8_t* reset, int S, int B) {
    if (!L || !input || S <= 0 || B <= 0 || !L->weights_input || !L->biases_input || !L->weights_hidden || !L->biases_hidden || !L->initial_hidden_state ||
        !L->post_activation || !L->n_pre_pre_activation || !L->output) return RLT_E_INVALID_ARGUMENT;
    const int I = L->input_dim, H = L->hidden_dim, H3 = 3 * H;
    std::vector<float> hprev((size_t)B * H);
    for (int t = 0; t < S; t++) {
        float* post = L->post_activation + (size_t)t * B * H3;
        float* npp = L->n_pre_pre_activation + (size_t)t * B * H;
        float* out = L->output + (size_t)t * B * H;
        const float* x = input + (size_t)t * B * I;
        for (int b = 0; b < B; b++) {
            const bool from_initial = t == 0 || (reset && reset[(size_t)t * B + b]);
            const float* src = from_initial ? L->initial_hidden_state : L->output + ((size_t)(t - 1) * B + b) * H;
            std::memcpy(&hprev[(size_t)b * H], src, sizeof(float) * H);
        }
        for (int b = 0; b < B; b++)                                       // W_h h + b_h (:262-288)
            for (int j = 0; j < H3; j++) {
                float acc = L->biases_hidden[j];
                for (int k = 0; k < H; k++) acc += hprev[(size_t)b * H + k] * L->weights_hidden[(size_t)j * H + k];
                post[(size_t)b * H3 + j] = acc;
            }
        for (int b = 0; b < B; b++)                                       // :290-291
            for (int j = 0; j < H; j++) { npp[(size_t)b * H + j] = post[(size_t)b * H3 + 2 * H + j]; post[(size_t)b * H3 + 2 * H + j] = 0; }
        for (int b = 0; b < B; b++)                                       // += W_i x + b_i (:293)
            for (int j = 0; j < H3; j++) {
                float acc = post[(size_t)b * H3 + j] + L->biases_input[j];
                for (int k = 0; k < I; k++) acc += x[(size_t)b * I + k] * L->weights_input[(size_t)j * I + k];
                post[(size_t)b * H3 + j] = acc;
            }
        for (int b = 0; b < B; b++) {
            float* p = post + (size_t)b * H3;
            for (int j = 0; j < 2 * H; j++) p[j] = L->fast_tanh ? 0.5f * fast_tanh(0.5f * p[j]) + 0.5f : 1 / (1 + std::exp(-p[j]));   // (fast_)sigmoid (:302-310)
            for (int j = 0; j < H; j++) p[2 * H + j] += npp[(size_t)b * H + j] * p[j];                 // :303
            for (int j = 0; j < H; j++) p[2 * H + j] = L->fast_tanh ? fast_tanh(p[2 * H + j]) : std::tanh(p[2 * H + j]);   // :312-320
            for (int j = 0; j < H; j++) {
                float o = 1 - p[H + j];                                                                 // one_minus (:313)
                o = o * p[2 * H + j];                                                                   // multiply (:314)
                o += p[H + j] * hprev[(size_t)b * H + j];                                               // multiply_accumulate (:315-330)
                out[(size_t)b * H + j] = o;
            }
        }
    }
    return 0;
}

// nn/layers/gru/operations_generic.h:594-760, step by step from the last to the first
int rlt_oracle_gru_backward(const rlt_gru_layer* L, const float* input, float* d_output, float* d_input, const uint8_t* reset, int S, int B, int want_w) {
    if (!L || !d_output || S <= 0 || B <= 0 || (!input && want_w)) return RLT_E_INVALID_ARGUMENT;
    if (want_w && (!L->d_weights_input || !L->d_biases_input || !L->d_weights_hidden || !L->d_biases_hidden)) return RLT_E_INVALID_ARGUMENT;
    const int I = L->input_dim, H = L->hidden_dim, H3 = 3 * H;
    std::vector<float> hprev((size_t)B * H), buf((size_t)B * H3);
    for (int t = S - 1; t >= 0; t--) {
        const float* post = L->post_activation + (size_t)t * B * H3;
        const float* npp = L->n_pre_pre_activation + (size_t)t * B * H;
        float* dout = d_output + (size_t)t * B * H;
        float* dprev = t > 0 ? d_output + (size_t)(t - 1) * B * H : nullptr;
        for (int b = 0; b < B; b++) {
            const bool from_initial = t == 0 || (reset && reset[(size_t)t * B + b]);
            const float* src = from_initial ? L->initial_hidden_state : L->output + ((size_t)(t - 1) * B + b) * H;
            std::memcpy(&hprev[(size_t)b * H], src, sizeof(float) * H);
            const float* p = post + (size_t)b * H3;
            float* bb = &buf[(size_t)b * H3];
            for (int j = 0; j < H; j++) {
                const float dh = dout[(size_t)b * H + j];
                if (!from_initial) dprev[(size_t)b * H + j] += dh * p[H + j];                            // :643-659
                bb[H + j] = dh * (hprev[(size_t)b * H + j] - p[2 * H + j]);                              // buffer_z (:624,660)
                bb[2 * H + j] = dh * (1 - p[H + j]) * (1 - p[2 * H + j] * p[2 * H + j]);                  // buffer_n (:668)
                bb[j] = bb[2 * H + j] * npp[(size_t)b * H + j];                                         // buffer_r (:669)
            }
            for (int j = 0; j < 2 * H; j++) bb[j] = bb[j] * p[j] * (1 - p[j]);                           // :670
        }
        if (want_w) {
            const float* x = input + (size_t)t * B * I;
            for (int j = 0; j < H3; j++)                                                                 // :677
                for (int k = 0; k < I; k++) {
                    float acc = L->d_weights_input[(size_t)j * I + k];
                    for (int b = 0; b < B; b++) acc += buf[(size_t)b * H3 + j] * x[(size_t)b * I + k];
                    L->d_weights_input[(size_t)j * I + k] = acc;
                }
            for (int j = 0; j < H3; j++) {                                                               // reduce_sum<true> (:678): sum first, then add
                float acc = 0;
                for (int b = 0; b < B; b++) acc += buf[(size_t)b * H3 + j];
                L->d_biases_input[j] = acc + L->d_biases_input[j];
            }
            for (int j = 0; j < 2 * H; j++) L->d_biases_hidden[j] = L->d_biases_input[j];                 // :679-681
        }
        if (d_input) {                                                                                   // :688
            float* dx = d_input + (size_t)t * B * I;
            for (int b = 0; b < B; b++)
                for (int k = 0; k < I; k++) {
                    float acc = 0;
                    for (int j = 0; j < H3; j++) acc += buf[(size_t)b * H3 + j] * L->weights_input[(size_t)j * I + k];
                    dx[(size_t)b * I + k] = acc;
                }
        }
        for (int b = 0; b < B; b++) for (int j = 0; j < H; j++) buf[(size_t)b * H3 + 2 * H + j] *= post[(size_t)b * H3 + j];   // :691
        if (want_w) {                                                                                    // :693-742
            for (int j = 0; j < H3; j++)
                for (int k = 0; k < H; k++) {
                    float acc = L->d_weights_hidden[(size_t)j * H + k];
                    for (int b = 0; b < B; b++) acc += buf[(size_t)b * H3 + j] * hprev[(size_t)b * H + k];
                    L->d_weights_hidden[(size_t)j * H + k] = acc;
                }
        }
        if (t > 0)
            for (int b = 0; b < B; b++) {
                if (reset && reset[(size_t)t * B + b]) continue;                                         // rows of reset samples are zeroed (:716-722)
                for (int k = 0; k < H; k++) {
                    float acc = dprev[(size_t)b * H + k];
                    for (int j = 0; j < H3; j++) acc += buf[(size_t)b * H3 + j] * L->weights_hidden[(size_t)j * H + k];
                    dprev[(size_t)b * H + k] = acc;
                }
            }
        if (want_w)                                                                                      // :745-749
            for (int j = 0; j < H; j++) {
                // the reference has zeroed the buffer rows of samples that were reset at this step (t > 0) by now (:716-722), so they do not
                // contribute to the b_hn gradient (they do contribute to everything above)
                float acc = 0;
                for (int b = 0; b < B; b++) acc += (t > 0 && reset && reset[(size_t)t * B + b]) ? 0.0f : buf[(size_t)b * H3 + 2 * H + j];
                L->d_biases_hidden[2 * H + j] = acc + L->d_biases_hidden[2 * H + j];
            }
    }
    return 0;
}

// --------------------------------------------------------------------------------------------- TD3
static inline float clamp_f(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }   // math::clamp

// nn/layers/td3_sampling/operations_generic.h:75-128
int rlt_oracle_td3_sampling_forward(const float* input, int ldin, const float* noise, int ldn, float std, float* pre_clip, int ldp,
                                    float* output, int ldo, int batch, int dim) {
    if (!input || !output || batch <= 0 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < batch; r++)
        for (int c = 0; c < dim; c++) {
            float mean = input[(size_t)r * ldin + c];
            float sample = noise ? mean + noise[(size_t)r * ldn + c] * std : mean;
            if (pre_clip) pre_clip[(size_t)r * ldp + c] = sample;
            output[(size_t)r * ldo + c] = clamp_f(sample, -1.0f, 1.0f);
        }
    return 0;
}
// td3_sampling/operations_generic.h:139-163
int rlt_oracle_td3_sampling_backward(const float* pre_clip, int ldp, const float* d_output, int lddo, float* d_input, int lddi, int batch, int dim) {
    if (!pre_clip || !d_output || !d_input || batch <= 0 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < batch; r++)
        for (int c = 0; c < dim; c++) {
            float pc = pre_clip[(size_t)r * ldp + c];
            d_input[(size_t)r * lddi + c] = (pc < -1 || pc > 1) ? 0.0f : d_output[(size_t)r * lddo + c];
        }
    return 0;
}
// rl/algorithms/td3/operations_generic.h:116-128; std::normal_distribution(mean, std) returns z * std + mean
int rlt_oracle_td3_target_action_noise(const float* z, float std, float clip, float* out, size_t count) {
    if (!z || !out) return RLT_E_INVALID_ARGUMENT;
    for (size_t i = 0; i < count; i++) out[i] = clamp_f(z[i] * std + 0.0f, -clip, clip);
    return 0;
}
// td3/operations_generic.h:129-145
int rlt_oracle_td3_noisy_next_actions(float* next_actions, int lda, const float* noise, int ldn, int batch, int dim) {
    if (!next_actions || !noise || batch <= 0 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int r = 0; r < batch; r++)
        for (int c = 0; c < dim; c++) {
            float a = next_actions[(size_t)r * lda + c] + noise[(size_t)r * ldn + c];
            next_actions[(size_t)r * lda + c] = clamp_f(a, -1.0f, 1.0f);
        }
    return 0;
}
// td3/operations_generic.h:146-169
int rlt_oracle_td3_target_action_values(const float* q1, const float* q2, const float* rewards, const uint8_t* terminated,
                                        float gamma, int ignore_termination, float* target, int batch) {
    if (!q1 || !q2 || !rewards || !terminated || !target || batch <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int b = 0; b < batch; b++) {
        float m = q1[b] < q2[b] ? q1[b] : q2[b];
        float future = (ignore_termination || !terminated[b]) ? gamma * m : 0.0f;
        target[b] = rewards[b] + future;
    }
    return 0;
}

// td3/operations_generic.h:170-235 with SEQUENCE_LENGTH = 1
int rlt_oracle_td3_train_critic(const rlt_td3_agent* A, int ci, const float* sampling_noise) {
    if (!A || ci < 0 || ci > 1 || !sampling_noise) return RLT_E_INVALID_ARGUMENT;
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const rlt_dense_layer* critic = A->critics[ci];
    int rc;
    if ((rc = rlt_oracle_mlp_zero_gradient(critic, A->n_critic_layers))) return rc;                                                  // :185
    const float* obs_next = A->observations_actions_base + (size_t)B * D;
    std::vector<float> mean((size_t)B * ACT);
    if ((rc = rlt_oracle_mlp_evaluate(A->actor_target, A->n_actor_layers, obs_next, D, mean.data(), ACT, B))) return rc;             // :191 (MLP part)
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = rlt_oracle_td3_sampling_forward(mean.data(), ACT, sampling_noise, ACT, A->sampling_std, nullptr, 0, next_actions, D, B, ACT))) return rc;
    if ((rc = rlt_oracle_td3_noisy_next_actions(next_actions, D, A->target_next_action_noise, ACT, B, ACT))) return rc;              // :192
    if (A->next_final_step_mask)                                                                                                   // :193-195
        if ((rc = rlt_oracle_mask_copy(obs_next + OBS, D, next_actions, D, A->next_final_step_mask, 1, B, ACT))) return rc;
    for (int b = 0; b < B; b++) std::memcpy(A->next_state_action_value_input + (size_t)b * D, obs_next + (size_t)b * D, sizeof(float) * OBS);   // :196
    for (int k = 0; k < 2; k++)                                                                                                    // :197-198
        if ((rc = rlt_oracle_mlp_evaluate(A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, A->next_q[k], 1, B))) return rc;
    if ((rc = rlt_oracle_td3_target_action_values(A->next_q[0], A->next_q[1], A->rewards, A->terminated, A->gamma, A->ignore_termination,
                                                 A->target_action_value, B))) return rc;                                           // :200
    if ((rc = rlt_oracle_mlp_forward(critic, A->n_critic_layers, A->observations_actions_base, D, B))) return rc;                   // :205
    float* q = critic[A->n_critic_layers - 1].output;
    // :207-212 loss_weight = 1 * (SEQ * B / num_final_steps)
    float n_final = (float)B;
    if (A->final_step_mask) rlt_oracle_cast_reduce_sum_u8(A->final_step_mask, B, &n_final);
    float loss_weight = 1.0f; loss_weight *= (float)(1 * B) / n_final;
    if ((rc = rlt_oracle_mse_gradient(q, 1, A->target_action_value, 1, A->d_output_critic, 1, B, 1, loss_weight, nullptr))) return rc;   // :217
    if (A->final_step_mask) {                                                                                                      // :218-227
        rlt_oracle_mask_zero(A->d_output_critic, 1, A->final_step_mask, 1, B, 1);
        rlt_oracle_mask_zero(q, 1, A->final_step_mask, 1, B, 1);                      // the logging block zeroes these in place
        rlt_oracle_mask_zero(A->target_action_value, 1, A->final_step_mask, 1, B, 1);
    }
    if ((rc = rlt_oracle_mlp_backward(critic, A->n_critic_layers, A->observations_actions_base, D, A->d_output_critic, 1, nullptr, 0, B, 1))) return rc;   // :233
    return adam_over(A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci]);                   // :234
}

// td3/operations_generic.h:236-281 with SEQUENCE_LENGTH = 1
int rlt_oracle_td3_train_actor(const rlt_td3_agent* A, const float* sampling_noise) {
    if (!A || !sampling_noise) return RLT_E_INVALID_ARGUMENT;
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const float* obs = A->observations_actions_base;
    int rc;
    if ((rc = rlt_oracle_mlp_forward(A->actor, A->n_actor_layers, obs, D, B))) return rc;                                          // :255 (MLP part)
    const float* mean = A->actor[A->n_actor_layers - 1].output;
    float* actions = A->state_action_value_input + OBS;
    if ((rc = rlt_oracle_td3_sampling_forward(mean, ACT, sampling_noise, ACT, A->sampling_std, A->actor_pre_clip, ACT, actions, D, B, ACT))) return rc;
    if (A->final_step_mask)                                                                                                        // :256-258
        if ((rc = rlt_oracle_mask_copy(obs + OBS, D, actions, D, A->final_step_mask, 1, B, ACT))) return rc;
    for (int b = 0; b < B; b++) std::memcpy(A->state_action_value_input + (size_t)b * D, obs + (size_t)b * D, sizeof(float) * OBS);  // :259
    const rlt_dense_layer* critic = A->critics[0];
    if ((rc = rlt_oracle_mlp_forward(critic, A->n_critic_layers, A->state_action_value_input, D, B))) return rc;                    // :261
    float n_final = (float)B;                                                                                                      // :262-267
    if (A->final_step_mask) rlt_oracle_cast_reduce_sum_u8(A->final_step_mask, B, &n_final);
    for (int b = 0; b < B; b++) A->d_output_actor[b] = (float)-1 / n_final;
    if (A->final_step_mask) rlt_oracle_mask_zero(A->d_output_actor, 1, A->final_step_mask, 1, B, 1);
    if ((rc = rlt_oracle_mlp_backward(critic, A->n_critic_layers, nullptr, 0, A->d_output_actor, 1, A->d_critic_input, D, B, 0))) return rc;   // :271
    float* d_actions = A->d_critic_input + OBS;                                                                                    // :272
    if (A->final_step_mask) rlt_oracle_mask_zero(d_actions, D, A->final_step_mask, 1, B, ACT);                                     // :273-275
    if ((rc = rlt_oracle_mlp_zero_gradient(A->actor, A->n_actor_layers))) return rc;                                                // :277
    // :278 sequential backward: the sampling layer's backward_full, then the MLP's backward
    if ((rc = rlt_oracle_td3_sampling_backward(A->actor_pre_clip, ACT, d_actions, D, A->d_actor_output, ACT, B, ACT))) return rc;
    if ((rc = rlt_oracle_mlp_backward(A->actor, A->n_actor_layers, obs, D, A->d_actor_output, ACT, nullptr, 0, B, 1))) return rc;
    return adam_over(A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age);                               // :280
}

static void polyak_mlp(const rlt_dense_layer* source, const rlt_dense_layer* target, int n, float polyak) {
    for (int l = 0; l < n; l++) {
        rlt_oracle_polyak_update(source[l].weights, target[l].weights, (size_t)source[l].in_dim * source[l].out_dim, polyak, 0);
        rlt_oracle_polyak_update(source[l].biases, target[l].biases, (size_t)source[l].out_dim, polyak, 0);
    }
}
// td3/operations_generic.h:317-321
int rlt_oracle_td3_update_critic_targets(const rlt_td3_agent* A) {
    if (!A) return RLT_E_INVALID_ARGUMENT;
    for (int k = 0; k < 2; k++) polyak_mlp(A->critics[k], A->critics_target[k], A->n_critic_layers, A->critic_polyak);
    return 0;
}
// td3/operations_generic.h:322-325
int rlt_oracle_td3_update_actor_target(const rlt_td3_agent* A) {
    if (!A) return RLT_E_INVALID_ARGUMENT;
    polyak_mlp(A->actor, A->actor_target, A->n_actor_layers, A->actor_polyak);
    return 0;
}

// --------------------------------------------------------------------------------------------- on-policy collection, normalisation
// nn/layers/standardize/operations_generic.h:54-67
int rlt_oracle_standardize_set_statistics(const float* mean, const float* std, float* layer_mean, float* layer_precision, int dim) {
    if (!mean || !std || !layer_mean || !layer_precision || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int i = 0; i < dim; i++) { layer_mean[i] = mean[i]; layer_precision[i] = std[i] == 0 ? 0.0f : 1 / std[i]; }
    return 0;
}
// standardize/operations_generic.h:68-86
int rlt_oracle_standardize_forward(const float* layer_mean, const float* layer_precision, const float* input, int ldin, float* output, int ldo, int batch, int dim) {
    if (!layer_mean || !layer_precision || !input || !output || batch <= 0 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int b = 0; b < batch; b++)
        for (int i = 0; i < dim; i++) {
            float v = input[(size_t)b * ldin + i] - layer_mean[i];
            if (layer_precision[i] != 0) v *= layer_precision[i];
            output[(size_t)b * ldo + i] = v;
        }
    return 0;
}
// standardize/operations_generic.h:101-120
int rlt_oracle_standardize_backward_input(const float* layer_precision, const float* d_output, int ldd, float* d_input, int ldi, int batch, int dim) {
    if (!layer_precision || !d_output || !d_input || batch <= 0 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    for (int b = 0; b < batch; b++)
        for (int i = 0; i < dim; i++) d_input[(size_t)b * ldi + i] = d_output[(size_t)b * ldd + i] * layer_precision[i];
    return 0;
}
// rl/components/running_normalizer/operations_generic.h:24-45 with mean / std of containers/matrix/operations_generic.h:640-691
int rlt_oracle_running_normalizer_update(const float* data, int ld, int rows, int dim, float* mean, float* std, uint32_t* age) {
    if (!data || !mean || !std || !age || rows < 2 || dim <= 0) return RLT_E_INVALID_ARGUMENT;
    *age += 1;
    for (int c = 0; c < dim; c++) {
        float acc = 0;
        for (int r = 0; r < rows; r++) acc += data[(size_t)r * ld + c];
        const float data_mean = acc / (rows * 1);
        float sq = 0;
        for (int r = 0; r < rows; r++) { const float diff = data[(size_t)r * ld + c] - data_mean; sq += diff * diff; }
        const float data_std = sq < 1e-6 ? 0.0f : std::sqrt(sq / (rows * 1 - 1));
        mean[c] = mean[c] + (data_mean - mean[c]) / (*age);
        std[c] = std[c] + (data_std - std[c]) / (*age);
    }
    return 0;
}

// rl/components/on_policy_runner/operations_generic.h:105-146 and operations_generic_per_env.h:8-74 for Pendulum environments.
// engine != nullptr: the draws come from it in the reference's order and are written to action_noise / initial_states; otherwise they are read.
static int on_policy_collect_impl(const rlt_pendulum_runner* rn, const rlt_on_policy_dataset* D, const rlt_dense_layer* actor, int n_layers, const float* log_std,
                                  const float* st_mean, const float* st_precision, float* action_noise, float* initial_states, int truncate_on_each_iteration,
                                  std::mt19937* engine) {
    if (!rn || !D || !actor || n_layers < 1 || !log_std || !action_noise || !rn->states || !rn->episode_step || !rn->episode_return || !rn->truncated) return RLT_E_INVALID_ARGUMENT;
    if (!D->observations || !D->actions_mean || !D->actions || !D->action_log_probs || !D->rewards || !D->terminated || !D->truncated || !D->all_reset) return RLT_E_INVALID_ARGUMENT;
    const int N = rn->n_envs, S = D->steps_per_env, ld = D->ld, OBS = 3, ACT = actor[n_layers - 1].out_dim;
    if (N <= 0 || S <= 0 || actor[0].in_dim != OBS || ACT != 1) return RLT_E_INVALID_ARGUMENT;     // the Pendulum takes one torque
    if (truncate_on_each_iteration) for (int e = 0; e < N; e++) rn->truncated[e] = 1;                                           // :112-114
    for (int e = 0; e < N; e++) D->all_reset[(size_t)e * ld] = rn->truncated[e];                                                  // :115-117 (reset aliases all_reset)
    std::vector<float> standardized((size_t)N * OBS);
    for (int step = 0; step < S; step++) {
        float* obs = D->observations + (size_t)step * N * ld;
        float* means = D->actions_mean + (size_t)step * N * ld;
        float* actions = D->actions + (size_t)step * N * ld;
        for (int e = 0; e < N; e++) {                                                                                          // prologue, per_env :8-35
            if (rn->truncated[e]) {
                rn->truncated[e] = 0; rn->episode_step[e] = 0; rn->episode_return[e] = 0;
                float* ini = initial_states ? initial_states + ((size_t)step * N + e) * 2 : nullptr;
                if (engine) {       // sample_initial_state, pendulum/operations_generic.h:66-77
                    const float th = std::uniform_real_distribution<float>(-(float)M_PI, (float)M_PI)(*engine);
                    const float thd = std::uniform_real_distribution<float>(-1.0f, 1.0f)(*engine);
                    if (ini) { ini[0] = th; ini[1] = thd; }
                    rn->states[2 * e] = th; rn->states[2 * e + 1] = thd;
                } else {
                    if (!ini) return RLT_E_INVALID_ARGUMENT;
                    rn->states[2 * e] = ini[0]; rn->states[2 * e + 1] = ini[1];
                }
            }
            pendulum_observe(rn->states[2 * e], rn->states[2 * e + 1], obs + (size_t)e * ld);
        }
        int rc;                                                                                                                 // :131 evaluate_step of the actor in Rollout mode
        if (st_mean) {
            if ((rc = rlt_oracle_standardize_forward(st_mean, st_precision, obs, ld, standardized.data(), OBS, N, OBS))) return rc;
            if ((rc = rlt_oracle_mlp_evaluate(actor, n_layers, standardized.data(), OBS, means, ld, N))) return rc;
        } else if ((rc = rlt_oracle_mlp_evaluate(actor, n_layers, obs, ld, means, ld, N))) return rc;
        for (int e = 0; e < N; e++) {                                                                                          // epilogue, per_env :37-74
            const size_t pos = (size_t)step * N + e;
            float log_prob = 0;
            for (int a = 0; a < ACT; a++) {
                const float mean = means[(size_t)e * ld + a];
                const float action_std = std::exp(log_std[a]);
                float* z = action_noise + pos * ACT + a;
                if (engine) { std::mt19937 copy = *engine; *z = std::normal_distribution<float>(0.0f, 1.0f)(copy); }
                // std::normal_distribution(mean, std) returns z * std + mean for the standard normal value z it generates
                const float noisy = engine ? std::normal_distribution<float>(mean, action_std)(*engine) : *z * action_std + mean;
                log_prob += normal_log_prob(mean, log_std[a], noisy);
                actions[(size_t)e * ld + a] = noisy;
            }
            D->action_log_probs[pos * ld] = log_prob;
            float nth, nthd, reward;
            pendulum_dynamics(&rn->env, rn->states[2 * e], rn->states[2 * e + 1], actions[(size_t)e * ld], &nth, &nthd, &reward);
            D->terminated[pos * ld] = 0.0f;                                                 // the Pendulum never terminates
            rn->episode_return[e] += reward;
            D->rewards[pos * ld] = reward;
            rn->episode_step[e] += 1;
            const bool truncated = rn->episode_step_limit > 0 && rn->episode_step[e] >= (uint32_t)rn->episode_step_limit;
            D->truncated[pos * ld] = truncated;
            D->all_reset[(pos + N) * ld] = truncated;
            rn->truncated[e] = truncated;
            rn->states[2 * e] = nth; rn->states[2 * e + 1] = nthd;
        }
    }
    for (int e = 0; e < N; e++) pendulum_observe(rn->states[2 * e], rn->states[2 * e + 1], D->observations + ((size_t)S * N + e) * ld);   // :137-144
    return 0;
}
int rlt_oracle_on_policy_collect(const rlt_pendulum_runner* runner, const rlt_on_policy_dataset* dataset, const rlt_dense_layer* actor, int n_actor_layers,
                                 const float* log_std, const float* standardize_mean, const float* standardize_precision, const float* action_noise,
                                 const float* initial_states, int truncate_on_each_iteration) {
    return on_policy_collect_impl(runner, dataset, actor, n_actor_layers, log_std, standardize_mean, standardize_precision, const_cast<float*>(action_noise),
                                  const_cast<float*>(initial_states), truncate_on_each_iteration, nullptr);
}
int rlt_oracle_on_policy_collect_with_rng(const rlt_pendulum_runner* runner, const rlt_on_policy_dataset* dataset, const rlt_dense_layer* actor, int n_actor_layers,
                                          const float* log_std, const float* standardize_mean, const float* standardize_precision, float* action_noise,
                                          float* initial_states, int truncate_on_each_iteration, char* rng_state, int rng_state_capacity) {
    if (!rng_state) return RLT_E_INVALID_ARGUMENT;
    std::mt19937 engine;
    { std::istringstream in(rng_state); in >> engine; if (in.fail()) return RLT_E_INVALID_ARGUMENT; }
    int rc = on_policy_collect_impl(runner, dataset, actor, n_actor_layers, log_std, standardize_mean, standardize_precision, action_noise, initial_states,
                                    truncate_on_each_iteration, &engine);
    if (rc) return rc;
    std::ostringstream out; out << engine;
    const std::string s = out.str();
    if ((int)s.size() + 1 > rng_state_capacity) return RLT_E_INVALID_ARGUMENT;
    std::memcpy(rng_state, s.c_str(), s.size() + 1);
    return 0;
}

}  // extern "C"
