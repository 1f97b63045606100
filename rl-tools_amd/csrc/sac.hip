// SAC-specific kernels: tanh-Gaussian head (sample_and_squash) forward/backward, TD target, min-Q gradient routing,
// masks, MSE gradient -- and train_critic / train_actor / update_critic_targets assembled from them.
// reference: nn/layers/sample_and_squash/operations_generic.h:148-398 (CUDA :17-115),
//            rl/algorithms/sac/operations_generic.h:133-527 (CUDA :12-128), nn/loss_functions/mse/operations_generic.h:9-97,
//            random/operations_generic.h:72-105.
#include "common.h"
#include "sac_update.h"
#include "mlp_rows.h"
#include <algorithm>

namespace {

__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }
// log N(value; mean, exp(log_std))
__device__ __forceinline__ float normal_log_prob(float mean, float log_std, float sd, float value) {
    const float neg_log_sqrt_2pi = -0.9189385332046727f;
    float z = (value - mean) / sd;
    return neg_log_sqrt_2pi - log_std - 0.5f * z * z;
}

__global__ __launch_bounds__(256) void sas_forward_kernel(rlt_sas_parameters p, const float* __restrict__ input, int ldin, const float* __restrict__ noise, int ldn,
                                                          float* __restrict__ actions, int lda, float* __restrict__ pre_squashing, int ldp,
                                                          float* __restrict__ log_probabilities, int batch, int dim) {
    for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < batch; r += gridDim.x * blockDim.x) {
        float log_prob = 0.0f;
        for (int c = 0; c < dim; c++) {
            float mean = input[(size_t)r * ldin + c];
            float log_std = clampf(input[(size_t)r * ldin + dim + c], p.log_std_lower_bound, p.log_std_upper_bound);
            float sd = expf(log_std);
            float sample = noise ? mean + noise[(size_t)r * ldn + c] * sd : mean;
            if (pre_squashing) pre_squashing[(size_t)r * ldp + c] = sample;
            float a = tanhf(sample);
            actions[(size_t)r * lda + c] = a;
            log_prob += normal_log_prob(mean, log_std, sd, sample) - logf(1.0f - a * a + p.log_probability_epsilon);
        }
        log_probabilities[r] = log_prob;
    }
}

// one workgroup of 1024 lanes; d_log_alpha += scale_num / count(reset) * sum_b alpha * (entropy_b - target_entropy)
__global__ __launch_bounds__(1024) void sas_backward_kernel(rlt_sas_parameters p, const float* __restrict__ input, int ldin, const float* __restrict__ noise, int ldn,
                                                            const float* __restrict__ actions, int lda, const float* __restrict__ pre_squashing, int ldp,
                                                            const float* __restrict__ d_output, int lddo, float* __restrict__ d_input, int lddi,
                                                            const float* __restrict__ log_alpha, float* __restrict__ d_log_alpha,
                                                            const uint8_t* __restrict__ reset, int batch, int dim) {
    __shared__ float partial[16];
    __shared__ float partial_n[16];
    const float alpha = expf(*log_alpha);
    const float alpha_over_b = alpha / (float)batch;
    float acc = 0.0f, nreset = 0.0f;
    for (int b = threadIdx.x; b < batch; b += blockDim.x) {
        float entropy = 0.0f;
        for (int a = 0; a < dim; a++) {
            float action = actions[(size_t)b * lda + a];
            float g = d_output[(size_t)b * lddo + a] * (1.0f - action * action);
            float eps = noise[(size_t)b * ldn + a];
            float log_std_raw = input[(size_t)b * ldin + dim + a];
            float log_std = clampf(log_std_raw, p.log_std_lower_bound, p.log_std_upper_bound);
            float sd = expf(log_std);
            float mu = input[(size_t)b * ldin + a];
            float sample = pre_squashing[(size_t)b * ldp + a];
            float z = (sample - mu) / sd;
            float dlp_dmean = z / sd, dlp_dsample = -z / sd, dlp_dlogstd = z * z - 1.0f;
            float d_mu = g + alpha_over_b * (dlp_dmean + dlp_dsample + 2.0f * action);
            float d_ls = sd * (g * eps) + alpha_over_b * (dlp_dlogstd + dlp_dsample * eps * sd + 2.0f * action * eps * sd);
            if (log_std_raw < p.log_std_lower_bound || log_std_raw > p.log_std_upper_bound) d_ls = 0.0f;
            d_input[(size_t)b * lddi + a] = d_mu;
            d_input[(size_t)b * lddi + dim + a] = d_ls;
            float lp = normal_log_prob(mu, log_std, sd, sample) - logf(1.0f - action * action + p.log_probability_epsilon);
            entropy -= lp;
        }
        acc += alpha * (entropy - p.target_entropy);
        nreset += reset ? (float)(reset[b] != 0) : 1.0f;
    }
    acc = rlt_wave_sum(acc); nreset = rlt_wave_sum(nreset);
    if ((threadIdx.x & 63) == 0) { partial[threadIdx.x >> 6] = acc; partial_n[threadIdx.x >> 6] = nreset; }
    __syncthreads();
    if (threadIdx.x == 0 && d_log_alpha) {
        float s = 0.0f, n = 0.0f;
        for (int i = 0; i < 16; i++) { s += partial[i]; n += partial_n[i]; }
        *d_log_alpha += s / n;
    }
}

__global__ __launch_bounds__(256) void target_q_kernel(const float* __restrict__ q1, const float* __restrict__ q2, const float* __restrict__ rewards,
                                                       const uint8_t* __restrict__ terminated, const float* __restrict__ next_log_probs,
                                                       const float* __restrict__ log_alpha, float gamma, int ignore_termination, float* __restrict__ target, int batch) {
    const float alpha = expf(*log_alpha);
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch; i += gridDim.x * blockDim.x) {
        float min_q = fminf(q1[i], q2[i]) - alpha * next_log_probs[i];
        float future = (ignore_termination || !terminated[i]) ? gamma * min_q : 0.0f;
        target[i] = rewards[i] + future;
    }
}
__global__ __launch_bounds__(256) void min_q_kernel(const float* __restrict__ q1, const float* __restrict__ q2, const float* __restrict__ d1, const float* __restrict__ d2,
                                                    int ld, int cdim, int adim, float* __restrict__ out, int ldo, int batch) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < batch * adim; i += gridDim.x * blockDim.x) {
        int b = i / adim, a = i % adim;
        const float* d = (q1[b] < q2[b]) ? d1 : d2;
        out[(size_t)b * ldo + a] = d[(size_t)b * ld + cdim - adim + a];
    }
}
__global__ __launch_bounds__(256) void mask_copy_kernel(const float* __restrict__ src, int lds, float* __restrict__ dst, int ldt, const uint8_t* __restrict__ mask,
                                                        int invert, int rows, int cols) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < rows * cols; i += gridDim.x * blockDim.x) {
        int r = i / cols, c = i % cols;
        bool m = (mask[r] != 0) != (invert != 0);
        if (m) dst[(size_t)r * ldt + c] = src[(size_t)r * lds + c];
    }
}
__global__ __launch_bounds__(256) void mask_zero_kernel(float* __restrict__ g, int ld, const uint8_t* __restrict__ mask, int invert, int rows, int cols) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < rows * cols; i += gridDim.x * blockDim.x) {
        int r = i / cols, c = i % cols;
        bool m = (mask[r] != 0) != (invert != 0);
        if (m) g[(size_t)r * ld + c] = 0.0f;
    }
}
__global__ __launch_bounds__(256) void mse_gradient_kernel(const float* __restrict__ a, int lda, const float* __restrict__ b, int ldb, float* __restrict__ d, int ldd,
                                                           int rows, int cols, float w, const float* __restrict__ w_dev) {
    const float weight = w_dev ? *w_dev : w;
    const float constant = 2.0f / ((float)rows * (float)cols) * weight;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < rows * cols; i += gridDim.x * blockDim.x) {
        int r = i / cols, c = i % cols;
        d[(size_t)r * ldd + c] = (a[(size_t)r * lda + c] - b[(size_t)r * ldb + c]) * constant;
    }
}
__global__ __launch_bounds__(1024) void mse_evaluate_kernel(const float* __restrict__ a, int lda, const float* __restrict__ b, int ldb, int rows, int cols, float w, float* out) {
    __shared__ float partial[16];
    float acc = 0.0f;
    for (int i = threadIdx.x; i < rows * cols; i += blockDim.x) {
        int r = i / cols, c = i % cols;
        float diff = a[(size_t)r * lda + c] - b[(size_t)r * ldb + c];
        acc += diff * diff;
    }
    acc = rlt_wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) { float s = 0.0f; for (int i = 0; i < 16; i++) s += partial[i]; *out = s * w / (float)(rows * cols); }
}
// strided row copy: dst[r][0:cols] = src[r][0:cols]
__global__ __launch_bounds__(256) void copy2d_kernel(const float* __restrict__ src, int lds, float* __restrict__ dst, int ldd, int rows, int cols) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < rows * cols; i += gridDim.x * blockDim.x) {
        int r = i / cols, c = i % cols;
        dst[(size_t)r * ldd + c] = src[(size_t)r * lds + c];
    }
}
// loss_weight handling of train_critic/train_actor in one launch: n = count(mask) (or rows);
//   critic: d[r] = (q[r] - y[r]) * 2/rows * (rows*0.5/n), zeroed where !mask   (sac/operations_generic.h:298-316)
//   actor : d[r] = -1/n, zeroed where !mask                                   (:437-453)
__global__ __launch_bounds__(1024) void sac_d_output_kernel(const float* __restrict__ q, const float* __restrict__ y, const uint8_t* __restrict__ mask,
                                                            float* __restrict__ d, int rows, int actor) {
    __shared__ float partial[16];
    __shared__ float n_final;
    float cnt = 0.0f;
    for (int i = threadIdx.x; i < rows; i += blockDim.x) cnt += mask ? (float)(mask[i] != 0) : 1.0f;
    cnt = rlt_wave_sum(cnt);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = cnt;
    __syncthreads();
    if (threadIdx.x == 0) { float s = 0.0f; for (int i = 0; i < 16; i++) s += partial[i]; n_final = s; }
    __syncthreads();
    // scale(loss_weight, s, reciprocal) is (1 / n) * s in the reference (containers/tensor/operations_generic.h:437-443): two roundings when n is no power of two
    const float loss_weight = (1.0f / n_final) * (actor ? -1.0f : (float)rows * 0.5f);
    const float constant = 2.0f / (float)rows * loss_weight;
    for (int i = threadIdx.x; i < rows; i += blockDim.x) {
        bool m = mask ? (mask[i] != 0) : true;
        float v = actor ? loss_weight : (q[i] - y[i]) * constant;
        d[i] = m ? v : 0.0f;
    }
}

int grid1(int n) { int b = (n + 255) / 256; return b > 1024 ? 1024 : (b < 1 ? 1 : b); }

}  // namespace

extern "C" {

int rlt_rocm_mse_gradient(rlt_rocm_device* device, const float* a, int lda, const float* b, int ldb, float* d_a, int ldda, int rows, int cols,
                          float loss_weight, const float* loss_weight_device) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(a && b && d_a && rows > 0 && cols > 0 && lda >= cols && ldb >= cols && ldda >= cols);
    hipLaunchKernelGGL(mse_gradient_kernel, dim3(grid1(rows * cols)), dim3(256), 0, device->stream, a, lda, b, ldb, d_a, ldda, rows, cols, loss_weight, loss_weight_device);
    return rlt_launch_status(device);
}
int rlt_rocm_mse_evaluate(rlt_rocm_device* device, const float* a, int lda, const float* b, int ldb, int rows, int cols, float loss_weight, float* out_loss) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(a && b && out_loss && rows > 0 && cols > 0 && lda >= cols && ldb >= cols);
    hipLaunchKernelGGL(mse_evaluate_kernel, dim3(1), dim3(1024), 0, device->stream, a, lda, b, ldb, rows, cols, loss_weight, out_loss);
    return rlt_launch_status(device);
}
int rlt_rocm_sas_forward(rlt_rocm_device* device, const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                         float* actions, int lda, float* pre_squashing, int ldp, float* log_probabilities, int batch, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(p && input && actions && log_probabilities && batch > 0 && dim > 0 && ldin >= 2 * dim && lda >= dim);
    RLT_REQUIRE((!noise || ldn >= dim) && (!pre_squashing || ldp >= dim));
    hipLaunchKernelGGL(sas_forward_kernel, dim3(grid1(batch)), dim3(256), 0, device->stream, *p, input, ldin, noise, ldn, actions, lda, pre_squashing, ldp,
                       log_probabilities, batch, dim);
    return rlt_launch_status(device);
}
static int sas_backward_impl(rlt_rocm_device* device, const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                             const float* actions, int lda, const float* pre_squashing, int ldp, const float* d_output, int lddo, float* d_input, int lddi,
                             const float* log_alpha, float* d_log_alpha, const uint8_t* reset, int batch, int dim) {
    RLT_REQUIRE(p && input && noise && actions && pre_squashing && d_output && d_input && log_alpha && batch > 0 && dim > 0);
    RLT_REQUIRE(ldin >= 2 * dim && ldn >= dim && lda >= dim && ldp >= dim && lddo >= dim && lddi >= 2 * dim);
    hipLaunchKernelGGL(sas_backward_kernel, dim3(1), dim3(1024), 0, device->stream, *p, input, ldin, noise, ldn, actions, lda, pre_squashing, ldp,
                       d_output, lddo, d_input, lddi, log_alpha, d_log_alpha, reset, batch, dim);
    return rlt_launch_status(device);
}
int rlt_rocm_sas_backward(rlt_rocm_device* device, const rlt_sas_parameters* p, const float* input, int ldin, const float* noise, int ldn,
                          const float* actions, int lda, const float* pre_squashing, int ldp, const float* d_output, int lddo, float* d_input, int lddi,
                          const float* log_alpha, float* d_log_alpha, int batch, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    return sas_backward_impl(device, p, input, ldin, noise, ldn, actions, lda, pre_squashing, ldp, d_output, lddo, d_input, lddi, log_alpha, d_log_alpha, nullptr, batch, dim);
}
int rlt_rocm_sac_target_action_values(rlt_rocm_device* device, const float* q1_next, const float* q2_next, const float* rewards, const uint8_t* terminated,
                                      const float* next_log_probabilities, const float* log_alpha, float gamma, int ignore_termination, float* target, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(q1_next && q2_next && rewards && terminated && next_log_probabilities && log_alpha && target && batch > 0);
    hipLaunchKernelGGL(target_q_kernel, dim3(grid1(batch)), dim3(256), 0, device->stream, q1_next, q2_next, rewards, terminated, next_log_probabilities, log_alpha,
                       gamma, ignore_termination, target, batch);
    return rlt_launch_status(device);
}
int rlt_rocm_sac_min_value_d_output(rlt_rocm_device* device, const float* q1, const float* q2, const float* d1, const float* d2, int ld, int cdim, int adim,
                                    float* d_actor_output, int ldo, int batch) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(q1 && q2 && d1 && d2 && d_actor_output && batch > 0 && adim > 0 && cdim >= adim && ld >= cdim && ldo >= adim);
    hipLaunchKernelGGL(min_q_kernel, dim3(grid1(batch * adim)), dim3(256), 0, device->stream, q1, q2, d1, d2, ld, cdim, adim, d_actor_output, ldo, batch);
    return rlt_launch_status(device);
}
int rlt_rocm_mask_copy(rlt_rocm_device* device, const float* source, int lds, float* target, int ldt, const uint8_t* mask, int invert, int rows, int cols) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(source && target && mask && rows > 0 && cols > 0 && lds >= cols && ldt >= cols);
    hipLaunchKernelGGL(mask_copy_kernel, dim3(grid1(rows * cols)), dim3(256), 0, device->stream, source, lds, target, ldt, mask, invert, rows, cols);
    return rlt_launch_status(device);
}
int rlt_rocm_mask_zero(rlt_rocm_device* device, float* gradient, int ld, const uint8_t* mask, int invert, int rows, int cols) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(gradient && mask && rows > 0 && cols > 0 && ld >= cols);
    hipLaunchKernelGGL(mask_zero_kernel, dim3(grid1(rows * cols)), dim3(256), 0, device->stream, gradient, ld, mask, invert, rows, cols);
    return rlt_launch_status(device);
}

static int copy2d(rlt_rocm_device* device, const float* src, int lds, float* dst, int ldd, int rows, int cols) {
    hipLaunchKernelGGL(copy2d_kernel, dim3(grid1(rows * cols)), dim3(256), 0, device->stream, src, lds, dst, ldd, rows, cols);
    return rlt_launch_status(device);
}
static bool agent_ok(const rlt_sac_agent* A) {
    return A && A->batch > 0 && A->observation_dim > 0 && A->action_dim > 0 && A->actor && A->critics[0] && A->critics[1] && A->critics_target[0] &&
           A->critics_target[1] && A->observations_actions_base && A->rewards && A->terminated && A->workspace &&
           A->n_actor_layers >= 1 && A->n_critic_layers >= 1 && A->log_alpha.parameters;
}

int rlt_rocm_sac_set_per_operation(rlt_rocm_device* device, int enabled) {
    if (!device) return RLT_E_NOT_INITIALISED;
    device->sac_per_operation = enabled != 0;
    return 0;
}


// rl/algorithms/sac/operations_generic.h:243-337: the fused kernels where they fit, else one launch per reference operation
int rlt_rocm_sac_train_critic(rlt_rocm_device* device, const rlt_sac_agent* A, int ci, const float* action_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && (ci == 0 || ci == 1) && action_noise);
    if (!device->sac_per_operation && rlt_sac_update_supported(device, A)) { const rlt_update_noise noise = {action_noise, 0, 0, nullptr}; return rlt_sac_update_critic(device, A, ci, noise); }
    if (!device->sac_per_operation && rlt_sac_wide_supported(device, A)) { const rlt_update_noise noise = {action_noise, 0, 0, nullptr}; return rlt_sac_wide_update_critics(device, A, ci, 1, noise, false); }
    RLT_REQUIRE(A->next_state_action_value_input && A->next_q[0] && A->next_q[1] && A->next_log_probabilities && A->target_action_value && A->d_output_critic[ci]);
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const rlt_dense_layer* critic = A->critics[ci];
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(critic, A->n_critic_layers, B) + (size_t)B * 2 * ACT * sizeof(float) + 256);
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(A->actor, A->n_actor_layers, B) + (size_t)B * 2 * ACT * sizeof(float) + 256);
    int rc;
    float* actor_out = (float*)A->workspace;
    void* ws = (char*)A->workspace + (((size_t)B * 2 * ACT * sizeof(float) + 255) & ~(size_t)255);
    size_t ws_bytes = A->workspace_bytes - ((char*)ws - (char*)A->workspace);
    if ((rc = rlt_rocm_mlp_zero_gradient(device, critic, A->n_critic_layers))) return rc;
    const float* obs_next = A->observations_actions_base + (size_t)B * D;
    if ((rc = rlt_rocm_mlp_evaluate(device, A->actor, A->n_actor_layers, obs_next, D, actor_out, 2 * ACT, B, ws, ws_bytes))) return rc;
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = rlt_rocm_sas_forward(device, &A->sas, actor_out, 2 * ACT, action_noise, ACT, next_actions, D, nullptr, 0, A->next_log_probabilities, B, ACT))) return rc;
    if (A->next_final_step_mask) if ((rc = rlt_rocm_mask_copy(device, obs_next + OBS, D, next_actions, D, A->next_final_step_mask, 1, B, ACT))) return rc;
    if ((rc = copy2d(device, obs_next, D, A->next_state_action_value_input, D, B, OBS))) return rc;
    if ((rc = rlt_mlp_forward_pair(device, A->critics_target[0], A->critics_target[1], A->n_critic_layers, A->next_state_action_value_input, D, A->next_q[0], A->next_q[1], 1, B, false, ws, ws_bytes))) return rc;
    if ((rc = rlt_rocm_sac_target_action_values(device, A->next_q[0], A->next_q[1], A->rewards, A->terminated, A->next_log_probabilities, A->log_alpha.parameters,
                                               A->gamma, 0, A->target_action_value, B))) return rc;
    if ((rc = rlt_rocm_mlp_forward(device, critic, A->n_critic_layers, A->observations_actions_base, D, B))) return rc;
    const float* q = critic[A->n_critic_layers - 1].output;
    hipLaunchKernelGGL(sac_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, q, (const float*)A->target_action_value, A->final_step_mask, A->d_output_critic[ci], B, 0);
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_mlp_backward(device, critic, A->n_critic_layers, A->observations_actions_base, D, A->d_output_critic[ci], 1, nullptr, 0, B, 1, ws, ws_bytes))) return rc;
    return rlt_rocm_adam_step(device, A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], 0.0f, nullptr);
}

// rl/algorithms/sac/operations_generic.h:488-527
int rlt_rocm_sac_update_critic_targets(rlt_rocm_device* device, const rlt_sac_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A));
    if (!device->sac_per_operation && 4 * A->n_critic_layers <= 64) {      // all tensors in one launch (per 16)
        const float* sources[64]; float* targets[64]; uint32_t counts[64];
        int n = 0;
        for (int k = 0; k < 2; k++)
            for (int l = 0; l < A->n_critic_layers; l++) {
                const rlt_dense_layer& s = A->critics[k][l]; const rlt_dense_layer& t = A->critics_target[k][l];
                sources[n] = s.weights; targets[n] = t.weights; counts[n++] = (uint32_t)s.in_dim * s.out_dim;
                sources[n] = s.biases; targets[n] = t.biases; counts[n++] = (uint32_t)s.out_dim;
            }
        return rlt_sac_polyak_list(device, sources, targets, counts, n, A->polyak);
    }
    for (int k = 0; k < 2; k++)
        for (int l = 0; l < A->n_critic_layers; l++) {
            const rlt_dense_layer& s = A->critics[k][l]; const rlt_dense_layer& t = A->critics_target[k][l];
            int rc;
            if ((rc = rlt_rocm_polyak_update(device, s.weights, t.weights, (size_t)s.in_dim * s.out_dim, A->polyak, 0))) return rc;
            if ((rc = rlt_rocm_polyak_update(device, s.biases, t.biases, (size_t)s.out_dim, A->polyak, 0))) return rc;
        }
    return 0;
}

// rl/algorithms/sac/operations_generic.h:395-468, one launch per reference operation
int rlt_rocm_sac_train_actor(rlt_rocm_device* device, const rlt_sac_agent* A, const float* action_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && action_noise);
    if (!device->sac_per_operation && rlt_sac_update_supported(device, A)) { const rlt_update_noise noise = {action_noise, 0, 0, nullptr}; return rlt_sac_update_actor(device, A, noise); }
    if (!device->sac_per_operation && rlt_sac_wide_supported(device, A)) { const rlt_update_noise noise = {action_noise, 0, 0, nullptr}; return rlt_sac_wide_update_actor(device, A, noise); }
    RLT_REQUIRE(A->state_action_value_input && A->d_output_actor_critics && A->d_critic_input[0] && A->d_critic_input[1] && A->d_actor_output_squashing &&
                A->d_actor_output && A->actor_pre_squashing && A->actor_log_probabilities && A->actor_actions && A->log_alpha.gradient);
    const int B = A->batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(A->critics[0], A->n_critic_layers, B));
    RLT_REQUIRE(A->workspace_bytes >= rlt_rocm_mlp_workspace_bytes(A->actor, A->n_actor_layers, B));
    void* ws = A->workspace; size_t ws_bytes = A->workspace_bytes;
    int rc;
    if ((rc = rlt_rocm_mlp_zero_gradient(device, A->actor, A->n_actor_layers))) return rc;
    if ((rc = rlt_rocm_fill_f32(device, A->log_alpha.gradient, 1, 1, 1, 0.0f))) return rc;
    const float* obs = A->observations_actions_base;
    if ((rc = rlt_rocm_mlp_forward(device, A->actor, A->n_actor_layers, obs, D, B))) return rc;
    const float* actor_out = A->actor[A->n_actor_layers - 1].output;
    if ((rc = rlt_rocm_sas_forward(device, &A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT,
                                   A->actor_log_probabilities, B, ACT))) return rc;
    float* sav_actions = A->state_action_value_input + OBS;
    if ((rc = copy2d(device, A->actor_actions, ACT, sav_actions, D, B, ACT))) return rc;
    if (A->final_step_mask) if ((rc = rlt_rocm_mask_copy(device, obs + OBS, D, sav_actions, D, A->final_step_mask, 1, B, ACT))) return rc;
    if ((rc = copy2d(device, obs, D, A->state_action_value_input, D, B, OBS))) return rc;
    if ((rc = rlt_mlp_forward_pair(device, A->critics[0], A->critics[1], A->n_critic_layers, A->state_action_value_input, D, nullptr, nullptr, 0, B, true, ws, ws_bytes))) return rc;
    hipLaunchKernelGGL(sac_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, (const float*)nullptr, (const float*)nullptr, A->final_step_mask,
                       A->d_output_actor_critics, B, 1);
    if ((rc = rlt_launch_status(device))) return rc;
    for (int k = 0; k < 2; k++)   // the critics' output activation is the identity, so d_output survives the first backward_input unchanged
        if ((rc = rlt_rocm_mlp_backward(device, A->critics[k], A->n_critic_layers, nullptr, 0, A->d_output_actor_critics, 1, A->d_critic_input[k], D, B, 0, ws, ws_bytes))) return rc;
    const float* q1 = A->critics[0][A->n_critic_layers - 1].output; const float* q2 = A->critics[1][A->n_critic_layers - 1].output;
    if ((rc = rlt_rocm_sac_min_value_d_output(device, q1, q2, A->d_critic_input[0], A->d_critic_input[1], D, D, ACT, A->d_actor_output_squashing, ACT, B))) return rc;
    if (A->final_step_mask) if ((rc = rlt_rocm_mask_zero(device, A->d_actor_output_squashing, ACT, A->final_step_mask, 1, B, ACT))) return rc;
    if ((rc = sas_backward_impl(device, &A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT,
                                A->d_actor_output_squashing, ACT, A->d_actor_output, 2 * ACT, A->log_alpha.parameters, A->log_alpha.gradient, A->reset, B, ACT))) return rc;
    if ((rc = rlt_rocm_mlp_backward(device, A->actor, A->n_actor_layers, obs, D, A->d_actor_output, 2 * ACT, nullptr, 0, B, 1, ws, ws_bytes))) return rc;
    if ((rc = rlt_rocm_adam_step(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, 0.0f, nullptr))) return rc;
    return rlt_rocm_adam_step(device, &A->log_alpha, 1, &A->alpha_adam, A->alpha_age, 0.0f, nullptr);
}

// both train_critic calls of a loop step with a shared batch (and update_critic_targets) as one launch where the fused kernel fits
static int train_critics(rlt_rocm_device* device, const rlt_sac_agent* A, const rlt_update_noise& noise, int update_targets) {
    if (!device->sac_per_operation && rlt_sac_update_supported(device, A)) return rlt_sac_update_critics(device, A, noise, update_targets != 0);
    if (!device->sac_per_operation && rlt_sac_wide_supported(device, A)) return rlt_sac_wide_update_critics(device, A, 0, 2, noise, update_targets != 0);
    int rc;
    const float* values = noise.values;
    if (!values) {
        RLT_REQUIRE(noise.drawn);
        if ((rc = rlt_rocm_randn_f32(device, noise.drawn, (size_t)A->batch * A->action_dim, noise.seed, noise.stream))) return rc;
        values = noise.drawn;
    }
    for (int k = 0; k < 2; k++)
        if ((rc = rlt_rocm_sac_train_critic(device, A, k, values))) return rc;
    return update_targets ? rlt_rocm_sac_update_critic_targets(device, A) : 0;
}
int rlt_rocm_sac_train_critics(rlt_rocm_device* device, const rlt_sac_agent* A, const float* action_noise, int update_targets) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && action_noise);
    const rlt_update_noise noise = {action_noise, 0, 0, nullptr};
    return train_critics(device, A, noise, update_targets);
}
int rlt_rocm_sac_train_critics_drawn(rlt_rocm_device* device, const rlt_sac_agent* A, float* drawn_noise, uint64_t seed, uint64_t stream, int update_targets) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A));
    const rlt_update_noise noise = {nullptr, seed, stream, drawn_noise};
    return train_critics(device, A, noise, update_targets);
}
int rlt_rocm_sac_train_actor_drawn(rlt_rocm_device* device, const rlt_sac_agent* A, float* drawn_noise, uint64_t seed, uint64_t stream) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A));
    if (!device->sac_per_operation && rlt_sac_update_supported(device, A)) { const rlt_update_noise noise = {nullptr, seed, stream, drawn_noise}; return rlt_sac_update_actor(device, A, noise); }
    if (!device->sac_per_operation && rlt_sac_wide_supported(device, A)) { const rlt_update_noise noise = {nullptr, seed, stream, drawn_noise}; return rlt_sac_wide_update_actor(device, A, noise); }
    RLT_REQUIRE(drawn_noise);
    const int rc = rlt_rocm_randn_f32(device, drawn_noise, (size_t)A->batch * A->action_dim, seed, stream);
    return rc ? rc : rlt_rocm_sac_train_actor(device, A, drawn_noise);
}

// rl/algorithms/sac/loop/core/operations_generic.h:110-155 past the warm-up, as a host loop over the entry points of this library
int rlt_rocm_sac_pendulum_loop_by_calls(rlt_rocm_device* device, const rlt_sac_agent* A, const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb, int n_steps,
                                        uint64_t seed, uint64_t step_offset, const rlt_sac_loop_scratch* S) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(agent_ok(A) && runner && rb && S && n_steps >= 0);
    RLT_REQUIRE(S->rollout_noise && S->noise_critic && S->noise_actor && S->env_indices && S->sample_offsets);
    RLT_REQUIRE(rb->observation_dim == A->observation_dim && rb->action_dim == A->action_dim && rb->n_envs == runner->n_envs);
    const int B = A->batch;
    int rc;
    for (int i = 0; i < n_steps; i++) {
        const uint64_t g = 8 * (step_offset + (uint64_t)i);
        // every draw is made by the kernel that consumes it (and echoed into the scratch arrays): four launches per step where the fused kernels fit
        if ((rc = rlt_rocm_pendulum_runner_step_drawn(device, runner, rb, A->actor, A->n_actor_layers, &A->sas, S->rollout_noise, seed, g + 1, g + 2))) return rc;
        if ((rc = rlt_rocm_gather_batch_drawn(device, rb, seed, g + 3, S->env_indices, S->sample_offsets, runner->episode_step_limit, B, A->observations_actions_base, A->rewards,
                                              A->terminated, nullptr, nullptr, nullptr, nullptr))) return rc;
        if ((rc = rlt_rocm_sac_train_critics_drawn(device, A, S->noise_critic, seed, g + 4, 1))) return rc;
        if ((rc = rlt_rocm_sac_train_actor_drawn(device, A, S->noise_actor, seed, g + 5))) return rc;
    }
    return 0;
}

// ---------------------------------------------------------------------------------------- sequence batches, sequential (recurrent) networks
static inline const float* seq_output(const rlt_seq_layer* layers, int n) { const rlt_seq_layer& L = layers[n - 1]; return L.kind ? L.gru.output : L.dense.output; }
static inline int seq_out_dim(const rlt_seq_layer* layers, int n) { const rlt_seq_layer& L = layers[n - 1]; return L.kind ? L.gru.hidden_dim : L.dense.out_dim; }
static bool sequence_agent_ok(const rlt_sac_sequence_agent* A) {
    if (!A || A->observation_dim <= 0 || A->action_dim <= 0 || A->n_actor_layers < 1 || A->n_critic_layers < 1) return false;
    if (!A->actor || !A->critics[0] || !A->critics[1] || !A->critics_target[0] || !A->critics_target[1] || !A->log_alpha.parameters) return false;
    const rlt_sequence_batch& K = A->batch;
    if (K.batch <= 0 || K.sequence_length <= 0 || !K.observations_actions_base || !K.rewards || !K.terminated || !K.reset || !K.next_reset_base || !K.final_step_mask ||
        !K.next_final_step_mask_base) return false;
    if (seq_out_dim(A->actor, A->n_actor_layers) != 2 * A->action_dim) return false;
    for (int k = 0; k < 2; k++) if (seq_out_dim(A->critics[k], A->n_critic_layers) != 1 || seq_out_dim(A->critics_target[k], A->n_critic_layers) != 1) return false;
    return A->workspace && A->workspace_bytes >= rlt_rocm_sac_sequence_workspace_bytes(A);
}

// what one pass of any of the agent's networks needs, rounded up so that the second half of a doubled workspace is aligned like the first
static size_t sequence_pass_workspace_bytes(const rlt_sac_sequence_agent* A, int T, int B) {
    size_t n = rlt_rocm_seq_workspace_bytes(A->actor, A->n_actor_layers, T, B);
    n = std::max(n, rlt_rocm_seq_workspace_bytes(A->critics[0], A->n_critic_layers, T, B));
    n = std::max(n, rlt_rocm_seq_workspace_bytes(A->critics_target[0], A->n_critic_layers, T, B));
    return (n + 255) & ~(size_t)255;
}
size_t rlt_rocm_sac_sequence_workspace_bytes(const rlt_sac_sequence_agent* A) {
    if (!A || !A->actor || !A->critics[0] || !A->critics_target[0]) return 0;
    const int T = A->batch.sequence_length + 1, B = A->batch.batch;
    // up to three passes run at the same time (rlt_side_begin), each in its own third; then the loss gradient of the first critic where both critics train in one call
    return 3 * sequence_pass_workspace_bytes(A, T, B) + ((sizeof(float) * (size_t)A->batch.sequence_length * B + 255) & ~(size_t)255);
}

// rl/algorithms/sac/operations_generic.h:243-337 on a sequence batch, one launch per reference operation
int rlt_rocm_sac_sequence_train_critic(rlt_rocm_device* device, const rlt_sac_sequence_agent* A, int ci, const float* action_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(sequence_agent_ok(A) && (ci == 0 || ci == 1) && action_noise);
    RLT_REQUIRE(A->next_state_action_value_input && A->next_q[0] && A->next_q[1] && A->next_log_probabilities && A->target_action_value && A->d_output);
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const int first = A->include_first_step_in_targets ? 1 : 0, T = S + first, next_offset = first ? 0 : 1;   // off_policy_runner/operations_generic.h:85-92
    const rlt_seq_layer* critic = A->critics[ci];
    // two halves of the workspace: passes that do not depend on each other run at the same time, one on the handle's side stream -- the trained critic's forward
    // pass next to the actor's on the next rows, then the second target critic next to the first (each recurrence fills a twentieth of the chip)
    const size_t ws_bytes = sequence_pass_workspace_bytes(A, S + 1, B);
    void* ws = A->workspace; void* ws_side = (char*)A->workspace + ws_bytes;
    const bool overlap = S >= 48;      // short sequences: a pass is shorter than the two events that fork and join a stream cost on the host
    int rc;
    if ((rc = rlt_rocm_seq_zero_gradient(device, critic, A->n_critic_layers))) return rc;                                                  // :263
    {
        const bool side = overlap && rlt_side_begin(device);
        rc = rlt_rocm_seq_forward(device, critic, A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B, side ? ws_side : ws, ws_bytes);   // :294
        rlt_side_end(device);
        if (rc) return rc;
    }
    const float* base_next = K.observations_actions_base + (size_t)next_offset * B * D;
    const uint8_t* next_reset = K.next_reset_base + (size_t)next_offset * B;
    const uint8_t* next_final = K.next_final_step_mask_base + (size_t)next_offset * B;
    if ((rc = rlt_rocm_seq_forward(device, A->actor, A->n_actor_layers, base_next, D, next_reset, T, B, ws, ws_bytes))) return rc;           // :266-273
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = rlt_rocm_sas_forward(device, &A->sas, seq_output(A->actor, A->n_actor_layers), 2 * ACT, action_noise, ACT, next_actions, D, nullptr, 0,
                                   A->next_log_probabilities, T * B, ACT))) return rc;
    if ((rc = rlt_rocm_mask_copy(device, base_next + OBS, D, next_actions, D, next_final, 1, T * B, ACT))) return rc;                      // :274-277
    if ((rc = copy2d(device, base_next, D, A->next_state_action_value_input, D, T * B, OBS))) return rc;                                   // :278
    for (int k = 1; k >= 0; k--) {                                                                                                         // :283-284 (target critic 1 on the side stream)
        const bool side = k == 1 && overlap && rlt_side_begin(device);
        rc = rlt_rocm_seq_forward(device, A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, next_reset, T, B, side ? ws_side : ws, ws_bytes);
        if (!rc) rc = rlt_rocm_memcpy_d2d(device, A->next_q[k], seq_output(A->critics_target[k], A->n_critic_layers), sizeof(float) * T * B);
        rlt_side_end(device);
        if (rc) return rc;
    }
    if (overlap && (rc = rlt_side_join(device))) return rc;
    // the value of the step after (offset B where the first step is included), the log-probability at the same index (:144-154)
    if ((rc = rlt_rocm_sac_target_action_values(device, A->next_q[0] + first * B, A->next_q[1] + first * B, K.rewards, K.terminated, A->next_log_probabilities,
                                               A->log_alpha.parameters, A->gamma, 0, A->target_action_value, S * B))) return rc;             // :289
    hipLaunchKernelGGL(sac_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, seq_output(critic, A->n_critic_layers), (const float*)A->target_action_value,
                       (const uint8_t*)K.final_step_mask, A->d_output, S * B, 0);                                                          // :298-316
    if ((rc = rlt_launch_status(device))) return rc;
    if ((rc = rlt_rocm_seq_backward(device, critic, A->n_critic_layers, K.observations_actions_base, D, A->d_output, nullptr, K.reset, S, B, 1, 0, ws, ws_bytes))) return rc;   // :329
    return rlt_rocm_adam_step(device, A->critic_adam_tensors[ci], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[ci], 0.0f, nullptr);   // :336
}

// Both critics on one batch and one set of noise (the loop's SHARED_BATCH case, rl/algorithms/sac/loop/core/operations_generic.h:127-138): what the two calls of
// train_critic would compute twice -- the actor on the next rows, its sample, both target critics, the target values -- is computed once, and the two critics'
// passes run next to each other on the handle's three streams: first side stream critic 0 forward, then target critic 1; second side stream critic 1 forward; main
// stream actor, sample, target critic 0; after the join the target values and both loss gradients, then critic 0's backward pass on the main stream next to critic 1's
// on a side stream, then both optimisers. Every pass is the launch sequence that the single calls make, on the same inputs: the results are theirs bit for bit.
int rlt_rocm_sac_sequence_train_critics(rlt_rocm_device* device, const rlt_sac_sequence_agent* A, const float* action_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(sequence_agent_ok(A) && action_noise);
    RLT_REQUIRE(A->next_state_action_value_input && A->next_q[0] && A->next_q[1] && A->next_log_probabilities && A->target_action_value && A->d_output);
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT;
    const int first = A->include_first_step_in_targets ? 1 : 0, T = S + first, next_offset = first ? 0 : 1;
    const size_t ws_bytes = sequence_pass_workspace_bytes(A, S + 1, B);
    void* ws = A->workspace; void* ws_side = (char*)A->workspace + ws_bytes; void* ws_second = (char*)A->workspace + 2 * ws_bytes;
    float* d_output_first = (float*)((char*)A->workspace + 3 * ws_bytes);      // critic 0's loss gradient; critic 1's goes to the agent's buffer, where two single calls leave it
    const bool overlap = S >= 48;      // short sequences: a pass is shorter than the two events that fork and join a stream cost on the host
    int rc;
    for (int k = 0; k < 2; k++) if ((rc = rlt_rocm_seq_zero_gradient(device, A->critics[k], A->n_critic_layers))) return rc;
    {
        if (overlap) rlt_side_begin(device);      // (without a second stream everything below simply runs in order on the one stream)
        rc = rlt_rocm_seq_forward(device, A->critics[0], A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B, device->side_return ? ws_side : ws, ws_bytes);
        rlt_side_end(device);
        if (rc) return rc;
        if (overlap) rlt_side_begin(device, 1);
        rc = rlt_rocm_seq_forward(device, A->critics[1], A->n_critic_layers, K.observations_actions_base, D, K.reset, S, B, device->side_return ? ws_second : ws, ws_bytes);
        rlt_side_end(device);
        if (rc) return rc;
    }
    const float* base_next = K.observations_actions_base + (size_t)next_offset * B * D;
    const uint8_t* next_reset = K.next_reset_base + (size_t)next_offset * B;
    const uint8_t* next_final = K.next_final_step_mask_base + (size_t)next_offset * B;
    if ((rc = rlt_rocm_seq_forward(device, A->actor, A->n_actor_layers, base_next, D, next_reset, T, B, ws, ws_bytes))) return rc;
    float* next_actions = A->next_state_action_value_input + OBS;
    if ((rc = rlt_rocm_sas_forward(device, &A->sas, seq_output(A->actor, A->n_actor_layers), 2 * ACT, action_noise, ACT, next_actions, D, nullptr, 0,
                                   A->next_log_probabilities, T * B, ACT))) return rc;
    if ((rc = rlt_rocm_mask_copy(device, base_next + OBS, D, next_actions, D, next_final, 1, T * B, ACT))) return rc;
    if ((rc = copy2d(device, base_next, D, A->next_state_action_value_input, D, T * B, OBS))) return rc;
    for (int k = 1; k >= 0; k--) {      // target critic 1 behind critic 0's forward pass on the side stream (it waits for the copies above), target critic 0 on the main stream
        if (k == 1 && overlap) rlt_side_begin(device);
        rc = rlt_rocm_seq_forward(device, A->critics_target[k], A->n_critic_layers, A->next_state_action_value_input, D, next_reset, T, B, device->side_return ? ws_side : ws, ws_bytes);
        if (!rc) rc = rlt_rocm_memcpy_d2d(device, A->next_q[k], seq_output(A->critics_target[k], A->n_critic_layers), sizeof(float) * T * B);
        rlt_side_end(device);
        if (rc) return rc;
    }
    if (overlap && (rc = rlt_side_join(device))) return rc;
    if ((rc = rlt_rocm_sac_target_action_values(device, A->next_q[0] + first * B, A->next_q[1] + first * B, K.rewards, K.terminated, A->next_log_probabilities,
                                               A->log_alpha.parameters, A->gamma, 0, A->target_action_value, S * B))) return rc;
    for (int k = 0; k < 2; k++) {
        hipLaunchKernelGGL(sac_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, seq_output(A->critics[k], A->n_critic_layers), (const float*)A->target_action_value,
                           (const uint8_t*)K.final_step_mask, k ? A->d_output : d_output_first, S * B, 0);
        if ((rc = rlt_launch_status(device))) return rc;
    }
    {
        if (overlap) rlt_side_begin(device);
        rc = rlt_rocm_seq_backward(device, A->critics[1], A->n_critic_layers, K.observations_actions_base, D, A->d_output, nullptr, K.reset, S, B, 1, 0, device->side_return ? ws_side : ws, ws_bytes);
        rlt_side_end(device);
        if (rc) return rc;
    }
    if ((rc = rlt_rocm_seq_backward(device, A->critics[0], A->n_critic_layers, K.observations_actions_base, D, d_output_first, nullptr, K.reset, S, B, 1, 0, ws, ws_bytes))) return rc;
    if (overlap && (rc = rlt_side_join(device))) return rc;
    for (int k = 0; k < 2; k++)
        if ((rc = rlt_rocm_adam_step(device, A->critic_adam_tensors[k], A->n_critic_adam_tensors, &A->critic_adam, A->critic_age[k], 0.0f, nullptr))) return rc;
    return 0;
}

// sac/operations_generic.h:486-527
int rlt_rocm_sac_sequence_update_critic_targets(rlt_rocm_device* device, const rlt_sac_sequence_agent* A) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(sequence_agent_ok(A) && A->n_critic_layers <= RLT_SEQ_MAX_LAYERS);
    // every tensor of both target critics in one launch per sixteen tensors
    const float* sources[2 * 5 * RLT_SEQ_MAX_LAYERS]; float* targets[2 * 5 * RLT_SEQ_MAX_LAYERS]; uint32_t counts[2 * 5 * RLT_SEQ_MAX_LAYERS];
    int n = 0;
    auto pair = [&](const float* source, float* target, size_t count) { sources[n] = source; targets[n] = target; counts[n++] = (uint32_t)count; };
    for (int k = 0; k < 2; k++)
        for (int l = 0; l < A->n_critic_layers; l++) {
            const rlt_seq_layer& s = A->critics[k][l]; const rlt_seq_layer& t = A->critics_target[k][l];
            RLT_REQUIRE(s.kind == t.kind);
            if (s.kind == 0) {
                pair(s.dense.weights, t.dense.weights, (size_t)s.dense.in_dim * s.dense.out_dim); pair(s.dense.biases, t.dense.biases, (size_t)s.dense.out_dim);
            } else {
                const size_t H = s.gru.hidden_dim, I = s.gru.input_dim;
                pair(s.gru.weights_input, t.gru.weights_input, 3 * H * I); pair(s.gru.biases_input, t.gru.biases_input, 3 * H);
                pair(s.gru.weights_hidden, t.gru.weights_hidden, 3 * H * H); pair(s.gru.biases_hidden, t.gru.biases_hidden, 3 * H);
                pair(s.gru.initial_hidden_state, t.gru.initial_hidden_state, H);
            }
        }
    for (int i = 0; i < n; i++) RLT_REQUIRE(sources[i] && targets[i]);
    return rlt_sac_polyak_list(device, sources, targets, counts, n, A->polyak);
}

// sac/operations_generic.h:395-468 on a sequence batch
int rlt_rocm_sac_sequence_train_actor(rlt_rocm_device* device, const rlt_sac_sequence_agent* A, const float* action_noise) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(sequence_agent_ok(A) && action_noise);
    RLT_REQUIRE(A->state_action_value_input && A->d_output && A->d_critic_input[0] && A->d_critic_input[1] && A->d_actor_output_squashing && A->d_actor_output &&
                A->actor_pre_squashing && A->actor_log_probabilities && A->actor_actions && A->log_alpha.gradient);
    const rlt_sequence_batch& K = A->batch;
    const int S = K.sequence_length, B = K.batch, OBS = A->observation_dim, ACT = A->action_dim, D = OBS + ACT, R = S * B;
    const size_t ws_bytes = sequence_pass_workspace_bytes(A, S + 1, B);
    void* ws = A->workspace; void* ws_side = (char*)A->workspace + ws_bytes;
    const bool overlap = S >= 48;      // short sequences: a pass is shorter than the two events that fork and join a stream cost on the host
    int rc;
    if ((rc = rlt_rocm_seq_zero_gradient(device, A->actor, A->n_actor_layers))) return rc;                                                  // :414
    if ((rc = rlt_rocm_fill_f32(device, A->log_alpha.gradient, 1, 1, 1, 0.0f))) return rc;
    const float* obs = K.observations_actions_base;
    if ((rc = rlt_rocm_seq_forward(device, A->actor, A->n_actor_layers, obs, D, K.reset, S, B, ws, ws_bytes))) return rc;                   // :427
    const float* actor_out = seq_output(A->actor, A->n_actor_layers);
    if ((rc = rlt_rocm_sas_forward(device, &A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT,
                                   A->actor_log_probabilities, R, ACT))) return rc;
    float* sav_actions = A->state_action_value_input + OBS;
    if ((rc = copy2d(device, A->actor_actions, ACT, sav_actions, D, R, ACT))) return rc;
    if ((rc = rlt_rocm_mask_copy(device, obs + OBS, D, sav_actions, D, K.final_step_mask, 1, R, ACT))) return rc;                           // :428-430
    if ((rc = copy2d(device, obs, D, A->state_action_value_input, D, R, OBS))) return rc;                                                   // :431
    // the gradient at the critics' outputs is a constant per row (:437-453): formed first, so that each critic's forward pass and its gradient towards the input
    // (:432-433, :458-459) can follow each other on a stream of their own -- critic 1 on the side stream, critic 0 on the main stream
    hipLaunchKernelGGL(sac_d_output_kernel, dim3(1), dim3(1024), 0, device->stream, (const float*)nullptr, (const float*)nullptr, (const uint8_t*)K.final_step_mask,
                       A->d_output, R, 1);
    if ((rc = rlt_launch_status(device))) return rc;
    // the inner layers of backward_input run without the reset mode (nn_models/sequential/operations_generic.h:399-407); the critics'
    // output layer has no activation function, so d_output survives the calls unchanged (both read it)
    for (int k = 1; k >= 0; k--) {
        const bool side = k == 1 && overlap && rlt_side_begin(device);
        void* w = side ? ws_side : ws;
        rc = rlt_rocm_seq_forward(device, A->critics[k], A->n_critic_layers, A->state_action_value_input, D, K.reset, S, B, w, ws_bytes);
        if (!rc) rc = rlt_rocm_seq_backward(device, A->critics[k], A->n_critic_layers, nullptr, 0, A->d_output, A->d_critic_input[k], K.reset, S, B, 0, 0, w, ws_bytes);
        rlt_side_end(device);
        if (rc) return rc;
    }
    if (overlap && (rc = rlt_side_join(device))) return rc;
    if ((rc = rlt_rocm_sac_min_value_d_output(device, seq_output(A->critics[0], A->n_critic_layers), seq_output(A->critics[1], A->n_critic_layers), A->d_critic_input[0],
                                             A->d_critic_input[1], D, D, ACT, A->d_actor_output_squashing, ACT, R))) return rc;             // :460
    if ((rc = rlt_rocm_mask_zero(device, A->d_actor_output_squashing, ACT, K.final_step_mask, 1, R, ACT))) return rc;                       // :461-463
    if ((rc = sas_backward_impl(device, &A->sas, actor_out, 2 * ACT, action_noise, ACT, A->actor_actions, ACT, A->actor_pre_squashing, ACT, A->d_actor_output_squashing, ACT,
                                A->d_actor_output, 2 * ACT, A->log_alpha.parameters, A->log_alpha.gradient, K.reset, R, ACT))) return rc;   // :464
    if ((rc = rlt_rocm_seq_backward(device, A->actor, A->n_actor_layers, obs, D, A->d_actor_output, nullptr, K.reset, S, B, 1, 0, ws, ws_bytes))) return rc;
    if ((rc = rlt_rocm_adam_step(device, A->actor_adam_tensors, A->n_actor_adam_tensors, &A->actor_adam, A->actor_age, 0.0f, nullptr))) return rc;   // :465
    return rlt_rocm_adam_step(device, &A->log_alpha, 1, &A->alpha_adam, A->alpha_age, 0.0f, nullptr);                                      // :466
}

}  // extern "C"
