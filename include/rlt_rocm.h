/*
 * rlt_rocm.h -- C ABI of the MI355X (gfx950) backend for the dense-network
 * training hot path of rl-tools.
 *
 * The reference library dispatches every operation by C++ overload on a device
 * tag (rl_tools/devices/cuda.h:52-122 is the tag this backend sits next to).
 * Each entry point below is what one such overload for a `devices::ROCM` tag
 * binds to; the comment above it names the reference function it stands in for.
 *
 * Conventions
 *  - every function returns 0 on success, a positive hipError_t value when the
 *    HIP runtime failed, or a negative RLT_E_* code for a rejected argument;
 *  - all data pointers are DEVICE pointers unless the name ends in `_host`;
 *  - matrices are row-major, fp32, with an explicit leading dimension (`ld*`,
 *    in elements) wherever a view of a wider matrix can be passed;
 *  - work is enqueued on the device handle's stream and returns without
 *    synchronising, except for the host<->device copies, which synchronise the
 *    stream like the reference's do (containers/matrix/operations_cuda.h:149-195);
 *  - boolean tensors of the reference (terminated, masks) are uint8_t here.
 */
#ifndef RLT_ROCM_H
#define RLT_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RLT_E_INVALID_ARGUMENT (-1) /* null pointer, non-positive dimension, ld too small */
#define RLT_E_UNSUPPORTED      (-2) /* shape outside what the kernels are built for      */
#define RLT_E_NOT_INITIALISED  (-3)
#define RLT_E_DEVICE_TIMEOUT   (-4) /* a persistent kernel gave up waiting for another workgroup (reported by check_status) */
#define RLT_E_WORKSPACE_TOO_SMALL (-5) /* the call needs more scratch memory than the fixed array of RLT_STATIC_SCRATCH_BYTES holds */
#define RLT_E_CAPTURING (-6)           /* the call allocates, frees, copies to or from the host or waits while the stream records a graph */

/* nn/activation_functions.h:11-18 -- same numbering as the reference enum */
enum rlt_activation {
    RLT_ACT_IDENTITY  = 0,
    RLT_ACT_RELU      = 1,
    RLT_ACT_GELU      = 2,
    RLT_ACT_TANH      = 3,
    RLT_ACT_FAST_TANH = 4,
    RLT_ACT_SIGMOID   = 5
};

/* Opaque device object: one HIP device + one stream (devices/cuda.h:52-77 holds
 * the same for CUDA plus a BLAS handle, which this backend has no use for). */
typedef struct rlt_rocm_device rlt_rocm_device;

/* ---------------------------------------------------------------- device -- */

/* init(device)            devices/cuda.h:130-154 */
int rlt_rocm_init(int hip_device_index, rlt_rocm_device** out_device);
/* (no counterpart: the reference never destroys its handle) */
int rlt_rocm_destroy(rlt_rocm_device* device);
/* check_status(device)    devices/cuda.h:156-174 -- synchronises, returns the sticky error */
int rlt_rocm_check_status(rlt_rocm_device* device);
/* Adopt a caller-owned hipStream_t (NULL selects the handle's own stream again). */
int rlt_rocm_set_stream(rlt_rocm_device* device, void* hip_stream);
void* rlt_rocm_get_stream(rlt_rocm_device* device);
/* Human-readable text for any code returned by this library. */
const char* rlt_rocm_error_string(int code);
/* Number of compute units and LDS bytes per workgroup the kernels were sized against. */
int rlt_rocm_device_info(rlt_rocm_device* device, int* compute_units, int* lds_bytes, char* name, int name_len);

/* ------------------------------------------------------------ containers -- */

/* malloc / free           containers/matrix/operations_cuda.h:16-45, tensor/operations_cuda.h:15-39 */
int rlt_rocm_malloc(rlt_rocm_device* device, void** out_ptr, size_t bytes);
int rlt_rocm_free(rlt_rocm_device* device, void* ptr);
/* copy (dense)            containers/matrix/operations_cuda.h:105-195 */
int rlt_rocm_memcpy_h2d(rlt_rocm_device* device, void* dst, const void* src_host, size_t bytes);
int rlt_rocm_memcpy_d2h(rlt_rocm_device* device, void* dst_host, const void* src, size_t bytes);
int rlt_rocm_memcpy_d2d(rlt_rocm_device* device, void* dst, const void* src, size_t bytes);
/* copy (strided views)    containers/matrix/operations_cuda.h:48-60,98-103 ; tensor copy2d :94-168
 * kind: 0 = device->device, 1 = host->device, 2 = device->host; widths/pitches in bytes. */
int rlt_rocm_memcpy2d(rlt_rocm_device* device, void* dst, size_t dst_pitch, const void* src, size_t src_pitch,
                      size_t width_bytes, size_t rows, int kind);
/* set_all                 containers/matrix/operations_cuda.h:62-74,201-207 */
int rlt_rocm_fill_f32(rlt_rocm_device* device, float* dst, int rows, int cols, int ld, float value);
int rlt_rocm_fill_u8(rlt_rocm_device* device, uint8_t* dst, size_t count, uint8_t value);
/* set_all(t, value tensor) containers/tensor/operations_cuda.h:341-347: every element becomes the scalar `value` points to on the DEVICE
 * (e.g. a loss weight computed by an earlier launch), no host round trip */
int rlt_rocm_fill_from_f32(rlt_rocm_device* device, float* dst, int rows, int cols, int ld, const float* value);
/* randn / rand            containers/tensor/operations_cuda.h:548-624
 * Counter-based (Philox4x32-10): element i of a call is word i % 4 of group i / 4 of the sequence that (seed, stream) selects --
 * key = seed, counter = (group index, stream). No state array exists. Calls with different `stream` values (or seeds) draw from
 * disjoint sequences of 2^64 groups whatever their lengths, so a caller that passes a fresh stream number per call (a counter it
 * increments, as the reference advances its generator state) never sees a value twice. rand is uniform on (low, high) from 24 bits
 * per value, randn is Box-Muller on the two word pairs of a group. */
int rlt_rocm_randn_f32(rlt_rocm_device* device, float* dst, size_t count, uint64_t seed, uint64_t stream);
int rlt_rocm_rand_f32(rlt_rocm_device* device, float* dst, size_t count, float low, float high, uint64_t seed, uint64_t stream);
/* The raw 32-bit words of the same sequence (no counterpart in the reference: lets a caller check the generator against the
 * published Philox4x32-10 vectors or build other distributions). */
int rlt_rocm_rand_bits_u32(rlt_rocm_device* device, uint32_t* dst, size_t count, uint64_t seed, uint64_t stream);
/* scale(t, s, reciprocal) containers/tensor/operations_generic.h:433-445,713 : x <- reciprocal ? (1/x)*s : x*s (rounded in that order) */
int rlt_rocm_scale_f32(rlt_rocm_device* device, float* x, size_t count, float s, int reciprocal);
/* cast_reduce_sum<T>(bool tensor) containers/tensor/operations_generic.h:928-985 (CUDA: <<<1,1>>>, operations_cuda.h:287-307) */
int rlt_rocm_cast_reduce_sum_u8(rlt_rocm_device* device, const uint8_t* mask, size_t count, float* out_sum);
/* sum / squared-sum of a float tensor (gradient_norm, nn/parameters/operations_generic.h) */
int rlt_rocm_reduce_sum_f32(rlt_rocm_device* device, const float* x, size_t count, int squared, float* out_sum);

/* unary_operation(device, op, t[, output])   containers/tensor/operations_generic.h:573-640 with the functors of :365-446, on a 2-D view
 * [rows x cols] (a contiguous tensor is one row); dst may be src. `parameter` is the functor's parameter (CONSTANT: the value; SCALE and
 * SCALE_RECIPROCAL: the factor, the latter computing 1 / a * factor as Scale<..., RECIPROCAL> does). SIGMOID saturates beyond +-20 as :395-400. */
enum { RLT_UNARY_NEGATE = 0, RLT_UNARY_ABS, RLT_UNARY_CONSTANT, RLT_UNARY_SIGMOID, RLT_UNARY_FAST_SIGMOID, RLT_UNARY_EXP, RLT_UNARY_TANH, RLT_UNARY_FAST_TANH,
       RLT_UNARY_ONE_MINUS, RLT_UNARY_SCALE, RLT_UNARY_SCALE_RECIPROCAL };
int rlt_rocm_unary_f32(rlt_rocm_device* device, int operation, float parameter, const float* src, int ld_src, float* dst, int ld_dst, int rows, int cols);
/* binary_operation(device, op, a, b, output)   :641-700 with Add / Subtract / Multiply / Divide (:448-471); dst may be a or b */
enum { RLT_BINARY_ADD = 0, RLT_BINARY_SUBTRACT, RLT_BINARY_MULTIPLY, RLT_BINARY_DIVIDE };
int rlt_rocm_binary_f32(rlt_rocm_device* device, int operation, const float* a, int lda, const float* b, int ldb, float* dst, int ld_dst, int rows, int cols);
/* ternary_operation with MultiplyAccumulate (:475-481, :701-760): dst = accumulator + a * b, the product rounded before the addition */
int rlt_rocm_multiply_accumulate_f32(rlt_rocm_device* device, const float* a, int lda, const float* b, int ldb, const float* accumulator, int ldc,
                                     float* dst, int ld_dst, int rows, int cols);
/* unary_associative_reduce with the abs-max operation (:762-800; CUDA <<<1,1>>>, operations_cuda.h:287-307): max |x| into a device scalar (0 for count 0) */
int rlt_rocm_reduce_abs_max_f32(rlt_rocm_device* device, const float* x, size_t count, float* out_max);

/* ------------------------------------------------------------ dense / MLP -- */

/* One dense layer as the reference stores it (nn/layers/dense/layer.h:82-135 plus the Adam
 * parameter instances, nn/optimizers/adam/adam.h:76-96). Unused members may be NULL. */
typedef struct rlt_dense_layer {
    float* weights;          /* [out_dim x in_dim], row-major, packed          */
    float* biases;           /* [out_dim]                                      */
    float* d_weights;        /* gradient accumulators (LayerGradient)          */
    float* d_biases;
    float* pre_activations;  /* [batch x out_dim] packed (LayerBackward)       */
    float* output;           /* [batch x out_dim] packed (LayerGradient)       */
    int32_t in_dim;
    int32_t out_dim;
    int32_t activation;      /* enum rlt_activation                            */
    int32_t reserved;
} rlt_dense_layer;

/* evaluate(dense)         nn/layers/dense/operations_cpu_blas.h:36-72, operations_cuda.h:237-276
 * y = act(x W^T + b); nothing is stored in the layer. */
int rlt_rocm_dense_evaluate(rlt_rocm_device* device, const rlt_dense_layer* layer,
                            const float* x, int ldx, float* y, int ldy, int batch);
/* forward(dense)          nn/layers/dense/operations_cpu_blas.h:74-116, operations_cuda.h:278-316
 * also stores layer->pre_activations and (if non-NULL) layer->output; y may be NULL. */
int rlt_rocm_dense_forward(rlt_rocm_device* device, const rlt_dense_layer* layer,
                           const float* x, int ldx, float* y, int ldy, int batch);
/* backward_input(dense)   operations_cpu_blas.h:219-223: d_output <- d_pre = act'(pre) * d_output, d_input = d_pre W */
int rlt_rocm_dense_backward_input(rlt_rocm_device* device, const rlt_dense_layer* layer,
                                  float* d_output, int ldd, float* d_input, int ldi, int batch);
/* backward(dense)         operations_cpu_blas.h:143-186: d_output <- d_pre, d_biases += sum_batch d_pre, d_weights += d_pre^T x */
int rlt_rocm_dense_backward(rlt_rocm_device* device, const rlt_dense_layer* layer,
                            const float* x, int ldx, float* d_output, int ldd, int batch);
/* backward(dense) WITHOUT ANY ALLOCATION. No counterpart in the reference. For callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. rlt_rocm_dense_backward splits the batch over
 * workgroups and keeps their partial sums in a workspace the handle grows on demand; this variant keeps them in a fixed array of
 * RLT_STATIC_SCRATCH_BYTES that is part of the library's device image (each GPU the library is initialised on holds one copy until
 * the process ends) and calls neither hipMalloc nor hipFree nor any allocating routine. Same arguments, same launches and bit for
 * bit the same results as rlt_rocm_dense_backward. It returns RLT_E_WORKSPACE_TOO_SMALL when
 * splits * (out_dim * in_dim + out_dim) * 4 bytes exceed the array (splits = min(ceil(batch / 256), about two workgroups per compute
 * unit divided by the number of output tiles); every 64-wide layer fits at any batch, a 256 x 256 layer up to batch 16,128).
 * All calls on one GPU share the array, whatever handle or stream they use: calls that overlap on one GPU race; order them. */
#define RLT_STATIC_SCRATCH_BYTES (16u << 20)
int rlt_rocm_dense_backward_static(rlt_rocm_device* device, const rlt_dense_layer* layer,
                                   const float* x, int ldx, float* d_output, int ldd, int batch);
/* backward_full(dense)    operations_cpu_blas.h:224-228 = backward + d_input */
int rlt_rocm_dense_backward_full(rlt_rocm_device* device, const rlt_dense_layer* layer,
                                 const float* x, int ldx, float* d_output, int ldd,
                                 float* d_input, int ldi, int batch);

/* Workspace an MLP call needs (the reference's tick/tock buffers, nn_models/mlp/network.h:127-140):
 * bytes for `batch` rows through `layers`. */
size_t rlt_rocm_mlp_workspace_bytes(const rlt_dense_layer* layers, int n_layers, int batch);
/* evaluate(mlp)           nn_models/mlp/operations_generic.h:77-102 */
int rlt_rocm_mlp_evaluate(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers,
                          const float* x, int ldx, float* y, int ldy, int batch,
                          void* workspace, size_t workspace_bytes);
/* forward(mlp)            nn_models/mlp/operations_generic.h:103-114 (stores pre_activations/output of every layer) */
int rlt_rocm_mlp_forward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers,
                         const float* x, int ldx, int batch);
/* backward / backward_full / backward_input (mlp)   nn_models/mlp/operations_generic.h:126-204
 *   want_weight_gradients = 0 -> backward_input, 1 -> backward (d_input == NULL) or backward_full.
 * d_output is overwritten with the last layer's d_pre, as in the reference. */
int rlt_rocm_mlp_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers,
                          const float* x, int ldx, float* d_output, int ldd,
                          float* d_input, int ldi, int batch, int want_weight_gradients,
                          void* workspace, size_t workspace_bytes);
/* zero_gradient(mlp)      nn_models/mlp/operations_generic.h:117-124 */
int rlt_rocm_mlp_zero_gradient(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers);

/* Fused forward + backward of a whole MLP for a caller that already holds the upstream gradient
 * (the standalone microbenchmark shape, and PPO's critic where d_output = mse gradient is fused via
 * `target`): one pass over the batch, activations never leave the chip.
 *   y           [batch x out] network output (may be NULL)
 *   d_output    [batch x out] upstream gradient, used when target == NULL (not modified)
 *   target      if non-NULL, d_output is formed as (y - target) * mse_scale instead
 * Weight/bias gradients are ACCUMULATED into the layers' d_weights/d_biases (beta = 1, as the
 * reference's backward does). No pre_activations/output are stored. */
int rlt_rocm_mlp_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers,
                                  const float* x, int ldx, float* y, int ldy,
                                  const float* d_output, int ldd,
                                  const float* target, int ldt, float mse_scale,
                                  int batch, void* workspace, size_t workspace_bytes);

/* The same with the gradient with respect to the input as a further output, d_input [batch x in] (overwritten): forward + loss gradient +
 * backward_full of a network that sits on top of another model, e.g. a head in -> 64 -> out on a recurrent layer's output, in one pass over
 * the batch where the network is in -> 64 -> out or in -> 64 -> 64 -> out (in <= 128, out <= 16). */
int rlt_rocm_mlp_forward_backward_input(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers,
                                        const float* x, int ldx, float* y, int ldy,
                                        const float* d_output, int ldd,
                                        const float* target, int ldt, float mse_scale,
                                        float* d_input, int ldi,
                                        int batch, void* workspace, size_t workspace_bytes);

/* -------------------------------------------------------- optimiser/polyak -- */

/* nn/optimizers/adam/adam.h:13-48 (Parameters<T>); the *_TENSORFLOW defaults are
 * alpha 1e-3, beta (0.9, 0.999), epsilon = epsilon_sqrt = 1e-7; *_PYTORCH uses 1e-8. */
typedef struct rlt_adam_parameters {
    float alpha, beta_1, beta_2, epsilon, epsilon_sqrt;
    float weight_decay;      /* applied to entries flagged is_weight when enable_weight_decay */
    float bias_lr_factor;    /* applied to entries flagged is_bias when enable_bias_lr_factor */
    int32_t enable_weight_decay;
    int32_t enable_bias_lr_factor;
    int32_t enable_gradient_clipping;
    float gradient_clip_value;
} rlt_adam_parameters;

/* One parameter tensor with its Adam state (nn/optimizers/adam/adam.h:76-96). */
typedef struct rlt_adam_tensor {
    float* parameters;
    float* gradient;
    float* first_moment;
    float* second_moment;
    float* polyak_target;   /* optional: target <- polyak*target + (1-polyak)*new_parameter, fused */
    uint32_t count;
    uint32_t flags;         /* bit0: is_weight, bit1: is_bias */
} rlt_adam_tensor;

/* step(optimizer, model)  nn/optimizers/adam/operations_generic.h:49-66 + instance/operations_generic.h:26-72
 * `age` is a device-resident uint32 (starts at 1, operations_generic.h:43-47); the bias corrections
 * 1/(1-beta^age) are computed on the device from it and it is incremented by the same launch, so no
 * host round trip is needed (the reference spends a <<<1,1>>> kernel on this, adam/operations_cuda.h:18-68).
 * `tensors_host` is a host array; it is copied into the launch. polyak is ignored where polyak_target == NULL.
 * If out_gradient_squared_norm is non-NULL it receives sum(g^2) over all tensors. */
int rlt_rocm_adam_step(rlt_rocm_device* device, const rlt_adam_tensor* tensors_host, int n_tensors,
                       const rlt_adam_parameters* parameters_host, uint32_t* age,
                       float polyak, float* out_gradient_squared_norm);
/* reset_optimizer_state   adam/operations_generic.h:43-47: age <- 1, moments <- 0 */
int rlt_rocm_adam_reset(rlt_rocm_device* device, const rlt_adam_tensor* tensors_host, int n_tensors, uint32_t* age);
/* utils::polyak::update / update_squared   utils/polyak/operations_generic.h:11-43, operations_cuda.h:13-48 */
int rlt_rocm_polyak_update(rlt_rocm_device* device, const float* source, float* target, size_t count,
                           float polyak, int squared);
/* The same soft update for a list of tensors (e.g. every tensor of both target critics) in one launch per 16 tensors. */
int rlt_rocm_polyak_update_list(rlt_rocm_device* device, const float* const* sources, float* const* targets, const uint32_t* counts,
                                int n_tensors, float polyak);

/* ------------------------------------------------------------------- loss -- */

/* mse::gradient           nn/loss_functions/mse/operations_generic.h:41-97, operations_cuda.h:13-57
 * d_a = (a - b) * 2/(rows*cols) * w ; w = *loss_weight_device if non-NULL else loss_weight. */
int rlt_rocm_mse_gradient(rlt_rocm_device* device, const float* a, int lda, const float* b, int ldb,
                          float* d_a, int ldda, int rows, int cols,
                          float loss_weight, const float* loss_weight_device);
/* mse::evaluate           mse/operations_generic.h:9-21 : out = sum((a-b)^2) * w / (rows*cols) */
int rlt_rocm_mse_evaluate(rlt_rocm_device* device, const float* a, int lda, const float* b, int ldb,
                          int rows, int cols, float loss_weight, float* out_loss);

/* ----------------------------------------------------- sample_and_squash -- */

/* nn/layers/sample_and_squash/layer.h:29-39 */
typedef struct rlt_sas_parameters {
    float log_std_lower_bound;   /* -20 */
    float log_std_upper_bound;   /*   2 */
    float log_probability_epsilon; /* 1e-6 */
    float target_entropy;        /* -action_dim */
} rlt_sas_parameters;

/* evaluate / forward      sample_and_squash/operations_generic.h:148-280, operations_cuda.h:17-56
 *   input  [batch x 2*dim] = [mean | log_std]; noise [batch x dim] (NULL = zeros, i.e. Evaluation mode
 *   without the sample path: action = tanh(mean)); actions [batch x dim];
 *   log_probabilities [batch]; pre_squashing [batch x dim] may be NULL (evaluate does not keep it). */
int rlt_rocm_sas_forward(rlt_rocm_device* device, const rlt_sas_parameters* p,
                         const float* input, int ldin, const float* noise, int ldn,
                         float* actions, int lda, float* pre_squashing, int ldp,
                         float* log_probabilities, int batch, int dim);
/* backward_full           sample_and_squash/operations_generic.h:289-398, operations_cuda.h:58-115
 *   d_input [batch x 2*dim]; d_log_alpha (device scalar) is INCREMENTED by
 *   mean_batch( alpha * (-log_prob - target_entropy) ), alpha = exp(*log_alpha). */
int rlt_rocm_sas_backward(rlt_rocm_device* device, const rlt_sas_parameters* p,
                          const float* input, int ldin, const float* noise, int ldn,
                          const float* actions, int lda, const float* pre_squashing, int ldp,
                          const float* d_output, int lddo, float* d_input, int lddi,
                          const float* log_alpha, float* d_log_alpha, int batch, int dim);

/* ------------------------------------------------------------------ SAC --- */

/* target_action_values    rl/algorithms/sac/operations_generic.h:133-179, operations_cuda.h:12-44
 *   y = r + gamma * (!terminated) * (min(q1, q2) - exp(log_alpha) * log_prob) */
int rlt_rocm_sac_target_action_values(rlt_rocm_device* device, const float* q1_next, const float* q2_next,
                                      const float* rewards, const uint8_t* terminated,
                                      const float* next_log_probabilities, const float* log_alpha,
                                      float gamma, int ignore_termination, float* target, int batch);
/* min_value_d_output      sac/operations_generic.h:358-393, operations_cuda.h:88-128 */
int rlt_rocm_sac_min_value_d_output(rlt_rocm_device* device, const float* q1, const float* q2,
                                    const float* d_critic_1_input, const float* d_critic_2_input, int ld_critic_input,
                                    int critic_input_dim, int action_dim, float* d_actor_output, int ldo, int batch);
/* mask_actions            sac/operations_generic.h:181-209, operations_cuda.h:47-66 : rows where (mask != invert) are copied */
int rlt_rocm_mask_copy(rlt_rocm_device* device, const float* source, int lds, float* target, int ldt,
                       const uint8_t* mask, int invert, int rows, int cols);
/* mask_gradient           sac/operations_generic.h:210-234, operations_cuda.h:68-86 : rows where (mask != invert) are zeroed */
int rlt_rocm_mask_zero(rlt_rocm_device* device, float* gradient, int ld, const uint8_t* mask, int invert, int rows, int cols);

/* Everything one SAC agent owns on the device (rl/algorithms/sac/sac.h:62-145 ActorCritic and the
 * Critic/ActorTrainingBuffers, plus the batch of rl/components/off_policy_runner/off_policy_runner.h:89-156
 * for SEQUENCE_LENGTH = 1). All networks are MLPs described by rlt_dense_layer arrays (host arrays of
 * descriptors whose pointers are device pointers). */
typedef struct rlt_sac_agent {
    int32_t batch, observation_dim, action_dim, n_actor_layers, n_critic_layers;
    float gamma, polyak, reserved0;
    rlt_sas_parameters sas;
    rlt_adam_parameters actor_adam, critic_adam, alpha_adam;
    const rlt_dense_layer* actor;            /* out_dim of last layer = 2*action_dim */
    const rlt_dense_layer* critics[2];
    const rlt_dense_layer* critics_target[2];
    const rlt_adam_tensor* actor_adam_tensors;      int32_t n_actor_adam_tensors;   int32_t pad0;
    const rlt_adam_tensor* critic_adam_tensors[2];  int32_t n_critic_adam_tensors;  int32_t pad1;
    /* log_alpha as an Adam parameter instance (count = 1) */
    rlt_adam_tensor log_alpha;
    uint32_t* actor_age; uint32_t* critic_age[2]; uint32_t* alpha_age;
    /* batch (SequentialBatch, SEQUENCE_LENGTH = 1): [2 x batch x (obs+act)] */
    float* observations_actions_base;
    float* rewards;            /* [batch] */
    uint8_t* terminated;       /* [batch] */
    /* masks of the batch; NULL means all true, which is what gather_batch yields for SEQUENCE_LENGTH = 1 */
    const uint8_t* final_step_mask;        /* [batch] */
    const uint8_t* next_final_step_mask;   /* [batch] */
    const uint8_t* reset;                  /* [batch] */
    /* training buffers */
    float* next_state_action_value_input;   /* [batch x (obs+act)] */
    float* next_q[2];                        /* [batch] each */
    float* next_log_probabilities;           /* [batch] */
    float* target_action_value;              /* [batch] */
    float* d_output_critic[2];               /* [batch] */
    float* state_action_value_input;         /* [batch x (obs+act)] (actor training) */
    float* d_output_actor_critics;           /* [batch] */
    float* d_critic_input[2];                /* [batch x (obs+act)] */
    float* d_actor_output_squashing;         /* [batch x act] */
    float* d_actor_output;                   /* [batch x 2*act] */
    float* actor_pre_squashing;              /* [batch x act] */
    float* actor_log_probabilities;          /* [batch] */
    float* actor_actions;                    /* [batch x act] (sample_and_squash layer output) */
    void* workspace; size_t workspace_bytes;
} rlt_sac_agent;

/* train_critic            rl/algorithms/sac/operations_generic.h:243-337 for critic `critic_index`;
 *   action_noise [batch x action_dim] is the externally drawn N(0,1) noise.
 *   Two implementations with the same results (to fp32 rounding). Where every network is in -> 64 -> 64 -> out with one hidden
 *   activation (not GELU) and no output activation, obs + act <= 128, act <= 8 and all three masks are NULL, train_critic and
 *   train_actor each run as two launches (all network passes of the update; sum of the workgroups' partial gradients + Adam, or three
 *   where the Adam tensors are not the network's gradient buffers) and update_critic_targets as one;
 *   of the training buffers only next_log_probabilities and target_action_value (critic), actor_log_probabilities, actor_actions and
 *   actor_pre_squashing (actor) are then written, and the gradients are overwritten without a prior zero_gradient. Every other
 *   agent, or any agent after rlt_rocm_sac_set_per_operation(device, 1), takes one launch per reference operation and fills every
 *   training buffer. */
int rlt_rocm_sac_train_critic(rlt_rocm_device* device, const rlt_sac_agent* agent, int critic_index,
                              const float* action_noise);
/* update_critic_targets   sac/operations_generic.h:488-527 */
int rlt_rocm_sac_update_critic_targets(rlt_rocm_device* device, const rlt_sac_agent* agent);
/* train_actor             sac/operations_generic.h:395-468 */
int rlt_rocm_sac_train_actor(rlt_rocm_device* device, const rlt_sac_agent* agent, const float* action_noise);
/* (no counterpart) enabled != 0: the three calls above, and rlt_rocm_td3_train_critic / _train_actor, always take the one-launch-per-operation path. */
int rlt_rocm_sac_set_per_operation(rlt_rocm_device* device, int enabled);

/* ------------------------------------------------- replay buffer / runner -- */

/* Replay storage of one off-policy runner (rl/components/replay_buffer/replay_buffer.h:32-62):
 * the reference keeps one ring per environment; here the rings of all environments live in one
 * allocation, ring e at rows [e*capacity, (e+1)*capacity). Row layout (floats):
 * [obs | action | reward | next_obs | terminated | truncated], row_dim = 2*obs + act + 3. */
typedef struct rlt_replay_buffer {
    float* data;              /* [n_envs*capacity x row_dim]                 */
    uint32_t* episode_start;  /* [n_envs*capacity]                           */
    uint32_t* position;       /* [n_envs] device-resident ring cursors       */
    uint32_t* current_episode_start; /* [n_envs]                             */
    uint8_t* full;            /* [n_envs]                                    */
    int32_t n_envs, capacity, observation_dim, action_dim;
} rlt_replay_buffer;

/* add                     replay_buffer/operations_generic.h:54-78, one transition per environment:
 *   observations/next_observations [n_envs x obs], actions [n_envs x act], rewards [n_envs],
 *   terminated/truncated [n_envs]. Advances every ring cursor on the device. */
int rlt_rocm_replay_add(rlt_rocm_device* device, const rlt_replay_buffer* rb,
                        const float* observations, const float* actions, const float* rewards,
                        const float* next_observations, const uint8_t* terminated, const uint8_t* truncated);

/* gather_batch (SEQUENCE_LENGTH = 1)   off_policy_runner/operations_generic.h:240-430, operations_cuda.h:37-55,170-181
 *   env_indices[i], sample_offsets[i]: the two draws the reference makes per sample (host-drawn and copied
 *   for parity, or produced by rlt_rocm_gather_draw). deterministic != 0 uses offset = i, env = 0
 *   (the reference's DETERMINISTIC template flag). max_episode_length enters the ring-wrap index
 *   (position + max_episode_length + offset) % capacity once a ring is full.
 *   Outputs: observations_actions_base [2 x batch x (obs+act)], rewards [batch], terminated [batch],
 *   and the masks (reset, next_reset_base[2 x batch], final_step_mask, next_final_step_mask_base[2 x batch];
 *   any may be NULL). */
int rlt_rocm_gather_batch(rlt_rocm_device* device, const rlt_replay_buffer* rb,
                          const uint32_t* env_indices, const uint32_t* sample_offsets, int deterministic,
                          int max_episode_length, int batch,
                          float* observations_actions_base, float* rewards, uint8_t* terminated,
                          uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base);
/* SequentialBatch for any SEQUENCE_LENGTH (off_policy_runner.h:102-156); padded = sequence_length + 1. */
typedef struct rlt_sequence_batch {
    float* observations_actions_base;    /* [padded x batch x (obs + act)] */
    float* rewards;                      /* [sequence_length x batch] */
    uint8_t* terminated;                 /* [sequence_length x batch] */
    uint8_t* reset;                      /* [sequence_length x batch] */
    uint8_t* next_reset_base;            /* [padded x batch] */
    uint8_t* final_step_mask;            /* [sequence_length x batch] */
    uint8_t* next_final_step_mask_base;  /* [padded x batch] */
    int32_t batch, sequence_length;
} rlt_sequence_batch;
/* SequentialBatchParameters (off_policy_runner.h:79-87; the defaults switch the first two on for sequence_length > 1) */
typedef struct rlt_sequence_sampling {
    int32_t always_sample_from_initial_state, random_seq_length, enable_nominal_sequence_length_probability;
    float nominal_sequence_length_probability;
    int32_t include_first_step_in_targets;   /* 0: the `next` views start at padded step 1 (the default for sequence_length = 1), so the first
                                                 next_reset flag lands in next_reset_base[1] (operations_generic.h:85-92,286) */
} rlt_sequence_sampling;
/* The random draws of gather_batch, per sample in the order the sample consumes each kind (k-th use by sample b = entry
 * [b][k]); a sample restarts at most `padded` times and decides a sequence length at most padded + 1 times. */
typedef struct rlt_sequence_draws {
    const uint32_t* env_indices;      /* [batch]                  uniform_int(0, n_envs - 1), :426                       */
    const uint32_t* sample_offsets;   /* [batch x padded]         uniform_int(0, eligible rows - 1) at every (re)start, :305 */
    const uint8_t* nominal;           /* [batch x (padded + 1)]   1 where uniform_real(0, 1) < nominal probability, :267,362 */
    const uint32_t* lengths;          /* [batch x (padded + 1)]   uniform_int(1, sequence_length - 1), used where nominal = 0, :272,367 */
} rlt_sequence_draws;
/* gather_batch / gather_batch_step for sequences, rl/components/off_policy_runner/operations_generic.h:239-430: every sample
 * walks `padded` steps through one environment's ring from a drawn row (or from the first step of that row's episode),
 * copies observation / action / reward / terminated, ends a sequence at an episode end, at the ring's cursor, after a drawn
 * length or at the last step, writes the next observation and a zero action into the following step and restarts there
 * from a new draw; reset / final-step masks mark the boundaries. Entries the reference leaves untouched are left untouched.
 * Bit-exact (copies and index arithmetic). With sequence_length = 1 and both switches off it equals rlt_rocm_gather_batch. */
int rlt_rocm_gather_sequence_batch(rlt_rocm_device* device, const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling,
                                   const rlt_sequence_draws* draws, int max_episode_length, const rlt_sequence_batch* batch);

/* Device-side draw of (env, offset) pairs, uniform over the eligible rows of each ring
 * (off_policy_runner/operations_generic.h:257,304,426): sample i takes words 0 and 1 of Philox group i of the sequence that
 * (seed, stream) selects (see rlt_rocm_randn_f32); pass a fresh stream number per call. */
int rlt_rocm_gather_draw(rlt_rocm_device* device, const rlt_replay_buffer* rb, int batch,
                         uint64_t seed, uint64_t stream, uint32_t* env_indices, uint32_t* sample_offsets);

/* Device-side draws for rlt_rocm_gather_sequence_batch: fills the four arrays of rlt_sequence_draws (sizes as documented there) with what
 * gather_batch draws per sample (off_policy_runner/operations_generic.h:257-275,304,362-371,426): the environment; an offset uniform over the
 * eligible rows of that environment's ring for each of the `padded` possible (re)starts (capacity - max_episode_length rows of a full ring when
 * sequences start at episode starts); for each of the padded + 1 possible length decisions whether the nominal length is taken
 * (uniform_real < nominal_sequence_length_probability) and a length uniform in [1, sequence_length - 1]. Sample b takes the words of Philox
 * groups [b G, (b + 1) G), G = ceil((3 padded + 3) / 4), of the sequence that (seed, stream) selects, in that order. */
int rlt_rocm_gather_sequence_draw(rlt_rocm_device* device, const rlt_replay_buffer* rb, const rlt_sequence_sampling* sampling,
                                  int max_episode_length, int batch, int sequence_length, uint64_t seed, uint64_t stream,
                                  uint32_t* env_indices, uint32_t* sample_offsets, uint8_t* nominal, uint32_t* lengths);

/* rl/environments/pendulum/pendulum.h:12-25 */
typedef struct rlt_pendulum_parameters {
    float g, max_speed, max_torque, dt, m, l;
} rlt_pendulum_parameters;

/* step + reward + observe  rl/environments/pendulum/operations_generic.h:79-101,131-160
 *   states [n_envs x 2] = (theta, theta_dot) updated in place; actions [n_envs] (un-clamped);
 *   observations (pre-step) and next_observations [n_envs x 3]; rewards [n_envs]. */
int rlt_rocm_pendulum_step(rlt_rocm_device* device, const rlt_pendulum_parameters* p, float* states,
                           const float* actions, float* observations, float* next_observations,
                           float* rewards, int n_envs);

/* rl/environments/acrobot/acrobot.h:14-37 (DefaultParameters; EasyParameters widen the torque range to +-10) */
typedef struct rlt_acrobot_parameters {
    float dt, link_length_1, link_length_2, link_mass_1, link_mass_2, link_com_pos_1, link_com_pos_2, link_moi;
    float max_vel_1, max_vel_2, min_torque, max_torque;
} rlt_acrobot_parameters;

/* step + reward + terminated + observe of the Acrobot (swingup = 0) or the AcrobotSwingup (swingup = 1)
 * rl/environments/acrobot/operations_generic.h:56-117 (dsdt, rk4), :118-144 (step), :145-171 (reward), :173-193 (observe, terminated)
 *   states [n_envs x 4] = (theta_1, theta_2, theta_1_dot, theta_2_dot) updated in place; actions [n_envs] (un-clamped, in [-1, 1]
 *   after clamping, scaled to [min_torque, max_torque]); observations (pre-step) and next_observations [n_envs x 6];
 *   rewards [n_envs]; terminated [n_envs] of the NEXT state. Any output may be NULL. */
int rlt_rocm_acrobot_step(rlt_rocm_device* device, const rlt_acrobot_parameters* p, int swingup, float* states, const float* actions,
                          float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n_envs);

/* rl/environments/car/car.h:13-33 (Parameters with the front / rear tire coefficients B, C, D) */
typedef struct rlt_car_parameters {
    float g, m, I, lf, lr, tf_B, tf_C, tf_D, tr_B, tr_C, tr_D, cm, cr0, cr2, vt, dt;
} rlt_car_parameters;

/* step + reward + terminated + observe of the Car (the variant without a track)
 * rl/environments/car/operations_generic.h:80-84 (terminated), :99-127 (step: single-track model with Pacejka tire forces, explicit
 * Euler), :128-135 (reward from the pre-step state), :143-155 (observe = the state)
 *   states [n_envs x 6] = (x, y, mu, vx, vy, omega) updated in place; actions [n_envs x 2] = (throttle / brake, steering), clamped
 *   to [-1, 1]; observations (pre-step) and next_observations [n_envs x 6]; rewards [n_envs]; terminated [n_envs] of the NEXT
 *   state. Any output may be NULL. */
int rlt_rocm_car_step(rlt_rocm_device* device, const rlt_car_parameters* p, float* states, const float* actions,
                      float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n_envs);

/* The Car on a track (CarTrack, rl/environments/car/car.h:34-41,101-108): `track` is a height x width bitmap (1 = drivable) of square cells
 * `track_scale` metres wide, centred on the origin, row 0 at the top (largest y).
 *   terminated (operations_generic.h:85-98): the next state's cell is not drivable or lies outside the bitmap
 *   reward (:136-141): the pre-step forward speed vx;  step: as rlt_rocm_car_step
 *   observe (:156-190): the state, then for the directions -20, 0, +20 degrees off the heading the distance to the first cell that is
 *   not drivable along a ray of 50 steps of half a cell, as a fraction of the ray's length. A ray that leaves the bitmap ends there
 *   (the reference reads past the array in that case).
 *   states [n_envs x 6], actions [n_envs x 2], observations and next_observations [n_envs x 9]. Any output may be NULL. */
int rlt_rocm_car_track_step(rlt_rocm_device* device, const rlt_car_parameters* p, const uint8_t* track, int height, int width, float track_scale,
                            float* states, const float* actions, float* observations, float* next_observations, float* rewards,
                            uint8_t* terminated, int n_envs);

/* Per-environment runner state (rl/components/off_policy_runner/off_policy_runner.h:184-221). */
typedef struct rlt_pendulum_runner {
    float* states;            /* [n_envs x 2]  */
    uint32_t* episode_step;   /* [n_envs]      */
    float* episode_return;    /* [n_envs]      */
    uint8_t* truncated;       /* [n_envs] initialised to 1 */
    int32_t n_envs, episode_step_limit;
    rlt_pendulum_parameters env;
} rlt_pendulum_runner;

/* One off-policy runner step for all environments in a single launch
 * (prologue/interlude/epilogue, off_policy_runner/operations_generic.h:183-238, _per_env.h:8-108,
 * operations_cuda.h:60-203): reset-if-truncated from `initial_states` [n_envs x 2] (consumed only where a
 * reset happens; may be NULL to re-draw on the device: environment e takes words 0 and 1 of Philox group e of the
 * sequence that (seed, stream) selects, a fresh stream number per call), observe, deterministic
 * tanh/identity actor MLP or tanh-Gaussian actor with `action_noise` [n_envs x act], env step, reward,
 * next observation, truncation, and the replay `add`.
 *   policy_kind: 0 = actions given in `actions_in` (e.g. uniform warm-up policy drawn by the host)
 *                1 = MLP whose output IS the action (e.g. 3->64->64->1 tanh)
 *                2 = MLP [mean | log_std] followed by sample_and_squash with action_noise */
int rlt_rocm_pendulum_runner_step(rlt_rocm_device* device, const rlt_pendulum_runner* runner,
                                  const rlt_replay_buffer* rb, int policy_kind,
                                  const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas,
                                  const float* actions_in, const float* action_noise,
                                  const float* initial_states, uint64_t seed, uint64_t stream);
/* The same runner step with a sequential (recurrent) policy whose last layer yields [mean | log_std]
 * (rl/components/off_policy_runner/operations_generic.h:189-206): the policy state of the environments that start a new
 * episode is reset, then one evaluate_step in Rollout mode (sample_and_squash with action_noise [n_envs x 1]).
 * Declared after rlt_seq_layer / rlt_seq_state. */


/* rl::utils::evaluation::evaluate  rl/utils/evaluation/operations_generic.h:106-233 (called by the evaluation loop step,
 * rl/loop/steps/evaluation/operations_generic.h:56-92) for the Pendulum environment: n_episodes episodes of step_limit steps
 * from `initial_states` [n_episodes x 2] (what sample_initial_state draws, or the deterministic initial state), the actor in
 * Evaluation mode:
 *   policy_kind 1 = the actor's output is the action; 2 = the actor's output is [mean | log_std] and the action is tanh(mean)
 *   (sample_and_squash with zero noise, nn/layers/sample_and_squash/operations_generic.h:149-195).
 * Device outputs: returns [n_episodes], episode_length [n_episodes], summary [6] = {returns_mean, returns_std,
 * episode_length_mean, episode_length_std, num_terminated, share_terminated} (Result, evaluation.h:54-68). Actors
 * 3 -> H -> H -> out with H <= 64 run all steps in one launch, a wavefront per episode. */
int rlt_rocm_pendulum_evaluate(rlt_rocm_device* device, const rlt_pendulum_parameters* env, int policy_kind,
                               const rlt_dense_layer* actor, int n_actor_layers, const float* initial_states,
                               int n_episodes, int step_limit, float* returns, uint32_t* episode_length, float* summary);
/* The same evaluation for an actor that starts with a standardize layer (nn/layers/standardize/operations_generic.h:69-135, the
 * observation normalisation of PPO's actors, rl/algorithms/ppo/loop/core/approximators_sequential.h): every observation enters the
 * first dense layer as (observation - observation_mean) * observation_precision, both [3] on the device; both NULL: no such layer. */
int rlt_rocm_pendulum_evaluate_standardized(rlt_rocm_device* device, const rlt_pendulum_parameters* env, int policy_kind,
                                            const rlt_dense_layer* actor, int n_actor_layers, const float* observation_mean,
                                            const float* observation_precision, const float* initial_states, int n_episodes,
                                            int step_limit, float* returns, uint32_t* episode_length, float* summary);

/* Host-drawn randomness for rlt_rocm_sac_pendulum_loop (parity runs feed the draws the reference's CPU RNG made); any member
 * may be NULL, in which case the kernel draws it itself: Philox4x32-10 groups keyed by the launch's seed, one stream per kind of
 * draw (1 initial state: words 0, 1 -> theta, theta_dot; 3 rollout noise; 4 gather offset: word 0 scaled to the eligible rows;
 * 5 / 6 critic / actor noise; normals are Box-Muller on words 0, 1), group index = step_offset + step, times batch plus the
 * sample where the draw is per sample. Launches that continue a run pass the same seed and the next step_offset. */
typedef struct rlt_sac_loop_inputs {
    const float* rollout_noise;       /* [n_steps x action_dim] exploration noise of the runner's actor                 */
    const float* initial_states;      /* [n_steps x 2] (theta, theta_dot), read at the steps where an episode resets    */
    const uint32_t* sample_offsets;   /* [n_steps x batch] gather offsets (the env index is always 0: one environment)  */
    const float* noise_critic;        /* [n_steps x batch x action_dim]                                                 */
    const float* noise_actor;         /* [n_steps x batch x action_dim]                                                 */
} rlt_sac_loop_inputs;
typedef struct rlt_sac_loop_outputs {  /* all optional */
    float* critic_loss;                /* [n_steps x 2] 0.5 * mean squared TD error of each critic at its update          */
    float* observations_actions_base;  /* [2 x batch x (obs+act)] the last step's batch                                   */
    float* rewards;                    /* [batch]                                                                         */
    uint8_t* terminated;               /* [batch]                                                                         */
    float* target_action_value;        /* [batch] the last step's TD targets                                              */
    uint64_t* phase_ticks;             /* [16] profiling aid: constant-rate (100 MHz) clock ticks workgroup 0 spent per phase,
                                          ADDED to what is there: 0 env step, 1 critic phase, 2/4/7/9 grid barriers, 3 critic Adam,
                                          5 critic weight refresh, 6 actor phase, 8 actor Adam, 10 actor weight refresh            */
    /* the draws every step used -- the caller's arrays echoed, or what the kernel drew itself -- in the layout of rlt_sac_loop_inputs,
     * so that a run on device-drawn randomness can be replayed step by step elsewhere */
    float* drawn_rollout_noise;        /* [n_steps]                                                                       */
    float* drawn_initial_states;       /* [n_steps x 2] written at the steps where an episode resets, untouched elsewhere */
    uint32_t* drawn_sample_offsets;    /* [n_steps x batch]                                                               */
    float* drawn_noise_critic;         /* [n_steps x batch]                                                               */
    float* drawn_noise_actor;          /* [n_steps x batch]                                                               */
    uint64_t* stage_ticks;             /* [48] profiling aid, ADDED to what is there: the same clock as phase_ticks, read by thread 0 of
                                          workgroup 0 after every stage and after every workgroup barrier of the critic phase (slots 0-18:
                                          even = a stage's own instructions, odd = the wait at the barrier behind it) and of the actor
                                          phase (slots 20-32). Reading the clock waits for the wavefront's outstanding LDS traffic, so a
                                          run with this output set is a few percent slower than one without.                         */
} rlt_sac_loop_outputs;

/* n_steps iterations of sac::loop::core::step (rl/algorithms/sac/loop/core/operations_generic.h:110-155, past the warm-up:
 * actor-driven environment step + replay add, gather_batch, train_critic x2, update_critic_targets, train_actor) in ONE
 * persistent launch of batch/16 workgroups that synchronise through device memory. Built for the Pendulum shapes of the
 * reference's example (observation 3, action 1, 3-layer ReLU networks of width 64, batch a multiple of 16 up to 1024, one
 * environment, networks laid out as contiguous [W1|b1|W2|b2|W3|b3] arenas, masks NULL); returns RLT_E_UNSUPPORTED otherwise and
 * the caller takes the per-operation entry points above. Gradient arenas hold the last step's summed gradients on return. */
int rlt_rocm_sac_pendulum_loop(rlt_rocm_device* device, const rlt_sac_agent* agent, const rlt_pendulum_runner* runner,
                               const rlt_replay_buffer* rb, int n_steps, uint64_t seed, uint64_t step_offset,
                               const rlt_sac_loop_inputs* inputs, const rlt_sac_loop_outputs* outputs);

/* The off-policy runner over any of the batched environments (rl/components/off_policy_runner/off_policy_runner.h:184-221 runner state,
 * :158-183 Buffers). env_kind selects the environment and with it the widths:
 *   RLT_ENV_PENDULUM          state 2, observation 3, action 1   (parameters: pendulum)
 *   RLT_ENV_ACROBOT           state 4, observation 6, action 1   (parameters: acrobot)
 *   RLT_ENV_ACROBOT_SWINGUP   state 4, observation 6, action 1   (parameters: acrobot)
 *   RLT_ENV_CAR               state 6, observation 6, action 2   (parameters: car)
 *   RLT_ENV_PENDULUM_POSITION state 3 (theta, theta_dot, last action), observation 2 (cos, sin), action 1   (parameters: pendulum): the Pendulum that hides its velocity,
 *                             rl/environments/pendulum/pendulum.h:117-124 (the environment of the reference's recurrent configurations) */
enum { RLT_ENV_PENDULUM = 0, RLT_ENV_ACROBOT = 1, RLT_ENV_ACROBOT_SWINGUP = 2, RLT_ENV_CAR = 3, RLT_ENV_PENDULUM_POSITION = 4 };
typedef struct rlt_env_runner {
    int32_t env_kind, n_envs, episode_step_limit, reserved;
    float* states;              /* [n_envs x state_dim] */
    uint32_t* episode_step;     /* [n_envs] */
    float* episode_return;      /* [n_envs] */
    uint8_t* truncated;         /* [n_envs] initialised to 1 */
    rlt_pendulum_parameters pendulum; rlt_acrobot_parameters acrobot; rlt_car_parameters car;    /* the one env_kind names is read */
    /* the runner's per-step buffers, written by every step */
    float* observations;        /* [n_envs x observation_dim] */
    float* actions;             /* [n_envs x action_dim] */
    float* next_observations;   /* [n_envs x observation_dim] */
    float* rewards;             /* [n_envs] */
    uint8_t* terminated;        /* [n_envs] */
} rlt_env_runner;
/* widths of an environment kind; each pointer may be NULL. RLT_E_INVALID_ARGUMENT for an unknown kind. */
int rlt_rocm_env_dims(int env_kind, int* state_dim, int* observation_dim, int* action_dim);
size_t rlt_rocm_env_runner_step_workspace_bytes(const rlt_env_runner* runner, int policy_kind, const rlt_dense_layer* actor, int n_actor_layers);
/* step<POLICY>(device, runner, policy, ...)   rl/components/off_policy_runner/operations_generic.h:183-238, operations_generic_per_env.h:8-108
 *   prologue: environments whose `truncated` flag is set start again from initial_states [n_envs x state_dim] (what sample_initial_state
 *   would draw; consumed only where a reset happens; the caller draws them, e.g. rlt_rocm_rand_f32 over (-0.1, 0.1) for the Acrobot), their
 *   counters are cleared and the last row of their replay ring is marked truncated; observe.  interlude: the policy, as in
 *   rlt_rocm_pendulum_runner_step (policy_kind 0 actions_in [n_envs x action_dim], 1 MLP -> action, 2 MLP -> [mean | log_std] + sample_and_squash
 *   with action_noise [n_envs x action_dim]).  epilogue: environment step, reward, next observation, terminated; episode_step += 1,
 *   episode_return += reward, truncated = terminated or episode_step == episode_step_limit; replay add. Five to seven launches. */
int rlt_rocm_env_runner_step(rlt_rocm_device* device, const rlt_env_runner* runner, const rlt_replay_buffer* rb, int policy_kind,
                             const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas,
                             const float* actions_in, const float* action_noise, const float* initial_states,
                             void* workspace, size_t workspace_bytes);

/* Device buffers that rlt_rocm_sac_pendulum_loop_by_calls draws into. */
typedef struct rlt_sac_loop_scratch {
    float* rollout_noise;       /* [n_envs x action_dim] */
    float* noise_critic;        /* [batch x action_dim]  */
    float* noise_actor;         /* [batch x action_dim]  */
    uint32_t* env_indices;      /* [batch] */
    uint32_t* sample_offsets;   /* [batch] */
} rlt_sac_loop_scratch;
/* The draws of a loop step made by the kernels that consume them instead of by launches before them. Each call leaves exactly what the
 * named sequence of calls leaves, bit for bit, and echoes what it drew into the arrays those calls would have filled (the arrays may be
 * NULL where the fused kernels serve the call; they are required where the call falls back to one launch per operation).
 *   rlt_rocm_pendulum_runner_step_drawn  = rlt_rocm_randn_f32(drawn_noise, n_envs, seed, noise_stream), then rlt_rocm_pendulum_runner_step
 *                                          with policy_kind 2, that noise, initial_states NULL and (seed, initial_state_stream)
 *   rlt_rocm_gather_batch_drawn          = rlt_rocm_gather_draw(seed, stream) into the two index arrays, then rlt_rocm_gather_batch on them
 *   rlt_rocm_sac_train_critics           = rlt_rocm_sac_train_critic for critic 0, then for critic 1, on the agent's batch with the same
 *                                          noise (the loop's SHARED_BATCH case, rl/algorithms/sac/loop/core/operations_generic.h:127-138: the
 *                                          two updates do not depend on each other), then, if update_targets, rlt_rocm_sac_update_critic_targets;
 *                                          one launch where the fused update kernel fits the agent
 *   rlt_rocm_sac_train_critics_drawn     = rlt_rocm_randn_f32(drawn_noise, batch x action_dim, seed, stream), then rlt_rocm_sac_train_critics
 *   rlt_rocm_sac_train_actor_drawn       = the same draw, then rlt_rocm_sac_train_actor */
int rlt_rocm_pendulum_runner_step_drawn(rlt_rocm_device* device, const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb,
                                        const rlt_dense_layer* actor, int n_actor_layers, const rlt_sas_parameters* sas, float* drawn_noise,
                                        uint64_t seed, uint64_t noise_stream, uint64_t initial_state_stream);
int rlt_rocm_gather_batch_drawn(rlt_rocm_device* device, const rlt_replay_buffer* rb, uint64_t seed, uint64_t stream,
                                uint32_t* drawn_env_indices, uint32_t* drawn_sample_offsets, int max_episode_length, int batch,
                                float* observations_actions_base, float* rewards, uint8_t* terminated,
                                uint8_t* reset, uint8_t* next_reset_base, uint8_t* final_step_mask, uint8_t* next_final_step_mask_base);
int rlt_rocm_sac_train_critics(rlt_rocm_device* device, const rlt_sac_agent* agent, const float* action_noise, int update_targets);
int rlt_rocm_sac_train_critics_drawn(rlt_rocm_device* device, const rlt_sac_agent* agent, float* drawn_noise, uint64_t seed, uint64_t stream,
                                     int update_targets);
int rlt_rocm_sac_train_actor_drawn(rlt_rocm_device* device, const rlt_sac_agent* agent, float* drawn_noise, uint64_t seed, uint64_t stream);

/* How the fused update kernels (SAC / TD3 / PPO minibatch, networks in -> 64 -> 64 -> out) finish. optimiser_in_kernel != 0 (default):
 * every workgroup waits (bounded, see rlt_rocm_set_wait_limit) until all have stored their partial gradients, then adds up a slice of them
 * in a fixed order and applies the optimiser's step (and the targets' soft update) to that slice, so an update is one launch (grids of up to
 * 64 workgroups); 0: the optimiser runs as a launch of its own after the kernel (same bits). one_xcd != 0 (default):
 * grids of at most 32 workgroups are placed on one XCD, whose L2 then serves the exchange; 0: spread over all XCDs. The environment
 * variables RLT_UPDATE_TAIL=0 and RLT_UPDATE_PLACEMENT=spread set the defaults of a process. No counterpart in the reference. */
int rlt_rocm_set_update_options(rlt_rocm_device* device, int optimiser_in_kernel, int one_xcd);
/* The kernels whose workgroups wait for each other (the persistent SAC loop; update kernels that end with the optimiser's step) poll a
 * bounded number of times, then give up: the kernel still ends normally, its results are void, and the next rlt_rocm_check_status returns
 * RLT_E_DEVICE_TIMEOUT. `polls` sets that bound (0: the default, about a second). With a bound of 1 every workgroup of an update kernel
 * but the last to arrive gives up without looking at the counter, which makes the give-up path testable from the host. No counterpart in
 * the reference. */
int rlt_rocm_set_wait_limit(rlt_rocm_device* device, unsigned polls);

/* The same n_steps iterations of sac::loop::core::step (rl/algorithms/sac/loop/core/operations_generic.h:110-155 past the warm-up,
 * SHARED_BATCH: runner step with the actor, one gather_batch and one critic noise draw for both train_critic calls,
 * update_critic_targets, actor noise draw, train_actor on the same batch) as a host loop over this library's own entry points, for
 * agents and runners of any size that rlt_rocm_sac_pendulum_loop does not cover: four launches per step where the fused kernels fit
 * (rlt_rocm_pendulum_runner_step_drawn, rlt_rocm_gather_batch_drawn, rlt_rocm_sac_train_critics_drawn with the target update,
 * rlt_rocm_sac_train_actor_drawn). Nothing synchronises with the host. Loop step g = step_offset + i draws from the Philox
 * sequences (seed, 8 g + k): k = 1 rollout noise, 2 initial states of episodes that reset, 3 batch indices, 4 critic noise,
 * 5 actor noise; the scratch arrays receive the draws of the last step. */
int rlt_rocm_sac_pendulum_loop_by_calls(rlt_rocm_device* device, const rlt_sac_agent* agent, const rlt_pendulum_runner* runner,
                                        const rlt_replay_buffer* rb, int n_steps, uint64_t seed, uint64_t step_offset,
                                        const rlt_sac_loop_scratch* scratch);

/* ------------------------------------------------------------ graph capture -- */

/* Recording the launches of a stretch of calls into a graph and replaying it, for host loops whose speed the launches set
 * (the reference's CUDA example captures its loop step into three graphs: src/rl/environments/pendulum/sac/cuda/sac.cu:122-164, with
 * devices::CUDA::graph_capture_active making check_status skip its wait: devices/cuda.h:59,163).
 *   rlt_rocm_graph_begin_capture  the handle's stream starts recording. Until rlt_rocm_graph_end_capture every entry point only records
 *                                 its launches: none may allocate, free, copy to or from the host or wait -- those that would return
 *                                 RLT_E_CAPTURING (rlt_rocm_malloc / _free / _memcpy_h2d / _d2h, a workspace of the library that would
 *                                 have to grow: issue the same calls once before the capture), rlt_rocm_check_status returns 0 at once.
 *   rlt_rocm_graph_end_capture    ends the recording (also after a failed call) and instantiates the graph.
 *   rlt_rocm_graph_launch         enqueues one replay on the handle's stream; pointers, sizes, seeds and stream numbers are those of the
 *                                 recording.
 * Random numbers under replay: every draw made on the device takes its values from the Philox sequence (seed, stream + offset), where
 * offset is a 64-bit word in device memory, zero after rlt_rocm_init. rlt_rocm_advance_streams enqueues offset += by, and can be
 * recorded: a graph that ends with it draws fresh values on every replay, the same ones as the unrecorded calls with their stream
 * numbers raised by `by` per repetition. rlt_rocm_set_stream_offset enqueues offset = value. */
typedef struct rlt_rocm_graph rlt_rocm_graph;
int rlt_rocm_graph_begin_capture(rlt_rocm_device* device);
int rlt_rocm_graph_end_capture(rlt_rocm_device* device, rlt_rocm_graph** out_graph);
int rlt_rocm_graph_launch(rlt_rocm_device* device, rlt_rocm_graph* graph);
int rlt_rocm_graph_destroy(rlt_rocm_device* device, rlt_rocm_graph* graph);
int rlt_rocm_advance_streams(rlt_rocm_device* device, uint64_t by);
int rlt_rocm_set_stream_offset(rlt_rocm_device* device, uint64_t value);

/* --------------------------------------------------------------------- PPO -- */

/* estimate_generalized_advantages   rl/algorithms/ppo/operations_generic.h:60-95
 *   rows are step-major: row = step*n_envs + env (on_policy_runner.h:38-72); every column is passed
 *   with the dataset's row stride `ld` (floats), flags are floats as in the reference dataset.
 *   all_values has (steps+1)*n_envs rows (the last n_envs rows bootstrap). */
int rlt_rocm_ppo_gae(rlt_rocm_device* device, const float* rewards, const float* terminated, const float* truncated,
                     const float* all_values, float* advantages, float* target_values, int ld,
                     int n_envs, int steps, float gamma, float lambda, int ignore_termination);

/* The part of rl/algorithms/ppo/ppo.h:13-40 (DefaultParameters) that the update reads. */
typedef struct rlt_ppo_parameters {
    float epsilon_clip;                 /* EPSILON_CLIP */
    float action_entropy_coefficient;   /* ACTION_ENTROPY_COEFFICIENT */
    float advantage_epsilon;            /* ADVANTAGE_EPSILON */
    int normalize_advantage;            /* NORMALIZE_ADVANTAGE: per-minibatch mean / std */
    int learn_action_std;               /* LEARN_ACTION_STD */
    int reserved[3];
} rlt_ppo_parameters;

/* Actor = MLP + state-independent action log_std (nn_models/mlp_unconditional_stddev/network.h), critic = MLP, their
 * optimisers (rl/algorithms/ppo/ppo.h:62-101). The layers' pre_activations/output buffers hold `batch` rows (the
 * minibatch size); actor_adam_tensors includes the log_std tensor. The workspace needs
 * rlt_rocm_ppo_workspace_bytes(agent) bytes. */
typedef struct rlt_ppo_agent {
    const rlt_dense_layer* actor;  int n_actor_layers;
    const rlt_dense_layer* critic; int n_critic_layers;
    float* log_std;                     /* [action_dim] */
    float* d_log_std;                   /* [action_dim] gradient */
    const rlt_adam_tensor* actor_adam_tensors;  int n_actor_adam_tensors;
    const rlt_adam_tensor* critic_adam_tensors; int n_critic_adam_tensors;
    rlt_adam_parameters actor_adam, critic_adam;
    uint32_t* actor_age; uint32_t* critic_age;
    int observation_dim, observation_privileged_dim, action_dim, batch;
    void* workspace; size_t workspace_bytes;
    /* optional standardize layers in front of the MLPs (nn/layers/standardize/operations_generic.h:68-86; the loop's approximators,
     * rl/algorithms/ppo/loop/core/config.h:51-83): the networks then read (x - mean) * precision (the factor only where it is not 0).
     * [observation_dim] / [observation_privileged_dim] floats; NULL = no such layer. The layer has no trainable parameters. */
    const float* actor_standardize_mean; const float* actor_standardize_precision;
    const float* critic_standardize_mean; const float* critic_standardize_precision;
} rlt_ppo_agent;

size_t rlt_rocm_ppo_workspace_bytes(const rlt_ppo_agent* agent);

/* The per-sample part of the update between the actor's forward and backward pass,
 * rl/algorithms/ppo/operations_generic.h:170-269 (ADAPTIVE_LEARNING_RATE off): advantage normalisation over the
 * minibatch, log-probability of the rollout action under the current policy (random/operations_generic.h:73-97),
 * ratio, clipping, d loss / d mean into d_action_means, and the entropy + surrogate terms ADDED to d_log_std.
 * Columns are passed with their row strides (floats). */
int rlt_rocm_ppo_surrogate_gradient(rlt_rocm_device* device, const float* action_means, int ld_means, const float* log_std,
                                    const float* actions, int ld_actions, const float* action_log_probs, int ld_log_probs,
                                    const float* advantages, int ld_advantages, const rlt_ppo_parameters* parameters,
                                    float* d_action_means, int ld_d, float* d_log_std, int batch, int action_dim);

/* One minibatch of train(), the body of the batch loop rl/algorithms/ppo/operations_generic.h:156-318: zero_gradient,
 * actor forward, surrogate gradient, actor backward, critic forward + MSE gradient (loss weight 0.5) + backward, Adam
 * step of both. The dataset columns are passed with the dataset's row stride `ld`; `row_indices` (device, `batch`
 * entries) selects the minibatch's rows -- the reference shuffles the dataset in place per epoch (:126-155), a caller
 * here passes that permutation instead -- NULL means rows [0, batch). out_critic_loss (device scalar, optional)
 * receives mse::evaluate of the critic on the minibatch before its update (:313). */
int rlt_rocm_ppo_train_minibatch(rlt_rocm_device* device, const rlt_ppo_agent* agent, const rlt_ppo_parameters* parameters,
                                 const float* observations, const float* observations_privileged, const float* actions,
                                 const float* action_log_probs, const float* advantages, const float* target_values, int ld,
                                 const uint32_t* row_indices, float* out_critic_loss);

/* One epoch of train(): the batch loop rl/algorithms/ppo/operations_generic.h:156-318 over the rows that the epoch's shuffle
 * (:126-155) put in place, given here as the permutation `row_indices` (device, n_minibatches x batch entries; minibatch i
 * takes entries [i * batch, (i + 1) * batch)). Same result as n_minibatches calls of rlt_rocm_ppo_train_minibatch; the
 * per-minibatch advantage statistics (:170-180) of the whole epoch are formed up front by one pair of launches.
 * out_critic_losses (device, optional) receives n_minibatches values. */
int rlt_rocm_ppo_train_epoch(rlt_rocm_device* device, const rlt_ppo_agent* agent, const rlt_ppo_parameters* parameters,
                             const float* observations, const float* observations_privileged, const float* actions,
                             const float* action_log_probs, const float* advantages, const float* target_values, int ld,
                             const uint32_t* row_indices, int n_minibatches, float* out_critic_losses);

/* --------------------------------------------------------------------- GRU -- */

/* nn/layers/gru/layer.h:96-217 (LayerForward / LayerBackward / LayerGradient): gate order r, z, n along the 3H rows
 * (the layout of torch.nn.GRU); LEARN_INITIAL_HIDDEN_STATE = false as in the reference's configuration (layer.h:14-24).
 * fast_tanh selects the reference's FAST_TANH switch (layer.h:12,18; operations_generic.h:302-320): the gates then use
 * math::fast_sigmoid / math::fast_tanh (math/operations_generic.h:247-255) in the forward pass, while the backward pass
 * keeps the derivative formulas of the exact functions on the stored outputs; the reference's SAC / TD3 GRU approximators
 * set it (rl/algorithms/sac/loop/core/approximators_gru.h:18). Tensors are [sequence x batch x features], row-major. */
typedef struct rlt_gru_layer {
    float* weights_input;          /* [3H x I] */
    float* biases_input;           /* [3H] */
    float* weights_hidden;         /* [3H x H] */
    float* biases_hidden;          /* [3H] */
    float* initial_hidden_state;   /* [H] */
    float* d_weights_input; float* d_biases_input; float* d_weights_hidden; float* d_biases_hidden;   /* gradients, accumulated */
    float* post_activation;        /* [S x B x 3H] r and z after the sigmoid, n after tanh (kept by forward for backward) */
    float* n_pre_pre_activation;   /* [S x B x H]  W_hn h + b_hn */
    float* output;                 /* [S x B x H]  hidden state of every step */
    int input_dim, hidden_dim;
    int fast_tanh, reserved;
} rlt_gru_layer;

size_t rlt_rocm_gru_workspace_bytes(const rlt_gru_layer* layer, int sequence_length, int batch);
/* forward (keeps the intermediates)   nn/layers/gru/operations_generic.h:231-341,418-421
 *   reset [S x B] (optional): a sample whose flag is set at step t starts that step from initial_hidden_state, as do all
 *   samples at step 0 (ResetMode, layer.h:56-68). */
int rlt_rocm_gru_forward(rlt_rocm_device* device, const rlt_gru_layer* layer, const float* input, const uint8_t* reset,
                         int sequence_length, int batch, void* workspace, size_t workspace_bytes);
/* backward / backward_full / backward_input through time   nn/layers/gru/operations_generic.h:594-795
 *   d_output [S x B x H] is modified (the gradient flowing back through the hidden state is accumulated into it, as in
 *   the reference); d_input [S x B x I] may be NULL; want_weight_gradients = 0 -> backward_input. */
int rlt_rocm_gru_backward(rlt_rocm_device* device, const rlt_gru_layer* layer, const float* input, float* d_output,
                          float* d_input, const uint8_t* reset, int sequence_length, int batch, int want_weight_gradients,
                          void* workspace, size_t workspace_bytes);

/* ------------------------------------- SAC on sequence batches (recurrent) -- */

/* One layer of a sequential model (nn_models/sequential/model.h:196-215 holds `content` and `next_module`): a dense layer,
 * applied to all steps x batch rows at once, or a GRU layer. The reference's recurrent approximators
 * (rl/algorithms/sac/loop/core/approximators_gru.h:13-74) are dense -> GRU [-> GRU] [-> dense] -> dense, for the actor
 * followed by the sample_and_squash layer, which lives in the agent below. The kept intermediates of every layer
 * (dense: pre_activations / output; GRU: post_activation / n_pre_pre_activation / output) hold steps x batch rows, with
 * steps = sequence_length + 1 where the network is also evaluated on the `next` views. */
typedef struct rlt_seq_layer {
    int32_t kind;                /* 0 dense, 1 GRU */
    int32_t reserved;
    rlt_dense_layer dense;
    rlt_gru_layer gru;
} rlt_seq_layer;

/* forward / evaluate of a sequential model   nn_models/sequential/operations_generic.h:277-347
 *   x [steps x batch x in] with leading dimension ldx (a GRU as first layer needs ldx = in); reset [steps x batch] or NULL
 *   (the ResetMode of nn/layers/gru/layer.h:56-68, handed to every layer); every layer keeps its intermediates, the result
 *   is the last layer's output. */
int rlt_rocm_seq_forward(rlt_rocm_device* device, const rlt_seq_layer* layers, int n_layers, const float* x, int ldx,
                         const uint8_t* reset, int steps, int batch, void* workspace, size_t workspace_bytes);
/* backward / backward_full / backward_input of a sequential model   nn_models/sequential/operations_generic.h:369-428
 *   d_output [steps x batch x out] packed, modified (every layer leaves its d_pre / accumulated hidden-state gradient in
 *   the buffer it was handed, as in the reference); d_input [steps x batch x in] packed or NULL;
 *   want_weight_gradients = 0 -> backward_input. The reference's backward_input hands the mode only to a model's first
 *   layer when that layer is also its last (operations_generic.h:399-407 call the inner layers without it), so in a deeper
 *   model the GRU layers run their backward_input as if no step had been a reset; reset_in_backward_input = 0 reproduces
 *   that, 1 hands the resets to every layer. Ignored when want_weight_gradients != 0 (those paths pass the mode on). */
int rlt_rocm_seq_backward(rlt_rocm_device* device, const rlt_seq_layer* layers, int n_layers, const float* x, int ldx,
                          float* d_output, float* d_input, const uint8_t* reset, int steps, int batch,
                          int want_weight_gradients, int reset_in_backward_input, void* workspace, size_t workspace_bytes);
int rlt_rocm_seq_zero_gradient(rlt_rocm_device* device, const rlt_seq_layer* layers, int n_layers);
size_t rlt_rocm_seq_workspace_bytes(const rlt_seq_layer* layers, int n_layers, int steps, int batch);

/* What a sequential model carries from one rollout step to the next (nn/layers/gru/layer.h State: hidden state and the
 * number of steps since its last reset, per batch row), indexed by layer; entries at dense layers are unused. */
#define RLT_SEQ_MAX_LAYERS 8
typedef struct rlt_seq_state {
    float* hidden[RLT_SEQ_MAX_LAYERS];     /* [batch x H] */
    uint32_t* step[RLT_SEQ_MAX_LAYERS];    /* [batch] */
} rlt_seq_state;
/* reset(model, state, mode)   nn_models/sequential/operations_generic.h:35-41, nn/layers/gru/operations_generic.h:87-120
 *   rows whose mask byte is set (all rows if mask == NULL) start again: hidden <- initial_hidden_state, step <- 0. */
int rlt_rocm_seq_reset_state(rlt_rocm_device* device, const rlt_seq_layer* layers, int n_layers, const rlt_seq_state* state,
                             const uint8_t* mask, int batch);
/* evaluate_step(model, input, state, output)   nn_models/sequential/operations_generic.h:303-327, nn/layers/gru/operations_generic.h:348-416
 *   one step of every layer on x [batch x in] (leading dimension ldx); GRU layers read and advance their state and, like the
 *   reference outside its NoAutoResetMode, start again from the initial hidden state once a row has run auto_reset_period
 *   steps (the SEQUENCE_LENGTH of the model's input shape; 0 switches that off). y [batch x out] with leading dimension ldy.
 *   The layers' kept intermediates are not touched. */
int rlt_rocm_seq_evaluate_step(rlt_rocm_device* device, const rlt_seq_layer* layers, int n_layers, const float* x, int ldx,
                               const rlt_seq_state* state, int auto_reset_period, float* y, int ldy, int batch,
                               void* workspace, size_t workspace_bytes);
size_t rlt_rocm_seq_evaluate_step_workspace_bytes(const rlt_seq_layer* layers, int n_layers, int batch);
/* runner step with a recurrent policy (see rlt_rocm_pendulum_runner_step) and the workspace it needs */
size_t rlt_rocm_pendulum_runner_step_recurrent_workspace_bytes(const rlt_seq_layer* policy, int n_policy_layers, int n_envs);
int rlt_rocm_pendulum_runner_step_recurrent(rlt_rocm_device* device, const rlt_pendulum_runner* runner, const rlt_replay_buffer* rb,
                                            const rlt_seq_layer* policy, int n_policy_layers, const rlt_seq_state* policy_state,
                                            int auto_reset_period, const rlt_sas_parameters* sas, const float* action_noise,
                                            const float* initial_states, void* workspace, size_t workspace_bytes);
/* rl::utils::evaluation::evaluate  rl/utils/evaluation/operations_generic.h:106-233 with a sequential (recurrent) policy on the
 * Pendulum (see rlt_rocm_pendulum_evaluate for the arguments and outputs): reset(policy, policy_state) before the first step
 * (:135), then evaluate_step per step in Evaluation mode (:163) -- GRU layers restart their hidden state every
 * auto_reset_period steps as in rlt_rocm_seq_evaluate_step. policy_state holds n_episodes rows and is left as the last
 * step left it. policy_kind 2: the policy's last layer yields [mean | log_std] and sample_and_squash follows (action
 * tanh(mean)); 1: its output is the action. */
size_t rlt_rocm_pendulum_evaluate_recurrent_workspace_bytes(const rlt_seq_layer* policy, int n_policy_layers, int n_episodes);
int rlt_rocm_pendulum_evaluate_recurrent(rlt_rocm_device* device, const rlt_pendulum_parameters* env, int policy_kind,
                                         const rlt_seq_layer* policy, int n_policy_layers, const rlt_seq_state* policy_state,
                                         int auto_reset_period, const float* initial_states, int n_episodes, int step_limit,
                                         float* returns, uint32_t* episode_length, float* summary, void* workspace,
                                         size_t workspace_bytes);

/* Everything one SAC agent with sequential (recurrent) networks owns on the device: rl/algorithms/sac/sac.h:62-145 for
 * SEQUENCE_LENGTH >= 1 and the batch of rl/components/off_policy_runner/off_policy_runner.h:102-156 as
 * rlt_rocm_gather_sequence_batch fills it. S = batch.sequence_length, B = batch.batch, T = S + 1 if
 * include_first_step_in_targets (then the `next` views start at padded step 0) else S (they start at step 1). */
typedef struct rlt_sac_sequence_agent {
    int32_t observation_dim, action_dim, n_actor_layers, n_critic_layers;
    int32_t include_first_step_in_targets, reserved0;
    float gamma, polyak;
    rlt_sas_parameters sas;
    rlt_adam_parameters actor_adam, critic_adam, alpha_adam;
    const rlt_seq_layer* actor;              /* last layer: out_dim = 2 * action_dim, intermediates for T x B rows */
    const rlt_seq_layer* critics[2];         /* intermediates for S x B rows */
    const rlt_seq_layer* critics_target[2];  /* intermediates for T x B rows */
    const rlt_adam_tensor* actor_adam_tensors;      int32_t n_actor_adam_tensors;   int32_t pad0;
    const rlt_adam_tensor* critic_adam_tensors[2];  int32_t n_critic_adam_tensors;  int32_t pad1;
    rlt_adam_tensor log_alpha;               /* count = 1 */
    uint32_t* actor_age; uint32_t* critic_age[2]; uint32_t* alpha_age;
    rlt_sequence_batch batch;
    /* training buffers (sac.h:73-131) */
    float* next_state_action_value_input;    /* [T x B x (obs + act)] */
    float* next_q[2];                        /* [T x B] */
    float* next_log_probabilities;           /* [T x B] */
    float* target_action_value;              /* [S x B] */
    float* d_output;                         /* [S x B] */
    float* state_action_value_input;         /* [S x B x (obs + act)] */
    float* d_critic_input[2];                /* [S x B x (obs + act)] */
    float* d_actor_output_squashing;         /* [S x B x act] */
    float* d_actor_output;                   /* [S x B x 2 act] */
    float* actor_actions;                    /* [T x B x act] sample_and_squash output */
    float* actor_pre_squashing;              /* [S x B x act] */
    float* actor_log_probabilities;          /* [S x B] */
    void* workspace; size_t workspace_bytes; /* >= rlt_rocm_sac_sequence_workspace_bytes */
} rlt_sac_sequence_agent;

/* The sequence updates below run network passes that do not depend on each other at the same time -- the trained critic's forward pass next to the (target) actor's,
 * the second target critic next to the first, in train_actor the second critic's forward pass and input gradient next to the first's -- the second of each pair on a
 * stream of the handle's own that waits for, and is waited for by, the stream the calls are enqueued on (each recurrence fills about a twentieth of the chip);
 * rlt_rocm_sac_sequence_train_critics uses two such streams. The workspace is three parts for that reason. Results are those of the passes in sequence, bit for bit. While the stream records a graph the passes stay in sequence. */
size_t rlt_rocm_sac_sequence_workspace_bytes(const rlt_sac_sequence_agent* agent);
/* train_critic on a sequence batch   rl/algorithms/sac/operations_generic.h:243-337
 *   action_noise [T x B x action_dim]: the N(0,1) noise of the actor's sample_and_squash layer on the `next` views.
 *   As in the reference, the target of step t takes the target critics' value of step t + 1 but the entropy bonus from the
 *   log-probability at index t of the evaluated `next` steps (operations_generic.h:144-154). */
int rlt_rocm_sac_sequence_train_critic(rlt_rocm_device* device, const rlt_sac_sequence_agent* agent, int critic_index, const float* action_noise);
/* train_critic for critic 0, then for critic 1, on the agent's batch with the same noise: the loop's SHARED_BATCH case (rl/algorithms/sac/loop/core/operations_generic.h:127-138,
 * where the second call repeats the actor's pass over the next rows, its sample, both target critics and the target values on unchanged inputs). Those are computed
 * once here, the two critics' own passes run next to each other on the handle's two streams, and the results are those of the two calls bit for bit (critic 1's loss
 * gradient is left in agent->d_output, as they leave it; critic 0's goes to the end of the workspace). */
int rlt_rocm_sac_sequence_train_critics(rlt_rocm_device* device, const rlt_sac_sequence_agent* agent, const float* action_noise);
/* update_critic_targets   sac/operations_generic.h:486-527 (dense and GRU layers, incl. the initial hidden state) */
int rlt_rocm_sac_sequence_update_critic_targets(rlt_rocm_device* device, const rlt_sac_sequence_agent* agent);
/* train_actor on a sequence batch   sac/operations_generic.h:395-468; action_noise [S x B x action_dim] */
int rlt_rocm_sac_sequence_train_actor(rlt_rocm_device* device, const rlt_sac_sequence_agent* agent, const float* action_noise);

/* --------------------------------------------------------------------- TD3 -- */

/* td3_sampling layer      nn/layers/td3_sampling/operations_generic.h:75-128
 *   sample = mean + noise * std (noise [batch x dim] are externally drawn N(0,1) values; NULL: sample = mean, the
 *   Evaluation mode), output = clamp(sample, -1, 1); pre_clip (optional) receives sample, as forward() keeps it. */
int rlt_rocm_td3_sampling_forward(rlt_rocm_device* device, const float* input, int ldin, const float* noise, int ldn, float std,
                                  float* pre_clip, int ldp, float* output, int ldo, int batch, int dim);
/* backward_full           td3_sampling/operations_generic.h:139-163 : d_input = (pre_clip < -1 || pre_clip > 1) ? 0 : d_output */
int rlt_rocm_td3_sampling_backward(rlt_rocm_device* device, const float* pre_clip, int ldp, const float* d_output, int lddo,
                                   float* d_input, int lddi, int batch, int dim);
/* target_action_noise     rl/algorithms/td3/operations_generic.h:116-128, operations_cuda.h:8-44
 *   from N(0,1) draws z: out = clamp(z * std + 0, -clip, clip) (the reference draws N(0, std) directly). */
int rlt_rocm_td3_target_action_noise(rlt_rocm_device* device, const float* standard_normal, float std, float clip, float* out, size_t count);
/* noisy_next_actions      td3/operations_generic.h:129-145, operations_cuda.h:46-75 : a = clamp(a + noise, -1, 1) in place */
int rlt_rocm_td3_noisy_next_actions(rlt_rocm_device* device, float* next_actions, int lda, const float* noise, int ldn, int batch, int dim);
/* target_action_values    td3/operations_generic.h:146-169, operations_cuda.h:77-110
 *   y = r + (ignore_termination || !terminated ? gamma * min(q1', q2') : 0) */
int rlt_rocm_td3_target_action_values(rlt_rocm_device* device, const float* q1_next, const float* q2_next, const float* rewards,
                                      const uint8_t* terminated, float gamma, int ignore_termination, float* target, int batch);

/* Everything one TD3 agent owns on the device (rl/algorithms/td3/td3.h ActorCritic, Critic/ActorTrainingBuffers, and the
 * batch of rl/components/off_policy_runner/off_policy_runner.h:89-156 for SEQUENCE_LENGTH = 1). The actor is an MLP
 * (output activation as configured, TANH in td3/loop/core/approximators_mlp.h:15-31) followed by the td3_sampling layer. */
typedef struct rlt_td3_agent {
    int32_t batch, observation_dim, action_dim, n_actor_layers, n_critic_layers, ignore_termination;
    float gamma, actor_polyak, critic_polyak;
    float sampling_std;                       /* std of the actor's td3_sampling layer (EXPLORATION_NOISE) */
    rlt_adam_parameters actor_adam, critic_adam;
    const rlt_dense_layer* actor;             /* out_dim of last layer = action_dim */
    const rlt_dense_layer* actor_target;
    const rlt_dense_layer* critics[2];
    const rlt_dense_layer* critics_target[2];
    const rlt_adam_tensor* actor_adam_tensors;      int32_t n_actor_adam_tensors;   int32_t pad0;
    const rlt_adam_tensor* critic_adam_tensors[2];  int32_t n_critic_adam_tensors;  int32_t pad1;
    uint32_t* actor_age; uint32_t* critic_age[2];
    /* batch (SequentialBatch, SEQUENCE_LENGTH = 1): [2 x batch x (obs+act)] */
    float* observations_actions_base;
    float* rewards;            /* [batch] */
    uint8_t* terminated;       /* [batch] */
    const uint8_t* final_step_mask;        /* [batch]; NULL = all true */
    const uint8_t* next_final_step_mask;   /* [batch]; NULL = all true */
    /* critic training buffers */
    float* target_next_action_noise;        /* [batch x act], already clamped (target_action_noise) */
    float* next_state_action_value_input;   /* [batch x (obs+act)] */
    float* next_q[2];                        /* [batch] each */
    float* target_action_value;              /* [batch] */
    float* d_output_critic;                  /* [batch] */
    /* actor training buffers */
    float* state_action_value_input;         /* [batch x (obs+act)] */
    float* actor_pre_clip;                   /* [batch x act] */
    float* d_output_actor;                   /* [batch] */
    float* d_critic_input;                   /* [batch x (obs+act)] */
    float* d_actor_output;                   /* [batch x act] */
    void* workspace; size_t workspace_bytes;
} rlt_td3_agent;

/* Two implementations with the same results (to fp32 rounding), as for SAC: where every network is in -> 64 -> 64 -> out with one hidden
 * activation (not GELU), the actors end in tanh, obs + act <= 128, act <= 8 and both masks are NULL, train_critic and train_actor each run
 * as two launches (all network passes of the update; sum of the workgroups' partial gradients + Adam); of the training buffers only
 * target_action_value (critic) and actor_pre_clip (actor) are then written, and the gradients are overwritten without a prior
 * zero_gradient. Every other agent, or any agent after rlt_rocm_sac_set_per_operation(device, 1), takes one launch per reference operation
 * and fills every training buffer.
 * train_critic            rl/algorithms/td3/operations_generic.h:170-235 for critic `critic_index`; sampling_noise [batch x act] are
 *   the N(0,1) draws of the target actor's sampling layer (its evaluate runs in the default mode, which samples). */
int rlt_rocm_td3_train_critic(rlt_rocm_device* device, const rlt_td3_agent* agent, int critic_index, const float* sampling_noise);
/* rlt_rocm_td3_train_critic for critic 0 with sampling_noise_first and then for critic 1 with sampling_noise_second on the agent's batch and target noise (the loop's shared
 * batch, rl/algorithms/td3/loop/core/operations_generic.h:98-112): same results bit for bit; for hidden widths up to 256 the two updates are one launch. */
int rlt_rocm_td3_train_critics(rlt_rocm_device* device, const rlt_td3_agent* agent, const float* sampling_noise_first, const float* sampling_noise_second);
/* The draws of a critic update on a shared batch: target_action_noise (td3/operations_generic.h:116-128: clamp(N(0, 1) * std, -clip, clip)) from
 * (seed, target_noise_stream), critic k's sampling noise from (seed, sampling_stream[k]); element i of a tensor is element i of rlt_rocm_randn_f32 on that stream. */
typedef struct rlt_td3_critic_draws {
    uint64_t seed, target_noise_stream, sampling_stream[2];
    float target_noise_std, target_noise_clip;
} rlt_td3_critic_draws;
/* target_action_noise into agent->target_next_action_noise and rlt_rocm_td3_train_critics with all three noise tensors drawn as `draws` says: same results bit for bit as
 * rlt_rocm_randn_f32 x 3, rlt_rocm_td3_target_action_noise and rlt_rocm_td3_train_critics. For hidden widths up to 256 the draws are made inside the one
 * launch; otherwise sampling_noise [2 x batch x act] receives the two sampling noises (it may be NULL where the draws are made inside). update_targets != 0:
 * rlt_rocm_td3_update_critic_targets afterwards as well (same bits; with the one launch, inside the optimisers' launch). */
int rlt_rocm_td3_train_critics_drawn(rlt_rocm_device* device, const rlt_td3_agent* agent, const rlt_td3_critic_draws* draws, float* sampling_noise, int update_targets);
/* train_actor             td3/operations_generic.h:236-281; sampling_noise as above, for the actor's forward pass */
int rlt_rocm_td3_train_actor(rlt_rocm_device* device, const rlt_td3_agent* agent, const float* sampling_noise);
/* rlt_rocm_td3_train_actor with the sampling noise drawn from (seed, stream) as rlt_rocm_randn_f32 draws it: inside the launch for hidden widths up to 256,
 * otherwise into sampling_noise [batch x act] first. */
int rlt_rocm_td3_train_actor_drawn(rlt_rocm_device* device, const rlt_td3_agent* agent, uint64_t seed, uint64_t stream, float* sampling_noise);
/* update_critic_targets   td3/operations_generic.h:317-321 */
int rlt_rocm_td3_update_critic_targets(rlt_rocm_device* device, const rlt_td3_agent* agent);
/* update_actor_target     td3/operations_generic.h:322-325 */
int rlt_rocm_td3_update_actor_target(rlt_rocm_device* device, const rlt_td3_agent* agent);

/* TD3 on sequence batches with sequential (recurrent) networks: rl/algorithms/td3/td3.h ActorCritic and training buffers for
 * SEQUENCE_LENGTH >= 1 with the approximators of td3/loop/core/approximators_gru.h:9-75 (GRU [-> GRU] [-> dense] -> dense, no
 * sampling layer, MASK_NON_TERMINAL). S, B, T as in rlt_sac_sequence_agent. */
typedef struct rlt_td3_sequence_agent {
    int32_t observation_dim, action_dim, n_actor_layers, n_critic_layers;
    int32_t include_first_step_in_targets, ignore_termination;
    float gamma, actor_polyak, critic_polyak, reserved0;
    rlt_adam_parameters actor_adam, critic_adam;
    const rlt_seq_layer* actor;              /* last layer: out_dim = action_dim, intermediates for S x B rows */
    const rlt_seq_layer* actor_target;       /* intermediates for T x B rows */
    const rlt_seq_layer* critics[2];         /* intermediates for S x B rows */
    const rlt_seq_layer* critics_target[2];  /* intermediates for T x B rows */
    const rlt_adam_tensor* actor_adam_tensors;      int32_t n_actor_adam_tensors;   int32_t pad0;
    const rlt_adam_tensor* critic_adam_tensors[2];  int32_t n_critic_adam_tensors;  int32_t pad1;
    uint32_t* actor_age; uint32_t* critic_age[2];
    rlt_sequence_batch batch;
    float* target_next_action_noise;         /* [T x B x act], already clamped (rlt_rocm_td3_target_action_noise) */
    float* next_state_action_value_input;    /* [T x B x (obs + act)] */
    float* next_q[2];                        /* [T x B] */
    float* target_action_value;              /* [S x B] */
    float* d_output;                         /* [S x B] */
    float* state_action_value_input;         /* [S x B x (obs + act)] */
    float* d_critic_input;                   /* [S x B x (obs + act)] */
    float* d_actor_output;                   /* [S x B x act] */
    float* actor_input;                      /* [T x B x obs]: the observation columns of the batch, contiguous, for an actor whose first layer is a GRU */
    void* workspace; size_t workspace_bytes; /* >= rlt_rocm_td3_sequence_workspace_bytes */
} rlt_td3_sequence_agent;

size_t rlt_rocm_td3_sequence_workspace_bytes(const rlt_td3_sequence_agent* agent);
/* train_critic on a sequence batch   rl/algorithms/td3/operations_generic.h:170-235: target actor and target critics over the
 * `next` views with next_reset, noisy clamped next actions, actions of non-final steps taken from the batch, targets from the
 * step after, loss reweighted by S*B / (number of final steps), gradient masked to the final steps */
int rlt_rocm_td3_sequence_train_critic(rlt_rocm_device* device, const rlt_td3_sequence_agent* agent, int critic_index);
/* rlt_rocm_td3_sequence_train_critic for critic 0 and then for critic 1 on the agent's batch and target noise (the loop's shared batch,
 * rl/algorithms/td3/loop/core/operations_generic.h:98-112): same results bit for bit; what the second call would repeat is computed once and independent passes run
 * side by side on the handle's side streams. */
int rlt_rocm_td3_sequence_train_critics(rlt_rocm_device* device, const rlt_td3_sequence_agent* agent);
/* train_actor on a sequence batch    td3/operations_generic.h:236-281 (through critic 0) */
int rlt_rocm_td3_sequence_train_actor(rlt_rocm_device* device, const rlt_td3_sequence_agent* agent);
/* update_critic_targets / update_actor_target   td3/operations_generic.h:283-325 (dense and GRU layers incl. the initial hidden state) */
int rlt_rocm_td3_sequence_update_critic_targets(rlt_rocm_device* device, const rlt_td3_sequence_agent* agent);
int rlt_rocm_td3_sequence_update_actor_target(rlt_rocm_device* device, const rlt_td3_sequence_agent* agent);

/* ------------------------------------------- on-policy collection, normalisation -- */

/* standardize layer       nn/layers/standardize/operations_generic.h:54-67 (set_statistics), :68-86 (evaluate / forward),
 *                         :101-120 (backward_input; backward is a no-op: the layer has no trainable parameters)
 *   set_statistics: layer_mean = mean, layer_precision = std == 0 ? 0 : 1 / std
 *   forward:        out = (in - layer_mean), times layer_precision where that is not 0
 *   backward_input: d_in = d_out * layer_precision */
int rlt_rocm_standardize_set_statistics(rlt_rocm_device* device, const float* mean, const float* std, float* layer_mean, float* layer_precision, int dim);
int rlt_rocm_standardize_forward(rlt_rocm_device* device, const float* layer_mean, const float* layer_precision, const float* input, int ldin,
                                 float* output, int ldo, int batch, int dim);
int rlt_rocm_standardize_backward_input(rlt_rocm_device* device, const float* layer_precision, const float* d_output, int ldd, float* d_input, int ldi,
                                        int batch, int dim);
/* running normaliser      rl/components/running_normalizer/operations_generic.h:18-45 (init: mean 0, std 1, age 0; update)
 *   update: age += 1; per column: m = mean(column), s = sqrt(sum (x - m)^2 / (rows - 1)) (0 if that sum < 1e-6,
 *   containers/matrix/operations_generic.h:640-691); mean += (m - mean) / age; std += (s - std) / age. age is a device counter. */
int rlt_rocm_running_normalizer_update(rlt_rocm_device* device, const float* data, int ld, int rows, int dim, float* mean, float* std, uint32_t* age);

/* The columns of the on-policy dataset that collect() writes (rl/components/on_policy_runner/on_policy_runner.h:38-72), each passed
 * with the dataset's row stride `ld`; rows are step-major (row = step * n_envs + env). observations and all_reset have
 * (steps_per_env + 1) * n_envs rows: the observation after the last step and the delayed reset flags go there. */
typedef struct rlt_on_policy_dataset {
    float* observations;       /* [(steps + 1) * n_envs x observation_dim] */
    float* actions_mean;       /* [steps * n_envs x action_dim] */
    float* actions;            /* [steps * n_envs x action_dim] */
    float* action_log_probs;   /* [steps * n_envs] */
    float* rewards;            /* [steps * n_envs] */
    float* terminated;         /* [steps * n_envs], flags as floats */
    float* truncated;          /* [steps * n_envs] */
    float* all_reset;          /* [(steps + 1) * n_envs] */
    int32_t ld, steps_per_env;
} rlt_on_policy_dataset;

size_t rlt_rocm_on_policy_collect_workspace_bytes(const rlt_pendulum_runner* runner, const rlt_dense_layer* actor, int n_actor_layers);
/* collect                 rl/components/on_policy_runner/operations_generic.h:105-146, operations_generic_per_env.h:8-74
 *   for the Pendulum environments of `runner` (episode_step_limit 0 = none): per step the prologue (reset where truncated from
 *   initial_states [steps x n_envs x 2], consumed only where a reset happens; observe), the actor (optional standardize layer,
 *   then the MLP giving the action means) and the epilogue (action = mean + exp(log_std) * action_noise [steps x n_envs x
 *   action_dim], its log-probability, environment step, reward, episode counters, truncation, delayed reset flag); at the end
 *   the final observation. The reference draws the noise and the initial states from its RNG while it goes; a caller here
 *   draws them beforehand (rlt_rocm_randn_f32 / rlt_rocm_rand_f32). */
int rlt_rocm_on_policy_collect(rlt_rocm_device* device, const rlt_pendulum_runner* runner, const rlt_on_policy_dataset* dataset,
                               const rlt_dense_layer* actor, int n_actor_layers, const float* log_std,
                               const float* standardize_mean, const float* standardize_precision,
                               const float* action_noise, const float* initial_states, int truncate_on_each_iteration,
                               void* workspace, size_t workspace_bytes);

/* The runner step of rlt_rocm_env_runner_step with a sequential policy (dense and GRU layers) and its rollout state
 * (rl/components/off_policy_runner/operations_generic.h:189-206): after the prologue the policy state of the environments that start a new
 * episode is reset, then one evaluate_step in Rollout mode, then the policy's last layer:
 *   head_kind 1  the output is the action
 *             2  the output is [mean | log_std]: sample_and_squash with action_noise (SAC; `sas` required)
 *             3  td3_sampling (nn/layers/td3_sampling/operations_generic.h:75-128): action = clamp(output + exploration_noise_std * action_noise, -1, 1) (TD3)
 * action_noise [n_envs x action_dim] standard normal values (unused for head_kind 1). policy_state may be NULL for a policy of dense layers. */
size_t rlt_rocm_env_runner_step_sequential_workspace_bytes(const rlt_env_runner* runner, const rlt_seq_layer* policy, int n_policy_layers);
int rlt_rocm_env_runner_step_sequential(rlt_rocm_device* device, const rlt_env_runner* runner, const rlt_replay_buffer* rb,
                                        const rlt_seq_layer* policy, int n_policy_layers, const rlt_seq_state* policy_state, int auto_reset_period,
                                        int head_kind, const rlt_sas_parameters* sas, float exploration_noise_std, const float* action_noise,
                                        const float* initial_states, void* workspace, size_t workspace_bytes);
/* The same step with every draw made by the launch itself, for at most 16 environments and a policy of at most 8 dense layers no wider than 256 (the loops that
 * step one or a few environments per training step): ONE launch for reset, observation, policy, head, dynamics, counters and the replay add.
 *   head_kind 0 (n_policy_layers = 0): uniform actions in (-1, 1), the exploration policy of the warm-up phase (nn_models/random_uniform/operations_generic.h:28-44);
 *   1, 2, 3 as above. Draws: element e * action_dim + c of stream noise_stream under `seed` (what rlt_rocm_randn_f32 would write there; for head_kind 0 what
 *   rlt_rocm_rand_f32(-1, 1) would), and for an environment that starts an episode state component i = initial_low[i] + (initial_high[i] - initial_low[i]) * u
 *   with u element e * state_dim + i of rlt_rocm_rand_f32(0, 1) on stream initial_state_stream (the environments' sample_initial_state, e.g.
 *   rl/environments/acrobot/operations_generic.h:39-52); initial_low and initial_high are HOST arrays of state_dim floats. drawn_noise (optional, device) [n_envs x action_dim] receives the noise or the uniform actions.
 * RLT_E_UNSUPPORTED for more environments, a recurrent or wider policy: draw into arrays and call rlt_rocm_env_runner_step_sequential then. */
int rlt_rocm_env_runner_step_drawn(rlt_rocm_device* device, const rlt_env_runner* runner, const rlt_replay_buffer* rb, const rlt_seq_layer* policy, int n_policy_layers,
                                   int head_kind, const rlt_sas_parameters* sas, float exploration_noise_std, const float* initial_low, const float* initial_high,
                                   float* drawn_noise, uint64_t seed, uint64_t noise_stream, uint64_t initial_state_stream);

/* collect for any of the batched environments and any sequential policy (dense and GRU layers): rl/components/on_policy_runner/
 * operations_generic.h:105-146 over operations_generic_per_env.h:8-74. Per step: reset(policy, policy_state) where the runner's truncated flag
 * is set (before the prologue clears it, :127-130; skipped when policy_state is NULL), the prologue (environments whose flag is set start
 * again from initial_states [steps x n_envs x state_dim], consumed only where a reset happens; observe into the dataset), evaluate_step of the
 * policy in Rollout mode (after the optional standardize layer) giving the action means, the epilogue (action = mean + exp(log_std) * noise
 * with action_noise [steps x n_envs x action_dim], its log-probability, the environment's step, reward and terminated flag, counters,
 * truncated = terminated or episode_step >= episode_step_limit > 0, the delayed reset flag); at the end the final observation. The runner's
 * per-step buffers (actions, rewards, terminated) are used as staging. A policy of dense layers only is an MLP policy. */
size_t rlt_rocm_env_on_policy_collect_workspace_bytes(const rlt_env_runner* runner, const rlt_seq_layer* policy, int n_policy_layers);
int rlt_rocm_env_on_policy_collect(rlt_rocm_device* device, const rlt_env_runner* runner, const rlt_on_policy_dataset* dataset,
                                   const rlt_seq_layer* policy, int n_policy_layers, const rlt_seq_state* policy_state, int auto_reset_period,
                                   const float* log_std, const float* standardize_mean, const float* standardize_precision,
                                   const float* action_noise, const float* initial_states, int truncate_on_each_iteration,
                                   void* workspace, size_t workspace_bytes);

/* rl::utils::evaluation::evaluate  rl/utils/evaluation/operations_generic.h:113-233 for any of the batched environments and any sequential
 * policy (dense and GRU layers): n_episodes episodes of at most step_limit steps from initial_states [n_episodes x state_dim]. Of `env` the
 * env_kind and the parameters it names are read. reset(policy, policy_state) before the first step (:135; policy_state may be NULL for a
 * policy of dense layers), then per step observe, the optional standardize layer (observation_mean / observation_precision [observation_dim],
 * both NULL: none), evaluate_step in Evaluation mode, the head (policy_kind 1: the output [action_dim] is the action; 2: the output is
 * [mean | log_std] and the action is tanh(mean)), the environment's step, reward and terminated. An episode counts rewards and steps up to and
 * including the step that terminates it (:187-197). Outputs as rlt_rocm_pendulum_evaluate: returns [n_episodes], episode_length [n_episodes],
 * summary [6] = {returns_mean, returns_std, episode_length_mean, episode_length_std, num_terminated, share_terminated}. */
size_t rlt_rocm_env_evaluate_workspace_bytes(int env_kind, const rlt_seq_layer* policy, int n_policy_layers, int n_episodes);
int rlt_rocm_env_evaluate(rlt_rocm_device* device, const rlt_env_runner* env, int policy_kind, const rlt_seq_layer* policy, int n_policy_layers,
                          const rlt_seq_state* policy_state, int auto_reset_period, const float* observation_mean, const float* observation_precision,
                          const float* initial_states, int n_episodes, int step_limit, float* returns, uint32_t* episode_length, float* summary,
                          void* workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif /* RLT_ROCM_H */
