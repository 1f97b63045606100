// Observation normalisation: the standardize layer and the running normaliser that feeds it.
// reference: nn/layers/standardize/operations_generic.h:54-120, rl/components/running_normalizer/operations_generic.h:18-45,
//            column mean / deviation: containers/matrix/operations_generic.h:640-691.
#include "common.h"

namespace {

__global__ __launch_bounds__(64) void standardize_set_statistics_kernel(const float* __restrict__ mean, const float* __restrict__ std, float* __restrict__ layer_mean,
                                                                        float* __restrict__ layer_precision, int dim) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < dim; i += gridDim.x * blockDim.x) {
        layer_mean[i] = mean[i];
        const float s = std[i];
        layer_precision[i] = s == 0.0f ? 0.0f : 1.0f / s;
    }
}

__global__ __launch_bounds__(256) void standardize_forward_kernel(const float* __restrict__ layer_mean, const float* __restrict__ layer_precision, const float* __restrict__ input,
                                                                  int ldin, float* __restrict__ output, int ldo, int batch, int dim) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < (size_t)batch * dim; i += (size_t)gridDim.x * blockDim.x) {
        const size_t b = i / dim; const int c = (int)(i - b * dim);
        float v = input[b * ldin + c] - layer_mean[c];
        const float p = layer_precision[c];
        if (p != 0.0f) v *= p;
        output[b * ldo + c] = v;
    }
}

__global__ __launch_bounds__(256) void standardize_backward_input_kernel(const float* __restrict__ layer_precision, const float* __restrict__ d_output, int ldd,
                                                                         float* __restrict__ d_input, int ldi, int batch, int dim) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < (size_t)batch * dim; i += (size_t)gridDim.x * blockDim.x) {
        const size_t b = i / dim; const int c = (int)(i - b * dim);
        d_input[b * ldi + c] = d_output[b * ldd + c] * layer_precision[c];
    }
}

// sum over a workgroup of 1024 lanes, result in every lane
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = rlt_wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.0f;
    for (int i = 0; i < 16; i++) s += scratch[i];
    return s;
}

// one workgroup per column: mean, then the sum of squared deviations from it, then the running update with age + 1
__global__ __launch_bounds__(1024) void running_normalizer_kernel(const float* __restrict__ data, int ld, int rows, float* __restrict__ mean, float* __restrict__ std,
                                                                  const uint32_t* __restrict__ age) {
    __shared__ float scratch[16];
    const int c = blockIdx.x;
    float acc = 0.0f;
    for (int r = threadIdx.x; r < rows; r += blockDim.x) acc += data[(size_t)r * ld + c];
    const float data_mean = block_sum(acc, scratch) / (float)rows;
    float sq = 0.0f;
    for (int r = threadIdx.x; r < rows; r += blockDim.x) { const float d = data[(size_t)r * ld + c] - data_mean; sq += d * d; }
    sq = block_sum(sq, scratch);
    if (threadIdx.x == 0) {
        const float data_std = sq < 1e-6f ? 0.0f : sqrtf(sq / (float)(rows - 1));
        const float a = (float)(*age + 1u);
        mean[c] = mean[c] + (data_mean - mean[c]) / a;
        std[c] = std[c] + (data_std - std[c]) / a;
    }
}
__global__ void increment_kernel(uint32_t* counter) { if (threadIdx.x == 0 && blockIdx.x == 0) *counter += 1u; }

int grid1(size_t n) { size_t b = (n + 255) / 256; return (int)(b > 2048 ? 2048 : (b < 1 ? 1 : b)); }

}  // namespace

extern "C" {

int rlt_rocm_standardize_set_statistics(rlt_rocm_device* device, const float* mean, const float* std, float* layer_mean, float* layer_precision, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(mean && std && layer_mean && layer_precision && dim > 0);
    hipLaunchKernelGGL(standardize_set_statistics_kernel, dim3(rlt_div_up(dim, 64)), dim3(64), 0, device->stream, mean, std, layer_mean, layer_precision, dim);
    return rlt_launch_status(device);
}

int rlt_rocm_standardize_forward(rlt_rocm_device* device, const float* layer_mean, const float* layer_precision, const float* input, int ldin, float* output, int ldo,
                                 int batch, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_mean && layer_precision && input && output && batch > 0 && dim > 0 && ldin >= dim && ldo >= dim);
    hipLaunchKernelGGL(standardize_forward_kernel, dim3(grid1((size_t)batch * dim)), dim3(256), 0, device->stream, layer_mean, layer_precision, input, ldin, output, ldo, batch, dim);
    return rlt_launch_status(device);
}

int rlt_rocm_standardize_backward_input(rlt_rocm_device* device, const float* layer_precision, const float* d_output, int ldd, float* d_input, int ldi, int batch, int dim) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(layer_precision && d_output && d_input && batch > 0 && dim > 0 && ldd >= dim && ldi >= dim);
    hipLaunchKernelGGL(standardize_backward_input_kernel, dim3(grid1((size_t)batch * dim)), dim3(256), 0, device->stream, layer_precision, d_output, ldd, d_input, ldi, batch, dim);
    return rlt_launch_status(device);
}

int rlt_rocm_running_normalizer_update(rlt_rocm_device* device, const float* data, int ld, int rows, int dim, float* mean, float* std, uint32_t* age) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(data && mean && std && age && rows >= 2 && dim > 0 && ld >= dim);
    hipLaunchKernelGGL(running_normalizer_kernel, dim3(dim), dim3(1024), 0, device->stream, data, ld, rows, mean, std, (const uint32_t*)age);
    int rc = rlt_launch_status(device);
    if (rc) return rc;
    hipLaunchKernelGGL(increment_kernel, dim3(1), dim3(64), 0, device->stream, age);
    return rlt_launch_status(device);
}

}  // extern "C"
