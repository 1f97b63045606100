// The Tensor elementwise operations as callable entries: unary_operation, binary_operation, ternary_operation and the abs-max reduction
// (reference: containers/tensor/operations_generic.h:365-481 functors, :573-760 the operations; CUDA: operations_cuda.h:172-283, 359-544, 287-307).
// Operands are 2-D views [rows x cols] with their own leading dimensions, so that a contiguous tensor is one row and a column block of a
// matrix is a view; dst may be any of the operands. Bound: HBM, 8-12 B per element.
#include "common.h"

namespace {
__device__ __forceinline__ float unary_apply(int op, float a, float parameter) {
    switch (op) {
        case RLT_UNARY_NEGATE: return -a;
        case RLT_UNARY_ABS: return fabsf(a);
        case RLT_UNARY_CONSTANT: return parameter;
        case RLT_UNARY_SIGMOID: return a < -20.0f ? 0.0f : (a > 20.0f ? 1.0f : 1.0f / (1.0f + expf(-a)));
        case RLT_UNARY_FAST_SIGMOID: return 0.5f * rlt_fast_tanh(0.5f * a) + 0.5f;
        case RLT_UNARY_EXP: return expf(a);
        case RLT_UNARY_TANH: return tanhf(a);
        case RLT_UNARY_FAST_TANH: return rlt_fast_tanh(a);
        case RLT_UNARY_ONE_MINUS: return 1.0f - a;
        case RLT_UNARY_SCALE: return a * parameter;
        case RLT_UNARY_SCALE_RECIPROCAL: return 1.0f / a * parameter;
        default: return a;
    }
}
__global__ __launch_bounds__(256) void unary_kernel(int op, float parameter, const float* src, int lds, float* dst, int ldd, int rows, int cols) {
    const size_t total = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / cols, c = i % cols;
        dst[r * ldd + c] = unary_apply(op, src[r * lds + c], parameter);
    }
}
__global__ __launch_bounds__(256) void binary_kernel(int op, const float* a, int lda, const float* b, int ldb, float* dst, int ldd, int rows, int cols) {
#pragma clang fp contract(off)
    const size_t total = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / cols, c = i % cols;
        const float x = a[r * lda + c], y = b[r * ldb + c];
        dst[r * ldd + c] = op == RLT_BINARY_ADD ? x + y : op == RLT_BINARY_SUBTRACT ? x - y : op == RLT_BINARY_MULTIPLY ? x * y : x / y;
    }
}
// acc + a * b with the product rounded before the addition, as the reference's CPU build computes it
__global__ __launch_bounds__(256) void multiply_accumulate_kernel(const float* a, int lda, const float* b, int ldb, const float* acc, int ldc, float* dst, int ldd, int rows, int cols) {
#pragma clang fp contract(off)
    const size_t total = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / cols, c = i % cols;
        const float product = a[r * lda + c] * b[r * ldb + c];
        dst[r * ldd + c] = acc[r * ldc + c] + product;
    }
}
// max |x| over a contiguous tensor: one workgroup, lanes stride through the data, wavefront butterflies, then the 16 wavefronts' maxima
__global__ __launch_bounds__(1024) void abs_max_kernel(const float* __restrict__ x, size_t count, float* __restrict__ out) {
    __shared__ float partial[16];
    float m = 0.0f;
    for (size_t i = threadIdx.x; i < count; i += blockDim.x) m = fmaxf(m, fabsf(x[i]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) { float r = 0.0f; for (int i = 0; i < 16; i++) r = fmaxf(r, partial[i]); *out = r; }
}
int grid_for(size_t n) { const size_t b = (n + 255) / 256; return (int)(b > 4096 ? 4096 : (b < 1 ? 1 : b)); }
}  // namespace

extern "C" {

int rlt_rocm_unary_f32(rlt_rocm_device* device, int operation, float parameter, const float* src, int ld_src, float* dst, int ld_dst, int rows, int cols) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(src && dst && rows > 0 && cols > 0 && ld_src >= cols && ld_dst >= cols && operation >= RLT_UNARY_NEGATE && operation <= RLT_UNARY_SCALE_RECIPROCAL);
    hipLaunchKernelGGL(unary_kernel, dim3(grid_for((size_t)rows * cols)), dim3(256), 0, device->stream, operation, parameter, src, ld_src, dst, ld_dst, rows, cols);
    return rlt_launch_status(device);
}
int rlt_rocm_binary_f32(rlt_rocm_device* device, int operation, const float* a, int lda, const float* b, int ldb, float* dst, int ld_dst, int rows, int cols) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(a && b && dst && rows > 0 && cols > 0 && lda >= cols && ldb >= cols && ld_dst >= cols && operation >= RLT_BINARY_ADD && operation <= RLT_BINARY_DIVIDE);
    hipLaunchKernelGGL(binary_kernel, dim3(grid_for((size_t)rows * cols)), dim3(256), 0, device->stream, operation, a, lda, b, ldb, dst, ld_dst, rows, cols);
    return rlt_launch_status(device);
}
int rlt_rocm_multiply_accumulate_f32(rlt_rocm_device* device, const float* a, int lda, const float* b, int ldb, const float* accumulator, int ldc, float* dst, int ld_dst,
                                     int rows, int cols) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(a && b && accumulator && dst && rows > 0 && cols > 0 && lda >= cols && ldb >= cols && ldc >= cols && ld_dst >= cols);
    hipLaunchKernelGGL(multiply_accumulate_kernel, dim3(grid_for((size_t)rows * cols)), dim3(256), 0, device->stream, a, lda, b, ldb, accumulator, ldc, dst, ld_dst, rows, cols);
    return rlt_launch_status(device);
}
int rlt_rocm_reduce_abs_max_f32(rlt_rocm_device* device, const float* x, size_t count, float* out_max) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(x && out_max);
    hipLaunchKernelGGL(abs_max_kernel, dim3(1), dim3(1024), 0, device->stream, x, count, out_max);
    return rlt_launch_status(device);
}

}  // extern "C"
