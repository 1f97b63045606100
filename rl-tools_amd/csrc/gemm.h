// Internal entry points of the dense-layer contraction kernels (gemm.hip).
#pragma once
#include "common.h"

// y/out/pre (each optional) = act(x W^T + bias); pre/out are packed [batch x out_dim], y has leading dimension ldy
int rlt_gemm_forward(rlt_rocm_device* device, const float* x, int ldx, const float* W, const float* bias, int act,
                     float* pre, float* out, float* y, int ldy, int batch, int in_dim, int out_dim);
// d_in = d_pre W, optionally multiplied elementwise by act'(.) of the layer below: dact_pre (packed [batch x in_dim]) holds that
// layer's pre-activations, or its outputs when dact_from_output is set
int rlt_gemm_backward_input(rlt_rocm_device* device, const float* d_pre, int ldd, const float* W, float* d_in, int ldi,
                            const float* dact_pre, int dact_kind, int dact_from_output, int batch, int in_dim, int out_dim);
// dW += d_pre^T x ; dbias += column sums of d_pre (dbias may be NULL). The partial sums of a split batch go to the handle's grow-only
// workspace, or, with static_scratch, to the library's fixed device array (RLT_E_WORKSPACE_TOO_SMALL beyond RLT_STATIC_SCRATCH_BYTES).
// narrow_long: the caller's layers are narrow (at most 192 x 160) and its batches long; such shapes then take the kernel that keeps the whole
// gradient in one workgroup's accumulators (another summation order than the tiled kernel's, so the dense-layer entry points, which promise
// each other's bits, do not ask for it).
int rlt_gemm_wgrad(rlt_rocm_device* device, const float* d_pre, int ldd, const float* x, int ldx, float* dW, float* dbias,
                   int batch, int in_dim, int out_dim, bool static_scratch = false, bool narrow_long = false);
// looks up, once per GPU, where that GPU keeps the fixed array (called by rlt_rocm_init with the handle's device)
int rlt_gemm_static_scratch_setup(rlt_rocm_device* device);
// dst <- act'(pre) * src (dst may alias src; then a no-op for the identity)
int rlt_dpre(rlt_rocm_device* device, const float* src, int lds, float* dst, int ldd, const float* pre, int rows, int cols, int act, int from_output);
// zeroes n tensors (mlp.hip): one launch per 16 runs of tensors that lie back to back
int rlt_zero_tensors(rlt_rocm_device* device, float* const* begins, const size_t* counts, int n);
