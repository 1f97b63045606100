// Single-pass forward + backward of a 3-layer MLP in -> 256 -> 256 -> out (mlp_fused.hip).
#pragma once
#include "common.h"

// bytes of workspace the fused path needs for this network and batch; 0 if the network does not have the supported shape
// (3 layers, in <= 32, both hidden widths 256, out <= 16, activations whose derivative follows from the output)
size_t rlt_mlp3_fused_workspace_bytes(const rlt_dense_layer* layers, int n_layers, int batch);
// same contract as rlt_rocm_mlp_forward_backward; RLT_E_UNSUPPORTED if the shape or the workspace does not fit
int rlt_mlp3_fused_forward_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy,
                                    const float* d_output, int ldd, const float* target, int ldt, float mse_scale, int batch,
                                    void* workspace, size_t workspace_bytes);
// forward(mlp) writing every layer's pre-activations and outputs; RLT_E_UNSUPPORTED if the shape does not fit
int rlt_mlp3_fused_forward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, int batch);
// backward(mlp) with weight gradients and no input gradient, from the outputs a forward() left in the layers; d_pre_last [batch x out] is the
// gradient at the last layer's pre-activations. RLT_E_UNSUPPORTED if the shape or the workspace does not fit
int rlt_mlp3_fused_backward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, const float* d_pre_last, int ldd,
                            int batch, void* workspace, size_t workspace_bytes);
