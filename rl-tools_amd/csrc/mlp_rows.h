// Internal entry point of the few-rows forward kernel (mlp_rows.hip).
#pragma once
#include "common.h"

// All layers of an MLP over a batch of at most RLT_MLP_ROWS_MAX_BATCH rows in one launch (every width at most 256, at most 8 layers).
// keep: the layers' pre_activations / output buffers are written (forward); y (optional when keep is set) receives the last layer's output.
// RLT_E_UNSUPPORTED when the shapes are not the kernel's: the caller then takes the per-layer kernels.
constexpr int RLT_MLP_ROWS_MAX_BATCH = 2048;
// RLT_MLP_ROWS=0 in the environment keeps such calls on the per-layer kernels (tests compare the two paths)
bool rlt_mlp_rows_enabled();
int rlt_mlp_rows_forward(rlt_rocm_device* device, const rlt_dense_layer* layers, int n_layers, const float* x, int ldx, float* y, int ldy, int batch, bool keep);
// The same for two networks of one depth on the same input rows in one launch (a pair of critics): outputs y_first / y_second (optional when keep is set).
int rlt_mlp_rows_forward_pair(rlt_rocm_device* device, const rlt_dense_layer* first, const rlt_dense_layer* second, int n_layers, const float* x, int ldx,
                              float* y_first, float* y_second, int ldy, int batch, bool keep);
// forward (keep) or evaluate of a pair of networks of one shape on the same rows: one launch for both when the few-rows kernel takes the shapes, else one network
// after the other through rlt_rocm_mlp_forward / rlt_rocm_mlp_evaluate (ws: the workspace those take)
int rlt_mlp_forward_pair(rlt_rocm_device* device, const rlt_dense_layer* first, const rlt_dense_layer* second, int n_layers, const float* x, int ldx, float* y_first,
                         float* y_second, int ldy, int batch, bool keep, void* ws, size_t ws_bytes);
