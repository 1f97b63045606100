// Networks in -> h -> h -> out with h < 64 on the kernels built for hidden width 64 (pad.hip).
#pragma once
#include "common.h"

// A 3-layer network whose hidden activation maps 0 to 0 (identity, relu, tanh, fast_tanh) computes the same outputs, and has the same gradients, as
// the width-64 network that has zero rows and columns added to its weights: the added units output act(0) = 0, feed nothing forward, and receive no
// gradient. rlt_pad_parameters writes that network's parameters (and room for its gradients) into `memory` and describes it; the one-launch kernels
// then run on the description, and rlt_unpad_gradients copies the h-wide blocks of the gradients they leave into the caller's gradient arrays
// (overwriting them, as those kernels do).
struct rlt_padded_net { rlt_dense_layer L[3]; };
bool rlt_pad_eligible(const rlt_dense_layer* layers, int n_layers);
size_t rlt_pad_floats(const rlt_dense_layer* layers, bool with_gradients);
int rlt_pad_parameters(rlt_rocm_device* device, const rlt_dense_layer* layers, float* memory, bool with_gradients, rlt_padded_net* out);
int rlt_unpad_gradients(rlt_rocm_device* device, const rlt_dense_layer* layers, const rlt_padded_net* padded);
// a second grow-only buffer of the handle, for the padded copies (the kernels that run on them take the first for their partial sums)
int rlt_pad_scratch(rlt_rocm_device* device, size_t bytes, void** out);
