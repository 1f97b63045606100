// Internal entry points of optim.hip.
#pragma once
#include "common.h"

// Gradients that are still blocks of partial sums (one block of `block_stride` floats per workgroup of the kernel that made them): the
// optimiser's launch adds them up, in the order of the small-MLP reduction kernel, stores the sums in the tensors' gradients and steps.
// offsets[t]: where tensor t's gradient starts within a block; scales[t]: factor on its sums.
struct rlt_adam_source { const float* partial; int groups, block_stride; const uint32_t* offsets; const float* scales; };

// rlt_rocm_adam_step for at most 12 tensors whose gradients are blocks of partial sums
int rlt_adam_step_from_partials(rlt_rocm_device* device, const rlt_adam_tensor* tensors, int n, const rlt_adam_parameters* parameters, uint32_t* age, const rlt_adam_source* source);

// rlt_rocm_adam_step for two optimisers (each with its own tensors, parameters and age) in one launch; each list at most 12 tensors
// where a source is given
int rlt_adam_step_pair(rlt_rocm_device* device, const rlt_adam_tensor* tensors_a, int n_a, const rlt_adam_parameters* parameters_a, uint32_t* age_a,
                       const rlt_adam_tensor* tensors_b, int n_b, const rlt_adam_parameters* parameters_b, uint32_t* age_b,
                       const rlt_adam_source* source_a = nullptr, const rlt_adam_source* source_b = nullptr);
