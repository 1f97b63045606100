// Internal entry points of optim.hip.
#pragma once
#include "common.h"

// rlt_rocm_adam_step for two optimisers (each with its own tensors, parameters and age) in one launch; each list at most 12 tensors
int rlt_adam_step_pair(rlt_rocm_device* device, const rlt_adam_tensor* tensors_a, int n_a, const rlt_adam_parameters* parameters_a, uint32_t* age_a,
                       const rlt_adam_tensor* tensors_b, int n_b, const rlt_adam_parameters* parameters_b, uint32_t* age_b);
