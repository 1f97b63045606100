// All neural-network operations of devices::ROCM: include after <rl_tools/nn/operations_cpu_mux.h> (which brings the layer types and
// the generic model code), the counterpart of the CUDA includes of nn/operations_cpu_mux.h.
#pragma once
#include <rl_tools/utils/polyak/operations_rocm.h>
#include <rl_tools/nn/layers/dense/operations_rocm.h>
#include <rl_tools/nn/layers/sample_and_squash/operations_rocm.h>
#include <rl_tools/nn/loss_functions/mse/operations_rocm.h>
#include <rl_tools/nn/optimizers/adam/operations_rocm.h>
