// All base operations of devices::ROCM (the counterpart of operations/cuda.h). Include it AFTER <rl_tools/operations/cpu_mux.h>:
// the ROCM tag builds on the CPU device (host-side math, logging, and the CPU <-> ROCM copies).
//
//     #include <rl_tools/operations/cpu_mux.h>
//     #include <rl_tools/operations/rocm.h>
//     #include <rl_tools/nn/operations_cpu_mux.h>
//     #include <rl_tools/nn/operations_rocm.h>
//
// and the program links against librlt_rocm.so. devices::DEVICE_FACTORY_ROCM<> names the default device type, as
// devices::DEVICE_FACTORY_CUDA<> does for CUDA (operations/cpu_mux.h:137-144).
#pragma once
#include <rl_tools/operations/rocm/group_1.h>
#include <rl_tools/operations/rocm/group_2.h>
#include <rl_tools/operations/rocm/group_3.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools::devices{
    template<typename DEV_SPEC = devices::DefaultROCMSpecification>
    using DEVICE_FACTORY_ROCM = devices::ROCM<DEV_SPEC>;
}
RL_TOOLS_NAMESPACE_WRAPPER_END
