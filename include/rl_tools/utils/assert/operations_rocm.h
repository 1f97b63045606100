// utils::assert_exit for devices::ROCM (utils/assert/operations_cpu.h:8-18 is the CPU's): host code, so it logs and aborts.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <cstdlib>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools::utils{
    template <typename DEV_SPEC, typename T>
    bool assert_exit(devices::ROCM<DEV_SPEC>& device, bool condition, T message){
        if(!condition){
            log(device, device.logger, message);
            std::abort();
        }
        return condition;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
