// Group 1 of the ROCM backend's operations (device tag, logging), the counterpart of operations/cuda/group_1.h:1-17. Included
// after the CPU groups (operations/cpu_mux.h): the tag reuses the CPU's math and logging.
#pragma once
#ifndef RL_TOOLS_OPERATIONS_ROCM_GROUP_1
    #define RL_TOOLS_OPERATIONS_ROCM_GROUP_1
    #include <rl_tools/devices/rocm.h>
    #include <rl_tools/numeric_types/policy.h>
    #include <rl_tools/utils/env/operations_generic.h>
#else
    #error "Group 1 already imported"
#endif
