// Group 2 of the ROCM backend's operations (assert, random numbers), the counterpart of operations/cuda/group_2.h:1-12.
#pragma once
#ifndef RL_TOOLS_OPERATIONS_ROCM_GROUP_2
    #define RL_TOOLS_OPERATIONS_ROCM_GROUP_2
    #include <rl_tools/utils/assert/operations_rocm.h>
    #include <rl_tools/random/operations_rocm.h>
#else
    #error "Group 2 already imported"
#endif
