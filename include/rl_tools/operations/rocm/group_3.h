// Group 3 of the ROCM backend's operations (containers), the counterpart of operations/cuda/group_3.h:1-12.
#pragma once
#ifndef RL_TOOLS_OPERATIONS_ROCM_GROUP_3
    #define RL_TOOLS_OPERATIONS_ROCM_GROUP_3
    #include <rl_tools/containers/matrix/operations_rocm.h>
    #include <rl_tools/containers/tensor/operations_rocm.h>
#else
    #error "Group 3 already imported"
#endif
