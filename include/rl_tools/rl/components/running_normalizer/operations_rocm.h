// The running normaliser on devices::ROCM: update (the generic version, rl/components/running_normalizer/operations_generic.h:25-45,
// is a host loop over columns and elements). init is the generic one (set_all + a host counter).
//
// normalizer.age stays a host member, as in the reference; the library's kernel reads and increments a counter in device memory, so
// each update uploads the host's value first (four bytes, once per loop step).
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/components/running_normalizer/running_normalizer.h>
#include <rl_tools/rl/components/running_normalizer/operations_generic.h>
#include <rl_tools/containers/matrix/operations_rocm.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    template <typename DEV_SPEC, typename SPEC, typename DATA_SPEC>
    void update(devices::ROCM<DEV_SPEC>& device, rl::components::RunningNormalizer<SPEC>& normalizer, Matrix<DATA_SPEC>& data){
        static_assert(DATA_SPEC::COLS == SPEC::DIM, "Data dimension must match normalizer dimension");
        static_assert(DATA_SPEC::ROWS > 1, "Data size must be greater than 1 and should be much greated than one");
        static_assert(utils::typing::is_same_v<typename DATA_SPEC::T, float> && DATA_SPEC::COL_PITCH == 1 && sizeof(typename SPEC::TI) >= 4);
        if constexpr(SPEC::DIM > 0){
            uint32_t* age = (uint32_t*)devices::rocm::scratch(device, sizeof(uint32_t));
            const uint32_t host_age = (uint32_t)normalizer.age;
            devices::rocm::check(rlt_rocm_memcpy_h2d(device.handle, age, &host_age, sizeof(uint32_t)), "update(running normaliser)");
            devices::rocm::check(rlt_rocm_running_normalizer_update(device.handle, data._data, containers::rocm::leading_dimension<DATA_SPEC>, (int)DATA_SPEC::ROWS, (int)SPEC::DIM,
                                                                    normalizer.mean._data, normalizer.std._data, age), "update(running normaliser)");
        }
        normalizer.age++;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
