// Polyak (soft) updates on devices::ROCM (the counterpart of utils/polyak/operations_cuda.h:9-50; signatures as in
// utils/polyak/operations_generic.h:9-40,77-97).
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/containers/matrix/operations_rocm.h>
#include <rl_tools/utils/polyak/operations_generic.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools::utils::polyak{
    namespace rocm{
        template<typename DEVICE>
        void update(DEVICE& device, const float* source, float* target, size_t count, float polyak, int squared, bool clip){
            utils::assert_exit(device, !clip, "polyak updates with clipping are not available on devices::ROCM");
            devices::rocm::check(rlt_rocm_polyak_update(device.handle, source, target, count, polyak, squared), "polyak::update");
        }
        template <typename SOURCE_SPEC, typename TARGET_SPEC>
        constexpr bool dense_matrices = containers::check_structure<SOURCE_SPEC, TARGET_SPEC> && containers::rocm::dense<SOURCE_SPEC> && containers::rocm::dense<TARGET_SPEC>;
    }
    // target = polyak * target + (1 - polyak) * source
    template<typename DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC, typename T_POLYAK>
    void update(devices::ROCM<DEV_SPEC>& device, const Matrix<SOURCE_SPEC>& source, Matrix<TARGET_SPEC>& target, const T_POLYAK polyak, bool clip = false, typename SOURCE_SPEC::T clip_value = 1){
        static_assert(rocm::dense_matrices<SOURCE_SPEC, TARGET_SPEC>, "polyak updates run over dense matrices");
        rocm::update(device, source._data, target._data, (size_t)SOURCE_SPEC::ROWS * SOURCE_SPEC::COLS, (float)polyak, 0, clip);
    }
    // target = polyak * target + (1 - polyak) * source^2
    template<typename DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC, typename T_POLYAK>
    void update_squared(devices::ROCM<DEV_SPEC>& device, const Matrix<SOURCE_SPEC>& source, Matrix<TARGET_SPEC>& target, const T_POLYAK polyak, bool clip = false, typename SOURCE_SPEC::T clip_value = 1){
        static_assert(rocm::dense_matrices<SOURCE_SPEC, TARGET_SPEC>, "polyak updates run over dense matrices");
        rocm::update(device, source._data, target._data, (size_t)SOURCE_SPEC::ROWS * SOURCE_SPEC::COLS, (float)polyak, 1, clip);
    }
    template<typename DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC, typename T_POLYAK>
    void update(devices::ROCM<DEV_SPEC>& device, const Tensor<SOURCE_SPEC>& source, Tensor<TARGET_SPEC>& target, const T_POLYAK polyak, const bool clip = false, typename SOURCE_SPEC::T clip_value = 1){
        static_assert(tensor::same_dimensions<SOURCE_SPEC, TARGET_SPEC>() && tensor::dense_row_major_layout<SOURCE_SPEC>() && tensor::dense_row_major_layout<TARGET_SPEC>());
        rocm::update(device, source._data, target._data, (size_t)SOURCE_SPEC::SIZE, (float)polyak, 0, clip);
    }
    template<typename DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC, typename T_POLYAK>
    void update_squared(devices::ROCM<DEV_SPEC>& device, const Tensor<SOURCE_SPEC>& source, Tensor<TARGET_SPEC>& target, const T_POLYAK polyak, const bool clip = false, typename SOURCE_SPEC::T clip_value = 1){
        static_assert(tensor::same_dimensions<SOURCE_SPEC, TARGET_SPEC>() && tensor::dense_row_major_layout<SOURCE_SPEC>() && tensor::dense_row_major_layout<TARGET_SPEC>());
        rocm::update(device, source._data, target._data, (size_t)SOURCE_SPEC::SIZE, (float)polyak, 1, clip);
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
