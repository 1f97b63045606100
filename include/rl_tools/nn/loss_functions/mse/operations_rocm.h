// Mean squared error on devices::ROCM (the counterpart of nn/loss_functions/mse/operations_cuda.h:10-60).
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/containers/matrix/operations_rocm.h>
#include <rl_tools/nn/loss_functions/mse/operations_generic.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools::nn::loss_functions::mse{
    // gradient                mse/operations_cuda.h:39-57: d_a = (a - b) * 2 / (rows * cols) * loss_weight, the weight read from the device when given
    template<typename DEV_SPEC, typename SPEC_A, typename SPEC_B, typename SPEC_DA, typename LOSS_WEIGHT_SPEC>
    void gradient(devices::ROCM<DEV_SPEC>& device, Matrix<SPEC_A>& a, Matrix<SPEC_B>& b, Matrix<SPEC_DA>& d_a, Tensor<LOSS_WEIGHT_SPEC>& loss_weight){
        static_assert(containers::check_structure<SPEC_A, SPEC_B> && containers::check_structure<SPEC_A, SPEC_DA>);
        static_assert(SPEC_A::COL_PITCH == 1 && SPEC_B::COL_PITCH == 1 && SPEC_DA::COL_PITCH == 1);
        static_assert(LOSS_WEIGHT_SPEC::SHAPE::LENGTH == 1);
        static_assert(LOSS_WEIGHT_SPEC::SHAPE::template GET<0> == 1 || LOSS_WEIGHT_SPEC::SHAPE::template GET<0> == 0);
        constexpr bool LOSS_WEIGHT_PROVIDED = LOSS_WEIGHT_SPEC::SHAPE::template GET<0> == 1;
        const float* weight = nullptr;
        if constexpr(LOSS_WEIGHT_PROVIDED){ weight = loss_weight._data; }
        devices::rocm::check(rlt_rocm_mse_gradient(device.handle, a._data, SPEC_A::ROW_PITCH, b._data, SPEC_B::ROW_PITCH, d_a._data, SPEC_DA::ROW_PITCH, SPEC_A::ROWS, SPEC_A::COLS, 1.0f, weight), "mse::gradient");
    }
    template<typename DEV_SPEC, typename SPEC_A, typename SPEC_B, typename SPEC_DA>
    void gradient(devices::ROCM<DEV_SPEC>& device, Matrix<SPEC_A>& a, Matrix<SPEC_B>& b, Matrix<SPEC_DA>& d_a, typename SPEC_A::T loss_weight = 1){
        static_assert(containers::check_structure<SPEC_A, SPEC_B> && containers::check_structure<SPEC_A, SPEC_DA>);
        static_assert(SPEC_A::COL_PITCH == 1 && SPEC_B::COL_PITCH == 1 && SPEC_DA::COL_PITCH == 1);
        devices::rocm::check(rlt_rocm_mse_gradient(device.handle, a._data, SPEC_A::ROW_PITCH, b._data, SPEC_B::ROW_PITCH, d_a._data, SPEC_DA::ROW_PITCH, SPEC_A::ROWS, SPEC_A::COLS, (float)loss_weight, nullptr), "mse::gradient");
    }
    // evaluate                mse/operations_generic.h:9-21: the value is read back, so the stream is waited for
    template<typename DEV_SPEC, typename SPEC_A, typename SPEC_B>
    typename SPEC_A::T evaluate(devices::ROCM<DEV_SPEC>& device, Matrix<SPEC_A>& a, Matrix<SPEC_B>& b, typename SPEC_A::T loss_weight = 1){
        static_assert(containers::check_structure<SPEC_A, SPEC_B> && SPEC_A::COL_PITCH == 1 && SPEC_B::COL_PITCH == 1);
        float* out = nullptr; float value = 0;
        devices::rocm::check(rlt_rocm_malloc(device.handle, (void**)&out, sizeof(float)), "mse::evaluate");
        devices::rocm::check(rlt_rocm_mse_evaluate(device.handle, a._data, SPEC_A::ROW_PITCH, b._data, SPEC_B::ROW_PITCH, SPEC_A::ROWS, SPEC_A::COLS, (float)loss_weight, out), "mse::evaluate");
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, &value, out, sizeof(float)), "mse::evaluate");
        devices::rocm::check(rlt_rocm_free(device.handle, out), "mse::evaluate");
        return value;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
