// Tensor containers on devices::ROCM: malloc / free / copy / set_all / scale / cast_reduce_sum / randn / rand (the counterpart of
// containers/tensor/operations_cuda.h:15-624). The reference's CUDA backend compiles any element-wise functor into a kernel of its
// own; this backend ships precompiled kernels, so the operations a caller can name are the ones the C ABI has an entry point for.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/containers/tensor/tensor.h>
#include <rl_tools/random/operations_rocm.h>
#include <new>
#include <type_traits>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    // malloc / free           containers/tensor/operations_cuda.h:15-39
    // Tensors of numbers and flags are device memory. Tensors of structs (environments, their parameters, an optimiser's
    // hyper-parameters) are read and written by host code only -- the precompiled kernels know no struct layouts -- and are host memory.
    template<typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE, bool CONST>
    void malloc(devices::ROCM<DEV_SPEC>& device, tensor::TensorDynamic<T, T_TI, SIZE, CONST>& tensor){
        constexpr size_t SIZE_BYTES = (size_t)SIZE * sizeof(T);
        if constexpr(std::is_arithmetic_v<T>){
            void* memory = nullptr;
            devices::rocm::check(rlt_rocm_malloc(device.handle, &memory, SIZE_BYTES > 0 ? SIZE_BYTES : 1), "malloc(tensor)");
            tensor._data = (T*)memory;
        }
        else{
            tensor._data = (T*)::operator new(SIZE_BYTES > 0 ? SIZE_BYTES : 1, std::align_val_t(64));
        }
        count_malloc(device, SIZE_BYTES);
    }
    template <typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE, bool CONST>
    void free(devices::ROCM<DEV_SPEC>& device, tensor::TensorDynamic<T, T_TI, SIZE, CONST>& tensor){
        if constexpr(std::is_arithmetic_v<T>){
            devices::rocm::check(rlt_rocm_free(device.handle, (void*)tensor._data), "free(tensor)");
        }
        else{
            ::operator delete((void*)tensor._data, std::align_val_t(64));
        }
        tensor._data = nullptr;
    }
    template<typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE>
    void malloc(devices::ROCM<DEV_SPEC>& device, tensor::TensorStatic<T, T_TI, SIZE>& tensor){}
    template<typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE>
    void free(devices::ROCM<DEV_SPEC>& device, tensor::TensorStatic<T, T_TI, SIZE>& tensor){}
    template<typename DEV_SPEC, typename T>
    void malloc(devices::ROCM<DEV_SPEC>& device, tensor::TensorStaticEmpty<T>& tensor){}
    template<typename DEV_SPEC, typename T>
    void free(devices::ROCM<DEV_SPEC>& device, tensor::TensorStaticEmpty<T>& tensor){}

    namespace tensor::rocm{
        template <typename SPEC>
        constexpr bool last_dimension_contiguous(){ return SPEC::STRIDE::LAST == 1 || SPEC::SHAPE::LAST == 1; }
        // kind: 0 device -> device, 1 host -> device, 2 device -> host (rlt_rocm_memcpy2d)
        template<typename DEVICE, typename FROM_DEVICE, typename TO_DEVICE, typename FROM_SPEC, typename TO_SPEC>
        void copy(DEVICE& device, FROM_DEVICE& from_device, TO_DEVICE& to_device, const Tensor<FROM_SPEC>& from, Tensor<TO_SPEC>& to, int kind){
            static_assert(tensor::same_dimensions<FROM_SPEC, TO_SPEC>(), "Dimensions must be the same");
            static_assert(utils::typing::is_same_v<utils::typing::remove_cv_t<typename FROM_SPEC::T>, utils::typing::remove_cv_t<typename TO_SPEC::T>>, "copies across the host / device boundary keep the element type");
            using T = typename TO_SPEC::T;
            using TI = typename DEVICE::index_t;
            if constexpr(!std::is_arithmetic_v<utils::typing::remove_cv_t<T>>){
                // containers of structs (an optimiser's hyper-parameters) are host memory on every device (malloc above): copied element by element on the host, whatever the direction
                static_assert(tensor::dense_row_major_layout<FROM_SPEC>() && tensor::dense_row_major_layout<TO_SPEC>(), "containers of structs are copied whole");
                for(size_t i = 0; i < (size_t)FROM_SPEC::SIZE; i++){ to._data[i] = from._data[i]; }
            }
            else if constexpr(tensor::dense_row_major_layout<FROM_SPEC>() && tensor::dense_row_major_layout<TO_SPEC>()){
                const size_t bytes = (size_t)FROM_SPEC::SIZE * sizeof(T);
                const int rc = kind == 0 ? rlt_rocm_memcpy_d2d(device.handle, (void*)to._data, (const void*)from._data, bytes)
                             : kind == 1 ? rlt_rocm_memcpy_h2d(device.handle, (void*)to._data, (const void*)from._data, bytes)
                                         : rlt_rocm_memcpy_d2h(device.handle, (void*)to._data, (const void*)from._data, bytes);
                devices::rocm::check(rc, "copy(tensor)");
            }
            else if constexpr(FROM_SPEC::SHAPE::LENGTH == 1){
                static_assert(last_dimension_contiguous<FROM_SPEC>() && last_dimension_contiguous<TO_SPEC>(), "strided one-dimensional views cannot be copied on devices::ROCM");
                devices::rocm::check(rlt_rocm_memcpy2d(device.handle, (void*)to._data, (size_t)FROM_SPEC::SHAPE::FIRST * sizeof(T), (const void*)from._data, (size_t)FROM_SPEC::SHAPE::FIRST * sizeof(T),
                                                       (size_t)FROM_SPEC::SHAPE::FIRST * sizeof(T), 1, kind), "copy(tensor)");
            }
            else if constexpr(FROM_SPEC::SHAPE::LENGTH == 2 && last_dimension_contiguous<FROM_SPEC>() && last_dimension_contiguous<TO_SPEC>()){
                constexpr TI ROWS = FROM_SPEC::SHAPE::template GET<0>, COLS = FROM_SPEC::SHAPE::template GET<1>;
                devices::rocm::check(rlt_rocm_memcpy2d(device.handle, (void*)to._data, (size_t)TO_SPEC::STRIDE::template GET<0> * sizeof(T), (const void*)from._data, (size_t)FROM_SPEC::STRIDE::template GET<0> * sizeof(T),
                                                       (size_t)COLS * sizeof(T), ROWS, kind), "copy(tensor view)");
            }
            else{
                static_assert(FROM_SPEC::SHAPE::LENGTH > 1, "this view cannot be copied on devices::ROCM");
                for(TI i = 0; i < FROM_SPEC::SHAPE::FIRST; ++i){
                    auto next_from = view(from_device, from, i);
                    auto next_to = view(to_device, to, i);
                    copy(device, from_device, to_device, next_from, next_to, kind);
                }
            }
        }
    }
    // copy ROCM -> ROCM       containers/tensor/operations_cuda.h:94-139
    template<typename FROM_DEV_SPEC, typename TO_DEV_SPEC, typename FROM_SPEC, typename TO_SPEC>
    void copy(devices::ROCM<FROM_DEV_SPEC>& from_device, devices::ROCM<TO_DEV_SPEC>& to_device, const Tensor<FROM_SPEC>& from, Tensor<TO_SPEC>& to){
        tensor::rocm::copy(from_device, from_device, to_device, from, to, 0);
    }
    // copy ROCM -> CPU        containers/tensor/operations_cuda.h:140-153 (synchronises)
    template<typename FROM_DEV_SPEC, typename TO_DEV_SPEC, typename FROM_SPEC, typename TO_SPEC>
    void copy(devices::ROCM<FROM_DEV_SPEC>& from_device, devices::CPU<TO_DEV_SPEC>& to_device, const Tensor<FROM_SPEC>& from, Tensor<TO_SPEC>& to){
        tensor::rocm::copy(from_device, from_device, to_device, from, to, 2);
    }
    // copy CPU -> ROCM        containers/tensor/operations_cuda.h:154-168
    template<typename FROM_DEV_SPEC, typename TO_DEV_SPEC, typename FROM_SPEC, typename TO_SPEC>
    void copy(devices::CPU<FROM_DEV_SPEC>& from_device, devices::ROCM<TO_DEV_SPEC>& to_device, const Tensor<FROM_SPEC>& from, Tensor<TO_SPEC>& to){
        tensor::rocm::copy(to_device, from_device, to_device, from, to, 1);
    }
    // set_all                 containers/tensor/operations_cuda.h:335-347
    template<typename DEV_SPEC, typename SPEC>
    void set_all(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& t, typename SPEC::T value){
        using T = typename SPEC::T;
        using TI = typename devices::ROCM<DEV_SPEC>::index_t;
        if constexpr(tensor::dense_row_major_layout<SPEC>()){
            if constexpr(utils::typing::is_same_v<T, float>){
                devices::rocm::check(rlt_rocm_fill_f32(device.handle, t._data, 1, (int)SPEC::SIZE, (int)SPEC::SIZE, (float)value), "set_all(tensor)");
            }
            else if constexpr(sizeof(T) == 1){
                devices::rocm::check(rlt_rocm_fill_u8(device.handle, (uint8_t*)t._data, (size_t)SPEC::SIZE, (uint8_t)value), "set_all(tensor)");
            }
            else{
                T* host = new T[(size_t)SPEC::SIZE];
                for(size_t i = 0; i < (size_t)SPEC::SIZE; i++){ host[i] = value; }
                devices::rocm::check(rlt_rocm_memcpy_h2d(device.handle, (void*)t._data, host, (size_t)SPEC::SIZE * sizeof(T)), "set_all(tensor)");
                delete[] host;
            }
        }
        else if constexpr(SPEC::SHAPE::LENGTH == 2 && tensor::rocm::last_dimension_contiguous<SPEC>() && utils::typing::is_same_v<T, float>){
            devices::rocm::check(rlt_rocm_fill_f32(device.handle, t._data, (int)SPEC::SHAPE::template GET<0>, (int)SPEC::SHAPE::template GET<1>, (int)SPEC::STRIDE::template GET<0>, (float)value), "set_all(tensor view)");
        }
        else{
            static_assert(SPEC::SHAPE::LENGTH > 1, "this view cannot be filled on devices::ROCM");
            for(TI i = 0; i < SPEC::SHAPE::FIRST; ++i){
                auto next = view(device, t, i);
                set_all(device, next, value);
            }
        }
    }
    // set_all from a one-element tensor on the device   containers/tensor/operations_cuda.h:341-347
    template<typename DEV_SPEC, typename SPEC, typename VALUE_SPEC>
    void set_all(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& t, Tensor<VALUE_SPEC>& value){
        static_assert(VALUE_SPEC::SHAPE::LENGTH == 1 && VALUE_SPEC::SHAPE::template GET<0> == 1);
        static_assert(utils::typing::is_same_v<typename SPEC::T, float> && utils::typing::is_same_v<typename VALUE_SPEC::T, float> && tensor::dense_row_major_layout<SPEC>());
        devices::rocm::check(rlt_rocm_fill_from_f32(device.handle, t._data, 1, (int)SPEC::SIZE, (int)SPEC::SIZE, value._data), "set_all(tensor, tensor)");
    }
    // scale                   containers/tensor/operations_cuda.h:348-355, operations_generic.h:433-445,713
    template<typename DEV_SPEC, typename SPEC>
    void scale(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& t, typename SPEC::T scale, bool reciprocal = false){
        static_assert(utils::typing::is_same_v<typename SPEC::T, float> && tensor::dense_row_major_layout<SPEC>(), "scale works on dense float tensors");
        devices::rocm::check(rlt_rocm_scale_f32(device.handle, t._data, (size_t)SPEC::SIZE, scale, reciprocal ? 1 : 0), "scale(tensor)");
    }
    // cast_reduce_sum         containers/tensor/operations_cuda.h:308-320: the number of set flags of a bool tensor, as a float
    template<typename TARGET_TYPE, typename DEV_SPEC, typename SPEC, typename RESULT_SPEC>
    void cast_reduce_sum(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& t, Tensor<RESULT_SPEC>& result){
        static_assert(RESULT_SPEC::SHAPE::LENGTH == 1 && RESULT_SPEC::SHAPE::template GET<0> == 1);
        static_assert(sizeof(typename SPEC::T) == 1 && utils::typing::is_same_v<TARGET_TYPE, float> && utils::typing::is_same_v<typename RESULT_SPEC::T, float> && tensor::dense_row_major_layout<SPEC>(),
                      "cast_reduce_sum counts the flags of a dense bool tensor into a float");
        devices::rocm::check(rlt_rocm_cast_reduce_sum_u8(device.handle, (const uint8_t*)t._data, (size_t)SPEC::SIZE, result._data), "cast_reduce_sum");
    }
    // sum / squared_sum       containers/tensor/operations_generic.h:497-520,803 (the value is read back: the stream is waited for)
    template<typename DEV_SPEC, typename SPEC>
    typename SPEC::T squared_sum(devices::ROCM<DEV_SPEC>& device, const Tensor<SPEC>& t){
        static_assert(utils::typing::is_same_v<utils::typing::remove_cv_t<typename SPEC::T>, float> && tensor::dense_row_major_layout<SPEC>());
        float* out = nullptr; float value = 0;
        devices::rocm::check(rlt_rocm_malloc(device.handle, (void**)&out, sizeof(float)), "squared_sum");
        devices::rocm::check(rlt_rocm_reduce_sum_f32(device.handle, t._data, (size_t)SPEC::SIZE, 1, out), "squared_sum");
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, &value, out, sizeof(float)), "squared_sum");
        devices::rocm::check(rlt_rocm_free(device.handle, out), "squared_sum");
        return value;
    }
    // unary_operation / binary_operation / ternary_operation   containers/tensor/operations_generic.h:573-760 (CUDA: operations_cuda.h:172-283, 359-544)
    // on dense float tensors: the functor's type selects the library's operation, its members travel as the parameter
    namespace tensor::rocm{
        template<typename OPERATION> struct UnaryId{ static constexpr int ID = -1; static float parameter(const OPERATION&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::Negate>{ static constexpr int ID = RLT_UNARY_NEGATE; static float parameter(const tensor::operations::unary::Negate&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::Abs>{ static constexpr int ID = RLT_UNARY_ABS; static float parameter(const tensor::operations::unary::Abs&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::Constant<float>>{ static constexpr int ID = RLT_UNARY_CONSTANT; static float parameter(const tensor::operations::unary::Constant<float>& op){ return op.constant; } };
        template<> struct UnaryId<tensor::operations::unary::Sigmoid>{ static constexpr int ID = RLT_UNARY_SIGMOID; static float parameter(const tensor::operations::unary::Sigmoid&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::FastSigmoid>{ static constexpr int ID = RLT_UNARY_FAST_SIGMOID; static float parameter(const tensor::operations::unary::FastSigmoid&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::Exp>{ static constexpr int ID = RLT_UNARY_EXP; static float parameter(const tensor::operations::unary::Exp&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::Tanh>{ static constexpr int ID = RLT_UNARY_TANH; static float parameter(const tensor::operations::unary::Tanh&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::FastTanh>{ static constexpr int ID = RLT_UNARY_FAST_TANH; static float parameter(const tensor::operations::unary::FastTanh&){ return 0; } };
        template<> struct UnaryId<tensor::operations::unary::OneMinus>{ static constexpr int ID = RLT_UNARY_ONE_MINUS; static float parameter(const tensor::operations::unary::OneMinus&){ return 0; } };
        template<typename OPERATION> struct BinaryId{ static constexpr int ID = -1; };
        template<> struct BinaryId<tensor::operations::binary::Add>{ static constexpr int ID = RLT_BINARY_ADD; };
        template<> struct BinaryId<tensor::operations::binary::Subtract>{ static constexpr int ID = RLT_BINARY_SUBTRACT; };
        template<> struct BinaryId<tensor::operations::binary::Multiply>{ static constexpr int ID = RLT_BINARY_MULTIPLY; };
        template<> struct BinaryId<tensor::operations::binary::Divide>{ static constexpr int ID = RLT_BINARY_DIVIDE; };
        template<typename SPEC> constexpr bool dense_float(){ return utils::typing::is_same_v<utils::typing::remove_cv_t<typename SPEC::T>, float> && tensor::dense_row_major_layout<SPEC>(); }
    }
    template<typename DEV_SPEC, typename OPERATION, typename SPEC, typename SPEC_OUTPUT>
    void unary_operation(devices::ROCM<DEV_SPEC>& device, const OPERATION& operation, Tensor<SPEC>& t, Tensor<SPEC_OUTPUT>& output){
        static_assert(tensor::rocm::UnaryId<OPERATION>::ID >= 0 || utils::typing::is_same_v<OPERATION, tensor::operations::unary::Scale<float>>, "this functor has no counterpart in the ROCm library");
        static_assert(tensor::rocm::dense_float<SPEC>() && tensor::rocm::dense_float<SPEC_OUTPUT>() && SPEC::SIZE == SPEC_OUTPUT::SIZE, "elementwise operations work on dense float tensors of one size");
        if constexpr(utils::typing::is_same_v<OPERATION, tensor::operations::unary::Scale<float>>)
            devices::rocm::check(rlt_rocm_unary_f32(device.handle, operation.reciprocal ? RLT_UNARY_SCALE_RECIPROCAL : RLT_UNARY_SCALE, operation.scale, t._data, (int)SPEC::SIZE, output._data, (int)SPEC::SIZE, 1, (int)SPEC::SIZE), "unary_operation");
        else
            devices::rocm::check(rlt_rocm_unary_f32(device.handle, tensor::rocm::UnaryId<OPERATION>::ID, tensor::rocm::UnaryId<OPERATION>::parameter(operation), t._data, (int)SPEC::SIZE, output._data, (int)SPEC::SIZE, 1, (int)SPEC::SIZE), "unary_operation");
    }
    template<typename DEV_SPEC, typename OPERATION, typename SPEC>
    void unary_operation(devices::ROCM<DEV_SPEC>& device, const OPERATION& operation, Tensor<SPEC>& t){
        unary_operation(device, operation, t, t);
    }
    template<typename DEV_SPEC, typename SPEC_1, typename SPEC_2, typename SPEC_OUT, typename OPERATION>
    void binary_operation(devices::ROCM<DEV_SPEC>& device, const OPERATION& operation, Tensor<SPEC_1>& t1, Tensor<SPEC_2>& t2, Tensor<SPEC_OUT>& result){
        static_assert(tensor::rocm::BinaryId<OPERATION>::ID >= 0, "this functor has no counterpart in the ROCm library");
        static_assert(tensor::rocm::dense_float<SPEC_1>() && tensor::rocm::dense_float<SPEC_2>() && tensor::rocm::dense_float<SPEC_OUT>() && SPEC_1::SIZE == SPEC_2::SIZE && SPEC_1::SIZE == SPEC_OUT::SIZE);
        devices::rocm::check(rlt_rocm_binary_f32(device.handle, tensor::rocm::BinaryId<OPERATION>::ID, t1._data, (int)SPEC_1::SIZE, t2._data, (int)SPEC_1::SIZE, result._data, (int)SPEC_1::SIZE, 1, (int)SPEC_1::SIZE), "binary_operation");
    }
    // the two-tensor form writes into the second operand (operations_generic.h:596-610)
    template<typename DEV_SPEC, typename SPEC_1, typename SPEC_2, typename OPERATION>
    void binary_operation(devices::ROCM<DEV_SPEC>& device, const OPERATION operation, const Tensor<SPEC_1>& t1, Tensor<SPEC_2>& t2){
        static_assert(tensor::rocm::BinaryId<OPERATION>::ID >= 0, "this functor has no counterpart in the ROCm library");
        static_assert(tensor::rocm::dense_float<SPEC_1>() && tensor::rocm::dense_float<SPEC_2>() && SPEC_1::SIZE == SPEC_2::SIZE);
        devices::rocm::check(rlt_rocm_binary_f32(device.handle, tensor::rocm::BinaryId<OPERATION>::ID, t1._data, (int)SPEC_1::SIZE, t2._data, (int)SPEC_1::SIZE, t2._data, (int)SPEC_1::SIZE, 1, (int)SPEC_1::SIZE), "binary_operation");
    }
    // multiply_accumulate(t1, t2, t_output): t_output += t1 * t2   (operations_generic.h:475-481 and the ternary operation around it)
    template<typename DEV_SPEC, typename SPEC_1, typename SPEC_2, typename SPEC_OUT>
    void multiply_accumulate(devices::ROCM<DEV_SPEC>& device, const Tensor<SPEC_1>& t1, const Tensor<SPEC_2>& t2, Tensor<SPEC_OUT>& t_output){
        static_assert(tensor::rocm::dense_float<SPEC_1>() && tensor::rocm::dense_float<SPEC_2>() && tensor::rocm::dense_float<SPEC_OUT>() && SPEC_1::SIZE == SPEC_2::SIZE && SPEC_1::SIZE == SPEC_OUT::SIZE);
        devices::rocm::check(rlt_rocm_multiply_accumulate_f32(device.handle, t1._data, (int)SPEC_1::SIZE, t2._data, (int)SPEC_1::SIZE, t_output._data, (int)SPEC_1::SIZE, t_output._data, (int)SPEC_1::SIZE, 1, (int)SPEC_1::SIZE), "multiply_accumulate");
    }
    // abs_max   operations_generic.h:820-825 (the value is read back: the stream is waited for)
    template<typename DEV_SPEC, typename SPEC>
    typename SPEC::T abs_max(devices::ROCM<DEV_SPEC>& device, const Tensor<SPEC>& t){
        static_assert(tensor::rocm::dense_float<SPEC>());
        float* out = nullptr; float value = 0;
        devices::rocm::check(rlt_rocm_malloc(device.handle, (void**)&out, sizeof(float)), "abs_max");
        devices::rocm::check(rlt_rocm_reduce_abs_max_f32(device.handle, t._data, (size_t)SPEC::SIZE, out), "abs_max");
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, &value, out, sizeof(float)), "abs_max");
        devices::rocm::check(rlt_rocm_free(device.handle, out), "abs_max");
        return value;
    }
    // get                     containers/tensor/operations_generic.h: one element, copied to the host (waits for the stream): for the odd value that
    // host code logs, never for loops
    template<typename DEV_SPEC, typename SPEC>
    typename SPEC::T get(devices::ROCM<DEV_SPEC>& device, const Tensor<SPEC>& tensor, typename devices::ROCM<DEV_SPEC>::index_t local_index){
        static_assert(std::is_arithmetic_v<typename SPEC::T> && SPEC::SHAPE::LENGTH == 1);
        utils::typing::remove_cv_t<typename SPEC::T> value;
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, &value, tensor._data + index(device, tensor, local_index), sizeof(value)), "get(tensor)");
        return value;
    }
    template<typename DEV_SPEC, typename SPEC, typename... INDICES>
    typename SPEC::T get(devices::ROCM<DEV_SPEC>& device, const Tensor<SPEC>& tensor, typename devices::ROCM<DEV_SPEC>::index_t first_index, const INDICES... indices){
        static_assert(std::is_arithmetic_v<typename SPEC::T> && SPEC::SHAPE::LENGTH == sizeof...(INDICES) + 1);
        utils::typing::remove_cv_t<typename SPEC::T> value;
        devices::rocm::check(rlt_rocm_memcpy_d2h(device.handle, &value, tensor._data + index(device, tensor, first_index, indices...), sizeof(value)), "get(tensor)");
        return value;
    }
#ifdef RL_TOOLS_ROCM_FORBID_HOST_ELEMENT_ACCESS
    // A tensor of numbers on this device is device memory: a reference to one element, or writing one element from the host, is never
    // what a caller of this backend means (on hosts that map device memory it works, slowly, and hides a missing overload: a generic
    // host loop running over device memory). With this macro such an access does not compile. The integration programs are checked with it.
    template<typename DEV_SPEC, typename SPEC, typename... INDICES, typename = utils::typing::enable_if_t<std::is_arithmetic_v<typename SPEC::T>>>
    typename SPEC::T& get_ref(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& tensor, typename devices::ROCM<DEV_SPEC>::index_t index, const INDICES... indices) = delete;
    template<typename DEV_SPEC, typename SPEC, typename... INDICES, typename = utils::typing::enable_if_t<std::is_arithmetic_v<typename SPEC::T>>>
    const typename SPEC::T& get_ref(devices::ROCM<DEV_SPEC>& device, const Tensor<SPEC>& tensor, typename devices::ROCM<DEV_SPEC>::index_t index, const INDICES... indices) = delete;
    template<typename DEV_SPEC, typename SPEC, typename TII, typename... INDICES, typename = utils::typing::enable_if_t<std::is_arithmetic_v<typename SPEC::T>>>
    void set(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& tensor, typename SPEC::T value, const TII index, const INDICES... indices) = delete;
    template<typename DEV_SPEC, typename SPEC, typename TII, typename... INDICES, typename = utils::typing::enable_if_t<std::is_arithmetic_v<typename SPEC::T>>>
    void increment(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& tensor, typename SPEC::T value, const TII index, const INDICES... indices) = delete;
#endif
    // randn / rand            containers/tensor/operations_cuda.h:545-624
    template<typename DEV_SPEC, typename SPEC, typename RNG>
    void randn(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& t, RNG& rng){
        using TI = typename devices::ROCM<DEV_SPEC>::index_t;
        static_assert(utils::typing::is_same_v<typename SPEC::T, float>);
        if constexpr(tensor::dense_row_major_layout<SPEC>()){
            devices::rocm::check(rlt_rocm_randn_f32(device.handle, t._data, (size_t)SPEC::SIZE, rng.seed, random::next_stream(rng)), "randn(tensor)");
        }
        else{
            static_assert(SPEC::SHAPE::LENGTH > 1, "this view cannot be filled on devices::ROCM");
            for(TI i = 0; i < SPEC::SHAPE::FIRST; ++i){
                auto next = view(device, t, i);
                randn(device, next, rng);
            }
        }
    }
    template<typename DEV_SPEC, typename SPEC, typename RNG>
    void rand(devices::ROCM<DEV_SPEC>& device, Tensor<SPEC>& t, RNG& rng, typename SPEC::T min = 0, typename SPEC::T max = 1){
        using TI = typename devices::ROCM<DEV_SPEC>::index_t;
        static_assert(utils::typing::is_same_v<typename SPEC::T, float>);
        if constexpr(tensor::dense_row_major_layout<SPEC>()){
            devices::rocm::check(rlt_rocm_rand_f32(device.handle, t._data, (size_t)SPEC::SIZE, min, max, rng.seed, random::next_stream(rng)), "rand(tensor)");
        }
        else{
            static_assert(SPEC::SHAPE::LENGTH > 1, "this view cannot be filled on devices::ROCM");
            for(TI i = 0; i < SPEC::SHAPE::FIRST; ++i){
                auto next = view(device, t, i);
                rand(device, next, rng, min, max);
            }
        }
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
