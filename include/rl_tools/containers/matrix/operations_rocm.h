// Matrix containers on devices::ROCM: malloc / free / copy / set_all / randn (the counterpart of
// containers/matrix/operations_cuda.h:16-222). A matrix is device memory; host code never dereferences `_data`.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/containers/matrix/matrix.h>
#include <rl_tools/random/operations_rocm.h>
#include <new>
#include <type_traits>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    // malloc / free           containers/matrix/operations_cuda.h:16-45
    // Matrices of numbers and flags are device memory. Matrices of structs (environments, their parameters) are read and written by
    // host code only -- the precompiled kernels know no struct layouts -- and are host memory; a component whose kernels do keep a struct
    // array on the device (the runners' environment states) allocates it itself.
    template<typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE_BYTES, bool T_CONST>
    void malloc(devices::ROCM<DEV_SPEC>& device, matrix::MatrixDynamic<T, T_TI, SIZE_BYTES, T_CONST>& matrix){
        if constexpr(std::is_arithmetic_v<T>){
            void* memory = nullptr;
            devices::rocm::check(rlt_rocm_malloc(device.handle, &memory, SIZE_BYTES > 0 ? SIZE_BYTES : 1), "malloc(matrix)");
            matrix._data = (T*)memory;
        }
        else{
            matrix._data = (T*)::operator new(SIZE_BYTES > 0 ? SIZE_BYTES : 1, std::align_val_t(64));
        }
        count_malloc(device, SIZE_BYTES);
    }
    template<typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE_BYTES, bool T_CONST>
    void free(devices::ROCM<DEV_SPEC>& device, matrix::MatrixDynamic<T, T_TI, SIZE_BYTES, T_CONST>& matrix){
        if constexpr(std::is_arithmetic_v<T>){
            devices::rocm::check(rlt_rocm_free(device.handle, (void*)matrix._data), "free(matrix)");
        }
        else{
            ::operator delete((void*)matrix._data, std::align_val_t(64));
        }
        matrix._data = nullptr;
    }
    template<typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE>
    void malloc(devices::ROCM<DEV_SPEC>& device, matrix::MatrixStatic<T, T_TI, SIZE>& matrix){}      // a statically allocated matrix lives where its owner lives
    template<typename DEV_SPEC, typename T, typename T_TI, T_TI SIZE>
    void free(devices::ROCM<DEV_SPEC>& device, matrix::MatrixStatic<T, T_TI, SIZE>& matrix){}

    namespace containers::rocm{
        // What the C ABI takes as the leading dimension of a matrix (elements between the starts of consecutive rows). A one-row view of a
        // one-dimensional tensor carries a row pitch of 1 (containers/tensor/operations_generic.h:1046-1056): its leading dimension is its width.
        template <typename SPEC>
        constexpr auto leading_dimension = (SPEC::ROWS == 1 && SPEC::ROW_PITCH < SPEC::COLS) ? SPEC::COLS : SPEC::ROW_PITCH;
        // all elements side by side in memory, row after row
        template <typename SPEC>
        constexpr bool dense = SPEC::COL_PITCH == 1 && (SPEC::ROWS == 1 || SPEC::ROW_PITCH == SPEC::COLS);
        // both matrices are rows of COLS contiguous elements of the same type: one strided copy moves them (kind as in rlt_rocm_memcpy2d)
        template <typename SOURCE_SPEC, typename TARGET_SPEC>
        constexpr bool strided_copy_possible = containers::check_structure<SOURCE_SPEC, TARGET_SPEC> && SOURCE_SPEC::COL_PITCH == 1 && TARGET_SPEC::COL_PITCH == 1
                                               && utils::typing::is_same_v<utils::typing::remove_cv_t<typename SOURCE_SPEC::T>, utils::typing::remove_cv_t<typename TARGET_SPEC::T>>;
        template <typename DEVICE, typename SOURCE_SPEC, typename TARGET_SPEC>
        void strided_copy(DEVICE& device, const Matrix<SOURCE_SPEC>& source, Matrix<TARGET_SPEC>& target, int kind){
            using T = typename TARGET_SPEC::T;
            if constexpr(!std::is_arithmetic_v<utils::typing::remove_cv_t<T>>){
                // matrices of structs are host memory on every device (malloc above): copied element by element on the host, whatever the direction
                for(size_t row = 0; row < (size_t)TARGET_SPEC::ROWS; row++){
                    for(size_t col = 0; col < (size_t)TARGET_SPEC::COLS; col++){ target._data[row * leading_dimension<TARGET_SPEC> + col] = source._data[row * leading_dimension<SOURCE_SPEC> + col]; }
                }
            }
            else if constexpr(dense<SOURCE_SPEC> && dense<TARGET_SPEC>){
                const size_t bytes = (size_t)TARGET_SPEC::ROWS * TARGET_SPEC::COLS * sizeof(T);
                const int rc = kind == 0 ? rlt_rocm_memcpy_d2d(device.handle, (void*)target._data, (const void*)source._data, bytes)
                             : kind == 1 ? rlt_rocm_memcpy_h2d(device.handle, (void*)target._data, (const void*)source._data, bytes)
                                         : rlt_rocm_memcpy_d2h(device.handle, (void*)target._data, (const void*)source._data, bytes);
                devices::rocm::check(rc, "copy(matrix)");
            }
            else{
                devices::rocm::check(rlt_rocm_memcpy2d(device.handle, (void*)target._data, (size_t)leading_dimension<TARGET_SPEC> * sizeof(T), (const void*)source._data, (size_t)leading_dimension<SOURCE_SPEC> * sizeof(T),
                                                       (size_t)TARGET_SPEC::COLS * sizeof(T), (size_t)TARGET_SPEC::ROWS, kind), "copy(matrix view)");
            }
        }
    }
    // copy ROCM -> ROCM       containers/matrix/operations_cuda.h:90-115
    template<typename SOURCE_DEV_SPEC, typename TARGET_DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC>
    void copy(devices::ROCM<SOURCE_DEV_SPEC>& source_device, devices::ROCM<TARGET_DEV_SPEC>& target_device, const Matrix<SOURCE_SPEC>& source, Matrix<TARGET_SPEC>& target){
        static_assert(containers::rocm::strided_copy_possible<SOURCE_SPEC, TARGET_SPEC>, "device-to-device copies need the same element type and unit column pitch on both sides");
        containers::rocm::strided_copy(source_device, source, target, 0);
    }
    // copy CPU -> ROCM        containers/matrix/operations_cuda.h:117-161 (synchronises, as there)
    template<typename SOURCE_DEV_SPEC, typename TARGET_DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC>
    void copy(devices::CPU<SOURCE_DEV_SPEC>& source_device, devices::ROCM<TARGET_DEV_SPEC>& target_device, const Matrix<SOURCE_SPEC>& source, Matrix<TARGET_SPEC>& target){
        static_assert(containers::check_structure<TARGET_SPEC, SOURCE_SPEC>);
        if constexpr(containers::rocm::strided_copy_possible<SOURCE_SPEC, TARGET_SPEC>){
            containers::rocm::strided_copy(target_device, source, target, 1);
        }
        else{   // another element type or a column-major side: convert on the host into a dense copy with the target's element type first
            Matrix<matrix::Specification<typename TARGET_SPEC::T, typename TARGET_SPEC::TI, TARGET_SPEC::ROWS, TARGET_SPEC::COLS, true>> staged;
            malloc(source_device, staged);
            copy(source_device, source_device, source, staged);
            containers::rocm::strided_copy(target_device, staged, target, 1);
            free(source_device, staged);
        }
    }
    // copy ROCM -> CPU        containers/matrix/operations_cuda.h:163-195
    template<typename SOURCE_DEV_SPEC, typename TARGET_DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC>
    void copy(devices::ROCM<SOURCE_DEV_SPEC>& source_device, devices::CPU<TARGET_DEV_SPEC>& target_device, const Matrix<SOURCE_SPEC>& source, Matrix<TARGET_SPEC>& target){
        static_assert(containers::check_structure<TARGET_SPEC, SOURCE_SPEC>);
        if constexpr(containers::rocm::strided_copy_possible<SOURCE_SPEC, TARGET_SPEC>){
            containers::rocm::strided_copy(source_device, source, target, 2);
        }
        else{
            static_assert(SOURCE_SPEC::COL_PITCH == 1, "column-major device matrices cannot be copied to the host directly");
            Matrix<matrix::Specification<utils::typing::remove_cv_t<typename SOURCE_SPEC::T>, typename TARGET_SPEC::TI, TARGET_SPEC::ROWS, TARGET_SPEC::COLS, true>> staged;
            malloc(target_device, staged);
            containers::rocm::strided_copy(source_device, source, staged, 2);
            copy(target_device, target_device, staged, target);
            free(target_device, staged);
        }
    }
    // set_all                 containers/matrix/operations_cuda.h:197-207
    template<typename DEV_SPEC, typename SPEC, typename VALUE_T>
    void set_all(devices::ROCM<DEV_SPEC>& device, Matrix<SPEC>& m, VALUE_T value){
        using T = typename SPEC::T;
        static_assert(SPEC::COL_PITCH == 1);
        if constexpr(utils::typing::is_same_v<T, float>){
            devices::rocm::check(rlt_rocm_fill_f32(device.handle, m._data, SPEC::ROWS, SPEC::COLS, containers::rocm::leading_dimension<SPEC>, (float)value), "set_all(matrix)");
        }
        else if constexpr(sizeof(T) == 1){
            for(typename SPEC::TI row = 0; row < (containers::rocm::dense<SPEC> ? 1 : SPEC::ROWS); row++){
                const size_t count = containers::rocm::dense<SPEC> ? (size_t)SPEC::ROWS * SPEC::COLS : (size_t)SPEC::COLS;
                devices::rocm::check(rlt_rocm_fill_u8(device.handle, (uint8_t*)m._data + (size_t)row * SPEC::ROW_PITCH, count, (uint8_t)(T)value), "set_all(matrix)");
            }
        }
        else{   // other element types (index matrices) are small and set rarely: stage the values on the host
            T* host = new T[(size_t)SPEC::ROWS * SPEC::COLS];
            for(size_t i = 0; i < (size_t)SPEC::ROWS * SPEC::COLS; i++){ host[i] = (T)value; }
            devices::rocm::check(rlt_rocm_memcpy2d(device.handle, (void*)m._data, (size_t)containers::rocm::leading_dimension<SPEC> * sizeof(T), host, (size_t)SPEC::COLS * sizeof(T), (size_t)SPEC::COLS * sizeof(T), SPEC::ROWS, 1), "set_all(matrix)");
            delete[] host;
        }
    }
    // randn                   containers/matrix/operations_cuda.h:208-222
    template<typename DEV_SPEC, typename SPEC, typename RNG>
    void randn(devices::ROCM<DEV_SPEC>& device, Matrix<SPEC>& m, typename SPEC::T mean, typename SPEC::T std, RNG& rng){
        static_assert(utils::typing::is_same_v<typename SPEC::T, float> && containers::rocm::dense<SPEC>, "randn fills dense float matrices");
        utils::assert_exit(device, mean == 0 && std == 1, "randn on devices::ROCM draws N(0, 1)");
        devices::rocm::check(rlt_rocm_randn_f32(device.handle, m._data, (size_t)SPEC::ROWS * SPEC::COLS, rng.seed, random::next_stream(rng)), "randn(matrix)");
    }
    template<typename DEV_SPEC, typename SPEC, typename RNG>
    void randn(devices::ROCM<DEV_SPEC>& device, Matrix<SPEC>& m, RNG& rng){
        randn(device, m, 0, 1, rng);
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
