// Adam on devices::ROCM (the counterpart of nn/optimizers/adam/operations_cuda.h:13-68 and instance/operations_cuda.h:10-70).
//
// The CUDA backend runs a <<<1,1>>> kernel for the bias corrections and then one kernel per parameter tensor. Here step() walks the
// model once on the host to collect its parameter tensors and hands the list to ONE launch (rlt_rocm_adam_step) that derives the bias
// corrections from the device-resident age, updates moments and parameters of every tensor and increments the age.
//
// Where the optimiser's members live: `age` on the device (the kernel reads and increments it); `parameters` (the hyper-parameter
// struct) and the two bias-correction scalars in HOST memory: host code sets and reads them (init, learning-rate schedules) and their
// values travel with each launch, so none of them needs a kernel of its own.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/nn/optimizers/adam/adam.h>
#include <rl_tools/nn/optimizers/adam/instance/operations_generic.h>
#include <rl_tools/nn/optimizers/adam/operations_generic.h>
#include <vector>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace nn::optimizers::adam::rocm{
        // The model walkers of the reference (nn_models/mlp/operations_generic.h:210-217, sequential :429-435, the layers' update) hand
        // an nn::optimizers::Adam<...> down to every parameter tensor. An Adam of this specification is the probe step() sends down that
        // path: the per-tensor overload below recognises it and records the tensor instead of updating it.
        template <typename T_SPEC>
        struct CollectSpecification{
            using T = typename T_SPEC::T;
            using TI = typename T_SPEC::TI;
            using DEFAULT_PARAMETERS = typename T_SPEC::DEFAULT_PARAMETERS;
            static constexpr bool ENABLE_WEIGHT_DECAY = T_SPEC::ENABLE_WEIGHT_DECAY;
            static constexpr bool ENABLE_BIAS_LR_FACTOR = T_SPEC::ENABLE_BIAS_LR_FACTOR;
            static constexpr bool DYNAMIC_ALLOCATION = false;
            static constexpr bool ROCM_COLLECT = true;
        };
        inline std::vector<rlt_adam_tensor>*& sink(){ static thread_local std::vector<rlt_adam_tensor>* list = nullptr; return list; }
        template <typename SPEC, typename = void> struct is_collector{ static constexpr bool value = false; };
        template <typename SPEC> struct is_collector<SPEC, utils::typing::enable_if_t<SPEC::ROCM_COLLECT>>{ static constexpr bool value = true; };
        template <typename DEVICE, typename SPEC, typename MODEL>
        std::vector<rlt_adam_tensor> collect(DEVICE& device, MODEL& model, bool for_reset){
            std::vector<rlt_adam_tensor> tensors;
            nn::optimizers::Adam<CollectSpecification<SPEC>> probe;
            sink() = &tensors;
            if(for_reset){ _reset_optimizer_state(device, model, probe); } else { update(device, model, probe); }
            sink() = nullptr;
            return tensors;
        }
        template <typename PARAMETER_SPEC>
        rlt_adam_tensor describe(nn::parameters::Adam::Instance<PARAMETER_SPEC>& p){
            using TENSOR = decltype(p.parameters);
            static_assert(utils::typing::is_same_v<typename TENSOR::T, float> && tensor::dense_row_major_layout<typename TENSOR::SPEC>(), "the ROCM backend updates dense fp32 tensors");
            rlt_adam_tensor t = {};
            t.parameters = p.parameters._data; t.gradient = p.gradient._data;
            t.first_moment = p.gradient_first_order_moment._data; t.second_moment = p.gradient_second_order_moment._data;
            t.polyak_target = nullptr;
            t.count = (uint32_t)TENSOR::SPEC::SIZE;
            t.flags = utils::typing::is_same_v<typename PARAMETER_SPEC::CATEGORY_TAG, nn::parameters::categories::Weights> ? 1u : (utils::typing::is_same_v<typename PARAMETER_SPEC::CATEGORY_TAG, nn::parameters::categories::Biases> ? 2u : 0u);
            return t;
        }
    }
    // malloc / free           nn/optimizers/adam/operations_generic.h:12-26
    template <typename DEV_SPEC, typename SPEC>
    void malloc(devices::ROCM<DEV_SPEC>& device, nn::optimizers::Adam<SPEC>& optimizer){
        static_assert(sizeof(typename SPEC::TI) == 4, "the optimiser's age is a 32-bit counter on the device");
        static_assert(SPEC::DYNAMIC_ALLOCATION, "optimisers on devices::ROCM are dynamically allocated");
        malloc(device, optimizer.age);
        optimizer.parameters._data = new typename nn::optimizers::Adam<SPEC>::PARAMETERS[1];
        optimizer.first_order_moment_bias_correction._data = new typename SPEC::T[1];
        optimizer.second_order_moment_bias_correction._data = new typename SPEC::T[1];
    }
    template <typename DEV_SPEC, typename SPEC>
    void free(devices::ROCM<DEV_SPEC>& device, nn::optimizers::Adam<SPEC>& optimizer){
        free(device, optimizer.age);
        delete[] optimizer.parameters._data; optimizer.parameters._data = nullptr;
        delete[] optimizer.first_order_moment_bias_correction._data; optimizer.first_order_moment_bias_correction._data = nullptr;
        delete[] optimizer.second_order_moment_bias_correction._data; optimizer.second_order_moment_bias_correction._data = nullptr;
    }
    // init                    nn/optimizers/adam/operations_cuda.h:13-40: the hyper-parameters of the specification (host memory, see above)
    template <typename DEV_SPEC, typename SPEC>
    void init(devices::ROCM<DEV_SPEC>& device, nn::optimizers::Adam<SPEC>& optimizer){
        using DEFAULTS = typename SPEC::DEFAULT_PARAMETERS;
        optimizer.parameters._data[0] = typename nn::optimizers::Adam<SPEC>::PARAMETERS{DEFAULTS::ALPHA, DEFAULTS::BETA_1, DEFAULTS::BETA_2, DEFAULTS::EPSILON, DEFAULTS::EPSILON_SQRT,
                                                                                        DEFAULTS::WEIGHT_DECAY, DEFAULTS::WEIGHT_DECAY_INPUT, DEFAULTS::WEIGHT_DECAY_OUTPUT, DEFAULTS::BIAS_LR_FACTOR};
    }
    // the per-tensor update   instance/operations_cuda.h:58-70. Reached through a model walk started by step() / reset_optimizer_state()
    template<typename DEV_SPEC, typename SPEC, typename ADAM_SPEC>
    void update(devices::ROCM<DEV_SPEC>& device, nn::parameters::Adam::Instance<SPEC>& parameter, nn::optimizers::Adam<ADAM_SPEC>& optimizer){
        if constexpr(nn::optimizers::adam::rocm::is_collector<ADAM_SPEC>::value){
            if constexpr(ADAM_SPEC::ENABLE_WEIGHT_DECAY){
                static_assert(utils::typing::is_same_v<typename SPEC::GROUP_TAG, nn::parameters::groups::Normal> || !utils::typing::is_same_v<typename SPEC::CATEGORY_TAG, nn::parameters::categories::Weights>,
                              "weight decay per parameter group (input / output layers) is not available on devices::ROCM");
            }
            nn::optimizers::adam::rocm::sink()->push_back(nn::optimizers::adam::rocm::describe(parameter));
        }
        else{
            utils::assert_exit(device, false, "devices::ROCM updates all tensors of a model in one launch: call step(device, optimizer, model)");
        }
    }
    template<typename DEV_SPEC, typename SPEC, typename PARAMETER_SPEC>
    void _reset_optimizer_state(devices::ROCM<DEV_SPEC>& device, nn::parameters::Adam::Instance<PARAMETER_SPEC>& parameter, nn::optimizers::Adam<SPEC>& optimizer){
        if constexpr(nn::optimizers::adam::rocm::is_collector<SPEC>::value){
            nn::optimizers::adam::rocm::sink()->push_back(nn::optimizers::adam::rocm::describe(parameter));
        }
        else{
            set_all(device, parameter.gradient_first_order_moment, 0);
            set_all(device, parameter.gradient_second_order_moment, 0);
        }
    }
    // reset_optimizer_state   nn/optimizers/adam/operations_cuda.h:41-48: age <- 1, moments <- 0, one launch
    template<typename DEV_SPEC, typename SPEC, typename MODEL>
    void reset_optimizer_state(devices::ROCM<DEV_SPEC>& device, nn::optimizers::Adam<SPEC>& optimizer, MODEL& model){
        auto tensors = nn::optimizers::adam::rocm::collect<devices::ROCM<DEV_SPEC>, SPEC>(device, model, true);
        if(tensors.empty()){
            set_all(device, optimizer.age, 1);
        }
        else{
            devices::rocm::check(rlt_rocm_adam_reset(device.handle, tensors.data(), (int)tensors.size(), (uint32_t*)optimizer.age._data), "reset_optimizer_state");
        }
    }
    // step                    nn/optimizers/adam/operations_cuda.h:57-65, operations_generic.h:49-66
    template<typename DEV_SPEC, typename SPEC, typename MODEL>
    void step(devices::ROCM<DEV_SPEC>& device, nn::optimizers::Adam<SPEC>& optimizer, MODEL& model){
        using DEFAULTS = typename SPEC::DEFAULT_PARAMETERS;
        auto tensors = nn::optimizers::adam::rocm::collect<devices::ROCM<DEV_SPEC>, SPEC>(device, model, false);
        if(tensors.empty()){ return; }
        const auto& hp = optimizer.parameters._data[0];
        rlt_adam_parameters p = {};
        p.alpha = hp.alpha; p.beta_1 = hp.beta_1; p.beta_2 = hp.beta_2; p.epsilon = hp.epsilon; p.epsilon_sqrt = hp.epsilon_sqrt;
        p.weight_decay = hp.weight_decay; p.bias_lr_factor = hp.bias_lr_factor;
        p.enable_weight_decay = SPEC::ENABLE_WEIGHT_DECAY; p.enable_bias_lr_factor = SPEC::ENABLE_BIAS_LR_FACTOR;
        p.enable_gradient_clipping = DEFAULTS::ENABLE_GRADIENT_CLIPPING; p.gradient_clip_value = DEFAULTS::GRADIENT_CLIP_VALUE;
        devices::rocm::check(rlt_rocm_adam_step(device.handle, tensors.data(), (int)tensors.size(), &p, (uint32_t*)optimizer.age._data, 0.0f, nullptr), "step(adam)");
    }
    // copies of the optimiser between devices: age on the device, hyper-parameters on the host (operations_generic.h:67-71 copies both). X -> ROCM resolves to the
    // reference's generic copy, whose two tensor copies land on the overloads of containers/tensor/operations_rocm.h (the hyper-parameters, a tensor of structs, stay on the host)
    template<typename SOURCE_DEV_SPEC, typename TARGET_DEVICE, typename SOURCE_SPEC, typename TARGET_SPEC>
    void copy(devices::ROCM<SOURCE_DEV_SPEC>& source_device, TARGET_DEVICE& target_device, const nn::optimizers::Adam<SOURCE_SPEC>& source, nn::optimizers::Adam<TARGET_SPEC>& target){
        copy(source_device, target_device, source.age, target.age);
        const auto& hp = source.parameters._data[0];
        typename nn::optimizers::Adam<TARGET_SPEC>::PARAMETERS converted = {(typename TARGET_SPEC::T)hp.alpha, (typename TARGET_SPEC::T)hp.beta_1, (typename TARGET_SPEC::T)hp.beta_2, (typename TARGET_SPEC::T)hp.epsilon,
            (typename TARGET_SPEC::T)hp.epsilon_sqrt, (typename TARGET_SPEC::T)hp.weight_decay, (typename TARGET_SPEC::T)hp.weight_decay_input, (typename TARGET_SPEC::T)hp.weight_decay_output, (typename TARGET_SPEC::T)hp.bias_lr_factor};
        set(target_device, target.parameters, converted, 0);
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
