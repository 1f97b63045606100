// devices::ROCM -- the device tag of the MI355X (gfx950) backend, next to devices::CPU and devices::CUDA of the reference
// (rl_tools/devices/cpu.h:17-66, rl_tools/devices/cuda.h:15-122).
//
// A backend of the reference is a tag type plus free-function overloads on it. The overloads for this tag live in the
// *_rocm.h headers beside this one; each forwards to one entry point of the C ABI in rlt_rocm.h (librlt_rocm.so), where the
// hand-written HIP kernels are. Host code compiled against this tag needs no HIP compiler: it is plain C++17.
//
// What differs from devices::CUDA:
//  * no BLAS handle and no per-thread generator states: the device object holds the C ABI's handle (one HIP device + one stream);
//  * math on the host side of the tag is the CPU's (devices::math::CPU): every function of this tag runs on the host and
//    only enqueues kernels, so a scalar sqrt / exp in generic code (initialiser bounds, logging) is a host computation;
//  * random numbers are counter based (random/operations_rocm.h): an engine is a (seed, counter) pair in host memory.
#pragma once
#include <rl_tools/rl_tools.h>
#include <rl_tools/utils/generic/typing.h>
#include <rl_tools/devices/devices.h>
#include <rl_tools/devices/cpu.h>
#include <rlt_rocm.h>

#include <cstdint>
#include <cstdlib>
#include <iostream>

RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    // Why the device type has a base class in namespace rl_tools. The reference's generic code calls operations unqualified with the device
    // as first argument (`update(device, layer.weights, optimizer)`), and a backend's overload is picked by overload resolution. An overload
    // declared AFTER the calling template is only found through argument-dependent lookup, which searches the namespaces of the argument
    // types -- for a device in rl_tools::devices, a parameter in rl_tools::nn::parameters and an optimiser in rl_tools::nn::optimizers that
    // does not include rl_tools, where every operation lives, and the generic host loop would silently run on device memory (the CUDA
    // backend avoids this by a fixed include order, src/rl/environments/pendulum/sac/cuda/sac.cu:6-27). A base class in rl_tools makes
    // rl_tools an associated namespace of the device, so the overloads of this backend are found wherever they are included.
    struct ROCMArgumentDependentLookupAnchor{};
}
RL_TOOLS_NAMESPACE_WRAPPER_END

RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools::devices{
    // devices.h:17-30 enumerates the known devices; until that enumeration has a ROCM entry the tag carries a value outside it
    // (the reference only compares DEVICE_ID for equality with the CPU ids, rl/algorithms/sac/operations_generic.h:252,401)
#ifndef RL_TOOLS_DEVICES_ROCM_DEVICE_ID
#define RL_TOOLS_DEVICES_ROCM_DEVICE_ID static_cast<::rl_tools::devices::DeviceId>(0x524F434D)
#endif
    namespace rocm{
        struct Base{
            static constexpr DeviceId DEVICE_ID = RL_TOOLS_DEVICES_ROCM_DEVICE_ID;
            using index_t = unsigned int;       // what index tensors hold on the device (episode_step, episode_start, cursors): 32 bits, as on CUDA
            static constexpr index_t MAX_INDEX = -1;
        };
    }
    namespace random{
        // counter-based engine (Philox4x32-10): key = seed, every draw consumes counter values; see random/operations_rocm.h
        struct ROCM: devices::random::Generic<devices::math::CPU>, rocm::Base{
            static constexpr Type TYPE = Type::random;
            template <typename T_NOTHING = void>
            struct ENGINE{
                uint64_t seed = 0;
                uint64_t counter = 0;      // the next unused stream number (device draws) / group index of stream 0 (host draws)
                uint64_t host_index = 0;
            };
        };
    }
    template <typename T_SPEC>
    struct ROCM: Device<T_SPEC>, rocm::Base, rl_tools::ROCMArgumentDependentLookupAnchor{
        template <typename OTHER_DEVICE>
        static constexpr bool compatible = OTHER_DEVICE::DEVICE_ID == rocm::Base::DEVICE_ID;
        using SPEC = T_SPEC;
        using EXECUTION_HINTS = devices::ExecutionHints;
        typename SPEC::MATH math;
        typename SPEC::RANDOM random;
        typename SPEC::LOGGING logger;          // a value, as in devices::CPU: the CPU's logging operations take it by reference
        rlt_rocm_device* handle = nullptr;      // rlt_rocm.h: one HIP device and the stream all work is enqueued on
        int hip_device_index = 0;
        bool initialized = false;
        index_t malloc_counter = 0;
        bool graph_capture_active = false;      // the stream records a graph (devices/cuda.h:59): check_status does not wait, nothing allocates; set by devices::rocm::begin_capture
        void* scratch = nullptr;                // grow-only device memory for the draws of gather_batch (devices::rocm::scratch)
        size_t scratch_bytes = 0;
        // Parity runs against another device: when set, TD3's train_critic / train_actor take the N(0, 1) draws of the td3_sampling layer (which the reference
        // samples inside the layer's forward pass, nn/layers/td3_sampling/operations_generic.h:75-128) from this device array [BATCH_SIZE x ACTION_DIM]
        // instead of drawing them, so that both devices can be given the draws one generator made. Null (the default): drawn on the device.
        const float* td3_sampling_noise_override = nullptr;
    };
    struct DefaultROCMSpecification{
        using MATH = devices::math::CPU;
        using MATH_DEVICE_ACCURATE = devices::math::CPU;
        using RANDOM = devices::random::ROCM;
        using LOGGING = devices::logging::CPU;
    };
    using DefaultROCM = ROCM<DefaultROCMSpecification>;
}
RL_TOOLS_NAMESPACE_WRAPPER_END

RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    namespace devices::rocm{
        // every C ABI call returns 0 or an error code; the reference's CUDA backend prints and carries on (devices/cuda.h:156-174),
        // here a failed call ends the program with the library's message
        inline void check(int code, const char* what){
            if(code != 0){
                std::cerr << "rl_tools ROCM backend: " << what << " failed: " << rlt_rocm_error_string(code) << std::endl;
                std::exit(100);
            }
        }
    }
    namespace devices::rocm{
        template <typename DEVICE>
        void* scratch(DEVICE& device, size_t bytes){
            if(bytes > device.scratch_bytes){
                if(device.graph_capture_active){ check(RLT_E_CAPTURING, "scratch (run the calls once before recording them, so that the buffer has its size)"); }
                if(device.scratch){ check(rlt_rocm_check_status(device.handle), "scratch"); check(rlt_rocm_free(device.handle, device.scratch), "scratch"); }
                const size_t want = bytes < 4096 ? 4096 : 2 * bytes;
                check(rlt_rocm_malloc(device.handle, &device.scratch, want), "scratch");
                device.scratch_bytes = want;
            }
            return device.scratch;
        }
    }
    // Recording a stretch of calls into a graph and replaying it (the reference's CUDA programs call cudaStreamBeginCapture / cudaGraphLaunch
    // themselves and set device.graph_capture_active around the recorded calls: src/rl/environments/pendulum/sac/cuda/sac.cu:122-164; programs
    // on this backend are plain C++ without the HIP runtime's headers, so the calls come from the library):
    //     devices::rocm::begin_capture(device);  step(device, ts);  auto* graph = devices::rocm::end_capture(device);
    //     while(...){ devices::rocm::replay(device, graph); }
    // Every operation between begin and end only records its launches. The recording ends with an advance of the device's stream offset by
    // REPLAY_STREAM_STRIDE, so every replay of any graph draws from Philox streams no other replay or unrecorded call uses (stream numbers
    // handed out by random::next_stream stay far below the stride).
    namespace devices::rocm{
        constexpr uint64_t REPLAY_STREAM_STRIDE = uint64_t(1) << 32;
        template <typename SPEC>
        void begin_capture(devices::ROCM<SPEC>& device){
            check(rlt_rocm_graph_begin_capture(device.handle), "begin_capture");
            device.graph_capture_active = true;
        }
        template <typename SPEC>
        rlt_rocm_graph* end_capture(devices::ROCM<SPEC>& device){
            rlt_rocm_graph* graph = nullptr;
            const int advance = rlt_rocm_advance_streams(device.handle, REPLAY_STREAM_STRIDE);
            const int end = rlt_rocm_graph_end_capture(device.handle, &graph);
            device.graph_capture_active = false;
            check(advance, "end_capture (stream advance)");
            check(end, "end_capture");
            return graph;
        }
        template <typename SPEC>
        void replay(devices::ROCM<SPEC>& device, rlt_rocm_graph* graph){ check(rlt_rocm_graph_launch(device.handle, graph), "replay"); }
        template <typename SPEC>
        void free_graph(devices::ROCM<SPEC>& device, rlt_rocm_graph* graph){ check(rlt_rocm_graph_destroy(device.handle, graph), "free_graph"); }
    }
    // init(device)            devices/cuda.h:130-154
    template <typename SPEC>
    void init(devices::ROCM<SPEC>& device){
        if(device.initialized){
            std::cerr << "ROCM device already initialized" << std::endl;
            return;
        }
        devices::rocm::check(rlt_rocm_init(device.hip_device_index, &device.handle), "rlt_rocm_init");
        device.initialized = true;
    }
    template <typename SPEC>
    void free(devices::ROCM<SPEC>& device){
        if(device.initialized){
            if(device.scratch){ rlt_rocm_free(device.handle, device.scratch); device.scratch = nullptr; device.scratch_bytes = 0; }
            rlt_rocm_destroy(device.handle);
            device.handle = nullptr;
            device.initialized = false;
        }
    }
    // check_status(device)    devices/cuda.h:156-174: waits for the stream and reports what went wrong since the last check
    template <typename SPEC>
    void check_status(devices::ROCM<SPEC>& device){
        if(device.graph_capture_active){ return; }      // devices/cuda.h:163
        devices::rocm::check(device.handle ? rlt_rocm_check_status(device.handle) : RLT_E_NOT_INITIALISED, "check_status");
    }
    template <typename DEV_SPEC, typename TI>
    void count_malloc(devices::ROCM<DEV_SPEC>& device, TI size){
        device.malloc_counter += size;
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
