// Device handle, memory and the small container operations of the C ABI
// (reference: devices/cuda.h:130-174, containers/matrix/operations_cuda.h:16-218, containers/tensor/operations_cuda.h:15-624).
#include "common.h"
#include "rng.h"
#include <cstdlib>
#include "gemm.h"
#include <cstdio>
#include <cstring>

int rlt_launch_status(rlt_rocm_device* device) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { device->sticky_error = (int)e; return (int)e; }
    return 0;
}

bool rlt_side_begin(rlt_rocm_device* device, int which) {
    if (which < 0 || which >= RLT_SIDE_STREAMS || !device->side_stream[which] || device->capturing || device->side_return) return false;
    if (hipEventRecord(device->fork_event[which], device->stream) != hipSuccess || hipStreamWaitEvent(device->side_stream[which], device->fork_event[which], 0) != hipSuccess) { (void)hipGetLastError(); return false; }
    device->side_return = device->stream;
    device->side_active = which;
    device->side_pending[which] = 1;
    device->stream = device->side_stream[which];
    return true;
}
void rlt_side_end(rlt_rocm_device* device) {
    if (device->side_return) { device->stream = device->side_return; device->side_return = nullptr; }
}
int rlt_side_join(rlt_rocm_device* device) {
    for (int k = 0; k < RLT_SIDE_STREAMS; k++) {
        if (!device->side_stream[k] || !device->side_pending[k]) continue;
        RLT_HIP(hipEventRecord(device->join_event[k], device->side_stream[k]));
        RLT_HIP(hipStreamWaitEvent(device->stream, device->join_event[k], 0));
        device->side_pending[k] = 0;
    }
    return 0;
}
int rlt_scratch(rlt_rocm_device* device, size_t bytes, void** out) {
    void*& buffer = device->side_return ? device->side_scratch[device->side_active] : device->scratch;       // work that goes to a side stream has a scratch buffer of its own
    size_t& have = device->side_return ? device->side_scratch_bytes[device->side_active] : device->scratch_bytes;
    if (bytes > have) {
        if (device->capturing) return RLT_E_CAPTURING;      // the workspace grows on a warm-up call before the capture
        if (buffer) RLT_HIP(hipFree(buffer));   // hipFree waits for the work that still uses it
        buffer = nullptr; have = 0;
        size_t want = bytes < (size_t)(1u << 20) ? (size_t)(1u << 20) : bytes + bytes / 4;
        RLT_HIP(hipMalloc(&buffer, want));
        have = want;
    }
    *out = buffer;
    return 0;
}

int rlt_counters(rlt_rocm_device* device, void** out) {
    *out = device->counters;
    return device->counters ? 0 : RLT_E_NOT_INITIALISED;
}

namespace {

__global__ __launch_bounds__(256) void fill_f32_kernel(float* __restrict__ dst, int rows, int cols, int ld, float value) {
    const size_t total = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i / cols, c = i % cols;
        dst[r * ld + c] = value;
    }
}
__global__ __launch_bounds__(256) void fill_from_f32_kernel(float* __restrict__ dst, int rows, int cols, int ld, const float* __restrict__ value) {
    const size_t total = (size_t)rows * cols;
    const float v = *value;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i / cols, c = i % cols;
        dst[r * ld + c] = v;
    }
}
__global__ __launch_bounds__(256) void fill_u8_kernel(uint8_t* __restrict__ dst, size_t count, uint8_t value) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) dst[i] = value;
}
__global__ __launch_bounds__(256) void scale_kernel(float* __restrict__ x, size_t count, float s, int reciprocal) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        x[i] = reciprocal ? (1.0f / x[i]) * s : x[i] * s;   // the reciprocal first, then the scale, as the reference's Scale operation rounds
}

// randn / rand: element i is word i % 4 of Philox group i / 4 of the call's stream (rng.h). Two calls with different `stream` values
// (or different seeds) share no group, whatever their lengths.
__global__ __launch_bounds__(256) void rand_kernel(float* __restrict__ dst, size_t count, float low, float high, uint64_t seed, uint64_t stream, int normal, const uint64_t* __restrict__ stream_offset) {
    const size_t quads = (count + 3) / 4;
    stream += *stream_offset;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (size_t)gridDim.x * blockDim.x) {
        const rlt_u32x4 r = rlt_philox(seed, stream, q);
        float v[4];
        if (normal) {   // Box-Muller, two normals per pair of uniforms
            float r0 = sqrtf(-2.0f * logf(rlt_u01(r.x))), r1 = sqrtf(-2.0f * logf(rlt_u01(r.z)));
            float s0, c0, s1, c1;
            sincosf(6.283185307179586f * rlt_u01(r.y), &s0, &c0);
            sincosf(6.283185307179586f * rlt_u01(r.w), &s1, &c1);
            v[0] = r0 * c0; v[1] = r0 * s0; v[2] = r1 * c1; v[3] = r1 * s1;
        } else {
            v[0] = low + (high - low) * rlt_u01(r.x); v[1] = low + (high - low) * rlt_u01(r.y);
            v[2] = low + (high - low) * rlt_u01(r.z); v[3] = low + (high - low) * rlt_u01(r.w);
        }
        for (int j = 0; j < 4; j++) if (q * 4 + j < count) dst[q * 4 + j] = v[j];
    }
}
// the raw 32-bit words of a stream, for checking the generator against a host restatement
__global__ __launch_bounds__(256) void rand_bits_kernel(uint32_t* __restrict__ dst, size_t count, uint64_t seed, uint64_t stream, const uint64_t* __restrict__ stream_offset) {
    const size_t quads = (count + 3) / 4;
    stream += *stream_offset;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (size_t)gridDim.x * blockDim.x) {
        const rlt_u32x4 r = rlt_philox(seed, stream, q);
        const uint32_t v[4] = {r.x, r.y, r.z, r.w};
        for (int j = 0; j < 4; j++) if (q * 4 + j < count) dst[q * 4 + j] = v[j];
    }
}

// single-workgroup reductions: 1024 lanes, wavefront butterflies then one pass over the 16 partials
template <int KIND>   // 0: uint8 != 0 count, 1: sum, 2: sum of squares
__global__ __launch_bounds__(1024) void reduce_kernel(const void* __restrict__ src, size_t count, float* __restrict__ out) {
    __shared__ float partial[16];
    float acc = 0.0f;
    for (size_t i = threadIdx.x; i < count; i += blockDim.x) {
        if (KIND == 0) acc += (float)(((const uint8_t*)src)[i] != 0);
        else { float v = ((const float*)src)[i]; acc += KIND == 1 ? v : v * v; }
    }
    acc = rlt_wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) { float s = 0.0f; for (int i = 0; i < 16; i++) s += partial[i]; *out = s; }
}

// which XCD every workgroup of a launch lands on (bits 3:0 of the XCC_ID hardware register)
__global__ __launch_bounds__(64) void xcd_probe_kernel(unsigned* __restrict__ out) {
    if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xf;
}

int grid_for(size_t n) { size_t b = (n + 255) / 256; return (int)(b > 8192 ? 8192 : (b < 1 ? 1 : b)); }

}  // namespace

extern "C" {

int rlt_rocm_init(int hip_device_index, rlt_rocm_device** out_device) {
    if (!out_device) return RLT_E_INVALID_ARGUMENT;
    rlt_rocm_device* device = nullptr;
    hipError_t e = hipSetDevice(hip_device_index);
    if (e != hipSuccess) return (int)e;
    device = new rlt_rocm_device();
    std::memset(device, 0, sizeof *device);
    device->hip_device = hip_device_index;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, hip_device_index);
    if (e != hipSuccess) { delete device; return (int)e; }
    device->compute_units = prop.multiProcessorCount;
    device->lds_bytes = (int)prop.sharedMemPerBlock;
    std::snprintf(device->name, sizeof device->name, "%s (%s)", prop.name, prop.gcnArchName);
    e = hipStreamCreate(&device->own_stream);   // default priority
    if (e != hipSuccess) { delete device; return (int)e; }
    device->stream = device->own_stream;
    e = hipMalloc(&device->counters, 8192);
    if (e == hipSuccess) e = hipMemset(device->counters, 0, 8192);
    if (e != hipSuccess) { (void)hipStreamDestroy(device->own_stream); delete device; return (int)e; }
    device->fault = (unsigned*)((char*)device->counters + 8192 - 64);   // the last 64 bytes of the block are never used as counters
    device->stream_offset = (uint64_t*)((char*)device->counters + 8192 - 128);      // zero: stream numbers mean what the caller passes
    // Dispatch order over the XCDs: probe twice with 64 workgroups; if workgroup b always shares its XCD with b + 8 (and with no
    // workgroup in between), persistent kernels may place a small grid on one XCD by using every 8th workgroup of a larger one.
    {
        unsigned* probe = (unsigned*)((char*)device->counters + 4096);
        unsigned host[64];
        bool ok = true;
        for (int rep = 0; rep < 2 && ok; rep++) {
            hipLaunchKernelGGL(xcd_probe_kernel, dim3(64), dim3(64), 0, device->stream, probe);
            ok = hipMemcpyAsync(host, probe, sizeof host, hipMemcpyDeviceToHost, device->stream) == hipSuccess && hipStreamSynchronize(device->stream) == hipSuccess;
            for (int b = 0; b < 64 && ok; b++) {
                if (b >= 8 && host[b] != host[b - 8]) ok = false;
                for (int k = 1; k < 8 && b >= k && ok; k++) if (host[b] == host[b - k]) ok = false;
            }
        }
        (void)hipMemsetAsync(probe, 0, sizeof host, device->stream);
        (void)hipStreamSynchronize(device->stream);
        device->xcd_stride = ok ? 8 : 0;
    }
    {   // where this GPU keeps the library's fixed scratch array (looked up once per GPU)
        const int rc = rlt_gemm_static_scratch_setup(device);
        if (rc) { (void)hipFree(device->counters); (void)hipStreamDestroy(device->own_stream); delete device; return rc; }
    }
    {   // defaults of rlt_rocm_set_update_options; RLT_UPDATE_TAIL=0 / RLT_UPDATE_PLACEMENT=spread switch them off for a whole process
        const char* t = std::getenv("RLT_UPDATE_TAIL"); const char* q = std::getenv("RLT_UPDATE_PLACEMENT");
        device->update_tail = !(t && std::strcmp(t, "0") == 0);
        device->update_one_xcd = !(q && std::strcmp(q, "spread") == 0);
        device->wait_limit = 1u << 20;
    }
    // streams for independent passes; without one (or its events) its work stays on the main stream
    for (int k = 0; k < RLT_SIDE_STREAMS; k++) {
        if (hipStreamCreate(&device->side_stream[k]) != hipSuccess) { device->side_stream[k] = nullptr; continue; }
        if (hipEventCreateWithFlags(&device->fork_event[k], hipEventDisableTiming) != hipSuccess) { (void)hipStreamDestroy(device->side_stream[k]); device->side_stream[k] = nullptr; continue; }
        if (hipEventCreateWithFlags(&device->join_event[k], hipEventDisableTiming) != hipSuccess) {
            (void)hipEventDestroy(device->fork_event[k]); (void)hipStreamDestroy(device->side_stream[k]); device->side_stream[k] = nullptr;
        }
    }
    (void)hipGetLastError();
    *out_device = device;
    return 0;
}
int rlt_rocm_set_update_options(rlt_rocm_device* device, int optimiser_in_kernel, int one_xcd) {
    if (!device) return RLT_E_NOT_INITIALISED;
    device->update_tail = optimiser_in_kernel != 0; device->update_one_xcd = one_xcd != 0;
    return 0;
}
int rlt_rocm_set_wait_limit(rlt_rocm_device* device, unsigned polls) {
    if (!device) return RLT_E_NOT_INITIALISED;
    device->wait_limit = polls ? polls : 1u << 20;
    return 0;
}
int rlt_rocm_destroy(rlt_rocm_device* device) {
    if (!device) return RLT_E_INVALID_ARGUMENT;
    (void)hipStreamSynchronize(device->own_stream);
    for (int k = 0; k < RLT_SIDE_STREAMS; k++) {
        if (!device->side_stream[k]) continue;
        (void)hipStreamSynchronize(device->side_stream[k]);
        (void)hipEventDestroy(device->fork_event[k]); (void)hipEventDestroy(device->join_event[k]);
        (void)hipStreamDestroy(device->side_stream[k]);
        if (device->side_scratch[k]) (void)hipFree(device->side_scratch[k]);
    }
    if (device->scratch) (void)hipFree(device->scratch);
    if (device->pad_scratch) (void)hipFree(device->pad_scratch);
    if (device->copy_scratch) (void)hipFree(device->copy_scratch);
    if (device->counters) (void)hipFree(device->counters);
    (void)hipStreamDestroy(device->own_stream);
    delete device;
    return 0;
}
int rlt_rocm_check_status(rlt_rocm_device* device) {
    if (!device) return RLT_E_NOT_INITIALISED;
    if (device->capturing) return 0;      // nothing runs while the stream records (devices/cuda.h:163: check_status does not wait under capture)
    hipError_t e = hipStreamSynchronize(device->stream);
    if (e != hipSuccess) device->sticky_error = (int)e;
    if (device->fault_armed && e == hipSuccess) {
        // word 0: a persistent kernel gave up waiting; word 1: a kernel met an index on the device that points outside its arrays (and skipped that element)
        unsigned fault[2] = {0, 0};
        device->fault_armed = 0;
        if (hipMemcpy(fault, device->fault, sizeof fault, hipMemcpyDeviceToHost) == hipSuccess && (fault[0] || fault[1])) {
            (void)hipMemset(device->fault, 0, sizeof fault);
            if (!device->sticky_error) device->sticky_error = fault[0] ? RLT_E_DEVICE_TIMEOUT : RLT_E_INVALID_ARGUMENT;
        }
    }
    int s = device->sticky_error;
    return s;
}
int rlt_rocm_set_stream(rlt_rocm_device* device, void* hip_stream) {
    if (!device) return RLT_E_NOT_INITIALISED;
    device->stream = hip_stream ? (hipStream_t)hip_stream : device->own_stream;
    return 0;
}
void* rlt_rocm_get_stream(rlt_rocm_device* device) { return device ? (void*)device->stream : nullptr; }
const char* rlt_rocm_error_string(int code) {
    if (code == 0) return "success";
    if (code == RLT_E_INVALID_ARGUMENT) return "rlt_rocm: invalid argument (null pointer, non-positive dimension or too small leading dimension)";
    if (code == RLT_E_UNSUPPORTED) return "rlt_rocm: shape outside what the kernels support";
    if (code == RLT_E_DEVICE_TIMEOUT) return "rlt_rocm: a persistent kernel gave up waiting for another workgroup; its results are invalid";
    if (code == RLT_E_NOT_INITIALISED) return "rlt_rocm: device handle not initialised";
    if (code == RLT_E_CAPTURING) return "rlt_rocm: the call allocates, frees, copies to or from the host or waits, which a stream that records a graph cannot do (size the workspaces with a call before the capture)";
    if (code == RLT_E_WORKSPACE_TOO_SMALL) return "rlt_rocm: the call needs more scratch memory than the library's fixed array (RLT_STATIC_SCRATCH_BYTES) holds; use the allocating entry point or a smaller batch";
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "rlt_rocm: unknown error";
}
int rlt_rocm_device_info(rlt_rocm_device* device, int* compute_units, int* lds_bytes, char* name, int name_len) {
    if (!device) return RLT_E_NOT_INITIALISED;
    if (compute_units) *compute_units = device->compute_units;
    if (lds_bytes) *lds_bytes = device->lds_bytes;
    if (name && name_len > 0) std::snprintf(name, (size_t)name_len, "%s", device->name);
    return 0;
}

int rlt_rocm_malloc(rlt_rocm_device* device, void** out_ptr, size_t bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_NOT_WHILE_CAPTURING();
    RLT_REQUIRE(out_ptr && bytes > 0);
    RLT_HIP(hipMalloc(out_ptr, bytes));
    return 0;
}
int rlt_rocm_free(rlt_rocm_device* device, void* ptr) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_NOT_WHILE_CAPTURING();
    if (!ptr) return 0;
    RLT_HIP(hipFree(ptr));
    return 0;
}
int rlt_rocm_memcpy_h2d(rlt_rocm_device* device, void* dst, const void* src_host, size_t bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_NOT_WHILE_CAPTURING();
    RLT_REQUIRE(dst && src_host);
    if (bytes == 0) return 0;
    RLT_HIP(hipMemcpyAsync(dst, src_host, bytes, hipMemcpyHostToDevice, device->stream));
    RLT_HIP(hipStreamSynchronize(device->stream));
    return 0;
}
int rlt_rocm_memcpy_d2h(rlt_rocm_device* device, void* dst_host, const void* src, size_t bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_NOT_WHILE_CAPTURING();
    RLT_REQUIRE(dst_host && src);
    if (bytes == 0) return 0;
    RLT_HIP(hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDeviceToHost, device->stream));
    RLT_HIP(hipStreamSynchronize(device->stream));
    return 0;
}
int rlt_rocm_memcpy_d2d(rlt_rocm_device* device, void* dst, const void* src, size_t bytes) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst && src);
    if (bytes == 0) return 0;
    RLT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, device->stream));
    return 0;
}
int rlt_rocm_memcpy2d(rlt_rocm_device* device, void* dst, size_t dst_pitch, const void* src, size_t src_pitch,
                      size_t width_bytes, size_t rows, int kind) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst && src && dst_pitch >= width_bytes && src_pitch >= width_bytes && kind >= 0 && kind <= 2);
    if (width_bytes == 0 || rows == 0) return 0;
    hipMemcpyKind k = kind == 0 ? hipMemcpyDeviceToDevice : (kind == 1 ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost);
    RLT_HIP(hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width_bytes, rows, k, device->stream));
    if (kind != 0) { RLT_NOT_WHILE_CAPTURING(); RLT_HIP(hipStreamSynchronize(device->stream)); }
    return 0;
}
int rlt_rocm_fill_f32(rlt_rocm_device* device, float* dst, int rows, int cols, int ld, float value) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst && rows > 0 && cols > 0 && ld >= cols);
    hipLaunchKernelGGL(fill_f32_kernel, dim3(grid_for((size_t)rows * cols)), dim3(256), 0, device->stream, dst, rows, cols, ld, value);
    return rlt_launch_status(device);
}
int rlt_rocm_fill_from_f32(rlt_rocm_device* device, float* dst, int rows, int cols, int ld, const float* value) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst && value && rows > 0 && cols > 0 && ld >= cols);
    hipLaunchKernelGGL(fill_from_f32_kernel, dim3(grid_for((size_t)rows * cols)), dim3(256), 0, device->stream, dst, rows, cols, ld, value);
    return rlt_launch_status(device);
}
int rlt_rocm_fill_u8(rlt_rocm_device* device, uint8_t* dst, size_t count, uint8_t value) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst);
    if (count == 0) return 0;
    hipLaunchKernelGGL(fill_u8_kernel, dim3(grid_for(count)), dim3(256), 0, device->stream, dst, count, value);
    return rlt_launch_status(device);
}
int rlt_rocm_rand_bits_u32(rlt_rocm_device* device, uint32_t* dst, size_t count, uint64_t seed, uint64_t stream) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst);
    if (count == 0) return 0;
    hipLaunchKernelGGL(rand_bits_kernel, dim3(grid_for((count + 3) / 4)), dim3(256), 0, device->stream, dst, count, seed, stream, (const uint64_t*)device->stream_offset);
    return rlt_launch_status(device);
}
int rlt_rocm_randn_f32(rlt_rocm_device* device, float* dst, size_t count, uint64_t seed, uint64_t stream) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst);
    if (count == 0) return 0;
    hipLaunchKernelGGL(rand_kernel, dim3(grid_for((count + 3) / 4)), dim3(256), 0, device->stream, dst, count, 0.0f, 1.0f, seed, stream, 1, (const uint64_t*)device->stream_offset);
    return rlt_launch_status(device);
}
int rlt_rocm_rand_f32(rlt_rocm_device* device, float* dst, size_t count, float low, float high, uint64_t seed, uint64_t stream) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(dst);
    if (count == 0) return 0;
    hipLaunchKernelGGL(rand_kernel, dim3(grid_for((count + 3) / 4)), dim3(256), 0, device->stream, dst, count, low, high, seed, stream, 0, (const uint64_t*)device->stream_offset);
    return rlt_launch_status(device);
}
int rlt_rocm_scale_f32(rlt_rocm_device* device, float* x, size_t count, float s, int reciprocal) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(x);
    if (count == 0) return 0;
    hipLaunchKernelGGL(scale_kernel, dim3(grid_for(count)), dim3(256), 0, device->stream, x, count, s, reciprocal);
    return rlt_launch_status(device);
}
int rlt_rocm_cast_reduce_sum_u8(rlt_rocm_device* device, const uint8_t* mask, size_t count, float* out_sum) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(mask && out_sum);
    hipLaunchKernelGGL(reduce_kernel<0>, dim3(1), dim3(1024), 0, device->stream, (const void*)mask, count, out_sum);
    return rlt_launch_status(device);
}
int rlt_rocm_reduce_sum_f32(rlt_rocm_device* device, const float* x, size_t count, int squared, float* out_sum) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(x && out_sum);
    if (squared) hipLaunchKernelGGL(reduce_kernel<2>, dim3(1), dim3(1024), 0, device->stream, (const void*)x, count, out_sum);
    else hipLaunchKernelGGL(reduce_kernel<1>, dim3(1), dim3(1024), 0, device->stream, (const void*)x, count, out_sum);
    return rlt_launch_status(device);
}

}  // extern "C"

namespace {
__global__ void advance_streams_kernel(uint64_t* __restrict__ offset, uint64_t by, int absolute) { *offset = absolute ? by : *offset + by; }
}
struct rlt_rocm_graph { hipGraph_t graph; hipGraphExec_t executable; };

extern "C" {
int rlt_rocm_advance_streams(rlt_rocm_device* device, uint64_t by) {
    if (!device) return RLT_E_NOT_INITIALISED;
    hipLaunchKernelGGL(advance_streams_kernel, dim3(1), dim3(1), 0, device->stream, device->stream_offset, by, 0);
    return rlt_launch_status(device);
}
int rlt_rocm_set_stream_offset(rlt_rocm_device* device, uint64_t value) {
    if (!device) return RLT_E_NOT_INITIALISED;
    hipLaunchKernelGGL(advance_streams_kernel, dim3(1), dim3(1), 0, device->stream, device->stream_offset, value, 1);
    return rlt_launch_status(device);
}
int rlt_rocm_graph_begin_capture(rlt_rocm_device* device) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_NOT_WHILE_CAPTURING();
    RLT_HIP(hipStreamBeginCapture(device->stream, hipStreamCaptureModeGlobal));
    device->capturing = 1;
    return 0;
}
int rlt_rocm_graph_end_capture(rlt_rocm_device* device, rlt_rocm_graph** out_graph) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(device->capturing);
    hipGraph_t graph = nullptr;
    const hipError_t e = hipStreamEndCapture(device->stream, &graph);      // ends the recording also where a recorded call failed
    device->capturing = 0;
    if (e != hipSuccess) { device->sticky_error = (int)e; if (out_graph) *out_graph = nullptr; return (int)e; }
    if (!out_graph) { (void)hipGraphDestroy(graph); return RLT_E_INVALID_ARGUMENT; }
    hipGraphExec_t executable = nullptr;
    const hipError_t e2 = hipGraphInstantiate(&executable, graph, nullptr, nullptr, 0);
    if (e2 != hipSuccess) { (void)hipGraphDestroy(graph); device->sticky_error = (int)e2; *out_graph = nullptr; return (int)e2; }
    *out_graph = new rlt_rocm_graph{graph, executable};
    return 0;
}
int rlt_rocm_graph_launch(rlt_rocm_device* device, rlt_rocm_graph* graph) {
    if (!device) return RLT_E_NOT_INITIALISED;
    RLT_REQUIRE(graph && graph->executable);
    RLT_NOT_WHILE_CAPTURING();
    device->fault_armed = 1;      // a recorded kernel may be one that waits for other workgroups
    RLT_HIP(hipGraphLaunch(graph->executable, device->stream));
    return 0;
}
int rlt_rocm_graph_destroy(rlt_rocm_device* device, rlt_rocm_graph* graph) {
    if (!device) return RLT_E_NOT_INITIALISED;
    if (!graph) return 0;
    RLT_NOT_WHILE_CAPTURING();
    RLT_HIP(hipStreamSynchronize(device->stream));
    (void)hipGraphExecDestroy(graph->executable);
    (void)hipGraphDestroy(graph->graph);
    delete graph;
    return 0;
}
}  // extern "C"
