// Hidden widths below 64 on the kernels built for 64: zero-padded copies of the parameters, and the way back for the gradients.
// (The reference's zoo trains PPO on the Pendulum at width 32, src/rl/zoo/pendulum-v1/ppo.h:17-18; without this such a network takes the
// per-layer kernels: about a thousand launches per PPO iteration of 64 environments x 128 steps instead of a few dozen.)
#include "pad.h"

namespace {
constexpr int PH = 64;
struct PadArgs {
    const float *W1, *b1, *W2, *b2, *W3, *b3;      // the caller's arrays ([h x in], [h], [h x h], [h], [out x h], [out])
    float *pW1, *pb1, *pW2, *pb2, *pW3, *pb3;      // the padded ones ([64 x in], [64], [64 x 64], [64], [out x 64], [out])
    int in, h, out;
};
__device__ __forceinline__ int pad_total(const PadArgs& a) { return PH * a.in + PH + PH * PH + PH + a.out * PH + a.out; }
// padded <- caller (zero outside the h-wide blocks)
__global__ __launch_bounds__(256) void pad_kernel(PadArgs a) {
    const int n1 = PH * a.in, n2 = n1 + PH, n3 = n2 + PH * PH, n4 = n3 + PH, n5 = n4 + a.out * PH, total = n5 + a.out;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        if (i < n1) { const int r = i / a.in, c = i - r * a.in; a.pW1[i] = r < a.h ? a.W1[r * a.in + c] : 0.f; }
        else if (i < n2) { const int r = i - n1; a.pb1[r] = r < a.h ? a.b1[r] : 0.f; }
        else if (i < n3) { const int j = i - n2, r = j >> 6, c = j & 63; a.pW2[j] = (r < a.h && c < a.h) ? a.W2[r * a.h + c] : 0.f; }
        else if (i < n4) { const int r = i - n3; a.pb2[r] = r < a.h ? a.b2[r] : 0.f; }
        else if (i < n5) { const int j = i - n4, r = j >> 6, c = j & 63; a.pW3[j] = c < a.h ? a.W3[r * a.h + c] : 0.f; }
        else a.pb3[i - n5] = a.b3[i - n5];
    }
}
// caller <- padded: here W1 ... b3 are the caller's GRADIENT arrays (written), pW1 ... pb3 the padded gradients (read)
struct UnpadArgs { float *W1, *b1, *W2, *b2, *W3, *b3; const float *pW1, *pb1, *pW2, *pb2, *pW3, *pb3; int in, h, out; };
__global__ __launch_bounds__(256) void unpad_kernel(UnpadArgs a) {
    const int n1 = a.h * a.in, n2 = n1 + a.h, n3 = n2 + a.h * a.h, n4 = n3 + a.h, n5 = n4 + a.out * a.h, total = n5 + a.out;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        if (i < n1) a.W1[i] = a.pW1[i];                                                     // rows 0 .. h - 1 of [64 x in] are its first h * in entries
        else if (i < n2) a.b1[i - n1] = a.pb1[i - n1];
        else if (i < n3) { const int j = i - n2, r = j / a.h, c = j - r * a.h; a.W2[j] = a.pW2[r * PH + c]; }
        else if (i < n4) a.b2[i - n3] = a.pb2[i - n3];
        else if (i < n5) { const int j = i - n4, r = j / a.h, c = j - r * a.h; a.W3[j] = a.pW3[r * PH + c]; }
        else a.b3[i - n5] = a.pb3[i - n5];
    }
}
bool zero_preserving(int act) { return act == RLT_ACT_IDENTITY || act == RLT_ACT_RELU || act == RLT_ACT_TANH || act == RLT_ACT_FAST_TANH; }
}  // namespace

bool rlt_pad_eligible(const rlt_dense_layer* L, int n) {
    if (!L || n != 3) return false;
    const int h = L[0].out_dim;
    return h >= 1 && h < PH && L[1].in_dim == h && L[1].out_dim == h && L[2].in_dim == h && L[0].in_dim >= 1 && L[2].out_dim >= 1 &&
           L[0].activation == L[1].activation && zero_preserving(L[0].activation) && L[0].weights && L[0].biases && L[1].weights && L[1].biases && L[2].weights && L[2].biases;
}
size_t rlt_pad_floats(const rlt_dense_layer* L, bool with_gradients) {
    const size_t one = (size_t)PH * L[0].in_dim + PH + (size_t)PH * PH + PH + (size_t)L[2].out_dim * PH + L[2].out_dim;
    return ((one + 63) & ~(size_t)63) * (with_gradients ? 2 : 1);
}
int rlt_pad_parameters(rlt_rocm_device* device, const rlt_dense_layer* L, float* memory, bool with_gradients, rlt_padded_net* out) {
    if (!rlt_pad_eligible(L, 3) || !memory || !out) return RLT_E_INVALID_ARGUMENT;
    const int in = L[0].in_dim, h = L[0].out_dim, o = L[2].out_dim;
    float* p = memory;
    PadArgs a = {L[0].weights, L[0].biases, L[1].weights, L[1].biases, L[2].weights, L[2].biases, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, in, h, o};
    a.pW1 = p; p += (size_t)PH * in; a.pb1 = p; p += PH; a.pW2 = p; p += (size_t)PH * PH; a.pb2 = p; p += PH; a.pW3 = p; p += (size_t)o * PH; a.pb3 = p;
    float* g = memory + rlt_pad_floats(L, false);
    for (int l = 0; l < 3; l++) out->L[l] = L[l];
    out->L[0].weights = a.pW1; out->L[0].biases = a.pb1; out->L[0].out_dim = PH;
    out->L[1].weights = a.pW2; out->L[1].biases = a.pb2; out->L[1].in_dim = PH; out->L[1].out_dim = PH;
    out->L[2].weights = a.pW3; out->L[2].biases = a.pb3; out->L[2].in_dim = PH;
    // the hidden layers' kept pre-activations / outputs of the caller are h wide: the one-launch kernels do not write them, and nothing else may run on the description
    out->L[0].pre_activations = nullptr; out->L[0].output = nullptr; out->L[1].pre_activations = nullptr; out->L[1].output = nullptr;
    if (with_gradients) {
        out->L[0].d_weights = g; g += (size_t)PH * in; out->L[0].d_biases = g; g += PH;
        out->L[1].d_weights = g; g += (size_t)PH * PH; out->L[1].d_biases = g; g += PH;
        out->L[2].d_weights = g; g += (size_t)o * PH; out->L[2].d_biases = g;
    } else {
        for (int l = 0; l < 3; l++) { out->L[l].d_weights = nullptr; out->L[l].d_biases = nullptr; }
    }
    const int total = PH * in + PH + PH * PH + PH + o * PH + o;
    hipLaunchKernelGGL(pad_kernel, dim3((total + 255) / 256), dim3(256), 0, device->stream, a);
    return rlt_launch_status(device);
}
int rlt_unpad_gradients(rlt_rocm_device* device, const rlt_dense_layer* L, const rlt_padded_net* P) {
    if (!rlt_pad_eligible(L, 3) || !P) return RLT_E_INVALID_ARGUMENT;
    for (int l = 0; l < 3; l++) if (!L[l].d_weights || !L[l].d_biases || !P->L[l].d_weights || !P->L[l].d_biases) return RLT_E_INVALID_ARGUMENT;
    const int in = L[0].in_dim, h = L[0].out_dim, o = L[2].out_dim;
    UnpadArgs a = {L[0].d_weights, L[0].d_biases, L[1].d_weights, L[1].d_biases, L[2].d_weights, L[2].d_biases,
                   P->L[0].d_weights, P->L[0].d_biases, P->L[1].d_weights, P->L[1].d_biases, P->L[2].d_weights, P->L[2].d_biases, in, h, o};
    const int total = h * in + h + h * h + h + o * h + o;
    hipLaunchKernelGGL(unpad_kernel, dim3((total + 255) / 256), dim3(256), 0, device->stream, a);
    return rlt_launch_status(device);
}
int rlt_pad_scratch(rlt_rocm_device* device, size_t bytes, void** out) {
    if (bytes > device->pad_scratch_bytes) {
        if (device->capturing) return RLT_E_CAPTURING;
        if (device->pad_scratch) RLT_HIP(hipFree(device->pad_scratch));      // hipFree waits for the work that still uses it
        device->pad_scratch = nullptr; device->pad_scratch_bytes = 0;
        const size_t want = bytes < (size_t)(1u << 18) ? (size_t)(1u << 18) : bytes + bytes / 4;
        RLT_HIP(hipMalloc(&device->pad_scratch, want));
        device->pad_scratch_bytes = want;
    }
    *out = device->pad_scratch;
    return 0;
}
