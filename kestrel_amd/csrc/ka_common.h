// Shared declarations of the kestrel_amd HIP kernels (gfx950 / CDNA4).
//
// Every entry point is `extern "C"`, takes raw device pointers, plain integers and
// a hipStream_t, validates its sizes on the host and returns 0 on success or a
// negative code; `ka_last_error()` then gives the reason as text. Entry points
// never allocate device memory and never synchronise (ka_linear_library_bf16 makes the
// vendor library's handle and its plan for a set of sizes at the first call with them).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define KA_API extern "C" __attribute__((visibility("default")))

// Element types of tensors crossing the C boundary.
enum KaDType : int { KA_F32 = 0, KA_BF16 = 1 };

typedef __bf16 bf16_t;

constexpr int KA_WAVE = 64;

// Error text of the last failed call in this thread (ka_error.hip; each library
// links its own copy).
void ka_set_error(const char* fmt, ...);

#define KA_CHECK(cond, ...)            \
    do {                               \
        if (!(cond)) {                 \
            ka_set_error(__VA_ARGS__); \
            return -1;                 \
        }                              \
    } while (0)

#define KA_LAUNCH_CHECK()                                                        \
    do {                                                                         \
        hipError_t e__ = hipGetLastError();                                      \
        if (e__ != hipSuccess) {                                                 \
            ka_set_error("%s: launch failed: %s", __func__, hipGetErrorString(e__)); \
            return -2;                                                           \
        }                                                                        \
    } while (0)

__device__ __forceinline__ float ka_to_float(float v) { return v; }
__device__ __forceinline__ float ka_to_float(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T ka_from_float(float v);
template <>
__device__ __forceinline__ float ka_from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t ka_from_float<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ float ka_wave_sum(float v) {
#pragma unroll
    for (int off = KA_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, KA_WAVE);
    return v;
}

__device__ __forceinline__ float ka_wave_max(float v) {
#pragma unroll
    for (int off = KA_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, KA_WAVE));
    return v;
}

// GELU with the tanh approximation: 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))).
__device__ __forceinline__ float ka_gelu_tanh(float x) {
    const float k0 = 0.7978845608028654f;
    const float k1 = 0.044715f;
    float inner = k0 * (x + k1 * x * x * x);
    return 0.5f * x * (1.0f + tanhf(inner));
}

// The same as x * sigmoid(2u), u = sqrt(2/pi) (x + 0.044715 x^3), on the hardware's exponential and
// reciprocal: 0.5 x (1 + tanh u) = x / (1 + e^(-2u)). Five ordinary instructions and two
// transcendental ones instead of the library routine's many (a kernel's epilogue applies this
// to 128 values a lane while the matrix pipes stand still). Exact to about 1e-7 relative, far
// below what a bf16 result keeps; the kernels that write bf16 activations use it.
__device__ __forceinline__ float ka_gelu_tanh_fast(float x) {
    const float c1 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;              // -2 sqrt(2/pi) log2(e)
    const float c3 = c1 * 0.044715f;
    const float e = __builtin_amdgcn_exp2f(x * fmaf(x * x, c3, c1));                  // e^(-2u): inf for very negative x, 0 for large x
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// Activations a linear kernel can apply in its epilogue. One table for every kernel family: a
// further activation is a code here, a case in each of the two functions below, and its name in
// the table of the Python face (ops/linear.py).
enum KaAct : int { KA_ACT_NONE = 0, KA_ACT_GELU_TANH = 1, KA_ACT_RELU = 2, KA_ACT_SILU = 3, KA_ACT_COUNT = 4 };

static inline bool ka_act_known(int act) { return act >= 0 && act < KA_ACT_COUNT; }

// Library-exact forms: the 32-bit path.
__device__ __forceinline__ float ka_activate(int act, float x) {
    switch (act) {
        case KA_ACT_GELU_TANH: return ka_gelu_tanh(x);
        case KA_ACT_RELU: return fmaxf(x, 0.f);
        case KA_ACT_SILU: return x / (1.0f + expf(-x));
        default: return x;
    }
}

// On the hardware's exponential and reciprocal: the kernels that write bf16 activations.
__device__ __forceinline__ float ka_activate_fast(int act, float x) {
    switch (act) {
        case KA_ACT_GELU_TANH: return ka_gelu_tanh_fast(x);
        case KA_ACT_RELU: return fmaxf(x, 0.f);
        case KA_ACT_SILU: return x * __fdividef(1.0f, 1.0f + __expf(-x));
        default: return x;
    }
}

// Compute units of the current device (asked once; 256, an MI355X, if the device will not say).
static inline int ka_compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cus = n;
        else
            cus = 256;
    }
    return cus;
}

static inline int ka_cdiv(long a, long b) { return (int)((a + b - 1) / b); }
