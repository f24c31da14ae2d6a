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

// Reductions over groups of neighbouring lanes inside the vector unit: lane moves that ride on the
// arithmetic instruction (DPP) up to a row of 16 lanes and the row and half-wave swaps of gfx950
// above that, where a shuffle (ds_bpermute) makes a trip through the LDS pipe for every step.
//
// ka_lanes_reduce<FROM, TO>(v, op): every lane gets op over its aligned group of TO lanes, given
// that the lanes of each aligned group of FROM lanes already hold one value (FROM = 1: any values).
// The steps of 4 and 8 lanes mirror a half row and a row, which pairs a lane with one of the other
// group, not with lane ^ 4 or lane ^ 8: that is the same only because of that condition. `op` must
// be commutative; every lane of a group ends with the same bits. All 64 lanes must be active.
struct KaSum { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };
struct KaMax { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct KaIntMax { __device__ __forceinline__ int operator()(int a, int b) const { return a > b ? a : b; } };
struct KaIntMin { __device__ __forceinline__ int operator()(int a, int b) const { return a < b ? a : b; } };

// `v` of the lane that the DPP control names, in the rows of 16 lanes that ROWS has a bit for; 0 in the
// other rows and, if ZERO_OUTSIDE, in a lane whose source lies outside its row.
template <int CTRL, typename T, int ROWS = 0xF, bool ZERO_OUTSIDE = true>
__device__ __forceinline__ T ka_dpp_move(T v) {
    static_assert(sizeof(T) == 4, "lane moves carry 32 bits");
    return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROWS, 0xF, ZERO_OUTSIDE));
}

// One step of such a reduction: `a` and `b` are the values of the two groups of STEP lanes that
// meet in this lane (which of them is this lane's own differs from lane to lane).
template <int STEP, typename T>
__device__ __forceinline__ void ka_lanes_pair(T v, T& a, T& b) {
    static_assert(sizeof(T) == 4 && STEP >= 1 && STEP < KA_WAVE && (STEP & (STEP - 1)) == 0, "a power of two within a wave");
    typedef __attribute__((ext_vector_type(2))) unsigned ka_u2;
    if constexpr (STEP <= 8) {
        a = v;
        if constexpr (STEP == 1) b = ka_dpp_move<0xB1>(v);            // quad_perm [1,0,3,2]
        else if constexpr (STEP == 2) b = ka_dpp_move<0x4E>(v);       // quad_perm [2,3,0,1]
        else if constexpr (STEP == 4) b = ka_dpp_move<0x141>(v);      // row_half_mirror
        else b = ka_dpp_move<0x140>(v);                               // row_mirror
    } else {
        const unsigned bits = __builtin_bit_cast(unsigned, v);
        ka_u2 s;
        // 16: rows 1 and 3 of the first register change places with rows 0 and 2 of the second;
        // 32: the upper half of the first with the lower half of the second
        if constexpr (STEP == 16) s = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
        else s = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        a = __builtin_bit_cast(T, (unsigned)s[0]);
        b = __builtin_bit_cast(T, (unsigned)s[1]);
    }
}

template <int FROM, int TO, typename T, typename Op>
__device__ __forceinline__ T ka_lanes_reduce(T v, Op op) {
    static_assert(TO <= KA_WAVE && (TO & (TO - 1)) == 0, "groups are powers of two within a wave");
    if constexpr (FROM >= TO) {
        return v;
    } else {
        T a, b;
        ka_lanes_pair<FROM>(v, a, b);
        return ka_lanes_reduce<FROM * 2, TO>(op(a, b), op);
    }
}

// Running sums along the lanes of a wave (lane i gets the sum of lanes 0..i), by the same means:
// four shifts inside each row of 16 (a lane that has no neighbour so far down gets 0), then the
// last lane of a row handed to the rows after it. All 64 lanes must be active.
__device__ __forceinline__ float ka_wave_running_sum(float v) {
    v += ka_dpp_move<0x111>(v);                          // row_shr:1
    v += ka_dpp_move<0x112>(v);                          // row_shr:2
    v += ka_dpp_move<0x114>(v);                          // row_shr:4
    v += ka_dpp_move<0x118>(v);                          // row_shr:8
    v += ka_dpp_move<0x142, float, 0xA, false>(v);       // row_bcast:15, into rows 1 and 3
    v += ka_dpp_move<0x143, float, 0xC, false>(v);       // row_bcast:31, into rows 2 and 3
    return v;
}

// The value of one lane (a number known at compile time or the same in every lane) in all lanes.
__device__ __forceinline__ float ka_lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

__device__ __forceinline__ float ka_wave_sum(float v) { return ka_lanes_reduce<1, KA_WAVE>(v, KaSum{}); }
__device__ __forceinline__ float ka_wave_max(float v) { return ka_lanes_reduce<1, KA_WAVE>(v, KaMax{}); }

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

// A gated linear layer (the first half of a feed-forward of the form act(x Wg^T) * (x Wu^T)): KA_ACT_GATED
// added to an activation's code says that the rows of the weights come in pairs, row 2j the gate's and
// row 2j + 1 the value's of output j (biases likewise), and that the epilogue writes
// out[m][j] = act(sum 2j) * (sum 2j + 1): N / 2 outputs from N weight rows, in the same pass. Every
// epilogue of this folder holds neighbouring columns in one thread, so the pair meets in registers
// (ka_gated_store below). Not together with accumulation into the output.
constexpr int KA_ACT_GATED = 0x100;

__host__ __device__ __forceinline__ bool ka_act_gated(int act) { return (act & KA_ACT_GATED) != 0; }
__host__ __device__ __forceinline__ int ka_act_base(int act) { return act & ~KA_ACT_GATED; }
static inline bool ka_act_known(int act) { return ka_act_base(act) >= 0 && ka_act_base(act) < KA_ACT_COUNT; }
// Columns of the output of a linear layer of N weight rows.
static inline int ka_act_outputs(int act, int N) { return ka_act_gated(act) ? N / 2 : N; }

// Library-exact forms: the 32-bit path.
__device__ __forceinline__ float ka_activate(int act, float x) {
    switch (ka_act_base(act)) {
        case KA_ACT_GELU_TANH: return ka_gelu_tanh(x);
        case KA_ACT_RELU: return fmaxf(x, 0.f);
        case KA_ACT_SILU: return x / (1.0f + expf(-x));
        default: return x;
    }
}

// On the hardware's exponential and reciprocal: the kernels that write bf16 activations.
__device__ __forceinline__ float ka_activate_fast(int act, float x) {
    switch (ka_act_base(act)) {
        case KA_ACT_GELU_TANH: return ka_gelu_tanh_fast(x);
        case KA_ACT_RELU: return fmaxf(x, 0.f);
        case KA_ACT_SILU: return x * __fdividef(1.0f, 1.0f + __expf(-x));
        default: return x;
    }
}

// The epilogue of a gated linear layer for the sums (biases added) of the weight rows n .. n + COUNT - 1 of
// output row m, n even: out[m][(n + 2p) / 2] = act(v[2p]) * v[2p + 1] for every pair inside N. FAST: the
// activations on the hardware's exponential (the kernels that write bf16), else the library's.
template <bool FAST, int COUNT>
__device__ __forceinline__ void ka_gated_store(void* out, int out_dtype, long ldo, int m, int n, int N, const float* v, int act) {
    static_assert(COUNT % 2 == 0, "pairs");
#pragma unroll
    for (int p = 0; p < COUNT / 2; ++p) {
        if (n + 2 * p + 1 >= N) continue;
        const float g = FAST ? ka_activate_fast(act, v[2 * p]) : ka_activate(act, v[2 * p]);
        const float y = g * v[2 * p + 1];
        const size_t o = (size_t)m * ldo + (n + 2 * p) / 2;
        if (out_dtype == KA_F32) reinterpret_cast<float*>(out)[o] = y;
        else reinterpret_cast<bf16_t*>(out)[o] = (bf16_t)y;
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
