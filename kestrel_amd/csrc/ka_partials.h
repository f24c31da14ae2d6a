// Partial sums of a linear layer whose K was cut into parts, and the kernel that adds them up.
//
// A kernel that cuts K writes the sums of part p as fp32 [M, N] at partial + p * M * N; the
// finishing kernel adds the parts in their order (no atomics: the same bits on every run) and
// applies what the linear's epilogue would have: biases, activation, accumulation into the output.
#pragma once
#include "ka_common.h"

typedef __attribute__((ext_vector_type(4))) float ka_floatx4;

// out = act(sum of the parts + biases) (+ out): one thread per four neighbouring outputs
static __global__ void __launch_bounds__(256)
ka_partials_finish_kernel(const float* __restrict__ partial, int splits, const float* __restrict__ bias,
                          const float* __restrict__ bias2, void* __restrict__ out, int out_dtype, long ldo, int M,
                          int N, int act, int accumulate) {
    const int quads = (N + 3) / 4;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= M * quads) return;
    const int m = idx / quads, n = (idx % quads) * 4;
    const bool whole = n + 3 < N && N % 4 == 0;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if (whole) {
        // eight parts' sums are asked for at once (a part past the last is the last again, and
        // left out of the sum), then added in the order of the parts
        for (int sp0 = 0; sp0 < splits; sp0 += 8) {
            ka_floatx4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = *reinterpret_cast<const ka_floatx4*>(partial + ((size_t)min(sp0 + u, splits - 1) * M + m) * N + n);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (sp0 + u < splits) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) s[i] += v[u][i];
                }
            }
        }
    } else {
        for (int sp = 0; sp < splits; ++sp) {
            const float* src = partial + ((size_t)sp * M + m) * N + n;
            for (int i = 0; i < 4 && n + i < N; ++i) s[i] += src[i];
        }
    }
    if (ka_act_gated(act)) {
        float v[4];
        for (int i = 0; i < 4; ++i) v[i] = n + i < N ? s[i] + (bias ? bias[n + i] : 0.f) + (bias2 ? bias2[n + i] : 0.f) : 0.f;
        ka_gated_store<true, 4>(out, out_dtype, ldo, m, n, N, v, act);
        return;
    }
    for (int i = 0; i < 4 && n + i < N; ++i) {
        float x = s[i] + (bias ? bias[n + i] : 0.f) + (bias2 ? bias2[n + i] : 0.f);
        if (act) x = ka_activate_fast(act, x);
        const size_t o = (size_t)m * ldo + n + i;
        if (out_dtype == KA_F32) {
            float* op = reinterpret_cast<float*>(out) + o;
            *op = accumulate ? *op + x : x;
        } else {
            reinterpret_cast<bf16_t*>(out)[o] = (bf16_t)x;
        }
    }
}


// A LayerNorm that follows a linear layer whose result lands in fp32 rows (the residual): the
// next block's first norm, computed where the rows are finished instead of in a launch of its own.
struct KaThenNorm {
    const float* gamma;
    const float* beta;      // may be null
    float eps;
    void* out;              // [M, N], rows ld apart
    int out_dtype;
    long ld;
};

constexpr int KA_ROW_THREADS = 512;
constexpr int KA_ROW_QUADS = 4;            // four neighbouring outputs per thread, this many times: rows up to 8192 wide
static inline bool ka_then_norm_fits(int N) { return N % 4 == 0 && N <= KA_ROW_THREADS * 4 * KA_ROW_QUADS; }

// One workgroup per row m: out[m] (+)= sum of the parts + biases (parts == 0: out[m] stands as it
// is), then normed[m] = LayerNorm(out[m]) with fp32 statistics over the row kept in registers.
// JN: fours of neighbouring outputs per thread (the row's width / 2048, rounded up). Everything a
// thread needs is asked for at once, from places moved inside the row where the thread has nothing
// there: one trip to memory whatever the width (a row of 2560, whose second four only a quarter of
// the threads have, took two: 6.6 us against 5.1 for a row of 2048).
template <int JN>
static __global__ void __launch_bounds__(KA_ROW_THREADS)
ka_partials_finish_norm_kernel(const float* __restrict__ partial, int splits, const float* __restrict__ bias,
                               const float* __restrict__ bias2, float* __restrict__ out, long ldo, int M, int N,
                               int accumulate, KaThenNorm then) {
    static_assert(JN >= 1 && JN <= KA_ROW_QUADS, "a row of at most 8192");
    constexpr int WAVES = KA_ROW_THREADS / KA_WAVE;
    __shared__ float red[2][WAVES];
    const int m = blockIdx.x, quads = N / 4;
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    ka_floatx4 x[JN], g[JN], b[JN], first[JN][8], extra[JN][2];
    const ka_floatx4 zero = ka_floatx4{0.f, 0.f, 0.f, 0.f};
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < JN; ++j) {
        const int n = min(threadIdx.x + j * KA_ROW_THREADS, quads - 1) * 4;
        g[j] = *reinterpret_cast<const ka_floatx4*>(then.gamma + n);
        b[j] = then.beta ? *reinterpret_cast<const ka_floatx4*>(then.beta + n) : zero;
        x[j] = *reinterpret_cast<const ka_floatx4*>(out + (size_t)m * ldo + n);
        if (splits > 0) {                                      // (the same for all threads)
#pragma unroll
            for (int u = 0; u < 8; ++u)
                first[j][u] = *reinterpret_cast<const ka_floatx4*>(partial + ((size_t)min(u, splits - 1) * M + m) * N + n);
            extra[j][0] = bias ? *reinterpret_cast<const ka_floatx4*>(bias + n) : zero;
            extra[j][1] = bias2 ? *reinterpret_cast<const ka_floatx4*>(bias2 + n) : zero;
        }
    }
#pragma unroll
    for (int j = 0; j < JN; ++j) {
        const int q = threadIdx.x + j * KA_ROW_THREADS;
        const bool mine = q < quads;
        const int n = min(q, quads - 1) * 4;
        ka_floatx4 v = x[j];
        if (splits > 0) {
            ka_floatx4 s = zero;
#pragma unroll
            for (int u = 0; u < 8; ++u)                        // the parts in their order
                if (u < splits) s += first[j][u];
            for (int sp0 = 8; sp0 < splits; sp0 += 8) {        // more than eight parts: eight more at a time
                ka_floatx4 p[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    p[u] = *reinterpret_cast<const ka_floatx4*>(partial + ((size_t)min(sp0 + u, splits - 1) * M + m) * N + n);
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (sp0 + u < splits) s += p[u];
            }
            s += extra[j][0];
            s += extra[j][1];
            v = accumulate ? v + s : s;
            if (mine) *reinterpret_cast<ka_floatx4*>(out + (size_t)m * ldo + n) = v;
        }
        x[j] = mine ? v : zero;
        if (mine) sum += (v[0] + v[1]) + (v[2] + v[3]);
    }
    sum = ka_wave_sum(sum);
    if (lane == 0) red[0][wave] = sum;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += red[0][w];
    const float mean = total / (float)N;
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < JN; ++j) {
        if (threadIdx.x + j * KA_ROW_THREADS < quads) {
#pragma unroll
            for (int i = 0; i < 4; ++i) sq += (x[j][i] - mean) * (x[j][i] - mean);
        }
    }
    sq = ka_wave_sum(sq);
    if (lane == 0) red[1][wave] = sq;
    __syncthreads();
    float var = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) var += red[1][w];
    const float rstd = 1.0f / sqrtf(var / (float)N + then.eps);
#pragma unroll
    for (int j = 0; j < JN; ++j) {
        const int q = threadIdx.x + j * KA_ROW_THREADS;
        if (q >= quads) continue;
        const int n = q * 4;
        float y[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = (x[j][i] - mean) * rstd * g[j][i] + b[j][i];
        const size_t o = (size_t)m * then.ld + n;
        if (then.out_dtype == KA_F32) {
            *reinterpret_cast<ka_floatx4*>(reinterpret_cast<float*>(then.out) + o) = ka_floatx4{y[0], y[1], y[2], y[3]};
        } else {
            typedef __attribute__((ext_vector_type(4))) __bf16 ka_bf16x4;
            ka_bf16x4 r;
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] = (bf16_t)y[i];
            *reinterpret_cast<ka_bf16x4*>(reinterpret_cast<bf16_t*>(then.out) + o) = r;
        }
    }
}

// (N: a multiple of 4, at most `ka_then_norm_fits` allows)
static inline void ka_launch_finish_norm(int M, int N, hipStream_t stream, const float* partial, int splits, const float* bias,
                                         const float* bias2, float* out, long ldo, int accumulate, const KaThenNorm& then) {
    const int fours = (N / 4 + KA_ROW_THREADS - 1) / KA_ROW_THREADS;
    switch (fours) {
        case 1: hipLaunchKernelGGL(ka_partials_finish_norm_kernel<1>, dim3(M), dim3(KA_ROW_THREADS), 0, stream, partial, splits, bias, bias2, out, ldo, M, N, accumulate, then); break;
        case 2: hipLaunchKernelGGL(ka_partials_finish_norm_kernel<2>, dim3(M), dim3(KA_ROW_THREADS), 0, stream, partial, splits, bias, bias2, out, ldo, M, N, accumulate, then); break;
        case 3: hipLaunchKernelGGL(ka_partials_finish_norm_kernel<3>, dim3(M), dim3(KA_ROW_THREADS), 0, stream, partial, splits, bias, bias2, out, ldo, M, N, accumulate, then); break;
        default: hipLaunchKernelGGL(ka_partials_finish_norm_kernel<4>, dim3(M), dim3(KA_ROW_THREADS), 0, stream, partial, splits, bias, bias2, out, ldo, M, N, accumulate, then); break;
    }
}
