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
static __global__ void __launch_bounds__(KA_ROW_THREADS)
ka_partials_finish_norm_kernel(const float* __restrict__ partial, int splits, const float* __restrict__ bias,
                               const float* __restrict__ bias2, float* __restrict__ out, long ldo, int M, int N,
                               int accumulate, KaThenNorm then) {
    constexpr int WAVES = KA_ROW_THREADS / KA_WAVE;
    __shared__ float red[2][WAVES];
    const int m = blockIdx.x, quads = N / 4;
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    ka_floatx4 x[KA_ROW_QUADS], g[KA_ROW_QUADS], b[KA_ROW_QUADS];
    float sum = 0.f;
    // (the norm's scale and shift are asked for with everything else: one trip to memory for the row)
#pragma unroll
    for (int j = 0; j < KA_ROW_QUADS; ++j) {
        const int n = min(threadIdx.x + j * KA_ROW_THREADS, quads - 1) * 4;
        g[j] = *reinterpret_cast<const ka_floatx4*>(then.gamma + n);
        b[j] = then.beta ? *reinterpret_cast<const ka_floatx4*>(then.beta + n) : ka_floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < KA_ROW_QUADS; ++j) {
        const int q = threadIdx.x + j * KA_ROW_THREADS;
        x[j] = ka_floatx4{0.f, 0.f, 0.f, 0.f};
        if (q >= quads) continue;
        const int n = q * 4;
        float* row = out + (size_t)m * ldo + n;
        ka_floatx4 v = *reinterpret_cast<const ka_floatx4*>(row);
        if (splits > 0) {
            ka_floatx4 s = ka_floatx4{0.f, 0.f, 0.f, 0.f};
            for (int sp0 = 0; sp0 < splits; sp0 += 8) {       // as in the kernel above: eight parts asked for at once, added in order
                ka_floatx4 p[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    p[u] = *reinterpret_cast<const ka_floatx4*>(partial + ((size_t)min(sp0 + u, splits - 1) * M + m) * N + n);
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (sp0 + u < splits) s += p[u];
            }
            if (bias) s += *reinterpret_cast<const ka_floatx4*>(bias + n);
            if (bias2) s += *reinterpret_cast<const ka_floatx4*>(bias2 + n);
            v = accumulate ? v + s : s;
            *reinterpret_cast<ka_floatx4*>(row) = v;
        }
        x[j] = v;
        sum += (v[0] + v[1]) + (v[2] + v[3]);
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
    for (int j = 0; j < KA_ROW_QUADS; ++j) {
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
    for (int j = 0; j < KA_ROW_QUADS; ++j) {
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
