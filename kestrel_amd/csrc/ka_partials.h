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

