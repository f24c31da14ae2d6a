// Skinny bf16 linear layer for decoding: out = act(A W^T + bias) with few rows (M <= 64).
//
// The weight matrix is streamed from HBM exactly once, and nothing is exchanged between
// workgroups (no fences, no atomics: on a part with eight L2s they cost more than the whole
// product). A workgroup owns a strip of 8 weight rows and all of K; its waves take interleaved
// 64-wide k-blocks and add up through LDS in wave order, so the result is the same on every
// run. 8 rows rather than the MFMA's 16 give N / 8 workgroups, enough to fill 256 CUs at
// N = 2048. v_mfma_f32_16x16x32_bf16 wants 16 row-operand rows: rows 0..7 carry the strip's
// k-block [k, k + 32), rows 8..15 the same weight rows' [k + 32, k + 64), so every lane's
// 16-byte load is useful. Two MFMAs per block then multiply with the activations of the first
// and of the second half; rows 0..7 of the first and rows 8..15 of the second are the wanted
// sums, the other halves are never read.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int SK_STRIP = 8;        // weight rows per workgroup
constexpr int SK_KBLOCK = 64;      // k per wave and step

__device__ __forceinline__ bf16x8 sk_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int MB, int WAVES>
__global__ void __launch_bounds__(WAVES * KA_WAVE)
skinny_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, long ldw,
              const float* __restrict__ bias, void* __restrict__ out, int out_dtype, long ldo, int M,
              int N, int K, int act, int accumulate) {
    __shared__ floatx4 red[WAVES][MB][KA_WAVE];
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * SK_STRIP;
    // Rows beyond N or M are clamped: their products land in places that are never stored.
    const int koff = (r / 8) * 32 + g * 8;            // this lane's place inside a 64-wide k-block
    const bf16_t* wp = W + (size_t)min(n0 + r % 8, N - 1) * ldw + koff;
    const bf16_t* ap[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) ap[mb] = A + (size_t)min(mb * 16 + r, M - 1) * lda + g * 8;
    floatx4 lo[MB], hi[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        lo[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
        hi[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int k = wave * SK_KBLOCK; k < K; k += WAVES * SK_KBLOCK) {
        // K is a multiple of 8: a lane's 8 values are all inside or all outside
        bf16x8 w = k + koff < K ? sk_load8(wp + k) : zero;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            bf16x8 xa = k + g * 8 < K ? sk_load8(ap[mb] + k) : zero;
            bf16x8 xb = k + 32 + g * 8 < K ? sk_load8(ap[mb] + k + 32) : zero;
            lo[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, xa, lo[mb], 0, 0, 0);
            hi[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, xb, hi[mb], 0, 0, 0);
        }
    }
    // A lane holds the MFMA rows g * 4 + i: lanes g < 2 keep rows 0..7 of `lo`, lanes g >= 2 rows
    // 8..15 of `hi`; lanes g and g + 2 hold the two halves of the same output elements.
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) red[wave][mb][lane] = g < 2 ? lo[mb] : hi[mb];
    __syncthreads();
    if (wave != 0 || lane >= 32) return;
    // 32 lanes finish: lane (g in {0, 1}, r) owns out[m = mb * 16 + r][n = n0 + g * 4 + i]
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < WAVES; ++w) s += red[w][mb][lane] + red[w][mb][lane + 32];
        int m = mb * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int n = n0 + g * 4 + i;
            if (n >= N) continue;
            float v = s[i] + (bias ? bias[n] : 0.f);
            if (act == 1) v = ka_gelu_tanh(v);
            size_t o = (size_t)m * ldo + n;
            if (out_dtype == KA_F32) {
                float* op = reinterpret_cast<float*>(out);
                op[o] = accumulate ? op[o] + v : v;
            } else {
                reinterpret_cast<bf16_t*>(out)[o] = (bf16_t)v;
            }
        }
    }
}

template <int MB>
static void launch_mb(int waves, dim3 grid, hipStream_t stream, const bf16_t* A, long lda, const bf16_t* W,
                      long ldw, const float* bias, void* out, int out_dtype, long ldo, int M, int N, int K,
                      int act, int accumulate) {
#define KA_SK(WV)                                                                                          \
    hipLaunchKernelGGL((skinny_kernel<MB, WV>), grid, dim3(WV * KA_WAVE), 0, stream, A, lda, W, ldw, bias, \
                       out, out_dtype, ldo, M, N, K, act, accumulate)
    if (waves >= 16) KA_SK(16);
    else if (waves >= 8) KA_SK(8);
    else if (waves >= 4) KA_SK(4);
    else KA_SK(2);
#undef KA_SK
}

// `target_waves`: waves the launch should put on the chip (about 16 to 32 per CU).
KA_API int ka_linear_skinny_bf16(const void* A, long lda, const void* W, long ldw, const float* bias,
                                 void* out, int out_dtype, long ldo, int M, int N, int K, int act,
                                 int accumulate, int target_waves, hipStream_t stream) {
    KA_CHECK(M > 0 && M <= 64, "ka_linear_skinny_bf16: M=%d outside 1..64", M);
    KA_CHECK(N > 0 && K > 0 && K % 8 == 0, "ka_linear_skinny_bf16: N=%d K=%d (K must be a multiple of 8)", N, K);
    KA_CHECK(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K, "ka_linear_skinny_bf16: row strides must be multiples of 8 and >= K");
    KA_CHECK(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "ka_linear_skinny_bf16: operands must be 16-byte aligned");
    KA_CHECK(ldo >= N, "ka_linear_skinny_bf16: output stride too small");
    KA_CHECK(act == 0 || act == 1, "ka_linear_skinny_bf16: unknown activation %d", act);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_linear_skinny_bf16: bad output type");
    KA_CHECK(!(accumulate && out_dtype != KA_F32), "ka_linear_skinny_bf16: accumulate needs an fp32 output");
    int strips = ka_cdiv(N, SK_STRIP);
    int MB = ka_cdiv(M, 16);
    // waves per workgroup: enough to fill the chip, never more than there are k-blocks
    int waves = ka_cdiv(target_waves, strips);
    int kblocks = ka_cdiv(K, SK_KBLOCK);
    if (waves > kblocks) waves = kblocks;
    if (MB > 2 && waves > 8) waves = 8;       // LDS of the final sum grows with MB
    dim3 grid(strips);
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    switch (MB) {
        case 1: launch_mb<1>(waves, grid, stream, a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate); break;
        case 2: launch_mb<2>(waves, grid, stream, a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate); break;
        case 3: launch_mb<3>(waves, grid, stream, a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate); break;
        default: launch_mb<4>(waves, grid, stream, a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate); break;
    }
    KA_LAUNCH_CHECK();
    return 0;
}
