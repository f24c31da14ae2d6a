// Skinny bf16 linear layer for decoding: out = act(A W^T + bias) with few rows (M <= 64).
//
// The weight matrix is streamed from HBM exactly once; the work is cut over N (strips of
// 16 weight rows per workgroup) and, where N alone gives too few workgroups to fill 256
// CUs, over K as well. The strip is the MFMA's row operand (v_mfma_f32_16x16x32_bf16: a lane
// holds 8 consecutive k of one weight row = one 16-byte load), the activations are the
// column operand, so 16 rows of A cost one MFMA per 32 k. The four waves of a workgroup
// take interleaved k-blocks and add up through LDS in wave order; K-splits add up through
// a scratch buffer in split order by the last workgroup to arrive (a counter per strip
// tells which), so the sum order, and with it the result, is the same on every run.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int SK_THREADS = 256;
constexpr int SK_WAVES = SK_THREADS / KA_WAVE;
constexpr int SK_STRIP = 16;       // weight rows per workgroup
constexpr int SK_KBLOCK = 32;      // k per MFMA

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int MB>
__global__ void __launch_bounds__(SK_THREADS)
skinny_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, long ldw,
              const float* __restrict__ bias, void* __restrict__ out, int out_dtype, long ldo, int M,
              int N, int K, int act, int accumulate, int ksplit, float* __restrict__ partial,
              unsigned* __restrict__ counters) {
    __shared__ floatx4 red[SK_WAVES][MB][KA_WAVE];
    const int strip = blockIdx.x, split = blockIdx.y, S = gridDim.y;
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int n0 = strip * SK_STRIP;
    const int kbeg = split * ksplit;
    const int kend = min(K, kbeg + ksplit);
    // Rows beyond N or M are clamped: their products land in output places that are never stored.
    const bf16_t* wp = W + (size_t)min(n0 + r, N - 1) * ldw + g * 8;
    const bf16_t* ap[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) ap[mb] = A + (size_t)min(mb * 16 + r, M - 1) * lda + g * 8;
    floatx4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 4
    for (int k = kbeg + wave * SK_KBLOCK; k < kend; k += SK_WAVES * SK_KBLOCK) {
        bool in = k + g * 8 < kend;       // K is a multiple of 8: a lane's 8 values are all in or all out
        bf16x8 w = in ? load8(wp + k) : zero;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            bf16x8 a = in ? load8(ap[mb] + k) : zero;
            acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, a, acc[mb], 0, 0, 0);
        }
    }
    // add up the waves in wave order
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) red[wave][mb][lane] = acc[mb];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        floatx4 s = red[0][mb][lane];
#pragma unroll
        for (int w = 1; w < SK_WAVES; ++w) s += red[w][mb][lane];
        acc[mb] = s;
    }
    if (S > 1) {
        float* mine = partial + ((size_t)(strip * S + split) * MB) * (KA_WAVE * 4);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            *reinterpret_cast<floatx4*>(mine + (mb * KA_WAVE + lane) * 4) = acc[mb];
        __threadfence();
        unsigned seen = 0;
        if (lane == 0) seen = atomicAdd(&counters[strip], 1u);
        seen = __shfl(seen, 0, KA_WAVE);
        if (seen != (unsigned)(S - 1)) return;
        if (lane == 0) atomicExch(&counters[strip], 0u);      // ready for the next launch
        __threadfence();
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < S; ++s) {
            const float* theirs = partial + ((size_t)(strip * S + s) * MB) * (KA_WAVE * 4);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const float* p = theirs + (mb * KA_WAVE + lane) * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[mb][i] += __hip_atomic_load(p + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    // epilogue: lane holds out[m = mb*16 + r][n = n0 + g*4 + i]
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        int m = mb * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int n = n0 + g * 4 + i;
            if (n >= N) continue;
            float v = acc[mb][i] + (bias ? bias[n] : 0.f);
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

// Scratch the K-splits add up through: `partial` floats and `counters` (zero before the
// first call; every call leaves them zero again). Calls that share scratch must not overlap.
KA_API long ka_skinny_partial_floats(int M, int N, int K, int target_workgroups) {
    int strips = ka_cdiv(N, SK_STRIP);
    int splits = strips >= target_workgroups ? 1 : ka_cdiv(target_workgroups, strips);
    int MB = ka_cdiv(M, 16);
    return (long)strips * splits * MB * KA_WAVE * 4;
}

KA_API int ka_linear_skinny_bf16(const void* A, long lda, const void* W, long ldw, const float* bias,
                                 void* out, int out_dtype, long ldo, int M, int N, int K, int act,
                                 int accumulate, float* partial, long partial_floats,
                                 unsigned* counters, int n_counters, int target_workgroups,
                                 hipStream_t stream) {
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
    // K-splits: enough workgroups to fill the chip, each at least one k-block per wave.
    int splits = 1;
    if (strips < target_workgroups) splits = ka_cdiv(target_workgroups, strips);
    int unit = SK_WAVES * SK_KBLOCK;
    int ksplit = ka_cdiv(ka_cdiv(K, splits), unit) * unit;
    splits = ka_cdiv(K, ksplit);
    if (splits > 1) {
        KA_CHECK(partial && counters, "ka_linear_skinny_bf16: scratch missing");
        KA_CHECK((long)strips * splits * MB * KA_WAVE * 4 <= partial_floats, "ka_linear_skinny_bf16: scratch too small");
        KA_CHECK(strips <= n_counters, "ka_linear_skinny_bf16: too few counters (%d strips)", strips);
        KA_CHECK(splits <= 65535, "ka_linear_skinny_bf16: too many splits");
    }
    dim3 grid(strips, splits), block(SK_THREADS);
#define KA_SK(MBV)                                                                                          \
    hipLaunchKernelGGL(skinny_kernel<MBV>, grid, block, 0, stream, (const bf16_t*)A, lda, (const bf16_t*)W, \
                       ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, ksplit, partial, counters)
    switch (MB) {
        case 1: KA_SK(1); break;
        case 2: KA_SK(2); break;
        case 3: KA_SK(3); break;
        default: KA_SK(4); break;
    }
#undef KA_SK
    KA_LAUNCH_CHECK();
    return 0;
}
