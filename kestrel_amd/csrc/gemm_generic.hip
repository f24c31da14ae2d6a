// Generic linear layer: out = act(A W^T + bias) or out += A W^T + bias.
//
// Plain FMA in fp32 with an LDS-tiled 64x64x16 block, any M, N, K, any mix of fp32
// and bf16 operands. Every output element is the sum over k = 0..K-1 in that order,
// whatever M and N are, so a row's result does not depend on what else is in the
// batch. This is the true 32-bit path and the fallback of the bf16 path.
#include "ka_common.h"

constexpr int GT = 64;   // tile edge in M and N
constexpr int GK = 16;   // tile depth

template <typename TA, typename TW, typename TOut>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const TA* __restrict__ A, long lda, const TW* __restrict__ W, long ldw,
                    const float* __restrict__ bias, TOut* __restrict__ out, long ldo, int M, int N,
                    int K, int act, int accumulate) {
    __shared__ float As[GK][GT + 4];
    __shared__ float Ws[GK][GT + 4];
    int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    float acc[4][4] = {};
    // Each thread loads 4 elements of each operand tile: row = tid / 4, k = (tid % 4) * 4 .. +4.
    int lr = threadIdx.x / 4, lk = (threadIdx.x % 4) * 4;
    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int k = k0 + lk + j;
            int m = m0 + lr, n = n0 + lr;
            As[lk + j][lr] = (m < M && k < K) ? ka_to_float(A[(size_t)m * lda + k]) : 0.f;
            Ws[lk + j][lr] = (n < N && k < K) ? ka_to_float(W[(size_t)n * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int m = m0 + ty * 4 + i;
        if (m >= M) continue;
        if (ka_act_gated(act)) {           // pairs of neighbouring columns make one output
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = acc[i][j] + (bias && n0 + tx * 4 + j < N ? bias[n0 + tx * 4 + j] : 0.f);
            ka_gated_store<false, 4>(out, sizeof(TOut) == 4 ? KA_F32 : KA_BF16, ldo, m, n0 + tx * 4, N, v, act);
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j] + (bias ? bias[n] : 0.f);
            if (act) v = ka_activate(act, v);
            size_t o = (size_t)m * ldo + n;
            if (accumulate) v += ka_to_float(out[o]);
            out[o] = ka_from_float<TOut>(v);
        }
    }
}

// Many rows in fp32 (prompts on the 32-bit path): the same sums, k in ascending order for every
// output, from a tile of 128 x 128 x 8 with 8 x 8 outputs a thread, 16-byte loads (rows and K
// must allow them: the host sends everything else to the kernel above) and two LDS stages.
constexpr int GF = 128;   // tile edge in M and N
constexpr int GFK = 8;    // tile depth

// (RM: output rows a thread holds, 8 or 4: tiles of 128 or 64 rows; the lower tile doubles the
// workgroups of a narrow output that would otherwise leave CUs with one or none)
template <int RM>
__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ A, long lda, const float* __restrict__ W, long ldw,
                const float* __restrict__ bias, float* __restrict__ out, long ldo, int M, int N, int K, int act,
                int accumulate) {
    typedef __attribute__((ext_vector_type(4))) float f4;
    constexpr int TM = 16 * RM;
    __shared__ __attribute__((aligned(16))) float As[2][GFK][TM + 4];
    __shared__ __attribute__((aligned(16))) float Ws[2][GFK][GF + 4];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * GF;
    // each thread brings four consecutive k of one row of each operand tile (rows past the end
    // are the last row again: their outputs are never stored)
    const int lr = threadIdx.x / 2, lk = (threadIdx.x % 2) * 4;
    const bool brings_a = lr < TM;
    const float* arow = A + (size_t)min(m0 + min(lr, TM - 1), M - 1) * lda + lk;
    const float* wrow = W + (size_t)min(n0 + lr, N - 1) * ldw + lk;
    const f4 zero = {0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int k0, f4& ra, f4& rw) {
        const bool ok = k0 + lk < K;             // K is a multiple of 4
        ra = ok ? *reinterpret_cast<const f4*>(arow + k0) : zero;
        rw = ok ? *reinterpret_cast<const f4*>(wrow + k0) : zero;
    };
    auto stash = [&](int buf, const f4& ra, const f4& rw) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (brings_a) As[buf][lk + j][lr] = ra[j];
            Ws[buf][lk + j][lr] = rw[j];
        }
    };
    float acc[RM][8] = {};
    f4 ra, rw;
    fetch(0, ra, rw);
    stash(0, ra, rw);
    __syncthreads();
    const int steps = (K + GFK - 1) / GFK;
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        if (s + 1 < steps) fetch((s + 1) * GFK, ra, rw);
#pragma unroll
        for (int k = 0; k < GFK; ++k) {
            float a[RM];
#pragma unroll
            for (int i = 0; i < RM; i += 4) {
                const f4 v = *reinterpret_cast<const f4*>(&As[buf][k][ty * RM + i]);
#pragma unroll
                for (int u = 0; u < 4; ++u) a[i + u] = v[u];
            }
            const f4 w0 = *reinterpret_cast<const f4*>(&Ws[buf][k][tx * 8]), w1 = *reinterpret_cast<const f4*>(&Ws[buf][k][tx * 8 + 4]);
#pragma unroll
            for (int i = 0; i < RM; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(a[i], j < 4 ? w0[j] : w1[j - 4], acc[i][j]);
        }
        if (s + 1 < steps) stash(buf ^ 1, ra, rw);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < RM; ++i) {
        const int m = m0 + ty * RM + i;
        if (m >= M) continue;
        if (ka_act_gated(act)) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = acc[i][j] + (bias && n0 + tx * 8 + j < N ? bias[n0 + tx * 8 + j] : 0.f);
            ka_gated_store<false, 8>(out, KA_F32, ldo, m, n0 + tx * 8, N, v, act);
            continue;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int n = n0 + tx * 8 + j;
            if (n >= N) continue;
            float v = acc[i][j] + (bias ? bias[n] : 0.f);
            if (act) v = ka_activate(act, v);
            const size_t o = (size_t)m * ldo + n;
            out[o] = accumulate ? out[o] + v : v;
        }
    }
}

// Few rows in fp32 (decoding on the 32-bit path): the tile above would put a sixteenth of its
// threads to work and read every weight through LDS. Here a wave owns one output column: its
// lanes walk over K with 16-byte loads of the weight row and of each activation row, every lane
// adds up its own k in their order, and the lanes' sums meet in a fixed tree. Plain fp32 FMA as
// above; the order of a sum is another than the tile's, the same for every M and N.
constexpr int GV_ROWS = 16;      // most rows
constexpr int GV_WAVES = 4;      // output columns per workgroup

typedef __attribute__((ext_vector_type(4))) float gv_float4;

__global__ void __launch_bounds__(GV_WAVES * KA_WAVE)
gemv_f32_kernel(const float* __restrict__ A, long lda, const float* __restrict__ W, long ldw,
                const float* __restrict__ bias, float* __restrict__ out, long ldo, int M, int N, int K, int act,
                int accumulate) {
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const int n = blockIdx.x * GV_WAVES + wave;
    if (n >= N) return;
    const float* wrow = W + (size_t)n * ldw;
    float acc[GV_ROWS];
#pragma unroll
    for (int m = 0; m < GV_ROWS; ++m) acc[m] = 0.f;
    for (int k = lane * 4; k < K; k += KA_WAVE * 4) {
        const gv_float4 w = *reinterpret_cast<const gv_float4*>(wrow + k);
#pragma unroll
        for (int m = 0; m < GV_ROWS; ++m) {
            if (m < M) {
                const gv_float4 a = *reinterpret_cast<const gv_float4*>(A + (size_t)m * lda + k);
                acc[m] = fmaf(a[3], w[3], fmaf(a[2], w[2], fmaf(a[1], w[1], fmaf(a[0], w[0], acc[m]))));
            }
        }
    }
#pragma unroll
    for (int m = 0; m < GV_ROWS; ++m) {
        if (m >= M) break;
        float v = ka_wave_sum(acc[m]);
        if (lane == 0) {
            v += bias ? bias[n] : 0.f;
            if (act) v = ka_activate(act, v);
            const size_t o = (size_t)m * ldo + n;
            out[o] = accumulate ? out[o] + v : v;
        }
    }
}

template <typename TA, typename TW, typename TOut>
static void launch(const void* A, long lda, const void* W, long ldw, const float* bias, void* out,
                   long ldo, int M, int N, int K, int act, int accumulate, hipStream_t stream) {
    dim3 grid(ka_cdiv(N, GT), ka_cdiv(M, GT)), block(256);
    hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TOut>), grid, block, 0, stream, (const TA*)A, lda,
                       (const TW*)W, ldw, bias, (TOut*)out, ldo, M, N, K, act, accumulate);
}

// A: [M, K] rows lda apart; W: [N, K] rows ldw apart; bias: fp32 [N] or null;
// out: [M, N] rows ldo apart. act: 0 none, 1 GELU-tanh. accumulate: out += result
// (only into fp32 out).
KA_API int ka_linear_generic(const void* A, int a_dtype, long lda, const void* W, int w_dtype,
                             long ldw, const float* bias, void* out, int out_dtype, long ldo,
                             int M, int N, int K, int act, int accumulate, hipStream_t stream) {
    KA_CHECK(M >= 0 && N > 0 && K > 0, "ka_linear_generic: bad sizes M=%d N=%d K=%d", M, N, K);
    KA_CHECK(ka_act_known(act), "ka_linear_generic: unknown activation %d", act);
    KA_CHECK(lda >= K && ldw >= K && ldo >= ka_act_outputs(act, N), "ka_linear_generic: strides too small");
    KA_CHECK(!ka_act_gated(act) || (N % 2 == 0 && !accumulate), "ka_linear_generic: a gated linear needs an even N and no accumulation");
    KA_CHECK(!(accumulate && out_dtype != KA_F32), "ka_linear_generic: accumulate needs an fp32 output");
    KA_CHECK(ka_cdiv(M, GT) <= 65535, "ka_linear_generic: M=%d too large for one launch", M);
    if (M == 0) return 0;
    int key = a_dtype * 4 + w_dtype * 2 + out_dtype;
    const bool vectors = key == 0 && K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && (uintptr_t)A % 16 == 0 &&
                         (uintptr_t)W % 16 == 0;
    if (vectors && M > GV_ROWS && ka_cdiv(M, 64) <= 65535) {
        if ((long)ka_cdiv(N, GF) * ka_cdiv(M, GF) >= 512)
            hipLaunchKernelGGL(gemm_f32_kernel<8>, dim3(ka_cdiv(N, GF), ka_cdiv(M, GF)), dim3(256), 0, stream, (const float*)A, lda,
                               (const float*)W, ldw, bias, (float*)out, ldo, M, N, K, act, accumulate);
        else
            hipLaunchKernelGGL(gemm_f32_kernel<4>, dim3(ka_cdiv(N, GF), ka_cdiv(M, 64)), dim3(256), 0, stream, (const float*)A, lda,
                               (const float*)W, ldw, bias, (float*)out, ldo, M, N, K, act, accumulate);
        KA_LAUNCH_CHECK();
        return 0;
    }
    if (vectors && M <= GV_ROWS && !ka_act_gated(act)) {      // (a wave per column there: the pair of a gate would meet nowhere)
        hipLaunchKernelGGL(gemv_f32_kernel, dim3(ka_cdiv(N, GV_WAVES)), dim3(GV_WAVES * KA_WAVE), 0, stream,
                           (const float*)A, lda, (const float*)W, ldw, bias, (float*)out, ldo, M, N, K, act, accumulate);
        KA_LAUNCH_CHECK();
        return 0;
    }
#define KA_CASE(k, TA, TW, TO) \
    case k: launch<TA, TW, TO>(A, lda, W, ldw, bias, out, ldo, M, N, K, act, accumulate, stream); break;
    switch (key) {
        KA_CASE(0, float, float, float)
        KA_CASE(1, float, float, bf16_t)
        KA_CASE(2, float, bf16_t, float)
        KA_CASE(3, float, bf16_t, bf16_t)
        KA_CASE(4, bf16_t, float, float)
        KA_CASE(5, bf16_t, float, bf16_t)
        KA_CASE(6, bf16_t, bf16_t, float)
        KA_CASE(7, bf16_t, bf16_t, bf16_t)
        default: KA_CHECK(false, "ka_linear_generic: unsupported dtypes a=%d w=%d out=%d", a_dtype, w_dtype, out_dtype);
    }
#undef KA_CASE
    KA_LAUNCH_CHECK();
    return 0;
}
