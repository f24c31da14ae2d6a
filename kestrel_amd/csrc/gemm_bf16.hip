// Tiled bf16 linear layer for prompts: out = act(A W^T + bias) or out += A W^T + bias.
//
// Both operands are K-contiguous (A [M, K], W [N, K]), which is exactly what the MFMA
// operand layout wants: a lane holds 8 consecutive k of one row. A workgroup of four
// waves computes a 128 (weight rows) x 128 (activation rows) tile in K-steps of 64 through
// double-buffered LDS (rows padded to 144 bytes, which makes the 16-byte operand reads
// bank-conflict free); each wave owns a 64 x 64 quarter as 2 x 2 v_mfma_f32_32x32x16_bf16
// tiles. The weight rows are the MFMA's row operand, so a lane ends up with four
// consecutive output columns of one output row and stores them as one vector. Bias,
// GELU-tanh and the fp32 residual accumulate run in the epilogue.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int GB_N = 128;          // weight rows per tile
constexpr int GB_K = 64;           // k per step
constexpr int GB_LD = GB_K + 8;    // padded LDS row (144 bytes)
constexpr int GB_THREADS = 256;
// Activation rows per tile: 64 * MT. MT = 2 is the square tile; MT = 1 doubles the number of
// workgroups where N x M alone would leave CUs idle (the N = dim products of a 2048-token prompt).
constexpr int gb_m(int mt) { return 64 * mt; }
constexpr int gb_smem(int mt) { return 2 * (GB_N + gb_m(mt)) * GB_LD * 2; }   // two buffers of both tiles

__device__ __forceinline__ bf16x8 gb_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int MT>
__global__ void __launch_bounds__(GB_THREADS)
gemm_bf16_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, long ldw,
                 const float* __restrict__ bias, void* __restrict__ out, int out_dtype, long ldo, int M,
                 int N, int K, int act, int accumulate, int tiles_n, int tiles_m) {
    extern __shared__ __attribute__((aligned(16))) unsigned char gb_lds[];
    bf16_t (*Ws)[GB_N][GB_LD] = reinterpret_cast<bf16_t (*)[GB_N][GB_LD]>(gb_lds);
    constexpr int GB_M = gb_m(MT);
    bf16_t (*Xs)[GB_M][GB_LD] = reinterpret_cast<bf16_t (*)[GB_M][GB_LD]>(gb_lds + 2 * GB_N * GB_LD * sizeof(bf16_t));
    // Tiles are numbered so that the workgroups one XCD gets (every 8th) walk down a column of
    // tiles that share the same weight rows, which then stay in that XCD's L2.
    int pid = blockIdx.x;
    int total = tiles_n * tiles_m;
    int per_xcd = (total + 7) / 8;
    int logical = (pid % 8) * per_xcd + pid / 8;
    if (logical >= total) return;
    int tn = logical / tiles_m, tm = logical % tiles_m;
    const int n0 = tn * GB_N, m0 = tm * gb_m(MT);
    const int tid = threadIdx.x, wave = tid / KA_WAVE, lane = tid % KA_WAVE;
    const int wn = wave / 2, wm = wave % 2;
    const int li = lane % 32, lg = lane / 32;

    floatx16 acc[2][MT];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 wreg[4], xreg[2 * MT];
    // chunk c = tid + i * 256: row c / 8, k-chunk c % 8
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int c = tid + i * GB_THREADS;
            int row = c >> 3, k = k0 + (c & 7) * 8;
            int n = n0 + row;
            wreg[i] = (n < N && k < K) ? gb_load8(W + (size_t)n * ldw + k) : zero;
        }
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) {
            int c = tid + i * GB_THREADS;
            int row = c >> 3, k = k0 + (c & 7) * 8;
            int m = m0 + row;
            xreg[i] = (m < M && k < K) ? gb_load8(A + (size_t)m * lda + k) : zero;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int c = tid + i * GB_THREADS;
            *reinterpret_cast<bf16x8*>(&Ws[buf][c >> 3][(c & 7) * 8]) = wreg[i];
        }
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) {
            int c = tid + i * GB_THREADS;
            *reinterpret_cast<bf16x8*>(&Xs[buf][c >> 3][(c & 7) * 8]) = xreg[i];
        }
    };

    const int steps = (K + GB_K - 1) / GB_K;
    fetch(0);
    stash(0);
    __syncthreads();
    for (int s = 0; s < steps; ++s) {
        int buf = s & 1;
        if (s + 1 < steps) fetch((s + 1) * GB_K);
#pragma unroll
        for (int ks = 0; ks < GB_K / 16; ++ks) {
            bf16x8 wa[2], xb[MT];
#pragma unroll
            for (int t = 0; t < 2; ++t)
                wa[t] = *reinterpret_cast<const bf16x8*>(&Ws[buf][wn * 64 + t * 32 + li][ks * 16 + lg * 8]);
#pragma unroll
            for (int t = 0; t < MT; ++t)
                xb[t] = *reinterpret_cast<const bf16x8*>(&Xs[buf][wm * 32 * MT + t * 32 + li][ks * 16 + lg * 8]);
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < MT; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[a], xb[b], acc[a][b], 0, 0, 0);
        }
        if (s + 1 < steps) stash(buf ^ 1);
        __syncthreads();
    }

    // epilogue: acc[a][b][v] is out[m][n] with n = n0 + wn*64 + a*32 + (v/4)*8 + lg*4 + v%4, m = m0 + wm*32*MT + b*32 + li
    const bool vec_ok = (N % 4 == 0) && (ldo % 4 == 0);
#pragma unroll
    for (int b = 0; b < MT; ++b) {
        int m = m0 + wm * 32 * MT + b * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                int n = n0 + wn * 64 + a * 32 + q * 8 + lg * 4;
                if (n >= N) continue;
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float x = acc[a][b][q * 4 + i];
                    if (bias && n + i < N) x += bias[n + i];
                    if (act == 1) x = ka_gelu_tanh(x);
                    v[i] = x;
                }
                size_t o = (size_t)m * ldo + n;
                if (out_dtype == KA_F32) {
                    float* op = reinterpret_cast<float*>(out) + o;
                    if (vec_ok) {
                        floatx4 cur = accumulate ? *reinterpret_cast<floatx4*>(op) : floatx4{0.f, 0.f, 0.f, 0.f};
                        floatx4 res = {cur[0] + v[0], cur[1] + v[1], cur[2] + v[2], cur[3] + v[3]};
                        *reinterpret_cast<floatx4*>(op) = res;
                    } else {
                        for (int i = 0; i < 4 && n + i < N; ++i) op[i] = accumulate ? op[i] + v[i] : v[i];
                    }
                } else {
                    bf16_t* op = reinterpret_cast<bf16_t*>(out) + o;
                    if (vec_ok) {
                        bf16x4 res = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
                        *reinterpret_cast<bf16x4*>(op) = res;
                    } else {
                        for (int i = 0; i < 4 && n + i < N; ++i) op[i] = (bf16_t)v[i];
                    }
                }
            }
        }
    }
}

KA_API int ka_linear_tiled_bf16(const void* A, long lda, const void* W, long ldw, const float* bias,
                                void* out, int out_dtype, long ldo, int M, int N, int K, int act,
                                int accumulate, hipStream_t stream) {
    KA_CHECK(M > 0 && N > 0 && K > 0 && K % 8 == 0, "ka_linear_tiled_bf16: M=%d N=%d K=%d (K must be a multiple of 8)", M, N, K);
    KA_CHECK(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K, "ka_linear_tiled_bf16: row strides must be multiples of 8 and >= K");
    KA_CHECK(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "ka_linear_tiled_bf16: operands must be 16-byte aligned");
    KA_CHECK(ldo >= N, "ka_linear_tiled_bf16: output stride too small");
    KA_CHECK(act == 0 || act == 1, "ka_linear_tiled_bf16: unknown activation %d", act);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_linear_tiled_bf16: bad output type");
    KA_CHECK(!(accumulate && out_dtype != KA_F32), "ka_linear_tiled_bf16: accumulate needs an fp32 output");
    uintptr_t obase = (uintptr_t)out;
    KA_CHECK(obase % 16 == 0, "ka_linear_tiled_bf16: output must be 16-byte aligned");
    int tiles_n = ka_cdiv(N, GB_N);
    // the square tile unless it would leave fewer than two workgroups per CU
    int mt = (long)tiles_n * ka_cdiv(M, gb_m(2)) < 512 ? 1 : 2;
    int tiles_m = ka_cdiv(M, gb_m(mt));
    long total = (long)tiles_n * tiles_m;
    long launched = ((total + 7) / 8) * 8;
    KA_CHECK(launched < (1L << 31), "ka_linear_tiled_bf16: too many tiles");
    static bool configured = false;
    if (!configured) {
        hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_kernel<1>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, gb_smem(1));
        hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_kernel<2>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, gb_smem(2));
        KA_CHECK(e1 == hipSuccess && e2 == hipSuccess, "ka_linear_tiled_bf16: cannot reserve %d bytes of LDS", gb_smem(2));
        configured = true;
    }
    if (mt == 1)
        hipLaunchKernelGGL(gemm_bf16_kernel<1>, dim3((unsigned)launched), dim3(GB_THREADS), gb_smem(1), stream,
                           (const bf16_t*)A, lda, (const bf16_t*)W, ldw, bias, out, out_dtype, ldo, M, N, K, act,
                           accumulate, tiles_n, tiles_m);
    else
        hipLaunchKernelGGL(gemm_bf16_kernel<2>, dim3((unsigned)launched), dim3(GB_THREADS), gb_smem(2), stream,
                           (const bf16_t*)A, lda, (const bf16_t*)W, ldw, bias, out, out_dtype, ldo, M, N, K, act,
                           accumulate, tiles_n, tiles_m);
    KA_LAUNCH_CHECK();
    return 0;
}
