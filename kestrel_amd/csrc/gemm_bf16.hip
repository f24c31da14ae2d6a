// Tiled bf16 linear layer for prompts: out = act(A W^T + bias) or out += A W^T + bias.
//
// Both operands are K-contiguous (A [M, K], W [N, K]), which is exactly what the MFMA
// operand layout wants: a lane holds 8 consecutive k of one row. A workgroup of four waves
// (2 x 2) computes a tile of 64 NT weight rows x 64 MT activation rows in K-steps of BK through
// double-buffered LDS (rows padded by 16 bytes, which keeps the 16-byte operand reads off each
// other's banks); each wave owns NT x MT v_mfma_f32_32x32x16_bf16 tiles. The weight rows are the
// MFMA's row operand, so a lane ends up with four consecutive output columns of one output row
// and stores them as one vector. Bias, GELU-tanh and the fp32 residual accumulate run in the
// epilogue.
//
// The 2 x 2 wave tile (128 x 128 per workgroup) is used where it gives every CU two workgroups,
// 2 x 1 otherwise; other shapes can be forced for measurements.
#include "ka_common.h"

#include <stdlib.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int GB_THREADS = 256;
constexpr int GB_PAD = 8;          // bf16 of padding per LDS row

constexpr int gb_smem(int nt, int mt, int bk) { return 2 * 64 * (nt + mt) * (bk + GB_PAD) * 2; }

__device__ __forceinline__ bf16x8 gb_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int NT, int MT, int BK>
__global__ void __launch_bounds__(GB_THREADS)
gemm_bf16_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, long ldw,
                 const float* __restrict__ bias, void* __restrict__ out, int out_dtype, long ldo, int M,
                 int N, int K, int act, int accumulate, int tiles_n, int tiles_m) {
    constexpr int BN = 64 * NT, BM = 64 * MT, LD = BK + GB_PAD;
    constexpr int CPR = BK / 8;                          // 16-byte chunks per tile row
    constexpr int WCH = BN * CPR / GB_THREADS;           // chunks of W a thread moves per k-step
    constexpr int XCH = BM * CPR / GB_THREADS;
    static_assert(BN * CPR % GB_THREADS == 0 && BM * CPR % GB_THREADS == 0, "tile does not divide over the threads");
    extern __shared__ __attribute__((aligned(16))) unsigned char gb_lds[];
    bf16_t (*Ws)[BN][LD] = reinterpret_cast<bf16_t (*)[BN][LD]>(gb_lds);
    bf16_t (*Xs)[BM][LD] = reinterpret_cast<bf16_t (*)[BM][LD]>(gb_lds + 2 * BN * LD * sizeof(bf16_t));
    // Tiles are numbered so that the workgroups one XCD gets (every 8th) walk down a column of
    // tiles that share the same weight rows, which then stay in that XCD's L2.
    int pid = blockIdx.x;
    int total = tiles_n * tiles_m;
    int per_xcd = (total + 7) / 8;
    int logical = (pid % 8) * per_xcd + pid / 8;
    if (logical >= total) return;
    int tn = logical / tiles_m, tm = logical % tiles_m;
    const int n0 = tn * BN, m0 = tm * BM;
    const int tid = threadIdx.x, wave = tid / KA_WAVE, lane = tid % KA_WAVE;
    const int wn = wave / 2, wm = wave % 2;
    const int li = lane % 32, lg = lane / 32;

    floatx16 acc[NT][MT];
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 wreg[WCH], xreg[XCH];
    // chunk c = tid + i * 256: row c / CPR, k-chunk c % CPR
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            int c = tid + i * GB_THREADS;
            int n = n0 + c / CPR, k = k0 + (c % CPR) * 8;
            wreg[i] = (n < N && k < K) ? gb_load8(W + (size_t)n * ldw + k) : zero;
        }
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            int c = tid + i * GB_THREADS;
            int m = m0 + c / CPR, k = k0 + (c % CPR) * 8;
            xreg[i] = (m < M && k < K) ? gb_load8(A + (size_t)m * lda + k) : zero;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            int c = tid + i * GB_THREADS;
            *reinterpret_cast<bf16x8*>(&Ws[buf][c / CPR][(c % CPR) * 8]) = wreg[i];
        }
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            int c = tid + i * GB_THREADS;
            *reinterpret_cast<bf16x8*>(&Xs[buf][c / CPR][(c % CPR) * 8]) = xreg[i];
        }
    };

    const int steps = (K + BK - 1) / BK;
    fetch(0);
    stash(0);
    __syncthreads();
    for (int s = 0; s < steps; ++s) {
        int buf = s & 1;
        if (s + 1 < steps) fetch((s + 1) * BK);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 wa[NT], xb[MT];
#pragma unroll
            for (int t = 0; t < NT; ++t)
                wa[t] = *reinterpret_cast<const bf16x8*>(&Ws[buf][wn * 32 * NT + t * 32 + li][ks * 16 + lg * 8]);
#pragma unroll
            for (int t = 0; t < MT; ++t)
                xb[t] = *reinterpret_cast<const bf16x8*>(&Xs[buf][wm * 32 * MT + t * 32 + li][ks * 16 + lg * 8]);
#pragma unroll
            for (int a = 0; a < NT; ++a)
#pragma unroll
                for (int b = 0; b < MT; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[a], xb[b], acc[a][b], 0, 0, 0);
        }
        if (s + 1 < steps) stash(buf ^ 1);
        __syncthreads();
    }

    // epilogue: acc[a][b][v] is out[m][n] with n = n0 + wn*32*NT + a*32 + (v/4)*8 + lg*4 + v%4,
    // m = m0 + wm*32*MT + b*32 + li
    const bool vec_ok = (N % 4 == 0) && (ldo % 4 == 0);
#pragma unroll
    for (int b = 0; b < MT; ++b) {
        int m = m0 + wm * 32 * MT + b * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < NT; ++a) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                int n = n0 + wn * 32 * NT + a * 32 + q * 8 + lg * 4;
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

template <int NT, int MT, int BK>
static int launch_config(const bf16_t* A, long lda, const bf16_t* W, long ldw, const float* bias, void* out,
                         int out_dtype, long ldo, int M, int N, int K, int act, int accumulate,
                         hipStream_t stream) {
    static bool configured = false;
    constexpr int smem = gb_smem(NT, MT, BK);
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_kernel<NT, MT, BK>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        KA_CHECK(e == hipSuccess, "ka_linear_tiled_bf16: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
        configured = true;
    }
    int tiles_n = ka_cdiv(N, 64 * NT), tiles_m = ka_cdiv(M, 64 * MT);
    long total = (long)tiles_n * tiles_m;
    long launched = ((total + 7) / 8) * 8;
    KA_CHECK(launched < (1L << 31), "ka_linear_tiled_bf16: too many tiles");
    hipLaunchKernelGGL((gemm_bf16_kernel<NT, MT, BK>), dim3((unsigned)launched), dim3(GB_THREADS), smem, stream, A, lda,
                       W, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, tiles_n, tiles_m);
    return 0;
}

// `config`: 0 chooses by size; 421 / 221 / 211 force the 4x2 (BK 32), 2x2 (BK 64), 2x1 (BK 64) tile.
KA_API int ka_linear_tiled_bf16(const void* A, long lda, const void* W, long ldw, const float* bias,
                                void* out, int out_dtype, long ldo, int M, int N, int K, int act,
                                int accumulate, int config, hipStream_t stream) {
    KA_CHECK(M > 0 && N > 0 && K > 0 && K % 8 == 0, "ka_linear_tiled_bf16: M=%d N=%d K=%d (K must be a multiple of 8)", M, N, K);
    KA_CHECK(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K, "ka_linear_tiled_bf16: row strides must be multiples of 8 and >= K");
    KA_CHECK(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "ka_linear_tiled_bf16: operands must be 16-byte aligned");
    KA_CHECK(ldo >= N, "ka_linear_tiled_bf16: output stride too small");
    KA_CHECK(act == 0 || act == 1, "ka_linear_tiled_bf16: unknown activation %d", act);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_linear_tiled_bf16: bad output type");
    KA_CHECK(!(accumulate && out_dtype != KA_F32), "ka_linear_tiled_bf16: accumulate needs an fp32 output");
    KA_CHECK((uintptr_t)out % 16 == 0, "ka_linear_tiled_bf16: output must be 16-byte aligned");
    if (config == 0) {
        // the square tile unless it leaves fewer than two workgroups per CU (measured: the bigger
        // 4 x 2 tile is slower at every size tried, the loop being bound by latency, not by LDS)
        long t22 = (long)ka_cdiv(N, 128) * ka_cdiv(M, 128);
        config = t22 >= 512 ? 221 : 211;
    }
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    int rc;
    switch (config) {
        case 421: rc = launch_config<4, 2, 32>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); break;
        case 221: rc = launch_config<2, 2, 64>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); break;
        case 211: rc = launch_config<2, 1, 64>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); break;
        case 222: rc = launch_config<2, 2, 32>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); break;
        case 441: rc = launch_config<4, 4, 32>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); break;
        default: KA_CHECK(false, "ka_linear_tiled_bf16: unknown tile configuration %d", config);
    }
    if (rc) return rc;
    KA_LAUNCH_CHECK();
    return 0;
}
