// Skinny bf16 linear layers for decoding (M <= 64 rows): out = act(A W^T + bias).
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
//
// At these sizes a kernel costs more in launch and memory latency than in bytes, so one launch
// does as much as the data flow allows:
//  * two K-segments into one output (out += A1 W1^T + A2 W2^T + b1 + b2): the attention
//    output projection and the second feed-forward linear of a parallel block in one pass;
//  * two outputs from one input (strips of W_a, then strips of W_b): the fused q|k|v
//    projection and the first feed-forward linear, which read the same normalised input;
//  * a LayerNorm prologue (M <= 16): the workgroup normalises the fp32 rows itself (one wave
//    per row, statistics in fp32, two passes) into LDS and feeds the MFMA from there.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int SK_STRIP = 8;        // weight rows per workgroup
constexpr int SK_KBLOCK = 64;      // k per wave and step
constexpr int SK_LN_ROWS = 16;     // most rows the LayerNorm prologue takes
constexpr int SK_PREFETCH = 4;     // weight blocks a wave loads before the LayerNorm prologue
constexpr int SK_XV = 8;           // float4 per lane of a row kept in registers (rows up to 2048 wide)
constexpr int SK_PAD = 8;          // bf16 of padding per LDS row (keeps 16-byte reads off each other's banks)

__device__ __forceinline__ bf16x8 sk_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
// Weights are read once and never again: a load that does not displace the activations,
// which every workgroup of a CU reads, from the caches.
__device__ __forceinline__ bf16x8 sk_load8_stream(const bf16_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
}

struct SkinnyTarget {       // one weight matrix and where its product goes
    const bf16_t* W;
    long ldw;
    const float* bias;
    void* out;
    long ldo;
    int out_dtype;
    int N;
    int act;
    int accumulate;
};

struct SkinnyArgs {
    // input: up to two K-segments (A[1] null: one), or fp32 rows to be normalised (ln_x)
    const bf16_t* A[2];
    long lda[2];
    int K[2];
    const bf16_t* W2;       // weights of the second segment, rows as in target a
    long ldw2;
    const float* bias2;
    const float* ln_x;      // fp32 [M, K[0]] rows to normalise instead of A[0]
    const float* ln_gamma;
    const float* ln_beta;
    float ln_eps;
    SkinnyTarget a, b;      // b.W null: one target
    int strips_a;
    int M;
};

template <int MB, int WAVES, bool LN>
__global__ void __launch_bounds__(WAVES * KA_WAVE) __attribute__((amdgpu_waves_per_eu(4)))
skinny_kernel(SkinnyArgs p) {
    __shared__ floatx4 red[WAVES][MB][KA_WAVE];
    extern __shared__ __attribute__((aligned(16))) unsigned char sk_dyn[];
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const int r = lane % 16, g = lane / 16;
    const bool second = (int)blockIdx.x >= p.strips_a;
    const SkinnyTarget& tg = second ? p.b : p.a;
    const int n0 = (second ? blockIdx.x - p.strips_a : blockIdx.x) * SK_STRIP;
    const int M = p.M, N = tg.N;
    const int koff = (r / 8) * 32 + g * 8;            // this lane's place inside a 64-wide k-block
    const size_t wrow = (size_t)min(n0 + r % 8, N - 1);

    floatx4 lo[MB], hi[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        lo[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
        hi[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    // What the 32 finishing lanes add at the end (bias, and the output's old value when the
    // product is accumulated) is fetched now: its latency hides behind the weight stream.
    floatx4 addend[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) addend[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    if (wave == 0 && lane < 32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int n = n0 + g * 4 + i;
            if (n >= N) continue;
            float b = tg.bias ? tg.bias[n] : 0.f;
            if (!second && p.bias2) b += p.bias2[n];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                int m = mb * 16 + r;
                float old = 0.f;
                if (tg.accumulate && m < M) old = reinterpret_cast<const float*>(tg.out)[(size_t)m * tg.ldo + n];
                addend[mb][i] = b;
                if (tg.accumulate) lo[mb][i] = old;     // wave 0's own sum starts from the old value
            }
        }
    }

    if constexpr (LN) {
        // Weight loads of this wave's first blocks go out first: they do not depend on the rows,
        // and their latency then hides behind the LayerNorm below.
        const int K = p.K[0];
        const bf16_t* wp = tg.W + wrow * tg.ldw + koff;
        bf16x8 wpre[SK_PREFETCH];
#pragma unroll
        for (int j = 0; j < SK_PREFETCH; ++j) {
            int k = (wave + j * WAVES) * SK_KBLOCK;
            wpre[j] = k + koff < K ? sk_load8_stream(wp + k) : zero;
        }
        // the rows go to LDS as [M][K + pad] bf16: copied as they are, or normalised on the way
        // (rows w, w + WAVES, ... by wave w)
        bf16_t* xs = reinterpret_cast<bf16_t*>(sk_dyn);
        const int ld = K + SK_PAD;
        if (p.ln_x == nullptr) {
            const int cpr = K / 8;
            for (int c = threadIdx.x; c < M * cpr; c += WAVES * KA_WAVE) {
                int m = c / cpr, kc = (c % cpr) * 8;
                *reinterpret_cast<bf16x8*>(xs + m * ld + kc) = sk_load8(p.A[0] + (size_t)m * p.lda[0] + kc);
            }
        }
        for (int m = wave; m < M && p.ln_x != nullptr; m += WAVES) {
            const float* src = p.ln_x + (size_t)m * K;
            {
                // the row stays in registers (K <= SK_XV * 256, checked by the host): one trip to memory
                floatx4 xv[SK_XV];
                float s = 0.f;
#pragma unroll
                for (int j = 0; j < SK_XV; ++j) {
                    int k = (j * KA_WAVE + lane) * 4;
                    xv[j] = k < K ? *reinterpret_cast<const floatx4*>(src + k) : floatx4{0.f, 0.f, 0.f, 0.f};
                    s += (xv[j][0] + xv[j][1]) + (xv[j][2] + xv[j][3]);
                }
                float mean = ka_wave_sum(s) / (float)K;
                float q = 0.f;
#pragma unroll
                for (int j = 0; j < SK_XV; ++j) {
                    int k = (j * KA_WAVE + lane) * 4;
                    if (k < K) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) q += (xv[j][i] - mean) * (xv[j][i] - mean);
                    }
                }
                float rstd = 1.0f / sqrtf(ka_wave_sum(q) / (float)K + p.ln_eps);
#pragma unroll
                for (int j = 0; j < SK_XV; ++j) {
                    int k = (j * KA_WAVE + lane) * 4;
                    if (k < K) {
                        floatx4 gm = *reinterpret_cast<const floatx4*>(p.ln_gamma + k);
                        bf16x4 y;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            float v = (xv[j][i] - mean) * rstd * gm[i];
                            if (p.ln_beta) v += p.ln_beta[k + i];
                            y[i] = (bf16_t)v;
                        }
                        *reinterpret_cast<bf16x4*>(xs + m * ld + k) = y;
                    }
                }
            }
        }
        __syncthreads();
        const bf16_t* xp = xs + min(r, M - 1) * ld + g * 8;
#pragma unroll
        for (int j = 0; j < SK_PREFETCH; ++j) {
            int k = (wave + j * WAVES) * SK_KBLOCK;
            if (k < K) {
                bf16x8 xa = k + g * 8 < K ? *reinterpret_cast<const bf16x8*>(xp + k) : zero;
                bf16x8 xb = k + 32 + g * 8 < K ? *reinterpret_cast<const bf16x8*>(xp + k + 32) : zero;
                lo[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wpre[j], xa, lo[0], 0, 0, 0);
                hi[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wpre[j], xb, hi[0], 0, 0, 0);
            }
        }
        for (int k = (wave + SK_PREFETCH * WAVES) * SK_KBLOCK; k < K; k += WAVES * SK_KBLOCK) {
            bf16x8 w = k + koff < K ? sk_load8(wp + k) : zero;
            bf16x8 xa = k + g * 8 < K ? *reinterpret_cast<const bf16x8*>(xp + k) : zero;
            bf16x8 xb = k + 32 + g * 8 < K ? *reinterpret_cast<const bf16x8*>(xp + k + 32) : zero;
            lo[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, xa, lo[0], 0, 0, 0);
            hi[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, xb, hi[0], 0, 0, 0);
        }
    } else {
#pragma unroll
        for (int seg = 0; seg < 2; ++seg) {
            if (seg == 1 && p.A[1] == nullptr) break;
            const int K = p.K[seg];
            const bf16_t* wp = (seg == 0 ? tg.W + wrow * tg.ldw : p.W2 + wrow * p.ldw2) + koff;
            const bf16_t* ap[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) ap[mb] = p.A[seg] + (size_t)min(mb * 16 + r, M - 1) * p.lda[seg] + g * 8;
            // K is a multiple of 8: a lane's 8 values are all inside or all outside. UN blocks at a
            // time, and ALL their loads (weights and activations) before the first MFMA: an
            // activation load issued between MFMAs puts a trip to L2 on the critical path per block.
            constexpr int UN = MB == 1 ? 4 : MB == 2 ? 2 : 1;
            for (int k0 = wave * SK_KBLOCK; k0 < K; k0 += UN * WAVES * SK_KBLOCK) {
                bf16x8 w[UN], xa[UN][MB], xb[UN][MB];
#pragma unroll
                for (int u = 0; u < UN; ++u) {
                    int k = k0 + u * WAVES * SK_KBLOCK;
                    w[u] = k + koff < K ? sk_load8_stream(wp + k) : zero;
                }
#pragma unroll
                for (int u = 0; u < UN; ++u) {
                    int k = k0 + u * WAVES * SK_KBLOCK;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const bool row = mb * 16 + r < M;      // rows past M are not fetched at all
                        xa[u][mb] = row && k + g * 8 < K ? sk_load8(ap[mb] + k) : zero;
                        xb[u][mb] = row && k + 32 + g * 8 < K ? sk_load8(ap[mb] + k + 32) : zero;
                    }
                }
#pragma unroll
                for (int u = 0; u < UN; ++u) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        lo[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u], xa[u][mb], lo[mb], 0, 0, 0);
                        hi[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u], xb[u][mb], hi[mb], 0, 0, 0);
                    }
                }
            }
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
            float v = s[i] + addend[mb][i];
            if (tg.act == 1) v = ka_gelu_tanh(v);
            size_t o = (size_t)m * tg.ldo + n;
            if (tg.out_dtype == KA_F32) {
                reinterpret_cast<float*>(tg.out)[o] = v;       // an accumulated product already holds the old value
            } else {
                reinterpret_cast<bf16_t*>(tg.out)[o] = (bf16_t)v;
            }
        }
    }
}

template <int MB, bool LN>
static int launch_mb(int waves, int strips, size_t dyn, hipStream_t stream, const SkinnyArgs& args) {
#define KA_SK(WV)                                                                                       \
    do {                                                                                                \
        if (dyn > 0) {                                                                                  \
            static size_t reserved = 0;                                                                 \
            if (dyn > reserved) {                                                                       \
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(skinny_kernel<MB, WV, LN>), \
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);   \
                KA_CHECK(e == hipSuccess, "skinny linear: cannot reserve %zu bytes of LDS", dyn);       \
                reserved = dyn;                                                                         \
            }                                                                                           \
        }                                                                                               \
        hipLaunchKernelGGL((skinny_kernel<MB, WV, LN>), dim3(strips), dim3(WV * KA_WAVE), dyn, stream, args); \
    } while (0)
    if (waves >= 16) KA_SK(16);
    else if (waves >= 8) KA_SK(8);
    else if (waves >= 4) KA_SK(4);
    else KA_SK(2);
#undef KA_SK
    return 0;
}

static int check_target(const char* who, const SkinnyTarget& t, int K) {
    KA_CHECK(t.W && t.out, "%s: weight or output missing", who);
    KA_CHECK(t.N > 0 && t.ldw % 8 == 0 && t.ldw >= K && (uintptr_t)t.W % 16 == 0, "%s: weight rows must be 16-byte aligned and >= K", who);
    KA_CHECK(t.ldo >= t.N, "%s: output stride too small", who);
    KA_CHECK(t.act == 0 || t.act == 1, "%s: unknown activation %d", who, t.act);
    KA_CHECK(t.out_dtype == KA_F32 || t.out_dtype == KA_BF16, "%s: bad output type", who);
    KA_CHECK(!(t.accumulate && t.out_dtype != KA_F32), "%s: accumulate needs an fp32 output", who);
    return 0;
}

// The general entry point. Segments: A1 [M, K1] with W (target a) and optionally A2 [M, K2] with
// W2 (same rows as target a; not with a second target). ln_x non-null: A1 is replaced by
// LayerNorm(ln_x) (M <= 16, K1 % 4 == 0). Target b (Wb non-null) shares the input.
KA_API int ka_linear_skinny_fused(const void* A1, long lda1, int K1, const void* A2, long lda2, int K2,
                                  const void* W2, long ldw2, const float* bias2, const float* ln_x,
                                  const float* ln_gamma, const float* ln_beta, float ln_eps, const void* Wa,
                                  long ldwa, const float* biasa, void* outa, int out_dtype_a, long ldoa, int Na,
                                  int acta, int accumulate_a, const void* Wb, long ldwb, const float* biasb,
                                  void* outb, int out_dtype_b, long ldob, int Nb, int actb, int M,
                                  int target_waves, hipStream_t stream) {
    const char* who = "ka_linear_skinny_fused";
    KA_CHECK(M > 0 && M <= 64, "%s: M=%d outside 1..64", who, M);
    KA_CHECK(K1 > 0 && K1 % 8 == 0, "%s: K=%d must be a positive multiple of 8", who, K1);
    SkinnyArgs args = {};
    args.M = M;
    args.K[0] = K1;
    args.a = SkinnyTarget{(const bf16_t*)Wa, ldwa, biasa, outa, ldoa, out_dtype_a, Na, acta, accumulate_a};
    if (check_target(who, args.a, K1)) return -1;
    const bool ln = ln_x != nullptr;
    if (ln) {
        KA_CHECK(M <= SK_LN_ROWS, "%s: the LayerNorm prologue takes at most %d rows", who, SK_LN_ROWS);
        KA_CHECK(K1 <= SK_XV * KA_WAVE * 4, "%s: the LayerNorm prologue takes rows of at most %d", who, SK_XV * KA_WAVE * 4);
        KA_CHECK(ln_gamma && ln_eps >= 0.f && (uintptr_t)ln_x % 16 == 0 && (uintptr_t)ln_gamma % 16 == 0, "%s: LayerNorm operands", who);
        KA_CHECK(A2 == nullptr, "%s: no second segment with a LayerNorm prologue", who);
        args.ln_x = ln_x; args.ln_gamma = ln_gamma; args.ln_beta = ln_beta; args.ln_eps = ln_eps;
    } else {
        KA_CHECK(A1 && lda1 % 8 == 0 && lda1 >= K1 && (uintptr_t)A1 % 16 == 0, "%s: input rows must be 16-byte aligned and >= K", who);
        args.A[0] = (const bf16_t*)A1; args.lda[0] = lda1;
    }
    if (A2) {
        KA_CHECK(Wb == nullptr, "%s: two segments and two targets cannot be combined", who);
        KA_CHECK(K2 > 0 && K2 % 8 == 0 && lda2 % 8 == 0 && lda2 >= K2 && (uintptr_t)A2 % 16 == 0, "%s: second segment", who);
        KA_CHECK(W2 && ldw2 % 8 == 0 && ldw2 >= K2 && (uintptr_t)W2 % 16 == 0, "%s: second segment's weights", who);
        args.A[1] = (const bf16_t*)A2; args.lda[1] = lda2; args.K[1] = K2;
        args.W2 = (const bf16_t*)W2; args.ldw2 = ldw2; args.bias2 = bias2;
    }
    int strips = ka_cdiv(Na, SK_STRIP);
    args.strips_a = strips;
    if (Wb) {
        args.b = SkinnyTarget{(const bf16_t*)Wb, ldwb, biasb, outb, ldob, out_dtype_b, Nb, actb, 0};
        if (check_target(who, args.b, K1)) return -1;
        strips += ka_cdiv(Nb, SK_STRIP);
    }
    int MB = ka_cdiv(M, 16);
    int waves = ka_cdiv(target_waves, strips);
    int kblocks = ka_cdiv(K1 + (A2 ? K2 : 0), SK_KBLOCK);
    if (waves < 4) waves = 4;                 // fewer waves leave too few loads in flight per CU
    if (waves > kblocks) waves = kblocks;
    if (MB > 2 && waves > 8) waves = 8;       // LDS of the final sum grows with MB
    int rc;
    // Staging plain rows in LDS (the copy path of the kernel) is measured slower than fetching
    // them block by block, so only the LayerNorm prologue goes through LDS.
    size_t dyn = (size_t)M * (K1 + SK_PAD) * sizeof(bf16_t);
    const bool staged = ln;
    if (staged) {
        if (ln || waves < 4) waves = ln ? 8 : 4;     // one or two rows per wave keep a LayerNorm prologue short
        KA_CHECK(dyn <= 96 * 1024, "%s: %d rows of %d do not fit in LDS", who, M, K1);
        rc = launch_mb<1, true>(waves, strips, dyn, stream, args);
    } else {
        switch (MB) {
            case 1: rc = launch_mb<1, false>(waves, strips, 0, stream, args); break;
            case 2: rc = launch_mb<2, false>(waves, strips, 0, stream, args); break;
            case 3: rc = launch_mb<3, false>(waves, strips, 0, stream, args); break;
            default: rc = launch_mb<4, false>(waves, strips, 0, stream, args); break;
        }
    }
    if (rc) return rc;
    KA_LAUNCH_CHECK();
    return 0;
}

// One input, one weight matrix, one output.
KA_API int ka_linear_skinny_bf16(const void* A, long lda, const void* W, long ldw, const float* bias,
                                 void* out, int out_dtype, long ldo, int M, int N, int K, int act,
                                 int accumulate, int target_waves, hipStream_t stream) {
    return ka_linear_skinny_fused(A, lda, K, nullptr, 0, 0, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0.f, W,
                                  ldw, bias, out, out_dtype, ldo, N, act, accumulate, nullptr, 0, nullptr, nullptr, 0,
                                  0, 0, 0, M, target_waves, stream);
}
