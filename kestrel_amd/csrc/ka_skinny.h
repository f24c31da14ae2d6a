// What the skinny bf16 linear kernels (gemv_bf16.hip) are made of, and the persistent kernel as a
// function of (workgroup, workgroups), so that more than one kernel can hold it: the plain launch
// and the launch that runs it beside the decode attention (decode_beside.hip).
#pragma once
#include "ka_common.h"

#include <type_traits>
#include <utility>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int SK_STRIP = 8;        // weight rows per strip
constexpr int SK_KBLOCK = 64;      // k per wave and step
constexpr int SK_LN_ROWS = 16;     // most rows the LayerNorm prologue takes
constexpr int SK_XV = 8;           // float4 per lane of a row kept in registers: rows up to 2048 wide
constexpr int SK_XV_WIDE = 16;     // ... and up to 4096 wide, then without the scale and shift beside them
constexpr int SK_PAD = 8;          // bf16 of padding per LDS row (keeps 16-byte reads off each other's banks)
constexpr int SP_WAVES = 8;        // waves of a persistent workgroup
constexpr int SP_MAX_PER = 8;      // most k-blocks per wave it keeps activations for

// Orders the LDS traffic of one wave: what its lanes wrote before is seen by its lanes after.
__device__ __forceinline__ void sk_wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// bf16 of LDS in which a wave of the persistent kernel turns one k-block of MB * 16 rows around
// (rows padded so that the lanes of a 16-byte read stay off each other's banks).
__host__ __device__ constexpr int sk_stage_elements(int MB) { return MB * 16 * (SK_KBLOCK + SK_PAD); }

// Every operand lives in global memory. Saying so at the load matters: a pointer that went
// through sk_pinned() below is "generic" to the compiler, and generic (flat) loads count as LDS
// traffic too, which forces a wait for everything in flight at each use.
#define SK_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ bf16x8 sk_load8(const bf16_t* p) { return *(const SK_GLOBAL bf16x8*)p; }
// Weights are read once and never again: a load that does not displace the activations,
// which every workgroup of a CU reads, from the caches.
__device__ __forceinline__ bf16x8 sk_load8_stream(const bf16_t* p) {
    return __builtin_nontemporal_load((const SK_GLOBAL bf16x8*)p);
}

// A kernel argument that is chosen between two at run time (target a or b, segment 1 or 2)
// is pinned in scalar registers first: left alone, the compiler turns "choose one of two
// loaded arguments" into "load from the chosen address", a trip to memory on which every
// weight load of the round then depends.
template <typename T>
__device__ __forceinline__ T sk_pinned(T v) {
    asm volatile("" : "+s"(v));
    return v;
}

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N - 1>): a loop whose index is a
// constant inside the body (register arrays are indexed by it).
template <int N, typename F, int... I>
__device__ __forceinline__ void sk_static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void sk_static_for(F&& f) {
    sk_static_for_impl<N>(f, std::make_integer_sequence<int, N>{});
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
    bf16_t* ln_store;       // non-null: workgroup 0 also stores the normalised rows here, [M, K[0]] rows ln_store_ld apart
    long ln_store_ld;
    SkinnyTarget a, b;      // b.W null: one target
    int strips_a;
    int M;
};

// bias[n .. n + 3] without a branch around the loads (values past N are never used).
__device__ __forceinline__ floatx4 sk_bias4(const float* bias, int n, int N) {
    floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
    if (bias == nullptr) return v;
    if (N % 4 == 0 && (reinterpret_cast<uintptr_t>(bias) & 15) == 0) {     // n is a multiple of 4
        v = *(const SK_GLOBAL floatx4*)(bias + min(n, N - 4));
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = *(const SK_GLOBAL float*)(bias + min(n + i, N - 1));
    }
    return v;
}

// The finishing lanes (g in {0, 1}, r; with HALF r < 8) own out[m = mb * 16 + r][n0 + g * 4 + i]:
// they add the waves' partial sums in wave order, then bias / old value, activation, store.
// `mine(mb)` says whether the calling wave finishes block mb of 16 rows.
template <int MB, bool HALF, int NW, typename Mine>
__device__ __forceinline__ void sk_finish(const floatx4 (*red)[MB][KA_WAVE], const floatx4 (&addend)[MB],
                                          const SkinnyTarget& tg, int n0, int M, int lane, Mine mine) {
    const int r = lane % 16, g = lane / 16;
    // the other half of an output element: MFMA rows 8..15, and with HALF columns 8..15 as well
    constexpr int OTHER = HALF ? 40 : 32;
    const int n = n0 + g * 4;
    const bool whole = n + 3 < tg.N && tg.ldo % 4 == 0 && (reinterpret_cast<uintptr_t>(tg.out) & 15) == 0;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        if (!mine(mb)) continue;
        floatx4 s = addend[mb];
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[w][mb][lane] + red[w][mb][lane + OTHER];
        const int m = mb * 16 + r;
        if (m >= M) continue;
        if (ka_act_gated(tg.act)) {         // the four sums are two pairs of gate and value
            const float v[4] = {s[0], s[1], s[2], s[3]};
            ka_gated_store<true, 4>(tg.out, tg.out_dtype, tg.ldo, m, n, tg.N, v, tg.act);
            continue;
        }
        if (tg.act) {
#pragma unroll
            for (int i = 0; i < 4; ++i) s[i] = ka_activate_fast(tg.act, s[i]);
        }
        const size_t o = (size_t)m * tg.ldo + n;
        if (whole) {
            if (tg.out_dtype == KA_F32) {
                *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(tg.out) + o) = s;
            } else {
                bf16x4 y;
#pragma unroll
                for (int i = 0; i < 4; ++i) y[i] = (bf16_t)s[i];
                *reinterpret_cast<bf16x4*>(reinterpret_cast<bf16_t*>(tg.out) + o) = y;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (n + i >= tg.N) continue;
                if (tg.out_dtype == KA_F32) reinterpret_cast<float*>(tg.out)[o + i] = s[i];
                else reinterpret_cast<bf16_t*>(tg.out)[o + i] = (bf16_t)s[i];
            }
        }
    }
}

// LayerNorm of rows wave, wave + NW, ... of fp32 x [M, K] into LDS as bf16 [M][K + SK_PAD]
// (statistics in fp32, two passes over a row kept in registers: K <= SK_XV * 256).
// A row to be normalised, with the scale and shift that meet it: fetched in one trip to memory
// (sk_fetch_row) and turned into bf16 in LDS later (sk_normalise_row), so that other loads can
// be issued in between without standing in front of these in the wave's queue.
// (XV float4 per lane; EARLY: scale and shift come with the row, else they are read when the row
// is normalised: a second trip, to L2 by then, that rows of more than 2048 pay for their registers)
template <int XV, bool EARLY>
struct RowOperands {
    floatx4 x[XV], gamma[EARLY ? XV : 1], beta[EARLY ? XV : 1];
};

template <int XV, bool EARLY>
__device__ __forceinline__ void sk_fetch_row(const SkinnyArgs& p, int m, int lane, RowOperands<XV, EARLY>& row) {
    const int K = p.K[0];
    const float* src = p.ln_x + (size_t)m * K;
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        const int k = min((j * KA_WAVE + lane) * 4, K - 4);
        row.x[j] = *reinterpret_cast<const floatx4*>(src + k);
        if constexpr (EARLY) {
            row.gamma[j] = *reinterpret_cast<const floatx4*>(p.ln_gamma + k);
            row.beta[j] = p.ln_beta ? *reinterpret_cast<const floatx4*>(p.ln_beta + k) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
    }
}

template <int XV, bool EARLY>
__device__ __forceinline__ void sk_normalise_row(const SkinnyArgs& p, bf16_t* xs, int m, int lane, RowOperands<XV, EARLY>& row) {
    const int K = p.K[0], ld = K + SK_PAD;
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        if ((j * KA_WAVE + lane) * 4 >= K) row.x[j] = floatx4{0.f, 0.f, 0.f, 0.f};
        s += (row.x[j][0] + row.x[j][1]) + (row.x[j][2] + row.x[j][3]);
    }
    float mean = ka_wave_sum(s) / (float)K;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        if ((j * KA_WAVE + lane) * 4 < K) {
#pragma unroll
            for (int i = 0; i < 4; ++i) q += (row.x[j][i] - mean) * (row.x[j][i] - mean);
        }
    }
    float rstd = 1.0f / sqrtf(ka_wave_sum(q) / (float)K + p.ln_eps);
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        const int k = (j * KA_WAVE + lane) * 4;
        if (k < K) {
            floatx4 gm, bt;
            if constexpr (EARLY) {
                gm = row.gamma[j];
                bt = row.beta[j];
            } else {
                gm = *reinterpret_cast<const floatx4*>(p.ln_gamma + k);
                bt = p.ln_beta ? *reinterpret_cast<const floatx4*>(p.ln_beta + k) : floatx4{0.f, 0.f, 0.f, 0.f};
            }
            bf16x4 y;
#pragma unroll
            for (int i = 0; i < 4; ++i) y[i] = (bf16_t)((row.x[j][i] - mean) * rstd * gm[i] + bt[i]);
            *reinterpret_cast<bf16x4*>(xs + m * ld + k) = y;
        }
    }
}

// ----------------------------------------------------------------------------
// The persistent kernel: workgroup `block` of `grid` takes strips block, block + grid, ...
// EARLY: the scale and shift of the LayerNorm prologue are fetched with the row (a trip to memory
// less, 64 registers more).
// ----------------------------------------------------------------------------
template <int PER, int MB, bool HALF, bool LN, int DEPTH, bool EARLY>
__device__ __forceinline__ void skinny_persistent_body(const SkinnyArgs& p, const int total_strips, const int block, const int grid) {
    static_assert(!HALF || MB == 1, "the half-column form is for at most 8 rows");
    static_assert(!LN || MB == 1, "the LayerNorm prologue takes at most 16 rows");
    __shared__ floatx4 red[2][SP_WAVES][MB][KA_WAVE];
    extern __shared__ __attribute__((aligned(16))) unsigned char sk_dyn[];
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int K = p.K[0], M = p.M;
    const int koff = (r / 8) * 32 + g * 8;            // this lane's place inside a 64-wide k-block (weights)
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const int mine = (total_strips - block + grid - 1) / grid;      // strips of this workgroup, >= 1

    // where this lane reads its PER weight blocks of a row (an offset past K is moved inside:
    // the activations that meet it are zero)
    int wofs[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) wofs[u] = min((wave + u * SP_WAVES) * SK_KBLOCK + koff, K - 8);

    bf16x8 w[DEPTH][PER];
    floatx4 addend[DEPTH][MB];
    const bf16_t* const Wa = sk_pinned(p.a.W);
    const bf16_t* const Wb = sk_pinned(p.b.W);
    const long ldwa = sk_pinned(p.a.ldw), ldwb = sk_pinned(p.b.ldw);
    const int Na = sk_pinned(p.a.N), Nb = sk_pinned(p.b.N);
    const float* const biasa = sk_pinned(p.a.bias);
    const float* const biasb = sk_pinned(p.b.bias);
    const int strips_a = sk_pinned(p.strips_a);

    auto issue = [&](int slot, int i) {
        const int strip = block + i * grid;
        const bool second = strip >= strips_a;
        const bf16_t* W = second ? Wb : Wa;
        const long ldw = second ? ldwb : ldwa;
        const int N = second ? Nb : Na;
        const float* bias = second ? biasb : biasa;
        const int n0 = (second ? strip - strips_a : strip) * SK_STRIP;
        const bf16_t* wp = W + (size_t)min(n0 + r % 8, N - 1) * ldw;
#pragma unroll
        for (int u = 0; u < PER; ++u) w[slot][u] = sk_load8_stream(wp + wofs[u]);
        // what the finishing lanes add at the end comes with the strip's weights. Every lane
        // asks (a load under a branch would break the stream), but all except the finishing
        // lanes of the strip's finishing waves ask for the bias's first line, which costs nothing
        // (exactly one load whatever the bias is: the host sends biases that are not 16-byte
        // aligned or whose N is no multiple of 4 to the split kernel, and "no bias" reads a
        // line of the weights and throws it away)
        const bool finisher = (wave - i % SP_WAVES + SP_WAVES) % SP_WAVES < MB && lane < 32;
        const float* bp = bias ? bias + (finisher ? min(n0 + (g & 1) * 4, N - 4) : 0) : reinterpret_cast<const float*>(Wa);
        floatx4 b4 = *(const SK_GLOBAL floatx4*)bp;
        if (!bias) b4 = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) addend[slot][mb] = b4;
    };

    // The first strips' weights are on their way while the activations come in. A wave's loads
    // come back in the order in which it asked, so the row that it is to normalise is asked for
    // before the weights: the LayerNorm would otherwise wait for them.
    RowOperands<PER <= 4 ? SK_XV : SK_XV_WIDE, EARLY> row;
    if constexpr (LN) {
        if (wave < M) sk_fetch_row(p, wave, lane, row);
        __builtin_amdgcn_sched_barrier(0);
    }
    issue(0, 0);
    sk_static_for<DEPTH - 2>([&](auto d) {
        if (d.value + 1 < mine) issue(d.value + 1, d.value + 1);
    });

    // activations of this wave's k-blocks wave, wave + 8, ...: fetched (or normalised) once
    constexpr int XH = HALF ? 1 : 2;
    bf16x8 x[PER][MB][XH];
    if constexpr (LN) {
        bf16_t* xs = reinterpret_cast<bf16_t*>(sk_dyn);
        __builtin_amdgcn_sched_barrier(0);
        if (wave < M) sk_normalise_row(p, xs, wave, lane, row);
        for (int m = wave + SP_WAVES; m < M; m += SP_WAVES) {
            sk_fetch_row(p, m, lane, row);
            sk_normalise_row(p, xs, m, lane, row);
        }
        __syncthreads();
        const int ld = K + SK_PAD;
        if (p.ln_store != nullptr && block == 0) {
            // (every workgroup has normalised the same rows; one of them leaves them for later launches)
            for (int c = threadIdx.x; c < M * (K / 8); c += SP_WAVES * KA_WAVE) {
                const int m = c / (K / 8), k = (c % (K / 8)) * 8;
                *reinterpret_cast<bf16x8*>(p.ln_store + (size_t)m * p.ln_store_ld + k) = *reinterpret_cast<const bf16x8*>(xs + m * ld + k);
            }
        }
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int k = (wave + u * SP_WAVES) * SK_KBLOCK;
            if constexpr (HALF) {
                const int m = r % 8;
                x[u][0][0] = m < M && k + koff < K ? *reinterpret_cast<const bf16x8*>(xs + m * ld + k + koff) : zero;
            } else {
                const bf16_t* xp = xs + min(r, M - 1) * ld + k + g * 8;
                x[u][0][0] = r < M && k + g * 8 < K ? *reinterpret_cast<const bf16x8*>(xp) : zero;
                x[u][0][1] = r < M && k + 32 + g * 8 < K ? *reinterpret_cast<const bf16x8*>(xp + 32) : zero;
            }
        }
    } else if constexpr (!HALF) {
        // More than 8 rows: an instruction that loaded a k-block for the multiplications directly
        // would touch half a cache line of each of 16 rows, 4 KB apart, and every line twice
        // (10 us for 64 rows of 2048, most of this kernel's time before its first strip). Here an
        // instruction takes whole lines of 8 rows, and the wave turns what it has loaded into the
        // multiplications' order through a piece of LDS of its own, k-block by k-block.
        constexpr int LDR = SK_KBLOCK + SK_PAD;
        bf16_t* stage = reinterpret_cast<bf16_t*>(sk_dyn) + (size_t)wave * sk_stage_elements(MB);
        const int srow = lane / 8, schunk = lane % 8;
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int k = (wave + u * SP_WAVES) * SK_KBLOCK;
#pragma unroll
            for (int j = 0; j < 2 * MB; ++j)
                x[u][j / 2][j % 2] = sk_load8(p.A[0] + (size_t)min(j * 8 + srow, M - 1) * p.lda[0] + min(k + schunk * 8, K - 8));
        }
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int k = (wave + u * SP_WAVES) * SK_KBLOCK;
            sk_wave_sync();                    // the k-block before has been read
#pragma unroll
            for (int j = 0; j < 2 * MB; ++j)
                *reinterpret_cast<bf16x8*>(stage + (j * 8 + srow) * LDR + schunk * 8) = x[u][j / 2][j % 2];
            sk_wave_sync();
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const int m = mb * 16 + r;
                const bf16x8 va = *reinterpret_cast<const bf16x8*>(stage + m * LDR + g * 8);
                const bf16x8 vb = *reinterpret_cast<const bf16x8*>(stage + m * LDR + 32 + g * 8);
                x[u][mb][0] = m < M && k + g * 8 < K ? va : zero;
                x[u][mb][1] = m < M && k + 32 + g * 8 < K ? vb : zero;
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int k = (wave + u * SP_WAVES) * SK_KBLOCK;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                if constexpr (HALF) {
                    const int m = r % 8;
                    bf16x8 v = sk_load8(p.A[0] + (size_t)min(m, M - 1) * p.lda[0] + min(k + koff, K - 8));
                    x[u][mb][0] = m < M && k + koff < K ? v : zero;
                } else {
                    const int m = mb * 16 + r;
                    const bf16_t* ap = p.A[0] + (size_t)min(m, M - 1) * p.lda[0];
                    bf16x8 va = sk_load8(ap + min(k + g * 8, K - 8));
                    bf16x8 vb = sk_load8(ap + min(k + 32 + g * 8, K - 8));
                    x[u][mb][0] = m < M && k + g * 8 < K ? va : zero;
                    x[u][mb][1] = m < M && k + 32 + g * 8 < K ? vb : zero;
                }
            }
        }
    }

    const bool finishing_lane = lane < 32 && (!HALF || r < 8);

    auto compute = [&](int slot, int i) {
        floatx4 lo[MB], hi[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            lo[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
            hi[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int u = 0; u < PER; ++u) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                lo[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[slot][u], x[u][mb][0], lo[mb], 0, 0, 0);
                if constexpr (!HALF) hi[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[slot][u], x[u][mb][1], hi[mb], 0, 0, 0);
            }
        }
        const int buf = i & 1;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red[buf][wave][mb][lane] = HALF || g < 2 ? lo[mb] : hi[mb];
        // One barrier per strip is enough: a buffer is written again two strips later, after the
        // barrier of the strip between, which the finishing wave reaches only when it has read it.
        __syncthreads();
        // the strip's blocks of 16 rows are finished by waves i, i + 1, ... (mod 8), one each
        const int turn = (wave - i % SP_WAVES + SP_WAVES) % SP_WAVES;
        if (turn >= MB || !finishing_lane) return;
        const int strip = block + i * grid;
        const bool second = strip >= strips_a;
        const int n0 = (second ? strip - strips_a : strip) * SK_STRIP;
        sk_finish<MB, HALF, SP_WAVES>(red[buf], addend[slot], second ? p.b : p.a, n0, M, lane,
                                      [turn](int mb) { return mb == turn; });
    };

    // Strip i + DEPTH - 1 is asked for before strip i is multiplied. No load of the loop stands
    // under a condition, and the last strips are written out case by case (one case per number of
    // strips left) without any: the compiler can then wait for exactly the strip it needs and leave
    // the others in flight. Strip s lives in slot s % DEPTH.
    int i = 0;
    for (; i + 2 * DEPTH - 1 <= mine; i += DEPTH) {
        sk_static_for<DEPTH>([&](auto j) {
            issue((j.value + DEPTH - 1) % DEPTH, i + j.value + DEPTH - 1);
            compute(j.value, i + j.value);
        });
    }
    // strips i .. mine - 1 are left, of which the first min(left, DEPTH - 1) are on their way
    const int left = mine - i;
    sk_static_for<2 * DEPTH - 2>([&](auto c) {
        constexpr int LEFT = c.value + 1;
        if (left != LEFT) return;
        sk_static_for<LEFT>([&](auto j) {
            if constexpr (j.value + DEPTH - 1 < LEFT) issue((j.value + DEPTH - 1) % DEPTH, i + j.value + DEPTH - 1);
            compute(j.value % DEPTH, i + j.value);
        });
    });
}

// ----------------------------------------------------------------------------
// host side: checks that every launch of these kernels makes first
// ----------------------------------------------------------------------------
// Whether the persistent kernel takes these sizes and operands (it reads four bias values of a
// strip with one aligned load).
static inline bool persistent_bias_ok(const SkinnyTarget& t) {
    return t.W == nullptr || t.bias == nullptr || (t.N % 4 == 0 && (uintptr_t)t.bias % 16 == 0);
}
static inline int check_target(const char* who, const SkinnyTarget& t, int K) {
    KA_CHECK(t.W && t.out, "%s: weight or output missing", who);
    KA_CHECK(t.N > 0 && t.ldw % 8 == 0 && t.ldw >= K && (uintptr_t)t.W % 16 == 0, "%s: weight rows must be 16-byte aligned and >= K", who);
    KA_CHECK(ka_act_known(t.act), "%s: unknown activation %d", who, t.act);
    KA_CHECK(t.ldo >= ka_act_outputs(t.act, t.N), "%s: output stride too small", who);
    KA_CHECK(!ka_act_gated(t.act) || (t.N % 2 == 0 && !t.accumulate), "%s: a gated linear needs an even N and no accumulation", who);
    KA_CHECK(t.out_dtype == KA_F32 || t.out_dtype == KA_BF16, "%s: bad output type", who);
    KA_CHECK(!(t.accumulate && t.out_dtype != KA_F32), "%s: accumulate needs an fp32 output", who);
    return 0;
}
