// Skinny bf16 linear layers for decoding (M <= 64 rows): out = act(A W^T + bias).
//
// The weight matrix is streamed from HBM exactly once, and nothing is exchanged between
// workgroups (no fences, no atomics: on a part with eight L2s they cost more than the whole
// product). The unit of work is a strip of 8 weight rows over all of K; the waves of a
// workgroup take interleaved 64-wide k-blocks of it and add up through LDS in wave order, so the
// result is the same on every run. 8 rows rather than the MFMA's 16 give N / 8 strips, enough
// to fill 256 CUs at N = 2048. v_mfma_f32_16x16x32_bf16 wants 16 row-operand rows: rows 0..7
// carry the strip's k-block [k, k + 32), rows 8..15 the same weight rows' [k + 32, k + 64), so
// every lane's 16-byte load is useful. Two MFMAs per block then multiply with the activations
// of the first and of the second half; rows 0..7 of the first and rows 8..15 of the second are
// the wanted sums, the other halves are never read. With at most 8 rows of activations (HALF)
// the activations play the same trick: MFMA columns 0..7 carry the rows' [k, k + 32), columns
// 8..15 their [k + 32, k + 64); one MFMA and one activation load per block, and the wanted sums
// are the two diagonal 8 x 8 quarters of the result.
//
// Every load of the inner loops is unconditional: an address that would fall outside is moved
// to the last valid place of the same row and the activation that multiplies it is zero. A
// load under a branch makes the compiler wait for ALL loads in flight before the next MFMA,
// and the loop then pays a trip to memory per round instead of streaming.
//
// Two kernels:
//  * persistent (one K-segment, K up to 64 * 8 * 8): a workgroup loads its share of the
//    activations into registers ONCE (normalising fp32 rows itself if asked to: the LayerNorm
//    prologue) and then walks over strips blockIdx.x, + gridDim.x, ...: only weights are
//    fetched inside the loop, one or two strips ahead of the arithmetic;
//  * split (any K, two K-segments into one output: out += A1 W1^T + A2 W2^T + b1 + b2, the
//    attention output projection and the second feed-forward linear of a parallel block in one
//    pass): one strip per workgroup, up to 16 waves over K, rounds of blocks double-buffered.
// Both take two targets (strips of W_a, then strips of W_b, from the same input): the fused
// q|k|v projection and the first feed-forward linear.
#include "ka_skinny.h"
#include "ka_partials.h"

// ----------------------------------------------------------------------------
// The persistent kernel (its body: ka_skinny.h).
// ----------------------------------------------------------------------------
template <int PER, int MB, bool HALF, bool LN, int DEPTH>
__global__ void __launch_bounds__(SP_WAVES * KA_WAVE)
skinny_persistent_kernel(SkinnyArgs p, int total_strips) {
    skinny_persistent_body<PER, MB, HALF, LN, DEPTH, PER <= 4>(p, total_strips, blockIdx.x, gridDim.x);
}

// ----------------------------------------------------------------------------
// The split kernel: one strip per workgroup, WAVES waves over the k-blocks of both segments.
// ----------------------------------------------------------------------------
template <int MB, int WAVES, bool HALF>
__global__ void __launch_bounds__(WAVES * KA_WAVE)
skinny_split_kernel(SkinnyArgs p) {
    static_assert(!HALF || MB == 1, "the half-column form is for at most 8 rows");
    __shared__ floatx4 red[WAVES][MB][KA_WAVE];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / KA_WAVE), lane = threadIdx.x % KA_WAVE;
    const int r = lane % 16, g = lane / 16;
    const bool second = (int)blockIdx.x >= p.strips_a;
    const SkinnyTarget& tg = second ? p.b : p.a;
    const int n0 = (second ? blockIdx.x - p.strips_a : blockIdx.x) * SK_STRIP;
    const int M = p.M, N = tg.N;
    const int koff = (r / 8) * 32 + g * 8;
    const size_t wrow = (size_t)min(n0 + r % 8, N - 1);
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

    // What the finishing lanes add at the end (biases, and the output's old value when the
    // product is accumulated) is fetched first: its latency hides behind the weight stream.
    floatx4 addend[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) addend[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    const bool finishing_lane = wave == 0 && lane < 32 && (!HALF || r < 8);
    if (finishing_lane) {
        floatx4 b4 = sk_bias4(tg.bias, n0 + g * 4, N);
        if (!second && p.bias2) b4 += sk_bias4(p.bias2, n0 + g * 4, N);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            addend[mb] = b4;
            // the old values of a row are read like a bias (rows and columns past the end are
            // moved inside and never used)
            if (tg.accumulate)
                addend[mb] += sk_bias4(reinterpret_cast<const float*>(tg.out) + (size_t)min(mb * 16 + r, M - 1) * tg.ldo,
                                       n0 + g * 4, N);
        }
    }

    const int nb1 = (p.K[0] + SK_KBLOCK - 1) / SK_KBLOCK;
    const int nb = nb1 + (p.A[1] ? (p.K[1] + SK_KBLOCK - 1) / SK_KBLOCK : 0);
    constexpr int UN = MB == 1 ? 4 : MB == 2 ? 2 : 1;      // blocks of a round
    constexpr int XH = HALF ? 1 : 2;
    const int rounds = (nb + WAVES * UN - 1) / (WAVES * UN);

    bf16x8 w[2][UN], x[2][UN][MB][XH];
    floatx4 lo[MB], hi[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        lo[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
        hi[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // this lane's rows of the weights and of the activations, per segment (the second segment's
    // are never followed when there is none)
    const int K0 = sk_pinned(p.K[0]), K1 = sk_pinned(p.K[1]);
    const bf16_t* const wrow0 = tg.W + wrow * tg.ldw;
    const bf16_t* const wrow1 = p.W2 + wrow * p.ldw2;
    const bf16_t* arow0[MB];
    const bf16_t* arow1[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = min(HALF ? r % 8 : mb * 16 + r, M - 1);
        arow0[mb] = p.A[0] + (size_t)m * p.lda[0];
        arow1[mb] = p.A[1] + (size_t)m * p.lda[1];
    }

    // (a round's weights are all asked for before its activations: the weights come from HBM, the
    // activations, which every workgroup reads, from L2)
    auto issue = [&](int slot, int round) {
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            // a block past the end reads the last one again and multiplies it with zeros
            const int bc = min(wave + (round * UN + u) * WAVES, nb - 1);
            const bool seg = bc >= nb1;
            const int Ks = seg ? K1 : K0;
            const int k = (seg ? bc - nb1 : bc) * SK_KBLOCK;
            const bf16_t* wp = seg ? wrow1 : wrow0;
            w[slot][u] = sk_load8_stream(wp + min(k + koff, Ks - 8));
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int b = wave + (round * UN + u) * WAVES;
            const bool live = b < nb;
            const int bc = min(b, nb - 1);
            const bool seg = bc >= nb1;
            const int Ks = seg ? K1 : K0;
            const int k = (seg ? bc - nb1 : bc) * SK_KBLOCK;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const bf16_t* ap = seg ? arow1[mb] : arow0[mb];
                if constexpr (HALF) {
                    const int m = r % 8;
                    bf16x8 v = sk_load8(ap + min(k + koff, Ks - 8));
                    x[slot][u][mb][0] = live && m < M && k + koff < Ks ? v : zero;
                } else {
                    const int m = mb * 16 + r;
                    bf16x8 va = sk_load8(ap + min(k + g * 8, Ks - 8));
                    bf16x8 vb = sk_load8(ap + min(k + 32 + g * 8, Ks - 8));
                    x[slot][u][mb][0] = live && m < M && k + g * 8 < Ks ? va : zero;
                    x[slot][u][mb][1] = live && m < M && k + 32 + g * 8 < Ks ? vb : zero;
                }
            }
        }
    };
    auto compute = [&](int slot) {
#pragma unroll
        for (int u = 0; u < UN; ++u) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                lo[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[slot][u], x[slot][u][mb][0], lo[mb], 0, 0, 0);
                if constexpr (!HALF) hi[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[slot][u], x[slot][u][mb][1], hi[mb], 0, 0, 0);
            }
        }
    };

    // round i + 1 is asked for before round i is multiplied; the tail is written out so that no
    // load of the loop stands under a condition
    issue(0, 0);
    int i = 0;
    for (; i + 2 < rounds; i += 2) {
        issue(1, i + 1);
        compute(0);
        issue(0, i + 2);
        compute(1);
    }
    if (rounds - i == 2) {
        issue(1, i + 1);
        compute(0);
        compute(1);
    } else {
        compute(0);
    }

#pragma unroll
    for (int mb = 0; mb < MB; ++mb) red[wave][mb][lane] = HALF || g < 2 ? lo[mb] : hi[mb];
    __syncthreads();
    if (!finishing_lane) return;
    sk_finish<MB, HALF, WAVES>(red, addend, tg, n0, M, lane, [](int) { return true; });
}

// ----------------------------------------------------------------------------
// The wide kernel, for 17 to 64 rows. With that many rows the activations are what the kernels
// above read most of: every strip of 8 weight rows meets all of them, from L2. Here a workgroup
// of eight waves takes eight neighbouring strips and a part of K, brings the activations of that
// part into LDS once (in chunks of 256 k, two buffers in turn) and every
// wave multiplies its own strip with them; the parts of K meet in fp32 partial sums that a
// second kernel adds up, in the order of the parts, with bias, activation and the output's old
// value. Nothing crosses between workgroups inside a launch.
//
// LDS layout of a chunk: row m is 512 bytes, its 16-byte unit u lies at place u ^ (m & 15): the
// 16 lanes that one pass of an MFMA operand read serves (16 rows, the same unit) then fall on 16
// different bank groups.
// ----------------------------------------------------------------------------
constexpr int WD_WAVES = 8;        // strips of a workgroup
constexpr int WD_CB = 4;           // k-blocks of a chunk
constexpr int WD_DEPTH = 2;        // chunks of weights in flight per wave
constexpr int WD_ROW_BYTES = WD_CB * SK_KBLOCK * 2;

struct WideArgs {
    const bf16_t* A[2];     // [M, K[s]] per segment (A[1] null: one segment)
    long lda[2];
    const bf16_t* W[2];     // [N, K[s]]
    long ldw[2];
    int K[2];
    int M, N, splits;
    float* partial;         // [splits, M, N]
};

// (Two workgroups per CU, which is what hides the trips to memory: at most 128 registers.)
template <int MB>
__global__ void __launch_bounds__(WD_WAVES * KA_WAVE) __attribute__((amdgpu_waves_per_eu(4, 4)))
skinny_wide_kernel(WideArgs p) {
    constexpr int ROWS = MB * 16;
    constexpr int XL = ROWS / 2 / WD_WAVES;            // loads of two rows per wave and chunk
    static_assert(XL * 2 * WD_WAVES == ROWS, "the rows of a chunk divide over the waves' loads");
    __shared__ __attribute__((aligned(16))) unsigned char xs[2][ROWS * WD_ROW_BYTES];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / KA_WAVE), lane = threadIdx.x % KA_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int M = p.M, N = p.N;
    const int split = blockIdx.y;
    const int n0 = (blockIdx.x * WD_WAVES + wave) * SK_STRIP;
    const int koff = (r / 8) * 32 + g * 8;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const int K0 = sk_pinned(p.K[0]), K1 = sk_pinned(p.K[1]);

    // this part's k-blocks of each segment, and its chunks: segment 0's first
    int kb_lo[2], kb_hi[2], chunks[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int nb = p.A[s] ? ((s ? K1 : K0) + SK_KBLOCK - 1) / SK_KBLOCK : 0;
        const int per = (nb + p.splits - 1) / p.splits;
        kb_lo[s] = min(split * per, nb);
        kb_hi[s] = min(kb_lo[s] + per, nb);
        chunks[s] = (kb_hi[s] - kb_lo[s] + WD_CB - 1) / WD_CB;
    }
    const int n_chunks = chunks[0] + chunks[1];

    const size_t wrow = (size_t)min(n0 + r % 8, N - 1);
    const bf16_t* const wrow0 = p.W[0] + wrow * p.ldw[0];
    const bf16_t* const wrow1 = p.A[1] ? p.W[1] + wrow * p.ldw[1] : wrow0;
    // what this lane brings of a chunk's activations: of the two rows 2 * (wave * XL + i) + lane / 32
    // the unit lane % 32, which goes to place unit ^ (row & 15)
    const bf16_t* const a0 = sk_pinned(p.A[0]);
    const bf16_t* const a1 = sk_pinned(p.A[1] ? p.A[1] : p.A[0]);
    const long lda0 = sk_pinned(p.lda[0]), lda1 = sk_pinned(p.A[1] ? p.lda[1] : p.lda[0]);
    int xm[XL], xplace[XL];
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        const int m = (wave * XL + i) * 2 + lane / 32;
        xplace[i] = m * WD_ROW_BYTES + (((lane % 32) ^ (m & 15)) * 16);
        xm[i] = min(m, M - 1);
    }

    // Where chunk c lies: first k-block, end of the part, segment. A chunk past the end is the
    // last one again: every load below is issued in every round, under no condition, so that the
    // compiler's counts of loads in flight are exact.
    auto chunk_of = [&](int c, int& kb, int& kb_end, int& seg) {
        const int cc = max(min(c, n_chunks - 1), 0);
        seg = chunks[1] > 0 && cc >= chunks[0];
        kb = kb_lo[seg] + (seg ? cc - chunks[0] : cc) * WD_CB;
        kb_end = c < n_chunks ? kb_hi[seg] : kb;
    };
    bf16x8 xr[XL];
    auto fetch_x = [&](int c) {
        int kb, kb_end, seg;
        chunk_of(c, kb, kb_end, seg);
        const int Ks = seg ? K1 : K0;
#pragma unroll
        for (int i = 0; i < XL; ++i)
            xr[i] = sk_load8((seg ? a1 : a0) + ((size_t)xm[i] * (seg ? lda1 : lda0) + min(kb * SK_KBLOCK + (lane % 32) * 8, Ks - 8)));
    };
    // activations past the part's end or past the end of K go to LDS as zeros (the weights that
    // meet them are then some other place of their row)
    auto store_x = [&](int buf, int c) {
        int kb, kb_end, seg;
        chunk_of(c, kb, kb_end, seg);
        const int k = kb * SK_KBLOCK + (lane % 32) * 8;
        const bool ok = k < min(kb_end * SK_KBLOCK, seg ? K1 : K0);
#pragma unroll
        for (int i = 0; i < XL; ++i) *reinterpret_cast<bf16x8*>(xs[buf] + xplace[i]) = ok ? xr[i] : zero;
    };
    bf16x8 w[WD_DEPTH][WD_CB];
    auto fetch_w = [&](int slot, int c) {
        int kb, kb_end, seg;
        chunk_of(c, kb, kb_end, seg);
        const int Ks = seg ? K1 : K0;
        const bf16_t* wp = seg ? wrow1 : wrow0;
#pragma unroll
        for (int j = 0; j < WD_CB; ++j) w[slot][j] = sk_load8_stream(wp + min((kb + j) * SK_KBLOCK + koff, Ks - 8));
    };

    floatx4 lo[MB], hi[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        lo[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
        hi[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    auto compute = [&](int buf, int slot) {
        const unsigned char* base = xs[buf];
#pragma unroll
        for (int j = 0; j < WD_CB; ++j) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const int m = mb * 16 + r;
                const bf16x8 xlo = *reinterpret_cast<const bf16x8*>(base + m * WD_ROW_BYTES + (((j * 8 + g) ^ r) * 16));
                const bf16x8 xhi = *reinterpret_cast<const bf16x8*>(base + m * WD_ROW_BYTES + (((j * 8 + 4 + g) ^ r) * 16));
                lo[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[slot][j], xlo, lo[mb], 0, 0, 0);
                hi[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[slot][j], xhi, hi[mb], 0, 0, 0);
            }
        }
    };
    // LDS writes of this wave done, then everybody's: what the barrier of __syncthreads() would
    // do too, but that one also waits for every load in flight
    auto lds_barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(0xc07f);      // lgkmcnt(0), the other counters at their maximum
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // Weights run up to WD_DEPTH chunks ahead (in registers), activations one (in registers
    // during the products of the chunk before, then in the LDS buffer that those products have
    // left: the barrier at the head of the round says that all waves have).
    fetch_x(0);
#pragma unroll
    for (int d = 0; d < WD_DEPTH; ++d) fetch_w(d, d);
    store_x(0, 0);
    for (int c = 0; c < n_chunks; c += WD_DEPTH) {
#pragma unroll
        for (int d = 0; d < WD_DEPTH; ++d) {
            if (c + d >= n_chunks) break;                 // (uniform; no load stands behind it)
            lds_barrier();
            fetch_x(c + d + 1);
            compute((c + d) & 1, d);
            fetch_w(d, c + d + WD_DEPTH);
            store_x((c + d + 1) & 1, c + d + 1);
        }
    }

    // rows 0..7 of the strip are in lo of the lanes g < 2, rows 8..15 (the other half of every
    // k-block) in hi of the lanes g >= 2: they meet in the lanes g < 2
    float* mine = p.partial + (size_t)split * M * N;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        floatx4 v = g < 2 ? lo[mb] : hi[mb];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = ka_lanes_reduce<32, KA_WAVE>(v[i], KaSum{});
        const int m = mb * 16 + r, n = n0 + g * 4;
        if (g < 2 && m < M) {
            float* dst = mine + (size_t)m * N + n;
            if (n + 3 < N && (N % 4) == 0) *reinterpret_cast<floatx4*>(dst) = v;
            else
                for (int i = 0; i < 4 && n + i < N; ++i) dst[i] = v[i];
        }
    }
}

// ----------------------------------------------------------------------------
// Host side
// ----------------------------------------------------------------------------
static int sk_compute_units() { return ka_compute_units(); }

// The persistent kernel is used wherever it fits; switching it off is for measurements and for
// tests of the split kernel on sizes that it otherwise never sees.
static int sk_persistent_enabled = 1;
KA_API void ka_skinny_set_persistent(int enabled) { sk_persistent_enabled = enabled; }
// The wide kernel (17 to 64 rows, activations through LDS, parts of K in scratch memory): 1 where
// it was measured faster, which is with two K-segments (a K too long for the persistent kernel's
// registers: 30 against 48 us for Moondream 2's output projection + fc2 at 64 rows; one segment
// of 2048: 21 against 15 us), 2 wherever it can run (for tests), 0 nowhere.
static int sk_wide_enabled = 1;
KA_API int ka_linear_skinny_pair_in_parts(int M, int N);
KA_API void ka_skinny_set_wide(int enabled) { sk_wide_enabled = enabled; }

template <int PER, int MB, bool HALF, bool LN>
static int launch_persistent_one(int grid, size_t dyn, int strips, hipStream_t stream, const SkinnyArgs& args) {
    // two strips ahead where one workgroup has a CU (and its registers) to itself (three, which the
    // registers would still hold, were measured slower: 6.56k against 6.72k tok/s at batch 8; for five
    // k-blocks a wave, K = 2560, likewise: 523 against 537 tok/s at one row)
    constexpr int DEPTH = LN && PER <= 4 ? 3 : 2;
    if (dyn > 0) {
        static size_t reserved = 0;
        if (dyn > reserved) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(skinny_persistent_kernel<PER, MB, HALF, LN, DEPTH>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);
            KA_CHECK(e == hipSuccess, "skinny linear: cannot reserve %zu bytes of LDS", dyn);
            reserved = dyn;
        }
    }
    hipLaunchKernelGGL((skinny_persistent_kernel<PER, MB, HALF, LN, DEPTH>), dim3(grid), dim3(SP_WAVES * KA_WAVE), dyn,
                       stream, args, strips);
    return 0;
}

template <int MB, bool HALF, bool LN>
static int launch_persistent_per(int per, int grid, size_t dyn, int strips, hipStream_t stream, const SkinnyArgs& args) {
    if (per <= 1) return launch_persistent_one<1, MB, HALF, LN>(grid, dyn, strips, stream, args);
    if (per <= 2) return launch_persistent_one<2, MB, HALF, LN>(grid, dyn, strips, stream, args);
    if (per <= 4) return launch_persistent_one<4, MB, HALF, LN>(grid, dyn, strips, stream, args);
    if constexpr (MB == 1) {
        // (a wave's k-blocks beyond K are loaded from inside and multiplied with zeros: a K of 2560, five blocks
        // a wave, took 26.6 us in the form for eight where the form for five takes its share of them)
        if (per <= 5) return launch_persistent_one<5, MB, HALF, LN>(grid, dyn, strips, stream, args);
        if (per <= 6) return launch_persistent_one<6, MB, HALF, LN>(grid, dyn, strips, stream, args);
        return launch_persistent_one<8, MB, HALF, LN>(grid, dyn, strips, stream, args);
    } else {
        if (per <= 5) return launch_persistent_one<5, MB, HALF, LN>(grid, dyn, strips, stream, args);
    }
    return 1;
}

// Most k-blocks a wave keeps activations for when there are more than 16 rows of them: K up to 2560 (at 64 rows
// the form for five blocks fills a lane's 256 registers and spills five of them).
constexpr int SP_MAX_PER_MANY_ROWS = 5;

static bool persistent_fits(int M, int kblocks, const SkinnyArgs& args) {
    const int per = ka_cdiv(kblocks, SP_WAVES);
    return per <= (M <= 16 ? SP_MAX_PER : SP_MAX_PER_MANY_ROWS) && persistent_bias_ok(args.a) && persistent_bias_ok(args.b);
}

static int launch_persistent(int strips, int M, int kblocks, bool ln, size_t dyn, hipStream_t stream,
                             const SkinnyArgs& args) {
    const int per = ka_cdiv(kblocks, SP_WAVES);
    const int MB = ka_cdiv(M, 16);
    // workgroups: as many as the chip holds at once (two of 8 waves per CU while registers
    // allow), cut so that every one walks over the same number of strips
    const bool two = MB <= 1 && per <= 4 && !ln;      // the LayerNorm prologue's registers leave room for one
    const int slots = sk_compute_units() * (two ? 2 : 1);
    const int rounds = ka_cdiv(strips, slots);
    const int grid = ka_cdiv(strips, rounds);
    if (ln) {
        if (M <= 8) return launch_persistent_per<1, true, true>(per, grid, dyn, strips, stream, args);
        return launch_persistent_per<1, false, true>(per, grid, dyn, strips, stream, args);
    }
    if (M <= 8) return launch_persistent_per<1, true, false>(per, grid, 0, strips, stream, args);
    switch (MB) {
        // (LDS in which every wave turns the activations it loads into the multiplications' order)
        case 1: return launch_persistent_per<1, false, false>(per, grid, SP_WAVES * sk_stage_elements(1) * sizeof(bf16_t), strips, stream, args);
        case 2: return launch_persistent_per<2, false, false>(per, grid, SP_WAVES * sk_stage_elements(2) * sizeof(bf16_t), strips, stream, args);
        case 3: return launch_persistent_per<3, false, false>(per, grid, SP_WAVES * sk_stage_elements(3) * sizeof(bf16_t), strips, stream, args);
        default: return launch_persistent_per<4, false, false>(per, grid, SP_WAVES * sk_stage_elements(4) * sizeof(bf16_t), strips, stream, args);
    }
}

template <int MB, bool HALF>
static int launch_split(int waves, int strips, hipStream_t stream, const SkinnyArgs& args) {
    // (rounded to the nearest of 4, 8 and 16)
    if (waves >= 12) {
        if constexpr (HALF) {      // 16 waves leave 128 registers a lane: enough only for the half-column form
            hipLaunchKernelGGL((skinny_split_kernel<MB, 16, HALF>), dim3(strips), dim3(16 * KA_WAVE), 0, stream, args);
            return 0;
        }
    }
    if (waves >= 6) hipLaunchKernelGGL((skinny_split_kernel<MB, 8, HALF>), dim3(strips), dim3(8 * KA_WAVE), 0, stream, args);
    else hipLaunchKernelGGL((skinny_split_kernel<MB, 4, HALF>), dim3(strips), dim3(4 * KA_WAVE), 0, stream, args);
    return 0;
}

// The general entry point. Segments: A1 [M, K1] with W (target a) and optionally A2 [M, K2] with
// W2 (same rows as target a; not with a second target). ln_x non-null: A1 is replaced by
// LayerNorm(ln_x) (M <= 16, K1 <= 2048). Target b (Wb non-null) shares the input.
struct SkinnyExtras {                 // what only some callers of skinny_fused bring
    const KaThenNorm* then = nullptr; // a norm of the finished rows
    void* ln_store = nullptr;         // where the LayerNorm prologue also leaves its normalised rows (bf16)
    long ln_store_ld = 0;
};

static int skinny_fused(const SkinnyExtras& extras, const void* A1, long lda1, int K1, const void* A2, long lda2, int K2,
                                  const void* W2, long ldw2, const float* bias2, const float* ln_x,
                                  const float* ln_gamma, const float* ln_beta, float ln_eps, const void* Wa,
                                  long ldwa, const float* biasa, void* outa, int out_dtype_a, long ldoa, int Na,
                                  int acta, int accumulate_a, const void* Wb, long ldwb, const float* biasb,
                                  void* outb, int out_dtype_b, long ldob, int Nb, int actb, int M,
                                  int target_waves, float* partials, long partial_floats, hipStream_t stream) {
    const char* who = "ka_linear_skinny_fused";
    const KaThenNorm* then = extras.then;
    KA_CHECK(M > 0 && M <= 64, "%s: M=%d outside 1..64", who, M);
    KA_CHECK(K1 > 0 && K1 % 8 == 0, "%s: K=%d must be a positive multiple of 8", who, K1);
    if (then) {
        KA_CHECK(out_dtype_a == KA_F32 && acta == KA_ACT_NONE && Wb == nullptr, "%s: a norm can follow one fp32 output without activation only", who);
        KA_CHECK(ka_then_norm_fits(Na), "%s: a norm cannot follow rows of %d (multiples of 4 up to %d)", who, Na, KA_ROW_THREADS * 4 * KA_ROW_QUADS);
        KA_CHECK(then->gamma && then->out && then->ld >= Na && ldoa % 4 == 0 && then->ld % 4 == 0 && (uintptr_t)outa % 16 == 0 &&
                     (uintptr_t)then->gamma % 16 == 0 && (uintptr_t)then->beta % 16 == 0 && (uintptr_t)then->out % 8 == 0 &&
                     (uintptr_t)biasa % 16 == 0 && (uintptr_t)bias2 % 16 == 0,
                 "%s: the operands of the norm that follows must be aligned to four elements", who);
        KA_CHECK(then->out_dtype == KA_F32 || then->out_dtype == KA_BF16, "%s: bad type of the normalised rows", who);
    }
    SkinnyArgs args = {};
    args.M = M;
    args.K[0] = K1;
    args.a = SkinnyTarget{(const bf16_t*)Wa, ldwa, biasa, outa, ldoa, out_dtype_a, Na, acta, accumulate_a};
    if (check_target(who, args.a, K1)) return -1;
    const bool ln = ln_x != nullptr;
    if (ln) {
        KA_CHECK(M <= SK_LN_ROWS, "%s: the LayerNorm prologue takes at most %d rows", who, SK_LN_ROWS);
        KA_CHECK(K1 <= SK_XV_WIDE * KA_WAVE * 4, "%s: the LayerNorm prologue takes rows of at most %d", who, SK_XV_WIDE * KA_WAVE * 4);
        KA_CHECK(ln_gamma && ln_eps >= 0.f && (uintptr_t)ln_x % 16 == 0 && (uintptr_t)ln_gamma % 16 == 0 &&
                     (uintptr_t)ln_beta % 16 == 0, "%s: LayerNorm operands must be 16-byte aligned", who);
        KA_CHECK(A2 == nullptr && !accumulate_a, "%s: no second segment and no accumulation with a LayerNorm prologue", who);
        args.ln_x = ln_x; args.ln_gamma = ln_gamma; args.ln_beta = ln_beta; args.ln_eps = ln_eps;
        if (extras.ln_store) {
            KA_CHECK(extras.ln_store_ld >= K1 && extras.ln_store_ld % 8 == 0 && (uintptr_t)extras.ln_store % 16 == 0,
                     "%s: the stored normalised rows must be 16-byte aligned and >= K apart", who);
            args.ln_store = (bf16_t*)extras.ln_store; args.ln_store_ld = extras.ln_store_ld;
        }
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
    const int MB = ka_cdiv(M, 16);
    const int kblocks = ka_cdiv(K1, SK_KBLOCK) + (A2 ? ka_cdiv(K2, SK_KBLOCK) : 0);
    if (ln) {
        const size_t dyn = (size_t)M * (K1 + SK_PAD) * sizeof(bf16_t);
        KA_CHECK(dyn <= 96 * 1024, "%s: %d rows of %d do not fit in LDS", who, M, K1);
        KA_CHECK(persistent_fits(M, kblocks, args), "%s: K=%d or the biases do not suit the LayerNorm prologue", who, K1);
        if (launch_persistent(strips, M, kblocks, true, dyn, stream, args)) return -1;
        KA_LAUNCH_CHECK();
        return 0;
    }
    // More than 16 rows of a K too long for the persistent kernel's registers: the split kernel
    // would read all activations from L2 once per strip (78 us for 48 rows, K = 2560, N = 17920;
    // the wide kernel shares them through LDS). Two targets go one after the other.
    const bool persistent_ok = !A2 && !accumulate_a && sk_persistent_enabled && persistent_fits(M, kblocks, args);
    if (M > 16 && Wb && partials && sk_wide_enabled && !persistent_ok) {
        int rc = skinny_fused(SkinnyExtras{}, A1, lda1, K1, nullptr, 0, 0, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0.f,
                                        Wa, ldwa, biasa, outa, out_dtype_a, ldoa, Na, acta, accumulate_a, nullptr, 0,
                                        nullptr, nullptr, 0, 0, 0, 0, M, target_waves, partials, partial_floats, stream);
        if (rc) return rc;
        return skinny_fused(SkinnyExtras{}, A1, lda1, K1, nullptr, 0, 0, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0.f,
                                      Wb, ldwb, biasb, outb, out_dtype_b, ldob, Nb, actb, 0, nullptr, 0, nullptr,
                                      nullptr, 0, 0, 0, 0, M, target_waves, partials, partial_floats, stream);
    }
    // Up to 16 rows of two segments: where there are more strips than CUs the split kernel,
    // which gives a strip to a workgroup, takes about twice the time that it takes with one
    // strip a CU (N = 2560, K = 2560 + 10240, 16 rows: 40 us; 25 us here).
    // With more than 8 rows of two segments the split kernel reads twice the weights' bytes in
    // activations (it multiplies 16 rows with strips of 8): 16.4 us here against 17.7 at 12 rows and
    // 18.3 at 16 (N = 2048, K = 2048 + 8192).
    const bool crowded = A2 && M <= 16 && ka_linear_skinny_pair_in_parts(M, Na);      // (a single row: 19 us against 24)
    if (!Wb && partials && ((sk_wide_enabled && (M > 16 ? (A2 || !persistent_ok) : crowded)) || sk_wide_enabled >= 2)) {
        WideArgs wide = {};
        wide.A[0] = args.A[0]; wide.lda[0] = args.lda[0]; wide.W[0] = args.a.W; wide.ldw[0] = args.a.ldw; wide.K[0] = K1;
        if (A2) { wide.A[1] = args.A[1]; wide.lda[1] = args.lda[1]; wide.W[1] = args.W2; wide.ldw[1] = args.ldw2; wide.K[1] = K2; }
        wide.M = M; wide.N = Na; wide.partial = partials;
        // parts of K: as many as give every CU one workgroup and none a second (measured at N = 2048,
        // K = 2048 + 8192, 32 groups of strips: 8 parts 18.1 us at 32 rows and 19.6 at 64, finishing
        // kernel included; 6 parts 21.4 and 22.3, 10 parts 22.6 and 27.4, 16 parts 21.1 and 25.1),
        // every part at least two chunks
        const int groups = ka_cdiv(Na, WD_WAVES * SK_STRIP);
        int splits = sk_compute_units() / groups;
        if (splits < 1) splits = 1;
        if (splits > ka_cdiv(kblocks, 2 * WD_CB)) splits = ka_cdiv(kblocks, 2 * WD_CB);
        while (splits > 1 && (long)splits * M * Na > partial_floats) --splits;
        if ((long)splits * M * Na <= partial_floats) {
            wide.splits = splits;
            dim3 grid(groups, splits);
            switch (MB) {
                case 1: hipLaunchKernelGGL(skinny_wide_kernel<1>, grid, dim3(WD_WAVES * KA_WAVE), 0, stream, wide); break;
                case 2: hipLaunchKernelGGL(skinny_wide_kernel<2>, grid, dim3(WD_WAVES * KA_WAVE), 0, stream, wide); break;
                case 3: hipLaunchKernelGGL(skinny_wide_kernel<3>, grid, dim3(WD_WAVES * KA_WAVE), 0, stream, wide); break;
                default: hipLaunchKernelGGL(skinny_wide_kernel<4>, grid, dim3(WD_WAVES * KA_WAVE), 0, stream, wide); break;
            }
            KA_LAUNCH_CHECK();
            if (then) {
                // the finishing kernel takes whole rows and normalises them as well
                ka_launch_finish_norm(M, Na, stream, partials, splits, biasa, A2 ? bias2 : nullptr, (float*)outa, ldoa, accumulate_a, *then);
            } else {
                const int quads = M * ka_cdiv(Na, 4);
                hipLaunchKernelGGL(ka_partials_finish_kernel, dim3(ka_cdiv(quads, 256)), dim3(256), 0, stream, partials, splits,
                                   biasa, A2 ? bias2 : nullptr, outa, out_dtype_a, ldoa, M, Na, acta, accumulate_a);
            }
            KA_LAUNCH_CHECK();
            return 0;
        }
    }
    // (where K was not cut into parts, a norm that follows is a launch of its own: the same kernel, no parts)
    auto norm_after = [&]() {
        if (then)
            ka_launch_finish_norm(M, Na, stream, nullptr, 0, nullptr, nullptr, (float*)outa, ldoa, 0, *then);
    };
    if (persistent_ok) {
        if (launch_persistent(strips, M, kblocks, false, 0, stream, args)) return -1;
        KA_LAUNCH_CHECK();
        norm_after();
        KA_LAUNCH_CHECK();
        return 0;
    }
    // waves over K: enough workgroups x waves to fill the chip, no more than there are rounds for
    int waves = ka_cdiv(target_waves, strips);
    const int un = MB == 1 ? 4 : MB == 2 ? 2 : 1;
    if (waves > ka_cdiv(kblocks, un)) waves = ka_cdiv(kblocks, un);
    int rc;
    if (M <= 8) rc = launch_split<1, true>(waves, strips, stream, args);
    else switch (MB) {
        case 1: rc = launch_split<1, false>(waves, strips, stream, args); break;
        case 2: rc = launch_split<2, false>(waves, strips, stream, args); break;
        case 3: rc = launch_split<3, false>(waves, strips, stream, args); break;
        default: rc = launch_split<4, false>(waves, strips, stream, args); break;
    }
    if (rc) return rc;
    KA_LAUNCH_CHECK();
    norm_after();
    KA_LAUNCH_CHECK();
    return 0;
}

KA_API int ka_linear_skinny_fused(const void* A1, long lda1, int K1, const void* A2, long lda2, int K2,
                                  const void* W2, long ldw2, const float* bias2, const float* ln_x,
                                  const float* ln_gamma, const float* ln_beta, float ln_eps, const void* Wa,
                                  long ldwa, const float* biasa, void* outa, int out_dtype_a, long ldoa, int Na,
                                  int acta, int accumulate_a, const void* Wb, long ldwb, const float* biasb,
                                  void* outb, int out_dtype_b, long ldob, int Nb, int actb, int M,
                                  int target_waves, float* partials, long partial_floats, hipStream_t stream) {
    return skinny_fused(SkinnyExtras{}, A1, lda1, K1, A2, lda2, K2, W2, ldw2, bias2, ln_x, ln_gamma, ln_beta, ln_eps, Wa, ldwa, biasa,
                        outa, out_dtype_a, ldoa, Na, acta, accumulate_a, Wb, ldwb, biasb, outb, out_dtype_b, ldob, Nb, actb, M,
                        target_waves, partials, partial_floats, stream);
}

// out (+)= A1 W1^T + b1 + A2 W2^T + b2 into fp32 rows, then normed = LayerNorm(out; gamma, beta, eps):
// the last linears of one block and the first norm of the next. Where K is cut into parts (more than
// 8 rows) the kernel that adds the parts up normalises the rows it has just finished; else the
// norm is a launch of its own behind the linear's.
// Whether `out += A1 W1^T + A2 W2^T` of M rows and N outputs goes through the kernel that cuts K into
// parts (a second kernel then finishes the rows, and can normalise them as well at no launch of its own).
KA_API int ka_linear_skinny_pair_in_parts(int M, int N) {
    if (!sk_wide_enabled || M < 1 || M > 64) return 0;
    const int strips = ka_cdiv(N, SK_STRIP);
    return M > 16 || (strips > sk_compute_units() && M > 4) || M > 8;
}

KA_API int ka_linear_skinny_pair_norm(const void* A1, long lda1, int K1, const void* A2, long lda2, int K2,
                                      const void* W1, long ldw1, const float* bias1, const void* W2, long ldw2,
                                      const float* bias2, float* out, long ldo, int N, int accumulate, int M,
                                      int target_waves, float* partials, long partial_floats, const float* gamma,
                                      const float* beta, float eps, void* normed, int normed_dtype, long ldn,
                                      hipStream_t stream) {
    const KaThenNorm then = {gamma, beta, eps, normed, normed_dtype, ldn};
    SkinnyExtras extras;
    extras.then = &then;
    return skinny_fused(extras, A1, lda1, K1, A2, lda2, K2, W2, ldw2, bias2, nullptr, nullptr, nullptr, 0.f, W1, ldw1, bias1, out,
                        KA_F32, ldo, N, KA_ACT_NONE, accumulate, nullptr, 0, nullptr, nullptr, 0, 0, 0, 0, M, target_waves,
                        partials, partial_floats, stream);
}

// out = act(LayerNorm(x; gamma, beta, eps) W^T + bias) as ka_linear_skinny_fused computes it with its
// LayerNorm prologue (at most 16 rows), and the normalised rows themselves in `normed` (bf16 [M, K],
// rows ldn apart), for launches that follow and read the same normalised input.
KA_API int ka_linear_skinny_norm_store(const float* x, const float* gamma, const float* beta, float eps, int K,
                                       const void* W, long ldw, const float* bias, void* out, int out_dtype, long ldo,
                                       int N, int act, int M, void* normed, long ldn, hipStream_t stream) {
    KA_CHECK(normed, "ka_linear_skinny_norm_store: nowhere to store the normalised rows");
    SkinnyExtras extras;
    extras.ln_store = normed;
    extras.ln_store_ld = ldn;
    return skinny_fused(extras, nullptr, 0, K, nullptr, 0, 0, nullptr, 0, nullptr, x, gamma, beta, eps, W, ldw, bias, out, out_dtype,
                        ldo, N, act, 0, nullptr, 0, nullptr, nullptr, 0, 0, 0, 0, M, 0, nullptr, 0, stream);
}

// One input, one weight matrix, one output.
KA_API int ka_linear_skinny_bf16(const void* A, long lda, const void* W, long ldw, const float* bias,
                                 void* out, int out_dtype, long ldo, int M, int N, int K, int act,
                                 int accumulate, int target_waves, float* partials, long partial_floats,
                                 hipStream_t stream) {
    return ka_linear_skinny_fused(A, lda, K, nullptr, 0, 0, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0.f, W,
                                  ldw, bias, out, out_dtype, ldo, N, act, accumulate, nullptr, 0, nullptr, nullptr, 0,
                                  0, 0, 0, M, target_waves, partials, partial_floats, stream);
}
