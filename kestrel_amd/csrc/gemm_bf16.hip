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
// That kernel takes any K (in steps of 8); where K is a multiple of 64 the large-tile kernel
// further down, which loads straight into LDS, is used instead.
#include "ka_common.h"
#include "ka_partials.h"

#include <stdlib.h>

#include <type_traits>

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
                if (ka_act_gated(act)) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = acc[a][b][q * 4 + i] + (bias && n + i < N ? bias[n + i] : 0.f);
                    ka_gated_store<true, 4>(out, out_dtype, ldo, m, n, N, v, act);
                    continue;
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float x = acc[a][b][q * 4 + i];
                    if (bias && n + i < N) x += bias[n + i];
                    if (act) x = ka_activate_fast(act, x);
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

// ----------------------------------------------------------------------------
// The large-tile kernel. Four (2 x 2) or eight (4 x 2) waves, each with WN x WM MFMA tiles of
// 32 x 32. K-steps of BK go from global memory straight into LDS (global_load_lds_dwordx4: no
// registers, no ds_write), NS stages, one barrier per step. Chunk c (16 bytes) of tile row r
// lies at place c ^ swizzle(r) of its row, chosen by which chunk each lane of the load asks
// for, so that the rows that one pass of a 16-byte LDS read touches fall on different banks
// without padding. Rows past the end of a matrix are read from its last row (and never stored);
// K must be a multiple of BK.
// ----------------------------------------------------------------------------
constexpr int gd_smem(int bn, int bm, int bk, int ns) { return ns * (bn + bm) * bk * 2; }

// A loop whose index is a compile-time constant in every round (the accumulators are up to 256
// registers: an index the compiler does not resolve would put them in memory).
template <int I, int N, typename F>
__device__ __forceinline__ void gd_static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        gd_static_for<I + 1, N>(f);
    }
}

#define GD_GLOBAL __attribute__((address_space(1)))
#define GD_LDS __attribute__((address_space(3)))

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters at their maximum)
template <int N>
__device__ __forceinline__ void gd_wait_loads() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}

// Waits until at most `younger` x LPW of this wave's loads are still in flight (the count of an
// s_waitcnt is an immediate: one instruction per value that can occur, at most MAX).
template <int LPW, int MAX>
__device__ __forceinline__ void gd_wait_younger(int younger) {
    static_assert(LPW * (MAX > 0 ? MAX : 0) <= 63, "more loads in flight than the counter holds");
    if constexpr (MAX <= 0) {
        gd_wait_loads<0>();
    } else {
        if (younger >= MAX) gd_wait_loads<LPW * MAX>();
        else gd_wait_younger<LPW, MAX - 1>(younger);
    }
}

// s_waitcnt lgkmcnt(0) alone: this wave's LDS reads have all arrived in its registers
__device__ __forceinline__ void gd_wait_lds() { __builtin_amdgcn_s_waitcnt(0xc07f); }

// The barrier alone, without the fence that __syncthreads() puts before it: that fence waits
// for every load in flight, the younger stages' too. What must be ordered here is ordered by
// hand: a wave has waited for its own loads of the stage (vmcnt) and for its LDS reads of the
// stage before (their values were used) when it arrives.
__device__ __forceinline__ void gd_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Orders the LDS traffic of one wave: what its lanes wrote before is seen by its lanes after.
__device__ __forceinline__ void at_epilogue_wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int WN, int WM, int GN, int GM, int BK, int NS, int SL>
__global__ void __launch_bounds__(KA_WAVE * GN * GM)
    __attribute__((amdgpu_waves_per_eu(GN * GM / 4, (WN * WM > 8 ? 1 : 2) * (GN * GM / 4))))
gemm_dma_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, long ldw,
                const float* __restrict__ bias, void* __restrict__ out, int out_dtype, long ldo, int M,
                int N, int K, int act, int accumulate, int tiles_n, int tiles_m, int k_per) {
    static_assert(BK == 32 || BK == 64, "K-steps of 32 or 64");
    // K cut into parts (grid y): part p multiplies the k_per columns from p * k_per on and writes
    // its sums as fp32 [M, N] of its own (the host passes the partial buffer as `out`, no bias,
    // no activation; a finishing kernel adds the parts up)
    if (k_per > 0) {
        const int part = blockIdx.y;
        A += (size_t)part * k_per;
        W += (size_t)part * k_per;
        K = min(k_per, K - part * k_per);
        out = reinterpret_cast<float*>(out) + (size_t)part * M * ldo;
    }
    static_assert(NS >= 2 && NS <= 8, "two to eight stages");
    static_assert(GN * GM == 4 || GN * GM == 8, "four or eight waves");
    constexpr int WAVES = GN * GM;
    constexpr int BN = 32 * WN * GN, BM = 32 * WM * GM;
    constexpr int ROW = BK * 2;                          // bytes of a tile row
    constexpr int CPR = BK / 8;                          // 16-byte chunks of a tile row
    constexpr int RPL = KA_WAVE / CPR;                   // rows that one load of 1 KB brings
    constexpr int STAGE = (BN + BM) * ROW;               // bytes of one stage: W rows, then X rows
    constexpr int W_LOADS = BN / RPL / WAVES, X_LOADS = BM / RPL / WAVES;   // loads per wave and stage
    static_assert(W_LOADS * RPL * WAVES == BN && X_LOADS * RPL * WAVES == BM, "the tile does not divide over the waves' loads");
    constexpr int LPW = W_LOADS + X_LOADS;
    extern __shared__ __attribute__((aligned(16))) unsigned char gb_lds[];
    int pid = blockIdx.x;
    int total = tiles_n * tiles_m;
    int per_xcd = (total + 7) / 8;
    int logical = (pid % 8) * per_xcd + pid / 8;
    if (logical >= total) return;
    int tn = logical / tiles_m, tm = logical % tiles_m;
    const int n0 = tn * BN, m0 = tm * BM;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / KA_WAVE), lane = tid % KA_WAVE;
    const int wn = wave / GM, wm = wave % GM;
    const int li = lane % 32, lg = lane / 32;

    floatx16 acc[WN][WM];
#pragma unroll
    for (int a = 0; a < WN; ++a)
#pragma unroll
        for (int b = 0; b < WM; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    // Chunk c of row r lies at place c ^ swizzle(r) of its row. One pass of a 16-byte LDS read
    // serves 16 lanes, which here read the same chunk of 16 consecutive rows, and the 64 banks
    // hold 256 bytes: two rows of 128 bytes, so rows of the same parity must differ in their
    // place ((r >> 1) & 7), or four rows of 64 bytes ((r >> 2) & 3). (Measured with r & 7: half
    // of the LDS cycles were bank conflicts, rows r and r + 8 meeting in one pass.)
    auto swizzle = [](int r) { return CPR == 8 ? ((r >> 1) & 7) : ((r >> 2) & 3); };
    // What this lane asks for in a load of RPL rows: row lane / CPR of them, and the chunk that
    // belongs at place lane % CPR of that row.
    const int lrow = lane / CPR;
    const bf16_t* wsrc[W_LOADS];
    const bf16_t* xsrc[X_LOADS];
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
        int r = (wave * W_LOADS + i) * RPL + lrow;
        wsrc[i] = W + (size_t)min(n0 + r, N - 1) * ldw + ((lane % CPR) ^ swizzle(r)) * 8;
    }
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) {
        int r = (wave * X_LOADS + i) * RPL + lrow;
        xsrc[i] = A + (size_t)min(m0 + r, M - 1) * lda + ((lane % CPR) ^ swizzle(r)) * 8;
    }
    auto fetch = [&](int stage, int k0) {
        unsigned char* base = gb_lds + stage * STAGE;
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i)
            __builtin_amdgcn_global_load_lds((const GD_GLOBAL void*)(wsrc[i] + k0),
                                             (GD_LDS void*)(base + (wave * W_LOADS + i) * RPL * ROW), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < X_LOADS; ++i)
            __builtin_amdgcn_global_load_lds((const GD_GLOBAL void*)(xsrc[i] + k0),
                                             (GD_LDS void*)(base + BN * ROW + (wave * X_LOADS + i) * RPL * ROW), 16, 0, 0);
    };

    // operand addresses inside a stage: tile row li of each of this wave's tiles; the k-chunk
    // of k-step ks is ks * 2 + lg
    int wrow_off[WN], xrow_off[WM];
#pragma unroll
    for (int a = 0; a < WN; ++a) wrow_off[a] = (wn * 32 * WN + a * 32 + li) * ROW;
#pragma unroll
    for (int b = 0; b < WM; ++b) xrow_off[b] = BN * ROW + (wm * 32 * WM + b * 32 + li) * ROW;
    const int swz = swizzle(li);

    // The K-steps' operands are read from LDS a group of SL k-slices (of 16) at a time, one group
    // ahead of the group that is being multiplied, also across the edge of a K-step: the MFMAs of a
    // stage's last group run while the first group of the next stage is on its way from LDS, so the
    // matrix pipes do not stand still at every K-step while both waves of a SIMD wait for LDS
    // together. For that the barrier of a K-step stands before the last group's MFMAs: a wave
    // arrives when its own loads of the next stage have landed and its own reads of this stage are
    // in its registers. After the barrier everybody's have, so the next stage may be read and this
    // stage's memory may be written: the load of stage s + NS goes out, and has NS - 1 K-steps to land.
    constexpr int G = BK / 16 / SL;                      // groups per K-step
    static_assert(G * SL * 16 == BK, "the groups of slices do not divide a K-step");
    const int steps = K / BK;
    // NS stages go out at once; the first has to be there before anything can be read
#pragma unroll
    for (int st = 0; st < NS; ++st)
        if (st < steps) fetch(st, st * BK);
    {
        const int younger = min(NS - 1, steps - 1);
        gd_wait_younger<LPW, NS - 1>(younger);
        gd_barrier();
    }
    bf16x8 wa[2][SL][WN], xb[2][SL][WM];
    auto operands = [&](auto slot_c, int stage, int g) {
        constexpr int slot = decltype(slot_c)::value;
        const unsigned char* base = gb_lds + (stage % NS) * STAGE;
#pragma unroll
        for (int i = 0; i < SL; ++i) {
            const int place = (((g * SL + i) * 2 + lg) ^ swz) * 16;
#pragma unroll
            for (int a = 0; a < WN; ++a) wa[slot][i][a] = *reinterpret_cast<const bf16x8*>(base + wrow_off[a] + place);
#pragma unroll
            for (int b = 0; b < WM; ++b) xb[slot][i][b] = *reinterpret_cast<const bf16x8*>(base + xrow_off[b] + place);
        }
    };
    const int groups = steps * G;
    // group t (stage t / G, its group t % G) is multiplied from the registers of slot t & 1
    auto group = [&](auto slot_c, int t) {
        constexpr int slot = decltype(slot_c)::value;
        const int st = t / G, g = t % G;
        if (g == G - 1 && st + 1 < steps) {
            // own loads of stage st + 1 landed (the stages after it may stay in flight), own reads of
            // stage st done (they are the operands of this group, needed below in any case)
            const int younger = min(NS - 2, steps - 2 - st);
            gd_wait_younger<LPW, NS - 2>(younger);
            gd_wait_lds();
            gd_barrier();
            if (st + NS < steps) fetch(st % NS, (st + NS) * BK);
        }
        // (always, also after the last group, whose "next" is read from memory nobody needs: a read
        // under a condition makes the compiler wait for every read in flight before the MFMAs,
        // the ones just asked for included)
        operands(std::integral_constant<int, slot ^ 1>{}, (t + 1) / G, (t + 1) % G);
#pragma unroll
        for (int i = 0; i < SL; ++i)
#pragma unroll
            for (int a = 0; a < WN; ++a)
#pragma unroll
                for (int b = 0; b < WM; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[slot][i][a], xb[slot][i][b], acc[a][b], 0, 0, 0);
        // The reads of the next group go out behind this group's second MFMA, into registers of
        // their own, and have the rest of the group's MFMAs to arrive. (Left to itself the compiler
        // gives both groups the same registers and asks for the next operands only after the
        // MFMAs that use the present ones, three MFMAs before they are needed. Asked for ahead of
        // the group's first MFMA they would be waited for at once: the compiler waits for every
        // read in flight where this loop needs the older ones only.)
        constexpr int FIRST = SL * WN * WM > 2 ? 2 : 1;
        __builtin_amdgcn_sched_group_barrier(0x008, FIRST, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, SL * (WN + WM), 0);
        __builtin_amdgcn_sched_group_barrier(0x008, SL * WN * WM - FIRST, 0);
    };
    // (Nothing but LDS reads may be in flight on the counter they share with scalar loads when the
    // loop is entered: with a scalar load among them the compiler can no longer count on arrival
    // in order and waits, in every round, for all reads, the ones just asked for included.)
    // (The arguments that only the epilogue uses are asked for here for the same reason: the
    // compiler otherwise fetches them, with scalar loads, as late as it can.)
    asm volatile("" ::"s"(bias), "s"(out), "s"(ldo), "s"(act), "s"(accumulate), "s"(out_dtype), "s"(M), "s"(N));
    gd_wait_lds();
    operands(std::integral_constant<int, 0>{}, 0, 0);
    int t = 0;
    for (; t + 1 < groups; t += 2) {
        group(std::integral_constant<int, 0>{}, t);
        group(std::integral_constant<int, 1>{}, t + 1);
    }
    if (t < groups) group(std::integral_constant<int, 0>{}, t);

    // Epilogue. acc[a][b][v] is out[m][n] with n = n0 + wn*32*WN + a*32 + (v/4)*8 + lg*4 + v%4 and
    // m = m0 + wm*32*WM + b*32 + li: a lane holds four neighbouring outputs of one row, and one
    // store instruction of the wave would touch 32 rows with 16 (bf16) or 32 bytes each, which the
    // memory system takes at a fraction of its rate (measured: 15 us of 79 for the 33 MB of the
    // first feed-forward linear of a 2,048-token prompt). So a wave passes its outputs through its
    // share of the stages' LDS, 32 rows at a time or more, and stores whole rows of its tile: 128
    // or 256 contiguous bytes per row, 16 bytes per lane. Bias and activation are applied on the
    // way in; an fp32 output that accumulates is read and added on the way out.
    gd_barrier();                                        // the last stage has been read by everybody
    const bool bias_vec = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(bias) % 16 == 0);
    auto staged = [&](auto* typed_out) {
        using T = std::remove_pointer_t<decltype(typed_out)>;
        constexpr int ES = sizeof(T);                    // 2 or 4
        constexpr int PER = 16 / ES;                     // outputs per 16-byte store
        constexpr int RB = 32 * WN * ES;                 // bytes of a row of the wave's tile
        constexpr int RS = RB + (ES == 2 ? 8 : 16);      // its place in LDS: padded so that the lanes' writes spread over the banks
        constexpr int SHARE = gd_smem(BN, BM, BK, NS) / WAVES;
        constexpr int BP = SHARE / (32 * RS) < WM ? SHARE / (32 * RS) : WM;      // blocks of 32 rows per pass
        static_assert(BP >= 1, "a wave's share of LDS does not hold 32 rows of its tile");
        constexpr int CH = RB / 16;                      // 16-byte chunks of a row
        constexpr int RPI = KA_WAVE / CH;                // rows one store instruction covers
        unsigned char* mine = gb_lds + wave * SHARE;
        const int n_wave = n0 + wn * 32 * WN, m_wave = m0 + wm * 32 * WM;
        const bool wide = (ldo * ES) % 16 == 0 && reinterpret_cast<uintptr_t>(typed_out) % 16 == 0 && n0 % PER == 0;
        gd_static_for<0, (WM + BP - 1) / BP>([&](auto pc) {
            constexpr int b0 = decltype(pc)::value * BP;
            constexpr int nb = b0 + BP <= WM ? BP : WM - b0;
            gd_static_for<0, nb>([&](auto bc) {
                constexpr int b = b0 + decltype(bc)::value;
                gd_static_for<0, WN>([&](auto ac) {
                    constexpr int a = decltype(ac)::value;
                    gd_static_for<0, 4>([&](auto qc) {
                        constexpr int q = decltype(qc)::value;
                        const int nl = a * 32 + q * 8 + lg * 4;
                        const int n = n_wave + nl;
                        floatx4 bv = {0.f, 0.f, 0.f, 0.f};
                        if (bias && n < N) {
                            if (bias_vec) bv = *reinterpret_cast<const floatx4*>(bias + n);       // n + 3 < N: N % 4 == 0
                            else
                                for (int i = 0; i < 4 && n + i < N; ++i) bv[i] = bias[n + i];
                        }
                        float v[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            float x = acc[a][b][q * 4 + i] + bv[i];
                            if (act) x = ka_activate_fast(act, x);
                            v[i] = x;
                        }
                        unsigned char* at = mine + ((b - b0) * 32 + li) * RS + nl * ES;
                        if constexpr (ES == 2) *reinterpret_cast<bf16x4*>(at) = bf16x4{(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
                        else *reinterpret_cast<floatx4*>(at) = floatx4{v[0], v[1], v[2], v[3]};
                    });
                });
            });
            at_epilogue_wave_sync();
#pragma unroll
            for (int r0 = 0; r0 < nb * 32; r0 += RPI) {
                const int rl = r0 + lane / CH, c = lane % CH;
                const int m = m_wave + b0 * 32 + rl, n = n_wave + c * PER;
                if (lane < RPI * CH && rl < nb * 32 && m < M && n < N) {      // (a row's chunks need not divide 64 lanes)
                    const unsigned char* from = mine + rl * RS + c * 16;
                    T* op = typed_out + (size_t)m * ldo + n;
                    if (wide && n + PER <= N) {
                        if constexpr (ES == 2) {
                            *reinterpret_cast<bf16x8*>(op) = *reinterpret_cast<const bf16x8*>(from);
                        } else {
                            floatx4 x = *reinterpret_cast<const floatx4*>(from);
                            if (accumulate) {
                                const floatx4 cur = *reinterpret_cast<const floatx4*>(op);
                                x = floatx4{cur[0] + x[0], cur[1] + x[1], cur[2] + x[2], cur[3] + x[3]};
                            }
                            *reinterpret_cast<floatx4*>(op) = x;
                        }
                    } else {
                        const T* src = reinterpret_cast<const T*>(from);
                        for (int i = 0; i < PER && n + i < N; ++i) {
                            if constexpr (ES == 2) op[i] = src[i];
                            else op[i] = accumulate ? op[i] + src[i] : src[i];
                        }
                    }
                }
            }
            at_epilogue_wave_sync();                     // the next pass writes over what was just read
        });
    };
    if (out_dtype == KA_F32) staged(reinterpret_cast<float*>(out));
    else staged(reinterpret_cast<bf16_t*>(out));
}

template <int WN, int WM, int GN, int GM, int BK, int NS, int SL = 1>
static int launch_dma(const bf16_t* A, long lda, const bf16_t* W, long ldw, const float* bias, void* out,
                      int out_dtype, long ldo, int M, int N, int K, int act, int accumulate, hipStream_t stream,
                      int parts = 1, int k_per = 0) {
    static bool configured = false;
    constexpr int BN = 32 * WN * GN, BM = 32 * WM * GM;
    constexpr int smem = gd_smem(BN, BM, BK, NS);
    static_assert(smem <= 160 * 1024, "the stages do not fit in LDS");
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_dma_kernel<WN, WM, GN, GM, BK, NS, SL>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        KA_CHECK(e == hipSuccess, "ka_linear_tiled_bf16: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
        configured = true;
    }
    int tiles_n = ka_cdiv(N, BN), tiles_m = ka_cdiv(M, BM);
    long total = (long)tiles_n * tiles_m;
    long launched = ((total + 7) / 8) * 8;
    KA_CHECK(launched < (1L << 31), "ka_linear_tiled_bf16: too many tiles");
    hipLaunchKernelGGL((gemm_dma_kernel<WN, WM, GN, GM, BK, NS, SL>), dim3((unsigned)launched, parts), dim3(KA_WAVE * GN * GM), smem,
                       stream, A, lda, W, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, tiles_n, tiles_m, k_per);
    return 0;
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

// `config`: 0 chooses by size; other values force a tile (for measurements and tests), with
// 1000000 * parts added to force K to be cut into that many parts as well. `partials`: scratch
// memory for the sums of such parts (null: K is never cut).
KA_API int ka_linear_tiled_bf16(const void* A, long lda, const void* W, long ldw, const float* bias,
                                void* out, int out_dtype, long ldo, int M, int N, int K, int act,
                                int accumulate, int config, float* partials, long partial_floats,
                                hipStream_t stream) {
    KA_CHECK(M > 0 && N > 0 && K > 0 && K % 8 == 0, "ka_linear_tiled_bf16: M=%d N=%d K=%d (K must be a multiple of 8)", M, N, K);
    KA_CHECK(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K, "ka_linear_tiled_bf16: row strides must be multiples of 8 and >= K");
    KA_CHECK(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "ka_linear_tiled_bf16: operands must be 16-byte aligned");
    KA_CHECK(ka_act_known(act), "ka_linear_tiled_bf16: unknown activation %d", act);
    KA_CHECK(ldo >= ka_act_outputs(act, N), "ka_linear_tiled_bf16: output stride too small");
    KA_CHECK(!ka_act_gated(act) || (N % 2 == 0 && !accumulate), "ka_linear_tiled_bf16: a gated linear needs an even N and no accumulation");
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_linear_tiled_bf16: bad output type");
    KA_CHECK(!(accumulate && out_dtype != KA_F32), "ka_linear_tiled_bf16: accumulate needs an fp32 output");
    KA_CHECK((uintptr_t)out % 16 == 0, "ka_linear_tiled_bf16: output must be 16-byte aligned");
    int parts = config >= 1000000 ? config / 1000000 : 0;      // 0: chosen below
    config %= 1000000;
    if (ka_act_gated(act) && config != 211 && config != 221) {
        // the pairs of a gated linear meet in the epilogue of the tiles that are staged through registers (the
        // large tiles write their outputs as whole rows through LDS, laid out for N columns)
        config = (long)ka_cdiv(N, 128) * ka_cdiv(M, 128) >= 512 ? 221 : 211;
        parts = 0;
    }
    if (config == 0) {
        if (K % 64 == 0) {
            // Tiles of 128 x 128 read 64 flops' worth of operands per byte from L2, which is what
            // bounds them (measured: 11 TB/s of L2 traffic at 800 TFLOP/s); 256 x 256 halves that
            // and wins where its tiles fill most of the CUs in every round (measured inside the
            // model at 2048 rows: N = 6144 and 8192). Where 128 x 128 tiles leave a CU with one
            // workgroup only, eight waves and three stages hide the trip to HBM that two
            // workgroups would otherwise hide for each other (N = 2048: 35 us of 120 at K = 8192).
            const int cus = ka_compute_units();
            long t256 = (long)ka_cdiv(N, 256) * ka_cdiv(M, 256);
            long t128 = (long)ka_cdiv(N, 128) * ka_cdiv(M, 128);
            long rounds = (t256 + cus - 1) / cus;
            // (192 x 256 where its tiles fill the CUs and those of 256 x 256 do not: N = 6144 at
            // 2048 rows is 192 tiles of the one, 256 of the other; measured 7 us of 74 faster)
            long t192 = (long)ka_cdiv(N, 192) * ka_cdiv(M, 256);
            long rounds192 = (t192 + cus - 1) / cus;
            if (t192 * 10 >= rounds192 * cus * 7 && t192 * rounds * 10 > t256 * rounds192 * 11) config = 22232;
            else if (t256 * 10 >= rounds * cus * 7) config = 22224;
            else if (t128 <= cus) {
                config = 23212;
                // Few tiles (a few hundred rows of a narrow output): K is cut into parts so that
                // about every CU gets a workgroup; a second kernel adds the parts up.
                if (parts == 0 && partials && t128 * 2 <= cus && K >= 1024) {
                    parts = (int)(cus / t128);
                    if (parts > K / 512) parts = K / 512;
                    if (parts > 8) parts = 8;
                }
            } else config = 12222;
        } else {
            long t22 = (long)ka_cdiv(N, 128) * ka_cdiv(M, 128);
            config = t22 >= 512 ? 221 : 211;
        }
    }
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    int rc;
    if (parts >= 2 && config == 23212 && K % 64 == 0) {
        int k_per = ka_cdiv(ka_cdiv(K, parts), 64) * 64;
        parts = ka_cdiv(K, k_per);
        if (parts >= 2 && partials && (long)parts * M * N <= partial_floats) {
            rc = launch_dma<1, 2, 4, 2, 64, 3, 4>(a, lda, w, ldw, nullptr, partials, KA_F32, N, M, N, K, 0, 0, stream, parts, k_per);
            if (rc) return rc;
            KA_LAUNCH_CHECK();
            const int quads = M * ka_cdiv(N, 4);
            hipLaunchKernelGGL(ka_partials_finish_kernel, dim3(ka_cdiv(quads, 256)), dim3(256), 0, stream, partials, parts,
                               bias, (const float*)nullptr, out, out_dtype, ldo, M, N, act, accumulate);
            KA_LAUNCH_CHECK();
            return 0;
        }
    }
    switch (config) {
        case 221: rc = launch_config<2, 2, 64>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); break;
        case 211: rc = launch_config<2, 1, 64>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); break;
#define KA_DMA(CODE, WNV, WMV, GNV, GMV, BKV, NSV, SLV)                                                               \
        case CODE:                                                                                                \
            KA_CHECK(K % BKV == 0, "ka_linear_tiled_bf16: this tile needs K to be a multiple of %d", BKV);        \
            rc = launch_dma<WNV, WMV, GNV, GMV, BKV, NSV, SLV>(a, lda, w, ldw, bias, out, out_dtype, ldo, M, N, K, act, accumulate, stream); \
            break;
        // 10000 (four waves, 2 x 2) or 20000 (eight waves, 4 x 2) + stages * 1000 + (K-step / 32) * 100 + wave tile
        KA_DMA(12222, 2, 2, 2, 2, 64, 2, 2)      // 128 x 128, two workgroups per CU
        KA_DMA(23212, 1, 2, 4, 2, 64, 3, 4)      // 128 x 128 by eight waves, three stages: for one workgroup per CU
        KA_DMA(22224, 2, 4, 4, 2, 64, 2, 1)      // 256 x 256, one workgroup of eight waves per CU
        KA_DMA(22232, 3, 2, 2, 4, 64, 2, 1)      // 192 x 256 (N x M), eight waves: for an N that 256 leaves CUs idle with
        KA_DMA(13122, 2, 2, 2, 2, 32, 3, 2)      // (slower everywhere; kept as the test of K-steps of 32)
#undef KA_DMA
        default: KA_CHECK(false, "ka_linear_tiled_bf16: unknown tile configuration %d", config);
    }
    if (rc) return rc;
    KA_LAUNCH_CHECK();
    return 0;
}
