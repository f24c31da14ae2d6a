// The decode attention kernel of the bf16 path as a function of (token, head, part of the keys),
// so that more than one kernel can hold it: the plain launch (attention_bf16.hip) and the launch
// that runs a linear layer on the compute units beside it (decode_beside.hip).
#pragma once
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int AT_PAGE = 16;
constexpr int AT_LDS_PAGES = 2048;        // block table entries of one row kept in LDS (32k keys)
constexpr float AT_LOG2E = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 at_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

// Orders the LDS traffic of one wave: what its lanes wrote before is seen by its lanes after.
__device__ __forceinline__ void at_wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ----------------------------------------------------------------------------------------------
// decode kernel
// ----------------------------------------------------------------------------------------------
constexpr int AD_TILE_PAGES = 4;          // pages of a wave's tile unless a kernel says otherwise (64 keys)
constexpr int ad_lanes_per_key(int hd) { int l = 1; while (l * 8 < hd) l *= 2; return l; }

// What the decode kernel needs to take over the rotary encoding and the cache write of the
// step's own token (slots null: that work was done before, and the token's key is in the cache).
struct DecodeFuse {
    const bf16_t* k_new;      // key and value rows of the tokens: [n, stride], heads side by side
    const bf16_t* v_new;
    long stride;
    const float* table;       // fp32 [positions, rot]: cos then sin
    int rot;
    const int* slots;         // page * 16 + offset the token's key and value go to, < 0: nowhere
    bf16_t* k_cache;
    bf16_t* v_cache;
};

// What a lane needs to rotate eight channels dg * 8 .. + 8 of one head row: the channels, their
// partners in the other half of the rotated part, and cos / sin of the position. Fetched in one
// go (at_fetch_rotary) and used later (at_rotated), so that the trip to memory overlaps others.
struct RotaryOperands {
    bf16x8 own, other;
};
struct RotaryAngles {        // of one position: the same for q and for the key
    floatx4 c[2], s[2];
};

// lanes past the rotated part fetch lane 0's operands (valid addresses, never used)
__device__ __forceinline__ RotaryOperands at_fetch_rotary(const bf16_t* head, int dg, int rot) {
    const int d0 = dg * 8, half = rot / 2;
    RotaryOperands r;
    r.own = at_load8(head + d0);
    const bool rotated = d0 < rot, first = d0 < half;
    r.other = at_load8(head + (rotated ? (first ? d0 + half : d0 - half) : 0));
    return r;
}

__device__ __forceinline__ RotaryAngles at_fetch_angles(const float* cs, int dg, int rot) {
    const int d0 = dg * 8, half = rot / 2;
    const bool rotated = d0 < rot, first = d0 < half;
    const int i0 = rotated ? (first ? d0 : d0 - half) : 0;
    RotaryAngles a;
    a.c[0] = *reinterpret_cast<const floatx4*>(cs + i0);
    a.c[1] = *reinterpret_cast<const floatx4*>(cs + i0 + 4);
    a.s[0] = *reinterpret_cast<const floatx4*>(cs + half + i0);
    a.s[1] = *reinterpret_cast<const floatx4*>(cs + half + i0 + 4);
    return a;
}

// The eight channels rotated (non-interleaved halves of the first `rot` channels), rounded to
// bf16 as the cache and the q buffer hold them.
__device__ __forceinline__ void at_rotated(const RotaryOperands& r, const RotaryAngles& a, int dg, int rot, float out[8]) {
    const int d0 = dg * 8, half = rot / 2;
    if (d0 >= rot) {
#pragma unroll
        for (int j = 0; j < 8; ++j) out[j] = (float)r.own[j];
        return;
    }
    const bool first = d0 < half;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float c = a.c[j / 4][j % 4], sn = a.s[j / 4][j % 4];
        float v = first ? (float)r.own[j] * c - (float)r.other[j] * sn : (float)r.own[j] * c + (float)r.other[j] * sn;
        out[j] = (float)(bf16_t)v;
    }
}

// How a row's keys are dealt out, page by page from the page that holds `lo` (keys below `lo` in it
// are masked). The units are the parts of the row x the waves of a workgroup; a unit walks over
// its keys in rounds of one tile (at most TP pages) each.
// EVEN (workgroups of four waves: many rows, the launch streams keys and values): the pages are cut
// evenly over the units, every unit gets a run of neighbouring pages, the first `rem` units one page
// more than the others, and walks over its run in rounds of equal size: the waves of a workgroup
// end together, whatever the number of pages.
// Otherwise (eight or sixteen waves: few rows, a chain of trips to memory in which a round costs the
// same whether its tile is full or not): whole tiles are dealt out in turn, unit u takes tiles u,
// u + units, ..., so that no round is spent on a tile that is partly empty except the row's last (cut
// evenly, 80 pages over sixteen waves are two rounds of 3 + 2 pages for every wave instead of a
// second round for four of them: 21.8 against 20.9 us a launch at 8 rows of 1,280 keys).
// Measured at 32 heads of 64, 8 and 64 rows, 1,024 to 1,280 keys: either way of dealing is within
// 1 us (the run-to-run spread) of the other at tiles of 4 pages; tiles of 6 and 8 pages, which hold
// a wave's pages in one round, are no faster at 1,040 to 1,280 keys and 1 us slower at 1,024 with
// the arithmetic of a tile's empty part jumped over, 4 us slower with it masked; and the loads of
// the empty part cannot be jumped over: under a condition they make the compiler wait for every
// load in flight (137 against 105 us a launch at 64 rows). At 64 rows the launch reads at 5.0 TB/s,
// what a copy of scattered 2 KB pieces reaches; a 17th page costs a wave a round of its own.
//
// AHEAD: the keys of a wave's next tile are asked for before its current tile is worked on (as
// many registers more as a tile's keys take): one trip to memory less per tile where a wave has more
// than one tile and the kernel is a chain of trips (few rows), no gain where it streams (many rows).
// (A tile's values asked for together with its keys instead: slower, 11.8 against 11.2 us for the
// attention of one row with eight waves.)
template <int HD, int WAVES, bool AHEAD = false, int TP = AD_TILE_PAGES>
__device__ __forceinline__ void
attn_decode_body(const bf16_t* __restrict__ q, long q_row_stride, const bf16_t* __restrict__ k_cache,
                 const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table, int max_pages,
                 const int* __restrict__ token_row, const int* __restrict__ kv_lo,
                 const int* __restrict__ kv_hi, bf16_t* __restrict__ out, long out_row_stride, float scale,
                 int H, int Hkv, float* __restrict__ partial, const DecodeFuse& fz,
                 const int t, const int h, const int split, const int S) {
    static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head sizes in steps of 16 up to 256");
    constexpr int CPK = HD / 8;            // 16-byte chunks of a key row
    constexpr int LPK = ad_lanes_per_key(HD);   // lanes per key row: the chunks, rounded up to a power of two
    constexpr int KPI = KA_WAVE / LPK;     // keys per load instruction
    constexpr int TILE = TP * AT_PAGE;     // keys of a full tile
    static_assert(TILE % KPI == 0, "a tile is a whole number of key loads");
    constexpr int KL = TILE / KPI;         // key loads per lane and tile
    constexpr int VU = (HD + 31) / 32;     // 16-byte value loads per lane and page (a lane takes channel u * 32 + lane / 2)
    // Where the head size is no power of two, the lanes past a key row's chunks, and past the
    // channels of a value page, ask for what another lane asks for and add nothing.
    constexpr int REC = HD + 2;            // floats of a partial result: m, l, o[HD]
    __shared__ float ps[WAVES][TILE];
    __shared__ float merge[WAVES][REC];
    __shared__ int pages[AT_LDS_PAGES];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / KA_WAVE), lane = threadIdx.x % KA_WAVE;
    const int kvh = h / (H / Hkv);
    const int row = token_row[t];
    const int lo = kv_lo ? kv_lo[t] : 0;
    const bool fused = fz.slots != nullptr && kv_hi[t] > 0;
    const int pos = kv_hi[t] - 1;                 // fused: the token's own position, whose key is not cached yet
    const int hi = fused ? pos : kv_hi[t];        // cached keys this token reads: [lo, hi)
    // this unit's rounds: round r holds the keys [tile0, tile_hi) of round_keys(r) (a row without keys,
    // hi <= lo, has no pages and no rounds: nothing of the cache is touched)
    constexpr bool EVEN = WAVES == 4;
    const int first_page = lo / AT_PAGE;
    const int n_pages_live = hi > lo ? (hi - 1) / AT_PAGE - first_page + 1 : 0;
    const int unit = split * WAVES + wave, units = S * WAVES;
    int rounds, per, mine0, mine_hi;
    if constexpr (EVEN) {
        const int base = n_pages_live / units, rem = n_pages_live % units;
        const int own = base + (unit < rem ? 1 : 0);
        mine0 = first_page + unit * base + min(unit, rem);
        rounds = (own + TP - 1) / TP;
        per = rounds > 0 ? (own + rounds - 1) / rounds : 0;
        mine_hi = min(hi, (mine0 + own) * AT_PAGE);       // keys of this unit end here
    } else {
        const int tiles = (n_pages_live + TP - 1) / TP;
        rounds = tiles > unit ? (tiles - unit + units - 1) / units : 0;
        per = TP;
        mine0 = first_page + unit * TP;
        mine_hi = hi;
    }
    const int ks = lane / LPK, dg_lane = lane % LPK;
    const bool chunk_live = dg_lane < CPK;             // this lane holds a chunk of the key row
    const int dg = chunk_live ? dg_lane : 0;
    const float sl2 = scale * AT_LOG2E;
    // this wave adds the token's own key and value: the last one, which is among those with the
    // fewest keys where they do not divide over the waves
    const bool takes_new = fused && wave == WAVES - 1 && split == 0;

    // The operands of q (and, for the wave that takes them, of the token's own key and value) are
    // asked for first and used after the first tile's keys and values have been asked for.
    const bf16_t* qhead = q + (size_t)t * q_row_stride + (size_t)h * HD;
    RotaryOperands qr, kr;
    RotaryAngles angles;
    bf16x8 qplain;
    bf16_t vnew[VU];
    if (fused) {
        qr = at_fetch_rotary(qhead, dg, fz.rot);
        angles = at_fetch_angles(fz.table + (size_t)pos * fz.rot, dg, fz.rot);
    } else {
        qplain = at_load8(qhead + dg * 8);
    }
    if (takes_new) {
        kr = at_fetch_rotary(fz.k_new + (size_t)t * fz.stride + (size_t)kvh * HD, dg, fz.rot);
        const bf16_t* vrow = fz.v_new + (size_t)t * fz.stride + (size_t)kvh * HD;
#pragma unroll
        for (int u = 0; u < VU; ++u) vnew[u] = vrow[min(u * 32 + lane / 2, HD - 1)];
    }

    const int* bt = block_table + (size_t)row * max_pages;
    {   // the row's block table goes to LDS once (see the prompt kernel)
        const int n_pages = (max(hi, 0) + AT_PAGE - 1) / AT_PAGE;
        if (n_pages <= AT_LDS_PAGES) {
            for (int i = threadIdx.x; i < n_pages; i += KA_WAVE * WAVES) pages[i] = bt[i];
            __syncthreads();
            bt = pages;
        }
    }
    // q, and the token's own key and value, have had the time of the block table's trip
    float qf[8];
    if (fused) at_rotated(qr, angles, dg, fz.rot, qf);
    else {
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[j] = (float)qplain[j];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) qf[j] = chunk_live ? qf[j] * sl2 : 0.f;
    float m_i = -INFINITY, l_i = 0.f;
    float acc[VU];
#pragma unroll
    for (int u = 0; u < VU; ++u) acc[u] = 0.f;
    if (takes_new) {
        // the token's own key and value: rotate the key, let one head of the group store both, and
        // start this wave's sums with them, straight from registers
        float kn[8];
        at_rotated(kr, angles, dg, fz.rot, kn);
        const int slot = fz.slots[t];
        if (slot >= 0 && h % (H / Hkv) == 0) {
            const size_t page = slot / AT_PAGE, off = slot % AT_PAGE;
            if (ks == 0 && chunk_live) {
                bf16x8 kb;
#pragma unroll
                for (int j = 0; j < 8; ++j) kb[j] = (bf16_t)kn[j];
                *reinterpret_cast<bf16x8*>(fz.k_cache + ((page * Hkv + kvh) * AT_PAGE + off) * HD + dg * 8) = kb;
            }
            if ((lane & 1) == 0) {
#pragma unroll
                for (int u = 0; u < VU; ++u) {
                    int d = u * 32 + lane / 2;
                    if (d < HD) fz.v_cache[((page * Hkv + kvh) * HD + d) * AT_PAGE + off] = vnew[u];
                }
            }
        }
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) dot = fmaf(qf[j], kn[j], dot);
        dot = ka_lanes_reduce<1, LPK>(dot, KaSum{});
        m_i = dot;                // the only key so far: its weight is 1
        l_i = 1.f;
#pragma unroll
        for (int u = 0; u < VU; ++u) acc[u] = (lane & 1) == 0 ? (float)vnew[u] : 0.f;
    }

    // All key loads of a tile go out before any arithmetic, and none stands under a condition (a load
    // under a branch makes the compiler wait for every load in flight: 137 against 105 us a launch at 64
    // rows): a place outside the tile's keys [max(tile0, lo), tile_hi) is moved to one inside and masked
    // afterwards (every page of a unit's run holds at least one key of [lo, hi), so there is one). A tile
    // has room for TP pages and may hold fewer: what it does not hold is masked like any other place
    // outside (jumping over its arithmetic, the same for all lanes, cuts the tile's straight run of
    // instructions into pieces: 1,215 against 1,247 tok/s at one row).
    auto load_keys = [&](int tile0, int tile_hi, bf16x8 (&dst)[KL]) {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            int key = tile0 + i * KPI + ks;
            int kc = max(min(key, tile_hi - 1), lo);   // a place that holds data (pages below lo may be gone)
            int page = bt[kc / AT_PAGE];
            dst[i] = at_load8(k_cache + (((size_t)page * Hkv + kvh) * AT_PAGE + kc % AT_PAGE) * HD + dg * 8);
        }
    };
    // round r of this unit: keys [tile0, tile_hi)
    auto round_keys = [&](int r, int& tile0, int& tile_hi) {
        const int page0 = mine0 + r * (EVEN ? per : units * TP);
        tile0 = page0 * AT_PAGE;
        tile_hi = min(mine_hi, (page0 + per) * AT_PAGE);
    };
    bf16x8 kreg[KL], knext[AHEAD ? KL : 1];
    if constexpr (AHEAD) {
        if (rounds > 0) {
            int t0, t1;
            round_keys(0, t0, t1);
            load_keys(t0, t1, kreg);
        }
    }
    for (int r = 0; r < rounds; ++r) {
        int tile0, tile_hi;
        round_keys(r, tile0, tile_hi);
        if constexpr (AHEAD) {
            // (past the last round: the last round's keys once more, which nobody uses)
            int n0, n1;
            round_keys(min(r + 1, rounds - 1), n0, n1);
            load_keys(n0, n1, knext);
        } else {
            load_keys(tile0, tile_hi, kreg);
        }
        __builtin_amdgcn_sched_barrier(0);     // all of them, before the first is used
        float sc[KL];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            int key = tile0 + i * KPI + ks;
            bool ok = key >= lo && key < tile_hi;
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) dot = fmaf(qf[j], (float)kreg[i][j], dot);
            dot = ka_lanes_reduce<1, LPK>(dot, KaSum{});           // the LPK lanes of a key
            sc[i] = ok ? dot : -INFINITY;
            mx = fmaxf(mx, sc[i]);
        }
        mx = ka_lanes_reduce<LPK, KA_WAVE>(mx, KaMax{});            // (the lanes of a key hold one value)
        float m_new = fmaxf(m_i, mx);                               // finite: the tile holds a key of [lo, hi)
        // the values: asked for as soon as the keys' registers are free, all at once; the softmax
        // below runs while they are on their way
        bf16x8 vreg[TP][VU];
#pragma unroll
        for (int pg = 0; pg < TP; ++pg) {
            int kc = max(min(tile0 + pg * AT_PAGE, tile_hi - 1), lo);
            int page = bt[kc / AT_PAGE];
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                int d = min(u * 32 + lane / 2, HD - 1);
                vreg[pg][u] = at_load8(v_cache + (((size_t)page * Hkv + kvh) * HD + d) * AT_PAGE + (lane & 1) * 8);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        float alpha = exp2f(m_i - m_new);
        float rowsum = 0.f;
        at_wave_sync();                        // the previous tile's probabilities have been read
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            float p = exp2f(sc[i] - m_new);
            rowsum += p;
            if (dg_lane == 0) ps[wave][i * KPI + ks] = p;
        }
        rowsum = ka_lanes_reduce<LPK, KA_WAVE>(rowsum, KaSum{});
        l_i = l_i * alpha + rowsum;
        m_i = m_new;
#pragma unroll
        for (int u = 0; u < VU; ++u) acc[u] *= alpha;
        at_wave_sync();
        // values: a page is HD rows of 16 keys; a lane holds 8 keys (half a row) per load
#pragma unroll
        for (int pg = 0; pg < TP; ++pg) {
            const int half = lane & 1;
            const int first = tile0 + pg * AT_PAGE + half * 8;
            float pv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) pv[j] = ps[wave][pg * AT_PAGE + half * 8 + j];
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                float sum = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    int key = first + j;                      // slots outside the data may hold anything
                    float x = key >= lo && key < tile_hi ? (float)vreg[pg][u][j] : 0.f;
                    sum = fmaf(pv[j], x, sum);
                }
                acc[u] += sum;
            }
        }
        if constexpr (AHEAD) {
#pragma unroll
            for (int i = 0; i < KL; ++i) kreg[i] = knext[i];
        }
    }
    // the two halves of a channel row
#pragma unroll
    for (int u = 0; u < VU; ++u) acc[u] = ka_lanes_reduce<1, 2>(acc[u], KaSum{});
    if (lane == 0) { merge[wave][0] = m_i; merge[wave][1] = l_i; }
    if ((lane & 1) == 0) {
#pragma unroll
        for (int u = 0; u < VU; ++u)
            if (u * 32 + lane / 2 < HD) merge[wave][2 + u * 32 + lane / 2] = acc[u];
    }
    __syncthreads();
    if (wave != 0) return;
    // wave 0: lane d (and d + 64 for hd 128) merges the waves in wave order
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) M = fmaxf(M, merge[w][0]);
    float L = 0.f;
    float od[(HD + KA_WAVE - 1) / KA_WAVE];
#pragma unroll
    for (int e = 0; e < (HD + KA_WAVE - 1) / KA_WAVE; ++e) od[e] = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        float mw = merge[w][0];
        float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
        L += merge[w][1] * f;
#pragma unroll
        for (int e = 0; e < (HD + KA_WAVE - 1) / KA_WAVE; ++e) {
            int d = e * KA_WAVE + lane;
            if (d < HD) od[e] += merge[w][2 + d] * f;
        }
    }
    if (S > 1) {
        float* mine = partial + ((size_t)(t * H + h) * S + split) * REC;
        if (lane == 0) { mine[0] = M; mine[1] = L; }
#pragma unroll
        for (int e = 0; e < (HD + KA_WAVE - 1) / KA_WAVE; ++e) {
            int d = e * KA_WAVE + lane;
            if (d < HD) mine[2 + d] = od[e];
        }
        return;            // the parts meet in attn_decode_merge_kernel
    }
    float inv = L > 0.f ? 1.0f / L : 0.f;
    bf16_t* op = out + (size_t)t * out_row_stride + (size_t)h * HD;
#pragma unroll
    for (int e = 0; e < (HD + KA_WAVE - 1) / KA_WAVE; ++e) {
        int d = e * KA_WAVE + lane;
        if (d < HD) op[d] = (bf16_t)(od[e] * inv);
    }
}

// The parts of a row's keys meet here, in the order of the parts: one wave per (token, head).
// A kernel of its own and no arrival counter inside the first: a workgroup that waits for the
// others' sums to become visible has to flush and refill its XCD's L2 (tens of microseconds).
template <int HD>
__global__ void __launch_bounds__(KA_WAVE)
attn_decode_merge_kernel(const float* __restrict__ partial, int S, bf16_t* __restrict__ out, long out_row_stride, int H) {
    constexpr int REC = HD + 2;
    constexpr int E = (HD + KA_WAVE - 1) / KA_WAVE;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* all = partial + (size_t)(t * H + h) * S * REC;
    float M = -INFINITY;
    for (int s = 0; s < S; ++s) M = fmaxf(M, all[s * REC]);
    float L = 0.f, od[E];
#pragma unroll
    for (int e = 0; e < E; ++e) od[e] = 0.f;
    for (int s = 0; s < S; ++s) {
        const float ms = all[s * REC];
        const float f = ms == -INFINITY ? 0.f : exp2f(ms - M);
        L += all[s * REC + 1] * f;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int d = e * KA_WAVE + lane;
            if (d < HD) od[e] += all[s * REC + 2 + d] * f;
        }
    }
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    bf16_t* op = out + (size_t)t * out_row_stride + (size_t)h * HD;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int d = e * KA_WAVE + lane;
        if (d < HD) op[d] = (bf16_t)(od[e] * inv);
    }
}

// ----------------------------------------------------------------------------------------------
// host side: what every launch of these kernels checks first
// ----------------------------------------------------------------------------------------------
static inline int check_common(const char* who, const void* q, long q_row_stride, const void* out, long out_row_stride,
                        int n, int H, int Hkv, int hd, int page_size, int max_pages) {
    KA_CHECK(n > 0 && H > 0 && Hkv > 0 && H % Hkv == 0, "%s: bad sizes n=%d H=%d Hkv=%d", who, n, H, Hkv);
    KA_CHECK(page_size == AT_PAGE, "%s: page size %d (the MFMA kernels need %d)", who, page_size, AT_PAGE);
    KA_CHECK(max_pages > 0, "%s: empty block table", who);
    KA_CHECK(q_row_stride % 8 == 0 && (uintptr_t)q % 16 == 0 && hd % 8 == 0, "%s: q must be 16-byte aligned", who);
    KA_CHECK(out_row_stride % 4 == 0 && (uintptr_t)out % 8 == 0, "%s: out must be 8-byte aligned", who);
    KA_CHECK(H <= 65535, "%s: too many heads", who);
    return 0;
}

KA_API int ka_attention_decode_supported(int hd, int page_size);
KA_API long ka_attention_decode_partial_floats(int n, int H, int hd, int splits);

// The operands of a decode launch; fills what the kernel needs to rotate and store the tokens' own
// keys and values (`slots` non-null).
static inline int decode_check(const char* who, const void* q, long q_row_stride, const void* out, long out_row_stride,
                               int n, int H, int Hkv, int hd, int page_size, int max_pages, int splits,
                               const float* partial, long partial_floats, const void* k_new, const void* v_new,
                               long new_stride, const float* table, int rot, const int* slots, void* k_cache_w,
                               void* v_cache_w, DecodeFuse* fz) {
    if (check_common(who, q, q_row_stride, out, out_row_stride, n, H, Hkv, hd, page_size, max_pages)) return -1;
    KA_CHECK(ka_attention_decode_supported(hd, page_size), "%s: head size %d not covered", who, hd);
    KA_CHECK(splits >= 1 && splits <= 65535, "%s: bad split count %d", who, splits);
    if (splits > 1) {
        KA_CHECK(partial, "%s: scratch missing", who);
        KA_CHECK(ka_attention_decode_partial_floats(n, H, hd, splits) <= partial_floats, "%s: scratch too small", who);
    }
    *fz = DecodeFuse{};
    if (slots) {
        // the kernel rotates q and the new key itself and stores the token's key and value
        KA_CHECK(k_new && v_new && k_cache_w && v_cache_w, "%s: fused mode needs the new key and value rows", who);
        KA_CHECK(rot > 0 && rot <= hd && rot % 16 == 0 && table, "%s: fused mode needs a rotary width that is a multiple of 16 (got %d)", who, rot);
        KA_CHECK(new_stride % 8 == 0 && (uintptr_t)k_new % 16 == 0 && (uintptr_t)v_new % 16 == 0, "%s: new key rows must be 16-byte aligned", who);
        *fz = DecodeFuse{(const bf16_t*)k_new, (const bf16_t*)v_new, new_stride, table, rot, slots, (bf16_t*)k_cache_w, (bf16_t*)v_cache_w};
    }
    return 0;
}
