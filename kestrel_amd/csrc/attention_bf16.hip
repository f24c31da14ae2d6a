// bf16 paged attention on the matrix cores: a prompt kernel and a decode kernel.
//
// Cache layout: keys [pages, Hkv, 16, hd], values [pages, Hkv, hd, 16] (transposed inside the
// page), page size 16. Every token t of the packed batch reads the keys [kv_lo[t], kv_hi[t]) of
// its row through the row's block table; the step's own keys are already in the cache.
//
// Prompt kernel. A workgroup owns one or two blocks of 32 consecutive queries of one row and one
// head; its four waves take every fourth tile of 32 keys (two pages) each and merge at the end; the
// next tile's keys and the current tile's values are in flight while the current scores are
// computed. Scores are computed transposed, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: the keys are
// the row operand (a lane loads half a key row straight from the cache), the queries the column
// operand (held in registers for the whole loop). A lane then holds, for ONE query, 16 scores:
// softmax needs only in-lane work and one exchange with the lane 32 apart, and most tiles take
// their exponentials from the reference point the query already has (the sum of a tile's
// exponentials tells when that point has to move). The key rows are fed to the MFMA in a permuted
// order (bits 2 and 3 of the row index swapped) so that the 8 probabilities a lane holds for a
// page are those of 8 consecutive keys: they are, as they stand, the column operand of
// O^T += V^T P^T, whose row operand is one 16-byte load from the transposed value page. LDS holds
// the row's block table and is used for the merge.
//
// Decode kernel. One query per row: a bandwidth problem. The keys of a row are cut into splits
// (grid z) and 64-key tiles (waves); 16-byte loads are fully coalesced for keys (8 lanes per key
// row at hd 64) and values (2 lanes per channel row of a page). Waves merge through LDS, splits
// through scratch memory in a second kernel, always in the same order.
#include "ka_attention_decode.h"
#include "ka_no_alloc.h"

#include <mutex>
#include <type_traits>

// A lane's value combined with that of the lane 32 away (the two hold the halves of one query's
// scores): v_permlane32_swap exchanges the halves of two registers inside the vector unit, where a
// shuffle would make a trip through LDS.
__device__ __forceinline__ float at_max_with_other_half(float x) {
    typedef __attribute__((ext_vector_type(2))) unsigned at_u2;
    const at_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float at_sum_with_other_half(float x) {
    typedef __attribute__((ext_vector_type(2))) unsigned at_u2;
    const at_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}


// ----------------------------------------------------------------------------------------------
// prompt kernel
// ----------------------------------------------------------------------------------------------
constexpr int AP_WAVES = 4;                 // waves of a workgroup: all on the same 32 queries, keys interleaved
constexpr int AP_QBLOCK = 32;               // queries per workgroup
constexpr float AP_MAX_SLACK = 8.0f;        // powers of two the running maximum may grow before the outputs are rescaled
constexpr float AP_SUM_LIMIT = 4096.0f;     // a query's exponentials of one tile may add up to this before the tile is run again with a new reference point
constexpr int AP_MAX_TABLE = 24576;         // most block table entries of one row kept in LDS (393k keys)
constexpr int ap_merge_floats(int hd) { return (hd + 31) / 32 * 16 + 2; }
// block table entries of one row that fit in LDS beside the merge at head size hd
constexpr int ap_max_table(int hd) {
    int left = (160 * 1024 - (AP_WAVES - 1) * ap_merge_floats(hd) * KA_WAVE * 4 - 256) / 4;
    return left < AP_MAX_TABLE ? left : AP_MAX_TABLE;
}

// Registers: with 256 a lane (two waves per SIMD) the compiler lets the MFMAs write ordinary
// registers; left to itself it puts their results in accumulator registers and then spends a third
// of the loop's instructions moving them to where the softmax can read them. Two blocks of queries
// fit in 256 registers up to head size 64 (the prompt attention of 2,048 tokens: 63 to 48 us a
// layer); beyond that they would take a SIMD's registers for one wave, which was measured far
// slower than one block and two waves (head size 80: 98 against 63 us, 128: 267 against 139 us).
// One block fits two waves a SIMD up to head size 128 (204 registers; told that one wave is enough
// the compiler spread out over 280: 124 against 107 to 111 us at head size 128, 94 against 73 to 77
// at 112, a prompt of 2,048 tokens with 32 heads).
constexpr int ap_waves_per_simd(int hd, int qb) { return qb == 1 ? (hd <= 128 ? 2 : 1) : (hd <= 64 ? 2 : 1); }

// QB blocks of 32 queries per workgroup: every tile of keys and values that a wave fetches serves
// QB tiles of scores (the fetches, their addresses and the block table look-ups are shared).
template <int HD, int QB>
__global__ void __launch_bounds__(KA_WAVE * AP_WAVES) __attribute__((amdgpu_waves_per_eu(ap_waves_per_simd(HD, QB))))
attn_prefill_kernel(const bf16_t* __restrict__ q, long q_row_stride, const bf16_t* __restrict__ k_cache,
                    const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table, int max_pages,
                    const int* __restrict__ qblk_row, const int* __restrict__ qblk_tok,
                    const int* __restrict__ cu_q, const int* __restrict__ kv_len,
                    const int* __restrict__ kv_lo, const int* __restrict__ kv_hi, bf16_t* __restrict__ out,
                    long out_row_stride, float scale, int H, int Hkv, int table_entries) {
    static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head sizes in steps of 16 up to 256");
    static_assert(QB == 1 || QB == 2, "one or two blocks of queries");
    constexpr int QC = HD / 16;          // 16-byte chunks of half a head row = MFMA steps of the score product
    constexpr int DB = (HD + 31) / 32;   // 32-channel blocks of the output
    // A head size that is no multiple of 32 leaves the last block half used: its lanes 16..31
    // load the channels of lanes 0..15 once more, and what they compute is never stored.
    constexpr bool HALF_BLOCK = HD % 32 != 0;
    constexpr int REC = ap_merge_floats(HD);   // floats a lane hands over at the merge: its outputs, m and l
    __shared__ float mrg[AP_WAVES - 1][REC][KA_WAVE];
    extern __shared__ int pages[];       // the row's block table: `table_entries` of them
    // Heads are the fast index of the grid: the workgroups that run side by side then have the
    // same amount of work (the host lists the blocks of queries with the most keys first, so
    // the launch ends with the short ones), and an XCD, which gets every eighth workgroup,
    // keeps to the keys and values of a few heads.
    const int h = blockIdx.x, blk = blockIdx.y;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / KA_WAVE), lane = threadIdx.x % KA_WAVE;
    const int li = lane % 32, lg = lane / 32;
    const int kvh = h / (H / Hkv);
    const int row = qblk_row[blk];
    const int tok_end = cu_q[row + 1];
    // A block that starts behind its row's last token holds no query (the unused end of a list of
    // blocks of fixed length, as a captured step has it): nothing to do, and nothing more to look up.
    if (qblk_tok[blk] >= tok_end) return;
    int t[QB], tq[QB], hi[QB], lo[QB];
    bool q_valid[QB];
    int wave_hi = 0, wave_lo = 0x7fffffff;
    // lowest end and highest start of the visible ranges of the wave's queries: a tile inside
    // [max_lo, min_hi) is seen whole by every query and needs no mask
    int min_hi = 0x7fffffff, max_lo = 0;
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        t[b] = qblk_tok[blk] + b * 32 + li;
        q_valid[b] = t[b] < tok_end;
        tq[b] = q_valid[b] ? t[b] : tok_end - 1;
        hi[b] = q_valid[b] ? kv_hi[tq[b]] : 0;
        lo[b] = kv_lo ? kv_lo[tq[b]] : 0;
        wave_hi = max(wave_hi, hi[b]);
        if (q_valid[b]) {
            wave_lo = min(wave_lo, lo[b]);
            min_hi = min(min_hi, hi[b]);
            max_lo = max(max_lo, lo[b]);
        }
    }
    wave_hi = ka_lanes_reduce<1, KA_WAVE>(wave_hi, KaIntMax{});
    wave_lo = ka_lanes_reduce<1, KA_WAVE>(wave_lo, KaIntMin{});
    min_hi = ka_lanes_reduce<1, KA_WAVE>(min_hi, KaIntMin{});
    max_lo = ka_lanes_reduce<1, KA_WAVE>(max_lo, KaIntMax{});
    const int limit = kv_len[row];       // keys of this row that hold data
    // (the same in every lane: told to the compiler, which then counts tiles and looks up whole
    // pages in scalar registers)
    wave_hi = __builtin_amdgcn_readfirstlane(min(wave_hi, limit));
    wave_lo = __builtin_amdgcn_readfirstlane(wave_lo);
    min_hi = __builtin_amdgcn_readfirstlane(min_hi);
    max_lo = __builtin_amdgcn_readfirstlane(max_lo);
    // The row's block table goes to LDS once: a look-up per tile in global memory would put a
    // second trip to memory in front of every load of keys and values. (The host sees to it that
    // the table is long enough for every row of the launch.)
    const int n_pages = min((limit + AT_PAGE - 1) / AT_PAGE, table_entries);
    {
        const int* bt = block_table + (size_t)row * max_pages;
        for (int i = threadIdx.x; i < n_pages; i += KA_WAVE * AP_WAVES) pages[i] = bt[i];
        __syncthreads();
    }
    // A block whose queries see no key at all (the rows that pad a captured batch): zeros, and no
    // load is made from a table that has no entry.
    if (wave_hi <= wave_lo || n_pages <= 0) {
        if (wave == 0) {
#pragma unroll
            for (int b = 0; b < QB; ++b) {
                if (!q_valid[b]) continue;
                bf16_t* op = out + (size_t)t[b] * out_row_stride + (size_t)h * HD + lg * (HD / 2);
#pragma unroll
                for (int c = 0; c < QC; ++c) *reinterpret_cast<bf16x8*>(op + c * 8) = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
            }
        }
        return;
    }

    // queries: lane (q = li, g = lg) holds channels [g * HD/2, (g + 1) * HD/2)
    bf16x8 qreg[QB][QC];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        const bf16_t* qp = q + (size_t)tq[b] * q_row_stride + (size_t)h * HD + lg * (HD / 2);
#pragma unroll
        for (int c = 0; c < QC; ++c) qreg[b][c] = at_load8(qp + c * 8);
    }
    floatx16 o[QB][DB];
    float m_i[QB], m_ref[QB], l_i[QB];
    bool settled = false;                // every live query of the wave has a reference point (the same in all lanes)
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        m_i[b] = -INFINITY;
        m_ref[b] = 0.f;                  // m_i, or 0 while that is -inf
        l_i[b] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[b][db][v] = 0.f;
    }
    const float sl2 = scale * AT_LOG2E;
    const int kperm = (li & 16) | ((li & 4) << 1) | ((li & 8) >> 1) | (li & 3);

    // Every load of the loop is issued whether its tile exists or not, from an address moved
    // inside the row's live keys: a load under a branch would make the compiler wait for
    // everything in flight, and the loop would pay a trip to the cache per tile.
    const int last_live = n_pages * AT_PAGE < limit ? n_pages * AT_PAGE - 1 : limit - 1;   // (inside the table in LDS, whatever the host said)
    const int first_live = min(wave_lo, last_live);                  // pages below wave_lo may have been given back
    const size_t page_stride = (size_t)Hkv * AT_PAGE * HD;           // elements of a page, keys or values
    const unsigned k_lane = (unsigned)(kvh * AT_PAGE * HD + lg * (HD / 2));
    const unsigned v_lane = (unsigned)((kvh * HD + li) * AT_PAGE + lg * 8);
    const unsigned v_lane_half = (unsigned)((kvh * HD + (DB - 1) * 32 + (li & 15)) * AT_PAGE + lg * 8);

    // half a key row of tile `key0` for this lane's (permuted) key
    auto key_address = [&](int key0) -> const bf16_t* {
        unsigned key = (unsigned)min(max(key0 + kperm, first_live), last_live);
        unsigned page = (unsigned)pages[key / AT_PAGE];
        return k_cache + ((size_t)page * page_stride + (k_lane + (key % AT_PAGE) * HD));
    };
    auto load_keys_at = [&](const bf16_t* kp, bf16x8* dst) {
#pragma unroll
        for (int c = 0; c < QC; ++c) dst[c] = at_load8(kp + c * 8);
    };
    auto load_keys = [&](int key0, bf16x8* dst) { load_keys_at(key_address(key0), dst); };

    // the two value pages of tile `key0`: lane (d = li, g) loads 8 consecutive keys of channel d.
    // The page is the same for all lanes: its address is made in scalar registers.
    // (the pages are looked up a tile ahead, `value_pages`: the loads of a tile then start at once)
    auto value_pages = [&](int key0, unsigned* page) {
#pragma unroll
        for (int pg = 0; pg < 2; ++pg) {
            unsigned kbase = (unsigned)min(max(key0 + pg * AT_PAGE, first_live), last_live);
            page[pg] = (unsigned)__builtin_amdgcn_readfirstlane(pages[kbase / AT_PAGE]);
        }
    };
    auto load_values = [&](const unsigned* page, bf16x8 (*dst)[DB]) {
#pragma unroll
        for (int pg = 0; pg < 2; ++pg) {
            const bf16_t* vp = v_cache + (size_t)page[pg] * page_stride;
#pragma unroll
            for (int db = 0; db < DB; ++db)
                dst[pg][db] = at_load8(vp + (HALF_BLOCK && db == DB - 1 ? v_lane_half : v_lane + db * 32 * AT_PAGE));
        }
    };
    // what of them may be used: nothing of a page outside the wave's keys (another page was
    // loaded in its place), and nothing past the row's data, whose slots may hold anything
    auto mask_values = [&](int key0, bf16x8 (*dst)[DB]) {
        const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int pg = 0; pg < 2; ++pg) {
            int kbase = key0 + pg * AT_PAGE;
            bool live = kbase < wave_hi && kbase + AT_PAGE > wave_lo;
            int first = kbase + lg * 8;      // first of the 8 keys this lane loaded
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (!live) dst[pg][db] = zero;
                else if (kbase + AT_PAGE > limit) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (first + j >= limit) dst[pg][db][j] = (bf16_t)0.f;
                }
            }
        }
    };

    constexpr int STRIDE = 32 * AP_WAVES;
    // One tile of 32 keys whose key rows are in `kr`, which the next tile's then take, in two forms.
    // Careful: the softmax looks for the tile's maximum and moves the queries' reference point where
    // it has to. Plain (most tiles): the exponentials are taken straight from the reference point the
    // queries have and no maximum is looked for; a tile whose scores lie far above that point shows
    // in the sum of its exponentials (an overflow as infinity): the tile then adds zeros and `false`
    // is returned, for the tile to be run again carefully.
    auto process = [&](auto careful_tag, int key0, bf16x8* kr, unsigned* vpage) -> bool {
        constexpr bool CAREFUL = decltype(careful_tag)::value;
        bf16x8 vr[2][DB];
        load_values(vpage, vr);                            // in flight during the scores and the softmax
        __builtin_amdgcn_sched_barrier(0);
        // where the next tile's keys and values are: worked out beside the matrix products
        const bf16_t* next_keys = key_address(key0 + STRIDE);
        value_pages(key0 + STRIDE, vpage);
        const bool whole = key0 >= max_lo && key0 + 32 <= min_hi;
        // the scores of all blocks of queries first: the matrix pipes work on the later ones while
        // the softmax of the first is computed, and the blocks' chains of dependent instructions
        // (exchange with the other half of the wave, exponentials, sum) interleave
        floatx16 s[QB];
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) s[b][v] = 0.f;
#pragma unroll
        for (int c = 0; c < QC; ++c)               // (the blocks take turns: an MFMA that adds to the one before it waits for it)
#pragma unroll
            for (int b = 0; b < QB; ++b) s[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kr[c], qreg[b][c], s[b], 0, 0, 0);
        // The next tile's key rows go into the registers that the products above have read: in flight
        // until the next tile. (Two sets of registers taken in turn made the compiler keep the
        // outputs in two places as well and copy all 64 registers of them over in every tile.)
        __builtin_amdgcn_sched_barrier(0);
        load_keys_at(next_keys, kr);
        __builtin_amdgcn_sched_barrier(0);
        // lane holds, for its query, the keys key0 + (v / 8) * 16 + lg * 8 + v % 8
        if (!whole) {
#pragma unroll
            for (int b = 0; b < QB; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int key = key0 + (v / 8) * 16 + lg * 8 + (v % 8);
                    if (!(key >= lo[b] && key < hi[b])) s[b][v] = -INFINITY;
                }
        }
        bf16x8 pb[QB][2];
        bool again = false;
        if constexpr (!CAREFUL) {
            float total[QB];
            bool over = false;
#pragma unroll
            for (int b = 0; b < QB; ++b) {
                float rowsum = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float p = __builtin_amdgcn_exp2f(fmaf(s[b][v], sl2, -m_ref[b]));
                    rowsum += p;
                    pb[b][v / 8][v % 8] = (bf16_t)p;
                }
                total[b] = at_sum_with_other_half(rowsum);
                over = over || !(total[b] <= AP_SUM_LIMIT);
            }
            if (__any(over)) {                  // (a side path that only clears what the tile would add)
                again = true;
#pragma unroll
                for (int b = 0; b < QB; ++b) {
                    total[b] = 0.f;
                    pb[b][0] = pb[b][1] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
                }
            }
#pragma unroll
            for (int b = 0; b < QB; ++b) l_i[b] += total[b];
        } else {
            float alpha[QB];
            bool moved = false, unset = false;
#pragma unroll
            for (int b = 0; b < QB; ++b) {
                float mx = s[b][0];
#pragma unroll
                for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[b][v]);
                mx = at_max_with_other_half(mx) * sl2;              // the scale is positive: max and scale commute
                // The reference point follows the maximum only when that has grown by more than
                // AP_MAX_SLACK (in powers of two): softmax does not care which point is taken, an
                // exponential of up to 2^AP_MAX_SLACK is as exact in fp32 and bf16 as one below 1, and the
                // outputs so far need no rescaling.
                const bool grow = mx > m_i[b] + AP_MAX_SLACK;       // (also from -inf to the first finite maximum)
                const float m_new = grow ? mx : m_i[b];
                const float m_use = m_new == -INFINITY ? 0.f : m_new;     // nothing visible yet: keep everything at zero
                alpha[b] = grow ? __builtin_amdgcn_exp2f(m_i[b] - m_use) : 1.0f;
                float rowsum = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float p = __builtin_amdgcn_exp2f(fmaf(s[b][v], sl2, -m_use));
                    rowsum += p;
                    pb[b][v / 8][v % 8] = (bf16_t)p;
                }
                rowsum = at_sum_with_other_half(rowsum);
                l_i[b] = l_i[b] * alpha[b] + rowsum;
                m_i[b] = m_new;
                m_ref[b] = m_use;
                moved = moved || alpha[b] != 1.0f;
                unset = unset || (q_valid[b] && m_new == -INFINITY);
            }
            settled = !__any(unset);
            if (__any(moved)) {
#pragma unroll
                for (int b = 0; b < QB; ++b)
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int v = 0; v < 16; ++v) o[b][db][v] *= alpha[b];
            }
        }
        // O^T[d][query] += V^T[d][key] P^T[key][query], one page per MFMA
        if (key0 + 32 > min(wave_hi, limit) || key0 < wave_lo) mask_values(key0, vr);
#pragma unroll
        for (int pg = 0; pg < 2; ++pg)
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int b = 0; b < QB; ++b)
                    o[b][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vr[pg][db], pb[b][pg], o[b][db], 0, 0, 0);
        return !again;
    };

    // the next tile's keys are always in flight while a tile is processed
    bf16x8 kr[QC];
    int key0 = (wave_lo & ~31) + wave * 32;
    // Careful tiles until every live query has a reference point (a wave's first tile at the least),
    // plain ones from there on, and back whenever a plain one has found scores too far above it.
    unsigned vpage[2];
    while (key0 < wave_hi) {
        load_keys(key0, kr);
        value_pages(key0, vpage);
        do {
            process(std::true_type{}, key0, kr, vpage);
            key0 += STRIDE;
        } while (key0 < wave_hi && !settled);
        while (key0 < wave_hi && process(std::false_type{}, key0, kr, vpage)) key0 += STRIDE;
    }
    // the waves took different keys of the same queries: merge in wave order, a block of queries at a time
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        if (b > 0) __syncthreads();                        // the first block's sums have been read
        if (wave > 0) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) mrg[wave - 1][db * 16 + v][lane] = o[b][db][v];
            mrg[wave - 1][DB * 16][lane] = m_i[b];
            mrg[wave - 1][DB * 16 + 1][lane] = l_i[b];
        }
        __syncthreads();
        if (wave > 0 || !q_valid[b]) continue;
        float M = m_i[b];
#pragma unroll
        for (int w = 0; w < AP_WAVES - 1; ++w) M = fmaxf(M, mrg[w][DB * 16][lane]);
        float f0 = m_i[b] == -INFINITY ? 0.f : exp2f(m_i[b] - M);
        float L = l_i[b] * f0;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[b][db][v] *= f0;
#pragma unroll
        for (int w = 0; w < AP_WAVES - 1; ++w) {
            float mw = mrg[w][DB * 16][lane];
            float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
            L += mrg[w][DB * 16 + 1][lane] * f;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[b][db][v] += mrg[w][db * 16 + v][lane] * f;
        }
        float inv = L > 0.f ? 1.0f / L : 0.f;
        bf16_t* op = out + (size_t)t[b] * out_row_stride + (size_t)h * HD;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                if (db * 32 + qd * 8 >= HD) continue;          // the unused half of the last block
                int d = db * 32 + qd * 8 + lg * 4;
                bf16x4 r = {(bf16_t)(o[b][db][qd * 4 + 0] * inv), (bf16_t)(o[b][db][qd * 4 + 1] * inv),
                            (bf16_t)(o[b][db][qd * 4 + 2] * inv), (bf16_t)(o[b][db][qd * 4 + 3] * inv)};
                *reinterpret_cast<bf16x4*>(op + d) = r;
            }
    }
}

// ----------------------------------------------------------------------------------------------
// decode kernel (its body: ka_attention_decode.h)
// ----------------------------------------------------------------------------------------------
// (four waves per SIMD are all that a workgroup of 16 waves allows; head sizes of 80 to 128 fit four
// a SIMD as well, in 120 to 124 registers (112: three; it would spill two), larger ones two; saying so
// keeps the compiler from trading loads in flight for an occupancy the kernel cannot have. Head size
// 80 at two a SIMD, as it was: 4.62k against 4.89k tok/s at batch 12, 6.75k against 7.32k at 24, 8.80k
// against 9.72k at 48, 9.79k against 9.98k at 64, at 32 layers of Phi-2's sizes. Workgroups of four waves, which many rows get, fit five to a
// CU with tiles of 64 keys: 15.7k to 16.1k tok/s at batch 64. With tiles of 32 keys they need 56
// registers a lane and fit eight to a CU: the 2,048 workgroups of 64 rows x 32 heads then run all at
// once instead of in a round of 1,280 and one of 768: 17.8k -> 18.0k tok/s at batch 64, 15.9k -> 16.5k
// at 48, 11.9k -> 12.8k at 24, measured at 1,024 keys a row.)
constexpr int ad_waves_per_simd(int HD, int WAVES, int TP) {
    return HD > 128 ? 2 : HD > 64 ? (HD > 96 && HD < 128 ? 3 : 4) : (WAVES == 4 && TP <= 2 ? 8 : WAVES == 4 && TP <= 4 ? 5 : 4);
}
constexpr int AD_SMALL_TILE_PAGES = 2;
constexpr int AD_SMALL_TILE_MAX_PAGES = 128;   // rows of up to this many pages get the small tiles

template <int HD, int WAVES, int TP>
__global__ void __launch_bounds__(KA_WAVE * WAVES)
    __attribute__((amdgpu_waves_per_eu(ad_waves_per_simd(HD, WAVES, TP), ad_waves_per_simd(HD, WAVES, TP))))
attn_decode_kernel(const bf16_t* __restrict__ q, long q_row_stride, const bf16_t* __restrict__ k_cache,
                   const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table, int max_pages,
                   const int* __restrict__ token_row, const int* __restrict__ kv_lo,
                   const int* __restrict__ kv_hi, bf16_t* __restrict__ out, long out_row_stride, float scale,
                   int H, int Hkv, float* __restrict__ partial, DecodeFuse fz) {
    attn_decode_body<HD, WAVES, false, TP>(q, q_row_stride, k_cache, v_cache, block_table, max_pages, token_row, kv_lo, kv_hi,
                                           out, out_row_stride, scale, H, Hkv, partial, fz, blockIdx.x, blockIdx.y, blockIdx.z,
                                           gridDim.z);
}

// ----------------------------------------------------------------------------------------------
// rotary encoding + cache write, a page's worth of tokens per workgroup
// ----------------------------------------------------------------------------------------------
// A group of workgroups (grid y) takes a run of up to 16 consecutive tokens of the packed batch: the
// runs the host lists (`run_first`, `run_count`: the tokens that fill a page of their row in order
// are a run of their own, whatever their place in the batch), else every 16 tokens. Queries are
// rotated in place and keys rotated into the cache with 16-byte loads and stores (8 channels of a
// head and their 8 partners in the other half of the rotated part per thread; the channels of a
// key that are not rotated are copied, those of a query left alone). Values: the cache keeps a
// page transposed, [channel][16 tokens]; when the 16 tokens fill one page in order (which they do
// inside a prompt that starts on a page boundary) they are turned through LDS, 256 channels at a
// time; other tokens are stored one by one. The first `light_parts`
// workgroups of a group share the queries and keys, one piece of work per thread and round, the
// others the values. (One workgroup of sixteen turning all the values in registers, its stores 256
// bytes apart, and threads that met a query's plain channels with nothing to do: 18.7 us for 2,048
// tokens of 32 heads of 64 launched back to back, against 13.1 us now.)
constexpr int RC_TOKENS = AT_PAGE;
constexpr int RC_THREADS = 256;
constexpr int RC_VCHANNELS = 256;           // channels of the values that a workgroup turns at a time

__global__ void __launch_bounds__(RC_THREADS)
rope_cache_pages_kernel(bf16_t* __restrict__ qkv, long row_stride, const int* __restrict__ positions,
                        const int* __restrict__ slots, const float* __restrict__ table,
                        bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int n, int H, int Hkv,
                        int hd, int rot, int light_parts, const int* __restrict__ run_first,
                        const int* __restrict__ run_count) {
    const int t0 = run_first ? run_first[blockIdx.x] : blockIdx.x * RC_TOKENS;
    const int n_here = run_first ? min(run_count[blockIdx.x], min(RC_TOKENS, n - t0)) : min(RC_TOKENS, n - t0);
    if (t0 < 0 || n_here <= 0) return;
    const int half = rot / 2;
    const int pair_units = half / 8;                  // per head: 8 channels + their 8 partners
    const int plain_units = (hd - rot) / 8;           // per head: 8 channels that are not rotated
    const size_t page_elems = (size_t)Hkv * AT_PAGE * hd;
    // (rows padded by 8 bytes: the two halves of the tokens, which neighbouring lanes read, then lie 16 banks apart)
    __shared__ __attribute__((aligned(8))) bf16_t vtile[RC_TOKENS][RC_VCHANNELS + 4];

    if ((int)blockIdx.y < light_parts) {
        // Rotated pairs of the queries: (token, head, unit), the order of the rows of `qkv`; of the keys:
        // (kv head, token, unit), the order of the page; then the plain channels of the keys, likewise:
        // neighbouring lanes write neighbouring addresses
        const int q_items = n_here * H * pair_units, k_items = slots ? n_here * Hkv * pair_units : 0;
        const int pair_items = q_items + k_items;
        const int items = pair_items + (slots ? n_here * Hkv * plain_units : 0);
        const int lanes = light_parts * RC_THREADS;
        for (int idx = blockIdx.y * RC_THREADS + threadIdx.x; idx < items; idx += lanes) {
            if (idx < pair_items) {
                const bool is_key = idx >= q_items;
                int i, head, c0;
                if (!is_key) {
                    i = idx / (H * pair_units);
                    head = idx % (H * pair_units) / pair_units;
                } else {
                    const int j = idx - q_items;
                    head = H + j / (n_here * pair_units);
                    i = j % (n_here * pair_units) / pair_units;
                }
                c0 = idx % pair_units * 8;                               // (q_items is a multiple of pair_units)
                const int t = t0 + i;
                const int slot = is_key ? slots[t] : -1;
                if (is_key && slot < 0) continue;                       // nothing is cached for this token
                bf16_t* src = qkv + (size_t)t * row_stride + (size_t)head * hd;     // the keys follow the queries
                bf16_t* dst = src;
                if (is_key) dst = k_cache + (size_t)(slot / AT_PAGE) * page_elems + ((size_t)(head - H) * AT_PAGE + slot % AT_PAGE) * hd;
                bf16x8 a = at_load8(src + c0), b = at_load8(src + half + c0);
                const float* cs = table + (size_t)positions[t] * rot;
                floatx4 c[2] = {*reinterpret_cast<const floatx4*>(cs + c0), *reinterpret_cast<const floatx4*>(cs + c0 + 4)};
                floatx4 sn[2] = {*reinterpret_cast<const floatx4*>(cs + half + c0), *reinterpret_cast<const floatx4*>(cs + half + c0 + 4)};
                bf16x8 ra, rb;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    float x = (float)a[j], y = (float)b[j], cc = c[j / 4][j % 4], ss = sn[j / 4][j % 4];
                    ra[j] = (bf16_t)(x * cc - y * ss);
                    rb[j] = (bf16_t)(y * cc + x * ss);
                }
                *reinterpret_cast<bf16x8*>(dst + c0) = ra;
                *reinterpret_cast<bf16x8*>(dst + half + c0) = rb;
            } else {
                const int j = idx - pair_items;                          // (kv head, token, unit): neighbouring lanes, neighbouring addresses in the page
                const int kvh = j / (n_here * plain_units), rest = j % (n_here * plain_units);
                const int i = rest / plain_units, c0 = rot + (rest % plain_units) * 8;
                const int t = t0 + i, slot = slots[t];
                if (slot < 0) continue;
                const bf16_t* src = qkv + (size_t)t * row_stride + (size_t)(H + kvh) * hd;
                bf16_t* dst = k_cache + (size_t)(slot / AT_PAGE) * page_elems + ((size_t)kvh * AT_PAGE + slot % AT_PAGE) * hd;
                *reinterpret_cast<bf16x8*>(dst + c0) = at_load8(src + c0);
            }
        }
        return;
    }
    if (!slots) return;

    // values
    const int lane_id = (blockIdx.y - light_parts) * RC_THREADS + threadIdx.x, lanes = (gridDim.y - light_parts) * RC_THREADS;
    const int first = slots[t0];
    bool whole_page = n_here == RC_TOKENS && first >= 0 && first % AT_PAGE == 0;
    if (whole_page) {
        for (int i = 1; i < RC_TOKENS; ++i) whole_page = whole_page && slots[t0 + i] == first + i;   // (the same for all threads)
    }
    const int vwidth = Hkv * hd;
    const bf16_t* vsrc = qkv + (size_t)t0 * row_stride + (size_t)(H + Hkv) * hd;
    if (whole_page) {
        // 256 channels of the 16 tokens at a time through LDS: read as 16-byte pieces of a token's row,
        // written as 16-byte pieces of a channel's row of the page (8 tokens), neighbouring lanes
        // neighbouring addresses both times
        bf16_t* vpage = v_cache + (size_t)(first / AT_PAGE) * page_elems;
        for (int cs = (blockIdx.y - light_parts) * RC_VCHANNELS; cs < vwidth; cs += (gridDim.y - light_parts) * RC_VCHANNELS) {
            if (cs != (int)(blockIdx.y - light_parts) * RC_VCHANNELS) __syncthreads();      // the slice before has been read
#pragma unroll
            for (int r = 0; r < RC_TOKENS * RC_VCHANNELS / 8 / RC_THREADS; ++r) {
                const int idx = threadIdx.x + r * RC_THREADS;
                const int i = idx / (RC_VCHANNELS / 8), c0 = idx % (RC_VCHANNELS / 8) * 8;
                if (cs + c0 < vwidth) {
                    const bf16x8 piece = at_load8(vsrc + (size_t)i * row_stride + cs + c0);
                    bf16x4* to = reinterpret_cast<bf16x4*>(&vtile[i][c0]);
                    to[0] = bf16x4{piece[0], piece[1], piece[2], piece[3]};
                    to[1] = bf16x4{piece[4], piece[5], piece[6], piece[7]};
                }
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < RC_VCHANNELS * 2 / RC_THREADS; ++r) {
                const int c = threadIdx.x / 2 + r * (RC_THREADS / 2), part = threadIdx.x % 2;
                if (cs + c < vwidth) {
                    bf16x8 piece;
#pragma unroll
                    for (int i = 0; i < 8; ++i) piece[i] = vtile[part * 8 + i][c];
                    // channel cs + c = (head, d): its 16 tokens are one row of the page
                    *reinterpret_cast<bf16x8*>(vpage + (size_t)(cs + c) * AT_PAGE + part * 8) = piece;
                }
            }
        }
    } else {
        // tokens of different rows, or of a page's middle: eight channels of a token per thread, one load
        // of 16 bytes and eight stores of one value into the token's column of its page
        const int chunks = vwidth / 8;
        for (int idx = lane_id; idx < n_here * chunks; idx += lanes) {
            const int i = idx / chunks, c0 = idx % chunks * 8;
            const int slot = slots[t0 + i];
            if (slot < 0) continue;
            const bf16x8 piece = at_load8(vsrc + (size_t)i * row_stride + c0);
            bf16_t* col = v_cache + (size_t)(slot / AT_PAGE) * page_elems + (size_t)c0 * AT_PAGE + slot % AT_PAGE;
#pragma unroll
            for (int j = 0; j < 8; ++j) col[j * AT_PAGE] = piece[j];
        }
    }
}

// Rotates q in place (the first `rot` channels of every head, halves paired) and writes rotated
// keys and the values into the paged cache (slots null: rotates q only; a slot < 0: that token is
// not cached). bf16, pages of 16, head size and rot / 2 multiples of 8, rows 16-byte aligned.
KA_API int ka_rope_cache_pages_supported(int hd, int rot, int page_size) {
    return page_size == AT_PAGE && hd % 8 == 0 && rot > 0 && rot % 16 == 0 && rot <= hd;
}

KA_API int ka_rope_cache_pages_bf16(void* qkv, long row_stride, const int* positions, const int* slots,
                                    const float* table, int table_rows, void* k_cache, void* v_cache, int n, int H,
                                    int Hkv, int hd, int rot, int page_size, const int* run_first,
                                    const int* run_count, int n_runs, hipStream_t stream) {
    const char* who = "ka_rope_cache_pages_bf16";
    KA_CHECK(n >= 0 && H > 0 && Hkv > 0, "%s: bad sizes", who);
    KA_CHECK(ka_rope_cache_pages_supported(hd, rot, page_size), "%s: head size %d, rotary size %d, page size %d not covered", who, hd, rot, page_size);
    KA_CHECK(row_stride >= (long)(H + 2 * Hkv) * hd && row_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0, "%s: rows must be 16-byte aligned and hold q, k and v", who);
    KA_CHECK(table && table_rows > 0 && (uintptr_t)table % 16 == 0, "%s: rotary table missing or not 16-byte aligned", who);
    KA_CHECK(!slots || (k_cache && v_cache && (uintptr_t)k_cache % 16 == 0 && (uintptr_t)v_cache % 16 == 0), "%s: cache tensors missing or not 16-byte aligned", who);
    KA_CHECK((run_first == nullptr) == (run_count == nullptr) && n_runs >= 0, "%s: the runs of tokens come as two lists", who);
    if (n == 0 || (run_first && n_runs == 0)) return 0;
    // (runs: every token in exactly one, none longer than 16: the host's promise)
    const int groups = run_first ? n_runs : ka_cdiv(n, RC_TOKENS);
    // workgroups per group of tokens: a piece of work per thread for queries and keys, as many for
    // the values as have a piece each, and no more than fill the chip a few times over
    const int pair_units = rot / 16, plain_units = (hd - rot) / 8;
    const long light_items = (long)RC_TOKENS * ((H + Hkv) * pair_units + (slots ? Hkv * plain_units : 0));
    int light_parts = ka_cdiv(light_items, RC_THREADS), value_parts = slots ? ka_cdiv((long)Hkv * hd, RC_VCHANNELS) : 0;
    const int most = groups >= 256 ? 16 : 64;
    if (light_parts > most) light_parts = most;
    if (value_parts > most / 4) value_parts = most / 4;
    hipLaunchKernelGGL(rope_cache_pages_kernel, dim3(groups, light_parts + value_parts), dim3(RC_THREADS), 0, stream,
                       (bf16_t*)qkv, row_stride, positions, slots, table, (bf16_t*)k_cache, (bf16_t*)v_cache, n, H, Hkv, hd,
                       rot, light_parts, run_first, run_count);
    KA_LAUNCH_CHECK();
    return 0;
}

// Head sizes in steps of 16 up to 128 and in steps of 32 up to 256.
static bool at_head_size_covered(int hd) {
    return hd >= 16 && hd <= 256 && hd % 16 == 0 && (hd <= 128 || hd % 32 == 0);
}

KA_API int ka_attention_prefill_supported(int hd, int page_size) {
    return page_size == AT_PAGE && at_head_size_covered(hd);
}

// Keys of one row that the prompt kernel takes at this head size (its block table lies in LDS).
KA_API int ka_attention_prefill_max_keys(int hd) {
    return at_head_size_covered(hd) ? ap_max_table(hd) * AT_PAGE : 0;
}

KA_API int ka_attention_decode_supported(int hd, int page_size) {
    return page_size == AT_PAGE && at_head_size_covered(hd);
}

// Queries of one row that a workgroup of the prompt kernel takes at this head size: the blocks the
// host lists (`qblk_row`, `qblk_tok`) must be cut to this size, or to 32, which every head size takes.
KA_API int ka_attention_prefill_query_block(int hd) {
    return at_head_size_covered(hd) && hd <= 64 ? 64 : 32;
}

KA_API int ka_attention_prefill_bf16(const void* q, long q_row_stride, const void* k_cache, const void* v_cache,
                                     const int* block_table, int max_pages, const int* qblk_row,
                                     const int* qblk_tok, int n_qblocks, const int* cu_q, const int* kv_len,
                                     const int* kv_lo, const int* kv_hi, void* out, long out_row_stride,
                                     float scale, int H, int Hkv, int hd, int page_size, int longest_row,
                                     int query_block, hipStream_t stream) {
    if (check_common("ka_attention_prefill_bf16", q, q_row_stride, out, out_row_stride, n_qblocks, H, Hkv, hd,
                     page_size, max_pages))
        return -1;
    KA_CHECK(ka_attention_prefill_supported(hd, page_size), "ka_attention_prefill_bf16: head size %d not covered", hd);
    // (the kernel takes maxima of unscaled scores and turns masked scores into -inf before it scales them)
    KA_CHECK(scale > 0.f && scale < INFINITY, "ka_attention_prefill_bf16: the scale must be positive and finite, got %g", (double)scale);
    KA_CHECK(query_block == 32 || (query_block == 64 && ka_attention_prefill_query_block(hd) == 64),
             "ka_attention_prefill_bf16: blocks of %d queries at head size %d (32%s)", query_block, hd,
             ka_attention_prefill_query_block(hd) == 64 ? " or 64" : " only");
    // `longest_row`: no row of the launch holds more keys than this (0: not known, the whole
    // width of the block table is kept in LDS)
    int table_entries = max_pages;
    if (longest_row > 0 && ka_cdiv(longest_row, AT_PAGE) < max_pages) table_entries = ka_cdiv(longest_row, AT_PAGE);
    KA_CHECK(table_entries <= ap_max_table(hd), "ka_attention_prefill_bf16: a row of %d keys is longer than the %d this kernel takes at head size %d",
             table_entries * AT_PAGE, ap_max_table(hd) * AT_PAGE, hd);
    const size_t table_bytes = (size_t)table_entries * sizeof(int);
    KA_CHECK(n_qblocks <= 65535, "ka_attention_prefill_bf16: more than 65535 blocks of queries in one launch");
    dim3 grid(H, n_qblocks), block(KA_WAVE * AP_WAVES);
#define KA_AP_LAUNCH(HDV, QBV)                                                                                      \
    {                                                                                                               \
        static bool configured = false;                                                                             \
        if (!configured) {                                                                                          \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_prefill_kernel<HDV, QBV>),        \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, ap_max_table(HDV) * sizeof(int)); \
            KA_CHECK(e == hipSuccess, "ka_attention_prefill_bf16: cannot reserve LDS: %s", hipGetErrorString(e));   \
            configured = true;                                                                                      \
        }                                                                                                           \
        hipLaunchKernelGGL((attn_prefill_kernel<HDV, QBV>), grid, block, table_bytes, stream, (const bf16_t*)q,     \
                           q_row_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages,    \
                           qblk_row, qblk_tok, cu_q, kv_len, kv_lo, kv_hi, (bf16_t*)out, out_row_stride, scale, H,  \
                           Hkv, table_entries);                                                                     \
    }
#define KA_AP(HDV)                                                                                                  \
    case HDV:                                                                                                       \
        if (query_block == 64) KA_AP_LAUNCH(HDV, 2) else KA_AP_LAUNCH(HDV, 1)                                       \
        break;
#define KA_AP1(HDV) \
    case HDV: KA_AP_LAUNCH(HDV, 1) break;
    switch (hd) {
        KA_AP(16) KA_AP(32) KA_AP(48) KA_AP(64)
        KA_AP1(80) KA_AP1(96) KA_AP1(112) KA_AP1(128) KA_AP1(160) KA_AP1(192) KA_AP1(224) KA_AP1(256)
    }
#undef KA_AP
#undef KA_AP1
#undef KA_AP_LAUNCH
    KA_LAUNCH_CHECK();
    return 0;
}

KA_API long ka_attention_decode_partial_floats(int n, int H, int hd, int splits) {
    return (long)n * H * splits * (hd + 2);
}

static int decode_launch(const char* who, const void* q, long q_row_stride, const void* k_cache, const void* v_cache,
                         const int* block_table, int max_pages, const int* token_row, const int* kv_lo,
                         const int* kv_hi, void* out, long out_row_stride, float scale, int n, int H,
                         int Hkv, int hd, int page_size, int splits, int waves, float* partial,
                         long partial_floats, const void* k_new,
                         const void* v_new, long new_stride, const float* table, int rot,
                         const int* slots, void* k_cache_w, void* v_cache_w, hipStream_t stream) {
    DecodeFuse fz = {};
    if (decode_check(who, q, q_row_stride, out, out_row_stride, n, H, Hkv, hd, page_size, max_pages, splits, partial,
                     partial_floats, k_new, v_new, new_stride, table, rot, slots, k_cache_w, v_cache_w, &fz))
        return -1;
    KA_CHECK(waves == 4 || waves == 8 || waves == 16, "%s: waves must be 4, 8 or 16", who);
    if (hd > 64 && waves == 16) waves = 8;   // measured at head size 80: 16 waves 26.4 against 23.6 us at two waves per SIMD; at four a SIMD 3.80k against 3.84k tok/s at batch 8
    dim3 grid(n, H, splits), block(KA_WAVE * waves);
    // Workgroups of four waves that the chip holds all at once when eight of them share a CU (and that are not
    // so few that most CUs would hold one or none: then the larger tile's loads in flight count for more):
    // tiles of two pages (see ad_waves_per_simd).
    const long groups = (long)n * H * splits;
    const int cus = ka_compute_units();
    // (Rows of up to 2,048 keys, going by the width of the block table: behind 4,096 keys a row the larger tile
    // came out 2 to 3 % ahead at 24 and 32 rows, level at 48 and 64.)
    const bool small_tiles = waves == 4 && hd <= 64 && max_pages <= AD_SMALL_TILE_MAX_PAGES && groups * 2 >= 3L * cus && groups <= 8L * cus;
#define KA_AD(HDV, WV, TPV)                                                                                         \
    hipLaunchKernelGGL((attn_decode_kernel<HDV, WV, TPV>), grid, block, 0, stream, (const bf16_t*)q, q_row_stride, \
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, token_row, kv_lo,   \
                       kv_hi, (bf16_t*)out, out_row_stride, scale, H, Hkv, partial, fz)
#define KA_AD_SMALL(HDV)                                                                                            \
    case HDV:                                                                                                       \
        if (small_tiles) KA_AD(HDV, 4, AD_SMALL_TILE_PAGES); else if (waves == 4) KA_AD(HDV, 4, 4);                \
        else if (waves == 8) KA_AD(HDV, 8, 4); else KA_AD(HDV, 16, 4);                                              \
        break
#define KA_AD_LARGE(HDV)                                                                                            \
    case HDV:                                                                                                       \
        if (waves == 4) KA_AD(HDV, 4, 4); else KA_AD(HDV, 8, 4);                                                    \
        break
    switch (hd) {
        KA_AD_SMALL(16); KA_AD_SMALL(32); KA_AD_SMALL(48); KA_AD_SMALL(64);
        KA_AD_LARGE(80); KA_AD_LARGE(96); KA_AD_LARGE(112); KA_AD_LARGE(128);
        KA_AD_LARGE(160); KA_AD_LARGE(192); KA_AD_LARGE(224); KA_AD_LARGE(256);
    }
#undef KA_AD_SMALL
#undef KA_AD_LARGE
#undef KA_AD
    KA_LAUNCH_CHECK();
    if (splits > 1) {
#define KA_ADM(HDV)                                                                                                 \
    case HDV:                                                                                                       \
        hipLaunchKernelGGL(attn_decode_merge_kernel<HDV>, dim3(n, H), dim3(KA_WAVE), 0, stream, partial, splits,    \
                           (bf16_t*)out, out_row_stride, H);                                                        \
        break
        switch (hd) {
            KA_ADM(16); KA_ADM(32); KA_ADM(48); KA_ADM(64); KA_ADM(80); KA_ADM(96); KA_ADM(112); KA_ADM(128);
            KA_ADM(160); KA_ADM(192); KA_ADM(224); KA_ADM(256);
        }
#undef KA_ADM
        KA_LAUNCH_CHECK();
    }
    return 0;
}

KA_API int ka_attention_decode_bf16(const void* q, long q_row_stride, const void* k_cache, const void* v_cache,
                                    const int* block_table, int max_pages, const int* token_row, const int* kv_lo,
                                    const int* kv_hi, void* out, long out_row_stride, float scale, int n, int H,
                                    int Hkv, int hd, int page_size, int splits, int waves, float* partial,
                                    long partial_floats, const void* k_new,
                                    const void* v_new, long new_stride, const float* table, int rot,
                                    const int* slots, void* k_cache_w, void* v_cache_w, hipStream_t stream) {
    return decode_launch("ka_attention_decode_bf16", q, q_row_stride, k_cache, v_cache, block_table, max_pages, token_row,
                         kv_lo, kv_hi, out, out_row_stride, scale, n, H, Hkv, hd, page_size, splits, waves, partial,
                         partial_floats, k_new, v_new, new_stride, table, rot, slots, k_cache_w, v_cache_w, stream);
}

// ----------------------------------------------------------------------------------------------
// the same without any memory from the caller beyond inputs and outputs (ka_no_alloc.h)
// ----------------------------------------------------------------------------------------------
// The partial results of the parts of a row's keys go through this array instead of a buffer the
// caller allocated. Each GPU the library runs on holds its own copy until the process ends. In
// host code the name stands for the symbol only; the address on a device is asked for once per
// device (`static_scratch`) and only that pointer is ever handed to a kernel.
static __device__ __align__(256) float scratch[KA_NO_ALLOC_SCRATCH_FLOATS];

constexpr int KA_NO_ALLOC_MAX_DEVICES = 64;
static float* g_scratch_ptr[KA_NO_ALLOC_MAX_DEVICES];
static std::mutex g_scratch_lock;

// The array's address on the current device, looked up at the first call on that device.
static int static_scratch(float** ptr) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    KA_CHECK(e == hipSuccess, "ka_attention_decode_bf16_no_alloc: no current device: %s", hipGetErrorString(e));
    KA_CHECK(device >= 0 && device < KA_NO_ALLOC_MAX_DEVICES, "ka_attention_decode_bf16_no_alloc: device %d beyond the %d this library keeps a scratch address for",
             device, KA_NO_ALLOC_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[device]) {
        float* found = nullptr;
        e = hipGetSymbolAddress((void**)&found, HIP_SYMBOL(scratch));
        KA_CHECK(e == hipSuccess && found, "ka_attention_decode_bf16_no_alloc: cannot find the scratch array on device %d: %s", device,
                 hipGetErrorString(e));
        g_scratch_ptr[device] = found;
    }
    *ptr = g_scratch_ptr[device];
    return 0;
}

KA_API int ka_attention_decode_bf16_no_alloc(const void* q, long q_row_stride, const void* k_cache, const void* v_cache,
                                             const int* block_table, int max_pages, const int* token_row,
                                             const int* kv_lo, const int* kv_hi, void* out, long out_row_stride,
                                             float scale, int n, int H, int Hkv, int hd, int page_size, int splits,
                                             int waves, const void* k_new, const void* v_new, long new_stride,
                                             const float* table, int rot, const int* slots, void* k_cache_w,
                                             void* v_cache_w, hipStream_t stream) {
    const char* who = "ka_attention_decode_bf16_no_alloc";
    KA_CHECK(n > 0 && H > 0 && hd > 0 && splits >= 1, "%s: bad sizes n=%d H=%d hd=%d splits=%d", who, n, H, hd, splits);
    const long needed = splits > 1 ? ka_attention_decode_partial_floats(n, H, hd, splits) : 0;
    KA_CHECK(needed <= KA_NO_ALLOC_SCRATCH_FLOATS,
             "%s: %d tokens x %d heads x %d parts of the keys need %ld floats of scratch, the static array holds %ld "
             "(fewer tokens a call, or ka_attention_decode_bf16 with a buffer of the caller's)",
             who, n, H, splits, needed, (long)KA_NO_ALLOC_SCRATCH_FLOATS);
    float* ptr = nullptr;
    if (static_scratch(&ptr)) return -1;
    // nothing in the array has to start at zero: every record that the merge reads was written by
    // the kernel before it in this call (there are no counters or flags in it)
    return decode_launch(who, q, q_row_stride, k_cache, v_cache, block_table, max_pages, token_row, kv_lo, kv_hi, out,
                         out_row_stride, scale, n, H, Hkv, hd, page_size, splits, waves, ptr, KA_NO_ALLOC_SCRATCH_FLOATS,
                         k_new, v_new, new_stride, table, rot, slots, k_cache_w, v_cache_w, stream);
}
