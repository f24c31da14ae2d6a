// Decode attention and a linear layer in one launch, side by side on the compute units.
//
// A decode step of a block whose mixer and feed-forward read the same normalised input has two
// pieces of work that do not depend on each other: attention over the cache (a chain of trips to
// memory at a few rows, a stream of keys and values at many) and the feed-forward's first linear
// (a stream of weights with a prologue and an epilogue). As two launches each pays its own start
// and end with the chip half idle; as one, the workgroups of both kinds share every compute unit
// (one of each at a time: 8 waves and at most 128 registers a lane each), and the stream of one
// fills the gaps in the other. Nothing passes between the two kinds: a workgroup is of one kind
// from start to end, chosen by its index (the kinds alternate while both last).
//
// The linear part is the persistent skinny kernel (ka_skinny.h) on bf16 rows that an earlier launch
// has left (the block's normalised input): at most 8 rows, K up to 2048. Normalising the rows here,
// in every workgroup's prologue, was measured and dropped: within half a CU's registers that
// prologue makes the linear part the longer of the two (13.8 against 11.3 us alone at one row).
// The attention part is the decode kernel (ka_attention_decode.h) with 8 waves a workgroup, head
// sizes up to 64 (larger heads need more registers than half a SIMD's).
#include "ka_attention_decode.h"
#include "ka_skinny.h"

constexpr int BS_WAVES = SP_WAVES;       // waves of a workgroup, of either kind
constexpr int BS_ROWS = 8;               // most rows (tokens) of a launch
constexpr int BS_MAX_PER = 4;            // k-blocks per wave that the linear part keeps activations for: K <= 2048
constexpr int BS_DEPTH = 3;              // strips of weights in flight per linear workgroup, the one at work included

struct BesideAttention {
    const bf16_t* q;
    long q_row_stride;
    const bf16_t* k_cache;
    const bf16_t* v_cache;
    const int* block_table;
    int max_pages;
    const int* token_row;
    const int* kv_lo;
    const int* kv_hi;
    bf16_t* out;
    long out_row_stride;
    float scale;
    int n, H, Hkv, splits;
    float* partial;
    DecodeFuse fz;
};

template <int HD, int PER>
__global__ void __launch_bounds__(BS_WAVES * KA_WAVE) __attribute__((amdgpu_waves_per_eu(4, 4)))
attn_decode_beside_kernel(BesideAttention a, SkinnyArgs p, int strips, int attention_groups, int linear_groups) {
    const int b = blockIdx.x;
    const int pairs = min(attention_groups, linear_groups);
    const bool linear = b < 2 * pairs ? (b & 1) != 0 : linear_groups > attention_groups;
    const int index = b < 2 * pairs ? b >> 1 : b - pairs;
    if (linear) {
        skinny_persistent_body<PER, 1, true, false, BS_DEPTH, false>(p, strips, index, linear_groups);
        return;
    }
    const int t = index % a.n, h = index / a.n % a.H, split = index / (a.n * a.H);
    attn_decode_body<HD, BS_WAVES, true>(a.q, a.q_row_stride, a.k_cache, a.v_cache, a.block_table, a.max_pages, a.token_row,
                                   a.kv_lo, a.kv_hi, a.out, a.out_row_stride, a.scale, a.H, a.Hkv, a.partial, a.fz, t, h,
                                   split, a.splits);
}

// Whether a launch of n tokens x H heads x `splits` parts of the keys at head size hd, with a linear
// layer of K inputs, is taken. Attention may fill at most a quarter of the chip's places (two
// workgroups per compute unit): measured on Moondream 2's sizes at 1024 keys, the launch then
// saves 3 to 5 % of a decode step (batch 1 to 4); with more attention workgroups it loses what it
// saves (batch 8) or more (batch 5 to 7: 3 to 12 %), the two kinds standing in each other's way.
KA_API int ka_attention_decode_beside_supported(int n, int H, int splits, int hd, int page_size, int K) {
    return n > 0 && n <= BS_ROWS && H > 0 && splits > 0 && (long)n * H * splits <= ka_compute_units() / 2 && hd <= 64 &&
           ka_attention_decode_supported(hd, page_size) && K > 0 && K % 8 == 0 &&
           ka_cdiv(ka_cdiv(K, SK_KBLOCK), SP_WAVES) <= BS_MAX_PER;
}

// Attention as ka_attention_decode_bf16 computes it (same operands, 8 waves a workgroup), and beside it
// lin_out = act(A @ W^T + bias) for the same n rows: A bf16 [n, K], rows lda apart.
KA_API int ka_attention_decode_beside_bf16(const void* q, long q_row_stride, const void* k_cache, const void* v_cache,
                                           const int* block_table, int max_pages, const int* token_row,
                                           const int* kv_lo, const int* kv_hi, void* out, long out_row_stride,
                                           float scale, int n, int H, int Hkv, int hd, int page_size, int splits,
                                           float* partial, long partial_floats, const void* k_new, const void* v_new,
                                           long new_stride, const float* table, int rot, const int* slots,
                                           void* k_cache_w, void* v_cache_w, const void* A, long lda, int K,
                                           const void* W, long ldw, const float* bias, void* lin_out, int lin_out_dtype,
                                           long ldo, int N, int act, hipStream_t stream) {
    const char* who = "ka_attention_decode_beside_bf16";
    BesideAttention a = {};
    if (decode_check(who, q, q_row_stride, out, out_row_stride, n, H, Hkv, hd, page_size, max_pages, splits, partial,
                     partial_floats, k_new, v_new, new_stride, table, rot, slots, k_cache_w, v_cache_w, &a.fz))
        return -1;
    KA_CHECK(ka_attention_decode_beside_supported(n, H, splits, hd, page_size, K),
             "%s: %d rows x %d heads x %d parts, head size %d, K=%d not covered (at most %d rows and %d workgroups of "
             "attention, head sizes up to 64, K up to %d)", who, n, H, splits, hd, K, BS_ROWS, ka_compute_units() / 2,
             BS_MAX_PER * SP_WAVES * SK_KBLOCK);
    a.q = (const bf16_t*)q; a.q_row_stride = q_row_stride;
    a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache;
    a.block_table = block_table; a.max_pages = max_pages; a.token_row = token_row; a.kv_lo = kv_lo; a.kv_hi = kv_hi;
    a.out = (bf16_t*)out; a.out_row_stride = out_row_stride; a.scale = scale;
    a.n = n; a.H = H; a.Hkv = Hkv; a.splits = splits; a.partial = partial;

    SkinnyArgs p = {};
    p.M = n;
    p.K[0] = K;
    p.a = SkinnyTarget{(const bf16_t*)W, ldw, bias, lin_out, ldo, lin_out_dtype, N, act, 0};
    if (check_target(who, p.a, K)) return -1;
    KA_CHECK(persistent_bias_ok(p.a), "%s: the bias must be 16-byte aligned and N a multiple of 4", who);
    KA_CHECK(A && lda % 8 == 0 && lda >= K && (uintptr_t)A % 16 == 0, "%s: the linear layer's input rows must be 16-byte aligned and >= K", who);
    p.A[0] = (const bf16_t*)A; p.lda[0] = lda;
    const int strips = ka_cdiv(N, SK_STRIP);
    p.strips_a = strips;
    const size_t dyn = 0;

    // linear workgroups: the chip holds two workgroups of this launch per compute unit; as many as
    // fill the places that attention leaves, and no more: a workgroup that has to wait for a place
    // starts when the first ones end, and the launch takes twice as long. Strips go round the
    // workgroups, so some walk over one strip more than others.
    const long attention_groups = (long)n * H * splits;
    const int cus = ka_compute_units();
    int linear_groups = (int)(2 * cus - attention_groups);
    if (linear_groups > strips) linear_groups = strips;
    KA_CHECK(attention_groups + linear_groups < (1L << 31), "%s: too many workgroups", who);
    const int per = ka_cdiv(ka_cdiv(K, SK_KBLOCK), SP_WAVES);
    dim3 grid((unsigned)(attention_groups + linear_groups)), block(BS_WAVES * KA_WAVE);
#define KA_BS_LAUNCH(HDV, PERV)                                                                                     \
    {                                                                                                               \
        static size_t reserved = 0;                                                                                 \
        if (dyn > reserved) {                                                                                       \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_decode_beside_kernel<HDV, PERV>), \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);               \
            KA_CHECK(e == hipSuccess, "%s: cannot reserve %zu bytes of LDS", who, dyn);                             \
            reserved = dyn;                                                                                         \
        }                                                                                                           \
        hipLaunchKernelGGL((attn_decode_beside_kernel<HDV, PERV>), grid, block, dyn, stream, a, p, strips,          \
                           (int)attention_groups, linear_groups);                                                   \
    }
#define KA_BS(HDV)                                                                                                  \
    case HDV:                                                                                                       \
        if (per <= 1) KA_BS_LAUNCH(HDV, 1) else if (per <= 2) KA_BS_LAUNCH(HDV, 2) else KA_BS_LAUNCH(HDV, 4)        \
        break;
    switch (hd) {
        KA_BS(16) KA_BS(32) KA_BS(48) KA_BS(64)
    }
#undef KA_BS
#undef KA_BS_LAUNCH
    KA_LAUNCH_CHECK();
    if (splits > 1) {
#define KA_BSM(HDV)                                                                                                 \
    case HDV:                                                                                                       \
        hipLaunchKernelGGL(attn_decode_merge_kernel<HDV>, dim3(n, H), dim3(KA_WAVE), 0, stream, partial, splits,    \
                           (bf16_t*)out, out_row_stride, H);                                                        \
        break
        switch (hd) {
            KA_BSM(16); KA_BSM(32); KA_BSM(48); KA_BSM(64);
        }
#undef KA_BSM
        KA_LAUNCH_CHECK();
    }
    return 0;
}
