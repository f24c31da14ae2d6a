// Generic paged attention: one wavefront per (token, query head), any head size up
// to 512, any page size, fp32 or bf16 storage, all arithmetic in fp32.
//
// Every token t of the packed batch belongs to request row token_row[t] and sees
// the cached keys at positions [kv_lo[t], kv_hi[t]) of that row (kv_lo optional,
// default 0). A causal token at position p has kv_hi = p + 1; a token inside a
// bidirectional block has kv_hi = end of its block; a window of w has
// kv_lo = max(0, p + 1 - w). The keys of this step are already in the cache.
// Key position k of row r lies at page block_table[r, k / page_size], offset
// k % page_size; key cache [pages, Hkv, page_size, hd], value cache [pages, Hkv, hd, page_size].
#include "ka_common.h"

constexpr int ATT_MAX_HD = 512;

// Four neighbouring elements with one load (the address must be a multiple of 4 elements).
template <typename T>
__device__ __forceinline__ void att_load4(const T* p, float v[4]) {
    typedef __attribute__((ext_vector_type(4))) T vec4;
    const vec4 x = *reinterpret_cast<const vec4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ka_to_float(x[i]);
}

template <typename T>
__global__ void __launch_bounds__(KA_WAVE)
attention_generic_kernel(const T* __restrict__ q, long q_row_stride, const T* __restrict__ k_cache,
                         const T* __restrict__ v_cache, const int* __restrict__ block_table,
                         int max_pages, const int* __restrict__ token_row,
                         const int* __restrict__ kv_lo, const int* __restrict__ kv_hi,
                         T* __restrict__ out, long out_row_stride, float scale, int H, int Hkv,
                         int hd, int page_size) {
    __shared__ float qs[ATT_MAX_HD];
    __shared__ float ps[KA_WAVE];
    __shared__ long offs[KA_WAVE];   // value cache offset of channel 0 of each key of the chunk
    int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    int kvh = h / (H / Hkv);
    int row = token_row[t];
    int lo = kv_lo ? kv_lo[t] : 0, hi = kv_hi[t];
    const T* qp = q + (size_t)t * q_row_stride + (size_t)h * hd;
    for (int d = lane; d < hd; d += KA_WAVE) qs[d] = ka_to_float(qp[d]) * scale;
    __syncthreads();
    const int* bt = block_table + (size_t)row * max_pages;
    const bool k_vectors = hd % 4 == 0 && reinterpret_cast<uintptr_t>(k_cache) % (4 * sizeof(T)) == 0;
    const bool v_vectors = page_size % 4 == 0 && reinterpret_cast<uintptr_t>(v_cache) % (4 * sizeof(T)) == 0;
    float m = -INFINITY, l = 0.f;
    float o[ATT_MAX_HD / KA_WAVE];
#pragma unroll
    for (int i = 0; i < ATT_MAX_HD / KA_WAVE; ++i) o[i] = 0.f;
    for (int base = lo; base < hi; base += KA_WAVE) {
        int key = base + lane;
        bool valid = key < hi;
        float s = -INFINITY;
        long off = 0;
        if (valid) {
            int page = bt[key / page_size];
            const T* kp = k_cache + (((long)page * Hkv + kvh) * page_size + key % page_size) * hd;
            off = ((long)page * Hkv + kvh) * hd * page_size + key % page_size;
            float acc = 0.f;
            if (k_vectors) {
                // four channels with one load, added in the same order as one by one
                for (int d = 0; d < hd; d += 4) {
                    float k4[4];
                    att_load4(kp + d, k4);
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc = fmaf(qs[d + u], k4[u], acc);
                }
            } else {
                for (int d = 0; d < hd; ++d) acc = fmaf(qs[d], ka_to_float(kp[d]), acc);
            }
            s = acc;
        }
        float m_new = fmaxf(m, ka_wave_max(s));
        float corr = expf(m - m_new);  // m = -inf at the first chunk gives 0
        float p = valid ? expf(s - m_new) : 0.f;
        l = l * corr + ka_wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        offs[lane] = off;
        __syncthreads();
        int count = min(KA_WAVE, hi - base);
#pragma unroll
        for (int i = 0; i < ATT_MAX_HD / KA_WAVE; ++i) {
            int d = lane + i * KA_WAVE;
            if (d < hd) {
                float acc = o[i] * corr;
                const T* vd = v_cache + (long)d * page_size;
                int j = 0;
                // A chunk that starts on a multiple of four keys: every four keys from there lie in
                // one page, their values side by side in the cache: one load, added in the same
                // order as one by one.
                if (v_vectors && (base & 3) == 0) {
                    for (; j + 3 < count; j += 4) {
                        float v4[4];
                        att_load4(vd + offs[j], v4);
#pragma unroll
                        for (int u = 0; u < 4; ++u) acc = fmaf(ps[j + u], v4[u], acc);
                    }
                }
                for (; j < count; ++j) acc = fmaf(ps[j], ka_to_float(vd[offs[j]]), acc);
                o[i] = acc;
            }
        }
    }
    float inv = l > 0.f ? 1.0f / l : 0.f;
    T* op = out + (size_t)t * out_row_stride + (size_t)h * hd;
#pragma unroll
    for (int i = 0; i < ATT_MAX_HD / KA_WAVE; ++i) {
        int d = lane + i * KA_WAVE;
        if (d < hd) op[d] = ka_from_float<T>(o[i] * inv);
    }
}

KA_API int ka_attention_generic(const void* q, int dtype, long q_row_stride, const void* k_cache,
                                const void* v_cache, const int* block_table, int max_pages,
                                const int* token_row, const int* kv_lo, const int* kv_hi, void* out,
                                long out_row_stride, float scale, int n, int H, int Hkv, int hd,
                                int page_size, hipStream_t stream) {
    KA_CHECK(n >= 0 && H > 0 && Hkv > 0 && hd > 0, "ka_attention_generic: bad sizes");
    KA_CHECK(H % Hkv == 0, "ka_attention_generic: %d query heads do not divide into %d kv heads", H, Hkv);
    KA_CHECK(hd <= ATT_MAX_HD, "ka_attention_generic: head size %d above %d", hd, ATT_MAX_HD);
    KA_CHECK(H <= 65535, "ka_attention_generic: too many heads %d", H);
    KA_CHECK(page_size > 0 && max_pages > 0, "ka_attention_generic: bad paging %d %d", page_size, max_pages);
    if (n == 0) return 0;
    dim3 grid(n, H), block(KA_WAVE);
    if (dtype == KA_F32)
        hipLaunchKernelGGL(attention_generic_kernel<float>, grid, block, 0, stream, (const float*)q, q_row_stride,
                           (const float*)k_cache, (const float*)v_cache, block_table, max_pages, token_row, kv_lo,
                           kv_hi, (float*)out, out_row_stride, scale, H, Hkv, hd, page_size);
    else if (dtype == KA_BF16)
        hipLaunchKernelGGL(attention_generic_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q, q_row_stride,
                           (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, token_row, kv_lo,
                           kv_hi, (bf16_t*)out, out_row_stride, scale, H, Hkv, hd, page_size);
    else
        KA_CHECK(false, "ka_attention_generic: unsupported dtype %d", dtype);
    KA_LAUNCH_CHECK();
    return 0;
}
