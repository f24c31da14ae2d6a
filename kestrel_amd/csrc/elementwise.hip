// Embedding gather, LayerNorm and rotary + paged cache write.
//
// The residual stream is fp32 in every precision mode; these kernels read and write
// it as fp32 and convert only at the boundary to the model's storage type.
#include "ka_common.h"

KA_API int ka_version() { return 1; }

// ----------------------------------------------------------------------------
// Embedding: out[t, :] = table[ids[t], :] as fp32. A row with ids[t] == -1 is left as it
// is (its embedding was given by the caller). ids[t] <= -2 names the entry -2 - ids[t] of
// `pending`, a device table of token ids that an earlier step's sampling filled: the id of
// a decoded token can so reach the next step without passing through the host.
// ----------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             const int* __restrict__ pending, int n_pending, int vocab,
                             float* __restrict__ out, int dim, float scale) {
    int t = blockIdx.x;
    int id = ids[t];
    if (id == -1) return;
    if (id < 0) {
        int at = -2 - id;
        if (!pending || at >= n_pending) return;
        id = pending[at];
        if ((unsigned)id >= (unsigned)vocab) id = 0;   // never an address outside the table
    }
    const T* src = table + (size_t)id * dim;
    float* dst = out + (size_t)t * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) dst[d] = ka_to_float(src[d]) * scale;
}

// `scale`: a factor on the looked-up rows (1 for none; rows with id -1, which are given from
// outside, are not touched).
KA_API int ka_embed(const void* table, int table_dtype, const int* ids, const int* pending, int n_pending,
                    int vocab, float* out, int n, int dim, float scale, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && vocab > 0 && n_pending >= 0, "ka_embed: bad sizes n=%d dim=%d vocab=%d", n, dim, vocab);
    if (n == 0) return 0;
    dim3 grid(n), block(256);
    if (table_dtype == KA_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, (const float*)table, ids, pending, n_pending,
                           vocab, out, dim, scale);
    else if (table_dtype == KA_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, ids, pending,
                           n_pending, vocab, out, dim, scale);
    else
        KA_CHECK(false, "ka_embed: unsupported table dtype %d", table_dtype);
    KA_LAUNCH_CHECK();
    return 0;
}

// logits *= scale; then, with cap > 0, logits = cap * tanh(logits / cap): what some architectures do
// to their logits before sampling.
__global__ void adjust_logits_kernel(float* __restrict__ logits, long count, float scale, float cap) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float x = logits[i] * scale;
    if (cap > 0.f) x = cap * tanhf(x / cap);
    logits[i] = x;
}

KA_API int ka_adjust_logits(float* logits, long count, float scale, float cap, hipStream_t stream) {
    KA_CHECK(count >= 0 && cap >= 0.f, "ka_adjust_logits: bad count %ld or cap %g", count, cap);
    if (count == 0) return 0;
    KA_CHECK((count + 255) / 256 < (1L << 31), "ka_adjust_logits: too many values");
    hipLaunchKernelGGL(adjust_logits_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, logits, count, scale, cap);
    KA_LAUNCH_CHECK();
    return 0;
}

// out[rows[i], :] = src[i, :] (given embeddings spliced into the stream); a negative row: nothing
// (the unused end of a list of fixed length).
template <typename T>
__global__ void scatter_rows_kernel(const T* __restrict__ src, const int* __restrict__ rows,
                                    float* __restrict__ out, int dim) {
    int i = blockIdx.x;
    if (rows[i] < 0) return;
    const T* s = src + (size_t)i * dim;
    float* dst = out + (size_t)rows[i] * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) dst[d] = ka_to_float(s[d]);
}

KA_API int ka_scatter_rows(const void* src, int src_dtype, const int* rows, float* out, int m,
                           int dim, hipStream_t stream) {
    KA_CHECK(m >= 0 && dim > 0, "ka_scatter_rows: bad sizes m=%d dim=%d", m, dim);
    if (m == 0) return 0;
    dim3 grid(m), block(256);
    if (src_dtype == KA_F32)
        hipLaunchKernelGGL(scatter_rows_kernel<float>, grid, block, 0, stream, (const float*)src, rows, out, dim);
    else if (src_dtype == KA_BF16)
        hipLaunchKernelGGL(scatter_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)src, rows, out, dim);
    else
        KA_CHECK(false, "ka_scatter_rows: unsupported dtype %d", src_dtype);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// LayerNorm over the last axis, statistics in fp32, two passes (mean, then the
// variance of the centred values). `rows` (optional) selects input rows, which
// fuses the gather of the wanted positions into the final norm.
// ----------------------------------------------------------------------------
constexpr int LN_THREADS = 256;

__device__ __forceinline__ float block_sum_256(float v, float* smem) {
    v = ka_wave_sum(v);
    int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < LN_THREADS / KA_WAVE; ++w) total += smem[w];
    return total;
}

template <typename TOut>
__global__ void __launch_bounds__(LN_THREADS)
layernorm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                 const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
                 TOut* __restrict__ out, int dim) {
    __shared__ float smem[LN_THREADS / KA_WAVE];
    int i = blockIdx.x;
    const float* src = x + (size_t)(rows ? rows[i] : i) * dim;
    TOut* dst = out + (size_t)i * dim;
    float s = 0.f;
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) s += src[d];
    float mean = block_sum_256(s, smem) / (float)dim;
    float v = 0.f;
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) {
        float c = src[d] - mean;
        v += c * c;
    }
    float var = block_sum_256(v, smem) / (float)dim;
    float rstd = 1.0f / sqrtf(var + eps);
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) {
        float y = (src[d] - mean) * rstd * gamma[d];
        if (beta) y += beta[d];
        dst[d] = ka_from_float<TOut>(y);
    }
}

// Rows of up to 256 * 4 * ITEMS values: every thread keeps its share of the row in registers, so
// the row is read once.
template <typename TOut, int ITEMS>
__global__ void __launch_bounds__(LN_THREADS)
layernorm_regs_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                      const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
                      TOut* __restrict__ out, int dim) {
    typedef __attribute__((ext_vector_type(4))) float floatx4;
    __shared__ float smem[LN_THREADS / KA_WAVE];
    int i = blockIdx.x;
    const float* src = x + (size_t)(rows ? rows[i] : i) * dim;
    TOut* dst = out + (size_t)i * dim;
    // (every load unconditional, from a place moved inside the row; a load under a branch would
    // make the compiler wait for each before the next is asked for)
    floatx4 v[ITEMS], g[ITEMS], b[ITEMS];
    float s = 0.f;
    const bool beta_vec = beta && (reinterpret_cast<uintptr_t>(beta) % 16 == 0);
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = min((j * LN_THREADS + (int)threadIdx.x) * 4, dim - 4);
        v[j] = *reinterpret_cast<const floatx4*>(src + d);
        g[j] = *reinterpret_cast<const floatx4*>(gamma + d);
        b[j] = beta_vec ? *reinterpret_cast<const floatx4*>(beta + d) : floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d >= dim) v[j] = floatx4{0.f, 0.f, 0.f, 0.f};
        if (beta && !beta_vec && d < dim) b[j] = floatx4{beta[d], beta[d + 1], beta[d + 2], beta[d + 3]};
        s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
    }
    float mean = block_sum_256(s, smem) / (float)dim;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d < dim) {
#pragma unroll
            for (int e = 0; e < 4; ++e) q += (v[j][e] - mean) * (v[j][e] - mean);
        }
    }
    float rstd = 1.0f / sqrtf(block_sum_256(q, smem) / (float)dim + eps);
    const bool out_vec = reinterpret_cast<uintptr_t>(dst) % (4 * sizeof(TOut)) == 0;      // (dim is a multiple of 4)
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d < dim) {
            TOut y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = ka_from_float<TOut>((v[j][e] - mean) * rstd * g[j][e] + b[j][e]);
            if (out_vec) {
                typedef TOut __attribute__((ext_vector_type(4))) out4;
                *reinterpret_cast<out4*>(dst + d) = out4{y[0], y[1], y[2], y[3]};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[d + e] = y[e];
            }
        }
    }
}

KA_API int ka_layernorm(const float* x, const int* rows, const float* gamma, const float* beta,
                        float eps, void* out, int out_dtype, int n, int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0, "ka_layernorm: bad sizes n=%d dim=%d", n, dim);
    KA_CHECK(eps >= 0.f, "ka_layernorm: negative eps");
    if (n == 0) return 0;
    dim3 grid(n), block(LN_THREADS);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_layernorm: unsupported out dtype %d", out_dtype);
    const bool aligned = dim % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)gamma % 16 == 0;
    if (aligned && dim <= LN_THREADS * 4 * 4) {
        // (as many loads per thread as the row needs: 1, 2 or 4 of 16 bytes)
#define KA_LN_REGS(ITEMS)                                                                                                     \
    if (out_dtype == KA_F32)                                                                                                  \
        hipLaunchKernelGGL((layernorm_regs_kernel<float, ITEMS>), grid, block, 0, stream, x, rows, gamma, beta, eps, (float*)out, dim); \
    else                                                                                                                      \
        hipLaunchKernelGGL((layernorm_regs_kernel<bf16_t, ITEMS>), grid, block, 0, stream, x, rows, gamma, beta, eps, (bf16_t*)out, dim)
        if (dim <= LN_THREADS * 4) { KA_LN_REGS(1); }
        else if (dim <= LN_THREADS * 4 * 2) { KA_LN_REGS(2); }
        else { KA_LN_REGS(4); }
#undef KA_LN_REGS
    } else if (out_dtype == KA_F32) {
        hipLaunchKernelGGL(layernorm_kernel<float>, grid, block, 0, stream, x, rows, gamma, beta, eps, (float*)out, dim);
    } else {
        hipLaunchKernelGGL(layernorm_kernel<bf16_t>, grid, block, 0, stream, x, rows, gamma, beta, eps, (bf16_t*)out, dim);
    }
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Rotary position encoding of the first `rot` channels of each head, applied in place to
// the q heads of a fused qkv row, and to the k heads on their way into the paged cache
// together with v. The table row of position p is [cos(p f_0..f_{rot/2-1}), sin(...)] in
// fp32; the rotation is computed in fp32. `interleaved` says which channels form the pair
// that angle i turns: 0 = channel i with channel i + rot/2 (halves), 1 = channel 2i with
// channel 2i + 1.
//
// qkv row: [H*hd q | Hkv*hd k | Hkv*hd v]. Key cache: [pages, Hkv, page_size, hd]; value cache:
// [pages, Hkv, hd, page_size] (transposed inside the page, so that the MFMA attention kernels
// read eight consecutive keys of one channel with a single 16-byte load).
// slots[t] = page * page_size + offset, or < 0 for "do not write" (a layer that
// reads another layer's cache).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void rope_cache_kernel(T* __restrict__ qkv, long row_stride,
                                  const int* __restrict__ positions, const int* __restrict__ slots,
                                  const float* __restrict__ table, T* __restrict__ k_cache,
                                  T* __restrict__ v_cache, int H, int Hkv, int hd, int rot,
                                  int page_size, int rotate, int interleaved) {
    int t = blockIdx.x;
    T* row = qkv + (size_t)t * row_stride;
    int pos = positions[t];
    const float* cs = table + (size_t)pos * rot;
    int half = rot / 2;
    // q heads: rotate in place. One thread per (head, pair).
    if (rotate) {
        for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
            int h = idx / half, i = idx % half;
            T* p = row + h * hd;
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            float a = ka_to_float(p[ia]), b = ka_to_float(p[ib]);
            float c = cs[i], s = cs[half + i];
            p[ia] = ka_from_float<T>(a * c - b * s);
            p[ib] = ka_from_float<T>(b * c + a * s);
        }
    }
    long slot = slots ? slots[t] : -1;
    if (slot < 0) return;
    long page = slot / page_size, off = slot % page_size;
    const T* krow = row + (size_t)H * hd;
    const T* vrow = krow + (size_t)Hkv * hd;
    for (int idx = threadIdx.x; idx < Hkv * hd; idx += blockDim.x) {
        int h = idx / hd, d = idx % hd;
        size_t dst = (((size_t)page * Hkv + h) * page_size + off) * hd + d;
        float kv = ka_to_float(krow[idx]);
        if (rotate && d < rot) {
            const int i = interleaved ? d / 2 : (d < half ? d : d - half);
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            float a = ka_to_float(krow[h * hd + ia]), b = ka_to_float(krow[h * hd + ib]);
            float c = cs[i], s = cs[half + i];
            kv = d == ia ? a * c - b * s : b * c + a * s;
        }
        k_cache[dst] = ka_from_float<T>(kv);
        size_t vdst = (((size_t)page * Hkv + h) * hd + d) * page_size + off;
        v_cache[vdst] = vrow[idx];
    }
}

KA_API int ka_rope_cache(void* qkv, int dtype, long row_stride, const int* positions,
                         const int* slots, const float* table, int table_rows, void* k_cache,
                         void* v_cache, int n, int H, int Hkv, int hd, int rot, int page_size,
                         int interleaved, hipStream_t stream) {
    KA_CHECK(n >= 0 && H > 0 && Hkv > 0 && hd > 0, "ka_rope_cache: bad sizes");
    KA_CHECK(interleaved == 0 || interleaved == 1, "ka_rope_cache: pairing must be 0 (halves) or 1 (interleaved)");
    KA_CHECK(rot >= 0 && rot <= hd && rot % 2 == 0, "ka_rope_cache: rotary dim %d must be even and <= head dim %d", rot, hd);
    KA_CHECK(row_stride >= (long)(H + 2 * Hkv) * hd, "ka_rope_cache: row stride %ld too small", row_stride);
    KA_CHECK(page_size > 0, "ka_rope_cache: page size %d", page_size);
    KA_CHECK(rot == 0 || (table != nullptr && table_rows > 0), "ka_rope_cache: rotary table missing");
    if (n == 0) return 0;
    dim3 grid(n), block(256);
    int rotate = rot > 0;
    if (dtype == KA_F32)
        hipLaunchKernelGGL(rope_cache_kernel<float>, grid, block, 0, stream, (float*)qkv, row_stride, positions, slots,
                           table, (float*)k_cache, (float*)v_cache, H, Hkv, hd, rot, page_size, rotate, interleaved);
    else if (dtype == KA_BF16)
        hipLaunchKernelGGL(rope_cache_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)qkv, row_stride, positions, slots,
                           table, (bf16_t*)k_cache, (bf16_t*)v_cache, H, Hkv, hd, rot, page_size, rotate, interleaved);
    else
        KA_CHECK(false, "ka_rope_cache: unsupported dtype %d", dtype);
    KA_LAUNCH_CHECK();
    return 0;
}
