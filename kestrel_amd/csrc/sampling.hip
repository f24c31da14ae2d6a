// Token selection from fp32 logits: argmax, and temperature + top-p sampling.
//
// One workgroup of 1024 threads per row. A row with temperature <= 1e-6 is greedy
// (the first index of the maximum). Otherwise the distribution is
// softmax(logits / T) restricted to the smallest set of most probable tokens whose
// mass reaches top_p, found by bisection on the probability threshold; the token is
// drawn by inversion with a uniform number from a counter-based generator keyed by
// (rng_key[row], rng_counter[row]), so a request's draws do not depend on what else
// is in the batch. Logits of value -inf are never chosen.
#include "ka_common.h"

constexpr int SM_THREADS = 1024;
constexpr int SM_WAVES = SM_THREADS / KA_WAVE;
constexpr float SM_GREEDY_EPS = 1e-6f;
constexpr int SM_PICKED = 4 * SM_THREADS;       // probabilities that the search for the nucleus gathers once so few are left

__device__ __forceinline__ float block_reduce_sum(float v, float* smem) {
    v = ka_wave_sum(v);
    __syncthreads();
    if (threadIdx.x % KA_WAVE == 0) smem[threadIdx.x / KA_WAVE] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < SM_WAVES; ++w) t += smem[w];
    return t;
}

__device__ __forceinline__ float block_reduce_max(float v, float* smem) {
    v = ka_wave_max(v);
    __syncthreads();
    if (threadIdx.x % KA_WAVE == 0) smem[threadIdx.x / KA_WAVE] = v;
    __syncthreads();
    float t = -INFINITY;
#pragma unroll
    for (int w = 0; w < SM_WAVES; ++w) t = fmaxf(t, smem[w]);
    return t;
}

// The greatest value of the wave and the lowest index that has it, in every lane.
template <int STEP = 1>
__device__ __forceinline__ void wave_argmax(float& best, int& best_i) {
    if constexpr (STEP < KA_WAVE) {
        float va, vb;
        int ia, ib;
        ka_lanes_pair<STEP>(best, va, vb);
        ka_lanes_pair<STEP>(best_i, ia, ib);
        const bool second = vb > va || (vb == va && ib < ia);
        best = second ? vb : va;
        best_i = second ? ib : ia;
        wave_argmax<STEP * 2>(best, best_i);
    }
}

// splitmix64 of (key + counter * odd constant): uniform in [0, 1) with 24 bits.
__host__ __device__ inline float ka_uniform(unsigned long long key, unsigned long long counter) {
    unsigned long long z = key + 0x9E3779B97F4A7C15ull * (counter + 1ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// The chosen token goes to out[r] and, if the caller keeps a device table of the requests'
// latest tokens, to pending[pending_at[r]] (a negative place is passed over).
struct PendingTable {
    int* tokens;          // nullptr: none kept
    const int* at;        // per row of logits: the place in `tokens`
    int n;                // places in `tokens`
};

__device__ __forceinline__ void ka_store_token(int* out, const PendingTable& pending, int r, int token) {
    out[r] = token;
    if (pending.tokens) {
        int at = pending.at[r];
        if (at >= 0 && at < pending.n) pending.tokens[at] = token;
    }
}

// Index of the maximum (lowest index on ties) of one row, by all threads.
__device__ int block_argmax(const float* __restrict__ row, int V, float* smem_f, int* smem_i) {
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    // eight loads in flight per thread: a row is read in a few trips to memory, not in V / threads
    constexpr int UN = 8;
    for (int base = threadIdx.x; base < V; base += SM_THREADS * UN) {
        float v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            int i = base + u * SM_THREADS;
            v[u] = i < V ? row[i] : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            int i = base + u * SM_THREADS;
            if (i < V && (v[u] > best || (v[u] == best && i < best_i))) { best = v[u]; best_i = i; }
        }
    }
    wave_argmax(best, best_i);
    __syncthreads();
    if (threadIdx.x % KA_WAVE == 0) { smem_f[threadIdx.x / KA_WAVE] = best; smem_i[threadIdx.x / KA_WAVE] = best_i; }
    __syncthreads();
    best = smem_f[0]; best_i = smem_i[0];
    for (int w = 1; w < SM_WAVES; ++w) {
        float ov = smem_f[w]; int oi = smem_i[w];
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    if (best_i == 0x7fffffff) best_i = 0;
    return best_i;
}

// The same for rows of at most R * 1024 logits, all of a thread's loads in flight at once (a row
// is then one trip to memory; block_argmax asks for eight values a thread and round).
template <int R>
__global__ void __launch_bounds__(SM_THREADS)
argmax_regs_kernel(const float* __restrict__ logits, long ld, int* __restrict__ out, int V,
                   PendingTable pending) {
    __shared__ float sf[SM_WAVES];
    __shared__ int si[SM_WAVES];
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * ld;
    float x[R];
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = row[min(j * SM_THREADS + tid, V - 1)];
    float best = -INFINITY;
    int best_i = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int i = j * SM_THREADS + tid;
        if (i < V && x[j] > best) { best = x[j]; best_i = i; }      // j rises with i: the first of equals stays
    }
    wave_argmax(best, best_i);
    if (tid % KA_WAVE == 0) { sf[tid / KA_WAVE] = best; si[tid / KA_WAVE] = best_i; }
    __syncthreads();
    if (tid != 0) return;
    best = sf[0]; best_i = si[0];
    for (int w = 1; w < SM_WAVES; ++w) {
        float ov = sf[w]; int oi = si[w];
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    ka_store_token(out, pending, r, best_i == 0x7fffffff ? 0 : best_i);
}

__global__ void __launch_bounds__(SM_THREADS)
argmax_kernel(const float* __restrict__ logits, long ld, int* __restrict__ out, int V,
              PendingTable pending) {
    __shared__ float sf[SM_WAVES];
    __shared__ int si[SM_WAVES];
    int r = blockIdx.x;
    int idx = block_argmax(logits + (size_t)r * ld, V, sf, si);
    if (threadIdx.x == 0) ka_store_token(out, pending, r, idx);
}

__global__ void __launch_bounds__(SM_THREADS)
sample_kernel(const float* __restrict__ logits, long ld, const float* __restrict__ temps,
              const float* __restrict__ top_ps, const unsigned long long* __restrict__ rng_key,
              const int* __restrict__ rng_counter, int* __restrict__ out, int V,
              PendingTable pending) {
    __shared__ float sf[SM_WAVES];
    __shared__ int si[SM_WAVES];
    __shared__ float wave_tot[SM_WAVES];
    __shared__ int found_idx;
    int r = blockIdx.x;
    const float* row = logits + (size_t)r * ld;
    float T = temps[r];
    int greedy = block_argmax(row, V, sf, si);
    if (!(T > SM_GREEDY_EPS)) {
        if (threadIdx.x == 0) ka_store_token(out, pending, r, greedy);
        return;
    }
    float inv_t = 1.0f / T;
    float mx = row[greedy];
    float z = 0.f;
    for (int i = threadIdx.x; i < V; i += SM_THREADS) z += expf((row[i] - mx) * inv_t);
    z = block_reduce_sum(z, sf);
    float inv_z = 1.0f / z;
    float top_p = top_ps ? top_ps[r] : 1.0f;
    float thresh = 0.f, mass = 1.0f;
    if (top_p < 1.0f) {
        // f(t) = mass of {p >= t} falls with t; keep the largest t with f(t) >= top_p.
        float lo = 0.f, hi = 1.0f + 1e-6f;
        for (int it = 0; it < 30; ++it) {
            float mid = 0.5f * (lo + hi);
            float f = 0.f;
            for (int i = threadIdx.x; i < V; i += SM_THREADS) {
                float p = expf((row[i] - mx) * inv_t) * inv_z;
                if (p >= mid) f += p;
            }
            f = block_reduce_sum(f, sf);
            if (f >= top_p) lo = mid; else hi = mid;
        }
        thresh = lo;
        float f = 0.f;
        for (int i = threadIdx.x; i < V; i += SM_THREADS) {
            float p = expf((row[i] - mx) * inv_t) * inv_z;
            if (p >= thresh) f += p;
        }
        mass = block_reduce_sum(f, sf);
    }
    float u = ka_uniform(rng_key[r], (unsigned long long)(unsigned)rng_counter[r]);
    float target = u * mass;
    // Inversion in index order: first i with cumulative mass > target.
    if (threadIdx.x == 0) found_idx = -1;
    __syncthreads();
    float running = 0.f;
    int lane = threadIdx.x % KA_WAVE, wave = threadIdx.x / KA_WAVE;
    for (int base = 0; base < V; base += SM_THREADS) {
        int i = base + threadIdx.x;
        float p = 0.f;
        if (i < V) {
            p = expf((row[i] - mx) * inv_t) * inv_z;
            if (p < thresh || p <= 0.f) p = 0.f;
        }
        // inclusive scan inside the wave
        const float scan = ka_wave_running_sum(p);
        __syncthreads();
        if (lane == KA_WAVE - 1) wave_tot[wave] = scan;
        __syncthreads();
        float before = running;
        for (int w = 0; w < wave; ++w) before += wave_tot[w];
        float chunk = 0.f;
#pragma unroll
        for (int w = 0; w < SM_WAVES; ++w) chunk += wave_tot[w];
        float incl = before + scan;
        if (p > 0.f && incl > target && incl - p <= target) atomicMax(&found_idx, i);
        running += chunk;
        __syncthreads();
        if (found_idx >= 0) break;
    }
    if (threadIdx.x == 0) ka_store_token(out, pending, r, found_idx >= 0 ? found_idx : greedy);
}

// The same selection for rows of at most R * 1024 logits, each read once: a thread keeps its R
// logits (then probabilities) in registers. The threshold of the nucleus is bisected between 0
// and the largest probability and the search ends as soon as no probability lies between its
// bounds (the set {p >= threshold} is then settled); once few probabilities are left between
// the bounds they are gathered, a few per thread, and the rounds after that look at those alone.
// The draw is located by wave sums of the
// groups of 64 neighbouring tokens, one scan of those, and one scan inside the group found.
// sample_kernel above passes over the row about 35 times (300 us at a vocabulary of 51200: a
// quarter of a decode step); this one takes about a tenth of that.
template <int R>
__global__ void __launch_bounds__(SM_THREADS)
sample_regs_kernel(const float* __restrict__ logits, long ld, const float* __restrict__ temps,
                   const float* __restrict__ top_ps, const unsigned long long* __restrict__ rng_key,
                   const int* __restrict__ rng_counter, int* __restrict__ out, int V,
                   PendingTable pending) {
    __shared__ float sf[SM_WAVES];
    __shared__ int si[SM_WAVES];
    __shared__ float group_sum[R * SM_WAVES];       // of tokens (j * 1024 + wave * 64) .. + 64, in that order
    __shared__ float round_sums[2][3][SM_WAVES];
    __shared__ float picked_list[SM_PICKED];
    __shared__ int found_group;
    __shared__ float found_before;
    const int r = blockIdx.x, tid = threadIdx.x;
    const int lane = tid % KA_WAVE, wave = tid / KA_WAVE;
    const float* row = logits + (size_t)r * ld;
    const float T = temps[r];
    // (every load unconditional, from a place moved inside the row: a load under a branch would
    // make the compiler wait for each one before the next is asked for)
    float x[R];
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = row[min(j * SM_THREADS + tid, V - 1)];
#pragma unroll
    for (int j = 0; j < R; ++j)
        if (j * SM_THREADS + tid >= V) x[j] = -INFINITY;
    // the maximum and its first index
    float best = -INFINITY;
    int best_i = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int i = j * SM_THREADS + tid;
        if (i < V && x[j] > best) { best = x[j]; best_i = i; }      // j rises with i: the first of equals stays
    }
    wave_argmax(best, best_i);
    if (lane == 0) { sf[wave] = best; si[wave] = best_i; }
    __syncthreads();
    best = sf[0]; best_i = si[0];
    for (int w = 1; w < SM_WAVES; ++w) {
        float ov = sf[w]; int oi = si[w];
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    const int greedy = best_i == 0x7fffffff ? 0 : best_i;
    if (!(T > SM_GREEDY_EPS)) {
        if (tid == 0) ka_store_token(out, pending, r, greedy);
        return;
    }
    const float inv_t = 1.0f / T, mx = best;
    float z = 0.f;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        x[j] = __expf((x[j] - mx) * inv_t);            // exp(-inf) = 0: masked tokens and the places past V (the hardware's exp2: 9 of the kernel's 33 us otherwise)
        z += x[j];
    }
    z = block_reduce_sum(z, sf);
    const float inv_z = 1.0f / z;
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] *= inv_z;
    const float top_p = top_ps ? top_ps[r] : 1.0f;
    float thresh = 0.f, mass = 1.0f;
    if (top_p < 1.0f) {
        // f(t) = mass of {p >= t} falls with t; keep the largest t with f(t) >= top_p. The lower
        // bound starts at the smallest normal number: what lies below it holds less than 1e-33
        // together and is never needed to reach top_p (at most 1 - 6e-8).
        float lo = 1.17549435e-38f, hi = inv_z * (1.0f + 1e-6f) + 1e-30f;      // hi: just above the largest probability
        float above = 0.f;                                                     // f(hi): the mass at and above hi
        // Once at most SM_PICKED probabilities are left between the bounds they are gathered, a few
        // per thread, and the rounds after that look at those alone (a round over all R registers
        // costs 2.4 us at R = 52, one over the few 0.4 us).
        bool picked = false;
        float c[SM_PICKED / SM_THREADS];
#pragma unroll
        for (int k = 0; k < SM_PICKED / SM_THREADS; ++k) c[k] = 0.f;
        for (int it = 0; it < 40; ++it) {
            // The first threshold tried is 1 / SM_PICKED: no more than SM_PICKED probabilities can be
            // that large, so if they reach top_p (a model that is sure of itself) the gathering
            // follows at once. After that, the middle of the bounds.
            const float first = 1.0f / (float)SM_PICKED;
            const float mid = it == 0 && first < hi ? first : 0.5f * (lo + hi);
            // the mass at and above mid (of the gathered ones: below hi), the number of probabilities
            // in [lo, hi) and of those in [mid, hi)
            float f = 0.f;
            int n_in = 0, n_up = 0;
            if (!picked) {
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    const bool up = x[j] >= mid, in = x[j] >= lo && x[j] < hi;
                    f += up ? x[j] : 0.f;
                    n_in += in ? 1 : 0;
                    n_up += in && up ? 1 : 0;
                }
            } else {
#pragma unroll
                for (int k = 0; k < SM_PICKED / SM_THREADS; ++k) {
                    const bool in = c[k] >= lo && c[k] < hi, up = in && c[k] >= mid;
                    f += up ? c[k] : 0.f;
                    n_in += in ? 1 : 0;
                    n_up += up ? 1 : 0;
                }
            }
            // three sums over the workgroup: a value per wave through LDS, in one of two sets of
            // places by turns, so that one barrier a round is enough (a wave that is a round ahead
            // writes the other set); each row of 16 lanes then adds up the 16 waves' values, all
            // in one order, so every lane decides alike
            static_assert(SM_WAVES == 16, "the waves' sums meet in a row of 16 lanes");
            f = ka_wave_sum(f);
            const float wave_in = ka_wave_sum((float)n_in), wave_up = ka_wave_sum((float)n_up);
            float* places = &round_sums[it & 1][0][0];
            if (lane == 0) { places[wave] = f; places[SM_WAVES + wave] = wave_in; places[2 * SM_WAVES + wave] = wave_up; }
            __syncthreads();
            const float mass_up = ka_lanes_reduce<1, SM_WAVES>(places[lane % SM_WAVES], KaSum{});
            const float all_in = ka_lanes_reduce<1, SM_WAVES>(places[SM_WAVES + lane % SM_WAVES], KaSum{});
            const float all_up = ka_lanes_reduce<1, SM_WAVES>(places[2 * SM_WAVES + lane % SM_WAVES], KaSum{});
            const float at_mid = picked ? above + mass_up : mass_up;           // f(mid)
            const bool exhausted = !(mid > lo && mid < hi);                   // no float left between the bounds
            const bool rises = at_mid >= top_p;
            float between;                                                    // probabilities between the new bounds
            if (rises) { lo = mid; between = all_up; }
            else { hi = mid; above = at_mid; between = all_in - all_up; }
            // f(lo) >= top_p > f(hi) throughout. With at most one probability in [lo, hi) the
            // tokens above hi do not reach top_p, so that one is needed: {p >= lo} is the nucleus,
            // the same set for the old and the new bounds.
            if (between <= 1.f || exhausted) break;
            if (!picked && between <= (float)SM_PICKED) {
                // every wave knows how many each wave brings (the sums above, per wave): its own
                // start in the list follows from those before it, and a lane's place from the
                // lanes before it
                int at = 0;
                for (int w = 0; w < wave; ++w)
                    at += (int)(rises ? places[2 * SM_WAVES + w] : places[SM_WAVES + w] - places[2 * SM_WAVES + w]);
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    const bool in = x[j] >= lo && x[j] < hi;
                    const unsigned long long holds = __ballot(in);
                    if (holds) {
                        const int before = __builtin_amdgcn_mbcnt_hi((unsigned)(holds >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)holds, 0u));
                        if (in) picked_list[min(at + before, SM_PICKED - 1)] = x[j];
                        at += __popcll(holds);
                    }
                }
                __syncthreads();
                const int n = (int)between;
#pragma unroll
                for (int k = 0; k < SM_PICKED / SM_THREADS; ++k) c[k] = k * SM_THREADS + tid < n ? picked_list[k * SM_THREADS + tid] : 0.f;
                picked = true;
            }
        }
        thresh = lo;
        float f = 0.f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (x[j] < thresh) x[j] = 0.f;
            f += x[j];
        }
        mass = block_reduce_sum(f, sf);
    }
    const float u = ka_uniform(rng_key[r], (unsigned long long)(unsigned)rng_counter[r]);
    const float target = u * mass;
    // Inversion in index order: the first token whose cumulative mass exceeds the target.
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; ++j) {
        float g = ka_wave_sum(x[j]);
        if (lane == 0) group_sum[j * SM_WAVES + wave] = g;
    }
    if (tid == 0) found_group = -1;
    __syncthreads();
    if (wave == 0) {
        // one wave walks over the R * 16 group sums, 64 at a time
        float running = 0.f;
        for (int base = 0; base < R * SM_WAVES; base += KA_WAVE) {
            const int gi = base + lane;
            const float v = gi < R * SM_WAVES ? group_sum[gi] : 0.f;
            const float scan = ka_wave_running_sum(v);
            // sums only grow along the lanes: the first one past the target is the group (its own
            // sum is then positive: the one before was not past it)
            const float incl = running + scan;
            const unsigned long long hit = __ballot(incl > target && v > 0.f);
            if (hit) {
                const int first = __ffsll((long long)hit) - 1;
                if (lane == first) { found_group = gi; found_before = incl - v; }
                break;
            }
            running += ka_lane_value(scan, KA_WAVE - 1);
        }
    }
    __syncthreads();
    const int grp = found_group;
    int token = greedy;
    if (grp >= 0) {
        const int j = grp / SM_WAVES, w = grp % SM_WAVES;
        if (wave == w) {
            float p = 0.f;
#pragma unroll
            for (int jj = 0; jj < R; ++jj)
                if (jj == j) p = x[jj];
            const float scan = ka_wave_running_sum(p);
            const float incl = found_before + scan;
            const unsigned long long past = __ballot(p > 0.f && incl > target);
            const unsigned long long any = __ballot(p > 0.f);
            // the first token past the target; if the two ways of summing disagree in the last
            // bit and none is, the group's last token with any mass
            int pick = -1;
            if (past) pick = __ffsll((long long)past) - 1;
            else if (any) pick = 63 - __clzll((long long)any);
            if (lane == (pick < 0 ? 0 : pick)) ka_store_token(out, pending, r, pick < 0 ? greedy : j * SM_THREADS + w * KA_WAVE + pick);
        }
        return;
    }
    if (tid == 0) ka_store_token(out, pending, r, token);
}

KA_API int ka_argmax(const float* logits, long ld, int* out, int rows, int V, int* pending,
                     const int* pending_at, int n_pending, hipStream_t stream) {
    KA_CHECK(!pending || (pending_at && n_pending > 0), "ka_argmax: a pending table needs its places");
    KA_CHECK(rows >= 0 && V > 0 && ld >= V, "ka_argmax: bad sizes rows=%d V=%d ld=%ld", rows, V, ld);
    if (rows == 0) return 0;
    const PendingTable table{pending, pending_at, n_pending};
    const int per_thread = ka_cdiv(V, SM_THREADS);
    if (per_thread <= 16)
        hipLaunchKernelGGL(argmax_regs_kernel<16>, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, out, V, table);
    else if (per_thread <= 52)
        hipLaunchKernelGGL(argmax_regs_kernel<52>, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, out, V, table);
    else
        hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, out, V, table);
    KA_LAUNCH_CHECK();
    return 0;
}

static int sm_passes_only = 0;

KA_API int ka_sample(const float* logits, long ld, const float* temps, const float* top_ps,
                     const unsigned long long* rng_key, const int* rng_counter, int* out, int rows,
                     int V, int* pending, const int* pending_at, int n_pending, hipStream_t stream) {
    KA_CHECK(rows >= 0 && V > 0 && ld >= V, "ka_sample: bad sizes rows=%d V=%d ld=%ld", rows, V, ld);
    KA_CHECK(!pending || (pending_at && n_pending > 0), "ka_sample: a pending table needs its places");
    KA_CHECK(temps && rng_key && rng_counter, "ka_sample: temperatures and generator state are required");
    if (rows == 0) return 0;
    const PendingTable table{pending, pending_at, n_pending};
    const int per_thread = ka_cdiv(V, SM_THREADS);
#define KA_SAMPLE_REGS(RV)                                                                                        \
    hipLaunchKernelGGL(sample_regs_kernel<RV>, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, temps, top_ps, \
                       rng_key, rng_counter, out, V, table)
    if (sm_passes_only || per_thread > 64)
        hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, temps, top_ps, rng_key,
                           rng_counter, out, V, table);
    else if (per_thread <= 8) KA_SAMPLE_REGS(8);
    else if (per_thread <= 16) KA_SAMPLE_REGS(16);
    else if (per_thread <= 32) KA_SAMPLE_REGS(32);
    else if (per_thread <= 40) KA_SAMPLE_REGS(40);
    else if (per_thread <= 52) KA_SAMPLE_REGS(52);
    else KA_SAMPLE_REGS(64);
#undef KA_SAMPLE_REGS
    KA_LAUNCH_CHECK();
    return 0;
}

// 1: every row goes through the kernel that passes over the row many times, whatever its length
// (otherwise rows longer than 65536 only): for tests of that kernel.
KA_API void ka_sample_set_passes_only(int on) { sm_passes_only = on; }

// ----------------------------------------------------------------------------
// Masks before sampling (kestrel/scheduler/scheduler.py:2563-2604,2854-2927): tokens a request
// suppresses get -inf; a request with an allow-list keeps only the tokens on it.
// ----------------------------------------------------------------------------
__global__ void suppress_kernel(float* __restrict__ logits, long ld, const int* __restrict__ rows,
                                const int* __restrict__ tokens, int n, int V) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int token = tokens[i];
    if (token >= 0 && token < V) logits[(size_t)rows[i] * ld + token] = -INFINITY;
}

// Row r keeps the tokens allowed[starts[r] .. starts[r + 1]) (sorted ascending); an empty list
// means no restriction.
__global__ void __launch_bounds__(256)
allow_kernel(float* __restrict__ logits, long ld, const int* __restrict__ starts,
             const int* __restrict__ allowed, int V) {
    const int r = blockIdx.y;
    const int lo0 = starts[r], hi0 = starts[r + 1];
    if (hi0 <= lo0) return;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < V; i += gridDim.x * blockDim.x) {
        int lo = lo0, hi = hi0;            // first entry >= i
        while (lo < hi) {
            int mid = (lo + hi) >> 1;
            if (allowed[mid] < i) lo = mid + 1; else hi = mid;
        }
        if (!(lo < hi0 && allowed[lo] == i)) logits[(size_t)r * ld + i] = -INFINITY;
    }
}

KA_API int ka_suppress_tokens(float* logits, long ld, const int* rows, const int* tokens, int n, int V,
                              hipStream_t stream) {
    KA_CHECK(n >= 0 && V > 0 && ld >= V, "ka_suppress_tokens: bad sizes n=%d V=%d ld=%ld", n, V, ld);
    if (n == 0) return 0;
    hipLaunchKernelGGL(suppress_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, logits, ld, rows, tokens, n, V);
    KA_LAUNCH_CHECK();
    return 0;
}

KA_API int ka_allow_tokens(float* logits, long ld, const int* starts, const int* allowed, int rows, int V,
                           hipStream_t stream) {
    KA_CHECK(rows >= 0 && V > 0 && ld >= V, "ka_allow_tokens: bad sizes rows=%d V=%d ld=%ld", rows, V, ld);
    if (rows == 0) return 0;
    int blocks = (V + 255) / 256;
    if (blocks > 64) blocks = 64;
    hipLaunchKernelGGL(allow_kernel, dim3(blocks, rows), dim3(256), 0, stream, logits, ld, starts, allowed, V);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Log-probability of the chosen token (kestrel/scheduler/scheduler.py:3019-3042): with a
// temperature above 1e-6, log softmax(logits / T)[token]; otherwise (greedy, or a row whose
// normaliser is not finite) 0 if the token is the argmax and -inf if not.
// ----------------------------------------------------------------------------
__global__ void __launch_bounds__(SM_THREADS)
logprob_kernel(const float* __restrict__ logits, long ld, const int* __restrict__ ids,
               const float* __restrict__ temps, float* __restrict__ out, int V) {
    __shared__ float sf[SM_WAVES];
    __shared__ int si[SM_WAVES];
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * ld;
    const int greedy = block_argmax(row, V, sf, si);
    const float T = temps ? fmaxf(temps[r], 0.f) : 0.f;
    const float eff = T > SM_GREEDY_EPS ? T : 1.0f;
    const float mx = row[greedy] / eff;
    float z = 0.f;
    for (int i = threadIdx.x; i < V; i += SM_THREADS) z += expf(row[i] / eff - mx);
    z = block_reduce_sum(z, sf);
    if (threadIdx.x != 0) return;
    const float normaliser = mx + logf(z);
    const int id = ids[r];
    const bool force_greedy = !(T > SM_GREEDY_EPS) || !isfinite(normaliser);
    float lp;
    if (force_greedy) lp = id == greedy ? 0.f : -INFINITY;
    else lp = (id >= 0 && id < V ? row[id] / eff : -INFINITY) - normaliser;
    out[r] = lp;
}

KA_API int ka_token_logprobs(const float* logits, long ld, const int* ids, const float* temps, float* out,
                             int rows, int V, hipStream_t stream) {
    KA_CHECK(rows >= 0 && V > 0 && ld >= V, "ka_token_logprobs: bad sizes rows=%d V=%d ld=%ld", rows, V, ld);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(logprob_kernel, dim3(rows), dim3(SM_THREADS), 0, stream, logits, ld, ids, temps, out, V);
    KA_LAUNCH_CHECK();
    return 0;
}

// The uniform number the kernel draws, for tests and host-side replay.
KA_API float ka_uniform_host(unsigned long long key, unsigned long long counter) { return ka_uniform(key, counter); }
