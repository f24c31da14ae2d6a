// Two measuring kernels: what this GPU reaches on a plain read stream and on a loop of matrix
// instructions that waits for nothing. The rooflines that bench.py reports against nominal
// figures (8 TB/s, 2.5 PFLOP/s) can be reported against these as well.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(4))) unsigned int ka_u4;
typedef __attribute__((ext_vector_type(8))) __bf16 ka_bf16x8;
typedef __attribute__((ext_vector_type(16))) float ka_floatx16;

constexpr int PK_THREADS = 256;
constexpr int PK_UNROLL = 8;

// Every thread reads 16 bytes eight times per round, the whole grid walking over the buffer.
__global__ void __launch_bounds__(PK_THREADS) peak_read_kernel(const ka_u4* __restrict__ p, long n16, unsigned* sink) {
    long i = (long)blockIdx.x * PK_THREADS * PK_UNROLL + threadIdx.x;
    const long stride = (long)gridDim.x * PK_THREADS * PK_UNROLL;
    unsigned acc = 0;
    for (; i + (long)PK_THREADS * (PK_UNROLL - 1) < n16; i += stride) {
        ka_u4 v[PK_UNROLL];
#pragma unroll
        for (int u = 0; u < PK_UNROLL; ++u) v[u] = p[i + (long)PK_THREADS * u];
#pragma unroll
        for (int u = 0; u < PK_UNROLL; ++u) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
    if (acc == 0x12345678u) sink[0] = acc;       // keeps the loads alive; practically never taken
}

// Eight independent accumulators per wave, operands in registers: nothing but v_mfma_f32_32x32x16_bf16.
__global__ void __launch_bounds__(PK_THREADS) peak_mfma_kernel(float* sink, int iters) {
    constexpr int NACC = 8;
    ka_floatx16 acc[NACC];
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[a][v] = 0.f;
    ka_bf16x8 x, y;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        x[j] = (__bf16)(float)((threadIdx.x + j) % 7);
        y[j] = (__bf16)(float)((threadIdx.x * 3 + j) % 5);
    }
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int a = 0; a < NACC; ++a) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[a], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += acc[a][v];
    if (s == 0.12345f) sink[0] = s;
}

// Reads `bytes` (a multiple of 16, 16-byte aligned) once with `workgroups` workgroups.
KA_API int ka_peak_read(const void* buffer, long bytes, int workgroups, void* sink, hipStream_t stream) {
    KA_CHECK(buffer && sink && bytes >= 16 && (uintptr_t)buffer % 16 == 0, "ka_peak_read: needs a 16-byte aligned buffer and a sink");
    KA_CHECK(workgroups > 0 && workgroups <= 1 << 20, "ka_peak_read: bad number of workgroups %d", workgroups);
    hipLaunchKernelGGL(peak_read_kernel, dim3(workgroups), dim3(PK_THREADS), 0, stream, (const ka_u4*)buffer, bytes / 16,
                       (unsigned*)sink);
    KA_LAUNCH_CHECK();
    return 0;
}

// `workgroups` x 4 waves x `iters` x 8 matrix instructions of 32 x 32 x 16 (32,768 flops each).
KA_API int ka_peak_mfma_bf16(void* sink, int workgroups, int iters, hipStream_t stream) {
    KA_CHECK(sink && workgroups > 0 && workgroups <= 1 << 16 && iters > 0, "ka_peak_mfma_bf16: bad sizes");
    hipLaunchKernelGGL(peak_mfma_kernel, dim3(workgroups), dim3(PK_THREADS), 0, stream, (float*)sink, iters);
    KA_LAUNCH_CHECK();
    return 0;
}
