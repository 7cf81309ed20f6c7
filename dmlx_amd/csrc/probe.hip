// Calibration kernels for the benchmark.
// (1) What the matrix cores reach when NOTHING else runs. Every wavefront repeats
// the 32 matrix instructions of one reduction step of the prefill kernels (4 x 2 accumulator tiles, four k-slices)
// on operands that stay in registers: no loads, no LDS, no decode inside the loop. The rate depends on the operand
// VALUES (all-zero operands toggle no multiplier inputs and draw less power), which is why the benchmark reports it
// for zero and for random operands next to the published peak.
#include "common.h"

namespace dmoe {

constexpr int kProbeWorkgroups = 512; // two per compute unit, like the prefill kernels
constexpr int kProbeThreads = 256;
constexpr int kProbeFragments = 24;   // 8 weight + 16 activation fragments of 8 bf16 per lane

__global__ __launch_bounds__(kProbeThreads, 2) void mfma_loop_kernel(float *__restrict__ out,
                                                                     const uint4 *__restrict__ in, int iters) {
    constexpr int MT = 4, NT = 2, NJ = 4;
    f32x16_t acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.0f;
    bf16x8_t wa[NJ][NT], xb[NJ][MT];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
#pragma unroll
        for (int n = 0; n < NT; ++n) wa[j][n] = __builtin_bit_cast(bf16x8_t, in[(j * NT + n) * kProbeThreads + threadIdx.x]);
#pragma unroll
        for (int m = 0; m < MT; ++m)
            xb[j][m] = __builtin_bit_cast(bf16x8_t, in[(NJ * NT + j * MT + m) * kProbeThreads + threadIdx.x]);
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[j][n], xb[j][m], acc[m][n], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
        // the operands stay opaque, so that nothing is hoisted out of the loop or merged
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int n = 0; n < NT; ++n) asm volatile("" : "+v"(wa[j][n]));
#pragma unroll
            for (int m = 0; m < MT; ++m) asm volatile("" : "+v"(xb[j][m]));
        }
    }
    float r = 0.0f;
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n)
#pragma unroll
            for (int q = 0; q < 16; ++q) r += acc[m][n][q];
    out[blockIdx.x * kProbeThreads + threadIdx.x] = r;
}

// What a kernel that ONLY reads can pull from memory: every wavefront streams a private contiguous region with eight
// 16-byte loads per lane in flight, with the streaming hint the decode kernel's weight loads carry.
constexpr int kReadUnroll = 8;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void read_stream_kernel(uint32_t *__restrict__ sink, const uint4 *__restrict__ src,
                                                          size_t vecs_per_wave) {
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const uint4 *q = src + wave * vecs_per_wave + (threadIdx.x & 63);
    uint32_t acc = 0;
    for (size_t i = 0; i + 64 * kReadUnroll <= vecs_per_wave; i += 64 * kReadUnroll) {
        u32x4_t v[kReadUnroll];
#pragma unroll
        for (int u = 0; u < kReadUnroll; ++u) v[u] = __builtin_nontemporal_load((const u32x4_t *)(q + i + 64 * u));
#pragma unroll
        for (int u = 0; u < kReadUnroll; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    // every load feeds the wavefront's checksum word, so that none of them can be dropped
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc ^= (uint32_t)__shfl_xor((int)acc, off, 64);
    if ((threadIdx.x & 63) == 0) sink[wave] = acc;
}

} // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_debug_read_stream(size_t *out_bytes_read, uint32_t *d_sink, const void *d_src, size_t bytes,
                                      int workgroups, dmoe_stream s) {
    DMOE_REQUIRE(out_bytes_read && d_sink && d_src, "debug_read_stream: null pointer");
    DMOE_REQUIRE(((uintptr_t)d_src % 16) == 0, "debug_read_stream: source must be 16-byte aligned");
    DMOE_REQUIRE(workgroups >= 1 && workgroups <= 65536, "debug_read_stream: workgroups=%d out of range [1, 65536]", workgroups);
    const size_t waves = (size_t)workgroups * 4, chunk = (size_t)64 * kReadUnroll;
    const size_t vecs_per_wave = (bytes / 16 / waves) / chunk * chunk; // whole chunks only: no access past `bytes`
    DMOE_REQUIRE(vecs_per_wave > 0, "debug_read_stream: %zu bytes are less than one 8 KiB chunk per wavefront", bytes);
    *out_bytes_read = vecs_per_wave * waves * 16;
    hipLaunchKernelGGL(read_stream_kernel, dim3((unsigned)workgroups), dim3(256), 0, to_hip(s), d_sink, (const uint4 *)d_src,
                       vecs_per_wave);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

extern "C" int dmoe_debug_mfma_loop(float *d_out, const uint16_t *d_operands, int iters, dmoe_stream s) {
    static_assert(kProbeWorkgroups * kProbeThreads == DMOE_MFMA_LOOP_OUT, "header constant out of date");
    static_assert(kProbeFragments * kProbeThreads * 8 == DMOE_MFMA_LOOP_OPERANDS, "header constant out of date");
    DMOE_REQUIRE(d_out && d_operands, "debug_mfma_loop: null pointer");
    DMOE_REQUIRE(((uintptr_t)d_operands % 16) == 0, "debug_mfma_loop: operands must be 16-byte aligned");
    DMOE_REQUIRE(iters >= 1 && iters <= (1 << 20), "debug_mfma_loop: iters=%d out of range [1, 2^20]", iters);
    hipLaunchKernelGGL(mfma_loop_kernel, dim3(kProbeWorkgroups), dim3(kProbeThreads), 0, to_hip(s), d_out,
                       (const uint4 *)d_operands, iters);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}
