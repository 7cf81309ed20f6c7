// Calibration kernel for the benchmark: what the matrix cores reach when NOTHING else runs. Every wavefront repeats
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

} // namespace dmoe

using namespace dmoe;

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
