// The step after the MoE layer in the transformer block: the residual add, or the hyper-connection post mix
// (out[t,i,:] = x[t,:] * post_mix[t,i] + sum_j comb[t,j,i] * residual[t,j,:], all in f32, rounded to bf16).
// Memory bound: one thread owns 8 columns of one token, reads its 16 bytes of x and of every residual stream
// once and writes hc_mult pieces; the hc_mult * (hc_mult + 1) mix coefficients of the token come through the
// scalar/constant path of the cache (every lane of a wavefront that shares the token reads the same words).
#include "common.h"

namespace dmoe {

constexpr int kMaxHcMult = 8;

__device__ __forceinline__ void widen8(const uint4 &v, float *f) {
    f[0] = bf16_bits_to_f32(v.x & 0xffffu), f[1] = bf16_bits_to_f32(v.x >> 16);
    f[2] = bf16_bits_to_f32(v.y & 0xffffu), f[3] = bf16_bits_to_f32(v.y >> 16);
    f[4] = bf16_bits_to_f32(v.z & 0xffffu), f[5] = bf16_bits_to_f32(v.z >> 16);
    f[6] = bf16_bits_to_f32(v.w & 0xffffu), f[7] = bf16_bits_to_f32(v.w >> 16);
}
__device__ __forceinline__ uint4 narrow8(const float *f) {
    uint4 o;
    o.x = (uint32_t)f32_to_bf16_bits(f[0]) | ((uint32_t)f32_to_bf16_bits(f[1]) << 16);
    o.y = (uint32_t)f32_to_bf16_bits(f[2]) | ((uint32_t)f32_to_bf16_bits(f[3]) << 16);
    o.z = (uint32_t)f32_to_bf16_bits(f[4]) | ((uint32_t)f32_to_bf16_bits(f[5]) << 16);
    o.w = (uint32_t)f32_to_bf16_bits(f[6]) | ((uint32_t)f32_to_bf16_bits(f[7]) << 16);
    return o;
}

__global__ __launch_bounds__(256) void residual_add_kernel(uint4 *__restrict__ out, const uint4 *__restrict__ x,
                                                           const uint4 *__restrict__ res, size_t n8) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    float a[8], b[8];
    widen8(x[i], a);
    widen8(res[i], b);
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] = b[k] + a[k];
    out[i] = narrow8(a);
}

// deepseek_v4.zig:2450-2499; M = hc_mult
template <int M>
__global__ __launch_bounds__(256) void mhc_post_kernel(uint4 *__restrict__ out, const uint4 *__restrict__ x,
                                                       const uint4 *__restrict__ res, const float *__restrict__ post_mix,
                                                       const float *__restrict__ comb_mix, int T, int d8) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)T * d8) return;
    const size_t t = i / (size_t)d8, c = i - t * (size_t)d8;
    float xv[8];
    widen8(x[i], xv);
    float rv[M][8];
#pragma unroll
    for (int j = 0; j < M; ++j) widen8(res[(t * M + j) * (size_t)d8 + c], rv[j]);
    const float *post = post_mix + t * M, *comb = comb_mix + t * M * M;
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const float pm = post[m];
        float o[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            float term2 = comb[m] * rv[0][k]; // comb is used transposed: coefficient [j][m] multiplies stream j
#pragma unroll
            for (int j = 1; j < M; ++j) term2 = fmaf(comb[j * M + m], rv[j][k], term2);
            o[k] = xv[k] * pm + term2;
        }
        out[(t * M + m) * (size_t)d8 + c] = narrow8(o);
    }
}

} // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_block_post(uint16_t *d_out, const uint16_t *d_ffn_out, const uint16_t *d_residual,
                               const float *d_post_mix, const float *d_comb_mix, int T, int D, int hc_mult,
                               dmoe_stream s) {
    DMOE_REQUIRE(T >= 0 && D > 0 && D % 8 == 0, "block_post: T=%d D=%d (D must be a multiple of 8)", T, D);
    DMOE_REQUIRE(hc_mult >= 0 && hc_mult <= kMaxHcMult, "block_post: hc_mult=%d (0..%d)", hc_mult, kMaxHcMult);
    if (T == 0) return DMOE_OK;
    DMOE_REQUIRE(d_out && d_ffn_out && d_residual, "block_post: null pointer");
    DMOE_REQUIRE(((uintptr_t)d_out % 16) == 0 && ((uintptr_t)d_ffn_out % 16) == 0 && ((uintptr_t)d_residual % 16) == 0,
                 "block_post: activations must be 16-byte aligned");
    hipStream_t st = to_hip(s);
    const int d8 = D / 8;
    const size_t n8 = (size_t)T * d8;
    const dim3 grid((unsigned)((n8 + 255) / 256)), block(256);
    if (hc_mult == 0) {
        hipLaunchKernelGGL(residual_add_kernel, grid, block, 0, st, (uint4 *)d_out, (const uint4 *)d_ffn_out,
                           (const uint4 *)d_residual, n8);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    DMOE_REQUIRE(d_post_mix && d_comb_mix, "block_post: hc_mult=%d needs post_mix and comb_mix", hc_mult);
#define DMOE_POST_CASE(M)                                                                                        \
    case M:                                                                                                      \
        hipLaunchKernelGGL(mhc_post_kernel<M>, grid, block, 0, st, (uint4 *)d_out, (const uint4 *)d_ffn_out,      \
                           (const uint4 *)d_residual, d_post_mix, d_comb_mix, T, d8);                             \
        break;
    switch (hc_mult) {
        DMOE_POST_CASE(1)
        DMOE_POST_CASE(2)
        DMOE_POST_CASE(3)
        DMOE_POST_CASE(4)
        DMOE_POST_CASE(5)
        DMOE_POST_CASE(6)
        DMOE_POST_CASE(7)
        DMOE_POST_CASE(8)
    }
#undef DMOE_POST_CASE
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}
