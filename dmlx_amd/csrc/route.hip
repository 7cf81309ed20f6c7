// Router top-k (one wavefront per token, shuffle reductions), index remap, expand / reduce,
// and the host-side Smelt mask / remap builders.
#include <math.h>
#include <string.h>

#include "common.h"
#include "route_device.h"

namespace dmoe {

constexpr int kRouteWaves = 4;

// One wavefront per token (route_tokens); EPL = experts per lane
template <int EPL>
__global__ __launch_bounds__(kRouteWaves * 64) void route_kernel(
    uint32_t *__restrict__ out_idx, float *__restrict__ out_w, const float *__restrict__ scores,
    const float *__restrict__ bias, const uint8_t *__restrict__ resident, int T, int E, int K,
    int normalize, int apply_scale, float route_scale) {
    const int wave = (int)(threadIdx.x >> 6), lane = lane_id();
    const int t = (int)blockIdx.x * kRouteWaves + wave;
    if (t >= T) return;
    const float *const rows[1] = {scores + (size_t)t * E};
    uint32_t my_idx[1];
    float w[1];
    route_tokens<1, EPL>(rows, bias, resident, E, K, normalize, apply_scale, route_scale, lane, my_idx, w);
    if (lane < K) {
        out_idx[(size_t)t * K + lane] = my_idx[0];
        out_w[(size_t)t * K + lane] = w[0];
    }
}

static int launch_route(uint32_t *out_idx, float *out_w, const float *scores, const float *bias,
                        const uint8_t *resident, int T, int E, int K, int normalize, int apply_scale,
                        float route_scale, hipStream_t st) {
    DMOE_REQUIRE(T >= 0 && E >= 1 && E <= 1024, "route: E=%d out of range [1,1024]", E);
    DMOE_REQUIRE(K >= 1 && K <= E && K <= 64, "route: K=%d must satisfy 1 <= K <= min(E,64)", K);
    if (T == 0) return DMOE_OK;
    DMOE_REQUIRE(out_idx && out_w && scores, "route: null pointer");
    dim3 grid((unsigned)ceil_div(T, kRouteWaves)), block(kRouteWaves * 64);
    if (E <= 256)
        hipLaunchKernelGGL(route_kernel<4>, grid, block, 0, st, out_idx, out_w, scores, bias, resident, T, E, K, normalize,
                           apply_scale, route_scale);
    else
        hipLaunchKernelGGL(route_kernel<16>, grid, block, 0, st, out_idx, out_w, scores, bias, resident, T, E, K, normalize,
                           apply_scale, route_scale);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

int launch_route(const RouteArgs &r, hipStream_t st) {
    return launch_route(r.out_idx, r.out_w, r.scores, r.bias, r.resident, r.T, r.E, r.K, r.normalize, r.apply_scale,
                        r.route_scale, st);
}

__global__ void remap_kernel(uint32_t *__restrict__ out, const int32_t *__restrict__ remap,
                             const uint32_t *__restrict__ idx, size_t n, uint32_t n_total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint32_t e = idx[i];
    // an id outside the table would read out of bounds; map it to slot 0 like an unloaded expert
    out[i] = e < n_total ? (uint32_t)remap[e] : 0u;
}

// out[(t*K+k), :] = x[t, :]: one thread per 16 bytes of x, read once and stored K times
__global__ void expand_kernel(uint4 *__restrict__ out, const uint4 *__restrict__ x, size_t row_vecs,
                              int K, size_t in_vecs) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= in_vecs) return;
    const size_t t = i / row_vecs, c = i - t * row_vecs;
    const uint4 v = x[i];
    uint4 *o = out + t * (size_t)K * row_vecs + c;
    for (int k = 0; k < K; ++k) o[(size_t)k * row_vecs] = v;
}
__global__ void expand_kernel_bytes(uint8_t *__restrict__ out, const uint8_t *__restrict__ x,
                                    size_t row_bytes, int K, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    size_t row = i / row_bytes, c = i - row * row_bytes;
    out[i] = x[(row / (size_t)K) * row_bytes + c];
}

template <bool BF16>
__global__ void reduce_kernel(float *__restrict__ out, const void *__restrict__ eo,
                              const float *__restrict__ w, int T, int K, int D) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)T * D) return;
    size_t t = i / (size_t)D, d = i - t * (size_t)D;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) {
        size_t r = t * (size_t)K + k;
        float v = BF16 ? bf16_bits_to_f32(((const uint16_t *)eo)[r * D + d]) : ((const float *)eo)[r * D + d];
        acc += v * w[r]; // separate multiply and add, k ascending
    }
    out[i] = acc;
}

// the same sums, 16 bytes of one expert row per load: a thread owns 8 (bf16) or 4 (f32) neighbouring columns of a token
template <bool BF16>
__global__ void reduce_vec_kernel(float4 *__restrict__ out, const uint4 *__restrict__ eo, const float *__restrict__ w,
                                  int T, int K, int vecs_per_row) {
    constexpr int NV = BF16 ? 8 : 4;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)T * vecs_per_row) return;
    const size_t t = i / (size_t)vecs_per_row, c = i - t * (size_t)vecs_per_row;
    float acc[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) acc[j] = 0.0f;
    for (int k = 0; k < K; ++k) {
        const size_t r = t * (size_t)K + k;
        const uint4 q = eo[r * (size_t)vecs_per_row + c];
        const float wk = w[r];
        float v[NV];
        if (BF16) {
            const uint32_t d[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[2 * j] = __uint_as_float(d[j] << 16);
                v[2 * j + 1] = __uint_as_float(d[j] & 0xffff0000u);
            }
        } else {
            v[0] = __uint_as_float(q.x), v[1] = __uint_as_float(q.y), v[2] = __uint_as_float(q.z), v[3] = __uint_as_float(q.w);
        }
#pragma unroll
        for (int j = 0; j < NV; ++j) acc[j] += v[j] * wk; // separate multiply and add, k ascending
    }
#pragma unroll
    for (int j = 0; j < NV / 4; ++j)
        out[i * (NV / 4) + j] = make_float4(acc[4 * j], acc[4 * j + 1], acc[4 * j + 2], acc[4 * j + 3]);
}

} // namespace dmoe

using namespace dmoe;

extern "C" {

int dmoe_topk_route(uint32_t *d_out_indices, float *d_out_weights, const float *d_scores, int T, int E,
                    int K, int normalize, dmoe_stream s) {
    return launch_route(d_out_indices, d_out_weights, d_scores, nullptr, nullptr, T, E, K, normalize, 0,
                        1.0f, to_hip(s));
}

int dmoe_gate_route(uint32_t *d_out_indices, float *d_out_weights, const float *d_scores,
                    const float *d_bias, const uint8_t *d_resident_mask, int T, int E, int K, int renorm,
                    float route_scale, dmoe_stream s) {
    return launch_route(d_out_indices, d_out_weights, d_scores, d_bias, d_resident_mask, T, E, K, renorm,
                        1, route_scale, to_hip(s));
}

int dmoe_remap_indices(uint32_t *d_out, const int32_t *d_remap, const uint32_t *d_indices, size_t n,
                       int n_total, dmoe_stream s) {
    if (n == 0) return DMOE_OK;
    DMOE_REQUIRE(d_out && d_remap && d_indices && n_total > 0, "remap: bad argument");
    hipLaunchKernelGGL(remap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, to_hip(s), d_out,
                       d_remap, d_indices, n, (uint32_t)n_total);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

int dmoe_expand_tokens(void *d_out, const void *d_x, int T, int D, int K, int elem_size, dmoe_stream s) {
    DMOE_REQUIRE(T >= 0 && D > 0 && K > 0 && (elem_size == 2 || elem_size == 4), "expand: bad shape");
    if (T == 0) return DMOE_OK;
    DMOE_REQUIRE(d_out && d_x, "expand: null pointer");
    size_t row_bytes = (size_t)D * elem_size;
    if (row_bytes % 16 == 0 && ((uintptr_t)d_out % 16 == 0) && ((uintptr_t)d_x % 16 == 0)) {
        size_t rv = row_bytes / 16, total = rv * (size_t)T;
        hipLaunchKernelGGL(expand_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, to_hip(s),
                           (uint4 *)d_out, (const uint4 *)d_x, rv, K, total);
    } else {
        size_t total = row_bytes * (size_t)T * K;
        hipLaunchKernelGGL(expand_kernel_bytes, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                           to_hip(s), (uint8_t *)d_out, (const uint8_t *)d_x, row_bytes, K, total);
    }
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

int dmoe_reduce_experts(float *d_out, const void *d_expert_outs, int outs_are_bf16, const float *d_weights,
                        int T, int K, int D, dmoe_stream s) {
    DMOE_REQUIRE(T >= 0 && D > 0 && K > 0, "reduce: bad shape");
    if (T == 0) return DMOE_OK;
    DMOE_REQUIRE(d_out && d_expert_outs && d_weights, "reduce: null pointer");
    const int nv = outs_are_bf16 ? 8 : 4;
    if (D % nv == 0 && ((uintptr_t)d_out % 16) == 0 && ((uintptr_t)d_expert_outs % 16) == 0) {
        const int vpr = D / nv;
        const size_t n = (size_t)T * vpr;
        dim3 vgrid((unsigned)((n + 255) / 256)), vblock(256);
        if (outs_are_bf16)
            hipLaunchKernelGGL(reduce_vec_kernel<true>, vgrid, vblock, 0, to_hip(s), (float4 *)d_out, (const uint4 *)d_expert_outs,
                               d_weights, T, K, vpr);
        else
            hipLaunchKernelGGL(reduce_vec_kernel<false>, vgrid, vblock, 0, to_hip(s), (float4 *)d_out, (const uint4 *)d_expert_outs,
                               d_weights, T, K, vpr);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    size_t total = (size_t)T * D;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (outs_are_bf16)
        hipLaunchKernelGGL(reduce_kernel<true>, grid, block, 0, to_hip(s), d_out, d_expert_outs, d_weights,
                           T, K, D);
    else
        hipLaunchKernelGGL(reduce_kernel<false>, grid, block, 0, to_hip(s), d_out, d_expert_outs,
                           d_weights, T, K, D);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

// ---- host-side builders (integers; no device work) -------------------------------------------------

int dmoe_smelt_build_mask(uint8_t *h_out_mask, int *out_n_resident, int n_experts, float load_fraction,
                          int strategy, int enabled) {
    DMOE_REQUIRE(h_out_mask && n_experts > 0, "smelt mask: bad argument");
    DMOE_REQUIRE(strategy == 0 || strategy == 1, "smelt mask: strategy must be 0 (uniform) or 1 (first)");
    memset(h_out_mask, 0, (size_t)n_experts);
    if (!enabled || load_fraction >= 1.0f) {
        memset(h_out_mask, 1, (size_t)n_experts);
    } else {
        // f32 arithmetic and round-half-away, as the reference's @round on f32
        long n_load = (long)roundf(load_fraction * (float)n_experts);
        if (n_load < 1) n_load = 1;
        if (n_load > n_experts) n_load = n_experts;
        if (strategy == 1) {
            for (long i = 0; i < n_load; ++i) h_out_mask[i] = 1;
        } else if (n_load == 1) {
            h_out_mask[0] = 1; // the reference divides by n_load-1 here; a single pick is expert 0
        } else {
            float step = (float)(n_experts - 1) / (float)(n_load - 1);
            for (long i = 0; i < n_load; ++i) {
                long idx = (long)roundf(step * (float)i);
                if (idx > n_experts - 1) idx = n_experts - 1;
                h_out_mask[idx] = 1;
            }
        }
    }
    if (out_n_resident) {
        int c = 0;
        for (int i = 0; i < n_experts; ++i) c += h_out_mask[i];
        *out_n_resident = c;
    }
    return DMOE_OK;
}

int dmoe_build_remap(int32_t *h_out_remap, const uint8_t *h_mask, int n_experts) {
    DMOE_REQUIRE(h_out_remap && h_mask && n_experts > 0, "build remap: bad argument");
    int32_t slot = 0;
    for (int e = 0; e < n_experts; ++e) h_out_remap[e] = h_mask[e] ? slot++ : 0;
    return DMOE_OK;
}

int dmoe_preload_remap(int32_t *h_out_remap, float *h_out_cache_bias, const uint32_t *h_expert_ids,
                       int n_ids, int n_total) {
    DMOE_REQUIRE(h_out_remap && (h_expert_ids || n_ids == 0) && n_total > 0 && n_ids >= 0,
                 "preload remap: bad argument");
    for (int e = 0; e < n_total; ++e) {
        h_out_remap[e] = 0;
        if (h_out_cache_bias) h_out_cache_bias[e] = -1000.0f;
    }
    for (int sidx = 0; sidx < n_ids; ++sidx) {
        DMOE_REQUIRE(h_expert_ids[sidx] < (uint32_t)n_total, "preload remap: expert id %u >= %d",
                     h_expert_ids[sidx], n_total);
        h_out_remap[h_expert_ids[sidx]] = sidx;
        if (h_out_cache_bias) h_out_cache_bias[h_expert_ids[sidx]] = 0.0f;
    }
    return DMOE_OK;
}

} // extern "C"
