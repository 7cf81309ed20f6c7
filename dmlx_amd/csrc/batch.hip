// batch_builder.build on the device (batch_builder.zig:90-214): the scheduler's requests arrive as one
// concatenated token array plus per-request (length, base position); positions, the token -> request map and
// the [T,T] block-diagonal causal mask are produced by kernels. The reference fills the mask on the host
// (O(T^2) floats, 268 MB at T = 8192) and copies it over; here it is written once at HBM speed.
#include <vector>

#include "common.h"

namespace dmoe {

// one thread per token: binary search of its request among the exclusive offsets
__global__ void batch_positions_kernel(int32_t *__restrict__ pos, uint32_t *__restrict__ req_of_token,
                                       const int32_t *__restrict__ offsets, const int32_t *__restrict__ base_pos,
                                       int n_req, int T) {
    const int t = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (t >= T) return;
    int lo = 0, hi = n_req - 1; // last request whose offset is <= t (empty requests share an offset: take the last)
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (offsets[mid] <= t) lo = mid;
        else hi = mid - 1;
    }
    if (pos) pos[t] = base_pos[lo] + (t - offsets[lo]);
    if (req_of_token) req_of_token[t] = (uint32_t)lo;
}

// mask[r][c] = 0 when r and c belong to the same request and c <= r, else -inf (batch_builder.zig:140-177);
// four columns per thread
__global__ void batch_mask_kernel(float4 *__restrict__ mask, const uint32_t *__restrict__ req_of_token, int T) {
    const int c4 = (int)(blockIdx.x * blockDim.x + threadIdx.x), r = (int)blockIdx.y;
    const int T4 = (T + 3) / 4;
    if (c4 >= T4) return;
    const uint32_t rr = req_of_token[r];
    const float ninf = -__builtin_inff();
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = c4 * 4 + i;
        v[i] = (c < T && c <= r && req_of_token[c] == rr) ? 0.0f : ninf;
    }
    if (c4 * 4 + 3 < T && (T & 3) == 0) {
        mask[(size_t)r * T4 + c4] = make_float4(v[0], v[1], v[2], v[3]);
    } else {
        float *row = (float *)mask + (size_t)r * T;
        for (int i = 0; i < 4; ++i)
            if (c4 * 4 + i < T) row[c4 * 4 + i] = v[i];
    }
}

} // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_batch_build(uint32_t *d_out_tokens, int32_t *d_out_positions, float *d_out_mask,
                                uint32_t *d_out_request_of_token, const uint32_t *h_tokens, const int32_t *h_seq_lens,
                                const int32_t *h_base_pos, int n_requests, int T, dmoe_workspace ws, dmoe_stream s) {
    DMOE_REQUIRE(n_requests >= 0 && T >= 0, "batch_build: negative size");
    if (T == 0) return DMOE_OK; // emptyBatch (batch_builder.zig:92-94, :129-131)
    DMOE_REQUIRE(n_requests >= 1 && h_seq_lens && h_base_pos, "batch_build: tokens without requests");
    long long sum = 0;
    for (int i = 0; i < n_requests; ++i) {
        DMOE_REQUIRE(h_seq_lens[i] >= 0 && h_base_pos[i] >= 0, "batch_build: request %d has a negative length or position", i);
        sum += h_seq_lens[i];
    }
    DMOE_REQUIRE(sum == T, "batch_build: request lengths sum to %lld, T is %d", sum, T);
    DMOE_REQUIRE(T <= 65535 || d_out_mask == nullptr, "batch_build: a [T,T] mask is limited to T <= 65535");
    hipStream_t st = to_hip(s);
    Bump b;
    const size_t o_off = b.take(sizeof(int32_t) * (size_t)n_requests), o_base = b.take(sizeof(int32_t) * (size_t)n_requests);
    const size_t o_req = b.take(d_out_request_of_token ? 0 : sizeof(uint32_t) * (size_t)T);
    Workspace *w = nullptr;
    DMOE_TRY(workspace_reserve(ws, b.off, &w));
    // request descriptors are tiny: staged through a pageable copy that is complete when the call returns
    std::vector<int32_t> offs((size_t)n_requests);
    int32_t run = 0;
    for (int i = 0; i < n_requests; ++i) {
        offs[(size_t)i] = run;
        run += h_seq_lens[i];
    }
    DMOE_HIP(hipMemcpyAsync(at<int32_t>(w, o_off), offs.data(), sizeof(int32_t) * (size_t)n_requests, hipMemcpyHostToDevice, st));
    DMOE_HIP(hipMemcpyAsync(at<int32_t>(w, o_base), h_base_pos, sizeof(int32_t) * (size_t)n_requests, hipMemcpyHostToDevice, st));
    if (d_out_tokens) {
        DMOE_REQUIRE(h_tokens != nullptr, "batch_build: token output requested without tokens");
        DMOE_HIP(hipMemcpyAsync(d_out_tokens, h_tokens, sizeof(uint32_t) * (size_t)T, hipMemcpyHostToDevice, st));
    }
    DMOE_HIP(hipStreamSynchronize(st)); // the host arrays (ours and the caller's) may go away after the call
    uint32_t *req = d_out_request_of_token ? d_out_request_of_token : at<uint32_t>(w, o_req);
    hipLaunchKernelGGL(batch_positions_kernel, dim3((unsigned)ceil_div(T, 256)), dim3(256), 0, st, d_out_positions, req,
                       at<int32_t>(w, o_off), at<int32_t>(w, o_base), n_requests, T);
    DMOE_LAUNCH_CHECK();
    if (d_out_mask) {
        DMOE_REQUIRE(((uintptr_t)d_out_mask % 16) == 0, "batch_build: mask must be 16-byte aligned");
        dim3 grid((unsigned)ceil_div((T + 3) / 4, 256), (unsigned)T);
        hipLaunchKernelGGL(batch_mask_kernel, grid, dim3(256), 0, st, (float4 *)d_out_mask, req, T);
        DMOE_LAUNCH_CHECK();
    }
    return DMOE_OK;
}
