// DSV4Gate.forward in one entry point (deepseek_v4.zig:546-681): router matmul -> scoring function -> selection.
//
//   logits = (x @ Wg^T) in bf16, widened to f32 (:556-565)
//   scores = softmax | sigmoid | sqrt(log(1 + exp(.))) (:567-585)
//   selection, weights, renormalisation, route scale: route.hip (dmoe_gate_route, :589-678)
//
// The selected expert ids must not depend on which machine computed the scores, so this file fixes the
// arithmetic that the reference leaves to MLX: the order of the f32 additions in the matmul and the evaluation
// of exp / log. The reduction dimension is cut into segments of 128 elements, each summed left to right from 0
// with one fma per element (a bf16 x bf16 product is exact in f32), and the segment sums are added left to
// right; exp and log are explicit polynomials over IEEE operations. A CPU that follows the same description
// gets the same bits.
//
// Layout: Wg is re-ordered once at creation into [D/8][E] 16-byte pieces, so that a wavefront whose lanes are
// 64 consecutive experts reads 1 KiB contiguous per 8 reduction elements. The activations of the workgroup's
// 8 tokens are the same for all lanes: each segment is widened to f32 into LDS and read back as broadcasts. Work per wavefront: 8 tokens x 64 experts
// x one segment (few tokens: the segment sums go to scratch and are added by the scoring kernel, which gives
// the launch enough wavefronts) or x all segments (many tokens). It is plain fp32 FMA work on the vector ALU:
// 2 T D E flop, 0.07 ms for 8192 tokens at the 137 TFLOP/s fp32 rate, small against the expert GEMMs.
#include <algorithm>
#include <new>

#include "common.h"
#include "route_device.h"

namespace dmoe {

constexpr int kGateSeg = 128;   // reduction elements per partial sum
constexpr int kGateTokens = 8;  // tokens per wavefront
constexpr int kGateTokensFew = 2; // ... for batches of at most kGateFewTokens tokens: four times the wavefronts, each a quarter as long
constexpr int kGateFewTokens = 256;
constexpr int kGateWaves = 4;
#ifndef DMOE_GATE_MFMA_MIN_TILES
#define DMOE_GATE_MFMA_MIN_TILES 640
#endif
constexpr size_t kGateMfmaMinTiles = DMOE_GATE_MFMA_MIN_TILES; // 32 x 32 output tiles from which the matrix-core kernel is the faster one

struct Gate {
    int device = 0;
    int E = 0, D = 0, K = 0, scoring = 0;
    float route_scale = 1.0f;
    uint16_t *wgp = nullptr; // [D/8][E][8] bf16
    float *bias = nullptr;   // [E] or null
    uint8_t *mask = nullptr; // [E] or null (1 = resident)
    int32_t *tid2eid = nullptr; // [vocab, K] or null: hash routing table
    int vocab = 0;
};

__global__ void gate_repack_kernel(uint4 *__restrict__ dst, const uint16_t *__restrict__ src, int E, int D) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; // (k8, e)
    const size_t n = (size_t)(D / 8) * E;
    if (i >= n) return;
    const int e = (int)(i % E), k8 = (int)(i / E);
    dst[i] = *(const uint4 *)(src + (size_t)e * D + (size_t)k8 * 8);
}

// partial[(t * n_out_seg + s) * E + e]: SPLIT -> a workgroup takes `segs_per_wave` consecutive segments (grid.z =
// group of segments) and stores every segment sum, n_out_seg = n_seg; otherwise it walks all segments and stores
// their left-to-right sum, n_out_seg = 1.
template <bool SPLIT, int TOK>
__global__ __launch_bounds__(kGateWaves * 64) void gate_logits_kernel(float *__restrict__ partial,
                                                                      const uint16_t *__restrict__ x,
                                                                      const uint4 *__restrict__ wgp, int T, int D,
                                                                      int E, int n_seg, int segs_per_wave) {
    __shared__ __attribute__((aligned(16))) float xs[TOK][kGateSeg]; // the tokens' segment, widened to f32
    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int e = ((int)blockIdx.x * kGateWaves + wave) * 64 + lane;
    const int t0 = (int)blockIdx.y * TOK;
    const bool e_on = e < E;
    const int ec = e_on ? e : E - 1;
    const int seg0 = SPLIT ? (int)blockIdx.z * segs_per_wave : 0;
    const int seg1 = SPLIT ? (seg0 + segs_per_wave < n_seg ? seg0 + segs_per_wave : n_seg) : n_seg;
    // staging: thread -> (token tid / 32, four elements at (tid % 32) * 4); surplus tokens repeat the last one
    const int st_tok = tid >> 5, st_k = (tid & 31) * 4;
    const uint16_t *st_src = x + (size_t)(t0 + st_tok < T ? t0 + st_tok : T - 1) * D;
    float total[TOK];
#pragma unroll
    for (int i = 0; i < TOK; ++i) total[i] = 0.0f;
    for (int seg = seg0; seg < seg1; ++seg) {
        const int k_begin = seg * kGateSeg, k_end = k_begin + kGateSeg < D ? k_begin + kGateSeg : D;
        // all weight pieces of the segment are requested before the first is used (one memory round trip per
        // segment instead of one per piece); pieces past a short last segment repeat the last one and are skipped
        constexpr int kPieces = kGateSeg / 8;
        uint4 wq[kPieces];
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
            const int k = k_begin + 8 * j < k_end ? k_begin + 8 * j : k_end - 8;
            wq[j] = wgp[(size_t)(k >> 3) * E + ec];
        }
        float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (st_tok < TOK && k_begin + st_k < k_end) { // D is a multiple of 8, so four elements are in or out together
            const uint2 v = *(const uint2 *)(st_src + k_begin + st_k);
            xv = make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                             __uint_as_float(v.y & 0xffff0000u));
        }
        __syncthreads(); // the previous segment has been consumed
        if (st_tok < TOK) *(float4 *)&xs[st_tok][st_k] = xv;
        __syncthreads();
        float part[TOK];
#pragma unroll
        for (int i = 0; i < TOK; ++i) part[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
            if (k_begin + 8 * j >= k_end) continue; // uniform
            float wf[8];
            wf[0] = __uint_as_float(wq[j].x << 16); wf[1] = __uint_as_float(wq[j].x & 0xffff0000u);
            wf[2] = __uint_as_float(wq[j].y << 16); wf[3] = __uint_as_float(wq[j].y & 0xffff0000u);
            wf[4] = __uint_as_float(wq[j].z << 16); wf[5] = __uint_as_float(wq[j].z & 0xffff0000u);
            wf[6] = __uint_as_float(wq[j].w << 16); wf[7] = __uint_as_float(wq[j].w & 0xffff0000u);
#pragma unroll
            for (int i = 0; i < TOK; ++i) {
                // every lane reads the same address: LDS broadcasts
                const float4 xa = *(const float4 *)&xs[i][8 * j], xb = *(const float4 *)&xs[i][8 * j + 4];
                part[i] = fmaf(xa.x, wf[0], part[i]);
                part[i] = fmaf(xa.y, wf[1], part[i]);
                part[i] = fmaf(xa.z, wf[2], part[i]);
                part[i] = fmaf(xa.w, wf[3], part[i]);
                part[i] = fmaf(xb.x, wf[4], part[i]);
                part[i] = fmaf(xb.y, wf[5], part[i]);
                part[i] = fmaf(xb.z, wf[6], part[i]);
                part[i] = fmaf(xb.w, wf[7], part[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < TOK; ++i) {
            if (SPLIT) {
                if (e_on && t0 + i < T) partial[((size_t)(t0 + i) * n_seg + seg) * E + e] = part[i];
            } else {
                total[i] = total[i] + part[i];
            }
        }
    }
    if (SPLIT || !e_on) return;
#pragma unroll
    for (int i = 0; i < TOK; ++i)
        if (t0 + i < T) partial[(size_t)(t0 + i) * E + e] = total[i];
}

// The same sums on the f32 matrix core, for batches large enough to fill it. v_mfma_f32_32x32x2_f32 adds its two
// products to the accumulator one after the other, each with one rounding: D = fma(a1, b1, fma(a0, b0, C)), bit for
// bit what two fmaf calls give (checked on the device against the C library over 20 480 outputs of 64-instruction
// chains, operands of both signs and of magnitudes six decades apart). A chain of these instructions over a
// segment's 128 elements, started from C = 0, is therefore the segment sum exactly as gate_logits_kernel and the CPU
// restatement form it, at twice the vector ALU's rate (the vector path has no packed fp32 here).
// Wavefront = 32 tokens x NB blocks of 32 experts, the whole reduction; lane (i = lane % 32, kk = lane / 32) feeds
// element kk of every pair of reduction elements for token i (A) and expert i of each block (B). Operands come
// straight from global memory, 16 bytes = 8 elements per lane and row, kGateMfmaAhead chunks ahead in registers
// (one wavefront per SIMD: nothing else hides the latency); both lane halves load the same 16 bytes and pick the
// even or the odd elements. No LDS, no barrier.
constexpr int kGateMfmaAhead = 4;
template <int NB>
__global__ __launch_bounds__(kGateWaves * 64) void gate_logits_mfma_kernel(float *__restrict__ logits,
                                                                           const uint16_t *__restrict__ x,
                                                                           const uint4 *__restrict__ wgp, int T, int D,
                                                                           int E) {
    const int tid = (int)threadIdx.x, lane = tid & 63, i = lane & 31, kk = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t0 = (int)blockIdx.y * 32;
    const int e0 = ((int)blockIdx.x * kGateWaves + wave) * 32 * NB;
    if (e0 >= E) return; // the whole wavefront is past the last expert
    const uint4 *const xrow = (const uint4 *)(x + (size_t)(t0 + i < T ? t0 + i : T - 1) * D);
    int ec[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) ec[b] = e0 + 32 * b + i < E ? e0 + 32 * b + i : E - 1;
    const int n_chunks = D >> 3;
    constexpr int CPS = kGateSeg / 8; // chunks per segment
    static_assert(CPS % kGateMfmaAhead == 0, "a segment is a whole number of turns of the ring");
    const uint32_t sh = kk ? 0u : 16u; // element kk of a dword: the low half moves up, the high half stays
    uint4 xr[kGateMfmaAhead], wr[kGateMfmaAhead][NB];
#pragma unroll
    for (int j = 0; j < kGateMfmaAhead; ++j) {
        const int c = j < n_chunks ? j : n_chunks - 1;
        xr[j] = xrow[c];
#pragma unroll
        for (int b = 0; b < NB; ++b) wr[j][b] = wgp[(size_t)c * E + ec[b]];
    }
    f32x16_t total[NB], part[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) total[b][r] = 0.0f;
    // the four pairs of one chunk: element kk of every dword
    auto pairs = [&](const uint4 &xv, const uint4 (&wv)[NB]) {
        const uint32_t xd[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const float a = __uint_as_float((xd[p] << sh) & 0xffff0000u);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t wd = p == 0 ? wv[b].x : p == 1 ? wv[b].y : p == 2 ? wv[b].z : wv[b].w;
                part[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, __uint_as_float((wd << sh) & 0xffff0000u), part[b], 0, 0, 0);
            }
        }
    };
    auto segment_done = [&]() {
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                total[b][r] = total[b][r] + part[b][r];
                part[b][r] = 0.0f;
            }
    };
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) part[b][r] = 0.0f;
    // Whole segments: straight-line code, the ring slot of every chunk known at compile time. The operands of chunk
    // c + 1 are widened to f32 between the matrix instructions of chunk c, into registers of their own (widening in
    // place, right in front of each matrix instruction, measured 5 % slower). What keeps the chain from the bare
    // instruction rate (28 ns per instruction measured, 150 TFLOP/s on the whole chip) are the load instructions: each
    // costs the wavefront about 30 ns of issue whatever the look-ahead (4, 8 or 16 chunks measure the same; without
    // the loads the kernel runs at the bare rate), which is why a wavefront takes two expert blocks per activation
    // chunk once there is work for more than two wavefronts per SIMD. Fetching a pair of chunks per load (one per lane
    // half, exchanged with v_permlane32_swap) halves the loads but costs the same again in swaps.
    const int n_whole = n_chunks / CPS;
    auto widen = [&](uint32_t d) { return __uint_as_float((d << sh) & 0xffff0000u); };
    float fa[4], fb[NB][4];
    {
        const uint32_t xd[4] = {xr[0].x, xr[0].y, xr[0].z, xr[0].w};
#pragma unroll
        for (int p = 0; p < 4; ++p) fa[p] = widen(xd[p]);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t wd[4] = {wr[0][b].x, wr[0][b].y, wr[0][b].z, wr[0][b].w};
#pragma unroll
            for (int p = 0; p < 4; ++p) fb[b][p] = widen(wd[p]);
        }
    }
    for (int seg = 0; seg < n_whole; ++seg) {
#pragma unroll
        for (int j = 0; j < CPS; ++j) {
            const int c = seg * CPS + j;
            constexpr int A = kGateMfmaAhead;
            const uint4 xn = xr[(j + 1) % A];
            const uint32_t xd[4] = {xn.x, xn.y, xn.z, xn.w};
            float na[4], nb[NB][4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
#pragma unroll
                for (int b = 0; b < NB; ++b) part[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[p], fb[b][p], part[b], 0, 0, 0);
                na[p] = widen(xd[p]);
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    const uint4 wn = wr[(j + 1) % A][b];
                    nb[b][p] = widen(p == 0 ? wn.x : p == 1 ? wn.y : p == 2 ? wn.z : wn.w);
                }
                __builtin_amdgcn_sched_barrier(0); // keeps the widening between the matrix instructions
            }
            // slot j % A was widened during the chunk before: request the chunk that will use it next (the barriers keep
            // the request HERE; left alone, the compiler sinks every load to just in front of its first use)
            const int cn = c + A < n_chunks ? c + A : n_chunks - 1; // the last ones are not used
            xr[j % A] = xrow[cn];
#pragma unroll
            for (int b = 0; b < NB; ++b) wr[j % A][b] = wgp[(size_t)cn * E + ec[b]];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                fa[p] = na[p];
#pragma unroll
                for (int b = 0; b < NB; ++b) fb[b][p] = nb[b][p];
            }
        }
        segment_done();
    }
    // a short last segment (D not a multiple of 128): its few chunks are fetched as they are used
    if (n_whole * CPS < n_chunks) {
        for (int c = n_whole * CPS; c < n_chunks; ++c) {
            const uint4 xv = xrow[c];
            uint4 wv[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) wv[b] = wgp[(size_t)c * E + ec[b]];
            pairs(xv, wv);
        }
        segment_done();
    }
    // accumulator r of lane (i, kk) is token 8 (r / 4) + 4 kk + r % 4, expert i of its block
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int e = e0 + 32 * b + i;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int t = t0 + 8 * (r >> 2) + 4 * kk + (r & 3);
            if (e < E && t < T) logits[(size_t)t * E + e] = total[b][r];
        }
    }
}

// exp(x) from IEEE operations only: Cody-Waite reduction by ln 2 in two parts, the degree-5 polynomial of the
// Cephes expf, scaling by two exact powers of two. Below -87: 0 (no denormal results); above 88.72: +inf.
__device__ __forceinline__ float det_expf(float x) {
    if (x != x) return x;
    if (x > 88.72283935546875f) return __uint_as_float(0x7f800000u);
    if (x < -87.0f) return 0.0f;
    const float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500E-4f;
    p = fmaf(p, r, 1.3981999507E-3f);
    p = fmaf(p, r, 8.3334519073E-3f);
    p = fmaf(p, r, 4.1665795894E-2f);
    p = fmaf(p, r, 1.6666665459E-1f);
    p = fmaf(p, r, 5.0000001201E-1f);
    float y = fmaf(p, r * r, r) + 1.0f;
    const int ni = (int)n, k1 = ni / 2, k2 = ni - k1;
    y = y * __uint_as_float((uint32_t)(k1 + 127) << 23);
    return y * __uint_as_float((uint32_t)(k2 + 127) << 23);
}

// log(x) for normal x > 0 (the Cephes logf); +inf -> +inf, 0 -> -inf, negative or NaN -> NaN
__device__ __forceinline__ float det_logf(float x) {
    if (x != x || x < 0.0f) return __uint_as_float(0x7fc00000u);
    if (x == 0.0f) return __uint_as_float(0xff800000u);
    const uint32_t u = __float_as_uint(x);
    if (u == 0x7f800000u) return x;
    int e = (int)((u >> 23) & 0xffu) - 126;
    float m = __uint_as_float((u & 0x007fffffu) | 0x3f000000u);
    if (m < 0.707106781186547524f) {
        e -= 1;
        m = (m + m) - 1.0f;
    } else {
        m = m - 1.0f;
    }
    const float z = m * m;
    float y = 7.0376836292E-2f;
    y = fmaf(y, m, -1.1514610310E-1f);
    y = fmaf(y, m, 1.1676998740E-1f);
    y = fmaf(y, m, -1.2420140846E-1f);
    y = fmaf(y, m, 1.4249322787E-1f);
    y = fmaf(y, m, -1.6668057665E-1f);
    y = fmaf(y, m, 2.0000714765E-1f);
    y = fmaf(y, m, -2.4999993993E-1f);
    y = fmaf(y, m, 3.3333331174E-1f);
    y = (y * m) * z;
    const float fe = (float)e;
    y = fmaf(fe, -2.12194440e-4f, y);
    y = fmaf(-0.5f, z, y);
    const float r = m + y;
    return fmaf(fe, 0.693359375f, r);
}

// softplus(x) = max(x, 0) + log1p(exp(-|x|)): log1p(u) for u in [0, 1] as log(w) * (u / (w - 1)) with w = 1 + u
// rounded (the quotient undoes the rounding of w to first order), u itself where w rounds to 1. No overflow for large
// x, no loss of the small results for very negative x.
__device__ __forceinline__ float det_softplusf(float x) {
    const float u = det_expf(-fabsf(x));
    const float w = 1.0f + u;
    const float l = w == 1.0f ? u : det_logf(w) * (u / (w - 1.0f));
    return (x > 0.0f ? x : 0.0f) + l;
}

// One wavefront per token: adds the segment sums left to right, rounds the logit to bf16, applies the scoring
// function and, with ROUTE, goes straight on to the selection (bias, Smelt mask, top-k, weights from the unbiased
// scores, renormalisation, route scale: deepseek_v4.zig:589-678) with the scores still in registers, so they make no
// round trip through memory; `scores` is written only when the caller wants them. Lane l owns experts l, l + 64, ...
// (EPL of them). Softmax: the sum is taken as one partial per lane (its experts in increasing order), folded by
// halves (lane i += lane i + 32, 16, .. 1).
template <int EPL, bool ROUTE, bool SPLIT>
__global__ __launch_bounds__(kGateWaves * 64) void gate_scores_kernel(float *__restrict__ scores,
                                                                      const float *__restrict__ partial, int T,
                                                                      int E, int n_seg, int scoring,
                                                                      uint32_t *__restrict__ out_idx,
                                                                      float *__restrict__ out_w,
                                                                      const float *__restrict__ bias,
                                                                      const uint8_t *__restrict__ resident, int K,
                                                                      int normalize, float route_scale) {
    const int lane = (int)threadIdx.x & 63;
    const int t = (int)blockIdx.x * kGateWaves + ((int)threadIdx.x >> 6);
    if (t >= T) return;
    float v[EPL];
    float mx = -__builtin_inff();
    // SPLIT (the matmul kernel stored every segment's sum): the segment sums of all of the lane's experts are requested
    // 64 at a time (one memory round trip per batch, not one per expert and eight segments) and added per expert in
    // segment order. Otherwise there is one sum per expert (n_seg == 1).
    constexpr int SB = SPLIT ? 64 / EPL : 1;
    const float *const p = partial + (size_t)t * n_seg * E;
#pragma unroll
    for (int i = 0; i < EPL; ++i) v[i] = 0.0f;
    for (int s0 = 0; s0 < n_seg; s0 += SB) {
        float q[EPL][SB];
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const int e = lane + 64 * i;
            const int ec = e < E ? e : E - 1;
#pragma unroll
            for (int j = 0; j < SB; ++j) q[i][j] = s0 + j < n_seg ? p[(size_t)(s0 + j) * E + ec] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < EPL; ++i)
#pragma unroll
            for (int j = 0; j < SB; ++j)
                if (s0 + j < n_seg) v[i] = v[i] + q[i][j];
    }
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int e = lane + 64 * i;
        if (e < E) {
            v[i] = bf16_bits_to_f32(f32_to_bf16_bits(v[i]));
            mx = v[i] > mx ? v[i] : mx;
        } else {
            v[i] = 0.0f;
        }
    }
    if (scoring == DMOE_SCORE_SOFTMAX) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float o = __shfl_xor(mx, off, 64);
            mx = o > mx ? o : mx;
        }
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < EPL; ++i)
            if (lane + 64 * i < E) {
                v[i] = det_expf(v[i] - mx);
                part = part + v[i];
            }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) part = part + __shfl_down(part, off, 64);
        const float sum = __shfl(part, 0, 64);
#pragma unroll
        for (int i = 0; i < EPL; ++i)
            if (lane + 64 * i < E) v[i] = v[i] / sum;
    } else {
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            if (lane + 64 * i >= E) continue;
            if (scoring == DMOE_SCORE_SIGMOID) v[i] = 1.0f / (1.0f + det_expf(-v[i]));
            else if (scoring == DMOE_SCORE_SQRTSOFTPLUS) v[i] = sqrtf(det_logf(1.0f + det_expf(v[i]))); // the reference's literal form (:575-583)
            else v[i] = sqrtf(det_softplusf(v[i]));
        }
    }
    if (scores) {
#pragma unroll
        for (int i = 0; i < EPL; ++i)
            if (lane + 64 * i < E) scores[(size_t)t * E + lane + 64 * i] = v[i];
    }
    if (ROUTE) {
        uint32_t my_idx;
        float w;
        route_from_registers<EPL>(v, bias, resident, E, K, normalize, 1, route_scale, lane, my_idx, w);
        if (lane < K) {
            out_idx[(size_t)t * K + lane] = my_idx;
            out_w[(size_t)t * K + lane] = w;
        }
    }
}

template <int EPL, bool ROUTE, typename... Args>
static void launch_scores(bool split, dim3 grid, dim3 block, hipStream_t st, Args... args) {
    if (split) hipLaunchKernelGGL((gate_scores_kernel<EPL, ROUTE, true>), grid, block, 0, st, args...);
    else hipLaunchKernelGGL((gate_scores_kernel<EPL, ROUTE, false>), grid, block, 0, st, args...);
}

// Hash routing (deepseek_v4.zig:619-636, then :655-678): the experts of a token come from a table indexed by its
// token id; the weights are the unbiased scores of those experts, divided by (their sum + 1e-20) unless the scoring
// function is softmax, times the route scale. One thread per token; the sum runs over k in increasing order.
__global__ void gate_hash_route_kernel(uint32_t *__restrict__ idx, float *__restrict__ w,
                                       const float *__restrict__ scores, const int32_t *__restrict__ tid2eid,
                                       const uint32_t *__restrict__ ids, int T, int E, int K, int vocab, int renorm,
                                       float route_scale) {
    const int t = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (t >= T) return;
    uint32_t id = ids[t];
    if (id >= (uint32_t)vocab) id = (uint32_t)vocab - 1; // ids are validated by the caller's contract; stay in bounds
    float sum = 0.0f;
    for (int j = 0; j < K; ++j) {
        int e = tid2eid[(size_t)id * K + j];
        e = e < 0 ? 0 : (e >= E ? E - 1 : e);
        const float s = scores[(size_t)t * E + e];
        idx[(size_t)t * K + j] = (uint32_t)e;
        w[(size_t)t * K + j] = s;
        sum = sum + s;
    }
    const float denom = sum + 1e-20f;
    for (int j = 0; j < K; ++j) {
        float v = w[(size_t)t * K + j];
        if (renorm) v = v / denom;
        w[(size_t)t * K + j] = v * route_scale;
    }
}

} // namespace dmoe

using namespace dmoe;

extern "C" {

int dmoe_gate_create(dmoe_gate *out, const dmoe_gate_desc *d, dmoe_stream s) {
    DMOE_REQUIRE(out && d, "gate_create: null argument");
    out->ctx = nullptr;
    DMOE_REQUIRE(d->weight != nullptr, "gate_create: weight is null");
    DMOE_REQUIRE(d->n_experts >= 1 && d->n_experts <= 1024 && d->top_k >= 1 && d->top_k <= d->n_experts,
                 "gate_create: bad expert count %d / top_k %d", d->n_experts, d->top_k);
    DMOE_REQUIRE(d->dim >= 8 && d->dim % 8 == 0, "gate_create: dim %d must be a positive multiple of 8", d->dim);
    DMOE_REQUIRE(d->scoring_func >= DMOE_SCORE_SOFTMAX && d->scoring_func <= DMOE_SCORE_SQRTSOFTPLUS_STABLE,
                 "gate_create: unknown scoring function %d", d->scoring_func);
    DMOE_REQUIRE(d->weight_source == DMOE_WEIGHTS_COPY_FROM_HOST || d->weight_source == DMOE_WEIGHTS_COPY_FROM_DEVICE,
                 "gate_create: weight_source must be a copying one (the weight is re-ordered)");
    DMOE_REQUIRE(!d->is_hash || (d->tid2eid != nullptr && d->vocab_size >= 1),
                 "gate_create: a hash gate needs tid2eid [vocab_size, top_k]");
    Gate *G = new (std::nothrow) Gate();
    DMOE_REQUIRE(G != nullptr, "gate_create: out of host memory");
    hipStream_t st = to_hip(s);
    const hipMemcpyKind kind = d->weight_source == DMOE_WEIGHTS_COPY_FROM_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
    const size_t wbytes = (size_t)d->n_experts * d->dim * 2;
    uint16_t *staging = nullptr;
    int rc = DMOE_OK;
    do {
        hipError_t e = hipGetDevice(&G->device);
        if (e != hipSuccess) { rc = hip_fail(e, "hipGetDevice"); break; }
        G->E = d->n_experts; G->D = d->dim; G->K = d->top_k; G->scoring = d->scoring_func; G->route_scale = d->route_scale;
        if ((e = hipMalloc((void **)&staging, wbytes)) != hipSuccess) { rc = hip_fail(e, "gate weight staging"); break; }
        if ((e = hipMalloc((void **)&G->wgp, wbytes)) != hipSuccess) { rc = hip_fail(e, "gate weight"); break; }
        if ((e = hipMemcpyAsync(staging, d->weight, wbytes, kind, st)) != hipSuccess) { rc = hip_fail(e, "gate weight upload"); break; }
        const size_t n = (size_t)(G->D / 8) * G->E;
        hipLaunchKernelGGL(gate_repack_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (uint4 *)G->wgp, staging, G->E, G->D);
        if ((e = hipGetLastError()) != hipSuccess) { rc = hip_fail(e, "gate repack"); break; }
        if (d->bias) {
            if ((e = hipMalloc((void **)&G->bias, sizeof(float) * (size_t)G->E)) != hipSuccess) { rc = hip_fail(e, "gate bias"); break; }
            if ((e = hipMemcpyAsync(G->bias, d->bias, sizeof(float) * (size_t)G->E, kind, st)) != hipSuccess) { rc = hip_fail(e, "gate bias upload"); break; }
        }
        if (d->resident_mask) {
            if ((e = hipMalloc((void **)&G->mask, (size_t)G->E)) != hipSuccess) { rc = hip_fail(e, "gate mask"); break; }
            if ((e = hipMemcpyAsync(G->mask, d->resident_mask, (size_t)G->E, kind, st)) != hipSuccess) { rc = hip_fail(e, "gate mask upload"); break; }
        }
        if (d->is_hash) {
            const size_t tb = sizeof(int32_t) * (size_t)d->vocab_size * G->K;
            G->vocab = d->vocab_size;
            if ((e = hipMalloc((void **)&G->tid2eid, tb)) != hipSuccess) { rc = hip_fail(e, "gate tid2eid"); break; }
            if ((e = hipMemcpyAsync(G->tid2eid, d->tid2eid, tb, kind, st)) != hipSuccess) { rc = hip_fail(e, "gate tid2eid upload"); break; }
        }
        // host sources may be pageable and may be released by the caller right after this call
        if ((e = hipStreamSynchronize(st)) != hipSuccess) { rc = hip_fail(e, "gate_create sync"); break; }
    } while (0);
    if (staging) (void)hipFree(staging);
    if (rc != DMOE_OK) {
        if (G->wgp) (void)hipFree(G->wgp);
        if (G->bias) (void)hipFree(G->bias);
        if (G->mask) (void)hipFree(G->mask);
        if (G->tid2eid) (void)hipFree(G->tid2eid);
        delete G;
        return rc;
    }
    out->ctx = G;
    return DMOE_OK;
}

int dmoe_gate_destroy(dmoe_gate gate) {
    Gate *G = (Gate *)gate.ctx;
    if (!G) return DMOE_OK;
    if (G->wgp) (void)hipFree(G->wgp);
    if (G->bias) (void)hipFree(G->bias);
    if (G->mask) (void)hipFree(G->mask);
    if (G->tid2eid) (void)hipFree(G->tid2eid);
    delete G;
    return DMOE_OK;
}

int dmoe_gate_forward(uint32_t *d_out_indices, float *d_out_weights, float *d_out_scores, dmoe_gate gate,
                      const uint16_t *d_x, const uint32_t *d_input_ids, int T, dmoe_workspace ws, dmoe_stream s) {
    Gate *G = (Gate *)gate.ctx;
    DMOE_REQUIRE(G != nullptr, "gate_forward: null gate");
    DMOE_REQUIRE(T >= 0, "gate_forward: T=%d", T);
    if (T == 0) return DMOE_OK;
    DMOE_REQUIRE(d_out_indices && d_out_weights && d_x, "gate_forward: null pointer");
    DMOE_REQUIRE(((uintptr_t)d_x % 16) == 0, "gate_forward: x must be 16-byte aligned");
    hipStream_t st = to_hip(s);
    const int n_seg = ceil_div(G->D, kGateSeg);
    // Few tokens: the segments are spread over several wavefronts so that the launch has about four wavefronts per
    // SIMD; the segment sums then travel through scratch (T * E * n_seg floats) to the scoring kernel.
    const int tok = T <= kGateFewTokens ? kGateTokensFew : kGateTokens;
    const size_t waves_whole = (size_t)ceil_div(T, tok) * ceil_div(G->E, 64);
    int groups = (int)std::min<size_t>((size_t)n_seg, (4096 + waves_whole - 1) / waves_whole);
    const int segs_per_wave = ceil_div(n_seg, groups);
    groups = ceil_div(n_seg, segs_per_wave);
    // enough 32-token x 32-expert tiles for one wavefront on most SIMDs of the chip: the matrix-core kernel (whole
    // sums); two tiles per wavefront once there are more than two wavefronts per SIMD
    const size_t mfma_tiles = (size_t)ceil_div(T, 32) * ceil_div(G->E, 32);
    const bool mfma = mfma_tiles >= kGateMfmaMinTiles;
    const int mfma_nb = mfma_tiles > 2048 ? 2 : 1;
    const bool split = groups > 1 && !mfma;
    const int n_out_seg = split ? n_seg : 1;
    Bump b;
    const size_t o_part = b.take(sizeof(float) * (size_t)T * G->E * n_out_seg);
    const bool hash = G->tid2eid && d_input_ids; // only the table lookup reads the scores back from memory
    const size_t o_scores = b.take(d_out_scores || !hash ? 0 : sizeof(float) * (size_t)T * G->E);
    Workspace *w = nullptr;
    DMOE_TRY(workspace_reserve(ws, b.off, &w));
    float *partial = at<float>(w, o_part);
    float *scores = d_out_scores ? d_out_scores : at<float>(w, o_scores);
    dim3 block(kGateWaves * 64);
    dim3 grid((unsigned)ceil_div(G->E, kGateWaves * 64), (unsigned)ceil_div(T, tok), (unsigned)groups);
    DMOE_REQUIRE(grid.y <= 65535u, "gate_forward: too many tokens for one launch (T=%d)", T);
    if (mfma) {
        const dim3 mgrid((unsigned)ceil_div(G->E, kGateWaves * 32 * mfma_nb), (unsigned)ceil_div(T, 32));
        if (mfma_nb == 2) hipLaunchKernelGGL(gate_logits_mfma_kernel<2>, mgrid, block, 0, st, partial, d_x, (const uint4 *)G->wgp, T, G->D, G->E);
        else hipLaunchKernelGGL(gate_logits_mfma_kernel<1>, mgrid, block, 0, st, partial, d_x, (const uint4 *)G->wgp, T, G->D, G->E);
    } else if (split && tok == kGateTokensFew)
        hipLaunchKernelGGL((gate_logits_kernel<true, kGateTokensFew>), grid, block, 0, st, partial, d_x, (const uint4 *)G->wgp, T, G->D, G->E, n_seg, segs_per_wave);
    else if (split)
        hipLaunchKernelGGL((gate_logits_kernel<true, kGateTokens>), grid, block, 0, st, partial, d_x, (const uint4 *)G->wgp, T, G->D, G->E, n_seg, segs_per_wave);
    else if (tok == kGateTokensFew)
        hipLaunchKernelGGL((gate_logits_kernel<false, kGateTokensFew>), grid, block, 0, st, partial, d_x, (const uint4 *)G->wgp, T, G->D, G->E, n_seg, segs_per_wave);
    else
        hipLaunchKernelGGL((gate_logits_kernel<false, kGateTokens>), grid, block, 0, st, partial, d_x, (const uint4 *)G->wgp, T, G->D, G->E, n_seg, segs_per_wave);
    DMOE_LAUNCH_CHECK();
    // the reference renormalises for every scoring function except softmax (:663)
    const int normalize = G->scoring != DMOE_SCORE_SOFTMAX ? 1 : 0;
    const dim3 sgrid((unsigned)ceil_div(T, kGateWaves));
    if (hash) { // hash layer with token ids: the table replaces the top-k (:619-636)
        if (G->E <= 256)
            launch_scores<4, false>(split, sgrid, block, st, scores, partial, T, G->E, n_out_seg, G->scoring, nullptr, nullptr,
                                    nullptr, nullptr, 0, 0, 1.0f);
        else
            launch_scores<16, false>(split, sgrid, block, st, scores, partial, T, G->E, n_out_seg, G->scoring, nullptr, nullptr,
                                     nullptr, nullptr, 0, 0, 1.0f);
        DMOE_LAUNCH_CHECK();
        hipLaunchKernelGGL(gate_hash_route_kernel, dim3((unsigned)ceil_div(T, 256)), dim3(256), 0, st, d_out_indices,
                           d_out_weights, scores, G->tid2eid, d_input_ids, T, G->E, G->K, G->vocab, normalize, G->route_scale);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    // scoring and selection in one launch; the scores leave the registers only if the caller asked for them
    DMOE_REQUIRE(G->K >= 1 && G->K <= G->E && G->K <= 64, "gate_forward: K=%d must satisfy 1 <= K <= min(E,64)", G->K);
    if (G->E <= 256)
        launch_scores<4, true>(split, sgrid, block, st, d_out_scores, partial, T, G->E, n_out_seg, G->scoring, d_out_indices,
                               d_out_weights, G->bias, G->mask, G->K, normalize, G->route_scale);
    else
        launch_scores<16, true>(split, sgrid, block, st, d_out_scores, partial, T, G->E, n_out_seg, G->scoring, d_out_indices,
                                d_out_weights, G->bias, G->mask, G->K, normalize, G->route_scale);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

} // extern "C"
