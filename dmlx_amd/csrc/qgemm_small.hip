// Grouped quantized GEMM, small-M path (decode): at most kSmallTileM rows per expert tile.
//
// The step is bound by streaming every live expert's packed weights once from HBM, so the layout is
// built around the weight stream: one wavefront owns a run of output columns; for each column its 64
// lanes read one contiguous 1 KiB piece of the packed row (16 bytes per lane), so every lane always
// covers the SAME slice of the reduction dimension and keeps the matching activations of the tile's
// rows in registers for the whole kernel. Products are formed with packed-bf16 dot instructions, f32
// accumulation, and one cross-lane sum per output value.
//
// 4-bit affine weights are never multiplied out: codes are turned into the bf16 numbers (128 + q) with
// one AND-OR per pair, and   sum_k x_k (q_k s + b) = s * sum_k x_k (128 + q_k) + (b - 128 s) * sum_k x_k
// is applied once per 32-value chunk.
#include "common.h"
#include "qformat.h"

namespace dmoe {

constexpr int kSmallWaves = 4;
constexpr int kColsGateUp = 16; // output columns per wavefront (each needs a gate row and an up row)
constexpr int kColsPlain = 32;

template <typename Fmt>
struct SmallTraits {
    static constexpr bool kFactored = false;
    __device__ static __forceinline__ void unpack(const uint4 &raw, Meta m, uint32_t *pairs) {
        Fmt::decode(raw, m, pairs);
    }
    __device__ static __forceinline__ void arrange_x(uint32_t *) {}
};

template <>
struct SmallTraits<FmtAffine4> {
    static constexpr bool kFactored = true;
    // pairs (q_i, q_{i+4}) of each 8-code word as bf16 (128 + q)
    __device__ static __forceinline__ void unpack_word(uint32_t w, uint32_t *o) {
        o[0] = (w & 0x000f000fu) | 0x43004300u;
        o[1] = ((w >> 4) & 0x000f000fu) | 0x43004300u;
        o[2] = ((w >> 8) & 0x000f000fu) | 0x43004300u;
        o[3] = ((w >> 12) & 0x000f000fu) | 0x43004300u;
    }
    __device__ static __forceinline__ void unpack(const uint4 &raw, Meta, uint32_t *pairs) {
        unpack_word(raw.x, pairs);
        unpack_word(raw.y, pairs + 4);
        unpack_word(raw.z, pairs + 8);
        unpack_word(raw.w, pairs + 12);
    }
    // natural pairs (x0,x1)(x2,x3)(x4,x5)(x6,x7) -> (x0,x4)(x1,x5)(x2,x6)(x3,x7), per 8 values
    __device__ static __forceinline__ void arrange_x(uint32_t *x /*[16]*/) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            uint32_t a = x[4 * w], b = x[4 * w + 1], c = x[4 * w + 2], d = x[4 * w + 3];
            x[4 * w] = (a & 0xffffu) | (c << 16);
            x[4 * w + 1] = (a >> 16) | (c & 0xffff0000u);
            x[4 * w + 2] = (b & 0xffffu) | (d << 16);
            x[4 * w + 3] = (b >> 16) | (d & 0xffff0000u);
        }
    }
};

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c,
                                           false);
}

template <typename Fmt, int ITERS, int NM>
struct ColData {
    uint4 raw[NM][ITERS];
    Meta meta[NM][ITERS];
};

template <typename Fmt, int ITERS, bool GATE_UP, int M>
__device__ __forceinline__ void small_run(const GemmArgs &g, const Tile &t, int wave, int lane) {
    using ST = SmallTraits<Fmt>;
    constexpr int NP = Fmt::kVals / 2;       // packed pairs per chunk
    constexpr int KSTEP = 64 * Fmt::kVals;   // reduction elements one wavefront covers per iteration
    constexpr int NM = GATE_UP ? 2 : 1;
    constexpr int CPW = GATE_UP ? kColsGateUp : kColsPlain;
    const int cols = g.b0.cols;
    const int n_out = g.b0.rows;

    // ---- activations of the tile's rows, this lane's slices, kept in registers -------------------
    uint32_t xp[M][ITERS][NP];
    float xs[M][ITERS];
#pragma unroll
    for (int r = 0; r < M; ++r) {
        const uint32_t p = t.row0 + (uint32_t)r;
        const size_t src = g.a_rows ? g.a_rows[p] : p;
        const uint16_t *xrow = g.a + src * (size_t)cols;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int k0 = it * KSTEP + lane * Fmt::kVals;
            float sum = 0.0f;
#pragma unroll
            for (int v = 0; v < NP / 4; ++v) {
                uint4 q = make_uint4(0, 0, 0, 0);
                if (k0 < cols) q = *(const uint4 *)(xrow + k0 + 8 * v);
                xp[r][it][4 * v] = q.x;
                xp[r][it][4 * v + 1] = q.y;
                xp[r][it][4 * v + 2] = q.z;
                xp[r][it][4 * v + 3] = q.w;
            }
            if (ST::kFactored) {
#pragma unroll
                for (int i = 0; i < NP; ++i)
                    sum += bf16_bits_to_f32(xp[r][it][i] & 0xffffu) + bf16_bits_to_f32(xp[r][it][i] >> 16);
            }
            xs[r][it] = sum;
            ST::arrange_x(xp[r][it]);
        }
    }

    const size_t e = t.expert;
    const int n_base = ((int)blockIdx.x * kSmallWaves + wave) * CPW;

    auto load_col = [&](int n, ColData<Fmt, ITERS, NM> &c) {
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            const QView &b = mi == 0 ? g.b0 : g.b1;
            const uint8_t *wrow = b.w + e * b.w_mat + (size_t)n * b.w_row;
            const uint8_t *srow = b.scales + e * b.s_mat + (size_t)n * b.s_row;
            const uint8_t *brow = b.biases ? b.biases + e * b.s_mat + (size_t)n * b.s_row : nullptr;
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int k0 = it * KSTEP + lane * Fmt::kVals;
                if (k0 < cols) {
                    c.raw[mi][it] = *(const uint4 *)(wrow + (size_t)(it * 64 + lane) * 16);
                    c.meta[mi][it] = Fmt::load_meta(b, srow, brow, k0);
                } else {
                    c.raw[mi][it] = make_uint4(0, 0, 0, 0);
                    c.meta[mi][it].s = 0.0f;
                    c.meta[mi][it].b = 0.0f;
                }
            }
        }
    };

    auto compute_col = [&](int n, const ColData<Fmt, ITERS, NM> &c) {
        float acc[NM][M];
#pragma unroll
        for (int mi = 0; mi < NM; ++mi)
#pragma unroll
            for (int r = 0; r < M; ++r) acc[mi][r] = 0.0f;
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                uint32_t pairs[NP];
                ST::unpack(c.raw[mi][it], c.meta[mi][it], pairs);
                const float s = c.meta[mi][it].s;
                const float boff = fmaf(-128.0f, s, c.meta[mi][it].b);
#pragma unroll
                for (int r = 0; r < M; ++r) {
                    float p0 = 0.0f, p1 = 0.0f; // two chains for instruction-level parallelism
#pragma unroll
                    for (int i = 0; i < NP; i += 2) {
                        p0 = dot2_bf16(pairs[i], xp[r][it][i], p0);
                        p1 = dot2_bf16(pairs[i + 1], xp[r][it][i + 1], p1);
                    }
                    if (ST::kFactored) acc[mi][r] = fmaf(s, p0 + p1, fmaf(boff, xs[r][it], acc[mi][r]));
                    else acc[mi][r] += p0 + p1;
                }
            }
        }
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            float rs = 1.0f;
            if (Fmt::kRowScale) {
                const QView &b = mi == 0 ? g.b0 : g.b1;
                rs = *(const float *)(b.scales + e * b.s_mat + (size_t)n * b.s_row);
            }
#pragma unroll
            for (int r = 0; r < M; ++r) acc[mi][r] = wave_sum(acc[mi][r]) * rs;
        }
#pragma unroll
        for (int r = 0; r < M; ++r) {
            if (lane == r) {
                const uint32_t p = t.row0 + (uint32_t)r;
                float v = GATE_UP ? limited_swiglu(acc[0][r], acc[NM - 1][r], g.swiglu_limit) : acc[0][r];
                if (g.row_scale) v *= g.row_scale[g.row_scale_idx ? g.row_scale_idx[p] : p];
                const size_t dst = g.out_rows ? g.out_rows[p] : p;
                g.out[dst * (size_t)g.ldo + n] = f32_to_bf16_bits(v);
            }
        }
    };

    ColData<Fmt, ITERS, NM> cur, nxt;
    if (n_base < n_out) load_col(n_base, cur);
#pragma unroll 2
    for (int c = 0; c < CPW; ++c) {
        const int n = n_base + c;
        if (n >= n_out) break;
        const bool more = (c + 1 < CPW) && (n + 1 < n_out);
        if (more) load_col(n + 1, nxt);
        compute_col(n, cur);
        if (more) cur = nxt;
    }
}

template <typename Fmt, int ITERS, bool GATE_UP>
__global__ __launch_bounds__(kSmallWaves * 64) void qgemm_small_kernel(GemmArgs g) {
    Tile t;
    const uint32_t slot = blockIdx.y;
    if (g.tiles) {
        if (slot >= *g.n_tiles) return;
        t = g.tiles[slot];
    } else {
        t.expert = 0;
        t.row0 = slot * (uint32_t)kSmallTileM;
        if ((int)t.row0 >= g.dense_rows) return;
        uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)kSmallTileM ? left : (uint32_t)kSmallTileM;
        t.pad = 0;
    }
    const int wave = (int)(threadIdx.x >> 6), lane = lane_id();
    switch (t.nrows) {
    case 1: small_run<Fmt, ITERS, GATE_UP, 1>(g, t, wave, lane); break;
    case 2: small_run<Fmt, ITERS, GATE_UP, 2>(g, t, wave, lane); break;
    case 3: small_run<Fmt, ITERS, GATE_UP, 3>(g, t, wave, lane); break;
    case 4: small_run<Fmt, ITERS, GATE_UP, 4>(g, t, wave, lane); break;
    default: break;
    }
}

static int small_iters(const QView &b, int vals) { return ceil_div(b.cols, 64 * vals); }

bool qgemm_small_supports(const QView &b) {
    int vals = (b.mode == DMOE_QUANT_AFFINE && b.bits == 4) || b.mode == DMOE_QUANT_MXFP4 ? 32 : 16;
    int it = small_iters(b, vals);
    return b.cols % vals == 0 && (it == 1 || it == 2 || (vals == 16 && it <= 4));
}

struct SmallLaunch {
    const GemmArgs &g;
    hipStream_t st;
    template <typename Fmt, int ITERS>
    int go() {
        const int cpw = g.gate_up ? kColsGateUp : kColsPlain;
        dim3 grid((unsigned)ceil_div(g.b0.rows, kSmallWaves * cpw), (unsigned)g.max_tiles), block(kSmallWaves * 64);
        if (g.gate_up) hipLaunchKernelGGL((qgemm_small_kernel<Fmt, ITERS, true>), grid, block, 0, st, g);
        else hipLaunchKernelGGL((qgemm_small_kernel<Fmt, ITERS, false>), grid, block, 0, st, g);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    template <typename Fmt>
    int operator()() {
        int it = small_iters(g.b0, Fmt::kVals);
        if (it == 1) return go<Fmt, 1>();
        if (it == 2) return go<Fmt, 2>();
        if (Fmt::kVals == 16 && it <= 4) return go<Fmt, (Fmt::kVals == 16 ? 4 : 2)>();
        set_error("small-M GEMM: reduction length %d not supported", g.b0.cols);
        return DMOE_ERR_UNSUPPORTED;
    }
};

int launch_qgemm_small(const GemmArgs &g, hipStream_t st) {
    DMOE_REQUIRE(qgemm_small_supports(g.b0), "small-M GEMM: unsupported weight shape (cols=%d)", g.b0.cols);
    DMOE_REQUIRE(g.max_tiles >= 0 && g.max_tiles <= 65535, "small-M GEMM: %d tiles exceed the grid limit",
                 g.max_tiles);
    DMOE_REQUIRE(g.a && g.out && g.ldo > 0, "small-M GEMM: null pointer");
    DMOE_REQUIRE(g.b0.cols % 8 == 0 && ((uintptr_t)g.a % 16) == 0, "small-M GEMM: activations must be 16-byte aligned");
    if (g.gate_up)
        DMOE_REQUIRE(g.b1.rows == g.b0.rows && g.b1.cols == g.b0.cols && g.b1.mode == g.b0.mode &&
                         g.b1.bits == g.b0.bits && g.b1.group == g.b0.group,
                     "small-M GEMM: gate and up projections differ in shape or format");
    if (g.max_tiles == 0) return DMOE_OK;
    return dispatch_format(g.b0, SmallLaunch{g, st});
}

} // namespace dmoe
