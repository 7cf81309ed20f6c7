// Grouped GEMM over UNQUANTIZED bf16 expert weights: the float arm of dispatchGatherMm (deepseek_v4.zig:969-979,
// ops.gatherMm) and of DSV4Expert.expertMatmul, for models whose experts were never quantized (the reference's own
// DSV4 smoke tests run this arm). Same tile list, same roles and same epilogue as the quantized kernels, so a layer
// of bf16 experts takes the same route -> pack -> gate/up -> down -> combine steps.
//
// One workgroup (4 wavefronts) = one tile of up to 128 rows of ONE expert segment against a strip of output columns;
// every wavefront owns 64 weight rows (gate_up: 32 gate + 32 up rows of the same 32 output columns) and feeds them as
// the A operand of v_mfma_f32_32x32x16_bf16 straight from global memory: lane (n = lane % 32, h = lane / 32) loads
// the 8 consecutive bf16 of weight row n at reduction offset 16 s + 8 h, exactly what its operand slots need. In the
// resident (re-ordered) layout the 64 lanes' 16-byte pieces of one step are contiguous, so a step is one linear
// 1 KiB read per wavefront. Activation rows are read the same way as the B operand (lane = token row); they are
// shared by the strips of a tile through the caches only. Two workgroups share a compute unit (the kernel stays under
// 256 registers), which is worth 30 % on an 8k-token prefill. Nothing here is tuned beyond that: the quantized formats
// are the hot path, this kernel is the correct and reasonably coalesced counterpart for float checkpoints.
#include "common.h"

namespace dmoe {

constexpr int kBf16Waves = 4;

template <bool GATE_UP, bool PACKED, int MT>
__device__ __forceinline__ void bf16_tile(const GemmArgs &g, const Tile &t) {
    constexpr int NT = 2;
    const int tid = (int)threadIdx.x, lane = tid & 63, ln = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cols = g.b0.cols, n_out = g.b0.rows;
    const int n_steps = (cols + 15) >> 4;
    const size_t e = t.expert;
    const int col_base = ((int)blockIdx.x * kBf16Waves + wave) * (GATE_UP ? 32 : 64);
    if (col_base >= n_out) return; // uniform over the wavefront; the kernel has no barriers

    const uint8_t *wp[NT];
    size_t wstep;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
        const int base = GATE_UP ? col_base : col_base + 32 * nt;
        const bool on = base < n_out;
        int n = base + ln;
        if (n >= n_out) n = n_out - 1; // keeps addresses valid; such rows are never stored
        if (PACKED) // piece ((nb * n_steps + s) * 2 + h) * 32 + ln of 16 bytes; rows are a multiple of 32 here
            wp[nt] = b.w + e * b.w_mat + ((((size_t)((on ? base : 0) >> 5) * n_steps) * 2 + h) * 32 + ln) * 16;
        else
            wp[nt] = b.w + e * b.w_mat + (size_t)n * b.w_row + (size_t)h * 16;
    }
    wstep = PACKED ? 1024 : 32;

    const uint8_t *xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int rl = mt * 32 + ln;
        if (rl >= (int)t.nrows) rl = (int)t.nrows - 1; // a valid row; its results are not stored
        const uint32_t p = t.row0 + (uint32_t)rl;
        const size_t src = g.a_rows ? g.a_rows[p] : p;
        xp[mt] = (const uint8_t *)g.a + (src * (size_t)cols + (size_t)h * 8) * 2;
    }

    f32x16_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

    auto step = [&](int s, bool live) {
        uint4 a[NT], x[MT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            a[nt] = live ? *(const uint4 *)(wp[nt] + (size_t)s * wstep) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            x[mt] = live ? *(const uint4 *)(xp[mt] + (size_t)s * 32) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[nt]),
                                                                      __builtin_bit_cast(bf16x8_t, x[mt]), acc[mt][nt],
                                                                      0, 0, 0);
    };
    const int full = cols >> 4; // whole steps of 16
    int s = 0;
    for (; s + 4 <= full; s += 4) {
#pragma unroll
        for (int u = 0; u < 4; ++u) step(s + u, true);
    }
    for (; s < full; ++s) step(s, true);
    // a reduction length that is a multiple of 8 but not of 16 leaves the upper half of a last step empty
    if (full < n_steps) step(full, h == 0);

    // ---- epilogue: lane = token row (ln), register r -> output column 8 * (r / 4) + 4 * h + r % 4 ----------------
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int rl = mt * 32 + ln;
        if (rl >= (int)t.nrows) continue;
        const uint32_t p = t.row0 + (uint32_t)rl;
        const size_t dst = g.out_rows ? g.out_rows[p] : p;
        float rscale = 1.0f;
        if (g.row_scale && p < g.row_scale_rows) rscale = g.row_scale[g.row_scale_idx ? g.row_scale_idx[p] : p];
        uint16_t *orow = g.out + dst * (size_t)g.ldo;
        const float limit = (t.flags & kTileDense) ? g.swiglu_limit_dense : g.swiglu_limit;
        if (GATE_UP) {
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const int n0 = col_base + 8 * rg + 4 * h;
                if (n0 >= n_out) continue;
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    v[i] = limited_swiglu(acc[mt][0][4 * rg + i], acc[mt][1][4 * rg + i], limit) * rscale;
                *(uint2 *)(orow + n0) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int rg = 0; rg < 4; ++rg) {
                    const int n0 = col_base + 32 * nt + 8 * rg + 4 * h;
                    if (n0 >= n_out) continue;
                    float v[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = acc[mt][nt][4 * rg + i] * rscale;
                    *(uint2 *)(orow + n0) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                }
        }
    }
}

template <bool GATE_UP, bool PACKED>
__global__ __launch_bounds__(kBf16Waves * 64, 2) void gemm_bf16_kernel(GemmArgs g) {
    Tile t;
    const uint32_t slot = blockIdx.y;
    if (g.tiles) {
        const uint32_t n_tiles = *g.n_tiles;
        if (slot >= n_tiles) return;
        t = g.tiles[slot];
        if ((int)t.nrows < g.min_rows || (int)t.nrows > g.max_rows || t.nrows == 0) return;
    } else {
        t.expert = 0;
        t.flags = 0;
        t.row0 = slot * (uint32_t)g.tile_m;
        if ((int)t.row0 >= g.dense_rows) return;
        const uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)g.tile_m ? left : (uint32_t)g.tile_m;
    }
    switch (__builtin_amdgcn_readfirstlane((int)((t.nrows + 31u) >> 5))) {
    case 1: bf16_tile<GATE_UP, PACKED, 1>(g, t); break;
    case 2: bf16_tile<GATE_UP, PACKED, 2>(g, t); break;
    case 3:
    case 4: bf16_tile<GATE_UP, PACKED, 4>(g, t); break;
    default: break;
    }
}

bool gemm_bf16_supports(const QView &b) { return b.mode == DMOE_QUANT_NONE && b.cols % 8 == 0 && b.rows % 4 == 0; }

template <bool GATE_UP, bool PACKED>
static int launch_variant(const GemmArgs &g, hipStream_t st) {
    const int cols_per_block = kBf16Waves * (GATE_UP ? 32 : 64);
    dim3 grid((unsigned)ceil_div(g.b0.rows, cols_per_block), (unsigned)g.max_tiles), block(kBf16Waves * 64);
    hipLaunchKernelGGL((gemm_bf16_kernel<GATE_UP, PACKED>), grid, block, 0, st, g);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

int launch_gemm_bf16(const GemmArgs &g, hipStream_t st) {
    DMOE_REQUIRE(gemm_bf16_supports(g.b0), "bf16 GEMM: weights must be unquantized bf16 with rows %% 4 == 0 and cols %% 8 == 0 (rows=%d cols=%d)",
                 g.b0.rows, g.b0.cols);
    DMOE_REQUIRE(g.tile_m > 0 && g.tile_m <= kMfmaTileM, "bf16 GEMM: bad tile size %d", g.tile_m);
    DMOE_REQUIRE(g.max_tiles >= 0 && g.max_tiles <= 65535, "bf16 GEMM: %d tiles exceed the grid limit", g.max_tiles);
    DMOE_REQUIRE(g.a && g.out && g.ldo > 0 && g.ldo % 4 == 0 && ((uintptr_t)g.out % 8) == 0 && ((uintptr_t)g.a % 16) == 0,
                 "bf16 GEMM: bad output / activation pointer or pitch");
    DMOE_REQUIRE(((uintptr_t)g.b0.w % 16) == 0, "bf16 GEMM: weights must be 16-byte aligned");
    if (g.gate_up)
        DMOE_REQUIRE(g.b1.mode == DMOE_QUANT_NONE && g.b1.rows == g.b0.rows && g.b1.cols == g.b0.cols &&
                         g.b1.packed == g.b0.packed && ((uintptr_t)g.b1.w % 16) == 0,
                     "bf16 GEMM: gate and up projections differ in shape or layout");
    if (g.max_tiles == 0) return DMOE_OK;
    if (g.b0.packed) return g.gate_up ? launch_variant<true, true>(g, st) : launch_variant<false, true>(g, st);
    return g.gate_up ? launch_variant<true, false>(g, st) : launch_variant<false, false>(g, st);
}

} // namespace dmoe
