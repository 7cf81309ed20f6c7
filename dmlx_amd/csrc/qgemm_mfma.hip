// Grouped quantized GEMM, MFMA path (prefill): bf16 matrix-core tiles with in-register dequantization.
//
// One workgroup (4 wavefronts) computes a tile of up to 128 rows of ONE expert segment against a strip
// of output columns. The four wavefronts split the strip, so every packed weight chunk is read and
// dequantized by exactly one wavefront, straight from global memory into the A operand of
// v_mfma_f32_32x32x16_bf16: lane (n = lane % 32, h = lane / 32) loads the 16-byte chunk h of weight row
// n for the current reduction step, i.e. exactly the values its MFMA operand slots need. The
// activations of the tile's rows are shared by all wavefronts through LDS (double-buffered, padded
// rows) and feed the B operand, so the accumulators hold out^T: lane = token row, registers = 16 output
// columns in runs of four, which lets the epilogue store 8 bytes at a time.
//
// A reduction step covers 2 chunks (64 values for 4-bit formats, 32 for 8-bit ones). The order of the
// products inside a step is permuted identically for both operands, which a sum does not see.
#include "common.h"
#include "qformat.h"

namespace dmoe {

constexpr int kMfmaWaves = 4;
constexpr int kMT = kMfmaTileM / 32; // 32-row MFMA tiles per workgroup tile

template <typename Fmt, bool GATE_UP, bool PACKED>
__global__ __launch_bounds__(kMfmaWaves * 64) void qgemm_mfma_kernel(GemmArgs g) {
    using CS = ChunkStream<Fmt, PACKED>;
    constexpr int KV = Fmt::kVals;     // values per 16-byte chunk
    constexpr int KSUB = 2 * KV;       // reduction elements per step
    constexpr int NJ = KV / 8;         // MFMAs (K = 16) per step and tile
    constexpr int LDA = KSUB + 8;      // LDS row pitch in bf16 elements (+16 bytes: conflict-free b128 reads)
    constexpr int CH = KSUB / 8;       // 16-byte pieces per activation row and step
    constexpr int RP = 256 / CH;       // rows staged per pass
    constexpr int PASSES = kMfmaTileM / RP;
    constexpr int NT = 2;              // 32-column MFMA tiles per wavefront

    __shared__ __attribute__((aligned(16))) uint16_t As[2][kMfmaTileM][LDA];

    Tile t;
    const uint32_t slot = blockIdx.y;
    if (g.tiles) {
        if (slot >= *g.n_tiles) return;
        t = g.tiles[slot];
    } else {
        t.expert = 0;
        t.row0 = slot * (uint32_t)kMfmaTileM;
        if ((int)t.row0 >= g.dense_rows) return;
        uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)kMfmaTileM ? left : (uint32_t)kMfmaTileM;
    }
    const int tid = (int)threadIdx.x, wave = tid >> 6, lane = tid & 63, ln = lane & 31, h = lane >> 5;
    const int cols = g.b0.cols, n_out = g.b0.rows;
    const int n_sub = cols / KSUB;
    const int n_mt = ((int)t.nrows + 31) >> 5;
    const size_t e = t.expert;

    // ---- this wavefront's weight rows -------------------------------------------------------------------
    // gate_up: tile 0 = gate rows, tile 1 = up rows of the same 32 output columns; plain: 64 output columns
    const int col_base = GATE_UP ? ((int)blockIdx.x * kMfmaWaves + wave) * 32 : ((int)blockIdx.x * kMfmaWaves + wave) * 64;
    const bool wave_on = col_base < n_out;
    CS cs[NT];
    bool tile_on[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
        const int base = GATE_UP ? col_base : col_base + 32 * nt;
        tile_on[nt] = wave_on && base < n_out;
        int n = base + ln;
        if (n >= n_out) n = n_out - 1; // keep addresses valid; such rows are never stored
        cs[nt].init(b, e, (tile_on[nt] ? base : 0) >> 5, ln, h, n);
    }

    // ---- activation staging: thread -> (row within pass, 16-byte piece) ------------------------------
    const int a_piece = tid % CH, a_row = tid / CH;
    const uint16_t *a_src[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        int r = a_row + p * RP;
        if (r < (int)t.nrows) {
            uint32_t pr = t.row0 + (uint32_t)r;
            size_t src = g.a_rows ? g.a_rows[pr] : pr;
            a_src[p] = g.a + src * (size_t)cols + a_piece * 8;
        } else {
            a_src[p] = nullptr;
        }
    }

    f32x16_t acc[kMT][NT];
#pragma unroll
    for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

    uint4 a_reg[PASSES];
    uint4 b_raw[NT];
    uint32_t b_sb[NT][2];

    auto load_a = [&](int ss) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            a_reg[p] = a_src[p] ? *(const uint4 *)(a_src[p] + (size_t)ss * KSUB) : make_uint4(0, 0, 0, 0);
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) *(uint4 *)&As[buf][a_row + p * RP][a_piece * 8] = a_reg[p];
    };
    auto load_b = [&](int ss) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
            b_raw[nt] = cs[nt].load_chunk(ss); // rows of a switched-off tile alias valid memory and are never stored
            cs[nt].load_meta(b, ss, b_sb[nt]);
        }
    };

    load_a(0);
    load_b(0);
    store_a(0);
    __syncthreads();

    for (int ss = 0; ss < n_sub; ++ss) {
        const int cur = ss & 1;
        uint32_t wp[NT][KV / 2];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) Fmt::decode_fast(b_raw[nt], CS::meta(b_sb[nt]), wp[nt]);
        const bool more = ss + 1 < n_sub;
        if (more) {
            load_a(ss + 1);
            load_b(ss + 1);
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            bf16x8_t wf[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                uint4 q = make_uint4(wp[nt][4 * j], wp[nt][4 * j + 1], wp[nt][4 * j + 2], wp[nt][4 * j + 3]);
                wf[nt] = __builtin_bit_cast(bf16x8_t, q);
            }
#pragma unroll
            for (int mt = 0; mt < kMT; ++mt) {
                if (mt < n_mt) {
                    uint4 q = *(const uint4 *)&As[cur][mt * 32 + ln][h * KV + 8 * j];
                    bf16x8_t xf = __builtin_bit_cast(bf16x8_t, q);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[nt], xf, acc[mt][nt], 0, 0, 0);
                }
            }
        }
        if (more) store_a(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane = token row (ln), registers r -> output column 8*(r/4) + 4*h + r%4 -------------
    if (!wave_on) return;
#pragma unroll
    for (int mt = 0; mt < kMT; ++mt) {
        if (mt >= n_mt) break;
        const int rl = mt * 32 + ln;
        if (rl >= (int)t.nrows) continue;
        const uint32_t p = t.row0 + (uint32_t)rl;
        const size_t dst = g.out_rows ? g.out_rows[p] : p;
        float rscale = 1.0f;
        if (g.row_scale) rscale = g.row_scale[g.row_scale_idx ? g.row_scale_idx[p] : p];
        uint16_t *orow = g.out + dst * (size_t)g.ldo;
        if (GATE_UP) {
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const int n0 = col_base + 8 * rg + 4 * h;
                if (n0 >= n_out) continue;
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float gv = acc[mt][0][4 * rg + i], uv = acc[mt][1][4 * rg + i];
                    if (Fmt::kRowScale) {
                        gv *= *(const float *)(g.b0.scales + e * g.b0.s_mat + (size_t)(n0 + i) * g.b0.s_row);
                        uv *= *(const float *)(g.b1.scales + e * g.b1.s_mat + (size_t)(n0 + i) * g.b1.s_row);
                    }
                    v[i] = limited_swiglu(gv, uv, g.swiglu_limit) * rscale;
                }
                *(uint2 *)(orow + n0) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int rg = 0; rg < 4; ++rg) {
                    const int n0 = col_base + 32 * nt + 8 * rg + 4 * h;
                    if (n0 >= n_out) continue;
                    float v[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        v[i] = acc[mt][nt][4 * rg + i];
                        if (Fmt::kRowScale)
                            v[i] *= *(const float *)(g.b0.scales + e * g.b0.s_mat + (size_t)(n0 + i) * g.b0.s_row);
                        v[i] *= rscale;
                    }
                    *(uint2 *)(orow + n0) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                }
            }
        }
    }
}

bool qgemm_mfma_supports(const QView &b) {
    int vals = (b.mode == DMOE_QUANT_AFFINE && b.bits == 4) || b.mode == DMOE_QUANT_MXFP4 ? 32 : 16;
    return b.cols % (2 * vals) == 0 && b.rows % 4 == 0;
}

struct MfmaLaunch {
    const GemmArgs &g;
    hipStream_t st;
    template <typename Fmt>
    int operator()() {
        const int cols_per_block = kMfmaWaves * (g.gate_up ? 32 : 64);
        dim3 grid((unsigned)ceil_div(g.b0.rows, cols_per_block), (unsigned)g.max_tiles), block(kMfmaWaves * 64);
        if (g.b0.packed) {
            if (g.gate_up) hipLaunchKernelGGL((qgemm_mfma_kernel<Fmt, true, true>), grid, block, 0, st, g);
            else hipLaunchKernelGGL((qgemm_mfma_kernel<Fmt, false, true>), grid, block, 0, st, g);
        } else {
            if (g.gate_up) hipLaunchKernelGGL((qgemm_mfma_kernel<Fmt, true, false>), grid, block, 0, st, g);
            else hipLaunchKernelGGL((qgemm_mfma_kernel<Fmt, false, false>), grid, block, 0, st, g);
        }
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
};

int launch_qgemm_mfma(const GemmArgs &g, hipStream_t st) {
    DMOE_REQUIRE(qgemm_mfma_supports(g.b0), "MFMA GEMM: unsupported weight shape (rows=%d cols=%d)", g.b0.rows,
                 g.b0.cols);
    DMOE_REQUIRE(g.max_tiles >= 0 && g.max_tiles <= 65535, "MFMA GEMM: %d tiles exceed the grid limit", g.max_tiles);
    DMOE_REQUIRE(g.a && g.out && g.ldo > 0 && g.ldo % 4 == 0 && ((uintptr_t)g.out % 8) == 0 &&
                     ((uintptr_t)g.a % 16) == 0,
                 "MFMA GEMM: bad output / activation pointer or pitch");
    if (g.gate_up)
        DMOE_REQUIRE(g.b1.rows == g.b0.rows && g.b1.cols == g.b0.cols && g.b1.mode == g.b0.mode &&
                         g.b1.bits == g.b0.bits && g.b1.group == g.b0.group && g.b1.packed == g.b0.packed,
                     "MFMA GEMM: gate and up projections differ in shape or format");
    if (g.max_tiles == 0) return DMOE_OK;
    return dispatch_format(g.b0, MfmaLaunch{g, st});
}

} // namespace dmoe
