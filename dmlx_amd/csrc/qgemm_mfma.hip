// Grouped quantized GEMM, MFMA path (prefill): bf16 matrix-core tiles with in-register dequantization.
//
// One workgroup (4 wavefronts) computes a tile of up to 128 rows of ONE expert segment against a strip
// of output columns. The four wavefronts split the strip, so every packed weight chunk is read and
// dequantized by exactly one wavefront, straight from global memory into the A operand of
// v_mfma_f32_32x32x16_bf16: lane (n = lane % 32, h = lane / 32) loads the 16-byte chunk h of weight row
// n for a reduction step, i.e. exactly the values its MFMA operand slots need. Those loads run through a
// register ring kMfmaRing steps deep. The activations of the tile's rows are shared by all wavefronts
// through LDS (double-buffered blocks of two steps, padded rows, one barrier per block) and feed the B
// operand, so the accumulators hold out^T: lane = token row, registers = 16 output columns in runs of
// four, which lets the epilogue store 8 bytes at a time.
//
// The loop is software-pipelined by hand: while the matrix core works through the 32 MFMAs of step s
// with the weights decoded during step s-1, the vector ALU decodes the weights of step s+1, so the two
// pipes overlap inside a single wavefront (the register budget leaves one wavefront per SIMD).
//
// A reduction step covers 2 chunks (64 values for 4-bit formats, 32 for 8-bit ones). The order of the
// products inside a step is permuted identically for both operands, which a sum does not see.
#include <type_traits>

#include "common.h"
#include "qformat.h"

namespace dmoe {

constexpr int kMfmaWaves = 4;
constexpr int kMfmaRing = 4;          // weight steps held in registers (kMfmaRing - 1 in flight)
constexpr int kStepsPerBlock = 2;     // reduction steps per LDS activation block

template <typename Fmt>
struct MfmaGeom {
    static constexpr int KV = Fmt::kVals;          // values per 16-byte chunk
    static constexpr int KSTEP = 2 * KV;           // reduction elements per step
    static constexpr int NJ = KV / 8;              // MFMAs (K = 16) per step and tile
    static constexpr int KB = kStepsPerBlock * KSTEP; // reduction elements per activation block
    static constexpr int LDA = KB + 8;             // LDS row pitch in bf16 elements (+16 bytes: conflict-free b128 reads)
    static constexpr int CH = KB / 8;              // 16-byte pieces per activation row and block
    static constexpr int RP = 256 / CH;            // rows staged per pass
    static constexpr int PASSES = kMfmaTileM / RP;
    static constexpr size_t kLdsBytes = 2ull * kMfmaTileM * LDA * 2;
};

// One tile with MT 32-row MFMA tiles (MT is a template parameter so that the reduction loop is straight-line
// code: the scheduler can then interleave the decode arithmetic with the matrix instructions).
template <typename Fmt, bool GATE_UP, bool PACKED, int MT>
__device__ __forceinline__ void mfma_tile(const GemmArgs &g, const Tile &t, uint16_t *mfma_lds) {
    using CS = ChunkStream<Fmt, PACKED>;
    using G = MfmaGeom<Fmt>;
    constexpr int KV = G::KV, KSTEP = G::KSTEP, NJ = G::NJ, KB = G::KB, LDA = G::LDA, CH = G::CH, RP = G::RP,
                  PASSES = G::PASSES;
    constexpr int NT = 2; // 32-column MFMA tiles per wavefront
    constexpr int n_mt = MT;
    const int tid = (int)threadIdx.x, lane = tid & 63, ln = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cols = g.b0.cols, n_out = g.b0.rows;
    const int n_steps = cols / KSTEP;
    const int n_blk = (n_steps + kStepsPerBlock - 1) / kStepsPerBlock;
    const size_t e = t.expert;

    // ---- this wavefront's weight rows -------------------------------------------------------------------
    // gate_up: tile 0 = gate rows, tile 1 = up rows of the same 32 output columns; plain: 64 output columns
    const int col_base = ((int)blockIdx.x * kMfmaWaves + wave) * (GATE_UP ? 32 : 64);
    const bool wave_on = col_base < n_out;
    CS cs[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
        const int base = GATE_UP ? col_base : col_base + 32 * nt;
        const bool on = wave_on && base < n_out;
        int n = base + ln;
        if (n >= n_out) n = n_out - 1; // keep addresses valid; such rows are never stored
        cs[nt].init(b, e, (on ? base : 0) >> 5, ln, h, n);
    }
    uint4 ring_raw[kMfmaRing][NT];
    uint32_t ring_sb[kMfmaRing][NT][2];
    auto load_b = [&](int step, int slot_) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
            ring_raw[slot_][nt] = cs[nt].load_chunk(step); // rows of a switched-off tile alias valid memory, never stored
            cs[nt].load_meta(b, step, ring_sb[slot_][nt]);
        }
    };
    // weight loads depend on the tile only: start them first
#pragma unroll
    for (int j = 0; j < kMfmaRing; ++j)
        if (j < n_steps) load_b(j, j);

    // ---- activation staging: thread -> (row within pass, 16-byte piece) ------------------------------
    const int a_piece = tid % CH, a_row = tid / CH;
    constexpr int rows_used = n_mt * 32;
    const uint16_t *a_src[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int r = a_row + p * RP;
        a_src[p] = nullptr;
        if (r < (int)t.nrows) {
            const uint32_t pr = t.row0 + (uint32_t)r;
            const size_t src = g.a_rows ? g.a_rows[pr] : pr;
            a_src[p] = g.a + src * (size_t)cols + a_piece * 8;
        }
    }
    uint4 a_reg[PASSES];
    auto load_a = [&](int blk) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            a_reg[p] = make_uint4(0, 0, 0, 0);
            // the last block may be half a block wide (n_steps odd): pieces past the row end stay zero
            if (a_src[p] && blk * KB + a_piece * 8 < cols) a_reg[p] = *(const uint4 *)(a_src[p] + (size_t)blk * KB);
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            if (p * RP < rows_used) // rows of MFMA tiles that are not computed are never read
                *(uint4 *)&mfma_lds[((size_t)buf * kMfmaTileM + a_row + p * RP) * LDA + a_piece * 8] = a_reg[p];
    };

    f32x16_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

    uint32_t wp[2][NT][KV / 2]; // decoded weights of the current / next step
    auto decode = [&](int slot_, int which) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) Fmt::decode_fast(ring_raw[slot_][nt], CS::meta(ring_sb[slot_][nt]), wp[which][nt]);
    };
    // One reduction step: the MT*NT*NJ matrix instructions of step s (weights wp[which], decoded one step
    // earlier) with the vector-ALU decode of step s+1 spread between them. Activation fragments are read
    // from LDS one MFMA group ahead. The scheduling-group barriers at the end pin that interleaving; left to
    // itself the compiler emits the whole decode first and the matrix instructions after it.
    auto step_body = [&](int slot_next, int which, int buf, int sb) {
        bf16x8_t xf[2][MT];
        auto read_x = [&](int j, int pp) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                uint4 q = *(const uint4 *)&mfma_lds[((size_t)buf * kMfmaTileM + mt * 32 + ln) * LDA + sb * KSTEP + h * KV + 8 * j];
                xf[pp][mt] = __builtin_bit_cast(bf16x8_t, q);
            }
        };
        read_x(0, 0);
        decode(slot_next, which ^ 1);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if (j + 1 < NJ) read_x(j + 1, (j + 1) & 1);
            bf16x8_t wf[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                uint4 q = make_uint4(wp[which][nt][4 * j], wp[which][nt][4 * j + 1], wp[which][nt][4 * j + 2],
                                     wp[which][nt][4 * j + 3]);
                wf[nt] = __builtin_bit_cast(bf16x8_t, q);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[nt], xf[j & 1][mt], acc[mt][nt], 0, 0, 0);
        }
        constexpr int kMfmas = NJ * MT * NT;
        constexpr int kValuPerMfma = (Fmt::kDecodeOps * NT + kMfmas - 1) / kMfmas;
        __builtin_amdgcn_sched_group_barrier(0x100, MT, 0); // LDS reads of the first group
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if (j + 1 < NJ) __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
#pragma unroll
            for (int k = 0; k < MT * NT; ++k) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);            // one matrix instruction
                __builtin_amdgcn_sched_group_barrier(0x002, kValuPerMfma, 0); // its share of the decode
            }
        }
    };

    load_a(0);
    store_a(0);
    __syncthreads();
    decode(0, 0);

    // kMfmaRing steps per trip so that ring slots, LDS buffers and the wp pair are compile-time indices. Full trips
    // run without any guard (loads past the end are clamped onto valid memory and their data is never used), so a
    // trip is straight-line code between barriers; a trailing partial trip runs the guarded copy.
    static_assert(kMfmaRing % (2 * kStepsPerBlock) == 0, "ring must cover whole pairs of activation blocks");
    auto trip = [&](int s0, auto guard) {
        constexpr bool GUARD = decltype(guard)::value;
#pragma unroll
        for (int j = 0; j < kMfmaRing; ++j) {
            const int s = s0 + j;
            if (!GUARD || s < n_steps) {
                const int blk = s / kStepsPerBlock;
                const int sb = j % kStepsPerBlock, buf = (j / kStepsPerBlock) & 1;
                const int s_ahead = s + kMfmaRing < n_steps ? s + kMfmaRing : n_steps - 1;
                load_b(s_ahead, j); // slot j was decoded one step ago
                if (sb == 0) load_a(blk + 1 < n_blk ? blk + 1 : n_blk - 1);
                step_body((j + 1) % kMfmaRing, j & 1, buf, sb);
                if (sb == kStepsPerBlock - 1 || (GUARD && s + 1 == n_steps)) {
                    store_a(buf ^ 1);
                    __syncthreads();
                }
            }
        }
    };
    int s0 = 0;
#pragma unroll 1
    for (; s0 + kMfmaRing <= n_steps; s0 += kMfmaRing) trip(s0, std::false_type{});
    if (s0 < n_steps) trip(s0, std::true_type{});

    // ---- epilogue: lane = token row (ln), registers r -> output column 8*(r/4) + 4*h + r%4 -------------
    if (!wave_on) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
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

template <typename Fmt, bool GATE_UP, bool PACKED>
__global__ __launch_bounds__(kMfmaWaves * 64) void qgemm_mfma_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint16_t mfma_lds[]; // As[2][kMfmaTileM][LDA]
    Tile t;
    const uint32_t slot = blockIdx.y;
    if (g.tiles) {
        const uint32_t n_tiles = *g.n_tiles;
        t = g.tiles[slot];
        if (slot >= n_tiles) return;
    } else {
        t.expert = 0;
        t.row0 = slot * (uint32_t)kMfmaTileM;
        if ((int)t.row0 >= g.dense_rows) return;
        uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)kMfmaTileM ? left : (uint32_t)kMfmaTileM;
    }
    switch ((t.nrows + 31u) >> 5) { // uniform over the workgroup
    case 1: mfma_tile<Fmt, GATE_UP, PACKED, 1>(g, t, mfma_lds); break;
    case 2: mfma_tile<Fmt, GATE_UP, PACKED, 2>(g, t, mfma_lds); break;
    case 3: mfma_tile<Fmt, GATE_UP, PACKED, 3>(g, t, mfma_lds); break;
    case 4: mfma_tile<Fmt, GATE_UP, PACKED, 4>(g, t, mfma_lds); break;
    default: break;
    }
}

bool qgemm_mfma_supports(const QView &b) {
    int vals = (b.mode == DMOE_QUANT_AFFINE && b.bits == 4) || b.mode == DMOE_QUANT_MXFP4 ? 32 : 16;
    return b.cols % (2 * vals) == 0 && b.rows % 4 == 0;
}

struct MfmaLaunch {
    const GemmArgs &g;
    hipStream_t st;
    template <typename Fmt, bool GATE_UP, bool PACKED>
    int go() {
        auto kern = qgemm_mfma_kernel<Fmt, GATE_UP, PACKED>;
        const size_t lds = MfmaGeom<Fmt>::kLdsBytes;
        static thread_local bool raised = false; // per instantiation: allow more than 64 KiB of dynamic LDS once
        if (!raised) {
            DMOE_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            raised = true;
        }
        const int cols_per_block = kMfmaWaves * (GATE_UP ? 32 : 64);
        dim3 grid((unsigned)ceil_div(g.b0.rows, cols_per_block), (unsigned)g.max_tiles), block(kMfmaWaves * 64);
        hipLaunchKernelGGL(kern, grid, block, lds, st, g);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    template <typename Fmt>
    int operator()() {
        if (g.b0.packed) return g.gate_up ? go<Fmt, true, true>() : go<Fmt, false, true>();
        return g.gate_up ? go<Fmt, true, false>() : go<Fmt, false, false>();
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
