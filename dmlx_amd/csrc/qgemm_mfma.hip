// Grouped quantized GEMM, MFMA path (prefill) for weights in the MLX layout: bf16 matrix-core tiles with in-register
// dequantization. (Stacks in the packed resident layout take the kernel in qgemm_wide.hip, which launch_qgemm_mfma
// forwards to.)
//
// One workgroup (4 wavefronts) computes a tile of up to 128 rows of ONE expert segment against a strip
// of output columns. The four wavefronts split the strip, so every packed weight chunk is read and
// dequantized by exactly one wavefront, straight from global memory into the A operand of
// v_mfma_f32_32x32x16_bf16: lane (n = lane % 32, h = lane / 32) loads the 16-byte chunk h of weight row
// n for a reduction step, i.e. exactly the values its MFMA operand slots need. Those loads run through a
// register ring kMfmaRing steps deep. The activations of the tile's rows are shared by all wavefronts
// through LDS (double-buffered blocks of kMfmaRing steps, padded rows, one barrier per block) and feed
// the B operand, so the accumulators hold out^T: lane = token row, registers = 16 output columns in runs
// of four, which lets the epilogue store 8 bytes at a time.
//
// The loop is software-pipelined by hand: while the matrix core works through the MFMAs of step s with
// the weights decoded during step s-1, the vector ALU decodes the weights of step s+1. A wavefront
// issues in order, so the two pipes only overlap if the instruction stream alternates between them:
// the step is written as units of [one MFMA | one slice of the decode] separated by scheduling barriers.
// Measured on MI355X a unit costs max(34, 13 + 4 * vector instructions) cycles, which is why the decode
// is kept under six instructions per MFMA.
//
// A reduction step covers 2 chunks (64 values for 4-bit formats, 32 for 8-bit ones). The order of the
// products inside a step is permuted identically for both operands, which a sum does not see.
#include <type_traits>

#include "common.h"
#include "qformat.h"

namespace dmoe {

constexpr int kMfmaWaves = 4;
constexpr int kMfmaRing = 4;  // reduction steps per LDS activation block
constexpr int kMfmaWRing = 2; // weight steps held in registers

template <typename Fmt>
struct MfmaGeom {
    static constexpr int KV = Fmt::kVals;          // values per 16-byte chunk
    static constexpr int KSTEP = 2 * KV;           // reduction elements per step
    static constexpr int NJ = KV / 8;              // MFMAs (K = 16) per step and tile
    static constexpr int KB = kMfmaRing * KSTEP;   // reduction elements per activation block
    static constexpr int LDA = KB + 8;             // LDS row pitch in bf16 elements (+16 bytes: conflict-free b128 reads)
    static constexpr int NI = KB / 64;             // 128-byte granules per activation row and block
    static constexpr size_t kBufBytes = (size_t)kMfmaTileM * LDA * 2;
    static constexpr size_t kLdsBytes = 2 * kBufBytes;
    static_assert(NJ % 2 == 0 && NI % 2 == 0, "fragment ping-pong and half-block staging need even counts");
};

// One tile with MT 32-row MFMA tiles (MT is a template parameter so that the reduction loop is straight-line code).
template <typename Fmt, bool GATE_UP, bool PACKED, int MT>
__device__ __forceinline__ void mfma_tile(const GemmArgs &g, const Tile &t, uint8_t *lds) {
    using CS = ChunkStream<Fmt, PACKED>;
    using G = MfmaGeom<Fmt>;
    constexpr int KV = G::KV, KSTEP = G::KSTEP, NJ = G::NJ, KB = G::KB, LDA = G::LDA, NI = G::NI;
    constexpr int NT = 2; // 32-column MFMA tiles per wavefront
    constexpr int WR = kMfmaWRing; // weight steps held in registers
    const int tid = (int)threadIdx.x, lane = tid & 63, ln = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cols = g.b0.cols, n_out = g.b0.rows;
    const int n_steps = cols / KSTEP;
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
    uint4 ring_raw[WR][NT];
    uint32_t ring_sb[WR][NT][2];
    auto load_b = [&](int step, int slot_) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
            ring_raw[slot_][nt] = cs[nt].load_chunk(step); // rows of a switched-off tile alias valid memory, never stored
            cs[nt].load_meta(b, step, ring_sb[slot_][nt]);
        }
    };
    // weight loads depend on the tile only: start them first (steps past the end are clamped, their data unused)
#pragma unroll
    for (int j = 0; j < WR; ++j) load_b(j < n_steps ? j : n_steps - 1, j);

    // ---- activation staging ------------------------------------------------------------------------------
    // thread -> (row a_row + 32 * p, 16-byte piece a_piece of each 128-byte granule): eight lanes cover one full
    // cache line of a row. A block is staged in two halves (granules [0, NI/2) and [NI/2, NI)) so that only half of
    // it sits in registers at a time. Rows past the segment end alias the tile's first row; they are never stored.
    const int a_piece = tid & 7, a_row = tid >> 3;
    const uint16_t *a_ptr[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int r = a_row + 32 * p;
        const uint32_t pr = t.row0 + (uint32_t)(r < (int)t.nrows ? r : 0);
        const size_t src = g.a_rows ? g.a_rows[pr] : pr;
        a_ptr[p] = g.a + src * (size_t)cols + a_piece * 8;
    }
    // One staging operation = one 16-byte load (or LDS store) per thread: piece ii of half `half` for the rows of
    // pass p. Both halves of a block have registers of their own, so that every load has two reduction steps to
    // arrive before its store, and the operations are issued one at a time between the MFMAs (a burst of them
    // stalls the wavefront's in-order issue while the memory pipes drain: ~50 cycles per LDS store).
    constexpr int kOpsPerHalf = MT * (NI / 2);
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4))); // a first-class value, unlike HIP's uint4 struct
    u32x4_t a_reg[2 * MT * (NI / 2)];
    auto load_a_op = [&](int blk, int half, int op) {
        const int p = op % MT, ii = op / MT;
        // uniform, clamped into the row: granules past the row end (the surplus steps of the last trip, or the
        // block after the last one) re-read the last granule and are zeroed in LDS by zero_tail
        int k0 = blk * KB + (half * (NI / 2) + ii) * 64;
        k0 = k0 < cols - 64 ? k0 : cols - 64;
        a_reg[(half * MT + p) * (NI / 2) + ii] = *(const u32x4_t *)(a_ptr[p] + k0);
    };
    uint8_t *const a_wr = lds + ((size_t)a_row * LDA + a_piece * 8) * 2;
    auto store_a_op = [&](uint32_t buf_off, int half, int op) {
        const int p = op % MT, ii = op / MT;
        *(u32x4_t *)(a_wr + buf_off + ((size_t)p * 32 * LDA + (half * (NI / 2) + ii) * 64) * 2) =
            a_reg[(half * MT + p) * (NI / 2) + ii];
    };
    // zero the granules of block blk that lie past the row end (only the last block of a reduction whose step count
    // is not a multiple of the trip length has any); runs after this thread's own stores to the same addresses
    auto zero_tail = [&](uint32_t buf_off, int blk) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
            if (blk * KB + i * 64 >= cols)
#pragma unroll
                for (int p = 0; p < MT; ++p)
                    *(uint4 *)(a_wr + buf_off + ((size_t)p * 32 * LDA + i * 64) * 2) = make_uint4(0, 0, 0, 0);
    };

    f32x16_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

    uint32_t wp[2][NT][KV / 2]; // decoded weights of the current / next step
    bf16x8_t xf[2][MT];         // activation fragments of the current / next MFMA group
    const uint8_t *const x_rd = lds + ((size_t)ln * LDA + h * KV) * 2;
    auto read_x = [&](uint32_t buf_off, int sb, int j, int mt, int pp) {
        uint4 q = *(const uint4 *)(x_rd + buf_off + ((size_t)mt * 32 * LDA + sb * KSTEP + 8 * j) * 2);
        xf[pp][mt] = __builtin_bit_cast(bf16x8_t, q);
    };
    // One reduction step: MT*NT*NJ units of [one MFMA of step s | the decode of a slice of step s+1's weights], with
    // a scheduling barrier after every unit (left to itself the compiler emits the whole decode first and the
    // MFMAs after it, which serialises the two pipes). Activation fragments are read from LDS one MFMA group
    // (MT*NT units) ahead of their use; the first group of the next step of the same block is fetched during the
    // last group of this one.
    auto step_body = [&](int slot_next, int which, uint32_t buf_off, int sb, auto side) {
        constexpr int NU = NJ * MT * NT; // units
        constexpr int NP = NT * (KV / 2); // packed pairs to decode for the next step
        Meta meta_next[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) meta_next[nt] = Fmt::pair_meta(CS::meta(ring_sb[slot_next][nt]));
        uint32_t dstate[Fmt::kPairState] = {};
        Fmt::pair_state(dstate);
        if (sb == 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) read_x(buf_off, 0, 0, mt, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const int u = (j * MT + mt) * NT + nt;
                    if (nt == 0) { // one fragment per unit pair, a whole MFMA group ahead of its use
                        if (j + 1 < NJ) read_x(buf_off, sb, j + 1, mt, (j + 1) & 1);
                        else if (sb + 1 < kMfmaRing) read_x(buf_off, sb + 1, 0, mt, 0);
                    }
                    side(u);
                    uint4 q = make_uint4(wp[which][nt][4 * j], wp[which][nt][4 * j + 1], wp[which][nt][4 * j + 2],
                                         wp[which][nt][4 * j + 3]);
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, q), xf[j & 1][mt],
                                                                          acc[mt][nt], 0, 0, 0);
#pragma unroll
                    for (int p = u * NP / NU; p < (u + 1) * NP / NU; ++p) {
                        Fmt::decode_pair(ring_raw[slot_next][p / (KV / 2)], meta_next[p / (KV / 2)], p % (KV / 2),
                                         wp[which ^ 1][p / (KV / 2)], dstate);
                        // pin the slice here: without it the optimiser sinks the decode of a trip's last step
                        // into the head of the next trip, where nothing overlaps it
                        asm volatile("" : "+v"(wp[which ^ 1][p / (KV / 2)][p % (KV / 2)]));
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int op = 0; op < kOpsPerHalf; ++op) load_a_op(0, half, op);
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int op = 0; op < kOpsPerHalf; ++op) store_a_op(0, half, op);
    const int n_trips = (n_steps + kMfmaRing - 1) / kMfmaRing;
    const bool ragged = n_steps % kMfmaRing != 0; // uniform, rare
    if (ragged && n_trips == 1) zero_tail(0, 0);
    __syncthreads();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) Fmt::decode_fast(ring_raw[0][nt], CS::meta(ring_sb[0][nt]), wp[0][nt]);

    // The loop always runs whole trips of kMfmaRing steps (one activation block): past the end of the reduction the
    // activation blocks are zero-filled and the weight loads are clamped onto the last valid step, so the surplus
    // steps add 0 * w and the loop body is one straight line with no guarded copy. While a trip computes from one
    // LDS buffer, the next block is staged into the other; one barrier per trip publishes it.
    static_assert(kMfmaRing == 4, "the staging schedule below is written for four steps per trip");
#pragma unroll 1
    for (int trip = 0; trip < n_trips; ++trip) {
        const int s0 = trip * kMfmaRing;
        const uint32_t rd_off = (trip & 1) ? (uint32_t)G::kBufBytes : 0u, wr_off = (uint32_t)G::kBufBytes - rd_off;
#pragma unroll
        for (int j = 0; j < kMfmaRing; ++j) {
            const int s = s0 + j;
            const int s_ahead = s + WR < n_steps ? s + WR : n_steps - 1;
            load_b(s_ahead, j % WR); // this slot was decoded one step ago
            // steps 0, 1: fetch the two halves of the next block; steps 2, 3: store them into the other buffer
            step_body((j + 1) % WR, j & 1, rd_off, j, [&](int u) {
                constexpr int NU = NJ * MT * NT, every = NU / kOpsPerHalf;
                static_assert(NU % kOpsPerHalf == 0, "staging operations must spread evenly over the units");
                if (u % every != 0) return;
                if (j < 2) load_a_op(trip + 1, j, u / every);
                else store_a_op(wr_off, j - 2, u / every);
            });
            if (j == 3) {
                if (ragged && trip + 2 == n_trips) zero_tail(wr_off, trip + 1);
                __syncthreads();
            }
        }
    }

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
// 8-bit formats: 70 KiB of LDS per workgroup, so two workgroups share a compute unit if a wavefront stays under 256
// registers; the 4-bit formats stage twice the reduction length per block (135 KiB) and run one workgroup per unit
__global__ __launch_bounds__(kMfmaWaves * 64, Fmt::kVals == 16 ? 2 : 1) void qgemm_mfma_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t mfma_lds[]; // bf16 As[2][kMfmaTileM][LDA]
    Tile t;
    const uint32_t slot = blockIdx.y;
    if (g.tiles) {
        const uint32_t n_tiles = *g.n_tiles;
        t = g.tiles[slot];
        if (slot >= n_tiles) return;
        if ((int)t.nrows < g.min_rows) return; // left to the weight-streaming kernel
    } else {
        t.expert = 0;
        t.row0 = slot * (uint32_t)g.tile_m;
        if ((int)t.row0 >= g.dense_rows) return;
        uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)g.tile_m ? left : (uint32_t)g.tile_m;
    }
    // the tile is the same for the whole workgroup; saying so keeps the four variants apart as scalar branches
    switch (__builtin_amdgcn_readfirstlane((int)((t.nrows + 31u) >> 5))) {
    case 1: mfma_tile<Fmt, GATE_UP, PACKED, 1>(g, t, mfma_lds); break;
    case 2: mfma_tile<Fmt, GATE_UP, PACKED, 2>(g, t, mfma_lds); break;
    case 3: mfma_tile<Fmt, GATE_UP, PACKED, 3>(g, t, mfma_lds); break;
    case 4: mfma_tile<Fmt, GATE_UP, PACKED, 4>(g, t, mfma_lds); break;
    default: break;
    }
}

bool qgemm_mfma_supports(const QView &b) {
    int vals = (b.mode == DMOE_QUANT_AFFINE && b.bits == 4) || b.mode == DMOE_QUANT_MXFP4 ? 32 : 16;
    // activation rows are staged in 128-byte granules; unquantized weights have their own kernel
    return b.mode != DMOE_QUANT_NONE && b.cols % (2 * vals) == 0 && b.cols % 64 == 0 && b.rows % 4 == 0;
}

template <typename Fmt, bool GATE_UP, bool PACKED>
static int mfma_raise_limit() {
    static LdsLimit limit; // per instantiation
    return raise_lds_limit(limit, (const void *)qgemm_mfma_kernel<Fmt, GATE_UP, PACKED>, (int)MfmaGeom<Fmt>::kLdsBytes);
}
template <typename Fmt>
static int mfma_prepare_format() {
    DMOE_TRY((mfma_raise_limit<Fmt, true, false>()));
    return mfma_raise_limit<Fmt, false, false>();
}
int qgemm_mfma_prepare() {
    DMOE_TRY(mfma_prepare_format<FmtAffine4>());
    DMOE_TRY(mfma_prepare_format<FmtAffine8>());
    DMOE_TRY(mfma_prepare_format<FmtMxfp4>());
    return mfma_prepare_format<FmtFp8Row>();
}

struct MfmaLaunch {
    const GemmArgs &g;
    hipStream_t st;
    template <typename Fmt, bool GATE_UP, bool PACKED>
    int go() {
        auto kern = qgemm_mfma_kernel<Fmt, GATE_UP, PACKED>;
        const size_t lds = MfmaGeom<Fmt>::kLdsBytes;
        DMOE_TRY((mfma_raise_limit<Fmt, GATE_UP, PACKED>())); // done by dmoe_init for its device; a flag test otherwise
        const int cols_per_block = kMfmaWaves * (GATE_UP ? 32 : 64);
        dim3 grid((unsigned)ceil_div(g.b0.rows, cols_per_block), (unsigned)g.max_tiles), block(kMfmaWaves * 64);
        hipLaunchKernelGGL(kern, grid, block, lds, st, g);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    template <typename Fmt>
    int operator()() {
        return g.gate_up ? go<Fmt, true, false>() : go<Fmt, false, false>();
    }
};

int launch_qgemm_mfma(const GemmArgs &g, hipStream_t st) {
    if (qgemm_wide_supports(g.b0)) return launch_qgemm_wide(g, st);
    DMOE_REQUIRE(g.tile_m > 0 && g.tile_m <= kMfmaTileM && g.tile_m % 32 == 0, "MFMA GEMM: bad tile size %d", g.tile_m);
    DMOE_REQUIRE(qgemm_mfma_supports(g.b0) && !g.b0.packed, "MFMA GEMM: unsupported weight shape (rows=%d cols=%d)",
                 g.b0.rows, g.b0.cols);
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
