// Grouped quantized GEMM, wide MFMA path (prefill, every quantized format in the packed resident layout).
//
// One workgroup (4 wavefronts) = one tile of up to 128 rows of ONE expert segment against a strip of output columns;
// each wavefront dequantizes its own 64 weight rows straight into the A operand of v_mfma_f32_32x32x16_bf16 and
// holds 128 x 64 f32 accumulators. The kernel is built so that TWO workgroups fit a compute unit (at most 256
// registers per wavefront, 64 KiB of LDS): a lone wavefront on a SIMD issues a vector instruction only every ~5
// cycles, two wavefronts every ~2.8, and the 4-bit decode (2.1 vector instructions per weight) is the largest
// item beside the MFMAs. A variant with 256-row tiles (every decoded fragment feeds eight MFMAs instead of four, but one
// wavefront per SIMD: all 512 registers, 128 KiB of LDS) measured 5 % slower on the 8k-token ragged prefill.
// The 8-bit formats run the same loop with two 16-byte chunk steps per 64-element step. Differences from the
// MLX-layout kernel in qgemm_mfma.hip:
//
//  * Activations go from global memory into LDS without passing through registers (global_load_lds_dwordx4).
//    One such instruction moves 1 KiB: 8 rows x 128 bytes (one reduction step of 64 bf16). Inside that KiB the
//    16-byte pieces of row r are stored at position piece ^ ((r >> 1) & 7). The LDS serves a 16-byte read
//    instruction 16 lanes (256 bytes, all 64 banks) per cycle, and a lane's place among the banks is
//    (row & 1) * 8 + position: rows 2q and 2q + 1 differ in the first term, the eight row pairs of a 16-lane group in
//    the second, so the MFMA operand reads (32 rows at the same reduction offset) run at the full 256 bytes per
//    cycle (position piece ^ (r & 7) made rows r and r + 8 collide: 155 bytes per cycle measured). The swizzle
//    costs nothing because each lane picks its global source address freely.
//  * Four LDS buffers of one reduction step each (4 x 16 KiB): while step s computes, the loads of step s+2
//    are in flight. The compiler does not know about these loads (they are issued from inline assembly), so
//    their completion is tracked by hand: VMEM operations return in order, hence "at most MT operations
//    outstanding" three quarters into step s implies that everything issued before this step's own MT loads
//    -- in particular the loads of step s+1 -- has landed. One s_barrier per step then publishes the buffer.
//  * The same in-order rule means a deep register ring of weight loads buys nothing (any wait for a staging request
//    also waits for every older weight load), so the weights of only two steps are in flight, which is what
//    keeps the wavefront under 256 registers.
//  * Activation fragments are single-buffered (except for tiles of at most 64 rows): the fragment of row tile mt
//    is reloaded for the next MFMA group right after its last use in this one, 2*MT-1 units before it is needed
//    again.
//
// The reduction loop is software-pipelined like the other MFMA kernel: units of [one MFMA | a slice of the decode
// of the next step's weights] separated by scheduling barriers.
#include <type_traits>

#include "common.h"
#include "qformat.h"

namespace dmoe {

constexpr int kWideWaves = 4;
constexpr int kWideRing = 4;                              // LDS activation buffers = steps per unrolled trip
constexpr int kWideWRing = 2;                             // weight steps held in registers (see the header)
constexpr int kWideBufBytes = kMfmaWideTileM * 128;       // one reduction step (64 bf16) of every row of the tile
constexpr size_t kWideLdsBytes = (size_t)kWideRing * kWideBufBytes;

// s_waitcnt immediates (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14])
constexpr int wait_vmcnt(int n) { return 0x0f70 | (n & 15) | ((n >> 4) << 14); }
constexpr int wait_vmcnt_lgkm0(int n) { return 0x0070 | (n & 15) | ((n >> 4) << 14); }
constexpr int kWaitLgkm0 = 0xc07f;

template <typename Fmt, bool GATE_UP, int MT>
__device__ __forceinline__ void wide_tile(const GemmArgs &g, const Tile &t, uint8_t *lds, const int strip) {
    using CS = ChunkStream<Fmt, true>;
    // A step is 64 reduction elements = one 128-byte activation granule. A lane's 16-byte weight chunk holds 32 (4-bit
    // formats) or 16 (8-bit formats) of them: the weights come in chunk steps of 2 * KV elements, CH of them per step,
    // and ring, decode and the double-buffered decoded operands advance by chunk steps.
    constexpr int KV = Fmt::kVals, KSTEP = 64, NJ = 4, NT = 2;
    constexpr int CH = 32 / KV;           // chunk steps per step
    static_assert(CH == 1 || CH == 2 || CH == 4, "chunks of 32, 16 or 8 values");
    constexpr int NJC = NJ / CH;          // MFMA groups per chunk step
    constexpr int NUC = NJC * MT * NT;    // units (MFMAs) per chunk step
    constexpr int NPC = NT * (KV / 2);    // packed pairs to decode per chunk step
    // chunk steps held in registers (twice as many for tiles of at most 64 rows moved the 8-bit mixed batch by nothing)
    // (unquantized weights: four chunk steps per step, so one step's worth keeps the ring at the 8-bit formats' size)
    constexpr int WRC = CH == 4 ? CH : kWideWRing * CH;
    static_assert(kWideRing % kWideWRing == 0 && (kWideRing * CH) % WRC == 0, "ring slots must line up across trips");
    const int tid = (int)threadIdx.x, lane = tid & 63, ln = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cols = g.b0.cols, n_out = g.b0.rows;
    const int n_steps = cols / KSTEP, n_csteps = n_steps * CH;
    const int n_trips = (n_steps + kWideRing - 1) / kWideRing;
    const size_t e = t.expert;

    // ---- this wavefront's weight rows (gate_up: tile 0 = gate, tile 1 = up rows of the same 32 columns) ----
    const int col_base = (strip * kWideWaves + wave) * (GATE_UP ? 32 : 64);
    const bool wave_on = col_base < n_out;
    CS cs[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
        const int base = GATE_UP ? col_base : col_base + 32 * nt;
        const bool on = wave_on && base < n_out;
        int n = base + ln;
        if (n >= n_out) n = n_out - 1;
        cs[nt].init(b, e, (on ? base : 0) >> 5, ln, h, n); // a switched-off tile aliases valid memory, never stored
    }
    uint4 ring_raw[WRC][NT];
    uint32_t ring_sb[WRC][NT][2];
    auto load_b = [&](int cstep, int slot_) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const QView &b = (GATE_UP && nt == 1) ? g.b1 : g.b0;
            ring_raw[slot_][nt] = cs[nt].load_chunk(cstep);
            cs[nt].load_meta(b, cstep, ring_sb[slot_][nt]);
        }
    };
#pragma unroll
    for (int j = 0; j < WRC; ++j) load_b(j < n_csteps ? j : n_csteps - 1, j);

    // ---- activation staging -------------------------------------------------------------------------------
    // operation i of this wavefront moves rows (wave + 4 i) * 8 .. + 7; lane = (row r8 of the eight, position c),
    // and fetches piece c ^ ((row >> 1) & 7) of its row. Rows past the segment end alias the tile's first row (never
    // stored).
    const int r8 = lane >> 3, c = lane & 7;
    const uint8_t *a_src[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int r = (wave + 4 * i) * 8 + r8;
        const uint32_t pr = t.row0 + (uint32_t)(r < (int)t.nrows ? r : 0);
        const size_t src = g.a_rows ? g.a_rows[pr] : pr;
        a_src[i] = (const uint8_t *)(g.a + src * (size_t)cols) + ((c ^ (((r >> 1) & 7))) * 16);
    }
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    auto stage_op = [&](int blk, int buf, int i) {
        const uint8_t *gp = a_src[i] + (size_t)blk * 128;
        const uint32_t la = lds_addr + (uint32_t)(buf * kWideBufBytes + (wave + 4 * i) * 1024); // uniform
        asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gp), "s"(la) : "memory"); // nothing else in this kernel uses M0
    };
    // surplus steps of the last trip (n_steps not a multiple of the ring) must multiply zeros
    auto zero_block = [&](int buf) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
            *(uint4 *)(lds + buf * kWideBufBytes + (wave + 4 * i) * 1024 + lane * 16) = make_uint4(0, 0, 0, 0);
        __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    };

    f32x16_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

    uint32_t wp[2][NT][KV / 2]; // decoded weights of the current / next step
    // activation fragment of each row tile for the current MFMA group; small tiles have registers to spare and too
    // few units per group to hide an LDS round trip, so they keep a second set and fetch a whole group ahead
    constexpr int XB = MT <= 2 ? 2 : 1;
    // blocks in flight ahead of the one being computed. A short step (small tile) does not cover a memory round
    // trip, so small tiles run three blocks ahead; that reuses the buffer read during the previous step, which is
    // only safe because those tiles also wait for their own LDS reads before each barrier (see below).
    constexpr int AHEAD = MT <= 2 ? 3 : 2;
    bf16x8_t xf[XB][MT];
    // fragment (mt, j) of a step: row mt * 32 + ln, the piece that holds this lane's eight reduction elements of MFMA
    // group j (chunk step c = j / NJC of the step, elements (2 c + h) * KV + 8 (j % NJC) onwards), stored at
    // piece ^ ((row >> 1) & 7)
    const uint8_t *x_rd[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int piece = ((2 * (j / NJC) + h) * KV + 8 * (j % NJC)) >> 3;
        x_rd[j] = lds + (ln >> 3) * 1024 + (ln & 7) * 128 + ((piece ^ ((ln >> 1) & 7)) * 16);
    }
    auto read_x = [&](int buf, int j, int mt) {
        uint4 q = *(const uint4 *)(x_rd[j] + buf * kWideBufBytes + mt * 4096);
        xf[j % XB][mt] = __builtin_bit_cast(bf16x8_t, q);
    };

    // ---- prologue: the first AHEAD blocks, first decode ----------------------------------------------------------
#pragma unroll
    for (int b = 0; b < AHEAD; ++b) {
        if (b < n_steps) {
#pragma unroll
            for (int i = 0; i < MT; ++i) stage_op(b, b, i);
        } else {
            zero_block(b);
        }
    }
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) Fmt::decode_fast(ring_raw[0][nt], CS::meta(ring_sb[0][nt]), wp[0][nt]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) read_x(0, 0, mt);

    // The loop always runs whole trips of kWideRing steps: surplus steps multiply zeroed activations with weights
    // clamped onto the last valid step. Step j of a trip computes from buffer j, requests block s + AHEAD into buffer
    // (j + AHEAD) % 4 during its first three MFMA groups, and at the start of the fourth waits for block s + 1 and
    // synchronises, so that the first fragments of the next step can be fetched during that last group.
#pragma unroll 1
    for (int trip = 0; trip < n_trips; ++trip) {
        const int s0 = trip * kWideRing;
#pragma unroll
        for (int j = 0; j < kWideRing; ++j) {
            const int s = s0 + j;
            const int buf_next = (j + 1) % kWideRing;
            const bool stage = s + AHEAD < n_steps; // uniform
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int ci = j * CH + c; // chunk step within the trip
                const int cs_ahead = s * CH + c + WRC < n_csteps ? s * CH + c + WRC : n_csteps - 1;
                load_b(cs_ahead, ci % WRC); // this slot was decoded one chunk step ago
                const int slot_next = (ci + 1) % WRC, which = ci & 1;
                Meta meta_next[NT];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) meta_next[nt] = Fmt::pair_meta(CS::meta(ring_sb[slot_next][nt]));
                uint32_t dstate[Fmt::kPairState] = {};
                Fmt::pair_state(dstate);
#pragma unroll
                for (int jc = 0; jc < NJC; ++jc) {
                    const int jj = c * NJC + jc; // MFMA group within the step
                    if (jj == NJ - 1) {
                        // block s + 1 must have landed; the AHEAD - 1 younger requests of MT operations each may still
                        // fly (fewer near the end of the reduction, when nothing is requested any more), and so may
                        // the weight chunks that the later chunk steps of this step have requested since (LATE, at
                        // least one load per weight tile each)
                        constexpr int LATE = (CH - 1) * NT;
                        if (AHEAD == 2) {
                            if (stage) __builtin_amdgcn_s_waitcnt(wait_vmcnt(MT + LATE));
                            else __builtin_amdgcn_s_waitcnt(wait_vmcnt(LATE));
                        } else {
                            // also drain this wavefront's LDS reads: the next step's requests overwrite the buffer
                            // that the reads issued during the previous MFMA group came from
                            if (stage) __builtin_amdgcn_s_waitcnt(wait_vmcnt_lgkm0(2 * MT + LATE));
                            else if (s + AHEAD - 1 < n_steps) __builtin_amdgcn_s_waitcnt(wait_vmcnt_lgkm0(MT + LATE));
                            else __builtin_amdgcn_s_waitcnt(wait_vmcnt_lgkm0(LATE));
                        }
                        asm volatile("" ::: "memory");
                        __builtin_amdgcn_s_barrier();
                        asm volatile("" ::: "memory");
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) {
                            const int uc = (jc * MT + mt) * NT + nt; // unit within the chunk step
                            const int u = c * NUC + uc;              // unit within the step
                            uint4 q = make_uint4(wp[which][nt][4 * jc], wp[which][nt][4 * jc + 1], wp[which][nt][4 * jc + 2],
                                                 wp[which][nt][4 * jc + 3]);
                            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, q),
                                                                                  xf[jj % XB][mt], acc[mt][nt], 0, 0, 0);
                            // fetch the fragment of the next group: after the last use of this one (one register set),
                            // or at the first (two sets)
                            if (nt == (XB == 1 ? NT - 1 : 0)) {
                                if (jj + 1 < NJ) read_x(j, jj + 1, mt);
                                else read_x(buf_next, 0, mt);
                            }
                            if (u % 6 == 0 && u / 6 < MT) { // the staging requests all fall into the first three groups
                                if (stage) stage_op(s + AHEAD, (j + AHEAD) % kWideRing, u / 6);
                            }
#pragma unroll
                            for (int p = uc * NPC / NUC; p < (uc + 1) * NPC / NUC; ++p) {
                                Fmt::decode_pair(ring_raw[slot_next][p / (KV / 2)], meta_next[p / (KV / 2)], p % (KV / 2),
                                                 wp[which ^ 1][p / (KV / 2)], dstate);
                                // pin the slice here (the optimiser would sink a trip's last decode into the next trip)
                                asm volatile("" : "+v"(wp[which ^ 1][p / (KV / 2)][p % (KV / 2)]));
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            }
            if (!stage && s + AHEAD < n_trips * kWideRing) zero_block((j + AHEAD) % kWideRing); // a surplus step: zeros
        }
    }

    // ---- epilogue: lane = token row (ln), registers r -> output column 8*(r/4) + 4*h + r%4 -------------
    // In that layout a store instruction would touch 32 rows with 16 bytes each. The tile goes through LDS instead
    // (the activation ring is free once every wavefront has left the loop; each wavefront uses its own 16 KiB): written
    // as held, read back row-major, so that a store instruction writes whole 64- or 128-byte runs of 16 or 8 rows.
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __syncthreads();
    if (!wave_on) return;
    constexpr int ROWB = GATE_UP ? 64 : 128;  // bytes of one output row held by this wavefront (32 / 64 columns)
    constexpr int PITCH = ROWB + 16;
    constexpr int LPR = ROWB / 16;            // lanes per row when reading back
    constexpr int RPI = 64 / LPR;             // rows per store instruction
    uint8_t *mine = lds + wave * (kWideLdsBytes / kWideWaves);
    const bool wide_store = (((uintptr_t)g.out | ((uintptr_t)g.ldo * 2)) % 16) == 0;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int rl = mt * 32 + ln;
        const uint32_t p = t.row0 + (uint32_t)(rl < (int)t.nrows ? rl : 0);
        const uint32_t dst = g.out_rows ? g.out_rows[p] : p;
        float rscale = 1.0f;
        if (g.row_scale) rscale = g.row_scale[g.row_scale_idx ? g.row_scale_idx[p] : p];
        uint8_t *wrow = mine + ln * PITCH;
        // per-row weight scales (FP8): output column n of register 4 rg + i is col_base (+ 32 nt) + 8 rg + 4 h + i
        auto wscale = [&](const QView &b, int n) {
            return *(const float *)(b.scales + e * b.s_mat + (size_t)(n < n_out ? n : n_out - 1) * b.s_row);
        };
        if (GATE_UP) {
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float gv = acc[mt][0][4 * rg + i], uv = acc[mt][1][4 * rg + i];
                    if (Fmt::kRowScale) {
                        gv *= wscale(g.b0, col_base + 8 * rg + 4 * h + i);
                        uv *= wscale(g.b1, col_base + 8 * rg + 4 * h + i);
                    }
                    v[i] = limited_swiglu(gv, uv, g.swiglu_limit) * rscale;
                }
                *(uint2 *)(wrow + (8 * rg + 4 * h) * 2) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int rg = 0; rg < 4; ++rg) {
                    float v[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        v[i] = acc[mt][nt][4 * rg + i];
                        if (Fmt::kRowScale) v[i] *= wscale(g.b0, col_base + 32 * nt + 8 * rg + 4 * h + i);
                        v[i] *= rscale;
                    }
                    *(uint2 *)(wrow + (32 * nt + 8 * rg + 4 * h) * 2) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                }
            }
        }
        // the same wavefront reads what it wrote: LDS operations of a wavefront complete in order
#pragma unroll
        for (int q = 0; q < 32 / RPI; ++q) {
            const int row = q * RPI + lane / LPR, piece = lane % LPR;
            const uint32_t drow = (uint32_t)__shfl((int)dst, row, 64); // lane `row` holds that row's destination
            const uint4 v = *(const uint4 *)(mine + row * PITCH + piece * 16);
            const int n0 = col_base + piece * 8;
            if (mt * 32 + row >= (int)t.nrows || n0 >= n_out) continue;
            uint16_t *o = g.out + (size_t)drow * (size_t)g.ldo + n0;
            if (wide_store && n0 + 8 <= n_out) {
                *(uint4 *)o = v;
            } else {
                *(uint2 *)o = make_uint2(v.x, v.y);
                if (n0 + 4 < n_out) *(uint2 *)(o + 4) = make_uint2(v.z, v.w);
            }
        }
    }
}

template <typename Fmt, bool GATE_UP>
__global__ __launch_bounds__(kWideWaves * 64, 2) void qgemm_wide_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t wide_lds[]; // [kWideRing][128 rows][128 bytes], swizzled
    Tile t;
    // Workgroups go to the eight XCDs round-robin in launch order; gridDim.y is a multiple of 8, which makes the maps
    // below permutations of the grid. XCD x = (tile class x / 2, strip half x % 2): it takes every fourth tile of the
    // list and one half of the tile's column strips, a tile's strips back to back. A tile's activations then enter two
    // L2s instead of eight, and consecutive tiles of an expert find the half of its weights they need in the L2 they
    // run on. Same box, against all strips of a tile on one XCD (the map before, kept for strip counts that are odd):
    // C3 step -0.7 % (down launch -1.6 %), C4 step -1.7 % (gate/up launch -2.4 %); four strip groups x two tile classes
    // -0.6 % / -1.3 %, eight strip groups (an XCD = two strips of every tile) +0.8 % / -0.9 %. (Giving an XCD runs of
    // 2..16 consecutive tiles with ALL their strips, so that the tiles of an expert could share its weights through
    // that L2, measured 0.5 % to 15 % slower the longer the run: an expert's weights do not fit one L2.)
    const uint32_t nx = gridDim.x, b = blockIdx.y * nx + blockIdx.x, k = b >> 3, xcd = b & 7u;
    uint32_t slot;
    int strip;
    if (nx % 2u == 0u) {
        const uint32_t half = nx / 2u;
        slot = 4u * (k / half) + (xcd >> 1);
        strip = (int)((xcd & 1u) * half + k % half);
    } else {
        slot = (k / nx) * 8u + xcd;
        strip = (int)(k % nx);
    }
    if (g.tiles) {
        const uint32_t n_tiles = *g.n_tiles;
        t = g.tiles[slot < (uint32_t)g.max_tiles ? slot : 0u];
        if (slot >= n_tiles) return;
        if ((int)t.nrows < g.min_rows) return; // left to the weight-streaming kernel
    } else {
        t.expert = 0;
        t.row0 = slot * (uint32_t)g.tile_m;
        if ((int)t.row0 >= g.dense_rows) return;
        uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)g.tile_m ? left : (uint32_t)g.tile_m;
    }
    // the tile is the same for the whole workgroup; saying so keeps the variants apart as scalar branches
    const int mt = __builtin_amdgcn_readfirstlane((int)((t.nrows + 31u) >> 5));
    if (mt <= 1) wide_tile<Fmt, GATE_UP, 1>(g, t, wide_lds, strip);
    else if (mt == 2) wide_tile<Fmt, GATE_UP, 2>(g, t, wide_lds, strip);
    else if (mt == 3) wide_tile<Fmt, GATE_UP, 3>(g, t, wide_lds, strip);
    else if (mt == 4) wide_tile<Fmt, GATE_UP, 4>(g, t, wide_lds, strip);
}

bool qgemm_wide_supports(const QView &b) {
    return b.mode != DMOE_QUANT_NONE && b.packed && b.cols % 64 == 0 && b.rows % 4 == 0;
}

template <typename Fmt, bool GATE_UP>
static int wide_raise_limit() {
    static LdsLimit limit; // per instantiation
    return raise_lds_limit(limit, (const void *)qgemm_wide_kernel<Fmt, GATE_UP>, (int)kWideLdsBytes);
}
template <typename Fmt>
static int wide_prepare_format() {
    DMOE_TRY((wide_raise_limit<Fmt, true>()));
    return wide_raise_limit<Fmt, false>();
}
int qgemm_wide_prepare() {
    DMOE_TRY(wide_prepare_format<FmtBf16>());
    DMOE_TRY(wide_prepare_format<FmtAffine4>());
    DMOE_TRY(wide_prepare_format<FmtAffine8>());
    DMOE_TRY(wide_prepare_format<FmtMxfp4>());
    return wide_prepare_format<FmtFp8Row>();
}

template <typename Fmt, bool GATE_UP>
static int launch_wide(const GemmArgs &g, hipStream_t st) {
    auto kern = qgemm_wide_kernel<Fmt, GATE_UP>;
    DMOE_TRY((wide_raise_limit<Fmt, GATE_UP>())); // done by dmoe_init for its device; a flag test otherwise
    const int cols_per_block = kWideWaves * (GATE_UP ? 32 : 64);
    dim3 grid((unsigned)ceil_div(g.b0.rows, cols_per_block), (unsigned)((g.max_tiles + 7) / 8 * 8)), block(kWideWaves * 64);
    hipLaunchKernelGGL(kern, grid, block, kWideLdsBytes, st, g);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

bool qgemm_wide_bf16_supports(const QView &b) {
    return b.mode == DMOE_QUANT_NONE && b.packed && b.cols % 64 == 0 && b.rows % 32 == 0 && ((uintptr_t)b.w % 16) == 0;
}

int launch_qgemm_wide(const GemmArgs &g, hipStream_t st) {
    DMOE_REQUIRE(qgemm_wide_supports(g.b0) || qgemm_wide_bf16_supports(g.b0),
                 "wide MFMA GEMM: unsupported weight format or shape (rows=%d cols=%d)", g.b0.rows, g.b0.cols);
    DMOE_REQUIRE(g.tile_m > 0 && g.tile_m <= kMfmaWideTileM && g.tile_m % 32 == 0, "wide MFMA GEMM: bad tile size %d",
                 g.tile_m);
    DMOE_REQUIRE(g.max_tiles >= 0 && g.max_tiles <= 65528, "wide MFMA GEMM: %d tiles exceed the grid limit", g.max_tiles);
    DMOE_REQUIRE(g.a && g.out && g.ldo > 0 && g.ldo % 4 == 0 && ((uintptr_t)g.out % 8) == 0 &&
                     ((uintptr_t)g.a % 16) == 0,
                 "wide MFMA GEMM: bad output / activation pointer or pitch");
    if (g.gate_up)
        DMOE_REQUIRE(g.b1.rows == g.b0.rows && g.b1.cols == g.b0.cols && g.b1.mode == g.b0.mode &&
                         g.b1.bits == g.b0.bits && g.b1.group == g.b0.group && g.b1.packed == g.b0.packed,
                     "wide MFMA GEMM: gate and up projections differ in shape or format");
    if (g.max_tiles == 0) return DMOE_OK;
    if (g.b0.mode == DMOE_QUANT_NONE)
        return g.gate_up ? launch_wide<FmtBf16, true>(g, st) : launch_wide<FmtBf16, false>(g, st);
    if (g.b0.mode == DMOE_QUANT_MXFP4)
        return g.gate_up ? launch_wide<FmtMxfp4, true>(g, st) : launch_wide<FmtMxfp4, false>(g, st);
    if (g.b0.mode == DMOE_QUANT_FP8_ROW)
        return g.gate_up ? launch_wide<FmtFp8Row, true>(g, st) : launch_wide<FmtFp8Row, false>(g, st);
    if (g.b0.bits == 8)
        return g.gate_up ? launch_wide<FmtAffine8, true>(g, st) : launch_wide<FmtAffine8, false>(g, st);
    return g.gate_up ? launch_wide<FmtAffine4, true>(g, st) : launch_wide<FmtAffine4, false>(g, st);
}

} // namespace dmoe
