// Grouped quantized GEMM, skinny path (decode): at most kSkinnyTileM (32) rows per expert tile.
//
// The step is bound by streaming every live expert's packed weights once from HBM. Each wavefront of a
// workgroup owns 32 weight rows of a projection and walks the whole reduction dimension on its own: lane
// (n = lane % 32, h = lane / 32) loads the 16-byte chunk h of row n for the current 64-wide step straight into
// registers, a ring of kSkinnyStages steps deep, so the wavefronts never wait for each other while several
// KiB per wavefront are in flight. The tile's activations sit in LDS (put there by direct global->LDS loads,
// requested ahead of the weight ring) and feed the A operand of v_mfma_f32_32x32x16_bf16; the weights feed the
// B operand, so every lane's accumulators belong to ITS weight row and rows 8j+4h..8j+4h+3 of the tile, and
// nothing has to be reduced across lanes.
//
// Up to 8 rows - nearly every tile at decode - the tile's rows stay whole in LDS and a lane keeps 4 accumulators.
// 9 to 32 rows: LDS holds a half or a quarter of every row, restaged on the way, and a lane keeps up to 16
// accumulators; an expert with many rows then still streams its weights once instead of once per 8 rows.
// Gate and up rows go to separate wavefronts (eight per workgroup, paired through LDS at the end): half the
// registers per wavefront, twice the wavefronts per SIMD to overlap decode, matrix and memory waits.
//
// 4-bit affine weights (group >= 64) are never multiplied out. Codes become the bf16 numbers (128 + q)
// with one AND-OR per pair; both halves of a step lie in the same scale group, so the matrix core
// produces P[m][n] = sum_k x[m][k] (128 + q[n][k]) for one group and the lane applies
//     acc += s[n] * P + (b[n] - 128 s[n]) * sum_k x[m][k]
// with its own row's scale and bias: two FMAs per accumulator and group. The AND-OR leaves the codes of
// a word in the order (0,4,1,5,2,6,3,7); the activations are stored in LDS in the same order, which a
// sum does not see. Other formats are decoded to bf16 values and accumulated directly.
#include "common.h"
#include <type_traits>

#include "qformat.h"

namespace dmoe {

constexpr int kSkinnyWaves = 4;          // 32-row blocks of weight rows per workgroup
constexpr int kSkinnyStages = 8;
constexpr int kSkinnySmallStages = 6;    // packed layout, tiles of one row block (see STAGES in skinny_tile)
constexpr int kSkinnyGroupedStages = 16; // ring depth when the loads are issued four steps at a time
constexpr int kSkinnyRowBlock = 8;       // tile rows per row block: the LDS window holds 8 whole rows of activations

__device__ __forceinline__ uint32_t vgpr_const32(uint32_t c) {
    uint32_t v;
    asm volatile("v_mov_b32 %0, %1" : "=v"(v) : "s"(c));
    return v;
}

// (q_i, q_{i+4}) of each 8-code word as packed bf16 (128 + q): element order 0,4,1,5,2,6,3,7
__device__ __forceinline__ void codes_to_bf16(uint32_t w, uint32_t mask, uint32_t magic, uint32_t *o) {
    o[0] = (w & mask) | magic;
    o[1] = ((w >> 4) & mask) | magic;
    o[2] = ((w >> 8) & mask) | magic;
    o[3] = ((w >> 12) & mask) | magic;
}

// s_waitcnt immediate for "at most n vector-memory loads outstanding" (gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14])
constexpr int skinny_wait_vmcnt(int n) { return 0x0f70 | (n & 15) | ((n >> 4) << 14); }

template <int CTRL>
__device__ __forceinline__ float skinny_dpp(float x) {
    const int v = __float_as_int(x);
    return __int_as_float(__builtin_amdgcn_update_dpp(v, v, CTRL, 0xf, 0xf, false));
}

template <int NM>
struct SkinnyStage {
    uint4 raw[NM];
    uint32_t sb[NM][2];
};

// One tile, start to finish. RJT = 1: tiles of one row block (4 accumulators per lane, no restaging); RJT = 4: larger
// tiles (16 accumulators; a tile of two row blocks computes four, the surplus rows are never stored). The kernel
// calls one or the other right after fetching the tile, so the two share nothing but the arguments and each keeps
// its own register allocation.
// `gate_up` (workgroup-uniform) is the role of the launch: gate and up projections with SwiGLU (their rows on
// separate wavefronts, paired through LDS at the end), or a single projection.
// `sync` (paired launch, workgroup-uniform): kSkinnySyncSignal = every workgroup of the tile adds 1 to
// g.tile_done[slot] once its stores have reached memory; kSkinnySyncWait = the workgroup waits for g.tile_done[slot] to
// reach g.tile_done_target before it reads its activations (the other role's output), its weight ring already in flight.
constexpr int kSkinnySyncNone = 0, kSkinnySyncSignal = 1, kSkinnySyncWait = 2;

// LDS: [activation window][sums of x per step][GROUPED only: 4 KiB per wavefront for turning weight lines]
__host__ __device__ constexpr size_t skinny_turn_offset(int cols, int kstep) {
    return (size_t)kSkinnyRowBlock * (size_t)cols * 2 + (size_t)kSkinnyTileM * 16 +
           (size_t)(cols / kstep) * kSkinnyRowBlock * sizeof(float) + 128;
}
constexpr size_t kSkinnyTurnBytes = (size_t)2 * kSkinnyWaves * 4 * 1024;
// where a tile's outputs are gathered before they are stored: behind the exchange areas of the epilogue (16 KiB)
constexpr size_t kSkinnyStageOffset = 16384, kSkinnyStageBytes = (size_t)kSkinnyTileM * 256 * 2;

// MBLK (MLX layout only): the scale / bias entries of a row are not fetched one per step (32 cache lines touched per
// load for 2 useful bytes each, again at every step: these loads, not the weights, bounded the MLX-layout path) but 16
// bytes at a time - eight bf16 or sixteen E8M0 entries, the next block requested while the current one is in use.
template <typename Fmt, bool FACTORED, bool PACKED, int RJT, bool MBLK, bool KSPLIT = false>
__device__ __forceinline__ void skinny_tile(const GemmArgs &g, const Tile &t, uint8_t *skinny_lds, const bool gate_up,
                                            const int sync, const uint32_t slot) {
    using CS = ChunkStream<Fmt, PACKED>;
    constexpr int KV = Fmt::kVals;   // values per 16-byte chunk
    constexpr int KSTEP = 2 * KV;    // reduction elements per step (both lane halves)
    constexpr int NJ = KV / 8;       // MFMAs (K = 16) per step
    // depth of the weight ring: the large-tile copy of the factored 4-bit form keeps 16 accumulators AND 16 products
    // per lane and takes a shallower ring to stay inside the same register budget (span boundaries stay whole ring
    // rounds either way); the other formats have the registers for the full ring (32 rows per expert, 256 live
    // experts, MXFP4: 4.2 -> 4.4 TB/s)
    // MLX layout, tiles of one row block (GROUPED): in the operand layout a wavefront's load would take 32 bytes out of
    // each of 32 rows (32 cache lines per instruction, a quarter of each used, the same lines again for the next three
    // steps; measured 2.7 TB/s at best). Instead lane l of load i fetches 16 bytes of row 8 i + l / 8, eight lanes
    // covering one 128-byte line = the row's codes of four steps; the four loads of such a group wait in the register
    // ring like any other stage, and when their steps come up the wavefront turns them into the operand layout through
    // 4 KiB of LDS of its own (written as loaded, read back per step; a wavefront's LDS operations complete in order, so
    // no barrier is involved).
    constexpr bool GROUPED = MBLK && RJT == 1;
    constexpr int LG = 4; // steps per 128-byte line = loads per group
    // The bulk of a decode step - packed weights, tiles of one row block - measured best with SIX stages (ring of 4 / 5 /
    // 6 / 8 / 10 stages, same box: 64-token step 0.2549 / 0.2525 / 0.2527 / 0.2553 / 0.2652 ms, MXFP4 step 0.1351 / 0.1340
    // / 0.1335 / 0.1343 / 0.1349 ms; smaller batches alike): what a deeper ring adds in flight it costs before the first step.
    constexpr int STAGES = GROUPED                           ? kSkinnyGroupedStages
                           : (PACKED && RJT == 1 && !MBLK)   ? kSkinnySmallStages
                           : (RJT == 1 || !FACTORED)         ? kSkinnyStages
                                                             : kSkinnyStages / 2;
    constexpr int PRE = GROUPED ? STAGES : STAGES - 1; // stages requested before the first step is consumed
    constexpr int ROUND = MBLK && STAGES < 8 ? 8 : STAGES;  // steps per unrolled round (MBLK: whole blocks of entries)
    static_assert(ROUND % STAGES == 0 && (!MBLK || ROUND % 8 == 0), "rounds are whole turns of the ring");
    constexpr int NM = 1;                           // projections per wavefront
    constexpr int WAVES = 2 * kSkinnyWaves;         // eight wavefronts share one staging of the tile's activations
    const int cg = gate_up ? kSkinnyWaves : WAVES;  // 32-row blocks of weight rows per workgroup
    const int tid = (int)threadIdx.x, lane = tid & 63, ln = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cols = g.b0.cols, n_out = g.b0.rows;
    const int n_steps = cols / KSTEP;
    const size_t e = t.expert;
    // Few tiles in the launch (a decode step of one or two sequences): the launch cannot fill the chip, every SIMD has
    // one wavefront, and that wavefront's chain of dependent steps sets the time. The reduction of a tile is then cut
    // in two: wavefronts 0-3 take the first half of the steps and 4-7 the second half for HALF as many weight rows
    // per workgroup (twice the workgroups), and the halves meet through LDS before the epilogue. Packed layout and
    // tiles of one row block only (the launcher builds no larger tiles then).
    static_assert(!KSPLIT || (PACKED && !MBLK && RJT == 1), "the split reduction exists for packed one-row-block tiles");
    constexpr bool ks = KSPLIT; // a kernel of its own: the other instantiations carry none of this
    const int kh = ks ? wave >> 2 : 0, wq = ks ? wave & 3 : wave; // reduction half, wavefront within the half
    const int n_loc = ks ? n_steps >> 1 : n_steps, sb0 = kh * n_loc; // this wavefront's steps: sb0 .. sb0 + n_loc - 1

    // ---- this lane's weight row ------------------------------------------------------------------------
    // A wavefront past the last block of weight rows repeats that block (and stores nothing): every wavefront
    // of the workgroup then runs the same control flow, which the barriers below rely on.
    const int proj = gate_up ? (wq & 1) : 0;        // gate/up: even wavefronts take gate rows, odd ones up rows
    const int col_raw = ((int)blockIdx.x * (ks ? cg >> 1 : cg) + (gate_up ? wq >> 1 : wq)) * 32;
    const QView &qv = proj ? g.b1 : g.b0;           // this wavefront's matrix stack
    const int col_last = ((n_out - 1) >> 5) << 5;
    const int col0 = col_raw < n_out ? col_raw : col_last;
    const bool store_on = col_raw + ln < n_out;
    int n = col0 + ln;
    if (n >= n_out) n = n_out - 1; // stay inside the matrix; such rows are never stored
    CS cs[NM];
#pragma unroll
    for (int mi = 0; mi < NM; ++mi) cs[mi].init(qv, e, col0 >> 5, ln, h, n);
    // GROUPED: byte offset of this lane's piece in load i of a group, from the matrix's first row. Piece c of row r
    // lands at position c ^ ((r >> 1) & 7) of the row's 128 bytes in LDS, so that the operand reads below (32 rows at
    // the same piece) spread over all banks; the lane simply fetches the piece that belongs at its position.
    uint32_t line_off[LG];
    const uint8_t *const wmat = qv.w + e * qv.w_mat;
    if (GROUPED) {
#pragma unroll
        for (int i = 0; i < LG; ++i) {
            const int r = 8 * i + (lane >> 3);
            int nr = col0 + r;
            if (nr >= n_out) nr = n_out - 1;
            line_off[i] = (uint32_t)nr * (uint32_t)qv.w_row + (uint32_t)(((lane & 7) ^ ((r >> 1) & 7)) * 16);
        }
    }
    // stage `step`: the chunk of reduction step `step`; GROUPED: load `step % 4` of group `step / 4` (i = step % 4 is
    // passed apart so that it stays a compile-time constant)
    auto load_stage = [&](int step, SkinnyStage<NM> &s, int i = 0) {
        if (GROUPED) {
            typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
            const u32x4_t v = __builtin_nontemporal_load((const u32x4_t *)(wmat + line_off[i] + (size_t)(step >> 2) * 128));
            s.raw[0] = make_uint4(v.x, v.y, v.z, v.w);
            return;
        }
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            s.raw[mi] = cs[mi].load_chunk_stream(step + sb0);
            if (!MBLK) cs[mi].load_meta(qv, step + sb0, s.sb[mi]);
        }
    };
    // ---- blocks of scale / bias entries (MBLK) -------------------------------------------------------------
    constexpr int kEntryBytes = Fmt::kMetaEntryBytes;                 // 2: bf16 scale + bf16 bias, 1: E8M0 scale
    constexpr int EPB = kEntryBytes ? 16 / kEntryBytes : 1;           // entries per 16-byte block
    const int last_block = MBLK ? (n_steps >> 3) - 1 : 0; // a block spans eight steps
    uint4 mblk_s[NM][2], mblk_b[NM][2]; // [.][0] in use, [.][1] requested for the steps after it
    auto load_mblock = [&](int block) {
        const int b = block < last_block ? block : last_block;
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            mblk_s[mi][1] = *(const uint4 *)(cs[mi].srow + (size_t)b * 16);
            mblk_b[mi][1] = cs[mi].brow ? *(const uint4 *)(cs[mi].brow + (size_t)b * 16) : make_uint4(0, 0, 0, 0);
        }
    };
    // Raw scale / bias entry of this lane for reduction step `gstep`, whose position in its block, `p8` = gstep % 8,
    // the caller knows at compile time (the launcher takes this path only when a block spans exactly eight steps, and
    // the unrolled rounds of the ring are whole multiples of eight). Steps must come in increasing order.
    auto mblock_meta = [&](int gstep, int p8, uint32_t (*sb)[2]) {
        if (p8 == 0) { // the step opens a block
#pragma unroll
            for (int mi = 0; mi < NM; ++mi) {
                mblk_s[mi][0] = mblk_s[mi][1];
                mblk_b[mi][0] = mblk_b[mi][1];
            }
            load_mblock((gstep >> 3) + 1);
        }
        // entries per step: one shared by both lane halves, or (groups of half a step) one for each half
        constexpr int EPS = EPB / 8;
        constexpr int per = 4 / (kEntryBytes ? kEntryBytes : 1); // entries per dword
        const int e0 = p8 * EPS, dw = e0 / per, sub = e0 - dw * per; // compile-time once unrolled
        const int shift = 8 * kEntryBytes * sub + (EPS == 2 ? 8 * kEntryBytes * h : 0);
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            const uint4 bs = mblk_s[mi][0], bb = mblk_b[mi][0];
            const uint32_t ws_ = dw == 0 ? bs.x : dw == 1 ? bs.y : dw == 2 ? bs.z : bs.w;
            const uint32_t wb_ = dw == 0 ? bb.x : dw == 1 ? bb.y : dw == 2 ? bb.z : bb.w;
            const uint32_t mask = kEntryBytes == 2 ? 0xffffu : 0xffu;
            sb[mi][0] = (ws_ >> shift) & mask;
            sb[mi][1] = (wb_ >> shift) & mask;
        }
    };

    // ---- activations of the tile in LDS -------------------------------------------------------------------
    // The LDS window holds 8 full rows' worth of activations. A tile of up to 8 rows (one row block, the bulk at
    // decode) keeps its rows whole; one of up to 16 (32) rows keeps a half (a quarter) of every row and is restaged
    // at the span boundaries, so that an expert with many rows still streams its weights only once. Only the rows
    // the tile has are staged: row m of the A operand only reaches accumulator row m, rows past the tile are never
    // stored. The matrix instruction always covers 32 rows; what grows with the tile is the number of accumulators
    // a lane scales and keeps (4 per row block), behind wave-uniform branches.
    const int nrows = __builtin_amdgcn_readfirstlane((int)t.nrows);
    const int rj = RJT == 1 ? 1 : nrows <= 2 * kSkinnyRowBlock ? 2 : 4; // row blocks = spans of the reduction
    const int rp = rj * kSkinnyRowBlock;             // rows the LDS layout is made for
    const int span_steps = n_steps / rj;             // the launcher only builds larger tiles when this divides
    const int span_bytes = span_steps * KSTEP * 2;   // bytes of one row in one span
    const int pitch = span_bytes + 16;               // +16 keeps neighbouring rows on different banks
    uint8_t *xs_lds = skinny_lds;
    float *gs_lds = (float *)(skinny_lds + kSkinnyRowBlock * cols * 2 + kSkinnyTileM * 16); // [span_steps][rp] sums of x
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)skinny_lds;
    // source rows of the tile: one load for all of them (lane r holds row r's), then uniform reads
    uint32_t src_of_lane = __builtin_amdgcn_readfirstlane(t.row0) + (uint32_t)(lane < nrows ? lane : 0);
    if (g.a_rows) src_of_lane = g.a_rows[src_of_lane];
    // requests span `span` of every row straight into LDS (no registers); completion is the caller's wait
    auto issue_x = [&](int span) {
        const int cpr = (span_bytes + 1023) >> 10; // 1 KiB operations per row
        const int ops = nrows * cpr;
        for (int o = wave; o < ops; o += WAVES) {
            const int r = o / cpr, c = (o - r * cpr) << 10;
            const size_t src = (uint32_t)__builtin_amdgcn_readlane((int)src_of_lane, r);
            const uint8_t *gp = (const uint8_t *)(g.a + src * (size_t)cols) + (size_t)span * span_bytes + c + lane * 16;
            const uint32_t la = lds_addr + (uint32_t)(r * pitch + c); // uniform; lane i lands at la + 16 i
            if (c + lane * 16 < span_bytes) {
                // nothing else in this kernel uses M0. A waiting consumer reads rows that workgroups on other XCDs
                // have just written with device-scope stores: its loads go past this XCD's L2 (sc1), no fence needed.
                if (sync == kSkinnySyncWait)
                    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off sc1" : : "v"(gp), "s"(la) : "memory");
                else
                    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gp), "s"(la) : "memory");
            }
        }
    };
    // factored form: per 16-byte piece (x0..x7) -> (x0,x4,x1,x5,x2,x6,x3,x7), the order the code pairs come out
    // in, and the sum of each step's 64 activations (eight pieces, eight neighbouring lanes)
    auto fix_x = [&]() {
        const int pieces = span_bytes >> 4;
        for (int idx = tid; idx < nrows * pieces; idx += WAVES * 64) {
            const int r = idx / pieces, pc = idx - r * pieces;
            uint4 *px = (uint4 *)(xs_lds + r * pitch + pc * 16);
            const uint4 v = *px;
            float sum = (bf16_bits_to_f32(v.x & 0xffffu) + bf16_bits_to_f32(v.x >> 16)) +
                        (bf16_bits_to_f32(v.y & 0xffffu) + bf16_bits_to_f32(v.y >> 16)) +
                        (bf16_bits_to_f32(v.z & 0xffffu) + bf16_bits_to_f32(v.z >> 16)) +
                        (bf16_bits_to_f32(v.w & 0xffffu) + bf16_bits_to_f32(v.w >> 16));
            uint4 o;
            o.x = (v.x & 0xffffu) | (v.z << 16);
            o.y = (v.x >> 16) | (v.z & 0xffff0000u);
            o.z = (v.y & 0xffffu) | (v.w << 16);
            o.w = (v.y >> 16) | (v.w & 0xffff0000u);
            *px = o;
            sum += skinny_dpp<0xB1>(sum);  // lane ^ 1 (quad_perm 1,0,3,2)
            sum += skinny_dpp<0x4E>(sum);  // lane ^ 2 (quad_perm 2,3,0,1)
            sum += skinny_dpp<0x141>(sum); // the other quad of the eight lanes (row_half_mirror)
            if ((pc & 7) == 0) gs_lds[(pc >> 3) * rp + r] = sum;
        }
    };

    SkinnyStage<NM> ring[STAGES];
    if (MBLK) load_mblock(0); // taken over by step 0, which requests block 1
    if (sync == kSkinnySyncWait) {
        // the activations are still being written: start the weight ring, then wait for the tile's producers (one
        // wavefront polls, the barrier holds the others), then fetch the rows
#pragma unroll
        for (int j = 0; j < PRE; ++j)
            if (j < n_loc) load_stage(j, ring[j], j % LG);
        if (wave == 0) {
            uint32_t polls = 0;
            while (__hip_atomic_load(&g.tile_done[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < g.tile_done_target &&
                   polls < g.spin_limit) {
                __builtin_amdgcn_s_sleep(8);
                ++polls;
            }
            // gave up: the launch still ends, the host learns about it from the workspace's counter
            if (polls >= g.spin_limit && lane == 0 && g.wait_expired &&
                __hip_atomic_load(&g.tile_done[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < g.tile_done_target)
                atomicAdd(g.wait_expired, 1u);
        }
        __syncthreads();
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) cs[mi].pin();
        issue_x(0);
        __builtin_amdgcn_s_waitcnt(skinny_wait_vmcnt(0));
    } else {
        // Loads return in issue order: the first span is requested ahead of the first stages of the weight ring, and
        // the wait below lets the ring stay in flight.
        issue_x(0);
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) cs[mi].pin(); // keeps the weight loads behind the requests above
#pragma unroll
        for (int j = 0; j < PRE; ++j)
            if (j < n_loc) load_stage(j, ring[j], j % LG);
        // every ring stage holds at least NM loads younger than the activation requests
        if (n_loc >= PRE) __builtin_amdgcn_s_waitcnt(skinny_wait_vmcnt(PRE * NM));
        else __builtin_amdgcn_s_waitcnt(skinny_wait_vmcnt(0));
    }
    __syncthreads();
    if (FACTORED) {
        fix_x();
        __syncthreads();
    }

    // A-operand source of this lane: tile row ln, reduction half h. Lanes past the tile's rows read row 0 again:
    // their operand rows only reach accumulator rows that are never stored.
    const uint8_t *xlane = xs_lds + (ln < nrows ? ln : 0) * pitch + h * KV * 2;
    const uint32_t mask = vgpr_const32(0x000f000fu), magic = vgpr_const32(0x43004300u);

    // accumulator registers 4 j + r of a lane belong to tile row 8 j + 4 h + r (row block j)
    {
        f32x16_t acc[NM];
#pragma unroll
        for (int mi = 0; mi < NM; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][r] = 0.0f;
        float facc[NM][4 * RJT];
#pragma unroll
        for (int mi = 0; mi < NM; ++mi)
#pragma unroll
            for (int r = 0; r < 4 * RJT; ++r) facc[mi][r] = 0.0f;

        // One step: decode every projection's chunk first, then issue the matrix instructions of the projections
        // alternately (independent accumulation chains), then apply the scales. `xs` = step within the span.
        auto consume = [&](int gstep, int p8, int xs, const SkinnyStage<NM> &s) {
            const uint8_t *xstep = xlane + (size_t)(xs + sb0) * KSTEP * 2;
            const float *gs_step = gs_lds + (xs + sb0) * rp + 4 * h;
            Meta meta[NM];
            if (MBLK) {
                uint32_t sbm[NM][2];
                mblock_meta(gstep, p8, sbm);
#pragma unroll
                for (int mi = 0; mi < NM; ++mi) meta[mi] = CS::meta(sbm[mi]);
            } else {
#pragma unroll
                for (int mi = 0; mi < NM; ++mi) meta[mi] = CS::meta(s.sb[mi]);
            }
            f32x16_t p[NM];
            if (FACTORED) {
                // word j of the chunk is exactly the B operand of the step's j-th matrix instruction: decode it
                // right before its use (the instructions of one projection are a dependent chain anyway), so only
                // one operand pair is live at a time
#pragma unroll
                for (int mi = 0; mi < NM; ++mi)
#pragma unroll
                    for (int r = 0; r < 16; ++r) p[mi][r] = 0.0f;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const uint4 xq = *(const uint4 *)(xstep + j * 16);
#pragma unroll
                    for (int mi = 0; mi < NM; ++mi) {
                        const uint32_t word = j == 0 ? s.raw[mi].x : j == 1 ? s.raw[mi].y : j == 2 ? s.raw[mi].z : s.raw[mi].w;
                        uint32_t wp[4];
                        codes_to_bf16(word, mask, magic, wp);
                        const uint4 q = make_uint4(wp[0], wp[1], wp[2], wp[3]);
                        p[mi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, xq), __builtin_bit_cast(bf16x8_t, q), p[mi], 0, 0, 0);
                    }
                }
            } else {
                bf16x8_t xf[NJ];
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    uint4 q = *(const uint4 *)(xstep + j * 16);
                    xf[j] = __builtin_bit_cast(bf16x8_t, q);
                }
                uint32_t wp[NM][KV / 2];
#pragma unroll
                for (int mi = 0; mi < NM; ++mi) Fmt::decode_fast(s.raw[mi], meta[mi], wp[mi]);
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
#pragma unroll
                    for (int mi = 0; mi < NM; ++mi) {
                        uint4 q = make_uint4(wp[mi][4 * j], wp[mi][4 * j + 1], wp[mi][4 * j + 2], wp[mi][4 * j + 3]);
                        acc[mi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[j], __builtin_bit_cast(bf16x8_t, q), acc[mi], 0, 0, 0);
                    }
                }
            }
            if (FACTORED) {
#pragma unroll
                for (int mi = 0; mi < NM; ++mi) {
                    const float boff = fmaf(-128.0f, meta[mi].s, meta[mi].b);
#pragma unroll
                    for (int j = 0; j < RJT; ++j) {
                        const float4 gsum = *(const float4 *)(gs_step + 8 * j); // past the tile's row blocks: stale sums, unused rows
                        facc[mi][4 * j + 0] = fmaf(meta[mi].s, p[mi][4 * j + 0], fmaf(boff, gsum.x, facc[mi][4 * j + 0]));
                        facc[mi][4 * j + 1] = fmaf(meta[mi].s, p[mi][4 * j + 1], fmaf(boff, gsum.y, facc[mi][4 * j + 1]));
                        facc[mi][4 * j + 2] = fmaf(meta[mi].s, p[mi][4 * j + 2], fmaf(boff, gsum.z, facc[mi][4 * j + 2]));
                        facc[mi][4 * j + 3] = fmaf(meta[mi].s, p[mi][4 * j + 3], fmaf(boff, gsum.w, facc[mi][4 * j + 3]));
                    }
                }
            }
            // with 16 products per lane alive, letting the next step's matrix instructions start before this step's
            // scaling has finished would double them: keep the steps apart (other wavefronts fill the wait)
            if ((RJT > 1 && FACTORED) || GROUPED) __builtin_amdgcn_sched_barrier(0);
        };

        // GROUPED: ring stages j .. j+3 (one group as loaded) -> the chunks of its four steps in the operand layout
        uint8_t *const turn_lds = skinny_lds + skinny_turn_offset(cols, KSTEP) + wave * (LG * 1024);
        const uint8_t *const turn_rd = turn_lds + ln * 128;
        const int turn_sw = (ln >> 1) & 7;
        uint4 turned_raw[LG];
        SkinnyStage<NM> turned;
        // A group is written one group ahead of its use, right behind the reads of the group before it (same
        // buffer: the reads have been issued, and the LDS keeps a wavefront's operations in order), so the reads at
        // the head of a group never wait for their own writes.
        auto turn_write = [&](int j) {
#pragma unroll
            for (int i = 0; i < LG; ++i) *(uint4 *)(turn_lds + i * 1024 + lane * 16) = ring[j + i].raw[0];
        };
        auto turn_read = [&]() {
#pragma unroll
            for (int jj = 0; jj < LG; ++jj) turned_raw[jj] = *(const uint4 *)(turn_rd + (((2 * jj + h) ^ turn_sw) * 16));
        };
        if (GROUPED) {
            turn_write(0);
#pragma unroll
            for (int i = 0; i < LG; ++i) // the stages of group 0 are free again: the group one round on
                load_stage(STAGES + i < n_loc ? STAGES + i : n_loc - LG + i, ring[i], i);
        }

        // Whole rounds of the ring run without guards, the rest in a guarded copy. Tiles of one row block end their
        // unguarded rounds where the look-ahead would pass the last step (LEAN_TAIL: no chunk is requested twice - the
        // repeated requests of a look-ahead clamped onto the last step, one per ring stage and wavefront, were a tenth
        // of a 64-step wavefront's loads); larger tiles need whole rounds per span and clamp instead.
        constexpr bool LEAN_TAIL = RJT == 1 && !GROUPED;
        const int full = LEAN_TAIL ? (n_loc > PRE ? (n_loc - PRE) / ROUND * ROUND : 0) : n_loc / ROUND * ROUND;
        int x0 = 0, next_span = span_steps; // first step of the span in LDS, first step of the next one
#pragma unroll 1
        for (int s0 = 0; s0 < full; s0 += ROUND) {
            if (RJT > 1 && s0 == next_span) {
                // the next span of the activations replaces the one in LDS (the weight ring stays in flight; its
                // loads are older than these requests, so the wait covers nothing that was not due anyway)
                __syncthreads();
                issue_x(s0 / span_steps);
                __builtin_amdgcn_s_waitcnt(skinny_wait_vmcnt(0));
                __syncthreads();
                if (FACTORED) {
                    fix_x();
                    __syncthreads();
                }
                x0 = s0;
                next_span += span_steps;
            }
#pragma unroll
            for (int j = 0; j < ROUND; ++j) {
                const int step = s0 + j, ahead = step + PRE;
                if (GROUPED) {
                    if (j % LG == 0) {
                        turn_read();
                        turn_write((j + LG) % STAGES); // the next group; its stages then take the loads a round later
#pragma unroll
                        for (int i = 0; i < LG; ++i) // past the end: the last group again (unused)
                            load_stage(ahead + LG + i < n_loc ? ahead + LG + i : n_loc - LG + i, ring[(j + LG) % STAGES + i], i);
                    }
                    turned.raw[0] = turned_raw[j % LG];
                    consume(step, j & 7, step - x0, turned);
                    continue;
                }
                load_stage(LEAN_TAIL || ahead < n_loc ? ahead : n_loc - 1, ring[(j + PRE) % STAGES]);
                consume(step, j & 7, step - x0, ring[j % STAGES]);
            }
        }
#pragma unroll 1
        for (int t0 = full; RJT == 1 && t0 < n_loc; t0 += ROUND) { // only tiles of one row block get here
#pragma unroll
            for (int j = 0; j < ROUND; ++j) {
                const int step = t0 + j;
                if (GROUPED) { // the reduction is a whole number of groups, and everything left is already in the ring
                    if (step < n_loc) {
                        if (j % LG == 0) {
                            turn_read();
                            if (step + LG < n_loc) turn_write((j + LG) % STAGES);
                        }
                        turned.raw[0] = turned_raw[j % LG];
                        consume(step, j & 7, step, turned);
                    }
                    continue;
                }
                if (step + PRE < n_loc) load_stage(step + PRE, ring[(j + PRE) % STAGES]);
                if (step < n_loc) consume(step, j & 7, step, ring[j % STAGES]);
            }
        }

        // ---- epilogue: this lane holds rows 8 j + 4 h + r of the tile for weight row n ----------------------
        float v[2][4 * RJT];
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            const float rs = Fmt::kRowScale ? *(const float *)(qv.scales + e * qv.s_mat + (size_t)n * qv.s_row) : 1.0f;
#pragma unroll
            for (int r = 0; r < 4 * RJT; ++r) v[mi][r] = (FACTORED ? facc[mi][r] : acc[mi][r]) * rs;
        }
        if (ks) { // the second half of the reduction joins the first (RJT == 1 here: four values per lane)
            float4 *kx = (float4 *)xs_lds + 256 * RJT + wq * 64 + lane; // bytes 4096 .. 8191, behind the gate/up exchange area below
            __syncthreads(); // every wavefront has left the main loop: the activation window is free
            if (kh == 1) kx[0] = make_float4(v[0][0], v[0][1], v[0][2], v[0][3]);
            __syncthreads();
            if (kh == 0) {
                const float4 u = kx[0];
                v[0][0] += u.x, v[0][1] += u.y, v[0][2] += u.z, v[0][3] += u.w;
            }
        }
        if (gate_up) {
            // the up wavefront hands its values to the gate wavefront of the same weight rows, through the
            // activation window (free once every wavefront has left the main loop)
            float4 *xch = (float4 *)xs_lds + ((wq >> 1) * 64 + lane) * RJT;
            __syncthreads();
            if (proj == 1 && kh == 0) {
#pragma unroll
                for (int j = 0; j < RJT; ++j) xch[j] = make_float4(v[0][4 * j], v[0][4 * j + 1], v[0][4 * j + 2], v[0][4 * j + 3]);
            }
            __syncthreads();
            if (proj == 0) {
#pragma unroll
                for (int j = 0; j < RJT; ++j) {
                    const float4 u = xch[j];
                    v[1][4 * j] = u.x, v[1][4 * j + 1] = u.y, v[1][4 * j + 2] = u.z, v[1][4 * j + 3] = u.w;
                }
            }
        }
        const bool storer = store_on && proj == 0 && kh == 0;
        const float swiglu_limit = (t.flags & kTileDense) ? g.swiglu_limit_dense : g.swiglu_limit;
        // A lane holds ONE column of up to 16 rows: stored from here that is a 2-byte store per row and lane, and a
        // tile of 32 rows spent 6-7 us of its workgroup's life on them. Instead the values go to LDS (behind the
        // exchange areas) and leave as 8-byte pieces of a row, one or two per thread. Output rows that cannot be cut
        // into such pieces keep the direct stores.
        const bool wide_out = (n_out & 3) == 0 && (g.ldo & 3) == 0 && ((uintptr_t)g.out & 7) == 0;
        const int cw_shift = (gate_up ? 7 : 8) - (ks ? 1 : 0); // log2 of the workgroup's output columns
        uint16_t *const stage = (uint16_t *)(skinny_lds + kSkinnyStageOffset); // [tile rows][columns of the workgroup]
        if (wide_out && !gate_up && !ks) __syncthreads(); // (the other roles have met at a barrier since the main loop)
#pragma unroll
        for (int j = 0; j < RJT; ++j) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 8 * j + 4 * h + r;
                if (proj != 0 || kh != 0 || i >= nrows || (!wide_out && !storer)) continue;
                const uint32_t p = t.row0 + (uint32_t)i;
                float val = gate_up ? limited_swiglu(v[0][4 * j + r], v[1][4 * j + r], swiglu_limit) : v[0][4 * j + r];
                if (g.row_scale && p < g.row_scale_rows) val *= g.row_scale[g.row_scale_idx ? g.row_scale_idx[p] : p];
                if (wide_out) {
                    stage[(i << cw_shift) + (gate_up ? wq >> 1 : wq) * 32 + ln] = f32_to_bf16_bits(val);
                    continue;
                }
                const size_t dst = g.out_rows ? g.out_rows[p] : p;
                // a producer's rows are read by workgroups on other XCDs within the same launch: device-scope
                // stores (written through this XCD's L2), so no cache-wide write-back is needed before the signal
                if (sync == kSkinnySyncSignal)
                    __hip_atomic_store(&g.out[dst * (size_t)g.ldo + n], f32_to_bf16_bits(val), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else
                    g.out[dst * (size_t)g.ldo + n] = f32_to_bf16_bits(val);
            }
        }
        if (wide_out) {
            __syncthreads();
            const int pp_shift = cw_shift - 2;                     // 4-column pieces per row
            const int strip0 = (int)blockIdx.x << cw_shift;        // the workgroup's first output column
            for (int idx = tid; idx < (nrows << pp_shift); idx += WAVES * 64) {
                const int r = idx >> pp_shift, c = (idx - (r << pp_shift)) * 4;
                if (strip0 + c >= n_out) continue;                 // a strip that ends past the matrix
                const uint32_t p = t.row0 + (uint32_t)r;
                const size_t dst = g.out_rows ? g.out_rows[p] : p;
                const uint64_t d = *(const uint64_t *)(stage + (r << cw_shift) + c);
                uint64_t *o = (uint64_t *)(g.out + dst * (size_t)g.ldo + strip0 + c);
                if (sync == kSkinnySyncSignal) __hip_atomic_store(o, d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else *o = d;
            }
        }
        if (sync == kSkinnySyncSignal) {
            __builtin_amdgcn_s_waitcnt(skinny_wait_vmcnt(0)); // this wavefront's stores have reached memory ...
            __syncthreads();                                   // ... and every other wavefront's of the workgroup ...
            if (tid == 0) __hip_atomic_fetch_add(&g.tile_done[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // ... before this
        }
    }
}

// `paired` = 0: one GEMM (`a`). `paired` = 1: gate/up (`a`) and down (`b`) of one tile list in one launch: workgroups
// y < a.max_tiles are the gate/up tiles, the next a.max_tiles the down tiles of the same list. The hardware starts
// workgroups in index order, so every producer of a tile is running or done by the time a consumer of it starts to
// wait; the down workgroups that become resident while the last gate/up workgroups drain stream their weights meanwhile.
template <typename Fmt, bool FACTORED, bool PACKED, bool MBLK = false, bool KSPLIT = false>
__global__ __launch_bounds__(2 * kSkinnyWaves * 64) void qgemm_skinny_kernel(GemmArgs a, GemmArgs b, int paired) {
    extern __shared__ __attribute__((aligned(16))) uint8_t skinny_lds[];
    const bool second = paired && blockIdx.y >= (uint32_t)a.max_tiles; // workgroup-uniform
    // The role's arguments, read from the kernel-argument segment with a uniform index (`a` sits at offset 0 and `b`
    // right behind it): taking the address of `a` or `b` instead would move both structs to scratch memory.
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const __attribute__((address_space(4))) GemmArgs *KernArgs;
    const GemmArgs g = ((KernArgs)__builtin_amdgcn_kernarg_segment_ptr())[second ? 1 : 0];
#else
    const GemmArgs g = a; // host pass of the compiler: never runs
#endif
    (void)b;
    const uint32_t slot = blockIdx.y - (second ? (uint32_t)a.max_tiles : 0u);
    const int sync = !paired ? kSkinnySyncNone : second ? kSkinnySyncWait : kSkinnySyncSignal;
    if ((int)blockIdx.x * (g.gate_up ? 1 : 2) * kSkinnyWaves * 32 >= (KSPLIT ? 2 : 1) * g.b0.rows) return; // the grid is sized for the wider role
    Tile t;
    if (g.tiles) {
        const uint32_t n_tiles = *g.n_tiles; // both loads are issued before either is needed
        t = g.tiles[slot];                   // the list has room for every launched slot
        if (slot >= n_tiles) return;
        if ((int)t.nrows > g.max_rows) return; // a list built for the matrix-core kernels: those take the larger tiles
    } else {
        t.expert = 0;
        t.flags = 0;
        t.row0 = slot * (uint32_t)g.tile_m;
        if ((int)t.row0 >= g.dense_rows) return;
        uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)g.tile_m ? left : (uint32_t)g.tile_m;
    }
    if (KSPLIT) { // the launcher builds no tile above one row block for this kernel
        skinny_tile<Fmt, FACTORED, PACKED, 1, MBLK, KSPLIT>(g, t, skinny_lds, g.gate_up, sync, slot);
        return;
    }
    if (__builtin_amdgcn_readfirstlane((int)t.nrows) <= kSkinnyRowBlock)
        skinny_tile<Fmt, FACTORED, PACKED, 1, MBLK>(g, t, skinny_lds, g.gate_up, sync, slot);
    else
        skinny_tile<Fmt, FACTORED, PACKED, kSkinnyTileM / kSkinnyRowBlock, MBLK>(g, t, skinny_lds, g.gate_up, sync, slot);
}

static int skinny_vals(const QView &b) {
    if (b.mode == DMOE_QUANT_NONE) return 8;
    return (b.mode == DMOE_QUANT_AFFINE && b.bits == 4) || b.mode == DMOE_QUANT_MXFP4 ? 32 : 16;
}
static size_t skinny_lds_bytes(const QView &b) {
    // a two-row-block tile reads (and ignores) up to 24 floats past its last step's sums: the 128 bytes in the offset.
    // At least 32 KiB: once the main loop is done the wavefronts exchange their sums through the start of the window
    // (gate/up pairs: 4 KiB per row block of the tile, up to 16 KiB; split reduction: bytes 4096 .. 8191) and gather
    // the tile's outputs behind that (up to 32 rows of 256 columns), which a short reduction dimension would not cover.
    return std::max(skinny_turn_offset(b.cols, 2 * skinny_vals(b)), kSkinnyStageOffset + kSkinnyStageBytes);
}

// Rows per tile to build tile lists with for this weight shape: a tile of 2 (4) row blocks splits the reduction
// into 2 (4) spans, each a whole number of ring rounds.
int qgemm_skinny_tile_m(const QView &b) {
    const int n_steps = b.cols / (2 * skinny_vals(b));
    if (n_steps % (4 * kSkinnyStages) == 0) return 4 * kSkinnyRowBlock;
    if (n_steps % (2 * kSkinnyStages) == 0) return 2 * kSkinnyRowBlock;
    return kSkinnyRowBlock;
}

bool qgemm_skinny_supports(const QView &b) {
    // unquantized weights: resident (re-ordered) stacks only, whole 32-row blocks
    if (b.mode == DMOE_QUANT_NONE && !(b.packed && b.rows % 32 == 0 && ((uintptr_t)b.w % 16) == 0)) return false;
    return b.cols % (2 * skinny_vals(b)) == 0 && skinny_lds_bytes(b) <= 150 * 1024;
}

// GemmArgs::ksplit needs the packed layout, two halves of the reduction that are whole ring rounds and start on a
// group boundary
bool qgemm_skinny_ksplit_ok(const QView &b) {
    if (!qgemm_skinny_supports(b) || !b.packed) return false;
    const int n_steps = b.cols / (2 * skinny_vals(b));
    if (n_steps % (2 * kSkinnyStages) != 0) return false;
    return b.group <= 0 || (b.cols / 2) % b.group == 0;
}

// rows of scales (and biases) that are 16-byte aligned and a whole number of 16-byte blocks long
static bool mlx_meta_blocks(const QView &b) {
    if (b.packed || b.group <= 0 || !b.scales) return false;
    const size_t esz = b.mode == DMOE_QUANT_MXFP4 ? 1 : 2, row = (size_t)(b.cols / b.group) * esz;
    if (b.mode != DMOE_QUANT_MXFP4 && b.mode != DMOE_QUANT_AFFINE) return false;
    // a block of entries must span exactly eight reduction steps (affine 4-bit: groups of 64; MXFP4: 32; 8-bit: 32)
    const int kstep = b.bits == 4 ? 64 : 32;
    if ((int)(16 / esz) * b.group != 8 * kstep) return false;
    if (skinny_lds_bytes(b) + kSkinnyTurnBytes > 150 * 1024 || b.w_row % 128 != 0 || ((uintptr_t)b.w % 16) != 0 || b.w_mat % 16 != 0 ||
        (uint64_t)b.rows * (uint64_t)b.w_row >= (1ull << 32))
        return false; // the line-wise weight loads of the small tiles: LDS to turn them in, whole lines per group
    return row >= 16 && row % 16 == 0 && b.s_row % 16 == 0 && b.s_mat % 16 == 0 && ((uintptr_t)b.scales % 16) == 0 &&
           (!b.biases || ((uintptr_t)b.biases % 16) == 0);
}

template <typename Fmt, bool FACTORED, bool PACKED, bool MBLK, bool KSPLIT = false>
static int skinny_raise_limit() {
    static LdsLimit limit; // per instantiation
    return raise_lds_limit(limit, (const void *)qgemm_skinny_kernel<Fmt, FACTORED, PACKED, MBLK, KSPLIT>, 150 * 1024);
}
// the instantiations SkinnyLaunch can pick for one format
template <typename Fmt>
static int skinny_prepare_format() {
    constexpr bool can_factor = std::is_same<Fmt, FmtAffine4>::value;
    constexpr bool has_entries = Fmt::kMetaEntryBytes != 0;
    DMOE_TRY((skinny_raise_limit<Fmt, can_factor, true, false>()));
    DMOE_TRY((skinny_raise_limit<Fmt, false, true, false>()));
    DMOE_TRY((skinny_raise_limit<Fmt, can_factor, true, false, true>()));
    DMOE_TRY((skinny_raise_limit<Fmt, false, true, false, true>()));
    DMOE_TRY((skinny_raise_limit<Fmt, can_factor, false, has_entries>()));
    DMOE_TRY((skinny_raise_limit<Fmt, false, false, has_entries>()));
    DMOE_TRY((skinny_raise_limit<Fmt, can_factor, false, false>()));
    return skinny_raise_limit<Fmt, false, false, false>();
}
int qgemm_skinny_prepare() {
    DMOE_TRY((skinny_raise_limit<FmtBf16, false, true, false>()));
    DMOE_TRY((skinny_raise_limit<FmtBf16, false, true, false, true>()));
    DMOE_TRY(skinny_prepare_format<FmtAffine4>());
    DMOE_TRY(skinny_prepare_format<FmtAffine8>());
    DMOE_TRY(skinny_prepare_format<FmtMxfp4>());
    return skinny_prepare_format<FmtFp8Row>();
}

struct SkinnyLaunch {
    const GemmArgs &g;
    hipStream_t st;
    const GemmArgs *second = nullptr; // paired launch: the down projection behind the gate/up GEMM `g`
    template <typename Fmt, bool FACTORED, bool PACKED, bool MBLK = false, bool KSPLIT = false>
    int go() {
        if constexpr (PACKED && !MBLK && !KSPLIT) {
            if (g.ksplit) return go<Fmt, FACTORED, PACKED, MBLK, true>(); // validated by the launch functions
        }
        auto kern = qgemm_skinny_kernel<Fmt, FACTORED, PACKED, MBLK, KSPLIT>;
        const size_t lds = skinny_lds_bytes(g.b0) + (MBLK ? kSkinnyTurnBytes : 0);
        DMOE_TRY((skinny_raise_limit<Fmt, FACTORED, PACKED, MBLK, KSPLIT>())); // done by dmoe_init for its device; a flag test otherwise
        // 8 wavefronts per workgroup: 128 output columns of gate AND up, or 256 of a single projection
        auto blocks_x = [](const GemmArgs &a) { return ceil_div((a.ksplit ? 2 : 1) * a.b0.rows, (a.gate_up ? 1 : 2) * kSkinnyWaves * 32); };
        dim3 block(2 * kSkinnyWaves * 64);
        if (second) {
            GemmArgs a = g, b = *second;
            a.tile_done_target = b.tile_done_target = (uint32_t)blocks_x(g);
            b.tile_done = a.tile_done;
            const size_t lds2 = std::max(lds, skinny_lds_bytes(second->b0) + (MBLK ? kSkinnyTurnBytes : 0));
            dim3 grid((unsigned)std::max(blocks_x(a), blocks_x(b)), (unsigned)(2 * g.max_tiles));
            hipLaunchKernelGGL(kern, grid, block, lds2, st, a, b, 1);
        } else {
            dim3 grid((unsigned)blocks_x(g), (unsigned)g.max_tiles);
            hipLaunchKernelGGL(kern, grid, block, lds, st, g, g, 0);
        }
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    template <typename Fmt>
    int operator()() {
        // the scale can be factored out of the matrix product when both halves of a step share a group
        constexpr bool can_factor = std::is_same<Fmt, FmtAffine4>::value;
        const bool factor = can_factor && g.b0.group >= 64;
        if (g.b0.packed) return factor ? go<Fmt, can_factor, true>() : go<Fmt, false, true>();
        // MLX layout: scale / bias entries in 16-byte blocks when every row of them is a whole number of blocks
        constexpr bool has_entries = Fmt::kMetaEntryBytes != 0;
        if (has_entries && mlx_meta_blocks(g.b0) && (!second || mlx_meta_blocks(second->b0)) && (!g.gate_up || mlx_meta_blocks(g.b1)))
            return factor ? go<Fmt, can_factor, false, has_entries>() : go<Fmt, false, false, has_entries>();
        return factor ? go<Fmt, can_factor, false>() : go<Fmt, false, false>();
    }
};

static bool skinny_factored(const QView &b) { return b.mode == DMOE_QUANT_AFFINE && b.bits == 4 && b.group >= 64; }

bool qgemm_skinny_pair_supports(const GemmArgs &gu, const GemmArgs &dn) {
    const QView &a = gu.b0, &b = dn.b0;
    return gu.gate_up && !dn.gate_up && gu.tiles && gu.tiles == dn.tiles && gu.n_tiles == dn.n_tiles &&
           gu.max_tiles == dn.max_tiles && gu.max_tiles > 0 && 2 * (long)gu.max_tiles <= 65535 &&
           a.packed == b.packed && a.mode == b.mode && a.bits == b.bits && skinny_factored(a) == skinny_factored(b) &&
           qgemm_skinny_supports(a) && qgemm_skinny_supports(b) && std::min(gu.tile_m, gu.max_rows) <= qgemm_skinny_tile_m(a) &&
           std::min(dn.tile_m, dn.max_rows) <= qgemm_skinny_tile_m(b) && gu.max_rows == dn.max_rows &&
           gu.tile_done != nullptr && dn.a == gu.out;
}

int launch_qgemm_skinny_pair(const GemmArgs &gu, const GemmArgs &dn, hipStream_t st) {
    DMOE_REQUIRE(qgemm_skinny_pair_supports(gu, dn), "skinny GEMM pair: arguments do not form a gate/up + down pair");
    DMOE_REQUIRE(!gu.ksplit && !dn.ksplit, "skinny GEMM pair: the split reduction is for single launches (steps of a few rows run as two)");
    DMOE_REQUIRE(gu.a && gu.out && dn.out && ((uintptr_t)gu.a % 16) == 0 && ((uintptr_t)dn.a % 16) == 0, "skinny GEMM pair: bad pointer");
    DMOE_REQUIRE(gu.b1.rows == gu.b0.rows && gu.b1.cols == gu.b0.cols && gu.b1.mode == gu.b0.mode && gu.b1.bits == gu.b0.bits &&
                     gu.b1.group == gu.b0.group && gu.b1.packed == gu.b0.packed,
                 "skinny GEMM pair: gate and up projections differ in shape or format");
    SkinnyLaunch l{gu, st};
    l.second = &dn;
    if (gu.b0.mode == DMOE_QUANT_NONE) return l.template go<FmtBf16, false, true>();
    return dispatch_format(gu.b0, l);
}

int launch_qgemm_skinny(const GemmArgs &g, hipStream_t st) {
    DMOE_REQUIRE(qgemm_skinny_supports(g.b0), "skinny GEMM: unsupported weight shape (cols=%d)", g.b0.cols);
    DMOE_REQUIRE(g.max_tiles >= 0 && g.max_tiles <= 65535, "skinny GEMM: %d tiles exceed the grid limit", g.max_tiles);
    DMOE_REQUIRE(g.a && g.out && g.ldo > 0 && ((uintptr_t)g.a % 16) == 0, "skinny GEMM: bad pointer");
    DMOE_REQUIRE(g.tile_m > 0 && std::min(g.tile_m, g.max_rows) <= qgemm_skinny_tile_m(g.b0),
                 "skinny GEMM: tiles of %d rows, this shape takes %d", std::min(g.tile_m, g.max_rows), qgemm_skinny_tile_m(g.b0));
    if (g.gate_up)
        DMOE_REQUIRE(g.b1.rows == g.b0.rows && g.b1.cols == g.b0.cols && g.b1.mode == g.b0.mode &&
                         g.b1.bits == g.b0.bits && g.b1.group == g.b0.group && g.b1.packed == g.b0.packed,
                     "skinny GEMM: gate and up projections differ in shape or format");
    DMOE_REQUIRE(!g.ksplit || (g.tile_m <= kSkinnyRowBlock && qgemm_skinny_ksplit_ok(g.b0) && (!g.gate_up || qgemm_skinny_ksplit_ok(g.b1))),
                 "skinny GEMM: a split reduction needs packed weights and tiles of at most %d rows", kSkinnyRowBlock);
    if (g.max_tiles == 0) return DMOE_OK;
    if (g.b0.mode == DMOE_QUANT_NONE) return SkinnyLaunch{g, st}.template go<FmtBf16, false, true>();
    return dispatch_format(g.b0, SkinnyLaunch{g, st});
}

} // namespace dmoe
