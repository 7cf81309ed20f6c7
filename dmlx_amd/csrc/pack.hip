// Token -> expert packing: a stable counting sort of the T*K routed expert ids.
//
// Each wavefront owns a contiguous sub-chunk of the flat (t*K+k) index space. Phase 1 builds one LDS
// histogram per sub-chunk; phase 2 turns the [sub-chunk][expert] counts into starting offsets (exclusive
// scan over sub-chunks inside each expert, then over experts) and emits counts / segment offsets / the
// tile list / the list of live experts; phase 3 re-reads the ids and places every row at
// base[sub-chunk][expert] + (number of earlier lanes with the same expert), found with ballots, so rows
// of one expert keep ascending flat index. No global atomics; the result is deterministic.
//
// Up to 1024 rows everything runs in ONE launch (16 wavefronts x 64 rows); above that in three.
#include "common.h"
#include "route_device.h"

namespace dmoe {

constexpr int kPackThreads = 1024;              // scan / fused kernels: one expert per thread
constexpr int kPackWaves = kPackThreads / 64;   // 16
constexpr int kSubGroups = 4;                   // multi-launch path: groups of 64 rows per wavefront
constexpr int kSubRows = 64 * kSubGroups;       // 256 rows per sub-chunk
constexpr int kScatterWaves = 4;                // wavefronts per block in the multi-launch path
constexpr uint32_t kPackSmallTileRows = 8;      // tiles of at most this many rows go behind the larger ones in the tile list

// one step of a wavefront-wide prefix sum: v += the value `CTRL` selects (0 where it selects nothing or the row is masked)
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t scan_dpp_step(uint32_t v) {
    return v + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
// inclusive prefix sum inside each row of 16 lanes
__device__ __forceinline__ uint32_t row_incl_scan(uint32_t v) {
    v = scan_dpp_step<0x111, 0xf>(v); // row_shr:1
    v = scan_dpp_step<0x112, 0xf>(v); // row_shr:2
    v = scan_dpp_step<0x114, 0xf>(v); // row_shr:4
    v = scan_dpp_step<0x118, 0xf>(v); // row_shr:8
    return v;
}
// inclusive prefix sum over the 64 lanes (all of them active)
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v) {
    v = row_incl_scan(v);
    v = scan_dpp_step<0x142, 0xa>(v); // row_bcast:15 into rows 1 and 3: the total of the row before
    v = scan_dpp_step<0x143, 0xc>(v); // row_bcast:31 into rows 2 and 3: the total of rows 0 and 1
    return v;
}

// exclusive scans of NV values per thread across a 1024-thread block in one pass; total[k] gets the block sums.
// One barrier: every wavefront adds up the 16 wavefront totals for itself. `sm` holds kPackWaves * NV words that nothing
// else touches (a kernel scans once).
template <int NV>
__device__ __forceinline__ void block_excl_scan(const uint32_t (&v)[NV], uint32_t (&excl)[NV], uint32_t (&total)[NV],
                                                uint32_t *sm) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t incl[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        incl[k] = wave_incl_scan(v[k]);
        if (lane == 63) sm[wave * NV + k] = incl[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const uint32_t t = row_incl_scan(lane < kPackWaves ? sm[lane * NV + k] : 0u); // lanes 0..15 = one row
        const uint32_t upto = (uint32_t)__builtin_amdgcn_readlane((int)t, wave);      // wavefronts 0..wave
        const uint32_t mine = (uint32_t)__builtin_amdgcn_readlane((int)incl[k], 63);  // this wavefront's total
        total[k] = (uint32_t)__builtin_amdgcn_readlane((int)t, kPackWaves - 1);
        excl[k] = upto - mine + incl[k] - v[k];
    }
}

// lanes of this wavefront that hold the same expert id (only among `active` lanes)
__device__ __forceinline__ uint64_t match_expert(uint32_t e, bool active, int nbits) {
    uint64_t peers = __ballot(active);
    for (int b = 0; b < nbits; ++b) {
        bool bit = (e >> b) & 1u;
        uint64_t bal = __ballot(active && bit);
        peers &= bit ? bal : ~bal;
    }
    return peers;
}

// the id as it is packed: through the optional slot map
__device__ __forceinline__ uint32_t packed_id(const PackOut &o, uint32_t e) {
    if (!o.remap) return e;
    return e < o.n_remap ? (uint32_t)o.remap[e] : 0u;
}

__device__ __forceinline__ int log2_ceil(int E) {
    int b = 0;
    while ((1 << b) < E) ++b;
    return b;
}

// phase 2 body shared by the fused and the stand-alone scan kernel. `count` is this thread's expert total.
__device__ uint32_t emit_segments(uint32_t count, int e, int E, size_t n, int tile_m, const PackOut &o,
                                  uint32_t *sm /*[4 * kPackWaves]*/) {
    // Tiles above kPackSmallTileRows rows first, then the rest, each group in expert order. On the decode path a
    // large tile takes about twice as long as a small one (it restages its activations on the way), so the few
    // of them start with the launch instead of stretching its tail. (Splitting further - full tiles of all experts
    // first, then the partial ones - measured 2-3 % slower at prefill: a partial tile then runs far from its
    // expert's full tiles and finds none of the weights in L2.)
    const uint32_t tm = tile_m > 0 ? (uint32_t)tile_m : 1u;
    const uint32_t nt = tile_m > 0 ? (count + tm - 1) / tm : 0u;
    const uint32_t last_rows = count - (nt ? (nt - 1) * tm : 0);           // rows of the expert's last tile
    const uint32_t n_big = nt == 0 ? 0 : (nt - 1) + (last_rows > kPackSmallTileRows ? 1u : 0u);
    // everything below depends on the expert's count only: segment start, rank among the live experts, first large
    // and first small tile come out of one scan
    const uint32_t in[4] = {count, count > 0 ? 1u : 0u, n_big, nt - n_big};
    uint32_t ex[4], tot[4];
    block_excl_scan<4>(in, ex, tot, sm);
    const uint32_t off = ex[0];
    if (e < E) {
        if (o.counts) o.counts[e] = count;
        if (o.offsets) o.offsets[e] = off;
    }
    if (e == 0 && o.offsets) o.offsets[E] = (uint32_t)n;
    if (count > 0 && o.live) o.live[ex[1]] = (uint32_t)e;
    if (e == 0 && o.n_live) *o.n_live = tot[1];
    for (uint32_t i = threadIdx.x; i < o.n_done; i += blockDim.x) o.tile_done[i] = 0;
    // the folded always-on expert: identity rows behind the routed ones, its tiles ahead of the routed tiles
    const uint32_t nt_dense = (o.dense_rows + tm - 1) / tm;
    for (uint32_t i = threadIdx.x; i < o.dense_rows; i += blockDim.x) {
        o.order[n + i] = (uint32_t)n + i;
        if (o.token) o.token[n + i] = i;
        if (o.sorted_e) o.sorted_e[n + i] = o.dense_expert;
    }
    if (tile_m > 0 && o.tiles) {
        for (uint32_t j = threadIdx.x; j < nt_dense; j += blockDim.x) {
            Tile t;
            t.expert = o.dense_expert;
            t.row0 = (uint32_t)n + j * tm;
            uint32_t left = o.dense_rows - j * tm;
            t.nrows = left < tm ? left : tm;
            t.flags = kTileDense;
            o.tiles[j] = t;
        }
        const uint32_t total_big = tot[2];
        for (uint32_t j = 0; j < nt; ++j) {
            Tile t;
            t.expert = (uint32_t)e;
            t.row0 = off + j * tm;
            uint32_t left = count - j * tm;
            t.nrows = left < tm ? left : tm;
            t.flags = 0;
            const uint32_t pos = j < n_big ? ex[2] + j : total_big + ex[3];
            o.tiles[nt_dense + pos] = t;
        }
        if (e == 0 && o.n_tiles) *o.n_tiles = nt_dense + tot[2] + tot[3];
    }
    return off;
}

__device__ __forceinline__ void place_row(const PackOut &o, uint32_t pos, uint32_t i, uint32_t e, int K) {
    o.order[pos] = i;
    if (o.inv) o.inv[i] = pos;
    if (o.token) o.token[pos] = i / (uint32_t)K;
    if (o.sorted_e) o.sorted_e[pos] = e;
}

// ---- one launch, n <= 1024 ---------------------------------------------------------------------------------
// `e` = this thread's expert id (row i = tid), `pack_sm` = hist[kPackWaves][E] in LDS
__device__ __forceinline__ void pack_fused_body(const PackOut &o, uint32_t e, bool active, uint32_t n, int K, int E,
                                                int tile_m, uint32_t *pack_sm, uint32_t *scan_sm) {
    const int tid = (int)threadIdx.x, lane = lane_id(), wave = tid >> 6;
    for (int i = tid; i < kPackWaves * E; i += kPackThreads) pack_sm[i] = 0;
    __syncthreads();
    if (active && e >= (uint32_t)E) { // a corrupt id: stay in bounds, and tell the host
        if (o.bad_ids) atomicAdd(o.bad_ids, 1u);
        e = (uint32_t)E - 1;
    }
    if (active) atomicAdd(&pack_sm[wave * E + e], 1u);
    __syncthreads();
    uint32_t count = 0;
    if (tid < E) {
        for (int w = 0; w < kPackWaves; ++w) {
            uint32_t c = pack_sm[w * E + tid];
            pack_sm[w * E + tid] = count;
            count += c;
        }
    }
    uint32_t off = emit_segments(count, tid, E, n, tile_m, o, scan_sm);
    if (tid < E)
        for (int w = 0; w < kPackWaves; ++w) pack_sm[w * E + tid] += off;
    __syncthreads();
    uint64_t peers = match_expert(e, active, log2_ceil(E));
    if (active) {
        uint32_t rank = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
        place_row(o, pack_sm[wave * E + e] + rank, (uint32_t)tid, e, K);
    }
}

__global__ __launch_bounds__(kPackThreads) void pack_fused_kernel(PackOut o, const uint32_t *__restrict__ idx,
                                                                  uint32_t n, int K, int E, int tile_m) {
    extern __shared__ uint32_t pack_sm[]; // hist[kPackWaves][E]
    __shared__ uint32_t scan_sm[4 * kPackWaves];
    const bool active = threadIdx.x < n;
    const uint32_t e = active ? packed_id(o, idx[threadIdx.x]) : 0u;
    pack_fused_body(o, e, active, n, K, E, tile_m, pack_sm, scan_sm);
}

// ---- one wavefront, n <= 64 ---------------------------------------------------------------------------------
// A decode step of a few sequences: lane i = row i, every other row's id comes over with v_readlane, and nothing needs
// LDS, a barrier or a histogram. Same outputs. The loops over the other rows are serial, so this only pays for one or
// two sequences (6 rows: 6.7 us against 7.2 us for the 1024-thread kernel, 48 rows: 16.9 against 7.5 us).
constexpr uint32_t kPackWaveRows = 16;
__device__ __forceinline__ uint32_t lane_value(uint32_t v, uint32_t j) { return (uint32_t)__builtin_amdgcn_readlane((int)v, (int)j); }

__device__ __forceinline__ void pack_wave_body(const PackOut &o, uint32_t e, bool active, uint32_t n, int K, int E,
                                               int tile_m, int lane) {
    if (active && e >= (uint32_t)E) { // a corrupt id: stay in bounds, and tell the host
        if (o.bad_ids) atomicAdd(o.bad_ids, 1u);
        e = (uint32_t)E - 1;
    }
    const uint32_t key = active ? e : 0xffffffffu;
    // rows of smaller experts, earlier rows of this expert, rows of this expert
    uint32_t below = 0, before = 0, same = 0;
    for (uint32_t j = 0; j < n; ++j) {
        const uint32_t ej = lane_value(key, j);
        below += ej < key ? 1u : 0u;
        same += ej == key ? 1u : 0u;
        before += (ej == key && j < (uint32_t)lane) ? 1u : 0u;
    }
    if (active) place_row(o, below + before, (uint32_t)lane, e, K);
    // the first row of an expert speaks for it: its tiles, its place among the live experts
    const bool first = active && before == 0;
    const uint32_t tm = tile_m > 0 ? (uint32_t)tile_m : 1u;
    const uint32_t nt = (tile_m > 0 && first) ? (same + tm - 1) / tm : 0u;
    const uint32_t last_rows = same - (nt ? (nt - 1) * tm : 0);
    const uint32_t n_big = nt == 0 ? 0 : (nt - 1) + (last_rows > kPackSmallTileRows ? 1u : 0u);
    const uint32_t n_small = nt - n_big;
    const uint64_t firsts = __ballot(first);
    uint32_t live_rank = 0, live_tot = 0, big_ex = 0, small_ex = 0, big_tot = 0, small_tot = 0;
    for (uint32_t j = 0; j < n; ++j) {
        if (!((firsts >> j) & 1ull)) continue; // uniform
        const uint32_t ej = lane_value(key, j), bj = lane_value(n_big, j), sj = lane_value(n_small, j);
        const bool lt = ej < key;
        live_rank += lt ? 1u : 0u;
        big_ex += lt ? bj : 0u;
        small_ex += lt ? sj : 0u;
        live_tot += 1u, big_tot += bj, small_tot += sj;
    }
    // rows per expert and where they start, for every expert of the layer
    for (uint32_t x = (uint32_t)lane; x < (uint32_t)E; x += 64) {
        uint32_t c = 0, lo = 0;
        for (uint32_t j = 0; j < n; ++j) {
            const uint32_t ej = lane_value(key, j);
            c += ej == x ? 1u : 0u;
            lo += ej < x ? 1u : 0u;
        }
        if (o.counts) o.counts[x] = c;
        if (o.offsets) o.offsets[x] = lo;
    }
    if (lane == 0 && o.offsets) o.offsets[E] = n;
    if (first && o.live) o.live[live_rank] = e;
    if (lane == 0 && o.n_live) *o.n_live = live_tot;
    for (uint32_t i = (uint32_t)lane; i < o.n_done; i += 64) o.tile_done[i] = 0;
    // the folded always-on expert: identity rows behind the routed ones, its tiles ahead of the routed tiles
    const uint32_t nt_dense = (o.dense_rows + tm - 1) / tm;
    for (uint32_t i = (uint32_t)lane; i < o.dense_rows; i += 64) {
        o.order[n + i] = n + i;
        if (o.token) o.token[n + i] = i;
        if (o.sorted_e) o.sorted_e[n + i] = o.dense_expert;
    }
    if (tile_m > 0 && o.tiles) {
        for (uint32_t j = (uint32_t)lane; j < nt_dense; j += 64) {
            Tile t;
            t.expert = o.dense_expert;
            t.row0 = n + j * tm;
            const uint32_t left = o.dense_rows - j * tm;
            t.nrows = left < tm ? left : tm;
            t.flags = kTileDense;
            o.tiles[j] = t;
        }
        for (uint32_t j = 0; j < nt; ++j) { // nt = 0 on every lane but an expert's first
            Tile t;
            t.expert = e;
            t.row0 = below + j * tm;
            const uint32_t left = same - j * tm;
            t.nrows = left < tm ? left : tm;
            t.flags = 0;
            o.tiles[nt_dense + (j < n_big ? big_ex + j : big_tot + small_ex)] = t;
        }
        if (lane == 0 && o.n_tiles) *o.n_tiles = nt_dense + big_tot + small_tot;
    }
}

__global__ __launch_bounds__(64) void pack_wave_kernel(PackOut o, const uint32_t *__restrict__ idx, uint32_t n, int K,
                                                       int E, int tile_m) {
    const int lane = lane_id();
    const bool active = (uint32_t)lane < n;
    const uint32_t e = active ? packed_id(o, idx[lane]) : 0u;
    pack_wave_body(o, e, active, n, K, E, tile_m, lane);
}

// selection and packing of one or two sequences in one launch: wavefront t routes token t, wavefront 0 packs
__global__ __launch_bounds__(kPackWaveRows * 64) void route_pack_tiny_kernel(PackOut o, RouteArgs r, int E, int tile_m) {
    __shared__ uint32_t ids[kPackWaveRows];
    const int lane = lane_id(), t = (int)(threadIdx.x >> 6);
    {
        const float *const rows[1] = {r.scores + (size_t)t * r.E};
        uint32_t my_idx[1];
        float w[1];
        route_tokens<1, 4>(rows, r.bias, r.resident, r.E, r.K, r.normalize, r.apply_scale, r.route_scale, lane, my_idx, w);
        if (lane < r.K) {
            const size_t at = (size_t)t * r.K + lane;
            r.out_idx[at] = my_idx[0];
            r.out_w[at] = w[0];
            ids[at] = my_idx[0];
        }
    }
    __syncthreads();
    if (t != 0) return;
    const uint32_t n = (uint32_t)(r.T * r.K);
    const bool active = (uint32_t)lane < n;
    const uint32_t e = active ? packed_id(o, ids[lane]) : 0u;
    pack_wave_body(o, e, active, n, r.K, E, tile_m, lane);
}

bool route_pack_tiny_supports(const RouteArgs &r) {
    return r.T >= 1 && r.K >= 1 && (size_t)r.T * (size_t)r.K <= (size_t)kPackWaveRows && r.E >= r.K && r.E <= 256;
}

int launch_route_pack_tiny(const PackOut &o, const RouteArgs &r, int E, int tile_m, hipStream_t st) {
    DMOE_REQUIRE(route_pack_tiny_supports(r), "route + pack: T=%d K=%d E=%d is not a batch of one or two sequences", r.T, r.K, r.E);
    DMOE_REQUIRE(E >= 1 && E <= kPackThreads, "pack: E=%d out of range [1,%d]", E, kPackThreads);
    DMOE_REQUIRE(r.out_idx && r.out_w && r.scores && o.order, "route + pack: null pointer");
    hipLaunchKernelGGL(route_pack_tiny_kernel, dim3(1), dim3((unsigned)r.T * 64), 0, st, o, r, E, tile_m);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

// ---- three launches, any n --------------------------------------------------------------------------------
__global__ __launch_bounds__(kScatterWaves * 64) void pack_hist_kernel(PackOut o, uint32_t *__restrict__ cnt,
                                                                       const uint32_t *__restrict__ idx,
                                                                       size_t n, int E, int n_sub) {
    extern __shared__ uint32_t pack_sm[]; // hist[kScatterWaves][E]
    const int tid = (int)threadIdx.x, lane = lane_id(), wave = tid >> 6;
    for (int i = tid; i < kScatterWaves * E; i += kScatterWaves * 64) pack_sm[i] = 0;
    __syncthreads();
    const int sub = (int)blockIdx.x * kScatterWaves + wave;
    if (sub < n_sub) {
        for (int g = 0; g < kSubGroups; ++g) {
            size_t i = (size_t)sub * kSubRows + (size_t)g * 64 + lane;
            if (i < n) {
                uint32_t e = packed_id(o, idx[i]);
                if (e >= (uint32_t)E) { // counted here once; the scatter kernel clamps the same way
                    if (o.bad_ids) atomicAdd(o.bad_ids, 1u);
                    e = (uint32_t)E - 1;
                }
                atomicAdd(&pack_sm[wave * E + e], 1u);
            }
        }
    }
    __syncthreads();
    if (sub < n_sub)
        for (int e = lane; e < E; e += 64) cnt[(size_t)sub * E + e] = pack_sm[wave * E + e];
}

__global__ __launch_bounds__(kPackThreads) void pack_scan_kernel(PackOut o, uint32_t *__restrict__ cnt,
                                                                 size_t n, int E, int n_sub, int tile_m) {
    __shared__ uint32_t scan_sm[4 * kPackWaves];
    const int tid = (int)threadIdx.x;
    uint32_t count = 0;
    if (tid < E) {
        // exclusive scan down this expert's column of sub-chunk counts, 32 independent loads at a time (one
        // dependent load per sub-chunk made this loop the longest part of packing a prefill batch)
        constexpr int kBatch = 32;
        for (int s0 = 0; s0 < n_sub; s0 += kBatch) {
            uint32_t c[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) c[j] = s0 + j < n_sub ? cnt[(size_t)(s0 + j) * E + tid] : 0u;
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                if (s0 + j < n_sub) cnt[(size_t)(s0 + j) * E + tid] = count;
                count += c[j];
            }
        }
    }
    uint32_t off = emit_segments(count, tid, E, n, tile_m, o, scan_sm);
    // the scatter kernel needs the segment starts even if the caller did not ask for offsets
    if (tid < E) cnt[(size_t)n_sub * E + tid] = off;
}

__global__ __launch_bounds__(kScatterWaves * 64) void pack_scatter_kernel(PackOut o,
                                                                          const uint32_t *__restrict__ cnt,
                                                                          const uint32_t *__restrict__ idx,
                                                                          size_t n, int K, int E, int n_sub) {
    extern __shared__ uint32_t pack_sm[]; // run[kScatterWaves][E]
    const int tid = (int)threadIdx.x, lane = lane_id(), wave = tid >> 6;
    const int sub = (int)blockIdx.x * kScatterWaves + wave;
    const bool wave_on = sub < n_sub;
    if (wave_on)
        for (int e = lane; e < E; e += 64)
            pack_sm[wave * E + e] = cnt[(size_t)sub * E + e] + cnt[(size_t)n_sub * E + e];
    __syncthreads();
    const int nbits = log2_ceil(E);
    for (int g = 0; g < kSubGroups; ++g) {
        size_t i = (size_t)sub * kSubRows + (size_t)g * 64 + lane;
        const bool active = wave_on && i < n;
        uint32_t e = active ? packed_id(o, idx[i]) : 0u;
        if (active && e >= (uint32_t)E) e = (uint32_t)E - 1;
        uint64_t peers = match_expert(e, active, nbits);
        uint32_t base = 0, rank = 0;
        if (active) {
            base = pack_sm[wave * E + e];
            rank = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
            place_row(o, base + rank, (uint32_t)i, e, K);
        }
        __syncthreads(); // every lane has read its base before any counter moves
        if (active && (peers >> lane) <= 1ull) // highest lane of its peer group
            pack_sm[wave * E + e] = base + rank + 1u;
        __syncthreads();
    }
}

size_t pack_scratch_bytes(size_t n, int E) {
    size_t n_sub = (n + kSubRows - 1) / kSubRows;
    return (n_sub + 1) * (size_t)E * sizeof(uint32_t);
}

int launch_pack(const PackOut &o, const uint32_t *d_idx, size_t n, int K, int E, int tile_m, void *d_scratch,
                hipStream_t st) {
    DMOE_REQUIRE(E >= 1 && E <= kPackThreads, "pack: E=%d out of range [1,%d]", E, kPackThreads);
    DMOE_REQUIRE(K >= 1, "pack: K=%d", K);
    DMOE_REQUIRE(n < (1ull << 31), "pack: too many rows");
    DMOE_REQUIRE(n == 0 || (o.order != nullptr && d_idx != nullptr), "pack: null pointer");
    if (n <= (size_t)kPackWaveRows) { // also covers n == 0: counts / offsets / n_tiles / n_live are still written (all zero)
        hipLaunchKernelGGL(pack_wave_kernel, dim3(1), dim3(64), 0, st, o, d_idx, (uint32_t)n, K, E, tile_m);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    if (n <= (size_t)kPackThreads) {
        size_t lds = sizeof(uint32_t) * (size_t)kPackWaves * E;
        hipLaunchKernelGGL(pack_fused_kernel, dim3(1), dim3(kPackThreads), lds, st, o, d_idx, (uint32_t)n, K, E,
                           tile_m);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    DMOE_REQUIRE(d_scratch != nullptr, "pack: scratch is null");
    uint32_t *cnt = (uint32_t *)d_scratch;
    int n_sub = (int)((n + kSubRows - 1) / kSubRows);
    dim3 grid((unsigned)ceil_div(n_sub, kScatterWaves)), block(kScatterWaves * 64);
    size_t lds = sizeof(uint32_t) * (size_t)kScatterWaves * E;
    hipLaunchKernelGGL(pack_hist_kernel, grid, block, lds, st, o, cnt, d_idx, n, E, n_sub);
    DMOE_LAUNCH_CHECK();
    hipLaunchKernelGGL(pack_scan_kernel, dim3(1), dim3(kPackThreads), 0, st, o, cnt, n, E, n_sub, tile_m);
    DMOE_LAUNCH_CHECK();
    hipLaunchKernelGGL(pack_scatter_kernel, grid, block, lds, st, o, cnt, d_idx, n, K, E, n_sub);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

} // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_pack(uint32_t *d_out_order, uint32_t *d_out_inv_order, uint32_t *d_out_token,
                         uint32_t *d_out_sorted_expert, uint32_t *d_out_counts, uint32_t *d_out_offsets,
                         uint32_t *d_out_live_experts, uint32_t *d_out_n_live, const uint32_t *d_indices, int T,
                         int K, int E, dmoe_workspace ws, dmoe_stream s) {
    DMOE_REQUIRE(T >= 0 && K >= 1, "pack: bad shape T=%d K=%d", T, K);
    size_t n = (size_t)T * K;
    Workspace *w = nullptr;
    DMOE_TRY(workspace_reserve(ws, pack_scratch_bytes(n, E > 0 ? E : 1), &w));
    PackOut o;
    o.order = d_out_order;
    o.inv = d_out_inv_order;
    o.token = d_out_token;
    o.sorted_e = d_out_sorted_expert;
    o.counts = d_out_counts;
    o.offsets = d_out_offsets;
    o.live = d_out_live_experts;
    o.n_live = d_out_n_live;
    o.bad_ids = w->flags + 1;
    return launch_pack(o, d_indices, n, K, E, 0, w->base, to_hip(s));
}
