// Grouped quantized GEMM, small-M path (decode): at most kSmallTileM rows per expert tile.
//
// The step is bound by streaming every live expert's packed weights once from HBM, so the layout is
// built around the weight stream. A workgroup has four wavefronts; the reduction dimension is cut into
// KS slices of 64 chunks (a chunk = 16 bytes of one packed row), one slice per wavefront, so a wavefront
// reads one contiguous 1 KiB piece of a weight row per load instruction and every lane always covers
// the SAME columns of the reduction dimension: the matching activations of the tile's rows are loaded
// once and stay in registers. The 4 / KS wavefronts that share a slice take different output columns.
// Loads run one batch of columns ahead of the arithmetic. Products are formed with packed-bf16 dot
// instructions and f32 accumulation; the per-lane partial sums of a batch are reduced across the
// wavefront with a transposing butterfly (V values cost V + 5 - log2 V shuffles instead of 6 V), the
// slices meet in LDS, and the epilogue (row scale, SwiGLU, routing weight, bf16) stores coalesced rows.
//
// 4-bit affine weights are never multiplied out: codes become the bf16 numbers (128 + q) with one
// AND-OR per pair, and   sum_k x_k (q_k s + b) = s * sum_k x_k (128 + q_k) + (b - 128 s) * sum_k x_k
// is applied once per 32-value chunk.
#include "common.h"
#include "qformat.h"

namespace dmoe {

constexpr int kSmallWaves = 4;
constexpr int kColsGateUp = 32; // output columns per wavefront (each needs a gate row and an up row)
constexpr int kColsPlain = 64;
constexpr int kBatch = 2;       // columns per load batch
constexpr int kStages = 4;      // batches in the load ring (kStages - 1 in flight ahead of the arithmetic)

__device__ __forceinline__ uint32_t vgpr_const(uint32_t c);

template <typename Fmt>
struct SmallTraits {
    static constexpr bool kFactored = false;
    __device__ static __forceinline__ void unpack(const uint4 &raw, Meta m, uint32_t *pairs) {
        Fmt::decode_fast(raw, m, pairs);
    }
    __device__ static __forceinline__ void arrange_x(uint32_t *) {}
};

template <>
struct SmallTraits<FmtAffine4> {
    static constexpr bool kFactored = true;
    // pairs (q_i, q_{i+4}) of each 8-code word as bf16 (128 + q)
    __device__ static __forceinline__ void unpack_word(uint32_t w, uint32_t mask, uint32_t magic, uint32_t *o) {
        o[0] = (w & mask) | magic;
        o[1] = ((w >> 4) & mask) | magic;
        o[2] = ((w >> 8) & mask) | magic;
        o[3] = ((w >> 12) & mask) | magic;
    }
    __device__ static __forceinline__ void unpack(const uint4 &raw, Meta, uint32_t *pairs) {
        const uint32_t mask = vgpr_const(0x000f000fu), magic = vgpr_const(0x43004300u);
        unpack_word(raw.x, mask, magic, pairs);
        unpack_word(raw.y, mask, magic, pairs + 4);
        unpack_word(raw.z, mask, magic, pairs + 8);
        unpack_word(raw.w, mask, magic, pairs + 12);
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

// Sum V per-lane values over the 64 lanes; afterwards lane l holds the total of value (l mod V).
template <int V>
__device__ __forceinline__ float transpose_reduce(float (&v)[V], int lane) {
    int n = V, bit = 1;
#pragma unroll
    for (int level = 0; level < 6; ++level) {
        if (n > 1) {
#pragma unroll
            for (int i = 0; i < V / 2; ++i) {
                if (i < n / 2) {
                    const bool up = (lane & bit) != 0;
                    float send = up ? v[2 * i] : v[2 * i + 1];
                    float keep = up ? v[2 * i + 1] : v[2 * i];
                    v[i] = keep + __shfl_xor(send, bit, 64);
                }
            }
            n >>= 1;
        } else {
            v[0] += __shfl_xor(v[0], bit, 64);
        }
        bit <<= 1;
    }
    return v[0];
}

template <int NM>
struct Batch {
    uint4 raw[kBatch][NM];
    uint32_t sb[kBatch][NM][2]; // raw scale / bias words (converted when the batch is consumed)
};

// a 32-bit constant the compiler must keep in a vector register (VOP3 on gfx9 reads one scalar at most,
// so "(w & mask) | magic" only becomes a single v_and_or_b32 when the constants are vector operands)
__device__ __forceinline__ uint32_t vgpr_const(uint32_t c) {
    uint32_t v;
    asm volatile("v_mov_b32 %0, %1" : "=v"(v) : "s"(c));
    return v;
}

template <typename Fmt, int KS, bool GATE_UP, int M>
__device__ __forceinline__ void small_run(const GemmArgs &g, const Tile &t, float *part) {
    using ST = SmallTraits<Fmt>;
    constexpr int NP = Fmt::kVals / 2;          // packed pairs per chunk
    constexpr int NM = GATE_UP ? 2 : 1;
    constexpr int CG = kSmallWaves / KS;        // wavefronts (column groups) per slice
    constexpr int CPW = GATE_UP ? kColsGateUp : kColsPlain;
    constexpr int CPB = CG * CPW;               // output columns per workgroup
    constexpr int NB = CPW / kBatch;            // batches per wavefront
    constexpr int MP = M == 3 ? 4 : M;          // rows padded to a power of two for the butterfly
    constexpr int V = kBatch * NM * MP;
    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: keeps addressing scalar
    const int slice = wave % KS, cg = wave / KS;
    const int cols = g.b0.cols, n_out = g.b0.rows;
    const int k0 = (slice * 64 + lane) * Fmt::kVals;   // first reduction element of this lane's chunk
    const bool k_on = k0 < cols;
    // lanes past the end of the row read chunk 0 instead (valid memory) and multiply it by zero activations
    const uint32_t w_off = k_on ? (uint32_t)(slice * 64 + lane) * 16u : 0u;
    const int k_meta = k_on ? k0 : 0;

    const size_t e = t.expert;
    const int block_col0 = (int)blockIdx.x * CPB;
    const int wave_col0 = block_col0 + cg * CPW;
    // scalar bases of this expert's matrices; per-column offsets are added as scalars too
    const uint8_t *wbase[NM], *sbase[NM], *bbase[NM];
#pragma unroll
    for (int mi = 0; mi < NM; ++mi) {
        const QView &q = mi == 0 ? g.b0 : g.b1;
        wbase[mi] = q.w + e * q.w_mat;
        sbase[mi] = q.scales + e * q.s_mat;
        bbase[mi] = q.biases ? q.biases + e * q.s_mat : nullptr;
    }

    auto load_batch = [&](int n0, Batch<NM> &b) {
#pragma unroll
        for (int c = 0; c < kBatch; ++c) {
            int n = n0 + c;
            if (n >= n_out) n = n_out - 1; // stay inside the matrix; such columns are never stored
#pragma unroll
            for (int mi = 0; mi < NM; ++mi) {
                const QView &q = mi == 0 ? g.b0 : g.b1;
                b.raw[c][mi] = *(const uint4 *)(wbase[mi] + (size_t)n * q.w_row + w_off);
                Fmt::load_meta_raw(q, sbase[mi] + (size_t)n * q.s_row,
                                   bbase[mi] ? bbase[mi] + (size_t)n * q.s_row : nullptr, k_meta, b.sb[c][mi]);
            }
        }
    };

    Batch<NM> ring[kStages];
    const bool wave_on = wave_col0 < n_out;
    if (wave_on) {
#pragma unroll
        for (int j = 0; j < kStages - 1; ++j)
            if (j < NB) load_batch(wave_col0 + j * kBatch, ring[j]);
    }

    // ---- activations of the tile's rows: this lane's chunk, kept in registers ---------------------------
    // (issued after the first weight loads, which depend on the tile only, so both latencies overlap)
    uint32_t xp[M][NP];
    float xs[M];
#pragma unroll
    for (int r = 0; r < M; ++r) {
        const uint32_t p = t.row0 + (uint32_t)r;
        const size_t src = g.a_rows ? g.a_rows[p] : p;
        const uint16_t *xrow = g.a + src * (size_t)cols;
#pragma unroll
        for (int v = 0; v < NP / 4; ++v) {
            uint4 q = make_uint4(0, 0, 0, 0);
            if (k_on) q = *(const uint4 *)(xrow + k0 + 8 * v);
            xp[r][4 * v] = q.x;
            xp[r][4 * v + 1] = q.y;
            xp[r][4 * v + 2] = q.z;
            xp[r][4 * v + 3] = q.w;
        }
        float sum = 0.0f;
        if (ST::kFactored) {
#pragma unroll
            for (int i = 0; i < NP; ++i) sum = dot2_bf16(xp[r][i], 0x3f803f80u, sum); // x . (1, 1)
        }
        xs[r] = sum;
        ST::arrange_x(xp[r]);
    }

    auto compute_batch = [&](int col_in_wave, const Batch<NM> &b) {
        float v[V];
#pragma unroll
        for (int c = 0; c < kBatch; ++c) {
#pragma unroll
            for (int mi = 0; mi < NM; ++mi) {
                uint32_t pairs[NP];
                const Meta meta = Fmt::meta_from_raw(b.sb[c][mi]);
                ST::unpack(b.raw[c][mi], meta, pairs);
                const float s = meta.s;
                const float boff = fmaf(-128.0f, s, meta.b);
#pragma unroll
                for (int r = 0; r < MP; ++r) {
                    float val = 0.0f;
                    if (r < M) {
                        float p0 = 0.0f, p1 = 0.0f; // two chains for instruction-level parallelism
#pragma unroll
                        for (int i = 0; i < NP; i += 2) {
                            p0 = dot2_bf16(pairs[i], xp[r][i], p0);
                            p1 = dot2_bf16(pairs[i + 1], xp[r][i + 1], p1);
                        }
                        val = ST::kFactored ? fmaf(s, p0 + p1, boff * xs[r]) : p0 + p1;
                    }
                    v[(c * NM + mi) * MP + r] = val;
                }
            }
        }
        float tot = transpose_reduce<V>(v, lane);
        if (lane < V) {
            const int r = lane % MP, mi = (lane / MP) % NM, c = lane / (MP * NM);
            if (r < M) part[((slice * CPB + cg * CPW + col_in_wave + c) * NM + mi) * 4 + r] = tot;
        }
    };

    // software pipeline over the batches of this wavefront: kStages - 1 batches of loads stay in flight
    // while one is consumed; the ring indices are compile-time constants
#pragma unroll 1
    for (int b0 = 0; b0 < NB; b0 += kStages) {
#pragma unroll
        for (int j = 0; j < kStages; ++j) {
            const int b = b0 + j;
            if (wave_on && b + kStages - 1 < NB)
                load_batch(wave_col0 + (b + kStages - 1) * kBatch, ring[(j + kStages - 1) % kStages]);
            if (wave_on && b < NB && wave_col0 + b * kBatch < n_out) compute_batch(b * kBatch, ring[j]);
        }
    }
    __syncthreads();

    // ---- epilogue: add the slices, scale, activate, store rows of consecutive columns ----------------
    for (int i = tid; i < CPB * M; i += kSmallWaves * 64) {
        const int col = i % CPB, r = i / CPB;
        const int n = block_col0 + col;
        if (n >= n_out) continue;
        float acc[NM];
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            float a = 0.0f;
#pragma unroll
            for (int sl = 0; sl < KS; ++sl) a += part[((sl * CPB + col) * NM + mi) * 4 + r];
            if (Fmt::kRowScale) {
                const QView &q = mi == 0 ? g.b0 : g.b1;
                a *= *(const float *)(q.scales + e * q.s_mat + (size_t)n * q.s_row);
            }
            acc[mi] = a;
        }
        const uint32_t p = t.row0 + (uint32_t)r;
        float val = GATE_UP ? limited_swiglu(acc[0], acc[NM - 1], g.swiglu_limit) : acc[0];
        if (g.row_scale) val *= g.row_scale[g.row_scale_idx ? g.row_scale_idx[p] : p];
        const size_t dst = g.out_rows ? g.out_rows[p] : p;
        g.out[dst * (size_t)g.ldo + n] = f32_to_bf16_bits(val);
    }
}

template <typename Fmt, int KS, bool GATE_UP>
__global__ __launch_bounds__(kSmallWaves * 64) void qgemm_small_kernel(GemmArgs g) {
    __shared__ float part[2048];
    Tile t;
    const uint32_t slot = blockIdx.y;
    if (g.tiles) {
        const uint32_t n_tiles = *g.n_tiles; // both loads are issued before either is needed
        t = g.tiles[slot];                   // the list has room for every launched slot
        if (slot >= n_tiles) return;
    } else {
        t.expert = 0;
        t.row0 = slot * (uint32_t)kSmallTileM;
        if ((int)t.row0 >= g.dense_rows) return;
        uint32_t left = (uint32_t)g.dense_rows - t.row0;
        t.nrows = left < (uint32_t)kSmallTileM ? left : (uint32_t)kSmallTileM;
        t.pad = 0;
    }
    switch (t.nrows) { // uniform over the workgroup
    case 1: small_run<Fmt, KS, GATE_UP, 1>(g, t, part); break;
    case 2: small_run<Fmt, KS, GATE_UP, 2>(g, t, part); break;
    case 3: small_run<Fmt, KS, GATE_UP, 3>(g, t, part); break;
    case 4: small_run<Fmt, KS, GATE_UP, 4>(g, t, part); break;
    default: break;
    }
}

static int small_slices(const QView &b, int vals) {
    int s = ceil_div(b.cols, 64 * vals);
    return s <= 1 ? 1 : (s == 2 ? 2 : (s <= 4 ? 4 : 0));
}

bool qgemm_small_supports(const QView &b) {
    int vals = (b.mode == DMOE_QUANT_AFFINE && b.bits == 4) || b.mode == DMOE_QUANT_MXFP4 ? 32 : 16;
    return b.cols % vals == 0 && small_slices(b, vals) != 0;
}

struct SmallLaunch {
    const GemmArgs &g;
    hipStream_t st;
    template <typename Fmt, int KS>
    int go() {
        const int cpb = (kSmallWaves / KS) * (g.gate_up ? kColsGateUp : kColsPlain);
        dim3 grid((unsigned)ceil_div(g.b0.rows, cpb), (unsigned)g.max_tiles), block(kSmallWaves * 64);
        if (g.gate_up) hipLaunchKernelGGL((qgemm_small_kernel<Fmt, KS, true>), grid, block, 0, st, g);
        else hipLaunchKernelGGL((qgemm_small_kernel<Fmt, KS, false>), grid, block, 0, st, g);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
    template <typename Fmt>
    int operator()() {
        switch (small_slices(g.b0, Fmt::kVals)) {
        case 1: return go<Fmt, 1>();
        case 2: return go<Fmt, 2>();
        case 4: return go<Fmt, 4>();
        default: break;
        }
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
