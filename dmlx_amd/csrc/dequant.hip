// dmoe_dequantize and the host-side description of quantized stacks.
#include "common.h"
#include "qformat.h"

namespace dmoe {

static size_t w_row_bytes(const dmoe_qweight *q) {
    if (q->mode == DMOE_QUANT_NONE) return (size_t)q->cols * 2;
    return q->mode == DMOE_QUANT_FP8_ROW ? (size_t)q->cols : (size_t)q->cols * (size_t)q->bits / 8;
}
static size_t s_row_bytes(const dmoe_qweight *q) {
    if (q->mode == DMOE_QUANT_NONE) return 0;
    if (q->mode == DMOE_QUANT_FP8_ROW) return 4;
    if (q->mode == DMOE_QUANT_MXFP4) return (size_t)q->cols / 32;
    return (size_t)(q->cols / q->group_size) * 2;
}
size_t qweight_w_bytes(const dmoe_qweight *q) { return w_row_bytes(q) * (size_t)q->rows * (size_t)q->n_mats; }
size_t qweight_s_bytes(const dmoe_qweight *q) { return s_row_bytes(q) * (size_t)q->rows * (size_t)q->n_mats; }
size_t qweight_b_bytes(const dmoe_qweight *q) {
    return (q->mode == DMOE_QUANT_AFFINE && q->biases) ? qweight_s_bytes(q) : 0;
}

int make_qview(QView *v, const dmoe_qweight *q, const char *name) {
    DMOE_REQUIRE(q != nullptr, "%s: descriptor is null", name);
    DMOE_REQUIRE(q->w && (q->scales || q->mode == DMOE_QUANT_NONE), "%s: weight / scales pointer is null", name);
    DMOE_REQUIRE(q->n_mats >= 1 && q->rows >= 1 && q->cols >= 1, "%s: bad shape [%d,%d,%d]", name, q->n_mats,
                 q->rows, q->cols);
    switch (q->mode) {
    case DMOE_QUANT_AFFINE:
        DMOE_REQUIRE(q->bits == 4 || q->bits == 8, "%s: affine bits must be 4 or 8 (got %d)", name, q->bits);
        DMOE_REQUIRE(q->group_size == 32 || q->group_size == 64 || q->group_size == 128,
                     "%s: affine group_size must be 32, 64 or 128 (got %d)", name, q->group_size);
        DMOE_REQUIRE(q->cols % q->group_size == 0, "%s: cols %d not a multiple of group_size %d", name, q->cols,
                     q->group_size);
        break;
    case DMOE_QUANT_MXFP4:
        DMOE_REQUIRE(q->bits == 4 && q->group_size == 32, "%s: mxfp4 needs bits=4, group_size=32", name);
        DMOE_REQUIRE(q->biases == nullptr, "%s: mxfp4 takes no biases", name);
        DMOE_REQUIRE(q->cols % 32 == 0, "%s: cols %d not a multiple of 32", name, q->cols);
        break;
    case DMOE_QUANT_FP8_ROW:
        DMOE_REQUIRE(q->bits == 8, "%s: fp8 needs bits=8", name);
        DMOE_REQUIRE(q->biases == nullptr, "%s: fp8 takes no biases", name);
        DMOE_REQUIRE(q->cols % 16 == 0, "%s: cols %d not a multiple of 16", name, q->cols);
        break;
    case DMOE_QUANT_NONE:
        DMOE_REQUIRE(q->bits == 16, "%s: unquantized weights are bf16 (bits=16, got %d)", name, q->bits);
        DMOE_REQUIRE(q->scales == nullptr && q->biases == nullptr, "%s: unquantized weights take no scales / biases", name);
        DMOE_REQUIRE(q->cols % 8 == 0 && q->rows % 4 == 0, "%s: unquantized weights need rows %% 4 == 0 and cols %% 8 == 0 (got [%d,%d])",
                     name, q->rows, q->cols);
        break;
    default:
        set_error("%s: unknown quantization mode %d", name, q->mode);
        return DMOE_ERR_INVALID;
    }
    DMOE_REQUIRE(((uintptr_t)q->w % 16) == 0 && (w_row_bytes(q) % 16) == 0,
                 "%s: packed rows must be 16-byte aligned (row = %zu bytes)", name, w_row_bytes(q));
    v->w = (const uint8_t *)q->w;
    v->scales = (const uint8_t *)q->scales;
    v->biases = (const uint8_t *)q->biases;
    v->w_row = w_row_bytes(q);
    v->s_row = s_row_bytes(q);
    v->w_mat = v->w_row * (size_t)q->rows;
    v->s_mat = v->s_row * (size_t)q->rows;
    v->rows = q->rows;
    v->cols = q->cols;
    v->n_mats = q->n_mats;
    v->mode = q->mode;
    v->bits = q->bits;
    v->group = q->mode == DMOE_QUANT_AFFINE ? q->group_size : 32;
    return DMOE_OK;
}

// one thread per 16-byte chunk of a row
template <typename Fmt>
__global__ void dequant_kernel(uint16_t *__restrict__ out, QView q, int mat) {
    const int chunks_per_row = q.cols / Fmt::kVals;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)q.rows * chunks_per_row) return;
    int row = (int)(i / chunks_per_row), c = (int)(i - (size_t)row * chunks_per_row);
    int k0 = c * Fmt::kVals;
    const uint8_t *wrow = q.w + (size_t)mat * q.w_mat + (size_t)row * q.w_row;
    const uint8_t *srow = q.scales + (size_t)mat * q.s_mat + (size_t)row * q.s_row;
    const uint8_t *brow = q.biases ? q.biases + (size_t)mat * q.s_mat + (size_t)row * q.s_row : nullptr;
    uint4 raw = *(const uint4 *)(wrow + (size_t)c * 16);
    Meta m = Fmt::load_meta(q, srow, brow, k0);
    uint32_t pairs[Fmt::kVals / 2];
    Fmt::decode(raw, m, pairs);
    if (Fmt::kRowScale) {
        float rs = *(const float *)srow;
#pragma unroll
        for (int p = 0; p < Fmt::kVals / 2; ++p)
            pairs[p] = pack_bf16x2(bf16_bits_to_f32(pairs[p] & 0xffffu) * rs, bf16_bits_to_f32(pairs[p] >> 16) * rs);
    }
    uint32_t *o = (uint32_t *)(out + (size_t)row * q.cols + k0);
#pragma unroll
    for (int p = 0; p < Fmt::kVals / 2; ++p) o[p] = pairs[p];
}

// The same matrix through the decoder that the matrix-core kernels run in registers (pair_meta / decode_pair), for
// tests that compare it bit for bit with decode().
template <typename Fmt>
__global__ void dequant_fused_kernel(uint16_t *__restrict__ out, QView q, int mat) {
    const int chunks_per_row = q.cols / Fmt::kVals;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)q.rows * chunks_per_row) return;
    int row = (int)(i / chunks_per_row), c = (int)(i - (size_t)row * chunks_per_row);
    int k0 = c * Fmt::kVals;
    const uint8_t *wrow = q.w + (size_t)mat * q.w_mat + (size_t)row * q.w_row;
    const uint8_t *srow = q.scales + (size_t)mat * q.s_mat + (size_t)row * q.s_row;
    const uint8_t *brow = q.biases ? q.biases + (size_t)mat * q.s_mat + (size_t)row * q.s_row : nullptr;
    uint4 raw = *(const uint4 *)(wrow + (size_t)c * 16);
    const Meta m = Fmt::pair_meta(Fmt::load_meta(q, srow, brow, k0));
    uint32_t pairs[Fmt::kVals / 2], st[Fmt::kPairState] = {};
    Fmt::pair_state(st);
#pragma unroll
    for (int p = 0; p < Fmt::kVals / 2; ++p) Fmt::decode_pair(raw, m, p, pairs, st);
    if (Fmt::kRowScale) {
        float rs = *(const float *)srow;
#pragma unroll
        for (int p = 0; p < Fmt::kVals / 2; ++p)
            pairs[p] = pack_bf16x2(bf16_bits_to_f32(pairs[p] & 0xffffu) * rs, bf16_bits_to_f32(pairs[p] >> 16) * rs);
    }
    uint32_t *o = (uint32_t *)(out + (size_t)row * q.cols + k0);
#pragma unroll
    for (int p = 0; p < Fmt::kVals / 2; ++p) o[p] = pairs[p];
}

struct DequantLaunch {
    uint16_t *out;
    QView q;
    int mat;
    hipStream_t st;
    bool fused = false;
    template <typename Fmt>
    int operator()() {
        size_t total = (size_t)q.rows * (q.cols / Fmt::kVals);
        if (fused)
            hipLaunchKernelGGL(dequant_fused_kernel<Fmt>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, out, q, mat);
        else
            hipLaunchKernelGGL(dequant_kernel<Fmt>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, out, q, mat);
        DMOE_LAUNCH_CHECK();
        return DMOE_OK;
    }
};

// FP8 E4M3 bytes [rows, cols] with one scale per block x block tile -> bf16. One thread per 16 bytes of a row (the
// launcher takes this kernel when a 16-byte piece never straddles two tiles), two 16-byte stores each.
template <bool E8M0>
__global__ void dequant_fp8_block_kernel(uint16_t *__restrict__ out, const uint8_t *__restrict__ w, const void *__restrict__ scale,
                                         int rows, int cols, int block, int scale_cols) {
    const int chunks_per_row = cols / 16;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * chunks_per_row) return;
    const int row = (int)(i / chunks_per_row), c = (int)(i - (size_t)row * chunks_per_row);
    const size_t si = (size_t)(row / block) * scale_cols + (size_t)(c * 16 / block);
    const float sc = E8M0 ? e8m0_to_f32(((const uint8_t *)scale)[si]) : ((const float *)scale)[si];
    const uint4 raw = *(const uint4 *)(w + (size_t)row * cols + (size_t)c * 16);
    uint32_t pairs[8];
    FmtFp8Row::decode(raw, Meta{1.0f, 0.0f}, pairs);
#pragma unroll
    for (int p = 0; p < 8; ++p)
        pairs[p] = pack_bf16x2(bf16_bits_to_f32(pairs[p] & 0xffffu) * sc, bf16_bits_to_f32(pairs[p] >> 16) * sc);
    uint4 *o = (uint4 *)(out + (size_t)row * cols + (size_t)c * 16);
    o[0] = make_uint4(pairs[0], pairs[1], pairs[2], pairs[3]);
    o[1] = make_uint4(pairs[4], pairs[5], pairs[6], pairs[7]);
}

// any shape, block size and alignment: one thread per value
template <bool E8M0>
__global__ void dequant_fp8_block_scalar_kernel(uint16_t *__restrict__ out, const uint8_t *__restrict__ w,
                                                const void *__restrict__ scale, int rows, int cols, int block, int scale_cols) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * cols) return;
    const int row = (int)(i / cols), col = (int)(i - (size_t)row * cols);
    const size_t si = (size_t)(row / block) * scale_cols + (size_t)(col / block);
    const float sc = E8M0 ? e8m0_to_f32(((const uint8_t *)scale)[si]) : ((const float *)scale)[si];
    out[i] = f32_to_bf16_bits(e4m3_to_f32(w[i]) * sc);
}

} // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_dequant_fp8_block(uint16_t *d_out, const uint8_t *d_weight, const void *d_scale, int scale_is_e8m0,
                                      int rows, int cols, int block_size, dmoe_stream s) {
    DMOE_REQUIRE(d_out && d_weight && d_scale, "dequant_fp8_block: null pointer");
    DMOE_REQUIRE(rows >= 0 && cols >= 0 && block_size >= 1, "dequant_fp8_block: bad shape [%d,%d] / block %d", rows, cols, block_size);
    if (rows == 0 || cols == 0) return DMOE_OK;
    const int scale_cols = ceil_div(cols, block_size);
    const size_t n = (size_t)rows * (size_t)cols;
    const bool wide = cols % 16 == 0 && block_size % 16 == 0 && ((uintptr_t)d_weight % 16) == 0 && ((uintptr_t)d_out % 16) == 0;
    const size_t threads = wide ? n / 16 : n;
    DMOE_REQUIRE((threads + 255) / 256 <= 0x7fffffffull, "dequant_fp8_block: [%d,%d] is too large for one call", rows, cols);
    const dim3 grid((unsigned)((threads + 255) / 256)), blk(256);
    hipStream_t st = to_hip(s);
    if (wide) {
        if (scale_is_e8m0) hipLaunchKernelGGL(dequant_fp8_block_kernel<true>, grid, blk, 0, st, d_out, d_weight, d_scale, rows, cols, block_size, scale_cols);
        else hipLaunchKernelGGL(dequant_fp8_block_kernel<false>, grid, blk, 0, st, d_out, d_weight, d_scale, rows, cols, block_size, scale_cols);
    } else {
        if (scale_is_e8m0) hipLaunchKernelGGL(dequant_fp8_block_scalar_kernel<true>, grid, blk, 0, st, d_out, d_weight, d_scale, rows, cols, block_size, scale_cols);
        else hipLaunchKernelGGL(dequant_fp8_block_scalar_kernel<false>, grid, blk, 0, st, d_out, d_weight, d_scale, rows, cols, block_size, scale_cols);
    }
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

static int dequantize_common(uint16_t *d_out, const dmoe_qweight *qw, int mat_index, bool fused, dmoe_stream s) {
    QView q;
    DMOE_TRY(make_qview(&q, qw, "dequantize"));
    DMOE_REQUIRE(d_out != nullptr, "dequantize: out is null");
    DMOE_REQUIRE(mat_index >= 0 && mat_index < q.n_mats, "dequantize: mat_index %d out of [0,%d)", mat_index,
                 q.n_mats);
    if (q.mode == DMOE_QUANT_NONE) { // nothing to decode: the matrix as it is
        DMOE_HIP(hipMemcpyAsync(d_out, q.w + (size_t)mat_index * q.w_mat, q.w_mat, hipMemcpyDeviceToDevice, to_hip(s)));
        return DMOE_OK;
    }
    DMOE_REQUIRE(q.cols % 32 == 0, "dequantize: cols %d not a multiple of 32", q.cols);
    return dispatch_format(q, DequantLaunch{d_out, q, mat_index, to_hip(s), fused});
}

extern "C" int dmoe_dequantize(uint16_t *d_out, const dmoe_qweight *qw, int mat_index, dmoe_stream s) {
    return dequantize_common(d_out, qw, mat_index, false, s);
}

extern "C" int dmoe_debug_dequantize_fused(uint16_t *d_out, const dmoe_qweight *qw, int mat_index, dmoe_stream s) {
    return dequantize_common(d_out, qw, mat_index, true, s);
}
