// One-time conversion of a stack of quantized matrices from the MLX layout (rows contiguous) to the
// packed layout the matrix-core kernels stream (see qformat.h). Runs when a layer is created.
#include "common.h"

namespace dmoe {

static int chunk_vals(const QView &v) {
    if (v.mode == DMOE_QUANT_NONE) return 8; // a 16-byte piece holds 8 bf16; a step of two pieces is one MFMA (K = 16)
    return (v.mode == DMOE_QUANT_AFFINE && v.bits == 4) || v.mode == DMOE_QUANT_MXFP4 ? 32 : 16;
}

bool can_pack(const QView &v) { return v.rows % 32 == 0 && v.cols % (2 * chunk_vals(v)) == 0; }

size_t packed_w_bytes(const QView &v) { return v.w_row * (size_t)v.rows * (size_t)v.n_mats; }

size_t packed_meta_bytes(const QView &v) {
    if (v.mode == DMOE_QUANT_AFFINE) return (size_t)v.n_mats * v.rows * (size_t)(v.cols / v.group) * 4;
    if (v.mode == DMOE_QUANT_MXFP4) return (size_t)v.n_mats * v.rows * (size_t)(v.cols / 32);
    return 0;
}

// one thread per 16-byte chunk
__global__ void repack_chunks_kernel(uint4 *__restrict__ out, QView q, int chunks_per_row, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t per_mat = (size_t)q.rows * chunks_per_row;
    const size_t mat = i / per_mat, rem = i - mat * per_mat;
    const int row = (int)(rem / chunks_per_row), c = (int)(rem - (size_t)row * chunks_per_row);
    const int nb = row >> 5, ln = row & 31, step = c >> 1, h = c & 1, n_steps = chunks_per_row >> 1;
    const uint4 v = *(const uint4 *)(q.w + mat * q.w_mat + (size_t)row * q.w_row + (size_t)c * 16);
    out[mat * per_mat + (((size_t)nb * n_steps + step) * 2 + h) * 32 + ln] = v;
}

// affine: {scale | bias << 16} per (row, group)
__global__ void repack_affine_meta_kernel(uint32_t *__restrict__ out, QView q, int n_groups, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t per_mat = (size_t)q.rows * n_groups;
    const size_t mat = i / per_mat, rem = i - mat * per_mat;
    const int row = (int)(rem / n_groups), g = (int)(rem - (size_t)row * n_groups);
    const uint32_t s = ((const uint16_t *)(q.scales + mat * q.s_mat + (size_t)row * q.s_row))[g];
    const uint32_t b = q.biases ? ((const uint16_t *)(q.biases + mat * q.s_mat + (size_t)row * q.s_row))[g] : 0u;
    out[mat * per_mat + ((size_t)(row >> 5) * n_groups + g) * 32 + (row & 31)] = s | (b << 16);
}

// mxfp4: one exponent byte per chunk
__global__ void repack_mxfp4_meta_kernel(uint8_t *__restrict__ out, QView q, int chunks_per_row, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t per_mat = (size_t)q.rows * chunks_per_row;
    const size_t mat = i / per_mat, rem = i - mat * per_mat;
    const int row = (int)(rem / chunks_per_row), c = (int)(rem - (size_t)row * chunks_per_row);
    const int n_steps = chunks_per_row >> 1;
    out[mat * per_mat + (((size_t)(row >> 5) * n_steps + (c >> 1)) * 2 + (c & 1)) * 32 + (row & 31)] =
        q.scales[mat * q.s_mat + (size_t)row * q.s_row + c];
}

int launch_repack(void *d_w, void *d_meta, const QView &src, hipStream_t st) {
    DMOE_REQUIRE(can_pack(src) && !src.packed, "repack: shape [%d,%d] cannot be packed", src.rows, src.cols);
    const int cpr = src.cols / chunk_vals(src);
    size_t total = (size_t)src.n_mats * src.rows * cpr;
    hipLaunchKernelGGL(repack_chunks_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (uint4 *)d_w, src, cpr,
                       total);
    DMOE_LAUNCH_CHECK();
    if (src.mode == DMOE_QUANT_AFFINE) {
        const int ng = src.cols / src.group;
        total = (size_t)src.n_mats * src.rows * ng;
        hipLaunchKernelGGL(repack_affine_meta_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                           (uint32_t *)d_meta, src, ng, total);
        DMOE_LAUNCH_CHECK();
    } else if (src.mode == DMOE_QUANT_MXFP4) {
        total = (size_t)src.n_mats * src.rows * cpr;
        hipLaunchKernelGGL(repack_mxfp4_meta_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                           (uint8_t *)d_meta, src, cpr, total);
        DMOE_LAUNCH_CHECK();
    }
    return DMOE_OK;
}

} // namespace dmoe
