// Device-side decoding of the quantized weight formats (MLX affine 4/8-bit, MXFP4, FP8-E4M3 per-row).
//
// Every format is read in 16-byte pieces ("chunks"): kVals values of one weight row that share one
// scale (and bias). Value i of a chunk is element (k0 + i) of the row, so pairs (2p, 2p+1) are adjacent
// along the reduction dimension.
//
// Two memory layouts exist for a stack of matrices:
//   MLX layout     rows are contiguous ([n, rows, cols*bits/32] u32 words), scales/biases per row.
//   packed layout  the resident layout of a dmoe_layer, built once at upload for the matrix-core
//                  kernels. Rows are taken in blocks of 32 and the reduction dimension in steps of
//                  two chunks; the 1 KiB that one wavefront consumes per step is contiguous:
//                      chunk (row = 32*nb + ln, step, h)  ->  16 bytes at
//                      w + mat*w_mat + (((nb*n_steps + step)*2 + h)*32 + ln) * 16
//                  so a wavefront streams its 32 rows as one linear run of memory. Scales and biases
//                  are interleaved the same way: affine {scale | bias << 16} words at
//                      meta + mat*m_mat + ((nb*n_groups + g)*32 + ln) * 4
//                  and MXFP4 exponents (one per chunk) at meta + mat*m_mat + ((nb*n_steps+step)*2+h)*32 + ln.
#pragma once

#include "common.h"

#if defined(__HIPCC__)
namespace dmoe {

// ---- scalar decoders (exact; used by dmoe_dequantize and as the definition of each format) -----------

// E8M0 shared exponent -> 2^(s-127); 255 is NaN
__device__ __forceinline__ float e8m0_to_f32(uint32_t s) {
    if (s == 255u) return __uint_as_float(0x7fc00000u);
    if (s == 0u) return __uint_as_float(0x00400000u); // 2^-127, an f32 subnormal
    return __uint_as_float(s << 23);
}

// E2M1 code (sign in bit 3) -> f32: 0, .5, 1, 1.5, 2, 3, 4, 6
__device__ __forceinline__ float e2m1_to_f32(uint32_t q) {
    uint32_t m = q & 7u;
    uint32_t bits = m >= 2u ? 0x3f800000u + ((m - 2u) << 22) : (m ? 0x3f000000u : 0u);
    return __uint_as_float(bits | ((q & 8u) << 28));
}

// OCP E4M3FN byte -> f32
__device__ __forceinline__ float e4m3_to_f32(uint32_t v) {
    uint32_t e = (v >> 3) & 15u, m = v & 7u, sign = (v & 0x80u) << 24;
    uint32_t bits;
    if (e == 15u && m == 7u) bits = 0x7fc00000u;
    else if (e == 0u) return __uint_as_float(__float_as_uint((float)m * 0.001953125f) | sign); // m * 2^-9
    else bits = ((e + 120u) << 23) | (m << 20);
    return __uint_as_float(bits | sign);
}

// ---- per-chunk decoders -------------------------------------------------------------------------------
// Fmt::kVals                          values per 16-byte chunk
// Fmt::kRowScale                      true: an f32 per-row scale is applied to the finished dot product
// Fmt::load_meta(q, row_s, row_b, k0) scale/bias of the chunk starting at column k0 (MLX layout)
// Fmt::load_meta_raw / meta_from_raw  the same in two steps: raw words while a load is in flight, f32 at use
// Fmt::packed_meta_base/_lane/_step, load_meta_at, meta_from_packed   raw word(s) from the packed layout
// Fmt::decode(raw, meta, out)         kVals/2 packed bf16 pairs, natural order, exact per-format arithmetic
// Fmt::decode_fast                    same values through the gfx950 packed conversion instructions

struct Meta {
    float s, b;
};

struct FmtAffine4 {
    static constexpr int kVals = 32;
    static constexpr int kMetaEntryBytes = 2; // MLX layout: bf16 scale (and bias) per group
    static constexpr int kDecodeOps = 96; // vector instructions to decode one chunk (scheduling hint only)
    static constexpr bool kRowScale = false;
    __device__ static __forceinline__ void load_meta_raw(const QView &q, const uint8_t *row_s, const uint8_t *row_b,
                                                         int k0, uint32_t *sb) {
        int g = k0 / q.group;
        sb[0] = ((const uint16_t *)row_s)[g];
        sb[1] = row_b ? ((const uint16_t *)row_b)[g] : 0u;
    }
    // Packed meta addressing, split into a part that is uniform over the wavefront (scalar arithmetic) and a
    // per-lane constant: word ((nb * n_groups + g) * 32 + ln) with g = (step * 2 + h) * kVals / group. Group sizes
    // are powers of two, and either a multiple of a step (g does not depend on h) or a divisor of a chunk, so g
    // splits exactly into a step term and an h term.
    __device__ static __forceinline__ size_t packed_meta_base(const QView &q, size_t mat, int nb) {
        return mat * q.m_mat + (size_t)nb * (size_t)(q.cols >> __builtin_ctz(q.group)) * 128;
    }
    __device__ static __forceinline__ uint32_t packed_meta_lane(const QView &q, int h, int ln) {
        return (uint32_t)((((h * kVals) >> __builtin_ctz(q.group)) * 32 + ln) * 4);
    }
    __device__ static __forceinline__ uint32_t packed_meta_step(const QView &q, int step) {
        return (uint32_t)(((step * 2 * kVals) >> __builtin_ctz(q.group)) * 128);
    }
    __device__ static __forceinline__ void load_meta_at(const uint8_t *p, uint32_t *sb) { sb[0] = *(const uint32_t *)p; }
    __device__ static __forceinline__ Meta meta_from_raw(const uint32_t *sb) {
        Meta m;
        m.s = bf16_bits_to_f32(sb[0]);
        m.b = bf16_bits_to_f32(sb[1]);
        return m;
    }
    __device__ static __forceinline__ Meta meta_from_packed(const uint32_t *sb) {
        Meta m;
        m.s = __uint_as_float(sb[0] << 16);
        m.b = __uint_as_float(sb[0] & 0xffff0000u);
        return m;
    }
    __device__ static __forceinline__ Meta load_meta(const QView &q, const uint8_t *row_s, const uint8_t *row_b,
                                                     int k0) {
        uint32_t sb[2];
        load_meta_raw(q, row_s, row_b, k0, sb);
        return meta_from_raw(sb);
    }
    __device__ static __forceinline__ void decode_word(uint32_t w, Meta m, uint32_t *out /*[4]*/) {
        uint32_t lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu; // nibbles 0,2,4,6 / 1,3,5,7 as bytes
        out[0] = pack_bf16x2(fmaf((float)(lo & 0xffu), m.s, m.b), fmaf((float)(hi & 0xffu), m.s, m.b));
        out[1] = pack_bf16x2(fmaf((float)((lo >> 8) & 0xffu), m.s, m.b), fmaf((float)((hi >> 8) & 0xffu), m.s, m.b));
        out[2] = pack_bf16x2(fmaf((float)((lo >> 16) & 0xffu), m.s, m.b), fmaf((float)((hi >> 16) & 0xffu), m.s, m.b));
        out[3] = pack_bf16x2(fmaf((float)(lo >> 24), m.s, m.b), fmaf((float)(hi >> 24), m.s, m.b));
    }
    __device__ static __forceinline__ void decode(const uint4 &raw, Meta m, uint32_t *out /*[16]*/) {
        decode_word(raw.x, m, out);
        decode_word(raw.y, m, out + 4);
        decode_word(raw.z, m, out + 8);
        decode_word(raw.w, m, out + 12);
    }
    __device__ static __forceinline__ void decode_fast(const uint4 &raw, Meta m, uint32_t *out) { decode(raw, m, out); }
    // Values (2q, 2q+1) of the chunk only, for callers that spread the decode between other instructions; q must
    // run upwards through a chunk. `m` must come from pair_meta() and `st` from pair_state(). A 4-bit code c masked
    // out in place IS an f16 number: the bit pattern c is the subnormal c * 2^-24, and a code that sits four bits up
    // in its half-word (pattern 16 c) is 16 c * 2^-24. v_fma_mix_f32 widens that half-word exactly inside an f32 fma,
    // so (c * 2^-24) * (s * 2^24) + b, respectively (16 c * 2^-24) * (s * 2^20) + b, is c * s + b rounded ONCE: bit for
    // bit what decode() computes with fmaf((float)c, s, b), for every bf16 scale and bias (the scaled s is exact up to
    // |s| < 2^103). Per word of 8 codes: one shift, four masks (codes i and i + 4 share a register), 8 fmas, 4 packs
    // = 17 instructions, against 23 with byte planes and v_cvt_f32_ubyteN.
    static constexpr int kPairState = 6;
    __device__ static __forceinline__ Meta pair_meta(Meta m) {
        m.s *= 16777216.0f; // s * 2^24, exact
        return m;
    }
    __device__ static __forceinline__ void pair_state(uint32_t *) {}
    __device__ static __forceinline__ void decode_pair(const uint4 &raw, Meta m, int q, uint32_t *out, uint32_t *st) {
        typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
        const uint32_t w = (q / 4) == 0 ? raw.x : (q / 4) == 1 ? raw.y : (q / 4) == 2 ? raw.z : raw.w;
        if (q == 0) st[5] = __float_as_uint(m.s * 0.0625f); // the scale of the codes that stay four bits up: s * 2^20
        if (q % 4 == 0) {
            st[0] = w & 0x000f000fu; // codes 0 | 4
            st[1] = w & 0x00f000f0u; // codes 1 | 5, sixteen-fold
        } else if (q % 4 == 1) {
            const uint32_t w8 = w >> 8;
            st[2] = w8 & 0x000f000fu; // codes 2 | 6
            st[3] = w8 & 0x00f000f0u; // codes 3 | 7, sixteen-fold
        }
        const f16x2_t a = __builtin_bit_cast(f16x2_t, st[(q % 2) * 2]), b = __builtin_bit_cast(f16x2_t, st[(q % 2) * 2 + 1]);
        const float va = (q % 4) < 2 ? (float)a.x : (float)a.y, vb = (q % 4) < 2 ? (float)b.x : (float)b.y;
        out[q] = pack_bf16x2(fmaf(va, m.s, m.b), fmaf(vb, __uint_as_float(st[5]), m.b));
    }
};

struct FmtAffine8 {
    static constexpr int kVals = 16;
    static constexpr int kMetaEntryBytes = 2;
    static constexpr int kDecodeOps = 44;
    static constexpr bool kRowScale = false;
    __device__ static __forceinline__ void load_meta_raw(const QView &q, const uint8_t *row_s, const uint8_t *row_b,
                                                         int k0, uint32_t *sb) {
        FmtAffine4::load_meta_raw(q, row_s, row_b, k0, sb);
    }
    // Packed meta addressing, split into a part that is uniform over the wavefront (scalar arithmetic) and a
    // per-lane constant: word ((nb * n_groups + g) * 32 + ln) with g = (step * 2 + h) * kVals / group. Group sizes
    // are powers of two, and either a multiple of a step (g does not depend on h) or a divisor of a chunk, so g
    // splits exactly into a step term and an h term.
    __device__ static __forceinline__ size_t packed_meta_base(const QView &q, size_t mat, int nb) {
        return mat * q.m_mat + (size_t)nb * (size_t)(q.cols >> __builtin_ctz(q.group)) * 128;
    }
    __device__ static __forceinline__ uint32_t packed_meta_lane(const QView &q, int h, int ln) {
        return (uint32_t)((((h * kVals) >> __builtin_ctz(q.group)) * 32 + ln) * 4);
    }
    __device__ static __forceinline__ uint32_t packed_meta_step(const QView &q, int step) {
        return (uint32_t)(((step * 2 * kVals) >> __builtin_ctz(q.group)) * 128);
    }
    __device__ static __forceinline__ void load_meta_at(const uint8_t *p, uint32_t *sb) { sb[0] = *(const uint32_t *)p; }
    __device__ static __forceinline__ Meta meta_from_raw(const uint32_t *sb) { return FmtAffine4::meta_from_raw(sb); }
    __device__ static __forceinline__ Meta meta_from_packed(const uint32_t *sb) { return FmtAffine4::meta_from_packed(sb); }
    __device__ static __forceinline__ Meta load_meta(const QView &q, const uint8_t *row_s, const uint8_t *row_b,
                                                     int k0) {
        return FmtAffine4::load_meta(q, row_s, row_b, k0);
    }
    __device__ static __forceinline__ void decode_word(uint32_t w, Meta m, uint32_t *out /*[2]*/) {
        out[0] = pack_bf16x2(fmaf((float)(w & 0xffu), m.s, m.b), fmaf((float)((w >> 8) & 0xffu), m.s, m.b));
        out[1] = pack_bf16x2(fmaf((float)((w >> 16) & 0xffu), m.s, m.b), fmaf((float)(w >> 24), m.s, m.b));
    }
    __device__ static __forceinline__ void decode(const uint4 &raw, Meta m, uint32_t *out /*[8]*/) {
        decode_word(raw.x, m, out);
        decode_word(raw.y, m, out + 2);
        decode_word(raw.z, m, out + 4);
        decode_word(raw.w, m, out + 6);
    }
    __device__ static __forceinline__ void decode_fast(const uint4 &raw, Meta m, uint32_t *out) { decode(raw, m, out); }
    // As for the 4-bit codes: a byte masked out in the low half of a half-word IS the f16 subnormal c * 2^-24, which
    // v_fma_mix_f32 widens exactly, so (c * 2^-24) * (s * 2^24) + b is c * s + b rounded once, the bits of decode(). Per
    // word of four codes: one shift, two masks (codes 0 | 2 and 1 | 3 share a register each), four fmas, two packs = 9
    // instructions against 10 with v_cvt_f32_ubyteN.
    static constexpr int kPairState = 2;
    __device__ static __forceinline__ Meta pair_meta(Meta m) {
        m.s *= 16777216.0f; // s * 2^24, exact
        return m;
    }
    __device__ static __forceinline__ void pair_state(uint32_t *) {}
    __device__ static __forceinline__ void decode_pair(const uint4 &raw, Meta m, int q, uint32_t *out, uint32_t *st) {
        typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
        const uint32_t w = (q / 2) == 0 ? raw.x : (q / 2) == 1 ? raw.y : (q / 2) == 2 ? raw.z : raw.w;
        if (q % 2 == 0) {
            st[0] = w & 0x00ff00ffu;        // codes 0 | 2
            st[1] = (w >> 8) & 0x00ff00ffu; // codes 1 | 3
        }
        const f16x2_t a = __builtin_bit_cast(f16x2_t, st[0]), b = __builtin_bit_cast(f16x2_t, st[1]);
        const float va = (q % 2) == 0 ? (float)a.x : (float)a.y, vb = (q % 2) == 0 ? (float)b.x : (float)b.y;
        out[q] = pack_bf16x2(fmaf(va, m.s, m.b), fmaf(vb, m.s, m.b));
    }
};

struct FmtMxfp4 {
    static constexpr int kVals = 32;
    static constexpr int kMetaEntryBytes = 1; // MLX layout: one E8M0 byte per group of 32
    static constexpr int kDecodeOps = 20;
    static constexpr bool kRowScale = false;
    __device__ static __forceinline__ void load_meta_raw(const QView &, const uint8_t *row_s, const uint8_t *, int k0,
                                                         uint32_t *sb) {
        sb[0] = row_s[k0 >> 5];
        sb[1] = 0u;
    }
    // packed meta: byte ((nb * n_steps + step) * 2 + h) * 32 + ln
    __device__ static __forceinline__ size_t packed_meta_base(const QView &q, size_t mat, int nb) {
        return mat * q.m_mat + (size_t)nb * (size_t)(q.cols / (2 * kVals)) * 64;
    }
    __device__ static __forceinline__ uint32_t packed_meta_lane(const QView &, int h, int ln) { return (uint32_t)(h * 32 + ln); }
    __device__ static __forceinline__ uint32_t packed_meta_step(const QView &, int step) { return (uint32_t)step * 64u; }
    __device__ static __forceinline__ void load_meta_at(const uint8_t *p, uint32_t *sb) { sb[0] = *p; }
    __device__ static __forceinline__ Meta meta_from_raw(const uint32_t *sb) {
        Meta m;
        m.s = e8m0_to_f32(sb[0]);
        m.b = 0.0f;
        return m;
    }
    __device__ static __forceinline__ Meta meta_from_packed(const uint32_t *sb) { return meta_from_raw(sb); }
    __device__ static __forceinline__ Meta load_meta(const QView &q, const uint8_t *row_s, const uint8_t *row_b,
                                                     int k0) {
        uint32_t sb[2];
        load_meta_raw(q, row_s, row_b, k0, sb);
        return meta_from_raw(sb);
    }
    __device__ static __forceinline__ void decode_word(uint32_t w, Meta m, uint32_t *out /*[4]*/) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            float a = e2m1_to_f32((w >> (8 * p)) & 15u) * m.s;
            float b = e2m1_to_f32((w >> (8 * p + 4)) & 15u) * m.s;
            out[p] = pack_bf16x2(a, b); // exact: 2 significant bits times a power of two
        }
    }
    __device__ static __forceinline__ void decode(const uint4 &raw, Meta m, uint32_t *out /*[16]*/) {
        decode_word(raw.x, m, out);
        decode_word(raw.y, m, out + 4);
        decode_word(raw.z, m, out + 8);
        decode_word(raw.w, m, out + 12);
    }
    // same values through the packed FP4 -> bf16 conversion (it scales by the exponent of `scale`)
    __device__ static __forceinline__ void fast_word(uint32_t w, float scale, uint32_t *out /*[4]*/) {
        out[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0));
        out[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1));
        out[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2));
        out[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3));
    }
    __device__ static __forceinline__ void decode_fast(const uint4 &raw, Meta m, uint32_t *out /*[16]*/) {
        fast_word(raw.x, m.s, out);
        fast_word(raw.y, m.s, out + 4);
        fast_word(raw.z, m.s, out + 8);
        fast_word(raw.w, m.s, out + 12);
    }
    static constexpr int kPairState = 1;
    __device__ static __forceinline__ Meta pair_meta(Meta m) { return m; }
    __device__ static __forceinline__ void pair_state(uint32_t *) {}
    __device__ static __forceinline__ void decode_pair(const uint4 &raw, Meta m, int q, uint32_t *out, uint32_t *) {
        const uint32_t w = (q / 4) == 0 ? raw.x : (q / 4) == 1 ? raw.y : (q / 4) == 2 ? raw.z : raw.w;
        switch (q % 4) { // the byte selector is an immediate
        case 0: out[q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, m.s, 0)); break;
        case 1: out[q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, m.s, 1)); break;
        case 2: out[q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, m.s, 2)); break;
        default: out[q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, m.s, 3)); break;
        }
    }
};

struct FmtFp8Row {
    static constexpr int kVals = 16;
    static constexpr int kMetaEntryBytes = 0; // no per-group entries
    static constexpr int kDecodeOps = 10;
    static constexpr bool kRowScale = true; // scales: one f32 per row, applied after the reduction
    __device__ static __forceinline__ void load_meta_raw(const QView &, const uint8_t *, const uint8_t *, int,
                                                         uint32_t *sb) {
        sb[0] = 0u;
        sb[1] = 0u;
    }
    __device__ static __forceinline__ size_t packed_meta_base(const QView &, size_t, int) { return 0; }
    __device__ static __forceinline__ uint32_t packed_meta_lane(const QView &, int, int) { return 0u; }
    __device__ static __forceinline__ uint32_t packed_meta_step(const QView &, int) { return 0u; }
    __device__ static __forceinline__ void load_meta_at(const uint8_t *, uint32_t *sb) { sb[0] = 0u; }
    __device__ static __forceinline__ Meta meta_from_raw(const uint32_t *) {
        Meta m;
        m.s = 1.0f;
        m.b = 0.0f;
        return m;
    }
    __device__ static __forceinline__ Meta meta_from_packed(const uint32_t *sb) { return meta_from_raw(sb); }
    __device__ static __forceinline__ Meta load_meta(const QView &, const uint8_t *, const uint8_t *, int) {
        return meta_from_raw(nullptr);
    }
    __device__ static __forceinline__ void decode_word(uint32_t w, Meta, uint32_t *out /*[2]*/) {
        out[0] = pack_bf16x2(e4m3_to_f32(w & 0xffu), e4m3_to_f32((w >> 8) & 0xffu)); // exact in bf16
        out[1] = pack_bf16x2(e4m3_to_f32((w >> 16) & 0xffu), e4m3_to_f32(w >> 24));
    }
    __device__ static __forceinline__ void decode(const uint4 &raw, Meta m, uint32_t *out /*[8]*/) {
        decode_word(raw.x, m, out);
        decode_word(raw.y, m, out + 2);
        decode_word(raw.z, m, out + 4);
        decode_word(raw.w, m, out + 6);
    }
    __device__ static __forceinline__ void fast_word(uint32_t w, uint32_t *out /*[2]*/) {
        out[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
        out[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true));
    }
    __device__ static __forceinline__ void decode_fast(const uint4 &raw, Meta, uint32_t *out /*[8]*/) {
        fast_word(raw.x, out);
        fast_word(raw.y, out + 2);
        fast_word(raw.z, out + 4);
        fast_word(raw.w, out + 6);
    }
    static constexpr int kPairState = 1;
    __device__ static __forceinline__ Meta pair_meta(Meta m) { return m; }
    __device__ static __forceinline__ void pair_state(uint32_t *) {}
    __device__ static __forceinline__ void decode_pair(const uint4 &raw, Meta, int q, uint32_t *out, uint32_t *) {
        const uint32_t w = (q / 2) == 0 ? raw.x : (q / 2) == 1 ? raw.y : (q / 2) == 2 ? raw.z : raw.w;
        if (q % 2 == 0) out[q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
        else out[q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true));
    }
};

// Unquantized bf16 weights seen as a "format" by the prefill kernel: a 16-byte chunk is eight values, i.e. exactly one
// matrix-instruction operand, and decoding is the identity. Not part of dispatch_format (which walks the quantized modes).
struct FmtBf16 {
    static constexpr int kVals = 8;
    static constexpr int kMetaEntryBytes = 0;
    static constexpr int kDecodeOps = 0;
    static constexpr bool kRowScale = false;
    __device__ static __forceinline__ void load_meta_raw(const QView &, const uint8_t *, const uint8_t *, int, uint32_t *sb) {
        sb[0] = 0u;
        sb[1] = 0u;
    }
    __device__ static __forceinline__ size_t packed_meta_base(const QView &, size_t, int) { return 0; }
    __device__ static __forceinline__ uint32_t packed_meta_lane(const QView &, int, int) { return 0u; }
    __device__ static __forceinline__ uint32_t packed_meta_step(const QView &, int) { return 0u; }
    __device__ static __forceinline__ void load_meta_at(const uint8_t *, uint32_t *sb) { sb[0] = 0u; }
    __device__ static __forceinline__ Meta meta_from_raw(const uint32_t *) {
        Meta m;
        m.s = 1.0f;
        m.b = 0.0f;
        return m;
    }
    __device__ static __forceinline__ Meta meta_from_packed(const uint32_t *sb) { return meta_from_raw(sb); }
    __device__ static __forceinline__ void decode_fast(const uint4 &raw, Meta, uint32_t *out /*[4]*/) {
        out[0] = raw.x, out[1] = raw.y, out[2] = raw.z, out[3] = raw.w;
    }
    static constexpr int kPairState = 1;
    __device__ static __forceinline__ Meta pair_meta(Meta m) { return m; }
    __device__ static __forceinline__ void pair_state(uint32_t *) {}
    __device__ static __forceinline__ void decode_pair(const uint4 &raw, Meta, int q, uint32_t *out, uint32_t *) {
        out[q] = q == 0 ? raw.x : q == 1 ? raw.y : q == 2 ? raw.z : raw.w;
    }
};

// dispatch a callable templated on the format: f.template operator()<Fmt>()
template <typename F>
inline int dispatch_format(const QView &q, F &&f) {
    if (q.mode == DMOE_QUANT_AFFINE && q.bits == 4) return f.template operator()<FmtAffine4>();
    if (q.mode == DMOE_QUANT_AFFINE && q.bits == 8) return f.template operator()<FmtAffine8>();
    if (q.mode == DMOE_QUANT_MXFP4) return f.template operator()<FmtMxfp4>();
    if (q.mode == DMOE_QUANT_FP8_ROW) return f.template operator()<FmtFp8Row>();
    set_error("unsupported quantization mode %d / bits %d", q.mode, q.bits);
    return DMOE_ERR_UNSUPPORTED;
}

// ---- addressing of one lane's chunk stream (lane = (ln = row within the 32-row block, h = step half)) ----
template <typename Fmt, bool PACKED>
struct ChunkStream {
    // packed layout: w / mbase are uniform over the wavefront, the lane's share is a 32-bit offset (so the loads can
    // take a scalar base); MLX layout: w is this lane's first chunk, srow / brow its row's scales / biases
    const uint8_t *w;
    const uint8_t *mbase;
    const uint8_t *srow;
    const uint8_t *brow;
    uint32_t wlane, mlane;
    int h;

    __device__ __forceinline__ void init(const QView &q, size_t mat, int row_block, int ln, int h_, int n_clamped) {
        h = h_;
        if (PACKED) {
            const int n_steps = q.cols / (2 * Fmt::kVals);
            w = q.w + mat * q.w_mat + (size_t)row_block * n_steps * 1024;
            wlane = (uint32_t)(h * 32 + ln) * 16u;
            mbase = q.meta + Fmt::packed_meta_base(q, mat, row_block);
            mlane = Fmt::packed_meta_lane(q, h, ln);
            srow = brow = nullptr;
        } else {
            w = q.w + mat * q.w_mat + (size_t)n_clamped * q.w_row + (size_t)h * 16;
            wlane = mlane = 0;
            mbase = nullptr;
            srow = q.scales + mat * q.s_mat + (size_t)n_clamped * q.s_row;
            brow = q.biases ? q.biases + mat * q.s_mat + (size_t)n_clamped * q.s_row : nullptr;
        }
    }
    // compiler-level fence on the chunk addresses: chunk loads issued after pin() stay behind every earlier asm
    // statement (used to keep them younger than hand-issued memory requests)
    __device__ __forceinline__ void pin() {
        if (PACKED) asm volatile("" : "+v"(wlane));
        else asm volatile("" : "+v"(w));
    }
    __device__ __forceinline__ uint4 load_chunk(int step) const {
        return *(const uint4 *)(w + (size_t)step * (PACKED ? 1024 : 32) + wlane);
    }
    // the same bytes with the streaming (non-temporal) hint, for kernels that are bound by the weight stream: a
    // plain read stream measures 7.1 instead of 6.0 TB/s with it, and tiles of one expert that run together
    // still find each other's lines in L2
    __device__ __forceinline__ uint4 load_chunk_stream(int step) const {
        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
        const u32x4_t v = __builtin_nontemporal_load((const u32x4_t *)(w + (size_t)step * (PACKED ? 1024 : 32) + wlane));
        return make_uint4(v.x, v.y, v.z, v.w);
    }
    __device__ __forceinline__ void load_meta(const QView &q, int step, uint32_t *sb) const {
        if (PACKED) Fmt::load_meta_at(mbase + Fmt::packed_meta_step(q, step) + mlane, sb);
        else Fmt::load_meta_raw(q, srow, brow, (step * 2 + h) * Fmt::kVals, sb);
    }
    __device__ static __forceinline__ Meta meta(const uint32_t *sb) {
        return PACKED ? Fmt::meta_from_packed(sb) : Fmt::meta_from_raw(sb);
    }
};

} // namespace dmoe
#endif
