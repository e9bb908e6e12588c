// Device layouts of the GGUF block formats and the per-lane "chunk" decoders used by
// the dequantisation and GEMV kernels.
//
// Block arithmetic follows crates/slai/src/quantization.rs of the reference
// (BlockQ8_0 :29-42, BlockQ4_0 :47-69, BlockQ6K :204-244, BlockQ5K :249-317,
// BlockQ4K :322-379, get_scale_min_k4 :381-389, decode_f16 :392-409).
//
// Device layout ("planes"): formats whose GGUF block size is not a multiple of 16
// bytes are split per row into 16-byte aligned planes so that every lane issues aligned
// 128-bit loads; the byte count per row is unchanged (up to <16 B of row padding).
//   Q8_0 row: [qs: nb*32 i8][d: nb f16]
//   Q4_0 row: [qs: nb*16 u8][d: nb f16]
//   Q6_K row: [ql: nb*128][qh: nb*64][scales: nb*16 i8][d: nb f16]
//   Q4_K / Q5_K / F16 / F32 rows: verbatim GGUF bytes (144 / 176 B blocks are 16-B multiples)
// Rows start at multiples of 16 bytes (row_stride).
//
// The same header compiles for the host (plain C++) so the index math can be checked
// on a CPU; SLAI_HD marks functions usable on both sides.
#pragma once
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#define SLAI_HD __host__ __device__ inline
#else
#define SLAI_HD inline
#include <math.h>
#endif

namespace slai {

enum : int { T_F32 = 0, T_F16 = 1, T_Q4_0 = 2, T_Q4_1 = 3, T_Q5_0 = 6, T_Q5_1 = 7, T_Q8_0 = 8, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14,
              T_Q8_K = 15 };

struct U4 { uint32_t x, y, z, w; };

SLAI_HD size_t align16(size_t v) { return (v + 15) & ~(size_t)15; }

SLAI_HD int block_elems(int t) {
    switch (t) { case T_F32: case T_F16: return 1; case T_Q4_0: case T_Q4_1: case T_Q5_0: case T_Q5_1: case T_Q8_0: return 32;
                 case T_Q4_K: case T_Q5_K: case T_Q6_K: case T_Q8_K: return 256; default: return 0; }
}
SLAI_HD int block_bytes(int t) {
    switch (t) { case T_F32: return 4; case T_F16: return 2; case T_Q4_0: return 18; case T_Q4_1: return 20; case T_Q5_0: return 22;
                 case T_Q5_1: return 24; case T_Q8_0: return 34; case T_Q4_K: return 144; case T_Q5_K: return 176; case T_Q6_K: return 210;
                 case T_Q8_K: return 292; default: return 0; }
}
// bytes of one row in GGUF order / in device order
SLAI_HD size_t gguf_row_bytes(int t, uint32_t ncols) { return (size_t)(ncols / block_elems(t)) * block_bytes(t); }
SLAI_HD size_t device_row_stride(int t, uint32_t ncols) { return align16(gguf_row_bytes(t, ncols)); }

SLAI_HD float bits_to_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
SLAI_HD uint32_t float_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

// quantization.rs:392-409.  Exact for every finite/infinite input; NaNs come out as the
// canonical quiet NaN with the input's sign, as the reference produces.
SLAI_HD float decode_f16(uint16_t h) {
#if defined(__HIP_DEVICE_COMPILE__)
    float f = __half2float(__ushort_as_half(h));
    if (f != f) return bits_to_float(((uint32_t)(h & 0x8000u) << 16) | 0x7fc00000u);
    return f;
#else
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff;
    if (e == 0) { float v = ldexpf((float)m, -24); return bits_to_float(float_to_bits(v) | sign); }
    if (e == 31) return bits_to_float(sign | (m ? 0x7fc00000u : 0x7f800000u));
    return bits_to_float(sign | ((e + 112) << 23) | (m << 13));
#endif
}
// binary16 -> binary32 inside the GEMV dot products (not the bit-exact dequantiser): the hardware converter on
// the device (one instruction; identical to decode_f16 for every non-NaN input), decode_f16 on the host.
SLAI_HD float gemv_f16(uint16_t h) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (float)__builtin_bit_cast(_Float16, h);
#else
    return decode_f16(h);
#endif
}

// IEEE binary32 -> binary16, round to nearest even (KV-cache store).
SLAI_HD uint16_t encode_f16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __half_as_ushort(__float2half_rn(f));
#else
    uint32_t x = float_to_bits(f), sign = (x >> 16) & 0x8000u, e = (x >> 23) & 0xffu, m = x & 0x7fffffu;
    if (e == 0xff) return (uint16_t)(sign | 0x7c00u | (m ? (0x200u | (m >> 13)) : 0));
    int ne = (int)e - 127 + 15;
    if (ne >= 31) return (uint16_t)(sign | 0x7c00u);
    if (ne <= 0) {
        if (ne < -10) return (uint16_t)sign;
        m |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - ne), hm = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t hm = m >> 13, rem = m & 0x1fffu, out = sign | ((uint32_t)ne << 10) | hm;
    if (rem > 0x1000u || (rem == 0x1000u && (hm & 1u))) out++;
    return (uint16_t)out;
#endif
}

SLAI_HD uint16_t ld16(const uint8_t *p) { uint16_t v; memcpy(&v, p, 2); return v; }
SLAI_HD U4 ld128(const uint8_t *p) {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint4 v = *reinterpret_cast<const uint4 *>(p);
    return U4{v.x, v.y, v.z, v.w};
#else
    U4 v; memcpy(&v, p, 16); return v;
#endif
}
// The same for weights that a kernel reads exactly once: the non-temporal hint keeps them from displacing what the caches
// are needed for (the vectors handed from launch to launch, or from workgroup to workgroup inside one).
SLAI_HD U4 ld128_stream(const uint8_t *p) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef uint32_t words4 __attribute__((ext_vector_type(4)));
    const words4 v = __builtin_nontemporal_load(reinterpret_cast<const words4 *>(p));
    return U4{v.x, v.y, v.z, v.w};
#else
    return ld128(p);
#endif
}
SLAI_HD uint32_t byte_of(const U4 &v, int k) {  // byte k (0..15) of a 128-bit value
    uint32_t w = (k < 8) ? ((k < 4) ? v.x : v.y) : ((k < 12) ? v.z : v.w);
    return (w >> (8 * (k & 3))) & 0xffu;
}

// quantization.rs:381-389 on the 12 scale bytes held in hdr.y/z/w (bytes 4..15 of the block).
SLAI_HD void scale_min_k4(const U4 &hdr, int j, uint32_t &sc, uint32_t &m) {
    if (j < 4) {
        sc = byte_of(hdr, 4 + j) & 63u;
        m = byte_of(hdr, 8 + j) & 63u;
    } else {
        uint32_t a = byte_of(hdr, 8 + j), b = byte_of(hdr, j), c = byte_of(hdr, 4 + j);
        sc = (a & 0xFu) | ((b >> 6) << 4);
        m = (a >> 4) | ((c >> 6) << 4);
    }
}

// ---------------------------------------------------------------------------
// Bit-exact single-element dequantisation from the device layout.  Multiplications and
// subtractions are separate roundings, as in the reference; the translation unit that
// uses this for the exactness contract is compiled with -ffp-contract=off.
// `row` points at the start of the row, nb = blocks per row.
// ---------------------------------------------------------------------------
SLAI_HD float dequant_elem(int t, const uint8_t *row, uint32_t nb, uint32_t col) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
    switch (t) {
    case T_F32: { float f; memcpy(&f, row + (size_t)col * 4, 4); return f; }
    case T_F16: return decode_f16(ld16(row + (size_t)col * 2));
    case T_Q8_0: {
        float d = decode_f16(ld16(row + (size_t)nb * 32 + (size_t)(col / 32) * 2));
        return (float)(int8_t)row[col] * d;
    }
    case T_Q4_0: {
        uint32_t b = col / 32, j = col % 32;
        float d = decode_f16(ld16(row + (size_t)nb * 16 + (size_t)b * 2));
        uint8_t byte = row[(size_t)b * 16 + (j & 15)];
        int q = (int)(j < 16 ? (byte & 0xF) : (byte >> 4)) - 8;
        return (float)q * d;
    }
    // Row layout of the remaining 32-element formats: [qs: 16 B per block][qh: 4 B per block (Q5_x)][d or (d, m) per block]
    case T_Q4_1: {      // BlockQ4_1, quantization.rs:74-99
        uint32_t b = col / 32, j = col % 32;
        const uint8_t *dm = row + (size_t)nb * 16 + (size_t)b * 4;
        float d = decode_f16(ld16(dm)), m = decode_f16(ld16(dm + 2));
        uint8_t byte = row[(size_t)b * 16 + (j & 15)];
        uint32_t q = j < 16 ? (byte & 0xFu) : (byte >> 4);
        return (float)q * d + m;
    }
    case T_Q5_0: case T_Q5_1: {     // BlockQ5_0 :103-128, BlockQ5_1 :134-161
        uint32_t b = col / 32, j = col % 32;
        uint32_t qh; memcpy(&qh, row + (size_t)nb * 16 + (size_t)b * 4, 4);
        uint8_t byte = row[(size_t)b * 16 + (j & 15)];
        uint32_t q = (j < 16 ? (byte & 0xFu) : (uint32_t)(byte >> 4)) | (((qh >> j) & 1u) << 4);
        if (t == T_Q5_0) {
            float d = decode_f16(ld16(row + (size_t)nb * 20 + (size_t)b * 2));
            return (float)((int)q - 16) * d;
        }
        const uint8_t *dm = row + (size_t)nb * 20 + (size_t)b * 4;
        float d = decode_f16(ld16(dm)), m = decode_f16(ld16(dm + 2));
        return (float)q * d + m;
    }
    case T_Q8_K: {      // BlockQ8K, quantization.rs:170-198: [qs: 256 B per block][d: f32 per block]; the block sums are not kept
        uint32_t b = col / 256;
        float d; memcpy(&d, row + (size_t)nb * 256 + (size_t)b * 4, 4);
        return d * (float)(int8_t)row[col];
    }
    case T_Q4_K: case T_Q5_K: {
        const uint32_t bs = (t == T_Q4_K) ? 144u : 176u;
        const uint8_t *blk = row + (size_t)(col / 256) * bs;
        uint32_t e = col % 256, jp = e / 64, w = e % 64, hi = w >= 32, l = w % 32;
        U4 hdr = ld128(blk);
        float d = decode_f16((uint16_t)(hdr.x & 0xffffu)), dmin = decode_f16((uint16_t)(hdr.x >> 16));
        uint32_t sc, m;
        scale_min_k4(hdr, (int)(jp * 2 + hi), sc, m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        const uint8_t *qs = blk + (t == T_Q4_K ? 16 : 48);
        uint8_t byte = qs[jp * 32 + l];
        uint32_t q = hi ? (byte >> 4) : (byte & 0xF);
        if (t == T_Q5_K) q += ((blk[16 + l] >> (2 * jp + hi)) & 1u) ? 16u : 0u;
        return d1 * (float)q - m1;
    }
    case T_Q6_K: {
        uint32_t b = col / 256, e = col % 256, i = e / 128, r = (e % 128) / 32, l = e % 32, is = l / 16;
        const uint8_t *ql = row + (size_t)b * 128, *qh = row + (size_t)nb * 128 + (size_t)b * 64;
        const int8_t *sc = (const int8_t *)(row + (size_t)nb * 192 + (size_t)b * 16);
        float d = decode_f16(ld16(row + (size_t)nb * 208 + (size_t)b * 2));
        uint8_t byte = ql[i * 64 + (r & 1) * 32 + l];
        uint32_t nib = (r < 2) ? (byte & 0xF) : (byte >> 4);
        uint32_t two = (qh[i * 32 + l] >> (2 * r)) & 3u;
        int q = (int)(int8_t)(nib | (two << 4)) - 32;
        return d * (float)sc[i * 8 + is + 2 * r] * (float)q;
    }
    default: return 0.0f;
    }
}

// Converts one GGUF block (verbatim bytes at `src`) into the device layout of row `dst_row`.
// b = block index within the row, nb = blocks per row.
SLAI_HD void repack_block(int t, const uint8_t *src, uint8_t *dst_row, uint32_t nb, uint32_t b) {
    switch (t) {
    case T_Q8_0:
        for (int i = 0; i < 32; ++i) dst_row[(size_t)b * 32 + i] = src[2 + i];
        dst_row[(size_t)nb * 32 + (size_t)b * 2] = src[0]; dst_row[(size_t)nb * 32 + (size_t)b * 2 + 1] = src[1];
        break;
    case T_Q4_0:
        for (int i = 0; i < 16; ++i) dst_row[(size_t)b * 16 + i] = src[2 + i];
        dst_row[(size_t)nb * 16 + (size_t)b * 2] = src[0]; dst_row[(size_t)nb * 16 + (size_t)b * 2 + 1] = src[1];
        break;
    case T_Q4_1:
        for (int i = 0; i < 16; ++i) dst_row[(size_t)b * 16 + i] = src[4 + i];
        for (int i = 0; i < 4; ++i) dst_row[(size_t)nb * 16 + (size_t)b * 4 + i] = src[i];
        break;
    case T_Q5_0:
        for (int i = 0; i < 16; ++i) dst_row[(size_t)b * 16 + i] = src[6 + i];
        for (int i = 0; i < 4; ++i) dst_row[(size_t)nb * 16 + (size_t)b * 4 + i] = src[2 + i];
        dst_row[(size_t)nb * 20 + (size_t)b * 2] = src[0]; dst_row[(size_t)nb * 20 + (size_t)b * 2 + 1] = src[1];
        break;
    case T_Q5_1:
        for (int i = 0; i < 16; ++i) dst_row[(size_t)b * 16 + i] = src[8 + i];
        for (int i = 0; i < 4; ++i) dst_row[(size_t)nb * 16 + (size_t)b * 4 + i] = src[4 + i];
        for (int i = 0; i < 4; ++i) dst_row[(size_t)nb * 20 + (size_t)b * 4 + i] = src[i];
        break;
    case T_Q8_K:
        for (int i = 0; i < 256; ++i) dst_row[(size_t)b * 256 + i] = src[4 + i];
        for (int i = 0; i < 4; ++i) dst_row[(size_t)nb * 256 + (size_t)b * 4 + i] = src[i];
        break;
    case T_Q6_K:
        for (int i = 0; i < 128; ++i) dst_row[(size_t)b * 128 + i] = src[i];
        for (int i = 0; i < 64; ++i) dst_row[(size_t)nb * 128 + (size_t)b * 64 + i] = src[128 + i];
        for (int i = 0; i < 16; ++i) dst_row[(size_t)nb * 192 + (size_t)b * 16 + i] = src[192 + i];
        dst_row[(size_t)nb * 208 + (size_t)b * 2] = src[208]; dst_row[(size_t)nb * 208 + (size_t)b * 2 + 1] = src[209];
        break;
    default: {
        int bb = block_bytes(t);
        for (int i = 0; i < bb; ++i) dst_row[(size_t)b * bb + i] = src[i];
    }
    }
}

// ---------------------------------------------------------------------------
// GEMV chunks.  A chunk is the unit one lane owns in every row: NRUN runs of RUNLEN
// consecutive columns whose activations the lane keeps in registers (x[r*RUNLEN+i]),
// together with the per-run sums xs[r] that absorb the formats' constant offsets:
//   sum_i (s*q_i - m) x_i = s * sum_i q_i x_i - m * sum_i x_i.
// fp32 accumulation throughout.
// ---------------------------------------------------------------------------
SLAI_HD float ub0(uint32_t w) { return (float)(w & 0xffu); }
SLAI_HD float ub1(uint32_t w) { return (float)((w >> 8) & 0xffu); }
SLAI_HD float ub2(uint32_t w) { return (float)((w >> 16) & 0xffu); }
SLAI_HD float ub3(uint32_t w) { return (float)(w >> 24); }
// sum of the four bytes of w times x[0..3]
SLAI_HD float dot4b(uint32_t w, const float *x, float acc) {
    acc = fmaf(ub0(w), x[0], acc); acc = fmaf(ub1(w), x[1], acc);
    acc = fmaf(ub2(w), x[2], acc); acc = fmaf(ub3(w), x[3], acc);
    return acc;
}
SLAI_HD float dot16b(const U4 &v, const float *x) {
    float a = dot4b(v.x, x, 0.0f);
    float b = dot4b(v.y, x + 4, 0.0f);
    a = dot4b(v.z, x + 8, a);
    b = dot4b(v.w, x + 12, b);
    return a + b;
}
SLAI_HD U4 and4(const U4 &v, uint32_t m) { return U4{v.x & m, v.y & m, v.z & m, v.w & m}; }
SLAI_HD U4 shr4(const U4 &v, int s) { return U4{v.x >> s, v.y >> s, v.z >> s, v.w >> s}; }
SLAI_HD U4 or4(const U4 &a, const U4 &b) { return U4{a.x | b.x, a.y | b.y, a.z | b.z, a.w | b.w}; }
SLAI_HD U4 shl4(const U4 &v, int s) { return U4{v.x << s, v.y << s, v.z << s, v.w << s}; }
SLAI_HD U4 xor4(const U4 &v, uint32_t m) { return U4{v.x ^ m, v.y ^ m, v.z ^ m, v.w ^ m}; }

template <int T> struct Chunk;

template <> struct Chunk<T_Q4_K> {
    static constexpr int NRUN = 2, RUNLEN = 16, E = 32;
    struct Data { U4 hdr, qs; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 32; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return (c >> 3) * 256 + ((c & 7) >> 1) * 64 + (c & 1) * 16 + r * 32; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        const uint8_t *blk = row + (size_t)(c >> 3) * 144;
        return Data{ld128(blk), ld128(blk + 16 + ((c & 7) >> 1) * 32 + (c & 1) * 16)};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        const int j = (c & 7) >> 1;
        float dd = gemv_f16((uint16_t)(d.hdr.x & 0xffffu)), dmin = gemv_f16((uint16_t)(d.hdr.x >> 16));
        uint32_t sc0, m0, sc1, m1;
        scale_min_k4(d.hdr, 2 * j, sc0, m0);
        scale_min_k4(d.hdr, 2 * j + 1, sc1, m1);
        float slo = dot16b(and4(d.qs, 0x0F0F0F0Fu), x);
        float shi = dot16b(and4(shr4(d.qs, 4), 0x0F0F0F0Fu), x + 16);
        return dd * ((float)sc0 * slo + (float)sc1 * shi) - dmin * ((float)m0 * xs[0] + (float)m1 * xs[1]);
    }
};

template <> struct Chunk<T_Q5_K> {
    static constexpr int NRUN = 2, RUNLEN = 16, E = 32;
    struct Data { U4 hdr, qh, qs; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 32; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return (c >> 3) * 256 + ((c & 7) >> 1) * 64 + (c & 1) * 16 + r * 32; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        const uint8_t *blk = row + (size_t)(c >> 3) * 176;
        return Data{ld128(blk), ld128(blk + 16 + (c & 1) * 16), ld128(blk + 48 + ((c & 7) >> 1) * 32 + (c & 1) * 16)};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        const int j = (c & 7) >> 1;
        float dd = gemv_f16((uint16_t)(d.hdr.x & 0xffffu)), dmin = gemv_f16((uint16_t)(d.hdr.x >> 16));
        uint32_t sc0, m0, sc1, m1;
        scale_min_k4(d.hdr, 2 * j, sc0, m0);
        scale_min_k4(d.hdr, 2 * j + 1, sc1, m1);
        U4 hlo = shl4(and4(shr4(d.qh, 2 * j), 0x01010101u), 4);
        U4 hhi = shl4(and4(shr4(d.qh, 2 * j + 1), 0x01010101u), 4);
        float slo = dot16b(or4(and4(d.qs, 0x0F0F0F0Fu), hlo), x);
        float shi = dot16b(or4(and4(shr4(d.qs, 4), 0x0F0F0F0Fu), hhi), x + 16);
        return dd * ((float)sc0 * slo + (float)sc1 * shi) - dmin * ((float)m0 * xs[0] + (float)m1 * xs[1]);
    }
};

template <> struct Chunk<T_Q6_K> {
    static constexpr int NRUN = 4, RUNLEN = 16, E = 64;
    struct Data { U4 ql0, ql32, qh; uint32_t sc_lo, sc_hi; uint16_t d; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 64; }
    // chunk c: block b=c/4, 128-half i=(c%4)/2, l-range m=c%2 (l = 16m..16m+15); run r = quadrant
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return (c >> 2) * 256 + ((c & 3) >> 1) * 128 + (c & 1) * 16 + r * 32; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        uint32_t b = c >> 2, i = (c & 3) >> 1, m = c & 1;
        const uint8_t *ql = row + (size_t)b * 128 + i * 64 + m * 16;
        const uint8_t *qh = row + (size_t)nb * 128 + (size_t)b * 64 + i * 32 + m * 16;
        const uint8_t *sc = row + (size_t)nb * 192 + (size_t)b * 16 + i * 8;
        Data d;
        d.ql0 = ld128(ql); d.ql32 = ld128(ql + 32); d.qh = ld128(qh);
        memcpy(&d.sc_lo, sc, 4); memcpy(&d.sc_hi, sc + 4, 4);
        d.d = ld16(row + (size_t)nb * 208 + (size_t)b * 2);
        return d;
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        const uint32_t m = c & 1;
        // scales[8i + m + {0,2,4,6}]
        float s0 = (float)(int8_t)((d.sc_lo >> (8 * m)) & 0xff), s1 = (float)(int8_t)((d.sc_lo >> (8 * (m + 2))) & 0xff);
        float s2 = (float)(int8_t)((d.sc_hi >> (8 * m)) & 0xff), s3 = (float)(int8_t)((d.sc_hi >> (8 * (m + 2))) & 0xff);
        U4 q1 = or4(and4(d.ql0, 0x0F0F0F0Fu), shl4(and4(d.qh, 0x03030303u), 4));
        U4 q2 = or4(and4(d.ql32, 0x0F0F0F0Fu), shl4(and4(shr4(d.qh, 2), 0x03030303u), 4));
        U4 q3 = or4(and4(shr4(d.ql0, 4), 0x0F0F0F0Fu), shl4(and4(shr4(d.qh, 4), 0x03030303u), 4));
        U4 q4 = or4(and4(shr4(d.ql32, 4), 0x0F0F0F0Fu), shl4(and4(shr4(d.qh, 6), 0x03030303u), 4));
        float a = s0 * (dot16b(q1, x) - 32.0f * xs[0]) + s1 * (dot16b(q2, x + 16) - 32.0f * xs[1]);
        float b = s2 * (dot16b(q3, x + 32) - 32.0f * xs[2]) + s3 * (dot16b(q4, x + 48) - 32.0f * xs[3]);
        return gemv_f16(d.d) * (a + b);
    }
};

template <> struct Chunk<T_Q8_0> {
    static constexpr int NRUN = 1, RUNLEN = 16, E = 16;
    struct Data { U4 qs; uint16_t d; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 16; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 16; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        return Data{ld128(row + (size_t)c * 16), ld16(row + (size_t)nb * 32 + (size_t)(c >> 1) * 2)};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        // int8 -> (q + 128) as unsigned bytes; the 128 comes back out through the run sum
        float s = dot16b(xor4(d.qs, 0x80808080u), x);
        return gemv_f16(d.d) * (s - 128.0f * xs[0]);
    }
};

template <> struct Chunk<T_Q4_0> {
    static constexpr int NRUN = 2, RUNLEN = 16, E = 32;
    struct Data { U4 qs; uint16_t d; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 32; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 32 + r * 16; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        return Data{ld128(row + (size_t)c * 16), ld16(row + (size_t)nb * 16 + (size_t)c * 2)};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        float slo = dot16b(and4(d.qs, 0x0F0F0F0Fu), x);
        float shi = dot16b(and4(shr4(d.qs, 4), 0x0F0F0F0Fu), x + 16);
        return gemv_f16(d.d) * ((slo + shi) - 8.0f * (xs[0] + xs[1]));
    }
};

// bit k of the low 4 bits of `nib` into bit 4 of byte k: the fifth bit of four 5-bit values
SLAI_HD uint32_t spread4(uint32_t nib) { return (((nib & 0xFu) * 0x00204081u) & 0x01010101u) << 4; }
SLAI_HD U4 high_bits16(uint32_t bits16) {   // bits 0..15 -> 0x10 in bytes 0..15
    return U4{spread4(bits16), spread4(bits16 >> 4), spread4(bits16 >> 8), spread4(bits16 >> 12)};
}

template <> struct Chunk<T_Q4_1> {     // one 32-element block: value = q*d + m
    static constexpr int NRUN = 2, RUNLEN = 16, E = 32;
    struct Data { U4 qs; uint32_t dm; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 32; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 32 + r * 16; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        uint32_t dm; memcpy(&dm, row + (size_t)nb * 16 + (size_t)c * 4, 4);
        return Data{ld128(row + (size_t)c * 16), dm};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        float slo = dot16b(and4(d.qs, 0x0F0F0F0Fu), x);
        float shi = dot16b(and4(shr4(d.qs, 4), 0x0F0F0F0Fu), x + 16);
        return gemv_f16((uint16_t)(d.dm & 0xffffu)) * (slo + shi) + gemv_f16((uint16_t)(d.dm >> 16)) * (xs[0] + xs[1]);
    }
};

template <> struct Chunk<T_Q5_0> {     // value = (q5 - 16) * d
    static constexpr int NRUN = 2, RUNLEN = 16, E = 32;
    struct Data { U4 qs; uint32_t qh; uint16_t d; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 32; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 32 + r * 16; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        uint32_t qh; memcpy(&qh, row + (size_t)nb * 16 + (size_t)c * 4, 4);
        return Data{ld128(row + (size_t)c * 16), qh, ld16(row + (size_t)nb * 20 + (size_t)c * 2)};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        float slo = dot16b(or4(and4(d.qs, 0x0F0F0F0Fu), high_bits16(d.qh)), x);
        float shi = dot16b(or4(and4(shr4(d.qs, 4), 0x0F0F0F0Fu), high_bits16(d.qh >> 16)), x + 16);
        return gemv_f16(d.d) * ((slo + shi) - 16.0f * (xs[0] + xs[1]));
    }
};

template <> struct Chunk<T_Q5_1> {     // value = q5 * d + m
    static constexpr int NRUN = 2, RUNLEN = 16, E = 32;
    struct Data { U4 qs; uint32_t qh, dm; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 32; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 32 + r * 16; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        uint32_t qh, dm;
        memcpy(&qh, row + (size_t)nb * 16 + (size_t)c * 4, 4);
        memcpy(&dm, row + (size_t)nb * 20 + (size_t)c * 4, 4);
        return Data{ld128(row + (size_t)c * 16), qh, dm};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        float slo = dot16b(or4(and4(d.qs, 0x0F0F0F0Fu), high_bits16(d.qh)), x);
        float shi = dot16b(or4(and4(shr4(d.qs, 4), 0x0F0F0F0Fu), high_bits16(d.qh >> 16)), x + 16);
        return gemv_f16((uint16_t)(d.dm & 0xffffu)) * (slo + shi) + gemv_f16((uint16_t)(d.dm >> 16)) * (xs[0] + xs[1]);
    }
};

template <> struct Chunk<T_Q8_K> {     // 16 of the 256 int8 of a block, f32 scale
    static constexpr int NRUN = 1, RUNLEN = 16, E = 16;
    struct Data { U4 qs; float d; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 16; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 16; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) {
        float d; memcpy(&d, row + (size_t)nb * 256 + (size_t)(c >> 4) * 4, 4);
        return Data{ld128(row + (size_t)c * 16), d};
    }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        float s = dot16b(xor4(d.qs, 0x80808080u), x);
        return d.d * (s - 128.0f * xs[0]);
    }
};

template <> struct Chunk<T_F16> {
    static constexpr int NRUN = 1, RUNLEN = 8, E = 8;
    struct Data { U4 v; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 8; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 8; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) { return Data{ld128(row + (size_t)c * 16)}; }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        const uint32_t w[4] = {d.v.x, d.v.y, d.v.z, d.v.w};
        float a = 0.0f;
        for (int i = 0; i < 4; ++i) {
            a = fmaf(gemv_f16((uint16_t)(w[i] & 0xffffu)), x[2 * i], a);
            a = fmaf(gemv_f16((uint16_t)(w[i] >> 16)), x[2 * i + 1], a);
        }
        return a;
    }
};

template <> struct Chunk<T_F32> {
    static constexpr int NRUN = 1, RUNLEN = 4, E = 4;
    struct Data { U4 v; };
    SLAI_HD static uint32_t nchunks(uint32_t ncols) { return ncols / 4; }
    SLAI_HD static uint32_t run_col(uint32_t c, int r) { return c * 4; }
    SLAI_HD static Data load(const uint8_t *row, uint32_t nb, uint32_t c) { return Data{ld128(row + (size_t)c * 16)}; }
    SLAI_HD static float dot(const Data &d, uint32_t c, const float *x, const float *xs) {
        float a = bits_to_float(d.v.x) * x[0];
        a = fmaf(bits_to_float(d.v.y), x[1], a);
        a = fmaf(bits_to_float(d.v.z), x[2], a);
        a = fmaf(bits_to_float(d.v.w), x[3], a);
        return a;
    }
};

}  // namespace slai
