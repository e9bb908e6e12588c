// "Tiled" device layout of quantized matrices and the per-lane block decoders of the
// row-per-lane GEMV (kernels_gemv_tiled.hip).
//
// Why a second layout: with the row-major layout every lane that shares a block decodes the
// block header again for every row.  Here a lane owns one ROW of a tile and walks whole
// 256-column super-blocks ("cblocks"), so a header is decoded once per 256 weights, there is no
// per-row cross-lane reduction, and every wave-wide load instruction reads 1024 contiguous bytes.
//
// Geometry: a wave covers a tile of ROWS rows x KQ cblocks, ROWS*KQ = 64, (ROWS,KQ) in
// {(16,4),(32,2),(64,1)}; lane = kq*ROWS + r.  A cblock is PT 16-byte "pieces" per row (+ an
// optional 2-byte tail).  Unit (tile t, column group g) lives at
//     base + (t*ngroups + g) * unit_bytes,   unit_bytes = PT*1024 (+128 tail),
// piece p of lane L at  unit + p*1024 + L*16, tail of lane L at unit + PT*1024 + L*2.
// Rows beyond nrows and cblocks beyond ncols/256 are zero-filled (they decode to 0).
//
//   Q4_K: cblock = one 144-byte block, pieces = [d,dmin,scales | qs x8]                  PT = 9
//   Q6_K: cblock = one block, pieces = [ql x8 | qh x4 | scales], tail = d               PT = 13
//   Q8_0: cblock = eight 34-byte blocks, pieces = [qs x16 | the eight f16 scales]        PT = 17
//
// Activations: a 16-lane DPP row holds the 256 activations of its cblock in 16 registers
// (register i, lane j <-> x[cb*256 + 16*i + j]); element (i, k) reaches every lane of the row
// through a row_newbcast:k DPP operand of the FMA, so x costs neither LDS nor shuffles.
//
// Block arithmetic follows crates/slai/src/quantization.rs (BlockQ4K :322-379,
// get_scale_min_k4 :381-389, BlockQ6K :204-244, BlockQ8_0 :29-42).
#pragma once
#include "quant_formats.h"

namespace slai {

struct TiledGeom {
    int type = 0;
    uint32_t nrows = 0, ncols = 0;
    uint32_t rows_log2 = 4;     // ROWS = 1 << rows_log2, KQ = 64 >> rows_log2
    uint32_t ncb = 0;           // cblocks per row = ncols / 256
    uint32_t ngroups = 0;       // ceil(ncb / KQ)
    uint32_t ntiles = 0;        // ceil(nrows / ROWS)
    uint32_t pieces = 0;        // PT
    uint32_t unit_bytes = 0;
};

SLAI_HD bool tiled_supported(int t) { return t == T_Q4_K || t == T_Q6_K || t == T_Q8_0; }
SLAI_HD uint32_t tiled_pieces(int t) { return t == T_Q4_K ? 9u : (t == T_Q6_K ? 13u : 17u); }
SLAI_HD uint32_t tiled_tail(int t) { return t == T_Q6_K ? 128u : 0u; }

SLAI_HD TiledGeom tiled_geom(int t, uint32_t nrows, uint32_t ncols) {
    TiledGeom g;
    g.type = t; g.nrows = nrows; g.ncols = ncols; g.ncb = ncols / 256;
    uint32_t kq;
    if (g.ncb % 4 == 0 || g.ncb >= 20) kq = 4;
    else if (g.ncb % 2 == 0 || g.ncb >= 10) kq = 2;
    else kq = 1;
    g.rows_log2 = kq == 4 ? 4 : (kq == 2 ? 5 : 6);
    g.ngroups = (g.ncb + kq - 1) / kq;
    const uint32_t rows = 1u << g.rows_log2;
    g.ntiles = (nrows + rows - 1) / rows;
    g.pieces = tiled_pieces(t);
    g.unit_bytes = g.pieces * 1024 + tiled_tail(t);
    return g;
}
SLAI_HD size_t tiled_bytes(const TiledGeom &g) { return (size_t)g.ntiles * g.ngroups * g.unit_bytes; }

// Address of logical byte `b` of the cblock (row, cb); b < PT*16 addresses the pieces, larger b the tail.
SLAI_HD size_t tiled_byte_offset(const TiledGeom &g, uint32_t row, uint32_t cb, uint32_t b) {
    const uint32_t rows = 1u << g.rows_log2, kq_n = 64u >> g.rows_log2;
    const uint32_t t = row >> g.rows_log2, r = row & (rows - 1), grp = cb / kq_n, kq = cb % kq_n;
    const uint32_t lane = kq * rows + r;
    const size_t unit = ((size_t)t * g.ngroups + grp) * g.unit_bytes;
    if (b < g.pieces * 16) return unit + (size_t)(b / 16) * 1024 + lane * 16 + (b % 16);
    return unit + (size_t)g.pieces * 1024 + lane * 2 + (b - g.pieces * 16);
}

// GGUF block `blk` of row `row` (verbatim bytes at src) into the tiled layout.
SLAI_HD void tiled_repack_block(const TiledGeom &g, const uint8_t *src, uint8_t *dst, uint32_t row, uint32_t blk) {
    switch (g.type) {
    case T_Q4_K:
        for (uint32_t b = 0; b < 144; ++b) dst[tiled_byte_offset(g, row, blk, b)] = src[b];
        break;
    case T_Q6_K:   // ql[128] qh[64] scales[16] are pieces 0..12; d is the tail
        for (uint32_t b = 0; b < 210; ++b) dst[tiled_byte_offset(g, row, blk, b)] = src[b];
        break;
    case T_Q8_0: { // cblock = blocks 8c..8c+7: logical bytes [qs: 32*bi + i][d: 256 + 2*bi]
        const uint32_t cb = blk / 8, bi = blk % 8;
        for (uint32_t i = 0; i < 32; ++i) dst[tiled_byte_offset(g, row, cb, 32 * bi + i)] = src[2 + i];
        dst[tiled_byte_offset(g, row, cb, 256 + 2 * bi)] = src[0];
        dst[tiled_byte_offset(g, row, cb, 256 + 2 * bi + 1)] = src[1];
        break;
    }
    default: break;
    }
}

// Bit-exact single-element dequantisation from the tiled layout (same arithmetic as dequant_elem).
SLAI_HD float tiled_dequant_elem(const TiledGeom &g, const uint8_t *base, uint32_t row, uint32_t col) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
    const uint32_t cb = col / 256, e = col % 256;
#define TB(b) base[tiled_byte_offset(g, row, cb, (b))]
    switch (g.type) {
    case T_Q4_K: {
        U4 hdr;
        uint8_t hb[16];
        for (int i = 0; i < 16; ++i) hb[i] = TB(i);
        memcpy(&hdr, hb, 16);
        float d = decode_f16((uint16_t)(hdr.x & 0xffffu)), dmin = decode_f16((uint16_t)(hdr.x >> 16));
        const uint32_t jp = e / 64, w = e % 64, hi = w >= 32, l = w % 32;
        uint32_t sc, m;
        scale_min_k4(hdr, (int)(jp * 2 + hi), sc, m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        uint8_t byte = TB(16 + jp * 32 + l);
        uint32_t q = hi ? (byte >> 4) : (byte & 0xF);
        return d1 * (float)q - m1;
    }
    case T_Q6_K: {
        const uint32_t i = e / 128, r = (e % 128) / 32, l = e % 32, is = l / 16;
        uint16_t dh = (uint16_t)(TB(208) | (TB(209) << 8));
        float d = decode_f16(dh);
        uint8_t byte = TB(i * 64 + (r & 1) * 32 + l);
        uint32_t nib = (r < 2) ? (byte & 0xF) : (byte >> 4);
        uint32_t two = (TB(128 + i * 32 + l) >> (2 * r)) & 3u;
        int q = (int)(int8_t)(nib | (two << 4)) - 32;
        return d * (float)(int8_t)TB(192 + i * 8 + is + 2 * r) * (float)q;
    }
    case T_Q8_0: {
        const uint32_t bi = e / 32;
        uint16_t dh = (uint16_t)(TB(256 + 2 * bi) | (TB(256 + 2 * bi + 1) << 8));
        return (float)(int8_t)TB(e) * decode_f16(dh);
    }
    default: return 0.0f;
    }
#undef TB
}

// ---------------------------------------------------------------------------
// Per-lane block dot products.  `X` provides the activations of the lane's cblock:
//   X.fma4<I,W>(w, acc) -> acc + sum_{b<4} byte_b(w) * x[16*I + 4*W + b]
//        (device: four byte->float conversions and four v_fmac_f32 whose x operand is a
//         row_newbcast DPP read of register I)
//   X.sum16(I)   -> sum_k x[16*I + k]  (row sums, loop invariant, precomputed).  Q4_K and Q8_0 only
//                   ever use sum16(2n) + sum16(2n+1); an accessor may keep that pair sum in the even
//                   slot and 0 in the odd one.
// ---------------------------------------------------------------------------
template <int I, class X> SLAI_HD float piece_dot(const X &x, const U4 &q, float acc) {
    // q holds sixteen unsigned byte values; byte k pairs with x[16*I + k]:  acc += q_k * x[16*I + k]
    acc = x.template fma4<I, 0>(q.x, acc);
    acc = x.template fma4<I, 1>(q.y, acc);
    acc = x.template fma4<I, 2>(q.z, acc);
    acc = x.template fma4<I, 3>(q.w, acc);
    return acc;
}

// Two independent accumulation chains interleaved word by word (keeps the FMA pipeline fed when a
// SIMD holds a single wave).
template <int I1, int I2, class X> SLAI_HD void piece_dot2(const X &x, const U4 &q1, const U4 &q2, float &a1, float &a2) {
    a1 = x.template fma4<I1, 0>(q1.x, a1); a2 = x.template fma4<I2, 0>(q2.x, a2);
    a1 = x.template fma4<I1, 1>(q1.y, a1); a2 = x.template fma4<I2, 1>(q2.y, a2);
    a1 = x.template fma4<I1, 2>(q1.z, a1); a2 = x.template fma4<I2, 2>(q2.z, a2);
    a1 = x.template fma4<I1, 3>(q1.w, a1); a2 = x.template fma4<I2, 3>(q2.w, a2);
}

template <int T> struct Tiled;

template <> struct Tiled<T_Q4_K> {
    static constexpr int PT = 9;
    static constexpr bool TAIL = false;
    struct Data { U4 p[9]; };
    template <int J, class X> SLAI_HD static void pair(const Data &d, const X &x, uint32_t scw, uint32_t mw, float &accd, float &accm) {
        // sub-blocks 2J (low nibbles) and 2J+1 (high nibbles) of qs pieces 2J, 2J+1
        const U4 &a = d.p[1 + 2 * J], &b = d.p[2 + 2 * J];
        float slo = 0.0f, shi = 0.0f;
        piece_dot2<4 * J, 4 * J + 2>(x, and4(a, 0x0F0F0F0Fu), and4(shr4(a, 4), 0x0F0F0F0Fu), slo, shi);
        piece_dot2<4 * J + 1, 4 * J + 3>(x, and4(b, 0x0F0F0F0Fu), and4(shr4(b, 4), 0x0F0F0F0Fu), slo, shi);
        constexpr int sh = (J & 1) * 16;
        accd = fmaf((float)((scw >> sh) & 0xffu), slo, accd);
        accd = fmaf((float)((scw >> (sh + 8)) & 0xffu), shi, accd);
        accm = fmaf((float)((mw >> sh) & 0xffu), x.sum16(4 * J) + x.sum16(4 * J + 1), accm);
        accm = fmaf((float)((mw >> (sh + 8)) & 0xffu), x.sum16(4 * J + 2) + x.sum16(4 * J + 3), accm);
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t /*tail*/, const X &x) {
        const U4 &h = d.p[0];
        const float dd = decode_f16((uint16_t)(h.x & 0xffffu)), dmin = decode_f16((uint16_t)(h.x >> 16));
        // all eight 6-bit scales / mins at once (quantization.rs:381-389 applied bytewise)
        const uint32_t sc_lo = h.y & 0x3f3f3f3fu, m_lo = h.z & 0x3f3f3f3fu;
        const uint32_t sc_hi = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);
        const uint32_t m_hi = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
        float accd = 0.0f, accm = 0.0f;
        pair<0>(d, x, sc_lo, m_lo, accd, accm);
        pair<1>(d, x, sc_lo, m_lo, accd, accm);
        pair<2>(d, x, sc_hi, m_hi, accd, accm);
        pair<3>(d, x, sc_hi, m_hi, accd, accm);
        return dd * accd - dmin * accm;
    }
};

template <> struct Tiled<T_Q6_K> {
    static constexpr int PT = 13;
    static constexpr bool TAIL = true;
    struct Data { U4 p[13]; };
    template <int I, int M, class X> SLAI_HD static float half_m(const Data &d, const X &x, float acc) {
        // l = 16M..16M+15 of the 128-half I: four quadrants, scales[8I + 2r + M]
        const U4 &ql0 = d.p[4 * I + M], &ql32 = d.p[4 * I + 2 + M], &qh = d.p[8 + 2 * I + M];
        const U4 &scp = d.p[12];
        const uint32_t scw = I == 0 ? scp.x : scp.z;    // scale bytes 8I .. 8I+3
        const uint32_t scw2 = I == 0 ? scp.y : scp.w;   // scale bytes 8I+4 .. 8I+7
        const U4 q1 = or4(and4(ql0, 0x0F0F0F0Fu), shl4(and4(qh, 0x03030303u), 4));
        const U4 q2 = or4(and4(ql32, 0x0F0F0F0Fu), shl4(and4(shr4(qh, 2), 0x03030303u), 4));
        const U4 q3 = or4(and4(shr4(ql0, 4), 0x0F0F0F0Fu), shl4(and4(shr4(qh, 4), 0x03030303u), 4));
        const U4 q4 = or4(and4(shr4(ql32, 4), 0x0F0F0F0Fu), shl4(and4(shr4(qh, 6), 0x03030303u), 4));
        const float s0 = (float)(int8_t)((scw >> (8 * M)) & 0xff), s1 = (float)(int8_t)((scw >> (8 * (M + 2))) & 0xff);
        const float s2 = (float)(int8_t)((scw2 >> (8 * M)) & 0xff), s3 = (float)(int8_t)((scw2 >> (8 * (M + 2))) & 0xff);
        float t1 = 0.0f, t2 = 0.0f, t3 = 0.0f, t4 = 0.0f;
        piece_dot2<8 * I + M, 8 * I + 2 + M>(x, q1, q2, t1, t2);
        piece_dot2<8 * I + 4 + M, 8 * I + 6 + M>(x, q3, q4, t3, t4);
        acc = fmaf(s0, t1 - 32.0f * x.sum16(8 * I + M), acc);
        acc = fmaf(s1, t2 - 32.0f * x.sum16(8 * I + 2 + M), acc);
        acc = fmaf(s2, t3 - 32.0f * x.sum16(8 * I + 4 + M), acc);
        acc = fmaf(s3, t4 - 32.0f * x.sum16(8 * I + 6 + M), acc);
        return acc;
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t tail, const X &x) {
        float acc = 0.0f;
        acc = half_m<0, 0>(d, x, acc);
        acc = half_m<0, 1>(d, x, acc);
        acc = half_m<1, 0>(d, x, acc);
        acc = half_m<1, 1>(d, x, acc);
        return decode_f16(tail) * acc;
    }
};

template <> struct Tiled<T_Q8_0> {
    static constexpr int PT = 17;
    static constexpr bool TAIL = false;
    struct Data { U4 p[17]; };
    template <int B, class X> SLAI_HD static float blk(const Data &d, const X &x, uint32_t dword, float acc) {
        // block B of the cblock: qs pieces 2B, 2B+1; int8 -> unsigned via ^0x80, the 128 comes back through the sums
        float s = 0.0f, s2 = 0.0f;
        piece_dot2<2 * B, 2 * B + 1>(x, xor4(d.p[2 * B], 0x80808080u), xor4(d.p[2 * B + 1], 0x80808080u), s, s2);
        s = (s + s2) - 128.0f * (x.sum16(2 * B) + x.sum16(2 * B + 1));
        const float dd = decode_f16((uint16_t)((B & 1) ? (dword >> 16) : (dword & 0xffffu)));
        return fmaf(dd, s, acc);
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t /*tail*/, const X &x) {
        const U4 &s = d.p[16];
        float acc = 0.0f;
        acc = blk<0>(d, x, s.x, acc); acc = blk<1>(d, x, s.x, acc);
        acc = blk<2>(d, x, s.y, acc); acc = blk<3>(d, x, s.y, acc);
        acc = blk<4>(d, x, s.z, acc); acc = blk<5>(d, x, s.z, acc);
        acc = blk<6>(d, x, s.w, acc); acc = blk<7>(d, x, s.w, acc);
        return acc;
    }
};

}  // namespace slai
