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
//   Q4_0: cblock = eight 18-byte blocks, pieces = [qs x8 (one block each) | the eight f16 scales]  PT = 9
//   Q5_K: cblock = one 176-byte block, pieces = [d,dmin,scales | qh x2 | qs x8]          PT = 11
//
// Activations: a 16-lane DPP row holds the 256 activations of its cblock in 16 registers
// (register i, lane j <-> x[cb*256 + 16*i + j]); element (i, k) reaches every lane of the row
// through a row_newbcast:k DPP operand of the FMA, so x costs neither LDS nor shuffles.
//
// Block arithmetic follows crates/slai/src/quantization.rs (BlockQ4K :322-379,
// get_scale_min_k4 :381-389, BlockQ6K :204-244, BlockQ8_0 :29-42).
#pragma once
#include <type_traits>
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

SLAI_HD bool tiled_supported(int t) { return t == T_Q4_K || t == T_Q6_K || t == T_Q8_0 || t == T_Q4_0 || t == T_Q5_K; }
SLAI_HD uint32_t tiled_pieces(int t) {
    switch (t) {
    case T_Q4_K: case T_Q4_0: return 9u;
    case T_Q5_K: return 11u;
    case T_Q6_K: return 13u;
    default: return 17u;
    }
}
SLAI_HD uint32_t tiled_tail(int t) { return t == T_Q6_K ? 128u : 0u; }

// force_rows_log2: 0 = choose by column count, else 4, 5 or 6.
SLAI_HD TiledGeom tiled_geom(int t, uint32_t nrows, uint32_t ncols, uint32_t force_rows_log2 = 0) {
    TiledGeom g;
    g.type = t; g.nrows = nrows; g.ncols = ncols; g.ncb = ncols / 256;
    uint32_t kq;
    if (force_rows_log2 >= 4 && force_rows_log2 <= 6) kq = 64u >> force_rows_log2;
    else if (g.ncb % 4 == 0 || g.ncb >= 20) kq = 4;
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
    case T_Q5_K:
        for (uint32_t b = 0; b < 176; ++b) dst[tiled_byte_offset(g, row, blk, b)] = src[b];
        break;
    case T_Q4_0: { // cblock = blocks 8c..8c+7: logical bytes [qs: 16*bi + i][d: 128 + 2*bi]
        const uint32_t cb = blk / 8, bi = blk % 8;
        for (uint32_t i = 0; i < 16; ++i) dst[tiled_byte_offset(g, row, cb, 16 * bi + i)] = src[2 + i];
        dst[tiled_byte_offset(g, row, cb, 128 + 2 * bi)] = src[0];
        dst[tiled_byte_offset(g, row, cb, 128 + 2 * bi + 1)] = src[1];
        break;
    }
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
    case T_Q4_K: case T_Q5_K: {
        U4 hdr;
        uint8_t hb[16];
        for (int i = 0; i < 16; ++i) hb[i] = TB(i);
        memcpy(&hdr, hb, 16);
        float d = decode_f16((uint16_t)(hdr.x & 0xffffu)), dmin = decode_f16((uint16_t)(hdr.x >> 16));
        const uint32_t jp = e / 64, w = e % 64, hi = w >= 32, l = w % 32;
        uint32_t sc, m;
        scale_min_k4(hdr, (int)(jp * 2 + hi), sc, m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        uint8_t byte = TB((g.type == T_Q4_K ? 16 : 48) + jp * 32 + l);
        uint32_t q = hi ? (byte >> 4) : (byte & 0xF);
        if (g.type == T_Q5_K) q += ((TB(16 + l) >> (2 * jp + hi)) & 1u) ? 16u : 0u;
        return d1 * (float)q - m1;
    }
    case T_Q4_0: {
        const uint32_t bi = e / 32, j = e % 32;
        uint16_t dh = (uint16_t)(TB(128 + 2 * bi) | (TB(128 + 2 * bi + 1) << 8));
        uint8_t byte = TB(16 * bi + (j & 15));
        int q = (int)(j < 16 ? (byte & 0xF) : (byte >> 4)) - 8;
        return (float)q * decode_f16(dh);
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
// Per-lane block dot products.  Every format walks its 256-column super-block in eight STAGES; a stage
// multiplies two 16-byte pieces of quantised values with two 16-element chunks (I1, I2) of the activations.
// `X` provides the activations of the lane's super-block:
//   X.stage<I1,I2>()          -> whatever X needs to serve chunks I1 and I2 (a tag for register-resident
//                                activations; the loaded values for activations fetched on demand).  The
//                                dot products request stage k+1 before they compute stage k.
//   X.fma4<SLOT,W>(st, w, acc) -> acc + sum_{b<4} byte_b(w) * x[16*I_SLOT + 4*W + b]
//   X.sum16(i)                -> sum_k x[16*i + k]; all uses come before the first stage.
// dotn<N> computes the dot products of N matrices' rows with the same activations in lockstep (N = 2: the
// gate/up pair), so that on-demand activations are fetched once.
// ---------------------------------------------------------------------------
// binary16 -> binary32 for block scales inside the dot products: the hardware converter on the device (one
// instruction; identical to decode_f16 for every non-NaN input), decode_f16 on the host.
SLAI_HD float scale_f16(uint16_t h) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (float)__builtin_bit_cast(_Float16, h);
#else
    return decode_f16(h);
#endif
}

// The quantised pieces may be fetched while the dot product runs: `L` (a "loader") issues the load of piece P of
// every matrix with L.piece<P>() (and L.tail() for the 2-byte tail); the dot products call lead() for what the
// first L::LEAD (>= L::DEPTH) stages need and ahead<K>() at stage K for what stage K + L::DEPTH needs, so a wave
// never has more than a few requests waiting to be issued and starts multiplying as soon as its first pieces arrive.  NoLoader is for
// data that is already in registers.
struct NoLoader {
    static constexpr int DEPTH = 8, LEAD = 8;
    template <int P> SLAI_HD void piece() const {}
    SLAI_HD void tail() const {}
};
#if defined(__HIP_DEVICE_COMPILE__)
#define SLAI_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
#else
#define SLAI_SCHED_FENCE() ((void)0)
#endif

template <class X, class S> SLAI_HD void stage_dot(const X &x, const S &st, const U4 &q1, const U4 &q2, float &a1, float &a2) {
    // q1 pairs with chunk I1, q2 with chunk I2; two independent accumulation chains interleaved word by word
    a1 = x.template fma4<0, 0>(st, q1.x, a1); a2 = x.template fma4<1, 0>(st, q2.x, a2);
    a1 = x.template fma4<0, 1>(st, q1.y, a1); a2 = x.template fma4<1, 1>(st, q2.y, a2);
    a1 = x.template fma4<0, 2>(st, q1.z, a1); a2 = x.template fma4<1, 2>(st, q2.z, a2);
    a1 = x.template fma4<0, 3>(st, q1.w, a1); a2 = x.template fma4<1, 3>(st, q2.w, a2);
}

// Whether an activation operand multiplies 4-bit weights unconverted (its nib8; see ScalarX): operands that do not say
// so do not.
template <class X, class = void> struct takes_nibbles : std::false_type {};
template <class X> struct takes_nibbles<X, std::void_t<decltype(X::NIBBLE_MIX)>> : std::bool_constant<X::NIBBLE_MIX> {};

template <int T> struct Tiled;

template <> struct Tiled<T_Q4_K> {
    static constexpr int PT = 9;
    static constexpr bool TAIL = false;
    struct Data { U4 p[9]; };
    // stage K: qs piece 1+K; low nibbles <-> chunk 4J+H (sub-block 2J), high nibbles <-> chunk 4J+2+H (sub-block 2J+1)
    static constexpr int c1(int K) { return 4 * (K / 2) + (K % 2); }
    static constexpr int c2(int K) { return 4 * (K / 2) + 2 + (K % 2); }
    template <int N> struct Acc { float accd[N], slo[N], shi[N]; uint32_t sc_lo[N], sc_hi[N]; };
    template <int K, int N, class X, class S> SLAI_HD static void compute(const Data *const *d, const X &x, const S &st, Acc<N> &a) {
        constexpr int J = K / 2, H = K % 2;
        for (int n = 0; n < N; ++n) {
            const U4 &q = d[n]->p[1 + K];
            // (operands that take the nibbles unconverted leave slo scaled by 2^-24 and shi by 2^-20: the 16 is taken
            // out of the high sub-block's scale here, the 2^-24 out of the block scale in dotn)
            if constexpr (takes_nibbles<X>::value) {
                x.template nib8<0>(st, q.x, a.slo[n], a.shi[n]); x.template nib8<1>(st, q.y, a.slo[n], a.shi[n]);
                x.template nib8<2>(st, q.z, a.slo[n], a.shi[n]); x.template nib8<3>(st, q.w, a.slo[n], a.shi[n]);
            } else {
                stage_dot(x, st, and4(q, 0x0F0F0F0Fu), and4(shr4(q, 4), 0x0F0F0F0Fu), a.slo[n], a.shi[n]);
            }
            if (H == 1) {
                const uint32_t scw = J < 2 ? a.sc_lo[n] : a.sc_hi[n];
                constexpr int sh = (J & 1) * 16;
                constexpr float hi_factor = takes_nibbles<X>::value ? 0.0625f : 1.0f;
                a.accd[n] = fmaf((float)((scw >> sh) & 0xffu), a.slo[n], a.accd[n]);
                a.accd[n] = fmaf((float)((scw >> (sh + 8)) & 0xffu) * hi_factor, a.shi[n], a.accd[n]);
                a.slo[n] = 0.0f; a.shi[n] = 0.0f;
            }
        }
    }
    // stage K reads piece 1 + K; the header is piece 0
    template <int P, class L> SLAI_HD static void lead_from(const L &ld) {
        if constexpr (P <= L::LEAD && P < PT) { ld.template piece<P>(); lead_from<P + 1>(ld); }
    }
    template <class L> SLAI_HD static void lead(const L &ld) { lead_from<0>(ld); }      // header + stages 0 .. LEAD-1
    template <int K, class L> SLAI_HD static void ahead(const L &ld) {
        if constexpr (1 + K + L::DEPTH < PT && 1 + K + L::DEPTH > L::LEAD) ld.template piece<1 + K + L::DEPTH>();
    }
    template <int K, int N, class X, class S, class L> SLAI_HD static void stages(const Data *const *d, const X &x, const S &st, Acc<N> &a, const L &ld) {
        ahead<K>(ld);
        SLAI_SCHED_FENCE();
        if constexpr (K < 7) {
            const auto nxt = x.template stage<c1(K + 1), c2(K + 1)>();
            compute<K, N>(d, x, st, a);
            stages<K + 1, N>(d, x, nxt, a, ld);
        } else {
            compute<K, N>(d, x, st, a);
        }
    }
    template <int N, class X, class L = NoLoader> SLAI_HD static void dotn(const Data *const *d, const uint16_t * /*tail*/, const X &x, float *out, const L &ld = L()) {
        Acc<N> a;
        float dd[N], dmin[N], accm[N];
        for (int n = 0; n < N; ++n) {
            const U4 &h = d[n]->p[0];
            dd[n] = scale_f16((uint16_t)(h.x & 0xffffu)); dmin[n] = scale_f16((uint16_t)(h.x >> 16));
            // all eight 6-bit scales / mins at once (quantization.rs:381-389 applied bytewise)
            a.sc_lo[n] = h.y & 0x3f3f3f3fu;
            a.sc_hi[n] = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);
            const uint32_t m_lo = h.z & 0x3f3f3f3fu;
            const uint32_t m_hi = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
            float am = 0.0f;
            for (int sb = 0; sb < 8; ++sb) {       // offset term: min of sub-block sb times the sum of its 32 activations
                const uint32_t mw = sb < 4 ? m_lo : m_hi;
                am = fmaf((float)((mw >> (8 * (sb & 3))) & 0xffu), x.sum16(2 * sb) + x.sum16(2 * sb + 1), am);
            }
            accm[n] = am; a.accd[n] = 0.0f; a.slo[n] = 0.0f; a.shi[n] = 0.0f;
        }
        const auto st0 = x.template stage<c1(0), c2(0)>();
        stages<0, N>(d, x, st0, a, ld);
        constexpr float unit = takes_nibbles<X>::value ? 16777216.0f : 1.0f;             // accd is in units of 2^-24 there
        for (int n = 0; n < N; ++n) out[n] = (dd[n] * unit) * a.accd[n] - dmin[n] * accm[n];
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t tail, const X &x) {
        const Data *dp[1] = {&d};
        float out[1];
        dotn<1>(dp, &tail, x, out);
        return out[0];
    }
};

template <> struct Tiled<T_Q6_K> {
    static constexpr int PT = 13;
    static constexpr bool TAIL = true;
    struct Data { U4 p[13]; };
    // stage K: 128-half I = K/4, l-range M = (K/2)%2 (l = 16M..16M+15), quadrant pair P = K%2:
    //   P = 0: quadrants 0,1 <-> chunks 8I+M, 8I+2+M;  P = 1: quadrants 2,3 <-> chunks 8I+4+M, 8I+6+M
    static constexpr int c1(int K) { return 8 * (K / 4) + 4 * (K % 2) + ((K / 2) % 2); }
    static constexpr int c2(int K) { return c1(K) + 2; }
    // scale of quadrant r (0..3) of (I, M): scales[8I + 2r + M]
    SLAI_HD static float scale_of(const Data &d, int I, int M, int r) {
        const U4 &scp = d.p[12];
        const uint32_t w = r < 2 ? (I == 0 ? scp.x : scp.z) : (I == 0 ? scp.y : scp.w);
        return (float)(int8_t)((w >> (8 * (M + 2 * (r & 1)))) & 0xff);
    }
    template <int K, int N, class X, class S> SLAI_HD static void compute(const Data *const *d, const X &x, const S &st, float *acc) {
        constexpr int I = K / 4, M = (K / 2) % 2, P = K % 2;
        for (int n = 0; n < N; ++n) {
            const U4 &ql0 = d[n]->p[4 * I + M], &ql32 = d[n]->p[4 * I + 2 + M], &qh = d[n]->p[8 + 2 * I + M];
            U4 qa, qb;
            if (P == 0) {
                qa = or4(and4(ql0, 0x0F0F0F0Fu), shl4(and4(qh, 0x03030303u), 4));
                qb = or4(and4(ql32, 0x0F0F0F0Fu), shl4(and4(shr4(qh, 2), 0x03030303u), 4));
            } else {
                qa = or4(and4(shr4(ql0, 4), 0x0F0F0F0Fu), shl4(and4(shr4(qh, 4), 0x03030303u), 4));
                qb = or4(and4(shr4(ql32, 4), 0x0F0F0F0Fu), shl4(and4(shr4(qh, 6), 0x03030303u), 4));
            }
            float ta = 0.0f, tb = 0.0f;
            stage_dot(x, st, qa, qb, ta, tb);
            acc[n] = fmaf(scale_of(*d[n], I, M, 2 * P), ta, acc[n]);
            acc[n] = fmaf(scale_of(*d[n], I, M, 2 * P + 1), tb, acc[n]);
        }
    }
    // stages 2G and 2G+1 (G = 0..3: I = G/2, M = G%2) read the piece group {4I+M, 4I+2+M, 8+2I+M}; the scales (piece
    // 12) and the tail are needed first
    template <int G, class L> SLAI_HD static void group(const L &ld) {
        constexpr int I = G / 2, M = G % 2;
        ld.template piece<4 * I + M>(); ld.template piece<4 * I + 2 + M>(); ld.template piece<8 + 2 * I + M>();
    }
    template <int G, class L> SLAI_HD static void lead_from(const L &ld) {
        if constexpr (2 * G < L::LEAD && G < 4) { group<G>(ld); lead_from<G + 1>(ld); }
    }
    template <class L> SLAI_HD static void lead(const L &ld) { ld.template piece<12>(); ld.tail(); lead_from<0>(ld); }
    template <int K, class L> SLAI_HD static void ahead(const L &ld) {
        // group G is first used at stage 2G: led when 2G < LEAD, otherwise requested at stage max(2G - DEPTH, 0)
        if constexpr ((K + L::DEPTH) % 2 == 0 && (K + L::DEPTH) / 2 < 4 && K + L::DEPTH >= L::LEAD) group<(K + L::DEPTH) / 2>(ld);
    }
    template <int K, int N, class X, class S, class L> SLAI_HD static void stages(const Data *const *d, const X &x, const S &st, float *acc, const L &ld) {
        ahead<K>(ld);
        SLAI_SCHED_FENCE();
        if constexpr (K < 7) {
            const auto nxt = x.template stage<c1(K + 1), c2(K + 1)>();
            compute<K, N>(d, x, st, acc);
            stages<K + 1, N>(d, x, nxt, acc, ld);
        } else {
            compute<K, N>(d, x, st, acc);
        }
    }
    template <int N, class X, class L = NoLoader> SLAI_HD static void dotn(const Data *const *d, const uint16_t *tail, const X &x, float *out, const L &ld = L()) {
        float acc[N];
        for (int n = 0; n < N; ++n) {
            // the -32 of every 6-bit value, through the activation sums: -32 * sum_j scale_j * sum16(chunk_j)
            float c = 0.0f;
            for (int I = 0; I < 2; ++I)
                for (int M = 0; M < 2; ++M)
                    for (int r = 0; r < 4; ++r) c = fmaf(scale_of(*d[n], I, M, r), x.sum16(8 * I + 2 * r + M), c);
            acc[n] = -32.0f * c;
        }
        const auto st0 = x.template stage<c1(0), c2(0)>();
        stages<0, N>(d, x, st0, acc, ld);
        for (int n = 0; n < N; ++n) out[n] = scale_f16(tail[n]) * acc[n];
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t tail, const X &x) {
        const Data *dp[1] = {&d};
        float out[1];
        dotn<1>(dp, &tail, x, out);
        return out[0];
    }
};

template <> struct Tiled<T_Q8_0> {
    static constexpr int PT = 17;
    static constexpr bool TAIL = false;
    struct Data { U4 p[17]; };
    // stage K = block K of the super-block: qs pieces 2K, 2K+1 <-> chunks 2K, 2K+1
    static constexpr int c1(int K) { return 2 * K; }
    static constexpr int c2(int K) { return 2 * K + 1; }
    SLAI_HD static float scale_of(const Data &d, int B) {
        const U4 &s = d.p[16];
        const uint32_t w = B < 2 ? s.x : (B < 4 ? s.y : (B < 6 ? s.z : s.w));
        return scale_f16((uint16_t)((B & 1) ? (w >> 16) : (w & 0xffffu)));
    }
    template <int K, int N, class X, class S> SLAI_HD static void compute(const Data *const *d, const X &x, const S &st, float *acc) {
        for (int n = 0; n < N; ++n) {
            // int8 -> unsigned via ^0x80; the 128 comes back through the activation sums
            float s = 0.0f, s2 = 0.0f;
            stage_dot(x, st, xor4(d[n]->p[2 * K], 0x80808080u), xor4(d[n]->p[2 * K + 1], 0x80808080u), s, s2);
            acc[n] = fmaf(scale_of(*d[n], K), s + s2, acc[n]);
        }
    }
    // stage K reads pieces 2K and 2K+1; the scales are piece 16
    template <int K, class L> SLAI_HD static void lead_from(const L &ld) {
        if constexpr (K < L::LEAD && K < 8) { ld.template piece<2 * K>(); ld.template piece<2 * K + 1>(); lead_from<K + 1>(ld); }
    }
    template <class L> SLAI_HD static void lead(const L &ld) { ld.template piece<16>(); lead_from<0>(ld); }
    template <int K, class L> SLAI_HD static void ahead(const L &ld) {
        if constexpr (K + L::DEPTH < 8 && K + L::DEPTH >= L::LEAD) { ld.template piece<2 * (K + L::DEPTH)>(); ld.template piece<2 * (K + L::DEPTH) + 1>(); }
    }
    template <int K, int N, class X, class S, class L> SLAI_HD static void stages(const Data *const *d, const X &x, const S &st, float *acc, const L &ld) {
        ahead<K>(ld);
        SLAI_SCHED_FENCE();
        if constexpr (K < 7) {
            const auto nxt = x.template stage<c1(K + 1), c2(K + 1)>();
            compute<K, N>(d, x, st, acc);
            stages<K + 1, N>(d, x, nxt, acc, ld);
        } else {
            compute<K, N>(d, x, st, acc);
        }
    }
    template <int N, class X, class L = NoLoader> SLAI_HD static void dotn(const Data *const *d, const uint16_t * /*tail*/, const X &x, float *out, const L &ld = L()) {
        float acc[N];
        for (int n = 0; n < N; ++n) {
            float c = 0.0f;
            for (int B = 0; B < 8; ++B) c = fmaf(scale_of(*d[n], B), x.sum16(2 * B) + x.sum16(2 * B + 1), c);
            acc[n] = -128.0f * c;
        }
        const auto st0 = x.template stage<c1(0), c2(0)>();
        stages<0, N>(d, x, st0, acc, ld);
        for (int n = 0; n < N; ++n) out[n] = acc[n];
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t tail, const X &x) {
        const Data *dp[1] = {&d};
        float out[1];
        dotn<1>(dp, &tail, x, out);
        return out[0];
    }
};

template <> struct Tiled<T_Q4_0> {
    static constexpr int PT = 9;
    static constexpr bool TAIL = false;
    struct Data { U4 p[9]; };
    // stage K = block K of the super-block: its 16 bytes are piece K; low nibbles <-> chunk 2K, high nibbles <-> chunk
    // 2K+1 (BlockQ4_0, quantization.rs:47-69); the -8 of every value comes back through the activation sums
    static constexpr int c1(int K) { return 2 * K; }
    static constexpr int c2(int K) { return 2 * K + 1; }
    SLAI_HD static float scale_of(const Data &d, int B) {
        const U4 &s = d.p[8];
        const uint32_t w = B < 2 ? s.x : (B < 4 ? s.y : (B < 6 ? s.z : s.w));
        return scale_f16((uint16_t)((B & 1) ? (w >> 16) : (w & 0xffffu)));
    }
    template <int K, class L> SLAI_HD static void lead_from(const L &ld) {
        if constexpr (K < L::LEAD && K < 8) { ld.template piece<K>(); lead_from<K + 1>(ld); }
    }
    template <class L> SLAI_HD static void lead(const L &ld) { ld.template piece<8>(); lead_from<0>(ld); }
    template <int K, class L> SLAI_HD static void ahead(const L &ld) {
        if constexpr (K + L::DEPTH < 8 && K + L::DEPTH >= L::LEAD) ld.template piece<K + L::DEPTH>();
    }
    template <int K, int N, class X, class S> SLAI_HD static void compute(const Data *const *d, const X &x, const S &st, float *acc) {
        for (int n = 0; n < N; ++n) {
            const U4 &q = d[n]->p[K];
            float s = 0.0f, s2 = 0.0f;
            stage_dot(x, st, and4(q, 0x0F0F0F0Fu), and4(shr4(q, 4), 0x0F0F0F0Fu), s, s2);
            acc[n] = fmaf(scale_of(*d[n], K), s + s2, acc[n]);
        }
    }
    template <int K, int N, class X, class S, class L> SLAI_HD static void stages(const Data *const *d, const X &x, const S &st, float *acc, const L &ld) {
        ahead<K>(ld);
        SLAI_SCHED_FENCE();
        if constexpr (K < 7) {
            const auto nxt = x.template stage<c1(K + 1), c2(K + 1)>();
            compute<K, N>(d, x, st, acc);
            stages<K + 1, N>(d, x, nxt, acc, ld);
        } else {
            compute<K, N>(d, x, st, acc);
        }
    }
    template <int N, class X, class L = NoLoader> SLAI_HD static void dotn(const Data *const *d, const uint16_t * /*tail*/, const X &x, float *out, const L &ld = L()) {
        float acc[N];
        for (int n = 0; n < N; ++n) {
            float c = 0.0f;
            for (int B = 0; B < 8; ++B) c = fmaf(scale_of(*d[n], B), x.sum16(2 * B) + x.sum16(2 * B + 1), c);
            acc[n] = -8.0f * c;
        }
        const auto st0 = x.template stage<c1(0), c2(0)>();
        stages<0, N>(d, x, st0, acc, ld);
        for (int n = 0; n < N; ++n) out[n] = acc[n];
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t tail, const X &x) {
        const Data *dp[1] = {&d};
        float out[1];
        dotn<1>(dp, &tail, x, out);
        return out[0];
    }
};

template <> struct Tiled<T_Q5_K> {
    static constexpr int PT = 11;
    static constexpr bool TAIL = false;
    struct Data { U4 p[11]; };
    // As Q4_K with a fifth bit (BlockQ5K, quantization.rs:249-317): stage K (J = K/2, H = K%2) reads qs piece 3 + K and
    // the high-bit piece 1 + H (bytes l = 16H..16H+15 of qh); bit 2J of qh[l] belongs to the low nibble (chunk 4J+H),
    // bit 2J+1 to the high nibble (chunk 4J+2+H)
    static constexpr int c1(int K) { return 4 * (K / 2) + (K % 2); }
    static constexpr int c2(int K) { return 4 * (K / 2) + 2 + (K % 2); }
    template <int N> struct Acc { float accd[N], slo[N], shi[N]; uint32_t sc_lo[N], sc_hi[N]; };
    template <int K, class L> SLAI_HD static void lead_from(const L &ld) {
        if constexpr (K < L::LEAD && K < 8) { ld.template piece<3 + K>(); lead_from<K + 1>(ld); }
    }
    template <class L> SLAI_HD static void lead(const L &ld) {
        ld.template piece<0>(); ld.template piece<1>(); ld.template piece<2>();
        lead_from<0>(ld);
    }
    template <int K, class L> SLAI_HD static void ahead(const L &ld) {
        if constexpr (K + L::DEPTH < 8 && K + L::DEPTH >= L::LEAD) ld.template piece<3 + K + L::DEPTH>();
    }
    template <int K, int N, class X, class S> SLAI_HD static void compute(const Data *const *d, const X &x, const S &st, Acc<N> &a) {
        constexpr int J = K / 2, H = K % 2;
        for (int n = 0; n < N; ++n) {
            const U4 &q = d[n]->p[3 + K], &qh = d[n]->p[1 + H];
            const U4 lo = or4(and4(q, 0x0F0F0F0Fu), shl4(and4(shr4(qh, 2 * J), 0x01010101u), 4));
            const U4 hi = or4(and4(shr4(q, 4), 0x0F0F0F0Fu), shl4(and4(shr4(qh, 2 * J + 1), 0x01010101u), 4));
            stage_dot(x, st, lo, hi, a.slo[n], a.shi[n]);
            if (H == 1) {
                const uint32_t scw = J < 2 ? a.sc_lo[n] : a.sc_hi[n];
                constexpr int sh = (J & 1) * 16;
                a.accd[n] = fmaf((float)((scw >> sh) & 0xffu), a.slo[n], a.accd[n]);
                a.accd[n] = fmaf((float)((scw >> (sh + 8)) & 0xffu), a.shi[n], a.accd[n]);
                a.slo[n] = 0.0f; a.shi[n] = 0.0f;
            }
        }
    }
    template <int K, int N, class X, class S, class L> SLAI_HD static void stages(const Data *const *d, const X &x, const S &st, Acc<N> &a, const L &ld) {
        ahead<K>(ld);
        SLAI_SCHED_FENCE();
        if constexpr (K < 7) {
            const auto nxt = x.template stage<c1(K + 1), c2(K + 1)>();
            compute<K, N>(d, x, st, a);
            stages<K + 1, N>(d, x, nxt, a, ld);
        } else {
            compute<K, N>(d, x, st, a);
        }
    }
    template <int N, class X, class L = NoLoader> SLAI_HD static void dotn(const Data *const *d, const uint16_t * /*tail*/, const X &x, float *out, const L &ld = L()) {
        Acc<N> a;
        float dd[N], dmin[N], accm[N];
        for (int n = 0; n < N; ++n) {
            const U4 &h = d[n]->p[0];
            dd[n] = scale_f16((uint16_t)(h.x & 0xffffu)); dmin[n] = scale_f16((uint16_t)(h.x >> 16));
            a.sc_lo[n] = h.y & 0x3f3f3f3fu;
            a.sc_hi[n] = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);
            const uint32_t m_lo = h.z & 0x3f3f3f3fu;
            const uint32_t m_hi = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
            float am = 0.0f;
            for (int sb = 0; sb < 8; ++sb) {
                const uint32_t mw = sb < 4 ? m_lo : m_hi;
                am = fmaf((float)((mw >> (8 * (sb & 3))) & 0xffu), x.sum16(2 * sb) + x.sum16(2 * sb + 1), am);
            }
            accm[n] = am; a.accd[n] = 0.0f; a.slo[n] = 0.0f; a.shi[n] = 0.0f;
        }
        const auto st0 = x.template stage<c1(0), c2(0)>();
        stages<0, N>(d, x, st0, a, ld);
        for (int n = 0; n < N; ++n) out[n] = dd[n] * a.accd[n] - dmin[n] * accm[n];
    }
    template <class X> SLAI_HD static float dot(const Data &d, uint16_t tail, const X &x) {
        const Data *dp[1] = {&d};
        float out[1];
        dotn<1>(dp, &tail, x, out);
        return out[0];
    }
};

}  // namespace slai
