// A chunk of up to 32 prompt tokens through one weight matrix on the matrix cores, gfx950.
//
// The reference has no such pass: its prompt loop runs the per-token GEMV (crates/slai/src/ops/gemv_quant.rs:206-312)
// once per prompt token (crates/slai-chat/src/chat_llama2.rs:105-158).  Here out[t][r] = sum_c deq(W[r][c]) * x[t][c]
// for all tokens t of the chunk in one pass over W, in fp32 throughout: the weights are dequantised exactly as the
// per-block `dequantize` of crates/slai/src/quantization.rs does (d * sc * q - dmin * m for Q4_K / Q5_K, d * sc * (q - 32)
// for Q6_K, d * q for Q8_0, d * (q - 8) for Q4_0) and fed to fp32 MFMA instructions, so the result differs from the GEMV's only in the order of the sum.
//
// The tiled weight layouts (quant_tiled.h) give every lane ONE ROW of a tile and whole 256-column super-blocks, which is
// the A-operand layout of the one-column-deep MFMA shapes:
//   64-row tiles (lane = row):            v_mfma_f32_32x32x1 (2 blocks): block = rows 0-31 / 32-63, both with the same
//                                         column k; B = x[token = lane % 32][k]; 64 rows x 32 tokens per instruction.
//   32-row tiles (lane = 32 * kq + row):  v_mfma_f32_32x32x1 (2 blocks): block kq = super-block 2g + kq, so one
//                                         instruction advances two columns for 32 rows x 32 tokens; the blocks are added
//                                         at the end.
//   16-row tiles (lane = 16 * kq + row):  v_mfma_f32_16x16x1 (4 blocks): block kq = super-block 4g + kq, so one
//                                         instruction advances FOUR columns (one per super-block) for 16 rows x 16
//                                         tokens; two instructions cover 32 tokens; the four blocks are added at the end.
// One lane register of weights thus feeds 64 x 32 multiply-adds; the activations (32 tokens x ncols floats, a few
// hundred KB) are read straight from L2, 16 bytes (four consecutive columns of the lane's token) per load.  They are
// stored "quad-major" for that: xq[(c / 4) * 32 + t] is the float4 of columns c .. c + 3 of token t, so the 32 tokens
// of one load instruction are 512 contiguous bytes (row-major activations would touch 32 cache lines per load and
// saturate L1 and L2 with quarter-used lines).  A wave owns whole super-blocks; the waves of a workgroup meet in LDS
// once per tile.
#include <algorithm>

#include "common.h"
#include "device_util.h"
#include "quant_tiled.h"

namespace slai {
namespace {

typedef float f32x32 __attribute__((ext_vector_type(32)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ float ub(uint32_t w, int b) { return (float)((w >> (8 * b)) & 0xffu); }
__device__ __forceinline__ uint32_t word(const U4 &q, int i) { return i == 0 ? q.x : (i == 1 ? q.y : (i == 2 ? q.z : q.w)); }

// The weights of stage K of a lane's super-block (see quant_tiled.h: a stage is two 16-element chunks c1(K), c2(K)),
// four at a time: quad<K, W>() gives elements 16 * c1 + 4W .. + 3 in lo[] and 16 * c2 + 4W .. + 3 in hi[].
template <int T> struct Deq;

template <> struct Deq<T_Q4_K> {
    using F = Tiled<T_Q4_K>;
    float d1[8], m1[8];                                        // d * sc and dmin * m of the eight sub-blocks
    __device__ __forceinline__ void head(const typename F::Data &d, uint16_t) {
        const U4 &h = d.p[0];
        const float dd = scale_f16((uint16_t)(h.x & 0xffffu)), dmin = scale_f16((uint16_t)(h.x >> 16));
        const uint32_t sc_lo = h.y & 0x3f3f3f3fu, sc_hi = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);     // quantization.rs:381-389
        const uint32_t m_lo = h.z & 0x3f3f3f3fu, m_hi = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            d1[sb] = dd * ub(sb < 4 ? sc_lo : sc_hi, sb & 3);
            m1[sb] = dmin * ub(sb < 4 ? m_lo : m_hi, sb & 3);
        }
    }
    __device__ __forceinline__ void scale(float s) {
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) { d1[sb] *= s; m1[sb] *= s; }
    }
    template <int K, int W> __device__ __forceinline__ void quad(const typename F::Data &d, float (&lo)[4], float (&hi)[4]) const {
        constexpr int J = K / 2;                                 // low nibbles: sub-block 2J, high nibbles: sub-block 2J + 1
        const uint32_t q = word(d.p[1 + K], W);
        const uint32_t ql = q & 0x0F0F0F0Fu, qh = (q >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int b = 0; b < 4; ++b) { lo[b] = d1[2 * J] * ub(ql, b) - m1[2 * J]; hi[b] = d1[2 * J + 1] * ub(qh, b) - m1[2 * J + 1]; }
    }
};

template <> struct Deq<T_Q5_K> {
    using F = Tiled<T_Q5_K>;
    float d1[8], m1[8];
    __device__ __forceinline__ void head(const typename F::Data &d, uint16_t) {
        const U4 &h = d.p[0];
        const float dd = scale_f16((uint16_t)(h.x & 0xffffu)), dmin = scale_f16((uint16_t)(h.x >> 16));
        const uint32_t sc_lo = h.y & 0x3f3f3f3fu, sc_hi = (h.w & 0x0f0f0f0fu) | (((h.y >> 6) & 0x03030303u) << 4);
        const uint32_t m_lo = h.z & 0x3f3f3f3fu, m_hi = ((h.w >> 4) & 0x0f0f0f0fu) | (((h.z >> 6) & 0x03030303u) << 4);
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            d1[sb] = dd * ub(sb < 4 ? sc_lo : sc_hi, sb & 3);
            m1[sb] = dmin * ub(sb < 4 ? m_lo : m_hi, sb & 3);
        }
    }
    __device__ __forceinline__ void scale(float s) {
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) { d1[sb] *= s; m1[sb] *= s; }
    }
    template <int K, int W> __device__ __forceinline__ void quad(const typename F::Data &d, float (&lo)[4], float (&hi)[4]) const {
        constexpr int J = K / 2, H = K % 2;
        const uint32_t q = word(d.p[3 + K], W), qb = word(d.p[1 + H], W);
        const uint32_t ql = (q & 0x0F0F0F0Fu) | (((qb >> (2 * J)) & 0x01010101u) << 4);
        const uint32_t qh = ((q >> 4) & 0x0F0F0F0Fu) | (((qb >> (2 * J + 1)) & 0x01010101u) << 4);
#pragma unroll
        for (int b = 0; b < 4; ++b) { lo[b] = d1[2 * J] * ub(ql, b) - m1[2 * J]; hi[b] = d1[2 * J + 1] * ub(qh, b) - m1[2 * J + 1]; }
    }
};

template <> struct Deq<T_Q6_K> {
    using F = Tiled<T_Q6_K>;
    float ds[16];                                              // d * scales[c] for the sixteen 16-element chunks
    __device__ __forceinline__ void head(const typename F::Data &d, uint16_t tail) {
        const float dd = scale_f16(tail);
#pragma unroll
        for (int I = 0; I < 2; ++I)
#pragma unroll
            for (int M = 0; M < 2; ++M)
#pragma unroll
                for (int r = 0; r < 4; ++r) ds[8 * I + 2 * r + M] = dd * F::scale_of(d, I, M, r);
    }
    __device__ __forceinline__ void scale(float s) {
#pragma unroll
        for (int c = 0; c < 16; ++c) ds[c] *= s;
    }
    template <int K, int W> __device__ __forceinline__ void quad(const typename F::Data &d, float (&lo)[4], float (&hi)[4]) const {
        constexpr int I = K / 4, M = (K / 2) % 2, P = K % 2;
        const uint32_t ql0 = word(d.p[4 * I + M], W), ql32 = word(d.p[4 * I + 2 + M], W), qh = word(d.p[8 + 2 * I + M], W);
        uint32_t qa, qb;
        if (P == 0) {
            qa = (ql0 & 0x0F0F0F0Fu) | ((qh & 0x03030303u) << 4);
            qb = (ql32 & 0x0F0F0F0Fu) | (((qh >> 2) & 0x03030303u) << 4);
        } else {
            qa = ((ql0 >> 4) & 0x0F0F0F0Fu) | (((qh >> 4) & 0x03030303u) << 4);
            qb = ((ql32 >> 4) & 0x0F0F0F0Fu) | (((qh >> 6) & 0x03030303u) << 4);
        }
        constexpr int C1 = F::c1(K), C2 = F::c2(K);
#pragma unroll
        for (int b = 0; b < 4; ++b) { lo[b] = ds[C1] * (ub(qa, b) - 32.0f); hi[b] = ds[C2] * (ub(qb, b) - 32.0f); }
    }
};

template <> struct Deq<T_Q8_0> {          // BlockQ8_0, quantization.rs:29-42: value = int8 * scale; stage K = block K
    using F = Tiled<T_Q8_0>;
    float sc[8], off[8];                                       // scale and -128 * scale of the eight 32-element blocks
    __device__ __forceinline__ void head(const typename F::Data &d, uint16_t) {
#pragma unroll
        for (int B = 0; B < 8; ++B) { sc[B] = F::scale_of(d, B); off[B] = -128.0f * sc[B]; }
    }
    __device__ __forceinline__ void scale(float s) {
#pragma unroll
        for (int B = 0; B < 8; ++B) { sc[B] *= s; off[B] *= s; }
    }
    template <int K, int W> __device__ __forceinline__ void quad(const typename F::Data &d, float (&lo)[4], float (&hi)[4]) const {
        // int8 -> unsigned through ^0x80 (one byte conversion instruction), the 128 taken off again with the scale
        const uint32_t qa = word(d.p[2 * K], W) ^ 0x80808080u, qb = word(d.p[2 * K + 1], W) ^ 0x80808080u;
#pragma unroll
        for (int b = 0; b < 4; ++b) { lo[b] = fmaf(sc[K], ub(qa, b), off[K]); hi[b] = fmaf(sc[K], ub(qb, b), off[K]); }
    }
};

template <> struct Deq<T_Q4_0> {          // BlockQ4_0, quantization.rs:47-69: value = (nibble - 8) * scale; stage K = block K
    using F = Tiled<T_Q4_0>;
    float sc[8], off[8];
    __device__ __forceinline__ void head(const typename F::Data &d, uint16_t) {
#pragma unroll
        for (int B = 0; B < 8; ++B) { sc[B] = F::scale_of(d, B); off[B] = -8.0f * sc[B]; }
    }
    __device__ __forceinline__ void scale(float s) {
#pragma unroll
        for (int B = 0; B < 8; ++B) { sc[B] *= s; off[B] *= s; }
    }
    template <int K, int W> __device__ __forceinline__ void quad(const typename F::Data &d, float (&lo)[4], float (&hi)[4]) const {
        const uint32_t q = word(d.p[K], W);
        const uint32_t ql = q & 0x0F0F0F0Fu, qh = (q >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int b = 0; b < 4; ++b) { lo[b] = fmaf(sc[K], ub(ql, b), off[K]); hi[b] = fmaf(sc[K], ub(qh, b), off[K]); }
    }
};

template <int T> __device__ __forceinline__ void load_unit(const uint8_t *unit, int lane, typename Tiled<T>::Data &d, uint16_t &tail) {
    using F = Tiled<T>;
#pragma unroll
    for (int P = 0; P < F::PT; ++P) d.p[P] = ld128_stream(unit + (size_t)P * 1024 + lane * 16);
    tail = F::TAIL ? ld16(unit + (size_t)F::PT * 1024 + lane * 2) : (uint16_t)0;
}

// The end of every kernel here: thread -> four consecutive rows (row .. row + 3) of token t whose partial sums lie
// `wave_stride` floats apart in LDS; adds them, then bias / old value, and stores (one float4 where alignment allows).
__device__ __forceinline__ void reduce_store4(const GemmChunkSeg &seg, float *out, const float *src, int nw, uint32_t wave_stride, uint32_t row, uint32_t t, bool quads,
                                              bool vec_ok) {
    float4 o = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll 4
    for (int w = 0; w < nw; ++w) {
        const float4 v = *(const float4 *)(src + (size_t)w * wave_stride);
        o.x += v.x; o.y += v.y; o.z += v.z; o.w += v.w;
    }
    float *dst = quads ? out + ((size_t)(row >> 2) * 32 + t) * 4 : out + (size_t)t * seg.out_stride + row;
    if (vec_ok && row + 3 < seg.nrows) {
        if (seg.flags & GEMV_BIAS) { const float4 b = *(const float4 *)(seg.bias + row); o.x += b.x; o.y += b.y; o.z += b.z; o.w += b.w; }
        if (seg.flags & GEMV_ACCUM) { const float4 a = *(const float4 *)dst; o.x += a.x; o.y += a.y; o.z += a.z; o.w += a.w; }
        *(float4 *)dst = o;
    } else {
        const float ov[4] = {o.x, o.y, o.z, o.w};
        for (uint32_t e = 0; e < 4 && row + e < seg.nrows; ++e) {
            float v = ov[e];
            if (seg.flags & GEMV_BIAS) v += seg.bias[row + e];
            if (seg.flags & GEMV_ACCUM) v = dst[e] + v;
            dst[e] = v;
        }
    }
}

// ---- 64-row tiles ------------------------------------------------------------------------------------------------------
struct X64 { float4 a[4], b[4]; };                             // the lane's token: chunks c1 and c2 of a stage, four columns per entry

// xcb: the lane's token in the first quad of the super-block; consecutive quads are 32 float4 apart
template <int T, int K> __device__ __forceinline__ void request_x64(const float4 *xcb, X64 &x) {
    using F = Tiled<T>;
#pragma unroll
    for (int W = 0; W < 4; ++W) {
        x.a[W] = xcb[(4 * F::c1(K) + W) * 32];
        x.b[W] = xcb[(4 * F::c2(K) + W) * 32];
    }
}

template <int T, int K, int W> __device__ __forceinline__ void mac64(const Deq<T> &q, const typename Tiled<T>::Data &d, const X64 &x, f32x32 &acc) {
    float lo[4], hi[4];
    q.template quad<K, W>(d, lo, hi);
    const float4 xa = x.a[W], xb = x.b[W];
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(lo[0], xa.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(hi[0], xb.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(lo[1], xa.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(hi[1], xb.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(lo[2], xa.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(hi[2], xb.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(lo[3], xa.w, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x1f32(hi[3], xb.w, acc, 0, 0, 0);
}

// stage K of the current super-block: request the activations of the next stage, multiply, move on
template <int T, int K> __device__ __forceinline__ void stages64(const Deq<T> &q, const typename Tiled<T>::Data &d, const float4 *xcb, X64 &x, f32x32 &acc) {
    X64 nx = x;
    if constexpr (K < 7) request_x64<T, K + 1>(xcb, nx);
    mac64<T, K, 0>(q, d, x, acc); mac64<T, K, 1>(q, d, x, acc); mac64<T, K, 2>(q, d, x, acc); mac64<T, K, 3>(q, d, x, acc);
    x = nx;
    if constexpr (K < 7) stages64<T, K + 1>(q, d, xcb, x, acc);
}

constexpr int G64_LDS_ROW = 68;                                // floats per token in the LDS partials (64 rows + padding)

// The activation loads run only a stage ahead of their use (more would not fit the registers), which is less than an
// L2 round trip: the matrix pipe is kept busy by several waves per SIMD instead, each with a super-block of its own.
template <int T>
__device__ __forceinline__ void gemm64_body(const GemmChunkParams &p, const GemmChunkSeg &seg, uint32_t tile, float *part) {
    using F = Tiled<T>;
    const int tid = threadIdx.x, lane = tid & 63, NW = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    const uint32_t token = min((uint32_t)(lane & 31), p.ntokens - 1);            // lanes past the chunk repeat its last token
    const float4 *xrow = (const float4 *)p.x + token;                             // + 64 * 32 per super-block
    f32x32 acc;
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = 0.0f;
    // the workgroup's range of super-blocks: all of them, or the blockIdx.y-th of ksplit ranges
    const uint32_t per = (p.ncb + p.ksplit - 1) / p.ksplit, cb0 = blockIdx.y * per, cb1 = min(p.ncb, cb0 + per);
    for (uint32_t cb = cb0 + wave; cb < cb1; cb += NW) {
        typename F::Data d;
        uint16_t dt = 0;
        X64 x;
        load_unit<T>(seg.W + ((size_t)tile * p.ncb + cb) * unit_bytes, lane, d, dt);
        request_x64<T, 0>(xrow + (size_t)cb * 2048, x);
        Deq<T> q;
        q.head(d, dt);
        stages64<T, 0>(q, d, xrow + (size_t)cb * 2048, x, acc);
    }
    // ---- the waves meet: part[wave][token][row]; register v of block b holds row 32b + 8(v/4) + 4(lane/32) + v%4 of token lane%32
    float *mine = part + (size_t)wave * 32 * G64_LDS_ROW + (size_t)(lane & 31) * G64_LDS_ROW + 4 * (lane >> 5);
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *(float4 *)(mine + 32 * b + 8 * g) = make_float4(acc[16 * b + 4 * g], acc[16 * b + 4 * g + 1], acc[16 * b + 4 * g + 2], acc[16 * b + 4 * g + 3]);
    lds_barrier();
    // four consecutive rows of a token per thread: float4 reads of the partials, one float4 store.  Consecutive threads
    // write consecutive addresses: the row quads of a token, or (quad-major output) the 32 tokens of a row quad.
    const bool quads = (seg.flags & GEMM_OUT_QUADS) != 0;
    float *out = seg.out + (size_t)blockIdx.y * seg.part_stride;
    const bool vec_ok = quads || (seg.out_stride % 4 == 0 && ((uintptr_t)out & 15) == 0);
    for (uint32_t idx = tid; idx < 512; idx += blockDim.x) {
        const uint32_t t = quads ? idx & 31u : idx >> 4, rq = quads ? idx >> 5 : idx & 15u;
        const uint32_t row = tile * 64 + 4 * rq;
        if (t >= p.ntokens || row >= seg.nrows) continue;
        reduce_store4(seg, out, part + (size_t)t * G64_LDS_ROW + 4 * rq, NW, 32 * G64_LDS_ROW, row, t, quads, vec_ok);
    }
}

// ---- 64-row tiles on the half-precision matrix cores ---------------------------------------------------------------------
// The f16 matrix rate is sixteen times the fp32 one.  Every dequantised weight w (scaled by 2^8, so that the remainder
// stays a normal f16 number) and every activation x is split into an f16 head and an f16 remainder, w = wh + wl,
// x = xh + xl, each pair keeping about 22 bits; wh*xh + wh*xl + wl*xh is accumulated in fp32 by three
// v_mfma_f32_32x32x16_f16 (the dropped wl*xl is below 2^-22 of the product).  Valid while |x| < 65504 and |w| < 255.
// The activations arrive split (split_quad in the kernels that write them, which also report values beyond the range).
// An instruction takes 32 rows x 16 columns: lanes 0-31 hold eight columns of chunk c1 for rows (A) / tokens (B) 0-31,
// lanes 32-63 eight columns of chunk c2.  The lane = row registers of the tile become the A operands of its two row
// halves through v_permlane32_swap: [c1 of rows 0-63], [c2 of rows 0-63] -> [c1 | c2 of rows 0-31], [c1 | c2 of rows 32-63].
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t H8 __attribute__((ext_vector_type(4)));       // eight f16

__device__ __forceinline__ void split8(const float (&a)[4], const float (&b)[4], H8 &h, H8 &l) {
    uint32_t h0, h1, h2, h3, l0, l1, l2, l3;
    split_pair_f16(a[0], a[1], h0, l0); split_pair_f16(a[2], a[3], h1, l1);
    split_pair_f16(b[0], b[1], h2, l2); split_pair_f16(b[2], b[3], h3, l3);
    h = H8{h0, h1, h2, h3}; l = H8{l0, l1, l2, l3};
}
// the activations arrive split (split_quad): heads and remainders of two quads as B operands
__device__ __forceinline__ void split_x(const H8 a, const H8 b, H8 &h, H8 &l) {
    h = __builtin_shufflevector(a, b, 0, 1, 4, 5);
    l = __builtin_shufflevector(a, b, 2, 3, 6, 7);
}
// a = [a of lanes 0-31 | b of lanes 0-31], b = [a of lanes 32-63 | b of lanes 32-63]
__device__ __forceinline__ void swap_halves(H8 &a, H8 &b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const auto r = __builtin_amdgcn_permlane32_swap(a[i], b[i], false, false);
        a[i] = r[0]; b[i] = r[1];
    }
}
__device__ __forceinline__ f32x16 mfma_h(const H8 &a, const H8 &b, f32x16 acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}

struct X64H { H8 a[4]; };                                  // the lane's token: its half's chunk of a stage, four columns per entry

// xl: the lane's token in the first quad of the super-block, moved on to chunk c2 for lanes 32-63
template <int T, int K> __device__ __forceinline__ void request_x64h(const H8 *xl, X64H &x) {
#pragma unroll
    for (int W = 0; W < 4; ++W) x.a[W] = xl[(4 * Tiled<T>::c1(K) + W) * 32];
}

template <int T, int K, int WP> __device__ __forceinline__ void mac64h(const Deq<T> &q, const typename Tiled<T>::Data &d, const X64H &x, f32x16 &top, f32x16 &bot) {
    float lo0[4], hi0[4], lo1[4], hi1[4];
    q.template quad<K, WP>(d, lo0, hi0);
    q.template quad<K, WP + 1>(d, lo1, hi1);
    H8 ah, al, bh, bl;                                         // a: chunk c1, b: chunk c2, columns 4WP .. 4WP + 7, all 64 rows
    split8(lo0, lo1, ah, al);
    split8(hi0, hi1, bh, bl);
    swap_halves(ah, bh);                                       // ah: rows 0-31, bh: rows 32-63
    swap_halves(al, bl);
    H8 xh, xl;
    split_x(x.a[WP], x.a[WP + 1], xh, xl);
    top = mfma_h(ah, xh, top); bot = mfma_h(bh, xh, bot);
    top = mfma_h(ah, xl, top); bot = mfma_h(bh, xl, bot);
    top = mfma_h(al, xh, top); bot = mfma_h(bl, xh, bot);
}

template <int T, int K> __device__ __forceinline__ void stages64h(const Deq<T> &q, const typename Tiled<T>::Data &d, const H8 *xl, X64H &x, f32x16 &top, f32x16 &bot) {
    X64H nx = x;
    if constexpr (K < 7) request_x64h<T, K + 1>(xl, nx);
    mac64h<T, K, 0>(q, d, x, top, bot);
    mac64h<T, K, 2>(q, d, x, top, bot);
    x = nx;
    if constexpr (K < 7) stages64h<T, K + 1>(q, d, xl, x, top, bot);
}

template <int T>
__device__ __forceinline__ void gemm64h_body(const GemmChunkParams &p, const GemmChunkSeg &seg, uint32_t tile, float *part) {
    using F = Tiled<T>;
    constexpr int D = F::c2(0) - F::c1(0);                     // chunk c2 of a stage is D chunks after c1
    static_assert(F::c2(3) - F::c1(3) == D && F::c2(7) - F::c1(7) == D, "c2 - c1 must not depend on the stage");
    const int tid = threadIdx.x, lane = tid & 63, NW = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    const uint32_t token = min((uint32_t)(lane & 31), p.ntokens - 1);            // lanes past the chunk repeat its last token
    const H8 *xrow = (const H8 *)p.x + token + (lane >> 5) * (4 * D * 32);
    f32x16 top, bot;
#pragma unroll
    for (int i = 0; i < 16; ++i) { top[i] = 0.0f; bot[i] = 0.0f; }
    const uint32_t per = (p.ncb + p.ksplit - 1) / p.ksplit, cb0 = blockIdx.y * per, cb1 = min(p.ncb, cb0 + per);
    for (uint32_t cb = cb0 + wave; cb < cb1; cb += NW) {
        typename F::Data d;
        uint16_t dt = 0;
        X64H x;
        load_unit<T>(seg.W + ((size_t)tile * p.ncb + cb) * unit_bytes, lane, d, dt);
        request_x64h<T, 0>(xrow + (size_t)cb * 2048, x);
        Deq<T> q;
        q.head(d, dt);
        q.scale(256.0f);
        stages64h<T, 0>(q, d, xrow + (size_t)cb * 2048, x, top, bot);
    }
    float *mine = part + (size_t)wave * 32 * G64_LDS_ROW + (size_t)(lane & 31) * G64_LDS_ROW + 4 * (lane >> 5);
    const float back = 1.0f / 256.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        *(float4 *)(mine + 8 * g) = make_float4(top[4 * g] * back, top[4 * g + 1] * back, top[4 * g + 2] * back, top[4 * g + 3] * back);
        *(float4 *)(mine + 32 + 8 * g) = make_float4(bot[4 * g] * back, bot[4 * g + 1] * back, bot[4 * g + 2] * back, bot[4 * g + 3] * back);
    }
    lds_barrier();
    const bool quads = (seg.flags & GEMM_OUT_QUADS) != 0;
    float *out = seg.out + (size_t)blockIdx.y * seg.part_stride;
    const bool vec_ok = quads || (seg.out_stride % 4 == 0 && ((uintptr_t)out & 15) == 0);
    for (uint32_t idx = tid; idx < 512; idx += blockDim.x) {
        const uint32_t t = quads ? idx & 31u : idx >> 4, rq = quads ? idx >> 5 : idx & 15u;
        const uint32_t row = tile * 64 + 4 * rq;
        if (t >= p.ntokens || row >= seg.nrows) continue;
        reduce_store4(seg, out, part + (size_t)t * G64_LDS_ROW + 4 * rq, NW, 32 * G64_LDS_ROW, row, t, quads, vec_ok);
    }
}

// grid = (tiles of all segments, ksplit), block = 64 * (waves: each takes every NW-th super-block)
template <int TT, int MAXT, bool H = false>
__global__ void __launch_bounds__(MAXT) gemm64_kernel(const GemmChunkParams p) {
    extern __shared__ float part[];                            // [waves][32 tokens][G64_LDS_ROW]
    touch_kernel_arguments<sizeof(GemmChunkParams)>();
    const uint32_t n0 = p.seg[0].ntiles, n1 = p.seg[1].ntiles;
    uint32_t tile = blockIdx.x;
    const int s = tile < n0 ? 0 : (tile - n0 < n1 ? 1 : 2);
    tile -= s == 0 ? 0u : (s == 1 ? n0 : n0 + n1);
    GemmChunkSeg seg;
    seg.W = s == 0 ? p.seg[0].W : (s == 1 ? p.seg[1].W : p.seg[2].W);
    seg.type = s == 0 ? p.seg[0].type : (s == 1 ? p.seg[1].type : p.seg[2].type);
    seg.nrows = s == 0 ? p.seg[0].nrows : (s == 1 ? p.seg[1].nrows : p.seg[2].nrows);
    seg.out = s == 0 ? p.seg[0].out : (s == 1 ? p.seg[1].out : p.seg[2].out);
    seg.out_stride = s == 0 ? p.seg[0].out_stride : (s == 1 ? p.seg[1].out_stride : p.seg[2].out_stride);
    seg.part_stride = s == 0 ? p.seg[0].part_stride : (s == 1 ? p.seg[1].part_stride : p.seg[2].part_stride);
    seg.bias = s == 0 ? p.seg[0].bias : (s == 1 ? p.seg[1].bias : p.seg[2].bias);
    seg.flags = s == 0 ? p.seg[0].flags : (s == 1 ? p.seg[1].flags : p.seg[2].flags);
    if constexpr (H) {
        if constexpr (TT != 0) {
            gemm64h_body<TT>(p, seg, tile, part);
        } else {
            switch (seg.type) {                                // uniform over the workgroup
            case T_Q4_K: gemm64h_body<T_Q4_K>(p, seg, tile, part); break;
            case T_Q6_K: gemm64h_body<T_Q6_K>(p, seg, tile, part); break;
            case T_Q5_K: gemm64h_body<T_Q5_K>(p, seg, tile, part); break;
            default: break;
            }
        }
    } else if constexpr (TT != 0) {
        gemm64_body<TT>(p, seg, tile, part);
    } else {
        switch (seg.type) {                                    // uniform over the workgroup
        case T_Q4_K: gemm64_body<T_Q4_K>(p, seg, tile, part); break;
        case T_Q6_K: gemm64_body<T_Q6_K>(p, seg, tile, part); break;
        case T_Q5_K: gemm64_body<T_Q5_K>(p, seg, tile, part); break;
        default: break;
        }
    }
}

// ---- 16-row tiles ------------------------------------------------------------------------------------------------------
// NACC = 2: the workgroup serves all 32 tokens (two accumulators: tokens lane % 16 and 16 + lane % 16); NACC = 1: 16 of
// them, the half given by blockIdx.y (narrow matrices: twice the workgroups, so that every SIMD has several waves).
template <int NACC> struct X16 { float4 a[NACC], b[NACC]; };    // four columns of chunk c1 (a) and c2 (b) per token

template <int T, int K, int W, int NACC> __device__ __forceinline__ void request_x16(const float4 *const (&xt)[NACC], X16<NACC> &x) {
    using F = Tiled<T>;
#pragma unroll
    for (int n = 0; n < NACC; ++n) { x.a[n] = xt[n][(4 * F::c1(K) + W) * 32]; x.b[n] = xt[n][(4 * F::c2(K) + W) * 32]; }
}

template <int T, int K, int W, int NACC> __device__ __forceinline__ void steps16(const Deq<T> &q, const typename Tiled<T>::Data &d, const float4 *const (&xt)[NACC],
                                                                                 X16<NACC> &x, f32x16 (&acc)[NACC]) {
    constexpr int NK = W == 3 ? K + 1 : K, NW = W == 3 ? 0 : W + 1;
    X16<NACC> nx = x;
    if constexpr (NK < 8) request_x16<T, NK, NW, NACC>(xt, nx);
    float lo[4], hi[4];
    q.template quad<K, W>(d, lo, hi);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
#pragma unroll
        for (int n = 0; n < NACC; ++n) {
            const float xa = b == 0 ? x.a[n].x : (b == 1 ? x.a[n].y : (b == 2 ? x.a[n].z : x.a[n].w));
            acc[n] = __builtin_amdgcn_mfma_f32_16x16x1f32(lo[b], xa, acc[n], 0, 0, 0);
        }
#pragma unroll
        for (int n = 0; n < NACC; ++n) {
            const float xb = b == 0 ? x.b[n].x : (b == 1 ? x.b[n].y : (b == 2 ? x.b[n].z : x.b[n].w));
            acc[n] = __builtin_amdgcn_mfma_f32_16x16x1f32(hi[b], xb, acc[n], 0, 0, 0);
        }
    }
    x = nx;
    if constexpr (NK < 8) steps16<T, NK, NW, NACC>(q, d, xt, x, acc);
}

// The same steps on the half-precision matrix cores (see the 64-row form): lane = 16 * kq + row is the A layout of
// v_mfma_f32_16x16x32_f16 as it stands, k group kq = the lane's super-block, eight columns (four of chunk c1, four of c2)
// per instruction, which adds up the four super-blocks itself.
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int NACC> struct X16H { H8 a[NACC], b[NACC]; };      // the split forms of four columns of chunk c1 (a) and c2 (b) per token
template <int T, int K, int W, int NACC> __device__ __forceinline__ void request_x16h(const H8 *const (&xt)[NACC], X16H<NACC> &x) {
    using F = Tiled<T>;
#pragma unroll
    for (int n = 0; n < NACC; ++n) { x.a[n] = xt[n][(4 * F::c1(K) + W) * 32]; x.b[n] = xt[n][(4 * F::c2(K) + W) * 32]; }
}
template <int T, int K, int W, int NACC> __device__ __forceinline__ void steps16h(const Deq<T> &q, const typename Tiled<T>::Data &d, const H8 *const (&xt)[NACC],
                                                                                  X16H<NACC> &x, f32x4 (&acc)[NACC]) {
    constexpr int NK = W == 3 ? K + 1 : K, NW = W == 3 ? 0 : W + 1;
    X16H<NACC> nx = x;
    if constexpr (NK < 8) request_x16h<T, NK, NW, NACC>(xt, nx);
    float lo[4], hi[4];
    q.template quad<K, W>(d, lo, hi);
    H8 ah, al;
    split8(lo, hi, ah, al);
#pragma unroll
    for (int n = 0; n < NACC; ++n) {
        H8 xh, xl;
        split_x(x.a[n], x.b[n], xh, xl);
        acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, ah), __builtin_bit_cast(f16x8, xh), acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, ah), __builtin_bit_cast(f16x8, xl), acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, al), __builtin_bit_cast(f16x8, xh), acc[n], 0, 0, 0);
    }
    x = nx;
    if constexpr (NK < 8) steps16h<T, NK, NW, NACC>(q, d, xt, x, acc);
}

constexpr int G16_LDS_ROW = 20;                                // floats per token in the LDS partials (16 rows + padding)

// grid = (tiles, 2 / NACC), block = 64 * ngroups (one wave per column group of four super-blocks)
template <int T, int MAXT, int NACC, bool H = false>
__global__ void __launch_bounds__(MAXT) gemm16_kernel(const GemmChunkParams p) {
    using F = Tiled<T>;
    extern __shared__ float part[];                            // [waves][16 * NACC tokens][G16_LDS_ROW]
    touch_kernel_arguments<sizeof(GemmChunkParams)>();
    const int tid = threadIdx.x, lane = tid & 63, NW = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t tile = blockIdx.x, tbase = NACC == 2 ? 0u : 16u * blockIdx.y;
    if (tbase >= p.ntokens) return;                            // (uniform) a short chunk has no second half
    const uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    const uint32_t g = p.group0 + wave;                        // this launch covers the column groups group0 .. group0 + NW - 1
    const uint32_t cb = min(g * 4 + (uint32_t)(lane >> 4), p.ncb - 1);   // (super-blocks past the end are zero weights)
    const float4 *xt[NACC];
#pragma unroll
    for (int n = 0; n < NACC; ++n) xt[n] = (const float4 *)p.x + (size_t)cb * 2048 + min(tbase + 16u * n + (uint32_t)(lane & 15), p.ntokens - 1);
    typename F::Data d;
    uint16_t dt = 0;
    load_unit<T>(p.seg[0].W + ((size_t)tile * p.ngroups + g) * unit_bytes, lane, d, dt);
    // Register v of a block (of the one block of the f16 form) holds row 4 * (lane / 16) + v of token lane % 16.
    float *mine = part + (size_t)wave * 16 * NACC * G16_LDS_ROW + 4 * (lane >> 4);
    if constexpr (H) {
        const H8 *xh[NACC];
#pragma unroll
        for (int n = 0; n < NACC; ++n) xh[n] = (const H8 *)xt[n];
        X16H<NACC> x;
        request_x16h<T, 0, 0, NACC>(xh, x);
        Deq<T> q;
        q.head(d, dt);
        f32x4 acc[NACC];
#pragma unroll
        for (int n = 0; n < NACC; ++n) acc[n] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        q.scale(256.0f);
        steps16h<T, 0, 0, NACC>(q, d, xh, x, acc);
        const float back = 1.0f / 256.0f;
#pragma unroll
        for (int n = 0; n < NACC; ++n)
            *(float4 *)(mine + (size_t)(16 * n + (lane & 15)) * G16_LDS_ROW) = make_float4(acc[n][0] * back, acc[n][1] * back, acc[n][2] * back, acc[n][3] * back);
    } else {
        X16<NACC> x;
        request_x16<T, 0, 0, NACC>(xt, x);
        Deq<T> q;
        q.head(d, dt);
        f32x16 acc[NACC];
#pragma unroll
        for (int n = 0; n < NACC; ++n)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[n][i] = 0.0f;
        steps16<T, 0, 0, NACC>(q, d, xt, x, acc);
        // the four blocks hold the same rows and tokens over different super-blocks: add them
#pragma unroll
        for (int n = 0; n < NACC; ++n) {
            float4 sm;
            sm.x = (acc[n][0] + acc[n][4]) + (acc[n][8] + acc[n][12]); sm.y = (acc[n][1] + acc[n][5]) + (acc[n][9] + acc[n][13]);
            sm.z = (acc[n][2] + acc[n][6]) + (acc[n][10] + acc[n][14]); sm.w = (acc[n][3] + acc[n][7]) + (acc[n][11] + acc[n][15]);
            *(float4 *)(mine + (size_t)(16 * n + (lane & 15)) * G16_LDS_ROW) = sm;
        }
    }
    lds_barrier();
    const GemmChunkSeg &seg = p.seg[0];
    const bool quads = (seg.flags & GEMM_OUT_QUADS) != 0;
    const bool vec_ok = quads || (seg.out_stride % 4 == 0 && ((uintptr_t)seg.out & 15) == 0);
    for (uint32_t idx = tid; idx < 64u * NACC; idx += blockDim.x) {     // four rows of a token per thread
        const uint32_t rq = idx & 3u, tl = idx >> 2, t = tbase + tl;
        const uint32_t row = tile * 16 + 4 * rq;
        if (t < p.ntokens && row < seg.nrows)
            reduce_store4(seg, seg.out, part + (size_t)tl * G16_LDS_ROW + 4 * rq, NW, 16 * NACC * G16_LDS_ROW, row, t, quads, vec_ok);
    }
}

// ---- 32-row tiles ------------------------------------------------------------------------------------------------------
constexpr int G32_LDS_ROW = 36;                                // floats per token in the LDS partials (32 rows + padding)

// grid = tiles, block = 64 * (column groups of this launch): one wave per group of two super-blocks, lane = 32 * kq + row
// f16 form: lane = 32 * kq + row is the A layout of v_mfma_f32_32x32x16_f16, k group kq = the lane's super-block
struct X32H { H8 a[4], b[4]; };
template <int T, int K> __device__ __forceinline__ void request_x32h(const H8 *xcb, X32H &x) {
    using F = Tiled<T>;
#pragma unroll
    for (int W = 0; W < 4; ++W) { x.a[W] = xcb[(4 * F::c1(K) + W) * 32]; x.b[W] = xcb[(4 * F::c2(K) + W) * 32]; }
}
template <int T, int K, int W> __device__ __forceinline__ void mac32h(const Deq<T> &q, const typename Tiled<T>::Data &d, const X32H &x, f32x16 &acc) {
    float lo[4], hi[4];
    q.template quad<K, W>(d, lo, hi);
    H8 ah, al, xh, xl;
    split8(lo, hi, ah, al);
    split_x(x.a[W], x.b[W], xh, xl);
    acc = mfma_h(ah, xh, acc); acc = mfma_h(ah, xl, acc); acc = mfma_h(al, xh, acc);
}
template <int T, int K> __device__ __forceinline__ void stages32h(const Deq<T> &q, const typename Tiled<T>::Data &d, const H8 *xcb, X32H &x, f32x16 &acc) {
    X32H nx = x;
    if constexpr (K < 7) request_x32h<T, K + 1>(xcb, nx);
    mac32h<T, K, 0>(q, d, x, acc); mac32h<T, K, 1>(q, d, x, acc); mac32h<T, K, 2>(q, d, x, acc); mac32h<T, K, 3>(q, d, x, acc);
    x = nx;
    if constexpr (K < 7) stages32h<T, K + 1>(q, d, xcb, x, acc);
}

template <int T, int MAXT, bool H = false>
__global__ void __launch_bounds__(MAXT) gemm32_kernel(const GemmChunkParams p) {
    using F = Tiled<T>;
    extern __shared__ float part[];                            // [waves][32 tokens][G32_LDS_ROW]
    touch_kernel_arguments<sizeof(GemmChunkParams)>();
    const int tid = threadIdx.x, lane = tid & 63, NW = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t tile = blockIdx.x;
    const uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    const uint32_t g = p.group0 + wave;
    const uint32_t cb = min(g * 2 + (uint32_t)(lane >> 5), p.ncb - 1);              // (a super-block past the end is zero weights)
    const float4 *xcb = (const float4 *)p.x + (size_t)cb * 2048 + min((uint32_t)(lane & 31), p.ntokens - 1);
    typename F::Data d;
    uint16_t dt = 0;
    load_unit<T>(p.seg[0].W + ((size_t)tile * p.ngroups + g) * unit_bytes, lane, d, dt);
    // Register v of a block (of the one block of the f16 form) holds row 8 * (v / 4) + 4 * (lane / 32) + v % 4 of token lane % 32.
    float *mine = part + (size_t)wave * 32 * G32_LDS_ROW + (size_t)(lane & 31) * G32_LDS_ROW + 4 * (lane >> 5);
    if constexpr (H) {
        X32H x;
        request_x32h<T, 0>((const H8 *)xcb, x);
        Deq<T> q;
        q.head(d, dt);
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
        q.scale(256.0f);
        stages32h<T, 0>(q, d, (const H8 *)xcb, x, acc);
        const float back = 1.0f / 256.0f;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
            *(float4 *)(mine + 8 * g4) = make_float4(acc[4 * g4] * back, acc[4 * g4 + 1] * back, acc[4 * g4 + 2] * back, acc[4 * g4 + 3] * back);
    } else {
        X64 x;
        request_x64<T, 0>(xcb, x);
        Deq<T> q;
        q.head(d, dt);
        f32x32 acc;
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] = 0.0f;
        stages64<T, 0>(q, d, xcb, x, acc);
        // the two blocks hold the same rows and tokens over different super-blocks: add them
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
            *(float4 *)(mine + 8 * g4) = make_float4(acc[4 * g4] + acc[16 + 4 * g4], acc[4 * g4 + 1] + acc[16 + 4 * g4 + 1],
                                                     acc[4 * g4 + 2] + acc[16 + 4 * g4 + 2], acc[4 * g4 + 3] + acc[16 + 4 * g4 + 3]);
    }
    lds_barrier();
    const GemmChunkSeg &seg = p.seg[0];
    const bool quads = (seg.flags & GEMM_OUT_QUADS) != 0;
    const bool vec_ok = quads || (seg.out_stride % 4 == 0 && ((uintptr_t)seg.out & 15) == 0);
    for (uint32_t idx = tid; idx < 256; idx += blockDim.x) {            // four rows of a token per thread
        const uint32_t rq = idx & 7u, t = idx >> 3;
        const uint32_t row = tile * 32 + 4 * rq;
        if (t < p.ntokens && row < seg.nrows)
            reduce_store4(seg, seg.out, part + (size_t)t * G32_LDS_ROW + 4 * rq, NW, 32 * G32_LDS_ROW, row, t, quads, vec_ok);
    }
}

// RMSNorm of token t = blockIdx.x (rms_norm.slang:48-67: (x * 1/sqrt(mean(x^2) + eps)) * w), written quad-major for the
// GEMM kernels above.  n % 4 == 0, n <= 16384 (16 float4 per thread).
__global__ void __launch_bounds__(256) rms_norm_quads_kernel(float4 *out, const float *x, const float *w, uint32_t n, uint32_t x_stride, float eps, int *split_flag) {
    __shared__ float red[4];
    const uint32_t t = blockIdx.x, nq = n / 4;
    const float4 *xr = (const float4 *)(x + (size_t)t * x_stride), *wr = (const float4 *)w;
    float4 v[16], g[16];
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const uint32_t i = threadIdx.x + 256u * j;
        if (i < nq) {
            v[j] = xr[i]; g[j] = wr[i];
            ss = fmaf(v[j].x, v[j].x, ss); ss = fmaf(v[j].y, v[j].y, ss); ss = fmaf(v[j].z, v[j].z, ss); ss = fmaf(v[j].w, v[j].w, ss);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float scale = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)n + eps);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const uint32_t i = threadIdx.x + 256u * j;
        if (i < nq) {
            const float4 r = make_float4((v[j].x * scale) * g[j].x, (v[j].y * scale) * g[j].y, (v[j].z * scale) * g[j].z, (v[j].w * scale) * g[j].w);
            if (split_flag) {                                  // (uniform) f16 heads and remainders; values beyond f16 are reported
                if (split_overflows(r)) *split_flag = 1;                // 1: a normalised row
                out[(size_t)i * 32 + t] = split_quad(r);
            } else {
                out[(size_t)i * 32 + t] = r;
            }
        }
    }
}

// LayerNorm of token t = blockIdx.x (ops/layernorm.rs:104-111: mean, centred values, variance = their squared norm / n,
// 1 / sqrt(variance + eps)), then * g + b, written quad-major.  n % 4 == 0, n <= 16384.
__global__ void __launch_bounds__(256) layernorm_quads_kernel(float4 *out, const float *x, const float *g, const float *b, uint32_t n, uint32_t x_stride, float eps,
                                                              int *split_flag) {
    __shared__ float red[4], red2[4];
    const uint32_t t = blockIdx.x, nq = n / 4;
    const float4 *xr = (const float4 *)(x + (size_t)t * x_stride), *gr = (const float4 *)g, *br = (const float4 *)b;
    float4 v[16];
    float sm = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const uint32_t i = threadIdx.x + 256u * j;
        v[j] = i < nq ? xr[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        sm += (v[j].x + v[j].y) + (v[j].z + v[j].w);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) sm += __shfl_xor(sm, m, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sm;
    __syncthreads();
    const float mean = ((red[0] + red[1]) + (red[2] + red[3])) / (float)n;
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const uint32_t i = threadIdx.x + 256u * j;
        if (i < nq) {
            v[j].x -= mean; v[j].y -= mean; v[j].z -= mean; v[j].w -= mean;
            ss = fmaf(v[j].x, v[j].x, ss); ss = fmaf(v[j].y, v[j].y, ss); ss = fmaf(v[j].z, v[j].z, ss); ss = fmaf(v[j].w, v[j].w, ss);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
    if ((threadIdx.x & 63) == 0) red2[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float scale = 1.0f / sqrtf(((red2[0] + red2[1]) + (red2[2] + red2[3])) / (float)n + eps);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const uint32_t i = threadIdx.x + 256u * j;
        if (i < nq) {
            const float4 gg = gr[i], bb = br[i];
            const float4 r = make_float4((v[j].x * scale) * gg.x + bb.x, (v[j].y * scale) * gg.y + bb.y, (v[j].z * scale) * gg.z + bb.z,
                                         (v[j].w * scale) * gg.w + bb.w);
            if (split_flag) {                                  // (uniform) f16 heads and remainders; values beyond f16 are reported
                if (split_overflows(r)) *split_flag = 1;
                out[(size_t)i * 32 + t] = split_quad(r);
            } else {
                out[(size_t)i * 32 + t] = r;
            }
        }
    }
}

// row-major [tokens][n] -> quad-major; thread = (quad, token), token fastest so that the stores are contiguous
__global__ void rows_to_quads_kernel(float4 *out, const float *x, uint32_t n, uint32_t x_stride, uint32_t ntokens, int *split_flag) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x, t = idx & 31u, qd = idx >> 5;
    if (qd < n / 4 && t < ntokens) {
        const float4 r = *(const float4 *)(x + (size_t)t * x_stride + 4 * qd);
        if (split_flag && split_overflows(r)) *split_flag = 1;
        out[(size_t)qd * 32 + t] = split_flag ? split_quad(r) : r;
    }
}

}  // namespace

bool gemm_chunk_supports(const slai_qmat *m) {
    if (!m || !m->tiled || !tiled_supported(m->type)) return false;
    return m->rows_log2 >= 4 && m->rows_log2 <= 6 && m->ngroups <= 64;
}

hipError_t launch_rms_norm_quads(hipStream_t s, float *out, const float *x, const float *w, uint32_t n, uint32_t ntokens, uint32_t x_stride, float eps, int *split_flag) {
    if (ntokens == 0 || ntokens > 32 || n == 0 || n % 4 || n > 16384 || x_stride % 4) return hipErrorInvalidValue;
    rms_norm_quads_kernel<<<ntokens, 256, 0, s>>>((float4 *)out, x, w, n, x_stride, eps, split_flag);
    return hipGetLastError();
}

hipError_t launch_layernorm_quads(hipStream_t s, float *out, const float *x, const float *g, const float *b, uint32_t n, uint32_t ntokens, uint32_t x_stride, float eps,
                                  int *split_flag) {
    if (ntokens == 0 || ntokens > 32 || n == 0 || n % 4 || n > 16384 || x_stride % 4) return hipErrorInvalidValue;
    layernorm_quads_kernel<<<ntokens, 256, 0, s>>>((float4 *)out, x, g, b, n, x_stride, eps, split_flag);
    return hipGetLastError();
}

hipError_t launch_rows_to_quads(hipStream_t s, float *out, const float *x, uint32_t n, uint32_t ntokens, uint32_t x_stride, int *split_flag) {
    if (ntokens == 0 || ntokens > 32 || n == 0 || n % 4 || x_stride % 4) return hipErrorInvalidValue;
    rows_to_quads_kernel<<<(n / 4 * 32 + 255) / 256, 256, 0, s>>>((float4 *)out, x, n, x_stride, ntokens, split_flag);
    return hipGetLastError();
}

hipError_t launch_gemm_chunk(slai_ctx *ctx, GemmChunkParams p) {
    if (p.nseg < 1 || p.nseg > 3 || p.ntokens == 0 || p.ntokens > 32 || p.ncb == 0 || p.ncols != p.ncb * 256 || ((uintptr_t)p.x & 15))
        return hipErrorInvalidValue;
    for (int i = 0; i < p.nseg; ++i) {
        const int t = p.seg[i].type;
        if (!tiled_supported(t)) return hipErrorInvalidValue;
        // segments of different formats in one launch: the K-quants only
        if (t != p.seg[0].type && (t == T_Q8_0 || t == T_Q4_0 || p.seg[0].type == T_Q8_0 || p.seg[0].type == T_Q4_0)) return hipErrorInvalidValue;
    }
    hipStream_t st = ctx->stream;
    if (p.rows_log2 == 6) {
        uint32_t tiles = 0;
        int tt = p.seg[0].type;
        for (int i = 0; i < p.nseg; ++i) {
            p.seg[i].ntiles = (p.seg[i].nrows + 63) / 64;
            tiles += p.seg[i].ntiles;
            if (p.seg[i].type != tt) tt = 0;
        }
        for (int i = p.nseg; i < 3; ++i) p.seg[i].ntiles = 0;
        // one wave per super-block of the workgroup's range, at most sixteen (every format fits the 128 registers per
        // lane that leaves)
        if (p.ksplit == 0 || p.ksplit > p.ncb) return hipErrorInvalidValue;
        if (p.ksplit > 1)
            for (int i = 0; i < p.nseg; ++i)
                if (p.seg[i].flags & (GEMV_BIAS | GEMV_ACCUM)) return hipErrorInvalidValue;
        const uint32_t per = (p.ncb + p.ksplit - 1) / p.ksplit;
        // (a Q8_0 super-block is 68 registers of weights per lane: eight waves, whose bound leaves 256 registers)
        const uint32_t nw = std::min(per, tt == T_Q8_0 ? 8u : 16u);
        const size_t smem = (size_t)nw * 32 * G64_LDS_ROW * sizeof(float);
        const int NT = (int)nw * 64;
        const dim3 grid(tiles, p.ksplit);
        if (p.split_f16) {
            // (up to eight waves: the bound that leaves 256 registers, which the mixed-format kernel needs not to spill)
#define SLAI_G64H(TY)                                                                      \
    do {                                                                                   \
        if (NT <= 512) gemm64_kernel<TY, 512, true><<<grid, NT, smem, st>>>(p);            \
        else gemm64_kernel<TY, 1024, true><<<grid, NT, smem, st>>>(p);                     \
    } while (0)
            switch (tt) {
            case T_Q4_K: SLAI_G64H(T_Q4_K); break;
            case T_Q5_K: SLAI_G64H(T_Q5_K); break;
            case T_Q6_K: SLAI_G64H(T_Q6_K); break;
            case T_Q4_0: SLAI_G64H(T_Q4_0); break;
            case T_Q8_0: gemm64_kernel<T_Q8_0, 512, true><<<grid, NT, smem, st>>>(p); break;
            default: SLAI_G64H(0); break;
            }
#undef SLAI_G64H
            return hipGetLastError();
        }
        switch (tt) {
        case T_Q4_K: gemm64_kernel<T_Q4_K, 1024><<<grid, NT, smem, st>>>(p); break;
        case T_Q5_K: gemm64_kernel<T_Q5_K, 1024><<<grid, NT, smem, st>>>(p); break;
        case T_Q6_K: gemm64_kernel<T_Q6_K, 1024><<<grid, NT, smem, st>>>(p); break;
        case T_Q4_0: gemm64_kernel<T_Q4_0, 1024><<<grid, NT, smem, st>>>(p); break;
        case T_Q8_0: gemm64_kernel<T_Q8_0, 512><<<grid, NT, smem, st>>>(p); break;
        default: gemm64_kernel<0, 1024><<<grid, NT, smem, st>>>(p); break;
        }
        return hipGetLastError();
    }
    if ((p.rows_log2 != 4 && p.rows_log2 != 5) || p.nseg != 1 || p.ngroups == 0 || p.ngroups > 64 || p.ksplit != 1) return hipErrorInvalidValue;
    // One wave per column group, at most 16 per workgroup: wider matrices take several launches over balanced slices
    // of the groups, the first one writing (or adding to the residual) and the others accumulating.
    const uint32_t nslices = (p.ngroups + 15) / 16, per_slice = (p.ngroups + nslices - 1) / nslices;
    const uint32_t rows = 1u << p.rows_log2;
    const uint32_t tiles = (p.seg[0].nrows + rows - 1) / rows;
    for (uint32_t sl = 0; sl < nslices; ++sl) {
        GemmChunkParams q = p;
        q.group0 = sl * per_slice;
        const uint32_t ng = std::min(per_slice, p.ngroups - q.group0);
        if (sl > 0) q.seg[0].flags = (q.seg[0].flags | GEMV_ACCUM) & ~GEMV_BIAS;
        const int NT = (int)ng * 64;
        if (p.rows_log2 == 5) {
            const size_t smem = (size_t)ng * 32 * G32_LDS_ROW * sizeof(float);
#define SLAI_G32H(TY, HH)                                                                  \
    do {                                                                                   \
        if (NT <= 256) gemm32_kernel<TY, 256, HH><<<tiles, NT, smem, st>>>(q);             \
        else if (NT <= 512) gemm32_kernel<TY, 512, HH><<<tiles, NT, smem, st>>>(q);        \
        else gemm32_kernel<TY, 1024, HH><<<tiles, NT, smem, st>>>(q);                      \
    } while (0)
#define SLAI_G32(TY)                                                                       \
    do {                                                                                   \
        if (p.split_f16) SLAI_G32H(TY, true); else SLAI_G32H(TY, false);                   \
    } while (0)
            switch (p.seg[0].type) {
            case T_Q4_K: SLAI_G32(T_Q4_K); break;
            case T_Q6_K: SLAI_G32(T_Q6_K); break;
            case T_Q8_0: SLAI_G32(T_Q8_0); break;
            case T_Q4_0: SLAI_G32(T_Q4_0); break;
            default: SLAI_G32(T_Q5_K); break;
            }
#undef SLAI_G32
#undef SLAI_G32H
        } else {
            // the thread bound decides the register budget (256 threads leave 256 registers per lane, 1024 leave 128);
            // narrow matrices (few waves per workgroup) split the tokens over two workgroups
            const size_t smem1 = (size_t)ng * 16 * G16_LDS_ROW * sizeof(float), smem2 = 2 * smem1;
#define SLAI_G16H(TY, HH)                                                                                  \
    do {                                                                                                   \
        if (NT <= 256) gemm16_kernel<TY, 256, 1, HH><<<dim3(tiles, 2), NT, smem1, st>>>(q);                \
        else if (NT <= 512) gemm16_kernel<TY, 512, 1, HH><<<dim3(tiles, 2), NT, smem1, st>>>(q);           \
        else if (NT <= 768) gemm16_kernel<TY, 768, 2, HH><<<tiles, NT, smem2, st>>>(q);                    \
        else gemm16_kernel<TY, 1024, 2, HH><<<tiles, NT, smem2, st>>>(q);                                  \
    } while (0)
#define SLAI_G16(TY)                                                                                       \
    do {                                                                                                   \
        if (p.split_f16) SLAI_G16H(TY, true); else SLAI_G16H(TY, false);                                   \
    } while (0)
            switch (p.seg[0].type) {
            case T_Q4_K: SLAI_G16(T_Q4_K); break;
            case T_Q6_K: SLAI_G16(T_Q6_K); break;
            case T_Q8_0: SLAI_G16(T_Q8_0); break;
            case T_Q4_0: SLAI_G16(T_Q4_0); break;
            default: SLAI_G16(T_Q5_K); break;
            }
#undef SLAI_G16
#undef SLAI_G16H
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace slai
