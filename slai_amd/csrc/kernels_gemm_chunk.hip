// A chunk of up to 32 prompt tokens through one weight matrix on the matrix cores, gfx950.
//
// The reference has no such pass: its prompt loop runs the per-token GEMV (crates/slai/src/ops/gemv_quant.rs:206-312)
// once per prompt token (crates/slai-chat/src/chat_llama2.rs:105-158).  Here out[t][r] = sum_c deq(W[r][c]) * x[t][c]
// for all tokens t of the chunk in one pass over W, in fp32 throughout: the weights are dequantised exactly as the
// per-block `dequantize` of crates/slai/src/quantization.rs does (d * sc * q - dmin * m for Q4_K / Q5_K, d * sc * (q - 32)
// for Q6_K) and fed to fp32 MFMA instructions, so the result differs from the GEMV's only in the order of the sum.
//
// The tiled weight layouts (quant_tiled.h) give every lane ONE ROW of a tile and whole 256-column super-blocks, which is
// the A-operand layout of the one-column-deep MFMA shapes:
//   64-row tiles (lane = row):            v_mfma_f32_32x32x1 (2 blocks): block = rows 0-31 / 32-63, both with the same
//                                         column k; B = x[token = lane % 32][k]; 64 rows x 32 tokens per instruction.
//   16-row tiles (lane = 16 * kq + row):  v_mfma_f32_16x16x1 (4 blocks): block kq = super-block 4g + kq, so one
//                                         instruction advances FOUR columns (one per super-block) for 16 rows x 16
//                                         tokens; two instructions cover 32 tokens; the four blocks are added at the end.
// One lane register of weights thus feeds 64 x 32 multiply-adds; the activations (32 tokens x ncols floats, a few
// hundred KB) are read straight from L2, 16 bytes (four consecutive columns of the lane's token) per load.  A wave
// owns whole super-blocks; the waves of a workgroup meet in LDS once per tile.
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

template <int T> __device__ __forceinline__ void load_unit(const uint8_t *unit, int lane, typename Tiled<T>::Data &d, uint16_t &tail) {
    using F = Tiled<T>;
#pragma unroll
    for (int P = 0; P < F::PT; ++P) d.p[P] = ld128(unit + (size_t)P * 1024 + lane * 16);
    tail = F::TAIL ? ld16(unit + (size_t)F::PT * 1024 + lane * 2) : (uint16_t)0;
}

// ---- 64-row tiles ------------------------------------------------------------------------------------------------------
struct X64 { float4 a[4], b[4]; };                             // the lane's token: chunks c1 and c2 of a stage, four columns per entry

template <int T, int K> __device__ __forceinline__ void request_x64(const float *xcb, X64 &x) {
    using F = Tiled<T>;
#pragma unroll
    for (int W = 0; W < 4; ++W) {
        x.a[W] = *(const float4 *)(xcb + 16 * F::c1(K) + 4 * W);
        x.b[W] = *(const float4 *)(xcb + 16 * F::c2(K) + 4 * W);
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

// stage K of the current super-block: request the activations of the next stage (`xnext`: those of stage 0 of the wave's
// next super-block after the last stage), multiply, move on
template <int T, int K> __device__ __forceinline__ void stages64(const Deq<T> &q, const typename Tiled<T>::Data &d, const float *xcb, const float *xcb_next,
                                                                  X64 &x, f32x32 &acc) {
    X64 nx;
    if constexpr (K < 7) request_x64<T, K + 1>(xcb, nx);
    else request_x64<T, 0>(xcb_next, nx);
    mac64<T, K, 0>(q, d, x, acc); mac64<T, K, 1>(q, d, x, acc); mac64<T, K, 2>(q, d, x, acc); mac64<T, K, 3>(q, d, x, acc);
    x = nx;
    if constexpr (K < 7) stages64<T, K + 1>(q, d, xcb, xcb_next, x, acc);
}

constexpr int G64_WAVES = 4;
constexpr int G64_LDS_ROW = 68;                                // floats per token in the LDS partials (64 rows + padding)

template <int T>
__device__ __forceinline__ void gemm64_body(const GemmChunkParams &p, const GemmChunkSeg &seg, uint32_t tile, float *part) {
    using F = Tiled<T>;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    const uint32_t token = min((uint32_t)(lane & 31), p.ntokens - 1);            // lanes past the chunk repeat its last token
    const float *xrow = p.x + (size_t)token * p.x_stride;
    f32x32 acc;
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = 0.0f;
    typename F::Data d, dn;
    uint16_t dt = 0, dnt = 0;
    uint32_t cb = wave;
    X64 x;
    if (cb < p.ncb) {
        load_unit<T>(seg.W + ((size_t)tile * p.ncb + cb) * unit_bytes, lane, d, dt);
        request_x64<T, 0>(xrow + (size_t)cb * 256, x);
    }
    while (cb < p.ncb) {
        const uint32_t nb = cb + G64_WAVES;
        const bool more = nb < p.ncb;
        if (more) load_unit<T>(seg.W + ((size_t)tile * p.ncb + nb) * unit_bytes, lane, dn, dnt);
        Deq<T> q;
        q.head(d, dt);
        stages64<T, 0>(q, d, xrow + (size_t)cb * 256, xrow + (size_t)(more ? nb : cb) * 256, x, acc);
        if (more) { d = dn; dt = dnt; }
        cb = nb;
    }
    // ---- the waves meet: part[wave][token][row]; register v of block b holds row 32b + 8(v/4) + 4(lane/32) + v%4 of token lane%32
    float *mine = part + (size_t)wave * 32 * G64_LDS_ROW + (size_t)(lane & 31) * G64_LDS_ROW + 4 * (lane >> 5);
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *(float4 *)(mine + 32 * b + 8 * g) = make_float4(acc[16 * b + 4 * g], acc[16 * b + 4 * g + 1], acc[16 * b + 4 * g + 2], acc[16 * b + 4 * g + 3]);
    lds_barrier();
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t idx = (uint32_t)tid + 256u * e, r = idx & 63u, t = idx >> 6;
        const uint32_t row = tile * 64 + r;
        if (t < p.ntokens && row < seg.nrows) {
            float o = 0.0f;
#pragma unroll
            for (int w = 0; w < G64_WAVES; ++w) o += part[(size_t)w * 32 * G64_LDS_ROW + (size_t)t * G64_LDS_ROW + r];
            float *dst = seg.out + (size_t)t * seg.out_stride + row;
            if (seg.flags & GEMV_BIAS) o += seg.bias[row];
            if (seg.flags & GEMV_ACCUM) o = *dst + o;
            *dst = o;
        }
    }
}

// grid = tiles of all segments, block = 256 (four waves, each a quarter of the super-blocks)
template <int TT>
__global__ void __launch_bounds__(256) gemm64_kernel(const GemmChunkParams p) {
    __shared__ float part[G64_WAVES * 32 * G64_LDS_ROW];
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
    seg.bias = s == 0 ? p.seg[0].bias : (s == 1 ? p.seg[1].bias : p.seg[2].bias);
    seg.flags = s == 0 ? p.seg[0].flags : (s == 1 ? p.seg[1].flags : p.seg[2].flags);
    if constexpr (TT != 0) {
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
struct X16 { float4 a0, b0, a1, b1; };                         // tokens lane%16 (0) and 16 + lane%16 (1): four columns of chunk c1 (a) and c2 (b)

template <int T, int K, int W> __device__ __forceinline__ void request_x16(const float *x0, const float *x1, X16 &x) {
    using F = Tiled<T>;
    x.a0 = *(const float4 *)(x0 + 16 * F::c1(K) + 4 * W); x.b0 = *(const float4 *)(x0 + 16 * F::c2(K) + 4 * W);
    x.a1 = *(const float4 *)(x1 + 16 * F::c1(K) + 4 * W); x.b1 = *(const float4 *)(x1 + 16 * F::c2(K) + 4 * W);
}

template <int T, int K, int W> __device__ __forceinline__ void steps16(const Deq<T> &q, const typename Tiled<T>::Data &d, const float *x0, const float *x1,
                                                                       X16 &x, f32x16 &acc0, f32x16 &acc1) {
    constexpr int NK = W == 3 ? K + 1 : K, NW = W == 3 ? 0 : W + 1;
    X16 nx = x;
    if constexpr (NK < 8) request_x16<T, NK, NW>(x0, x1, nx);
    float lo[4], hi[4];
    q.template quad<K, W>(d, lo, hi);
    const float xa0[4] = {x.a0.x, x.a0.y, x.a0.z, x.a0.w}, xb0[4] = {x.b0.x, x.b0.y, x.b0.z, x.b0.w};
    const float xa1[4] = {x.a1.x, x.a1.y, x.a1.z, x.a1.w}, xb1[4] = {x.b1.x, x.b1.y, x.b1.z, x.b1.w};
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        acc0 = __builtin_amdgcn_mfma_f32_16x16x1f32(lo[b], xa0[b], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x1f32(lo[b], xa1[b], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_16x16x1f32(hi[b], xb0[b], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x1f32(hi[b], xb1[b], acc1, 0, 0, 0);
    }
    x = nx;
    if constexpr (NK < 8) steps16<T, NK, NW>(q, d, x0, x1, x, acc0, acc1);
}

constexpr int G16_LDS_ROW = 20;                                // floats per token in the LDS partials (16 rows + padding)

// grid = tiles, block = 64 * ngroups (one wave per column group of four super-blocks)
template <int T, int MAXT>
__global__ void __launch_bounds__(MAXT) gemm16_kernel(const GemmChunkParams p) {
    using F = Tiled<T>;
    extern __shared__ float part[];                            // [waves][32 tokens][G16_LDS_ROW]
    touch_kernel_arguments<sizeof(GemmChunkParams)>();
    const int tid = threadIdx.x, lane = tid & 63, NW = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t tile = blockIdx.x;
    const uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    const uint32_t cb = min((uint32_t)wave * 4 + (uint32_t)(lane >> 4), p.ncb - 1);   // (super-blocks past the end are zero weights)
    const uint32_t t0 = min((uint32_t)(lane & 15), p.ntokens - 1), t1 = min(16u + (uint32_t)(lane & 15), p.ntokens - 1);
    const float *x0 = p.x + (size_t)t0 * p.x_stride + (size_t)cb * 256, *x1 = p.x + (size_t)t1 * p.x_stride + (size_t)cb * 256;
    typename F::Data d;
    uint16_t dt = 0;
    load_unit<T>(p.seg[0].W + ((size_t)tile * p.ngroups + wave) * unit_bytes, lane, d, dt);
    X16 x;
    request_x16<T, 0, 0>(x0, x1, x);
    f32x16 acc0, acc1;
#pragma unroll
    for (int i = 0; i < 16; ++i) { acc0[i] = 0.0f; acc1[i] = 0.0f; }
    Deq<T> q;
    q.head(d, dt);
    steps16<T, 0, 0>(q, d, x0, x1, x, acc0, acc1);
    // the four blocks hold the same rows and tokens over different super-blocks: add them.  Register v of a block holds
    // row 4 * (lane / 16) + v of token lane % 16.
    float4 s0, s1;
    s0.x = (acc0[0] + acc0[4]) + (acc0[8] + acc0[12]); s0.y = (acc0[1] + acc0[5]) + (acc0[9] + acc0[13]);
    s0.z = (acc0[2] + acc0[6]) + (acc0[10] + acc0[14]); s0.w = (acc0[3] + acc0[7]) + (acc0[11] + acc0[15]);
    s1.x = (acc1[0] + acc1[4]) + (acc1[8] + acc1[12]); s1.y = (acc1[1] + acc1[5]) + (acc1[9] + acc1[13]);
    s1.z = (acc1[2] + acc1[6]) + (acc1[10] + acc1[14]); s1.w = (acc1[3] + acc1[7]) + (acc1[11] + acc1[15]);
    float *mine = part + (size_t)wave * 32 * G16_LDS_ROW + 4 * (lane >> 4);
    *(float4 *)(mine + (size_t)(lane & 15) * G16_LDS_ROW) = s0;
    *(float4 *)(mine + (size_t)(16 + (lane & 15)) * G16_LDS_ROW) = s1;
    lds_barrier();
    for (uint32_t idx = tid; idx < 512; idx += blockDim.x) {
        const uint32_t r = idx & 15u, t = idx >> 4;
        const uint32_t row = tile * 16 + r;
        if (t < p.ntokens && row < p.seg[0].nrows) {
            float o = 0.0f;
            for (int w = 0; w < NW; ++w) o += part[(size_t)w * 32 * G16_LDS_ROW + (size_t)t * G16_LDS_ROW + r];
            float *dst = p.seg[0].out + (size_t)t * p.seg[0].out_stride + row;
            if (p.seg[0].flags & GEMV_BIAS) o += p.seg[0].bias[row];
            if (p.seg[0].flags & GEMV_ACCUM) o = *dst + o;
            *dst = o;
        }
    }
}

// out[t][i] = (x[t][i] * 1/sqrt(mean(x[t]^2) + eps)) * w[i] (rms_norm.slang:48-67), one workgroup per token
__global__ void __launch_bounds__(256) rms_norm_rows_kernel(float *out, const float *x, const float *w, uint32_t n, uint32_t out_stride, uint32_t x_stride, float eps) {
    __shared__ float red[4];
    const float *xr = x + (size_t)blockIdx.x * x_stride;
    float *o = out + (size_t)blockIdx.x * out_stride;
    float ss = 0.0f;
    for (uint32_t i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float scale = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)n + eps);
    for (uint32_t i = threadIdx.x; i < n; i += 256) o[i] = (xr[i] * scale) * w[i];
}

}  // namespace

bool gemm_chunk_supports(const slai_qmat *m) {
    if (!m || !m->tiled || (m->type != T_Q4_K && m->type != T_Q6_K && m->type != T_Q5_K)) return false;
    if (m->rows_log2 == 6) return true;
    return m->rows_log2 == 4 && m->ngroups <= 16;
}

hipError_t launch_rms_norm_rows(hipStream_t s, float *out, const float *x, const float *w, uint32_t n, uint32_t rows, uint32_t out_stride, uint32_t x_stride, float eps) {
    if (rows == 0 || n == 0) return hipErrorInvalidValue;
    rms_norm_rows_kernel<<<rows, 256, 0, s>>>(out, x, w, n, out_stride, x_stride, eps);
    return hipGetLastError();
}

hipError_t launch_gemm_chunk(slai_ctx *ctx, GemmChunkParams p) {
    if (p.nseg < 1 || p.nseg > 3 || p.ntokens == 0 || p.ntokens > 32 || p.ncb == 0 || p.ncols != p.ncb * 256 || p.x_stride % 4 || ((uintptr_t)p.x & 15))
        return hipErrorInvalidValue;
    for (int i = 0; i < p.nseg; ++i)
        if (p.seg[i].type != T_Q4_K && p.seg[i].type != T_Q6_K && p.seg[i].type != T_Q5_K) return hipErrorInvalidValue;
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
        switch (tt) {
        case T_Q4_K: gemm64_kernel<T_Q4_K><<<tiles, 256, 0, st>>>(p); break;
        case T_Q6_K: gemm64_kernel<T_Q6_K><<<tiles, 256, 0, st>>>(p); break;
        case T_Q5_K: gemm64_kernel<T_Q5_K><<<tiles, 256, 0, st>>>(p); break;
        default: gemm64_kernel<0><<<tiles, 256, 0, st>>>(p); break;
        }
        return hipGetLastError();
    }
    if (p.rows_log2 != 4 || p.nseg != 1 || p.ngroups == 0 || p.ngroups > 16) return hipErrorInvalidValue;
    const uint32_t tiles = (p.seg[0].nrows + 15) / 16;
    const int NT = (int)p.ngroups * 64;
    const size_t smem = (size_t)p.ngroups * 32 * G16_LDS_ROW * sizeof(float);
    // the thread bound decides the register budget (256 threads leave 256 registers per lane, 1024 leave 128)
#define SLAI_G16(TY)                                                                         \
    do {                                                                                     \
        if (NT <= 256) gemm16_kernel<TY, 256><<<tiles, NT, smem, st>>>(p);                   \
        else if (NT <= 512) gemm16_kernel<TY, 512><<<tiles, NT, smem, st>>>(p);              \
        else if (NT <= 768) gemm16_kernel<TY, 768><<<tiles, NT, smem, st>>>(p);              \
        else gemm16_kernel<TY, 1024><<<tiles, NT, smem, st>>>(p);                            \
    } while (0)
    switch (p.seg[0].type) {
    case T_Q4_K: SLAI_G16(T_Q4_K); break;
    case T_Q6_K: SLAI_G16(T_Q6_K); break;
    default: SLAI_G16(T_Q5_K); break;
    }
#undef SLAI_G16
    return hipGetLastError();
}

}  // namespace slai
