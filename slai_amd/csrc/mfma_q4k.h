// Q4_K rows times an f32 vector on the matrix cores, for the row-per-lane tiled layout (quant_tiled.h).
//
// A lane owns one row of one 256-column super-block: nine 16-byte pieces, the header and 128 bytes of 4-bit values.  The
// dot product of such a row with 256 activations costs the vector unit about 2.3 instructions per weight (extract, convert,
// multiply-add); a layer's weights arrive faster than that.  v_mfma_f32_16x16x32_f16 takes eight f16 per lane and operand
// and multiplies a 16 x 32 by a 32 x 16 matrix in the time of four vector instructions, and two facts make it usable here
// without moving a weight between lanes:
//
//   * a 4-bit value n masked in place -- (w & 0x000f000f), ((w >> 8) & 0x000f000f), and the high nibbles through
//     0x00f000f0 -- IS a pair of f16 numbers: the subnormals n * 2^-24 (16 n * 2^-24 for a high nibble).  The matrix cores
//     take subnormal inputs exactly, so the operand costs 5/8 of an instruction per weight and nothing is rounded;
//   * the instruction's A operand wants, from lane (g, r) = (lane / 16, lane % 16), eight values of row r and "k group" g.
//     The 64 lanes of a wave hold 64 different (row, super-block) pairs, not 16 rows with four k groups each -- but if the
//     B operand of k group g is non-zero in column g only, column g of the result is the dot product of the lanes of group
//     g alone: C[r][g] = (eight weights of lane (g, r)) . (their eight activations).  Columns g and 4 + g carry the high
//     and low halves of the activations, columns 8 + g and 12 + g the same for the steps that take the high nibbles, so
//     one accumulator holds the two sub-blocks (scales) of a 64-column quarter apart.
//
// Activations: x * 2^k = hi + lo with hi, lo in f16 (22 bits of x; 2^k, per super-block, brings the largest magnitude to
// [2^14, 2^15)), staged once per super-block in LDS in the order the masks above deliver the weights: 32 steps of
// (8 hi | 8 lo).  A lane reads its operand from the block of its super-block if its column is one of the two that are live
// in the step, and from a block of zeros otherwise; the choice is in the base address, the step in the immediate offset.
// The products n * hi and n * lo are exact in f32 and the matrix cores accumulate in f32, so the result differs from the
// f32 multiply-add chain of the vector path by accumulation order and by the 2^-22 of the split only.
//
// After the eight steps of a quarter the accumulator (rows 4 q .. 4 q + 3 of column c in lane (q, c)) goes through LDS to
// the lanes that own the rows, which apply the sub-block scales as before (quantization.rs:322-389).
#pragma once
#include "quant_tiled.h"

namespace slai {
namespace mq {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t w32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t w32x2 __attribute__((ext_vector_type(2)));

// ---- LDS layout, in bytes --------------------------------------------------------------------------------------------------
// One staged super-block: 32 steps x (8 hi | 8 lo) f16, then the sums of its activations (eight of 32 for Q4_K, sixteen of
// 16 for Q6_K; f32) and 2^-k.
constexpr uint32_t SB_STEPS = 32, SB_STEP_BYTES = 32, SB_B_BYTES = SB_STEPS * SB_STEP_BYTES;
constexpr uint32_t SB_SUMS = SB_B_BYTES, SB_INV = SB_B_BYTES + 64, SB_BYTES = SB_B_BYTES + 80;
// the accumulator of one matrix on its way to the lanes that own the rows: [16 columns][16 rows] f32
constexpr uint32_t CS_BYTES = 16 * 16 * 4;
SLAI_HD uint32_t step_of(uint32_t K, uint32_t h, uint32_t nib) { return K * 4 + h * 2 + nib; }   // Q4_K: piece 1 + K, words (x, y) | (z, w), low | high nibbles
// Q6_K: 128-half I, l-range M (l = 16 M ..), quadrant r, words (x, y) | (z, w): the sixteen weights of scale 8 I + 2 r + M in two steps
SLAI_HD uint32_t step_of_q6k(uint32_t I, uint32_t M, uint32_t r, uint32_t h) { return ((I * 2 + M) * 4 + r) * 2 + h; }

__device__ __forceinline__ uint32_t lane_now() {
    uint32_t l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}
// Lane exchanges as operand modifiers (no LDS round trip, no lane index): within quads, half rows (8 lanes) and rows (16).
template <int CTRL> __device__ __forceinline__ float dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E;               // quad_perm [1,0,3,2], [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141, DPP_MIRROR = 0x140;    // lane i <-> 7 - i of its half row, 15 - i of its row
// sum over the 8 lanes of a half row, in all of them
__device__ __forceinline__ float sum8(float v) {
    v += dpp<DPP_XOR1>(v); v += dpp<DPP_XOR2>(v); v += dpp<DPP_HALF_MIRROR>(v);
    return v;
}
// max(m, the word of the lane CTRL names), unsigned: zero, what a lane without a source reads, is neutral, so the exchange
// folds into the instruction (and an integer maximum needs no canonical operands, as a float one does)
template <int CTRL> __device__ __forceinline__ uint32_t dpp_umax(uint32_t m) {
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, CTRL, 0xf, 0xf, true);
    return m > o ? m : o;
}
// the largest of a non-negative value's bit patterns over the wave, as a wave-uniform word (such patterns order like the values)
__device__ __forceinline__ uint32_t max64_bits(float v) {
    uint32_t m = __builtin_bit_cast(uint32_t, v);
    m = dpp_umax<DPP_XOR1>(m); m = dpp_umax<DPP_XOR2>(m); m = dpp_umax<DPP_HALF_MIRROR>(m); m = dpp_umax<DPP_MIRROR>(m);
    const int b = (int)m;
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane(b, 0), r1 = (uint32_t)__builtin_amdgcn_readlane(b, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane(b, 32), r3 = (uint32_t)__builtin_amdgcn_readlane(b, 48);
    const uint32_t a = r0 > r1 ? r0 : r1, c = r2 > r3 ? r2 : r3;
    return a > c ? a : c;
}
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_f16(_Float16 a, _Float16 b) { return __builtin_bit_cast(uint32_t, half2v{a, b}); }

// Stages the 256 activations of one super-block: lane i of the wave holds elements 4 i .. 4 i + 3 in `x`.  `sb`: the
// super-block's block in LDS (SB_BYTES, 16-byte aligned).  Q4_K: element e = 64 J + 32 nib + 16 H + 8 h + i' belongs to
// step (K = 2 J + H, h, nib); Q6_K: e = 128 I + 32 r + 16 M + 8 h + i' to step (I, M, r, h).  In both it stands at position
// [0, 2, 1, 3, 4, 6, 5, 7]^-1 (i') of the step's eight: the order in which the masks deliver the weights of bytes
// 8 h .. 8 h + 7 of a piece.
template <int T>
__device__ __forceinline__ void stage_superblock(float4 x, char *sb) {
    static_assert(T == T_Q4_K || T == T_Q6_K, "formats with a matrix-core path");
    const uint32_t i = lane_now();
    const float mx = fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w)));
    uint32_t E = (max64_bits(mx) >> 23) & 0xffu;                                // biased exponent of the largest magnitude
    E = E < 30u ? 30u : E;
    const float up = __uint_as_float((268u - E) << 23), down = __uint_as_float((E - 14u) << 23);   // 2^k, 2^-k: k = 14 - (E - 127)
    const float a = x.x * up, b = x.y * up, c = x.z * up, d = x.w * up;
    const _Float16 ha = (_Float16)a, hb = (_Float16)b, hc = (_Float16)c, hd = (_Float16)d;
    const _Float16 la = (_Float16)(a - (float)ha), lb = (_Float16)(b - (float)hb), lc = (_Float16)(c - (float)hc), ld = (_Float16)(d - (float)hd);
    uint32_t step;
    if constexpr (T == T_Q4_K) {
        const float s = sum8((x.x + x.y) + (x.z + x.w));                       // the 32 activations of a sub-block: 8 lanes
        if ((i & 7u) == 0) reinterpret_cast<float *>(sb + SB_SUMS)[i >> 3] = s;
        step = step_of(2 * (i >> 4) + ((i >> 2) & 1u), (i >> 1) & 1u, (i >> 3) & 1u);
    } else {
        float s = (x.x + x.y) + (x.z + x.w);                                   // the 16 activations of a scale: 4 lanes
        s += dpp<DPP_XOR1>(s); s += dpp<DPP_XOR2>(s);
        if ((i & 3u) == 0) reinterpret_cast<float *>(sb + SB_SUMS)[i >> 2] = s;
        step = step_of_q6k(i >> 5, (i >> 2) & 1u, (i >> 3) & 3u, (i >> 1) & 1u);
    }
    char *blk = sb + step * SB_STEP_BYTES + (i & 1u) * 8u;
    *reinterpret_cast<w32x2 *>(blk) = w32x2{pack_f16(ha, hc), pack_f16(hb, hd)};
    *reinterpret_cast<w32x2 *>(blk + 16) = w32x2{pack_f16(la, lc), pack_f16(lb, ld)};
    if (i == 0) *reinterpret_cast<float *>(sb + SB_INV) = down;
}

// The dot products of this lane's row of N matrices (the same row and super-block of each: a gated pair shares the
// activations) with the staged super-block `sb`.  `zeros`: SB_BYTES of zeros (a lane without a super-block may name it as `sb`); `cs`: 2 N * CS_BYTES for this wave alone.
// Every lane of the wave takes part, whatever its row holds.
template <int N>
__device__ __forceinline__ void dot_q4k(const Tiled<T_Q4_K>::Data *const *d, const char *sb, const char *zeros, char *cs, float *out) {
    const uint32_t lane = lane_now(), g = lane >> 4, col = lane & 15u;
    // low-nibble steps live in columns g (hi half of x) and 4 + g (lo half); high-nibble steps in 8 + g and 12 + g
    const char *b_even = col == g ? sb : (col == 4u + g ? sb + 16 : zeros);
    const char *b_odd = col == 8u + g ? sb : (col == 12u + g ? sb + 16 : zeros);
    float acc[N], accm[N], dd[N], dmin[N];
    uint32_t sc_lo[N], sc_hi[N];
    const f32x4 s0 = *reinterpret_cast<const f32x4 *>(sb + SB_SUMS), s1 = *reinterpret_cast<const f32x4 *>(sb + SB_SUMS + 16);
    const float down = *reinterpret_cast<const float *>(sb + SB_INV);
    const float sums[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
    for (int n = 0; n < N; ++n) {
        const U4 &hd = d[n]->p[0];
        dd[n] = scale_f16((uint16_t)(hd.x & 0xffffu)); dmin[n] = scale_f16((uint16_t)(hd.x >> 16));
        // all eight 6-bit scales / mins at once (quantization.rs:381-389 applied bytewise)
        sc_lo[n] = hd.y & 0x3f3f3f3fu;
        sc_hi[n] = (hd.w & 0x0f0f0f0fu) | (((hd.y >> 6) & 0x03030303u) << 4);
        const uint32_t m_lo = hd.z & 0x3f3f3f3fu;
        const uint32_t m_hi = ((hd.w >> 4) & 0x0f0f0f0fu) | (((hd.z >> 6) & 0x03030303u) << 4);
        float am = 0.0f;
#pragma unroll
        for (int s = 0; s < 8; ++s) am = fmaf((float)(((s < 4 ? m_lo : m_hi) >> (8 * (s & 3))) & 0xffu), sums[s], am);
        accm[n] = am; acc[n] = 0.0f;
    }
    // Latencies are hidden by hand (four waves per SIMD do not hide them): the operands of step pair i + 1 are read from LDS
    // before the products of pair i are issued, and the accumulator of quarter J comes back from LDS -- transposed to the
    // lanes that own the rows -- while quarter J + 1 is multiplied (two blocks per matrix, used in turn).
    constexpr uint32_t LO = 0x000f000fu, HI = 0x00f000f0u;
    const auto read_b = [&](int it, half8 &be, half8 &bo) {     // step pair `it`: piece 1 + it / 2, words (x, y) | (z, w)
        be = __builtin_bit_cast(half8, *reinterpret_cast<const w32x4 *>(b_even + step_of(it >> 1, it & 1, 0) * SB_STEP_BYTES));
        bo = __builtin_bit_cast(half8, *reinterpret_cast<const w32x4 *>(b_odd + step_of(it >> 1, it & 1, 1) * SB_STEP_BYTES));
    };
    // lane (q, col) holds rows 4 q .. 4 q + 3 of column col; lane (g, r) wants row r of columns g, 4 + g, 8 + g, 12 + g
    const auto cs_of = [&](int n, int J) { return reinterpret_cast<float *>(cs + (n * 2 + (J & 1)) * CS_BYTES); };
    const auto take_back = [&](int J, float (&back)[N][4]) {
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const float *t = cs_of(n, J);
            back[n][0] = t[g * 16u + col]; back[n][1] = t[(4u + g) * 16u + col];
            back[n][2] = t[(8u + g) * 16u + col]; back[n][3] = t[(12u + g) * 16u + col];
        }
    };
    const auto add_back = [&](int J, const float (&back)[N][4]) {
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const uint32_t scw = J < 2 ? sc_lo[n] : sc_hi[n];
            const int sh = (J & 1) * 16;
            acc[n] = fmaf((float)((scw >> sh) & 0xffu), back[n][0] + back[n][1], acc[n]);
            acc[n] = fmaf((float)((scw >> (sh + 8)) & 0xffu) * 0.0625f, back[n][2] + back[n][3], acc[n]);   // (high nibbles were taken as 16 n)
        }
    };
    half8 be, bo;
    read_b(0, be, bo);
#pragma unroll
    for (int J = 0; J < 4; ++J) {
        f32x4 c[N];
        float back[N][4];
        __builtin_amdgcn_sched_barrier(0);
        if (J > 0) take_back(J - 1, back);                        // (asked for now, used after this quarter's products)
#pragma unroll
        for (int n = 0; n < N; ++n) c[n] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            const int it = 4 * J + i4, K = it >> 1, h = it & 1;
            half8 be_next = be, bo_next = bo;
            if (it + 1 < 16) read_b(it + 1, be_next, bo_next);
#pragma unroll
            for (int n = 0; n < N; ++n) {
                const U4 &q = d[n]->p[1 + K];
                const uint32_t w0 = h ? q.z : q.x, w1 = h ? q.w : q.y;
                const uint32_t v0 = w0 >> 8, v1 = w1 >> 8;
                const half8 ae = __builtin_bit_cast(half8, w32x4{w0 & LO, v0 & LO, w1 & LO, v1 & LO});
                const half8 ao = __builtin_bit_cast(half8, w32x4{w0 & HI, v0 & HI, w1 & HI, v1 & HI});
                c[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ae, be, c[n], 0, 0, 0);
                c[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ao, bo, c[n], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            be = be_next; bo = bo_next;
        }
#pragma unroll
        for (int n = 0; n < N; ++n) {
            asm volatile("" ::: "memory");
            *reinterpret_cast<f32x4 *>(cs_of(n, J) + col * 16u + 4u * g) = c[n];
            asm volatile("" ::: "memory");
        }
        if (J > 0) add_back(J - 1, back);
    }
    {
        float back[N][4];
        take_back(3, back);
        add_back(3, back);
    }
#pragma unroll
    for (int n = 0; n < N; ++n) out[n] = (dd[n] * 16777216.0f * down) * acc[n] - dmin[n] * accm[n];
}

// The same for a Q6_K row (quantization.rs:204-244): value = d * scale * (q - 32), q = low 4 bits | high 2 bits << 4.  The six
// bits of a weight are put together in place -- (ql & 0x000f000f) | ((qh << 4) & 0x00300030) and its relatives -- into the
// subnormal q * 2^-24 (16 q * 2^-24 for the weights whose low bits are a high nibble); the sixteen weights of a scale
// are two steps, two scales share an accumulator (columns g, 4 + g and 8 + g, 12 + g), and the -32 goes through the
// sums of the activations.  `tail`: d.
__device__ __forceinline__ float dot_q6k(const Tiled<T_Q6_K>::Data &d, uint16_t tail, const char *sb, const char *zeros, char *cs) {
    const uint32_t lane = lane_now(), g = lane >> 4, col = lane & 15u;
    const char *b_even = col == g ? sb : (col == 4u + g ? sb + 16 : zeros);
    const char *b_odd = col == 8u + g ? sb : (col == 12u + g ? sb + 16 : zeros);
    const float down = *reinterpret_cast<const float *>(sb + SB_INV);
    const U4 scp = d.p[12];
    const auto scale = [scp](int I, int M, int r) {              // scales[8 I + 2 r + M]
        const uint32_t w = r < 2 ? (I == 0 ? scp.x : scp.z) : (I == 0 ? scp.y : scp.w);
        return (float)(int8_t)((w >> (8 * (M + 2 * (r & 1)))) & 0xff);
    };
    float acc = 0.0f, c32 = 0.0f;
#pragma unroll
    for (int IM = 0; IM < 4; ++IM) {
        const int I = IM / 2, M = IM % 2;
        const U4 &ql0 = d.p[4 * I + M], &ql32 = d.p[4 * I + 2 + M], &qh = d.p[8 + 2 * I + M];
#pragma unroll
        for (int rp = 0; rp < 2; ++rp) {                         // quadrants 2 rp (low bits in ql0) and 2 rp + 1 (in ql32)
            const uint32_t mlo = rp ? 0x00f000f0u : 0x000f000fu, mhi = rp ? 0x03000300u : 0x00300030u;
            __builtin_amdgcn_sched_barrier(0);
            f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                __builtin_amdgcn_sched_barrier(0);
                // the high bits of quadrant r of bytes (0, 2) | (1, 3), moved next to the low bits: r even <- bits 0-1 | 4-5 of
                // the byte, r odd <- bits 2-3 | 6-7.  (One quadrant after the other: fewer values alive at a time.)
                const uint32_t h0 = h ? qh.z : qh.x, h1 = h ? qh.w : qh.y;
                {
                    const uint32_t a0 = h ? ql0.z : ql0.x, a1 = h ? ql0.w : ql0.y;
                    const half8 ae = __builtin_bit_cast(half8, w32x4{((h0 << 4) & mhi) | (a0 & mlo), ((h0 >> 4) & mhi) | ((a0 >> 8) & mlo),
                                                                      ((h1 << 4) & mhi) | (a1 & mlo), ((h1 >> 4) & mhi) | ((a1 >> 8) & mlo)});
                    const half8 be = __builtin_bit_cast(half8, *reinterpret_cast<const w32x4 *>(b_even + step_of_q6k(I, M, 2 * rp, h) * SB_STEP_BYTES));
                    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(ae, be, c, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                {
                    const uint32_t b0 = h ? ql32.z : ql32.x, b1 = h ? ql32.w : ql32.y;
                    const half8 ao = __builtin_bit_cast(half8, w32x4{((h0 << 2) & mhi) | (b0 & mlo), ((h0 >> 6) & mhi) | ((b0 >> 8) & mlo),
                                                                      ((h1 << 2) & mhi) | (b1 & mlo), ((h1 >> 6) & mhi) | ((b1 >> 8) & mlo)});
                    const half8 bo = __builtin_bit_cast(half8, *reinterpret_cast<const w32x4 *>(b_odd + step_of_q6k(I, M, 2 * rp + 1, h) * SB_STEP_BYTES));
                    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(ao, bo, c, 0, 0, 0);
                }
            }
            float *t = reinterpret_cast<float *>(cs);
            asm volatile("" ::: "memory");
            *reinterpret_cast<f32x4 *>(t + col * 16u + 4u * g) = c;
            asm volatile("" ::: "memory");
            const float even = t[g * 16u + col] + t[(4u + g) * 16u + col];
            const float odd = t[(8u + g) * 16u + col] + t[(12u + g) * 16u + col];
            asm volatile("" ::: "memory");
            const float f = rp ? 0.0625f : 1.0f;                 // (the weights of quadrants 2 and 3 were taken as 16 q)
            acc = fmaf(scale(I, M, 2 * rp) * f, even, acc);
            acc = fmaf(scale(I, M, 2 * rp + 1) * f, odd, acc);
        }
    }
    // (the -32 of every weight last, when the registers of the weights are free)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const f32x4 s4 = *reinterpret_cast<const f32x4 *>(sb + SB_SUMS + 16 * q);      // sums 4 q .. 4 q + 3: I = q / 2, r = 2 (q % 2) + {0, 0, 1, 1}, M = {0, 1, 0, 1}
        const int I = q / 2, r0 = 2 * (q % 2);
        c32 = fmaf(scale(I, 0, r0), s4.x, c32); c32 = fmaf(scale(I, 1, r0), s4.y, c32);
        c32 = fmaf(scale(I, 0, r0 + 1), s4.z, c32); c32 = fmaf(scale(I, 1, r0 + 1), s4.w, c32);
    }
    return scale_f16(tail) * (16777216.0f * down * acc - 32.0f * c32);
}

}  // namespace mq
}  // namespace slai
