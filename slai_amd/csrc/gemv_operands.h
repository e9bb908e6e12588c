// Device-side pieces shared by the GEMV kernels over the tiled weight layouts: how a lane gets its activations (as a
// wave-uniform scalar operand streamed through the scalar cache, or as a DPP broadcast out of registers), the loader that
// issues a unit's 16-byte weight pieces on request of the dot products in quant_tiled.h, and small reductions.
#pragma once
#include "common.h"
#include "quant_tiled.h"

namespace slai {
namespace lanes {

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory, which on this target means
// waiting for every outstanding global load (vmcnt(0)) -- it would serialise the weight stream behind each reduction step.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ float gelu_f(float x) {
    const float GELU_COEF_A = 0.044715f, SQRT_2_OVER_PI = 0.7978846f;   // ops/unary.rs:81-85
    return 0.5f * x * (1.0f + tanhf(SQRT_2_OVER_PI * x * (1.0f + GELU_COEF_A * x * x)));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// Sum over each 16-lane DPP row, result in every lane of the row: an inclusive scan with row_shr
// (lanes shifted in from outside the row read 0), then lane 15 is broadcast to the row.
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_mov<0x111>(v);   // row_shr:1
    v += dpp_mov<0x112>(v);   // row_shr:2
    v += dpp_mov<0x114>(v);   // row_shr:4
    v += dpp_mov<0x118>(v);   // row_shr:8
    return dpp_mov<0x15F>(v); // row_newbcast:15
}

typedef const float __attribute__((address_space(4))) cfloat;   // constant address space: scalar loads
typedef float fx16 __attribute__((ext_vector_type(16)));
typedef const fx16 __attribute__((address_space(4))) cfx16;

// Activations of one super-block, wave-uniform, fetched through the scalar cache one stage ahead of their use.
struct ScalarX {
    cfloat *x;   // 256 activations
    cfloat *s;   // 16 sums of 16 consecutive activations
    struct St { fx16 a, b; };
    template <int I1, int I2> __device__ __forceinline__ St stage() const {
        return St{*(cfx16 *)(x + 16 * I1), *(cfx16 *)(x + 16 * I2)};
    }
    // acc += sum_b byte_b(w) * x[16*I_SLOT + 4*W + b].  The conversions are spelled out because the compiler
    // otherwise extracts bytes 1..3 with a bit-field instruction first.
    template <int SLOT, int W> __device__ __forceinline__ float fma4(const St &st, uint32_t w, float acc) const {
        float t0, t1, t2, t3;
        asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(t0) : "v"(w));
        asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(t1) : "v"(w));
        asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(t2) : "v"(w));
        asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(t3) : "v"(w));
        const fx16 &c = SLOT ? st.b : st.a;
        acc = fmaf(t0, c[4 * W], acc);
        acc = fmaf(t1, c[4 * W + 1], acc);
        acc = fmaf(t2, c[4 * W + 2], acc);
        acc = fmaf(t3, c[4 * W + 3], acc);
        return acc;
    }
    __device__ __forceinline__ float sum16(int i) const { return s[i]; }
    // Eight 4-bit weights of one word at once, without converting them: a nibble n left in the low bits of a 16-bit half
    // is the half-precision subnormal n * 2^-24 (in bits 4..7: 16 n * 2^-24), and v_fma_mix_f32 multiplies such a half
    // by the f32 activation into an f32 sum.  Low nibbles (chunk I1) go to `lo`, high nibbles (chunk I2) to `hi`, in the
    // element order of fma4, so `lo` ends as 2^-24 and `hi` as 2^-20 times what fma4 gives -- exactly, powers of two
    // commute with every rounding here -- and the caller folds the factors into the block scale.
    static constexpr bool NIBBLE_MIX = true;
    template <int HALF> static __device__ __forceinline__ float mix(uint32_t halves, float xs, float acc) {
        float o;
        if constexpr (HALF == 0) asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(o) : "v"(halves), "s"(xs), "v"(acc));
        else asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(o) : "v"(halves), "s"(xs), "v"(acc));
        return o;
    }
    template <int W> __device__ __forceinline__ void nib8(const St &st, uint32_t w, float &lo, float &hi) const {
        const uint32_t b02l = w & 0x000F000Fu, b02h = w & 0x00F000F0u;      // bytes 0 and 2
        const uint32_t t = w >> 8;
        const uint32_t b13l = t & 0x000F000Fu, b13h = t & 0x00F000F0u;      // bytes 1 and 3
        lo = mix<0>(b02l, st.a[4 * W], lo);     hi = mix<0>(b02h, st.b[4 * W], hi);
        lo = mix<0>(b13l, st.a[4 * W + 1], lo); hi = mix<0>(b13h, st.b[4 * W + 1], hi);
        lo = mix<1>(b02l, st.a[4 * W + 2], lo); hi = mix<1>(b02h, st.b[4 * W + 2], hi);
        lo = mix<1>(b13l, st.a[4 * W + 3], lo); hi = mix<1>(b13h, st.b[4 * W + 3], hi);
    }
};

// Activations of a super-block held in 16 registers of a 16-lane DPP row.
struct DevX {
    float x[16];    // register i, lane j of the DPP row <-> x[cb*256 + 16*i + j]
    float s[16];    // s[i] = sum over the row of x[i]
    // acc += sum_b byte_b(w) * x[16*I + 4*W + b].  Lane k of every 16-lane row of register I is broadcast
    // to the row by the DPP operand (row_newbcast:k), so the activation costs no instruction of its own.
    // Written as assembly: the compiler forms DPP operands only on two-address encodings, which an FMA
    // does not have before register allocation, and it would otherwise hoist all 256 conversions of a
    // super-block ahead of the FMAs and run out of registers.
    static constexpr bool NIBBLE_MIX = false;
    template <int I1, int I2> struct St {};                   // activations are register resident: a stage is a tag
    template <int I1, int I2> __device__ __forceinline__ St<I1, I2> stage() const { return {}; }
    template <int SLOT, int W, int I1, int I2> __device__ __forceinline__ float fma4(St<I1, I2>, uint32_t w, float acc) const {
        constexpr int I = SLOT ? I2 : I1;
        float t0, t1, t2, t3;
        asm("v_cvt_f32_ubyte0 %1, %5\n\t"
            "v_cvt_f32_ubyte1 %2, %5\n\t"
            "v_cvt_f32_ubyte2 %3, %5\n\t"
            "v_cvt_f32_ubyte3 %4, %5\n\t"
            "v_fmac_f32_dpp %0, %6, %1 row_newbcast:%7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %6, %2 row_newbcast:%8 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %6, %3 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %6, %4 row_newbcast:%10 row_mask:0xf bank_mask:0xf"
            : "+v"(acc), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3)
            : "v"(w), "v"(x[I]), "n"(4 * W), "n"(4 * W + 1), "n"(4 * W + 2), "n"(4 * W + 3));
        return acc;
    }
    __device__ __forceinline__ float sum16(int i) const { return s[i]; }
};

// Issues the 16-byte pieces of one unit (of both matrices of a gated pair) on request of the dot product.
template <int T, int N, int LD> struct UnitLoader {
    static constexpr int DEPTH = LD;              // stages requested ahead of the one being multiplied
    static constexpr int LEAD = LD;               // stages requested before the dot product starts (>= DEPTH)
    using F = Tiled<T>;
    const uint8_t *unit[N];                       // + lane * 16 already applied
    const uint8_t *tailp[N];
    typename F::Data *d[N];
    uint16_t *t[N];
    template <int P> __device__ __forceinline__ void piece() const {
#pragma unroll
        for (int n = 0; n < N; ++n) d[n]->p[P] = ld128_stream(unit[n] + (size_t)P * 1024);
    }
    __device__ __forceinline__ void tail() const {
#pragma unroll
        for (int n = 0; n < N; ++n) *t[n] = ld16(tailp[n]);
    }
};

}  // namespace lanes
}  // namespace slai
