// Small device-side helpers shared by the kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace slai {

// Kernel arguments live in memory that no cache holds when a dispatch starts.  The compiler fetches the fields it
// needs as it goes, and every first touch of a 64-byte line is a round trip to memory; fields that are only known
// after a branch or a dependent index make those round trips serial.  Reading one word of every line of the
// argument block first makes all of them a single, overlapped round trip; later reads hit the scalar cache.
template <int BYTES> __device__ __forceinline__ void touch_kernel_arguments() {
    typedef const uint32_t __attribute__((address_space(4))) cu32;
    cu32 *ka = (cu32 *)__builtin_amdgcn_kernarg_segment_ptr();
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < BYTES; i += 64) w |= ka[i / 4];
    asm volatile("" : : "s"(w));
}

// A lane-broadcast word as an unsigned value (the builtin returns `int`; see join_words in resident_plan.h).
__device__ __forceinline__ uint32_t uniform_word(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// ---- data exchanged between workgroups of one running kernel ---------------------------------------------------------
// The eight dies of the device have an L2 each, and a die's L2 is not kept coherent with what other dies write while a
// kernel runs.  Accesses at agent scope (the sc1 cache-policy bit) are: a store is written through to memory, a load does
// not take a line that another die may since have changed.  Producer and consumer workgroups of one launch therefore
// exchange data with these accesses only, and the data itself says when it has arrived: the buffers are filled with
// FLOW_EMPTY (a NaN no computation produces) before the launch, and a reader repeats its load until no element is empty.
constexpr uint32_t FLOW_EMPTY = 0xFFFFFFFFu;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float flow_load(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void flow_store(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// 16 bytes at once (the compiler has no 16-byte atomic): the load is issued and waited for
__device__ __forceinline__ u32x4 flow_load16(const void *p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void flow_store16(void *p, u32x4 v) { asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory"); }
__device__ __forceinline__ bool flow_empty(u32x4 v) { return v.x == FLOW_EMPTY || v.y == FLOW_EMPTY || v.z == FLOW_EMPTY || v.w == FLOW_EMPTY; }

// A value as an f16 head plus an f16 remainder (both rounded toward zero; value - head is exact in f32), about
// 22 bits together: the form in which the prompt-chunk GEMM reads activations for the half-precision matrix cores.
// split_quad packs four values as {heads 0-1, heads 2-3, remainders 0-1, remainders 2-3} into the 16 bytes of the float4.
__device__ __forceinline__ void split_pair_f16(float a, float b, uint32_t &h, uint32_t &l) {
    h = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
    // value - head, the head converted inside the instruction (the compiler would emit a conversion and a subtraction)
    float ra, rb;
    asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(ra) : "v"(h), "v"(a));
    asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(rb) : "v"(h), "v"(b));
    l = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(ra, rb));
}
__device__ __forceinline__ float4 split_quad(float4 v) {
    uint32_t h0, h1, l0, l1;
    split_pair_f16(v.x, v.y, h0, l0);
    split_pair_f16(v.z, v.w, h1, l1);
    return make_float4(__uint_as_float(h0), __uint_as_float(h1), __uint_as_float(l0), __uint_as_float(l1));
}
// true when a value does not fit the f16 head (NaN included)
__device__ __forceinline__ bool split_overflows(float4 v) {
    return !(fabsf(v.x) < 65504.0f && fabsf(v.y) < 65504.0f && fabsf(v.z) < 65504.0f && fabsf(v.w) < 65504.0f);
}

}  // namespace slai
