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

}  // namespace slai
