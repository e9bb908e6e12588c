// One launch per token for the Llama-2 layer stack: every layer's RMSNorm + q/k/v, RoPE + cache write + attention,
// output projection, RMSNorm + gate/up + SiLU and down projection, then the final RMSNorm and the output matrix
// (`Llama2::launch`, crates/slai/src/models/llama2/transformer.rs:316-381), in a grid that stays resident.
//
// Why: at batch 1 a layer is four points at which every workgroup needs a vector that all the others produced, and a
// kernel boundary at each of them costs about as much as streaming the weights between them.  Here the workgroups stay
// where they are and hand the vectors over themselves:
//   * a producer writes its slice of the vector with agent-scope stores into a buffer that was filled with FLOW_EMPTY
//     before the launch (one buffer per layer and vector, so nothing is ever reused inside a launch);
//   * a consumer repeats its agent-scope load of a piece until no element of it is empty -- the data is its own flag, so
//     a hand-off is one store and one load deep, with no counter or barrier round trip in between;
//   * the waves that multiply request ALL the weights of their next unit first and only then wait: the weights travel
//     while the activations are still being produced.  Loads retire in issue order, so the waiting is done by other waves
//     of the workgroup ("stagers", which hold no outstanding weight requests) and handed over through LDS or through a
//     per-workgroup slot that the multiplying waves read with scalar loads.
// The arithmetic is that of the separate kernels (kernels_gemv_rowtile.hip, kernels_gemv_tiled.hip, attention_fast.h):
// 64-row tiles with wave-uniform activations for q/k/v, gate/up and the output matrix, 16-row tiles with DPP-broadcast
// activations for the two projections that add into the residual, one workgroup per head for the attention.
//
// Every wait is bounded.  A reader that gives up sets a flag the host turns into an error, and from then on no reader of
// the launch waits again, so a launch always ends.  The grid is exactly as large as the device can keep resident.
#include "common.h"
#include "attention_fast.h"
#include <cstddef>
#include "device_util.h"
#include "gemv_operands.h"
#include "quant_tiled.h"

namespace slai {
namespace {

using namespace lanes;

constexpr int PNT = 1024, PNW = 16;                 // threads and waves of a workgroup

// The thread index as a value the compiler cannot follow: what a phase derives from it (lane offsets, addresses) is then
// computed inside the phase instead of being kept alive across the whole layer loop, where it would not fit the registers.
__device__ __forceinline__ int phase_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

// Optional time stamps (the constant 100 MHz clock) for a per-phase time line of every workgroup: profilers see one long
// kernel.  `row` is null unless the host asked for a trace.
__device__ __forceinline__ void stamp(uint64_t *row, uint32_t k) {
    if (row && threadIdx.x == 0) row[k] = wall_clock64();
}

// ---- waiting for data -------------------------------------------------------------------------------------------------
constexpr uint64_t FLOW_WAIT_TICKS = 2u * 1000u * 1000u;      // 20 ms of the 100 MHz clock: what a reader waits before it gives up (a token takes about 1)

struct Flow {
    uint32_t *abort_flag;     // device word: non-zero once any reader of the launch has given up
    bool dead;                // wave-uniform: this wave no longer waits
};

// One round of a failed wait: sleep a little, look at the clock and at the flag.  `deadline` is 0 until the first failure.
__device__ __forceinline__ void flow_backoff(Flow &f, uint64_t &deadline) {
    __builtin_amdgcn_s_sleep(8);
    const uint64_t now = wall_clock64();
    if (deadline == 0) deadline = now + FLOW_WAIT_TICKS;
    if (now > deadline) {
        f.dead = true;
        if ((phase_tid() & 63) == 0) __hip_atomic_store(f.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if (__hip_atomic_load(f.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
        f.dead = true;
    }
}

// Waits until the 16 bytes at `probe` (one address for the whole wave: one request per round) are no longer empty.  A
// wave that arrives long before its input is produced polls this one piece only; the pieces it actually needs are
// fetched afterwards, when most of them are there.
__device__ __forceinline__ void flow_probe(const float *probe, Flow &f) {
    uint64_t deadline = 0;
    while (!f.dead) {
        const u32x4 v = flow_load16(probe);
        if (!__any(flow_empty(v))) break;
        flow_backoff(f, deadline);
    }
}

// N (4 or 12) pieces of 16 bytes per lane, each once none of its words is empty: piece k of a lane sits `off0 + k * stride`
// bytes into the vector at `base` and is requested when k < nlive.  One round trip for all of them, repeated by the whole
// wave while any is incomplete (after a time-out the values are whatever was there; pieces not requested stay zero).
// Everything between the first request and the arrival of the last result is ONE assembly block: the compiler does not
// know that a register named by an earlier block is still being filled, and has been seen to copy such registers before
// a wait placed in a later block.  Inside the block the loads run under an execution mask (no lane asks for a piece it
// does not need) and the offset register is stepped by the stride.
#define SLAI_FLOW_PIECE(K)                                                                                   \
    "v_cmp_lt_u32 vcc, " #K ", %[nl]\n\ts_and_b64 exec, %[sv], vcc\n\t"                                      \
    "global_load_dwordx4 %[v" #K "], %[t], %[base] sc1\n\ts_mov_b64 exec, %[sv]\n\tv_add_u32 %[t], %[st], %[t]\n\t"
template <int N>
__device__ __forceinline__ void flow_acquire(const float *base, uint32_t off0, uint32_t stride, uint32_t nlive, u32x4 (&v)[N], Flow &f) {
    static_assert(N == 4 || N == 12, "four or twelve pieces");
    const uint64_t base_bits = join_words(uniform_word((uint32_t)(uintptr_t)base), uniform_word((uint32_t)((uintptr_t)base >> 32)));
    const uint32_t st = uniform_word(stride);
#pragma unroll
    for (int k = 0; k < N; ++k) v[k] = u32x4{0, 0, 0, 0};
    uint64_t deadline = 0;
    for (;;) {
        uint64_t saved;
        uint32_t t;
        if constexpr (N == 4) {
            asm volatile("s_mov_b64 %[sv], exec\n\tv_mov_b32 %[t], %[off0]\n\t"
                         SLAI_FLOW_PIECE(0) SLAI_FLOW_PIECE(1) SLAI_FLOW_PIECE(2) SLAI_FLOW_PIECE(3)
                         "s_waitcnt vmcnt(0)"
                         : [v0] "+v"(v[0]), [v1] "+v"(v[1]), [v2] "+v"(v[2]), [v3] "+v"(v[3]), [sv] "=&s"(saved), [t] "=&v"(t)
                         : [base] "s"(base_bits), [off0] "v"(off0), [st] "s"(st), [nl] "v"(nlive)
                         : "memory", "vcc", "scc");
        } else {
            asm volatile("s_mov_b64 %[sv], exec\n\tv_mov_b32 %[t], %[off0]\n\t"
                         SLAI_FLOW_PIECE(0) SLAI_FLOW_PIECE(1) SLAI_FLOW_PIECE(2) SLAI_FLOW_PIECE(3) SLAI_FLOW_PIECE(4) SLAI_FLOW_PIECE(5)
                         SLAI_FLOW_PIECE(6) SLAI_FLOW_PIECE(7) SLAI_FLOW_PIECE(8) SLAI_FLOW_PIECE(9) SLAI_FLOW_PIECE(10) SLAI_FLOW_PIECE(11)
                         "s_waitcnt vmcnt(0)"
                         : [v0] "+v"(v[0]), [v1] "+v"(v[1]), [v2] "+v"(v[2]), [v3] "+v"(v[3]), [v4] "+v"(v[4]), [v5] "+v"(v[5]), [v6] "+v"(v[6]),
                           [v7] "+v"(v[7]), [v8] "+v"(v[8]), [v9] "+v"(v[9]), [v10] "+v"(v[10]), [v11] "+v"(v[11]), [sv] "=&s"(saved), [t] "=&v"(t)
                         : [base] "s"(base_bits), [off0] "v"(off0), [st] "s"(st), [nl] "v"(nlive)
                         : "memory", "vcc", "scc");
        }
        bool hole = false;
#pragma unroll
        for (int k = 0; k < N; ++k) hole = hole || ((uint32_t)k < nlive && flow_empty(v[k]));
        if (!__any(hole) || f.dead) break;
        flow_backoff(f, deadline);
    }
}
#undef SLAI_FLOW_PIECE

// ---- a 64-row tile (q / k / v, gate + up, output matrix) -----------------------------------------------------------------
struct TileIn {
    const float *x;           // the input vector (n floats)
    bool flow;                // written by this launch: read with flow_acquire16; else ordinary memory from before the launch
    const float *norm_w;      // RMSNorm weights
    uint32_t n;               // columns
    float eps;
};

// Stages the normalised-but-unscaled input (x * w, then the n/16 sums of 16) into `slot` and the sum of squares into
// red[0..3]: the last four waves of the workgroup, up to four 16-byte pieces per lane (n <= 4096).  rms_norm.slang:48-67;
// the scale is applied to the finished dot product.
__device__ __forceinline__ void stage_tile_input(const TileIn &in, float *slot, float *red, Flow &f) {
    const int tid = phase_tid(), lane = tid & 63, wave = tid >> 6;
    const uint32_t l = tid - (PNW - 4) * 64;                       // 0 .. 255
    uint32_t idx[4];
    bool live[4];
    float4 w[4];
    uint32_t nlive = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {                                   // the norm weights first: they depend on nothing
        idx[k] = l + 256 * k;
        live[k] = idx[k] < in.n / 4;
        nlive += live[k] ? 1u : 0u;
        w[k] = *reinterpret_cast<const float4 *>(in.norm_w + 4 * (live[k] ? idx[k] : l));
    }
    u32x4 raw[4];
    if (in.flow) {
        const uint32_t first = 64u * (uint32_t)(wave - (PNW - 4));       // the first piece of this wave's share
        flow_probe(in.x + 4 * (size_t)(first < in.n / 4 ? first : 0), f);
        flow_acquire<4>(in.x, l * 16u, 256u * 16u, nlive, raw, f);
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) raw[k] = *reinterpret_cast<const u32x4 *>(in.x + 4 * (live[k] ? idx[k] : l));
    }
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float4 v = make_float4(__uint_as_float(raw[k].x), __uint_as_float(raw[k].y), __uint_as_float(raw[k].z), __uint_as_float(raw[k].w));
        if (!live[k]) v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss);
        v.x *= w[k].x; v.y *= w[k].y; v.z *= w[k].z; v.w *= w[k].w;
        float s4 = (v.x + v.y) + (v.z + v.w);
        s4 += __shfl_xor(s4, 1, 64);
        s4 += __shfl_xor(s4, 2, 64);                               // lanes 4q..4q+3 hold 16 consecutive activations
        if (live[k]) {
            *reinterpret_cast<float4 *>(slot + 4 * idx[k]) = v;
            if ((lane & 3) == 0) slot[in.n + (idx[k] >> 2)] = s4;
        }
    }
    ss = wave_sum(ss);
    if (lane == 0) red[wave - (PNW - 4)] = ss;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");               // the slot is in L2 before the barrier lets the readers go
}

// One tile: rows tile*64 .. +63 of W (and W2) times the staged input; returns, in threads 0..63, the finished value of the
// thread's row (scaled; gate/up combined with SiLU when DUAL).  `stage`: false when the slot still holds this input.
// smem: partial[2][16][64], red[2][4] (red alternates between calls so that a fast wave cannot overwrite it early).
template <int T, bool DUAL>
__device__ __forceinline__ float tile64_phase(const uint8_t *W, const uint8_t *W2, uint32_t tile, uint32_t ncb, const TileIn &in, bool stage,
                                              float *slot, float *partial, float *red, Flow &f, uint64_t *tr) {
    using F = Tiled<T>;
    const int tid = phase_tid(), lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    constexpr int NM = DUAL ? 2 : 1;
    const bool has_unit = (uint32_t)wave < ncb;
    const bool stager = wave >= PNW - 4;
    typename F::Data d, e;
    uint16_t dt = 0, et = 0;
    // As much of the unit as the registers hold without spilling is requested before the wait (a spill of a requested
    // piece would make the wave wait for it before the barrier); the rest follows while the first stages are multiplied.
    UnitLoader<T, NM, DUAL ? 4 : (F::PT > 9 ? 6 : 8)> ld;
    auto request = [&]() {
        const size_t off = ((size_t)tile * ncb + wave) * unit_bytes;
        ld.unit[0] = W + off + lane * 16; ld.tailp[0] = W + off + (size_t)F::PT * 1024 + lane * 2; ld.d[0] = &d; ld.t[0] = &dt;
        if constexpr (DUAL) { ld.unit[1] = W2 + off + lane * 16; ld.tailp[1] = W2 + off + (size_t)F::PT * 1024 + lane * 2; ld.d[1] = &e; ld.t[1] = &et; }
        F::lead(ld);
    };
    stamp(tr, 0);
    if (stager && stage) {                                        // (either role, never both: the registers hold one at a time)
        stage_tile_input(in, slot, red, f);
        if (has_unit) request();
    } else if (has_unit) {
        request();
    }
    lds_barrier();
    stamp(tr, 1);
    float v = 0.0f, v2 = 0.0f;
    if (has_unit) {
        // The slot was rewritten with vector stores; the scalar cache may still hold what it held before.  Drop that,
        // and hand the compiler the pointer only now: loads through the constant address space move freely otherwise.
        asm volatile("s_dcache_inv\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
        uint64_t slot_bits = (uint64_t)(uintptr_t)slot;
        asm volatile("" : "+s"(slot_bits) : : "memory");
        cfloat *xsc = (cfloat *)slot_bits;
        ScalarX X{xsc + (size_t)wave * 256, xsc + in.n + (size_t)wave * 16};
        const typename F::Data *dp[NM];
        uint16_t tails[NM];
        float o2[NM];
        dp[0] = &d; tails[0] = dt;
        if constexpr (DUAL) { dp[1] = &e; tails[1] = et; }
        F::template dotn<NM>(dp, tails, X, o2, ld);
        v = o2[0];
        if constexpr (DUAL) v2 = o2[1];
    }
    stamp(tr, 2);
    partial[wave * 64 + lane] = v;
    if constexpr (DUAL) partial[(PNW + wave) * 64 + lane] = v2;
    lds_barrier();
    stamp(tr, 3);
    float o = 0.0f;
    if (tid < 64) {
        const float t = (red[0] + red[1]) + (red[2] + red[3]);
        const float scale = 1.0f / sqrtf(t / (float)in.n + in.eps);
        for (uint32_t w = 0; w < ncb; ++w) o += partial[w * 64 + tid];
        o *= scale;
        if constexpr (DUAL) {
            float up = 0.0f;
            for (uint32_t w = 0; w < ncb; ++w) up += partial[(PNW + w) * 64 + tid];
            up *= scale;
            o = up * (o / (1.0f + expf(-o)));                      // silu.slang:8-26
        }
    }
    return o;
}

// ---- a 16-row tile (attention output projection, down projection) -------------------------------------------------------
// Rows tile*16 .. +15 of W times the n-vector at `x` (written by this launch); returns the row's dot product in threads
// 0..15.  Waves 0 .. ngroups-1 multiply (one unit of 16 rows x 4 super-blocks each), the others fetch the vector into xs.
template <int T>
__device__ __forceinline__ float tile16_phase(const uint8_t *W, uint32_t tile, uint32_t ncb, uint32_t ngroups, const float *x, uint32_t n, float *xs,
                                              float *partial, Flow &f, uint64_t *tr) {
    using F = Tiled<T>;
    const int tid = phase_tid(), lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);
    const bool has_unit = (uint32_t)wave < ngroups;
    const uint32_t first_stager = ngroups < 12 ? ngroups : 12;
    const bool stager = (uint32_t)wave >= first_stager;
    typename F::Data d;
    uint16_t dt = 0;
    UnitLoader<T, 1, (F::PT > 9 ? 6 : 8)> ld;
    auto request = [&]() {
        const size_t off = ((size_t)tile * ngroups + wave) * unit_bytes;
        ld.unit[0] = W + off + lane * 16; ld.tailp[0] = W + off + (size_t)F::PT * 1024 + lane * 2; ld.d[0] = &d; ld.t[0] = &dt;
        F::lead(ld);
    };
    stamp(tr, 0);
    if (!stager) {
        if (has_unit) request();
    } else {
        // lane l of the nl stager lanes takes pieces l, l + nl, ...: four per round trip, or twelve when there are many
        const uint32_t nl = (PNW - first_stager) * 64, l = tid - first_stager * 64;
        const uint32_t chunks = n / 4;
        {
            const uint32_t first = (uint32_t)(wave - first_stager) * 64;            // the wave's first piece (if it has one)
            flow_probe(x + 4 * (size_t)(first < chunks ? first : 0), f);
        }
        if (chunks > 4 * nl) {
            const uint32_t trips = (chunks + 12 * nl - 1) / (12 * nl);
            for (uint32_t j = 0; j < trips; ++j) {                     // whole waves call the acquire
                const uint32_t i0 = 12 * j * nl + l;
                const uint32_t nlive = i0 < chunks ? min(12u, (chunks - i0 + nl - 1) / nl) : 0u;
                u32x4 raw[12];
                flow_acquire<12>(x, i0 * 16u, nl * 16u, nlive, raw, f);
#pragma unroll
                for (int k = 0; k < 12; ++k)
                    if ((uint32_t)k < nlive) *reinterpret_cast<u32x4 *>(xs + 4 * (size_t)(i0 + k * nl)) = raw[k];
            }
        } else {
            const uint32_t nlive = l < chunks ? min(4u, (chunks - l + nl - 1) / nl) : 0u;
            u32x4 raw[4];
            flow_acquire<4>(x, l * 16u, nl * 16u, nlive, raw, f);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if ((uint32_t)k < nlive) *reinterpret_cast<u32x4 *>(xs + 4 * (size_t)(l + k * nl)) = raw[k];
        }
        if (has_unit) request();
    }
    lds_barrier();
    stamp(tr, 1);
    float v = 0.0f;
    if (has_unit) {
        const int kq = lane >> 4, lane16 = lane & 15;
        const uint32_t cb = (uint32_t)wave * 4 + kq;
        const bool valid = cb < ncb;
        DevX X;
#pragma unroll
        for (int i = 0; i < 16; ++i) X.x[i] = valid ? xs[(size_t)cb * 256 + 16 * i + lane16] : 0.0f;
        if constexpr (T == T_Q6_K) {
#pragma unroll
            for (int i = 0; i < 16; ++i) X.s[i] = row16_sum(X.x[i]);
        } else {
#pragma unroll
            for (int i = 0; i < 16; i += 2) { X.s[i] = row16_sum(X.x[i] + X.x[i + 1]); X.s[i + 1] = 0.0f; }
        }
        const typename F::Data *dp[1] = {&d};
        uint16_t tails[1] = {dt};
        float o1[1];
        F::template dotn<1>(dp, tails, X, o1, ld);
        v = o1[0];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);                                // across the four super-blocks of the wave
    }
    stamp(tr, 2);
    if (lane < 16) partial[wave * 64 + lane] = v;
    lds_barrier();
    stamp(tr, 3);
    float o = 0.0f;
    if (tid < 16)
        for (uint32_t w = 0; w < ngroups; ++w) o += partial[w * 64 + tid];
    return o;
}

template <bool DUAL>
__device__ __forceinline__ float tile64_any(int type, const uint8_t *W, const uint8_t *W2, uint32_t tile, uint32_t ncb, const TileIn &in, bool stage,
                                            float *slot, float *partial, float *red, Flow &f, uint64_t *tr) {
    switch (type) {                                                // uniform over the workgroup
    case T_Q6_K: if constexpr (!DUAL) return tile64_phase<T_Q6_K, false>(W, W2, tile, ncb, in, stage, slot, partial, red, f, tr); else return 0.0f;
    case T_Q5_K: if constexpr (!DUAL) return tile64_phase<T_Q5_K, false>(W, W2, tile, ncb, in, stage, slot, partial, red, f, tr); else return 0.0f;
    default: return tile64_phase<T_Q4_K, DUAL>(W, W2, tile, ncb, in, stage, slot, partial, red, f, tr);
    }
}
__device__ __forceinline__ float tile16_any(int type, const uint8_t *W, uint32_t tile, uint32_t ncb, uint32_t ngroups, const float *x, uint32_t n, float *xs,
                                            float *partial, Flow &f, uint64_t *tr) {
    if (type == T_Q6_K) return tile16_phase<T_Q6_K>(W, tile, ncb, ngroups, x, n, xs, partial, f, tr);
    return tile16_phase<T_Q4_K>(W, tile, ncb, ngroups, x, n, xs, partial, f, tr);
}

// ---- the kernel ------------------------------------------------------------------------------------------------------------
// Workgroup roles.  q/k/v: workgroup i < 6 * n_heads takes tile (i / 8) % 6 of head (i % 8) + 8 * (i / 48) (two tiles each
// of v, k, q: the six tiles of a head run on one XCD, like the attention workgroup a0 + h of that head, a0 = 6 * n_heads;
// their hand-off goes through that XCD's L2, see kernels_gemv_rowtile.hip).  Projections: workgroup b takes rows 16b .. 16b+15
// and keeps their residual values from layer to layer.  gate/up: workgroup b takes rows 64b .. 64b+63.
template <bool F16>
__global__ void __launch_bounds__(PNT) llama_decode_persistent_kernel(const PersistentParams p) {
    extern __shared__ __align__(16) float smem[];
    __shared__ uint32_t wg_dead;                                   // the attention hand-off of this workgroup timed out
    // The description of the current layer and of the next one.  Read from memory at the moment of use, its lines (which
    // the weight stream has long pushed out of L2) would cost a round trip to memory each, one after the other.
    constexpr int LWORDS = sizeof(PersistentLayer) / 4;
    __shared__ uint32_t layer_words[2][LWORDS];
    float *partial = smem;                                         // [2][16][64]
    float *red = smem + 2 * PNW * 64;                              // [2][4]
    float *xs = red + 8;                                           // [max(dim, hidden)]
    touch_kernel_arguments<sizeof(PersistentParams)>();
    const uint32_t b = blockIdx.x;
    // A launch after one in which a reader gave up does nothing: the host has not looked yet (it queues many tokens), and
    // every further token would only wait out the same time limits.
    if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
    Flow f{p.abort_flag, false};
    const uint32_t dim = p.dim, hid = p.hidden, nh = p.n_heads;
    const uint32_t ncb = dim / 256, ncb_h = hid / 256, ng_o = ncb / 4, ng_d = (ncb_h + 3) / 4;
    const uint32_t a0 = 6 * nh;
    float *slot = p.slots + (size_t)b * p.slot_stride;
    // time stamps: 16 per layer (4 per phase: entered, input staged, multiplied, reduced), then 4 for the output matrix and the end
    uint64_t *trace = p.trace ? p.trace + (size_t)b * (16 * p.n_layers + 8) : nullptr;
    uint32_t phase = 0;                                            // parity picks the red[] half
    // the residual value of row 16b + tid: the embedding row the launch before this one left in p.x
    float xres = 0.0f;
    if (b < dim / 16 && threadIdx.x < 16) xres = p.x[16 * b + threadIdx.x];
    if (threadIdx.x == 0) wg_dead = 0;
    if (threadIdx.x < LWORDS && p.n_layers) layer_words[0][threadIdx.x] = reinterpret_cast<const uint32_t *>(p.layers)[threadIdx.x];
    __syncthreads();

    for (uint32_t l = 0; l < p.n_layers; ++l) {
        // this layer's description comes out of LDS field by field, as wave-uniform values, where it is used; the next
        // one's is requested now and parked in LDS at the end of the layer
        const uint32_t *lw = layer_words[l & 1u];
#define LPTR(T, field) ((T)(uintptr_t)join_words(uniform_word(lw[offsetof(PersistentLayer, field) / 4]), uniform_word(lw[offsetof(PersistentLayer, field) / 4 + 1])))
#define LINT(field) ((int)uniform_word(lw[offsetof(PersistentLayer, field) / 4]))
        uint32_t next_word = 0;
        if (threadIdx.x < LWORDS && l + 1 < p.n_layers) next_word = reinterpret_cast<const uint32_t *>(p.layers + l + 1)[threadIdx.x];
        uint64_t *tl = trace ? trace + 16 * l : nullptr;
        float *xa = p.xa + (size_t)l * dim, *xb = p.xb + (size_t)l * dim, *xm = p.xm + (size_t)l * dim, *hb = p.hb + (size_t)l * hid;
        // ---- q / k / v and the attention ---------------------------------------------------------------------------
        if (b < a0) {
            const uint32_t j = b >> 3, t = j % 6, h = (b & 7u) + 8u * (j / 6);
            const int s = (int)(t >> 1);                           // 0: v, 1: k, 2: q
            const uint32_t tile = 2 * h + (t & 1u);
            const uint8_t *W = s == 0 ? LPTR(const uint8_t *, wv) : (s == 1 ? LPTR(const uint8_t *, wk) : LPTR(const uint8_t *, wq));
            const int type = s == 0 ? LINT(tv) : (s == 1 ? LINT(tk) : LINT(tq));
            float *out = s == 0 ? p.vcol : (s == 1 ? p.kcol : p.q);
            const TileIn in{l == 0 ? p.x : xa, l != 0, LPTR(const float *, attn_norm), dim, p.eps};
            const float o = tile64_any<false>(type, W, nullptr, tile, ncb, in, true, slot, partial, red + 4 * (phase & 1u), f, tl);
            const uint32_t tid = phase_tid();
            if (tid < 64) {
                flow_store(out + (size_t)tile * 64 + tid, o);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (tid == 0) __hip_atomic_fetch_add(p.counters + (size_t)h * 32, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            ++phase;
        } else if (b < a0 + nh) {
            const uint32_t h = b - a0;
            AttnLaunch a{};
            a.q = p.q; a.knew = p.kcol; a.vnew = p.vcol;
            a.kcache = LPTR(void *, kcache); a.vcache = LPTR(void *, vcache); a.kv_f16 = F16;
            a.n_heads = nh; a.kv_mul = 1; a.head_size = 128; a.kv_dim = dim; a.seq_len = p.seq_len;
            a.pos_ptr = p.pos_ptr;
            a.qbias = LPTR(const float *, bq); a.kbias = LPTR(const float *, bk); a.vbias = LPTR(const float *, bv);
            a.rope_variant = p.rope_variant; a.rope_base = p.rope_base; a.rope_theta = p.rope_theta;
            a.out = xb; a.scratch = nullptr; a.n_splits = 1;
            uint32_t *counter = p.counters + (size_t)h * 32;
            const uint32_t tid = phase_tid();
            stamp(tl, 0);
            attn::attn_fast_body<F16, PNT, 128, true, true, 8, true>(a, h, 0u, tid, [&]() {
                if (tid == 0) {
                    uint32_t seen = 0, spins = 0;
                    uint64_t deadline = 0;
                    bool gave_up = f.dead;                         // (f.dead: uniform over the workgroup here)
                    while (!gave_up) {
                        // a read-modify-write that returns the value executes in the L2 the producers' atomics went to
                        const uint32_t zero = 0;
                        asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=&v"(seen) : "v"(counter), "v"(zero) : "memory");
                        if (seen >= 6u) break;
                        if ((++spins & 15u) == 0) {
                            const uint64_t now = wall_clock64();
                            if (deadline == 0) deadline = now + FLOW_WAIT_TICKS;
                            gave_up = now > deadline || __hip_atomic_load(f.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
                        }
                    }
                    if (gave_up) { wg_dead = 1; __hip_atomic_store(f.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
                    *counter = 0u;                                 // for the next layer; nobody else touches it until then
                }
                __syncthreads();
                asm volatile("" ::: "memory");
            });
            if (wg_dead) f.dead = true;
            stamp(tl, 3);
        }
        // ---- attention output projection into the residual ---------------------------------------------------------
        if (b < dim / 16) {
            const float o = tile16_any(LINT(to), LPTR(const uint8_t *, wo), b, ncb, ng_o, xb, dim, xs, partial, f, tl ? tl + 4 : nullptr);
            const uint32_t tid = phase_tid();
            if (tid < 16) { xres += o; flow_store(xm + 16 * b + tid, xres); }          // transformer.rs:352-355
        }
        // ---- RMSNorm + gate / up + SiLU ---------------------------------------------------------------------------------
        if (b < hid / 64) {
            const TileIn in{xm, true, LPTR(const float *, ffn_norm), dim, p.eps};
            const float o = tile64_any<true>(LINT(tg), LPTR(const uint8_t *, wgate), LPTR(const uint8_t *, wup), b, ncb, in, true, slot, partial, red + 4 * (phase & 1u), f, tl ? tl + 8 : nullptr);
            if (phase_tid() < 64) flow_store(hb + 64 * b + phase_tid(), o);
            ++phase;
        }
        // ---- down projection into the residual ----------------------------------------------------------------------------
        if (b < dim / 16) {
            const float o = tile16_any(LINT(td), LPTR(const uint8_t *, wdown), b, ncb_h, ng_d, hb, hid, xs, partial, f, tl ? tl + 12 : nullptr);
            float *next = p.xa + (size_t)(l + 1) * dim;
            const uint32_t tid = phase_tid();
            if (tid < 16) { xres += o; flow_store(next + 16 * b + tid, xres); }      // transformer.rs:362-365
        }
        if (threadIdx.x < LWORDS) layer_words[(l + 1) & 1u][threadIdx.x] = next_word;
        lds_barrier();
#undef LPTR
#undef LINT
    }
    // ---- final RMSNorm and the output matrix: tiles b, b + grid, ... -------------------------------------------------------
    {
        const uint32_t ntiles = (p.vocab + 63) / 64;
        const float *xl = p.n_layers ? p.xa + (size_t)p.n_layers * dim : p.x;
        const TileIn in{xl, p.n_layers != 0, p.out_norm, dim, p.eps};
        bool first = true;
        const uint32_t par = phase & 1u;                            // the input is staged once: its sum of squares stays where it is
        for (uint32_t tile = b; tile < ntiles; tile += gridDim.x) {
            const float o = tile64_any<false>(p.tout, p.wout, nullptr, tile, ncb, in, first, slot, partial, red + 4 * par, f, first && trace ? trace + 16 * p.n_layers : nullptr);
            const uint32_t tid = phase_tid();
            const uint32_t row = tile * 64 + tid;
            if (tid < 64 && row < p.vocab) p.logits[row] = o;
            first = false;
            lds_barrier();                                         // partial[] is reused by the next tile
        }
        stamp(trace ? trace + 16 * p.n_layers : nullptr, 4);
    }
}

// Fills the hand-off buffers of a launch with FLOW_EMPTY (16 bytes per thread and step).
__global__ void flow_fill_kernel(u32x4 *buf, size_t n16) {
    const u32x4 e = {FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) buf[i] = e;
}

}  // namespace

size_t persistent_smem_bytes(const PersistentParams &p) {
    return ((size_t)2 * PNW * 64 + 8 + (p.dim > p.hidden ? p.dim : p.hidden)) * sizeof(float);
}

// How many workgroups of the kernel the device keeps resident at once (0: it cannot run at all).
hipError_t persistent_capacity(const PersistentParams &p, int device, uint32_t *resident) {
    *resident = 0;
    const size_t smem = persistent_smem_bytes(p);
    const void *fn = p.kv_f16 ? (const void *)llama_decode_persistent_kernel<true> : (const void *)llama_decode_persistent_kernel<false>;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    int per_cu = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, PNT, smem);
    if (e != hipSuccess) return e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return e;
    *resident = (uint32_t)(per_cu > 0 ? per_cu : 0) * (uint32_t)prop.multiProcessorCount;
    return hipSuccess;
}

hipError_t launch_flow_fill(hipStream_t s, void *buf, size_t bytes) {
    if (bytes % 16 || (uintptr_t)buf % 16) return hipErrorInvalidValue;
    flow_fill_kernel<<<64, 1024, 0, s>>>((u32x4 *)buf, bytes / 16);
    return hipGetLastError();
}

hipError_t launch_decode_persistent(hipStream_t s, const PersistentParams &p, uint32_t grid) {
    const size_t smem = persistent_smem_bytes(p);
    if (p.kv_f16) llama_decode_persistent_kernel<true><<<grid, PNT, smem, s>>>(p);
    else llama_decode_persistent_kernel<false><<<grid, PNT, smem, s>>>(p);
    return hipGetLastError();
}

}  // namespace slai
