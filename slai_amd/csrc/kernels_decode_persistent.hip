// One launch per token for the Llama-2 layer stack: every layer's RMSNorm + q/k/v, RoPE + cache write + attention,
// output projection, RMSNorm + gate/up + SiLU and down projection, then the final RMSNorm and the output matrix
// (`Llama2::launch`, crates/slai/src/models/llama2/transformer.rs:316-381), in a grid that stays resident.
//
// Why: at batch 1 a layer is four points at which every workgroup needs a vector that all the others produced, and a
// kernel boundary at each of them costs about as much as streaming the weights between them.  Here the workgroups stay
// where they are and hand the vectors over themselves:
//   * a producer writes its slice of the vector with agent-scope stores into a buffer that was filled with FLOW_EMPTY
//     before the launch (one buffer per layer and vector, so nothing is ever reused inside a launch);
//   * a consumer watches one word of the vector until it is there, then asks for its whole part, and the lanes that see
//     an empty word in theirs ask again until none does -- the data is its own flag: no counter, no fence, no barrier
//     round trip;
//   * a wave asks for the weights of its NEXT phase as soon as the registers of the current one are free, right after its
//     dot product: the weights travel while the hand-off is waited for.  Loads retire in issue order, so a wave's poll
//     waits behind its own requests: every wave waits for its own input itself, with the unit it multiplies next asked
//     for one phase earlier (and nothing may be spilled: a scratch reload waits behind the requested weights too).
// The workgroups that multiply q, k and v also add the bias, rotate, and write the cache row; the attention of a head is
// one workgroup that asks for the cached rows before the query exists.  Q4_K and Q6_K dot products run on the matrix
// cores (mfma_q4k.h), Q5_K on the vector unit with wave-uniform activations (kernels_gemv_rowtile.hip's arithmetic).
// Work is cut into units of equal size rather than whole tiles (resident_plan.h): a unit of a 64-row-tile matrix is any
// run of up to 64 rows, so that every compute unit streams the same number of bytes in a phase.
//
// Where things are: every offset the kernel forms comes from resident_plan.h, which a host program walks for every
// (workgroup, wave, lane, layer) against the sizes of the allocations.  Weights, norm vectors and hand-off vectors are
// read through buffer descriptors that carry those sizes, so an access outside of them reads zero (or is dropped)
// instead of faulting.
//
// Every wait is bounded.  A reader that gives up sets a flag the host turns into an error, and from then on no reader of
// the launch waits again, so a launch always ends.  The grid is never larger than what the device keeps resident.
#include "common.h"
#include "attention_fast.h"
#include <cstddef>
#include "device_util.h"
#include "gemv_operands.h"
#include "mfma_q4k.h"
#include "quant_tiled.h"
#include "resident_plan.h"

namespace slai {
namespace {

using namespace lanes;

constexpr int PNT = plan::WG_THREADS, PNW = plan::WG_WAVES;   // threads and waves of a workgroup

// Who a thread is: the wave index is a wave-uniform value handed down from the top of the kernel, the lane index is
// recomputed where it is needed.  The thread index itself must not live in a vector register across the layer loop: it
// gets spilled there, and a reload of it behind the weights requested ahead waits for all of them.
__device__ __forceinline__ uint32_t lane_id() {
    uint32_t l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));      // (volatile: recomputed at every use, never kept)
    return l;
}

// A wave-uniform value as one the compiler cannot follow: what is derived from it (comparisons, conversions) is computed
// where it is used instead of once before the layer loop -- hoisted, a flag or a converted constant lives in a vector
// register across the whole loop, is spilled there, and its reload waits behind the weights requested ahead.
__device__ __forceinline__ uint32_t fresh(uint32_t v) {
    asm volatile("" : "+s"(v));
    return v;
}

// Lane exchanges inside the phases.  The library forms (__shfl_xor) derive their lane index once, the compiler then keeps
// every `lane ^ mask` alive across the whole layer loop -- in spilled registers, and a reload of one behind the weights
// requested ahead waits for all of them.  These recompute the index where it is used.
__device__ __forceinline__ float lane_xor(float v, int mask) {
    const int l = (int)lane_id();
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(((l ^ mask) & 63) << 2, __builtin_bit_cast(int, v)));
}
__device__ __forceinline__ float wave_total(float v) {            // the sum over the wave, in every lane
    v += mq::dpp<mq::DPP_XOR1>(v); v += mq::dpp<mq::DPP_XOR2>(v); v += mq::dpp<mq::DPP_HALF_MIRROR>(v); v += mq::dpp<mq::DPP_MIRROR>(v);
    const int b = __builtin_bit_cast(int, v);                   // every lane of a row of 16 holds the row's sum
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// Optional time stamps (the constant 100 MHz clock) for a per-phase time line of every workgroup: profilers see one long
// kernel.  `row` is null unless the host asked for a trace.
__device__ __forceinline__ void stamp(uint64_t *row, uint32_t k, uint32_t wave) {
    if (row && fresh(wave) == 0 && lane_id() == 0) row[k] = wall_clock64();
}

// ---- memory seen through buffer descriptors ------------------------------------------------------------------------------
// A descriptor holds the address and the size in bytes of one matrix or vector; loads and stores name a byte offset, and
// the hardware compares it with the size: outside of it a load returns zero and a store is dropped.
using Rsrc = __amdgpu_buffer_rsrc_t;
typedef uint32_t u32x4b __attribute__((ext_vector_type(4)));
constexpr int RSRC_WORD3 = 0x00020000;                        // untyped 32-bit data, no swizzle
constexpr int AUX_PLAIN = 0;
constexpr int AUX_STREAM = 2;                                 // non-temporal: weights, read exactly once per launch, should not displace the hand-off vectors in the caches (+1.5 % tok/s)
constexpr int AUX_FLOW = (int)0x80000010u;                    // agent scope (sc1): not served by a cache of this die; never merged or hoisted
constexpr int AUX_ONCE = (int)0x80000000u;                    // through the caches like any load, but never merged or hoisted
struct DevBuf {                                               // wave-uniform
    Rsrc rs;
    const void *ptr;
    uint32_t bytes;
    int type;
};
__device__ __forceinline__ Rsrc make_rsrc(const void *p, uint32_t bytes) { return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), (short)0, (int)bytes, RSRC_WORD3); }
__device__ __forceinline__ DevBuf dev_buf(const void *p, uint32_t bytes, int type = 0) { return DevBuf{make_rsrc(p, bytes), p, bytes, type}; }
__device__ __forceinline__ DevBuf dev_buf(const ResidentBuf &b) { return dev_buf(b.ptr, b.bytes, (int)b.type); }
// entry `word` (in 32-bit words) of the layer description parked in LDS, as wave-uniform values
__device__ __forceinline__ DevBuf layer_buf(const uint32_t *lw, uint32_t word) {
    const uint64_t bits = join_words(uniform_word(lw[word]), uniform_word(lw[word + 1]));
    return dev_buf((const void *)(uintptr_t)bits, uniform_word(lw[word + 2]), (int)uniform_word(lw[word + 3]));
}
#define LAYER_BUF(lw, field) layer_buf(lw, (uint32_t)(offsetof(PersistentLayer, field) / 4))
static_assert(sizeof(ResidentBuf) == 16 && offsetof(ResidentBuf, ptr) == 0 && offsetof(ResidentBuf, bytes) == 8 && offsetof(ResidentBuf, type) == 12, "layer_buf reads these words");

template <int AUX> __device__ __forceinline__ u32x4 buf_load16(Rsrc rs, uint32_t off, uint32_t soff = 0) {
    const u32x4b v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, (int)soff, AUX);
    return u32x4{v.x, v.y, v.z, v.w};
}
__device__ __forceinline__ float4 as_float4(u32x4 v) { return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)); }
// one float of a hand-off vector, at agent scope
__device__ __forceinline__ void flow_put(Rsrc rs, uint32_t index, float v) { __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rs, (int)(index * 4u), 0, AUX_FLOW); }

// Issues the 16-byte pieces of one unit (of both matrices of a gated pair) on request of the dot product, through the
// matrices' descriptors.  voff: byte offset of this lane's 16 bytes of piece 0; piece P lies P * 1024 further.
template <int T, int N, int LD> struct BufUnitLoader {
    static constexpr int DEPTH = LD;
    static constexpr int LEAD = LD;
    using F = Tiled<T>;
    Rsrc rs[N];
    uint32_t voff[N], toff[N];
    typename F::Data *d[N];
    uint16_t *t[N];
    template <int P> __device__ __forceinline__ void piece() const {
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const u32x4b v = __builtin_amdgcn_raw_buffer_load_b128(rs[n], (int)voff[n], P * 1024, AUX_STREAM);
            d[n]->p[P] = U4{v.x, v.y, v.z, v.w};
        }
    }
    __device__ __forceinline__ void tail() const {
#pragma unroll
        for (int n = 0; n < N; ++n) *t[n] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs[n], (int)toff[n], 0, AUX_PLAIN);
    }
};

// ---- waiting for data -------------------------------------------------------------------------------------------------
constexpr uint64_t FLOW_WAIT_TICKS = 2u * 1000u * 1000u;      // 20 ms of the 100 MHz clock: what a reader waits before it gives up (a token takes about 1)
constexpr uint32_t LDS_WAIT_ROUNDS = 1u << 22;                 // rounds of a wait on a word of LDS (at least 60 ns each: a quarter of a second, beyond every bounded wait of the waves it waits for)

struct Flow {
    uint32_t *abort_flag;     // device word: non-zero once any reader of the launch has given up
    bool dead;                // wave-uniform: this wave no longer waits
};

// One round of a failed wait.  A round is a round trip to memory (about a microsecond), so the clock is looked at every
// 16th and the flag of the launch every 64th round only: neither may add a dependent memory access to every poll.
__device__ __forceinline__ void flow_backoff(Flow &f, uint64_t &deadline, uint32_t &rounds) {
    ++rounds;
    if ((rounds & 15u) != 0) return;
    const uint64_t now = wall_clock64();
    if (deadline == 0) deadline = now + FLOW_WAIT_TICKS;
    if (now > deadline) {
        f.dead = true;
        if (lane_id() == 0) __hip_atomic_store(f.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if ((rounds & 63u) == 0 && __hip_atomic_load(f.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
        f.dead = true;
    }
}

// A word of LDS that the waves of a workgroup count themselves in on (real LDS instructions: a flat access would return
// behind the wave's outstanding weight requests).
typedef __attribute__((address_space(3))) uint32_t LdsWord;
__device__ __forceinline__ void lds_count_in(LdsWord *c) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");         // what the wave left in LDS comes first
    if (lane_id() == 0) __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// Waits until `need` waves have counted themselves in, and clears the word for its next use (which lies behind a
// workgroup barrier).  Every wave that counts does so unconditionally after waits that are bounded themselves; the
// rounds here are bounded all the same.
__device__ __forceinline__ void lds_count_wait(LdsWord *c, uint32_t need, Flow &f) {
    uint32_t rounds = 0;
    while (__hip_atomic_load(c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < need) {
        __builtin_amdgcn_s_sleep(1);
        if (++rounds > LDS_WAIT_ROUNDS) {
            f.dead = true;
            if (lane_id() == 0) __hip_atomic_store(f.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    if (lane_id() == 0) __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Every wave of the device waits for its input at some point, most of them for many microseconds, and a request for a
// hand-off vector is served by memory itself: what the waiting waves ask for competes with the weights.  So a wave first
// watches a single word -- every lane the same one: one request of one line per round -- and only when that word is there
// asks for its whole part, which the other producers have then written as well or are about to.
__device__ __forceinline__ void flow_watch(Rsrc x, uint32_t word, Flow &f) {
    uint64_t deadline = 0;
    uint32_t rounds = 0;
    for (;;) {
        const uint32_t w = __builtin_amdgcn_raw_buffer_load_b32(x, (int)(word * 4u), 0, AUX_FLOW);
        if (w != FLOW_EMPTY || f.dead) return;
        flow_backoff(f, deadline, rounds);
    }
}
// The 16 bytes of piece `piece` of a hand-off vector for every lane of the wave, once no word of any lane's piece is
// empty: one request per lane and round, repeated by the whole wave (after a time-out the values are whatever was there).
__device__ __forceinline__ u32x4 flow_take(Rsrc x, uint32_t piece, Flow &f) {
    uint64_t deadline = 0;
    uint32_t rounds = 0;
    flow_watch(x, uniform_word(piece) * 4u + 255u, f);           // the last word of the wave's 64 pieces
    // Every workgroup takes the whole vector: asked of memory 256 times over, that is what a hand-off costs.  The first
    // request therefore goes through the die's L2 like any load, and the workgroups of a die share one fetch.  A line
    // that was cached before its producer wrote it shows empty words (a word only ever changes from empty to its value,
    // and no line survives from an earlier launch: the caches are invalidated when a kernel starts), and then the
    // requests go to memory as before.
    u32x4 v = buf_load16<AUX_ONCE>(x, piece * 16u);
    // only the lanes whose piece shows an empty word ask again: what the late producers wrote, not the whole part
    for (;;) {
        const bool hole = flow_empty(v);
        if (!__any(hole) || f.dead) return v;
        if (hole) v = buf_load16<AUX_FLOW>(x, piece * 16u);
        flow_backoff(f, deadline, rounds);
    }
}
// Four pieces per lane (piece0 + 64 k: the same lane's piece of four consecutive super-blocks; k >= n is not asked for
// and comes back as zeros), under the same rule.
__device__ __forceinline__ void flow_take4(Rsrc x, uint32_t piece0, uint32_t n, u32x4 (&out)[4], Flow &f) {
    uint64_t deadline = 0;
    uint32_t rounds = 0;
    flow_watch(x, (uniform_word(piece0) + 64u * (n - 1u)) * 4u + 255u, f);
#pragma unroll
    for (int k = 0; k < 4; ++k) {                                 // (through the die's L2 first: see flow_take)
        out[k] = u32x4{0u, 0u, 0u, 0u};
        if ((uint32_t)k < n) out[k] = buf_load16<AUX_ONCE>(x, (piece0 + 64u * k) * 16u);
    }
    for (;;) {
        bool hole = false;
#pragma unroll
        for (int k = 0; k < 4; ++k) hole = hole || flow_empty(out[k]);
        if (!__any(hole) || f.dead) return;
#pragma unroll
        for (int k = 0; k < 4; ++k)                               // (a piece past n is zeros: never empty)
            if (flow_empty(out[k])) out[k] = buf_load16<AUX_FLOW>(x, (piece0 + 64u * k) * 16u);
        flow_backoff(f, deadline, rounds);
    }
}
// ---- weights on their way ---------------------------------------------------------------------------------------------------
// A phase's multiply cannot start before its input exists, but its weights do not depend on anything: each wave asks
// for the unit of its NEXT phase as soon as the registers of the current one are free (right after its dot product,
// before the partial sums are reduced and handed over -- except wave 0 of a 16-row-tile phase, which adds up and hands the
// rows on first: finish16), so the weights travel while the hand-off is waited for.
struct Unit {                 // the 16-byte pieces a wave requested ahead (which ones depends on the block format)
    U4 a[13], b[9];           // first matrix / second matrix of a gated pair
    uint16_t ta;              // 2-byte tail of the first matrix (Q6_K)
};
struct Req {                  // where the wave's unit lies: kept from the request to the multiply, which asks for the rest
    Rsrc rs[2];
    uint32_t voff, toff;
};
// Every piece (and the tail) of a single matrix's unit: the block format only decides how many pieces there are, so the
// request needs no code per format (the registers of a Unit hold the largest).
// (The fences keep the requests where they are written: moved up into the multiply before them, they would need its
// registers as well.)
__device__ __forceinline__ void request_fence() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
__device__ __forceinline__ void request_all(Unit &u, const Req &r, int type) {
    const uint32_t pt = tiled_pieces(type);
    request_fence();
    u = Unit{};                                                  // (nothing of an earlier unit stays alive in the registers)
#pragma unroll
    for (int P = 0; P < 13; ++P) {
        if ((uint32_t)P < pt) {
            const u32x4b v = __builtin_amdgcn_raw_buffer_load_b128(r.rs[0], (int)r.voff, P * 1024, AUX_STREAM);
            u.a[P] = U4{v.x, v.y, v.z, v.w};
        }
    }
    if (tiled_tail(type)) u.ta = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r.rs[0], (int)r.toff, 0, AUX_PLAIN);
    request_fence();
}
// A gated pair of Q4_K matrices: the header and the first GATED_LEAD stages of both (8: everything); the multiply asks
// for the rest.
constexpr int GATED_LEAD = 8;
__device__ __forceinline__ void request_gated(Unit &u, const Req &r) {
    u = Unit{};
    request_fence();
#pragma unroll
    for (int P = 0; P <= GATED_LEAD; ++P) {
        const u32x4b v = __builtin_amdgcn_raw_buffer_load_b128(r.rs[0], (int)r.voff, P * 1024, AUX_STREAM);
        const u32x4b w = __builtin_amdgcn_raw_buffer_load_b128(r.rs[1], (int)r.voff, P * 1024, AUX_STREAM);
        u.a[P] = U4{v.x, v.y, v.z, v.w};
        u.b[P] = U4{w.x, w.y, w.z, w.w};
    }
    request_fence();
}

// ---- a unit of up to 64 rows of a 64-row-tile matrix (q / k / v, gate + up, output matrix) -------------------------------
struct TileIn {
    Rsrc x;                   // the input vector (n floats)
    bool flow;                // written by this launch: read with flow_take; else ordinary memory from before the launch
    Rsrc norm_w;              // RMSNorm weights (n floats)
    uint32_t n;               // columns
    float eps;
};

// Rows unit.row0 .. + unit.nrows - 1 of W (and W2), super-block `wave`: lane i owns row unit.row0 + i (lanes past the
// unit repeat its last row and their results are dropped).
template <bool DUAL>
__device__ __forceinline__ void request64(Unit &u, Req &r, const DevBuf &W, const DevBuf &W2, const plan::RowUnit unit, uint32_t ncb, uint32_t wave_) {
    const uint32_t lane = lane_id(), wave = fresh(wave_);
    if (wave >= ncb) { u = Unit{}; return; }
    const uint32_t unit_bytes = plan::unit_bytes_of(W.type);
    const uint32_t row = plan::unit_row(unit, lane);
    r.rs[0] = W.rs; r.rs[1] = W2.rs;
    r.voff = plan::tile64_piece0(row, wave, ncb, unit_bytes);
    r.toff = plan::tile64_tail(row, wave, ncb, unit_bytes, tiled_pieces(W.type));
    if constexpr (DUAL) request_gated(u, r);
    else request_all(u, r, W.type);
}

// The multiply of a requested unit: wave w waits for the 256 input values of super-block w (one 16-byte piece per lane),
// leaves x * w and the sums of 16 in its part of the workgroup's slot (rms_norm.slang:48-67; the scale is applied to the
// finished dot product), reads them back as scalar operands, multiplies, and leaves its partial sums in LDS.  `stage`:
// false when the slot still holds this input.  partial[2][16][64], red[16].
template <int T, bool DUAL>
__device__ __forceinline__ void mult64(const Unit &u, const Req &r, uint32_t ncb, const TileIn &in, bool stage, float *slot, char *lds, float *partial, float *red, Flow &f,
                                       uint64_t *tr, const uint32_t wave_) {
    using F = Tiled<T>;
    const int lane = (int)lane_id();
    const uint32_t wave = fresh(wave_);
    constexpr int NM = DUAL ? 2 : 1;
    float v = 0.0f, v2 = 0.0f;
    if constexpr (T == T_Q4_K || T == T_Q6_K) {
        // on the matrix cores (mfma_q4k.h): the wave stages its super-block in LDS, for itself alone
        if ((uint32_t)wave < ncb) {
            char *sb = lds + plan::lds_mq_sb(wave, 0);
            if (stage) {
                const uint32_t piece = plan::wave_piece((uint32_t)wave, (uint32_t)lane);
                const float4 w = as_float4(buf_load16<AUX_PLAIN>(in.norm_w, piece * 16u));
                float4 x = as_float4(in.flow ? flow_take(in.x, piece, f) : buf_load16<AUX_PLAIN>(in.x, piece * 16u));
                float ss = fmaf(x.x, x.x, fmaf(x.y, x.y, fmaf(x.z, x.z, x.w * x.w)));
                ss = wave_total(ss);
                if (lane == 0) red[wave] = ss;
                x.x *= w.x; x.y *= w.y; x.z *= w.z; x.w *= w.w;
                mq::stage_superblock<T>(x, sb);
            }
            stamp(tr, 1, wave);
            typename F::Data d, e;
#pragma unroll
            for (int i = 0; i < F::PT; ++i) d.p[i] = u.a[i];
            if constexpr (DUAL) {
#pragma unroll
                for (int i = 0; i < F::PT; ++i) e.p[i] = u.b[i];
            }
            if constexpr (T == T_Q6_K) {
                static_assert(!DUAL, "gated pairs are Q4_K");
                v = mq::dot_q6k(d, u.ta, sb, lds + plan::lds_mq_zero(), lds + plan::lds_mq_cs(wave));
            } else {
                const typename F::Data *dp[NM];
                float o2[NM];
                dp[0] = &d;
                if constexpr (DUAL) dp[1] = &e;
                mq::dot_q4k<NM>(dp, sb, lds + plan::lds_mq_zero(), lds + plan::lds_mq_cs(wave), o2);
                v = o2[0];
                if constexpr (DUAL) v2 = o2[1];
            }
        }
    } else if ((uint32_t)wave < ncb) {
        if (stage) {
            const uint32_t piece = plan::wave_piece((uint32_t)wave, (uint32_t)lane);
            const float4 w = as_float4(buf_load16<AUX_PLAIN>(in.norm_w, piece * 16u));
            float4 x = as_float4(in.flow ? flow_take(in.x, piece, f) : buf_load16<AUX_PLAIN>(in.x, piece * 16u));
            float ss = fmaf(x.x, x.x, fmaf(x.y, x.y, fmaf(x.z, x.z, x.w * x.w)));
            ss = wave_total(ss);
            if (lane == 0) red[wave] = ss;
            x.x *= w.x; x.y *= w.y; x.z *= w.z; x.w *= w.w;
            float s4 = (x.x + x.y) + (x.z + x.w);
            s4 += lane_xor(s4, 1);
            s4 += lane_xor(s4, 2);                                     // lanes 4q..4q+3 hold 16 consecutive activations
            *reinterpret_cast<float4 *>(slot + 4 * piece) = x;
            if ((lane & 3) == 0) slot[in.n + (piece >> 2)] = s4;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");           // the wave's part of the slot is in L2
        }
        stamp(tr, 1, wave);
        // The slot was rewritten with vector stores; the scalar cache may still hold what it held before.  Drop that,
        // and hand the compiler the pointer only now: loads through the constant address space move freely otherwise.
        asm volatile("s_dcache_inv\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
        uint64_t slot_bits = (uint64_t)(uintptr_t)slot;
        asm volatile("" : "+s"(slot_bits) : : "memory");
        cfloat *xsc = (cfloat *)slot_bits;
        ScalarX X{xsc + plan::slot_x((uint32_t)wave), xsc + in.n + (size_t)wave * 16};
        typename F::Data d, e;
#pragma unroll
        for (int i = 0; i < F::PT; ++i) d.p[i] = u.a[i];
        if constexpr (DUAL) {
#pragma unroll
            for (int i = 0; i < F::PT; ++i) e.p[i] = u.b[i];
        }
        uint16_t dt = u.ta, et = 0;
        const typename F::Data *dp[NM];
        uint16_t tails[NM];
        float o2[NM];
        dp[0] = &d; tails[0] = dt;
        if constexpr (DUAL) {
            dp[1] = &e; tails[1] = et;
            BufUnitLoader<T, 2, GATED_LEAD> ld;                        // asks for the pieces that were not requested ahead
            ld.rs[0] = r.rs[0]; ld.voff[0] = r.voff; ld.toff[0] = r.toff; ld.d[0] = &d; ld.t[0] = &dt;
            ld.rs[1] = r.rs[1]; ld.voff[1] = r.voff; ld.toff[1] = r.toff; ld.d[1] = &e; ld.t[1] = &et;
            F::template dotn<2>(dp, tails, X, o2, ld);
        } else {
            F::template dotn<1>(dp, tails, X, o2);                   // the whole unit was requested ahead
        }
        v = o2[0];
        if constexpr (DUAL) v2 = o2[1];
    }
    stamp(tr, 2, wave);
    partial[wave * 64 + lane] = v;
    if constexpr (DUAL) partial[(PNW + wave) * 64 + lane] = v2;
}

// After the barrier: thread i < 64 of the workgroup adds up row i of the unit (scaled; gate / up combined with SiLU).
template <bool DUAL>
__device__ __forceinline__ float finish64(uint32_t ncb, const TileIn &in, const float *partial, const float *red, uint64_t *tr, uint32_t wave_) {
    const uint32_t wave = fresh(wave_);
    lds_barrier();
    stamp(tr, 3, wave);
    const int tid = (int)(wave * 64u + lane_id());
    float o = 0.0f;
    if (tid < 64) {
        float t = 0.0f;
        for (uint32_t w = 0; w < ncb; ++w) { t += red[w]; o += partial[w * 64 + tid]; }
        const float scale = 1.0f / sqrtf(t / (float)fresh(in.n) + in.eps);
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

// ---- 16-row tiles (attention output projection, down projection) ---------------------------------------------------------
// Rows tile*16 .. +15 of W times an n-vector written by this launch, plus the residual.  A tile takes `ngroups` waves (one
// unit of 16 rows x 4 super-blocks each); a workgroup runs up to two tiles side by side (plan::Tiles16): waves
// k * ngroups .. (k + 1) * ngroups - 1 multiply tile k.  Each wave waits for the 1024 input values of its four
// super-blocks, 16 per lane, straight into the registers they are used from.
__device__ __forceinline__ void request16(Unit &u, Req &r, const DevBuf &W, const plan::Tiles16 t, uint32_t ngroups, uint32_t wave_) {
    const uint32_t lane = lane_id(), wave = fresh(wave_);
    if (wave >= ngroups * t.n) { u = Unit{}; return; }
    const uint32_t unit_bytes = plan::unit_bytes_of(W.type);
    const uint32_t k = wave / ngroups, g = wave - k * ngroups;
    r.rs[0] = W.rs; r.rs[1] = W.rs;
    r.voff = plan::tile16_piece0(plan::tiles16_tile(t, k), g, ngroups, unit_bytes, lane);
    r.toff = plan::tile16_tail(plan::tiles16_tile(t, k), g, ngroups, unit_bytes, tiled_pieces(W.type), lane);
    request_all(u, r, W.type);
}
// `res`: the vector the result is added to (complete long before this phase).  Thread i < 16 * t.n receives, in `residual`,
// element 16 * tile + i % 16 of it: asked for first, so that it is there when the reduction needs it.
template <int T>
__device__ __forceinline__ void mult16(const Unit &u, const plan::Tiles16 t, uint32_t ncb, uint32_t ngroups, Rsrc x, Rsrc res, bool res_flow, float &residual, char *lds,
                                       float *partial, LdsWord *arrived, Flow &f, uint64_t *tr, const uint32_t wave_) {
    using F = Tiled<T>;
    const int lane = (int)lane_id();
    const uint32_t wave = fresh(wave_);
    float v = 0.0f;
    residual = 0.0f;
    if (wave == 0 && (uint32_t)lane < 16u * t.n) {
        const uint32_t off = (plan::tiles16_row(t, (uint32_t)lane)) * 4u;
        residual = __uint_as_float(res_flow ? __builtin_amdgcn_raw_buffer_load_b32(res, (int)off, 0, AUX_FLOW) : __builtin_amdgcn_raw_buffer_load_b32(res, (int)off, 0, AUX_PLAIN));
    }
    // on the matrix cores (mfma_q4k.h): the wave stages its four super-blocks in LDS, for itself alone
    static_assert(T == T_Q4_K || T == T_Q6_K, "the projections into the residual are Q4_K or Q6_K");
    if (wave < ngroups * t.n) {
        const uint32_t g = wave % ngroups;
        const uint32_t n = plan::umin(4u, ncb - plan::tile16_sb(g, 0));
        u32x4 xv[4];
        flow_take4(x, plan::tile16_piece(g, 0, (uint32_t)lane), n, xv, f);
#pragma unroll
        for (int k = 0; k < 4; ++k) mq::stage_superblock<T>(as_float4(xv[k]), lds + plan::lds_mq_sb(wave, k));   // (past the end: zeros)
        stamp(tr, 1, wave);
        typename F::Data d;
#pragma unroll
        for (int i = 0; i < F::PT; ++i) d.p[i] = u.a[i];
        const char *sb = lds + plan::lds_mq_sb(wave, (uint32_t)lane >> 4);
        if constexpr (T == T_Q6_K) {
            v = mq::dot_q6k(d, u.ta, sb, lds + plan::lds_mq_zero(), lds + plan::lds_mq_cs(wave));
        } else {
            const typename F::Data *dp[1] = {&d};
            float o1[1];
            mq::dot_q4k<1>(dp, sb, lds + plan::lds_mq_zero(), lds + plan::lds_mq_cs(wave), o1);
            v = o1[0];
        }
        v += lane_xor(v, 16);
        v += lane_xor(v, 32);                                      // across the four super-blocks of the wave
    }
    stamp(tr, 2, wave);
    if (lane < 16) partial[wave * 64 + lane] = v;
    if (wave < ngroups * t.n) lds_count_in(arrived);
}
// The rows of the tiles are added up by wave 0 (thread i < 16 * t.n: row plan::tiles16_row(t, i)) as soon as the waves that
// multiplied have left their partial sums -- not behind the workgroup barrier: the other waves ask for the weights of
// their next phase before they get there, and a compute unit takes its requests at the rate memory answers them (the
// barrier came 1.3 us after the last product in the attention output projection, 2.3 us in the down projection).  The
// caller hands the result on, asks for wave 0's own next weights, and only then joins the barrier of the phase.
__device__ __forceinline__ float finish16(const plan::Tiles16 t, uint32_t ngroups, const float *partial, LdsWord *arrived, Flow &f, uint64_t *tr, uint32_t wave_) {
    const uint32_t wave = fresh(wave_);
    float o = 0.0f;
    if (wave == 0 && t.n != 0) {
        lds_count_wait(arrived, ngroups * t.n, f);
        stamp(tr, 3, wave);
        const uint32_t tid = lane_id();
        if (tid < 16u * t.n) {
            const uint32_t k = tid >> 4, j = tid & 15u;
            for (uint32_t w = 0; w < ngroups; ++w) o += partial[(k * ngroups + w) * 64 + j];
        }
    }
    return o;
}

// the block format is uniform over the workgroup
template <bool DUAL>
__device__ __forceinline__ void mult64_any(int type, const Unit &u, const Req &r, uint32_t ncb, const TileIn &in, bool stage, float *slot, char *lds, float *partial, float *red,
                                           Flow &f, uint64_t *tr, uint32_t wave) {
    switch (type) {
    case T_Q6_K: if constexpr (!DUAL) mult64<T_Q6_K, false>(u, r, ncb, in, stage, slot, lds, partial, red, f, tr, wave); break;
    case T_Q5_K: if constexpr (!DUAL) mult64<T_Q5_K, false>(u, r, ncb, in, stage, slot, lds, partial, red, f, tr, wave); break;
    default: mult64<T_Q4_K, DUAL>(u, r, ncb, in, stage, slot, lds, partial, red, f, tr, wave); break;
    }
}
__device__ __forceinline__ void mult16_any(int type, const Unit &u, const plan::Tiles16 t, uint32_t ncb, uint32_t ngroups, Rsrc x, Rsrc res, bool res_flow, float &residual,
                                           char *lds, float *partial, LdsWord *arrived, Flow &f, uint64_t *tr, uint32_t wave) {
    if (type == T_Q6_K) mult16<T_Q6_K>(u, t, ncb, ngroups, x, res, res_flow, residual, lds, partial, arrived, f, tr, wave);
    else mult16<T_Q4_K>(u, t, ncb, ngroups, x, res, res_flow, residual, lds, partial, arrived, f, tr, wave);
}

// ---- the attention of one head (transformer.rs:342-350: RoPE, cache write, scores, softmax, weighted values) ------------
// The workgroups that multiply q, k and v also add the bias, rotate, and write the cache row (rotate_and_store); what is
// left here is the part that needs the whole head.  Everything that depends on the position only -- the cached keys and
// values of up to ATT_PRE passes, all of them for the first 384 positions of an f16 cache -- is requested before the
// query exists.  Every wave runs a softmax of its own over the positions it owns; the newest position, whose key and
// value are produced in this launch, joins when the waves are merged.
template <bool F16> struct AttPass {
    static constexpr int KP = F16 ? 2 : 4, VP = F16 ? 1 : 2;    // 16-byte pieces of a lane's sixteen key / eight value elements
    U4 k[KP], v[2][VP];
};
template <bool F16> __device__ __forceinline__ void att_decode8(const U4 *r, float (&o)[8]) {
    if constexpr (F16) {
        const uint32_t u[4] = {r[0].x, r[0].y, r[0].z, r[0].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[2 * i] = attn::h2f((uint16_t)(u[i] & 0xffffu)); o[2 * i + 1] = attn::h2f((uint16_t)(u[i] >> 16)); }
    } else {
        o[0] = __uint_as_float(r[0].x); o[1] = __uint_as_float(r[0].y); o[2] = __uint_as_float(r[0].z); o[3] = __uint_as_float(r[0].w);
        o[4] = __uint_as_float(r[1].x); o[5] = __uint_as_float(r[1].y); o[6] = __uint_as_float(r[1].z); o[7] = __uint_as_float(r[1].w);
    }
}
__device__ __forceinline__ U4 as_u4(u32x4 v) { return U4{v.x, v.y, v.z, v.w}; }

constexpr int DPP_ROW_ROR8 = 0x128;                           // lane i of a row of 16 takes lane (i + 8) % 16

template <bool F16> struct Attention {
    using P = AttPass<F16>;
    static constexpr uint32_t ES = F16 ? 2 : 4;                 // bytes of a cache element
    static constexpr int ATT_PRE = F16 ? 3 : 1;                 // passes requested before the query is waited for
    const plan::Shape &sh;
    Rsrc kc, vc;              // the layer's caches
    uint32_t head, T;         // T: cached positions (= the position of this token)
    uint32_t wave;
    float m, lsum, o[8];      // this wave's running maximum and sum, this lane's eight outputs

    __device__ __forceinline__ void request(P &ps, uint32_t tb) const {
        const uint32_t lane = lane_id();
        // lanes without a position read position 0: a valid address (there is at least one cached position when any pass runs)
        const uint32_t t = plan::att_k_pos(tb, wave, lane);
        const uint32_t koff = plan::cache_elem(sh, t < T ? t : 0u, plan::att_k_elem(head, lane)) * ES;
#pragma unroll
        for (int j = 0; j < P::KP; ++j) ps.k[j] = as_u4(buf_load16<AUX_PLAIN>(kc, koff + 16u * j));
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const uint32_t tv = plan::att_v_pos(tb, wave, u, lane);
            const uint32_t voff = plan::cache_elem(sh, tv < T ? tv : 0u, plan::att_v_elem(head, lane)) * ES;
#pragma unroll
            for (int j = 0; j < P::VP; ++j) ps.v[u][j] = as_u4(buf_load16<AUX_PLAIN>(vc, voff + 16u * j));
        }
    }
    // scores of this wave's eight positions of the pass, softmax update, weighted values (cpu.rs:505-560 in one sweep)
    __device__ __forceinline__ void consume(const P &ps, uint32_t tb, const float (&qr)[16]) {
        const uint32_t lane = lane_id();
        const bool live = plan::att_k_pos(tb, wave, lane) < T;
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            float kv[8];
            att_decode8<F16>(ps.k + j * (P::KP / 2), kv);
#pragma unroll
            for (int q = 0; q < 8; ++q) part = fmaf(qr[8 * j + q], kv[q], part);
        }
        part = mq::sum8(part);                                   // over the eight lanes of the position
        const float sc = live ? part / sqrtf(128.0f) : -FLT_MAX;             // cpu.rs:521
        // the largest of the wave's eight scores: the row's two positions, then the four rows
        const float mrow = fmaxf(sc, mq::dpp<mq::DPP_MIRROR>(sc));
        const int mb = __builtin_bit_cast(int, mrow);
        const float mx = fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 0)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 16))),
                               fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 32)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(mb, 48))));
        const float mn = fmaxf(m, mx);
        const float resc = expf(m - mn);                        // 0 on the first live pass, 1 while nothing was live
        const float pr = live ? expf(sc - mn) : 0.0f;
        lsum = fmaf(lsum, resc, (lane & 7u) == 0 ? pr : 0.0f);
#pragma unroll
        for (int q = 0; q < 8; ++q) o[q] *= resc;
        m = mn;
        // The weights of the row's two positions (plan::att_v_pos: value lanes of row r take positions 2 r and 2 r + 1):
        // lanes 0-7 of the row scored the first, lanes 8-15 the second.
        const float other = mq::dpp<DPP_ROW_ROR8>(pr);
        const bool second = (lane & 8u) != 0;
        const float pw[2] = {second ? other : pr, second ? pr : other};
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            float vv[8];
            att_decode8<F16>(ps.v[u], vv);
#pragma unroll
            for (int q = 0; q < 8; ++q) o[q] = fmaf(pw[u], vv[q], o[q]);
        }
    }
};

// The products of the newest position's score this lane owns: lane (i, jj) = (lane % 8, lane / 8 % 4) holds elements
// 16 i + 4 jj .. + 3 of the key in `kn` (and sixteen of the query in qr).
template <bool F16> __device__ __forceinline__ float att_new_score(const float (&qr)[16], u32x4 kn) {
    using C = attn::KV<F16>;                                    // (what the cache row holds: rounded to its element type)
    const uint32_t jj = (lane_id() >> 3) & 3u;
    float part = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float d = qr[4 * j] * C::round(__uint_as_float(kn.x));
        d = fmaf(qr[4 * j + 1], C::round(__uint_as_float(kn.y)), d);
        d = fmaf(qr[4 * j + 2], C::round(__uint_as_float(kn.z)), d);
        d = fmaf(qr[4 * j + 3], C::round(__uint_as_float(kn.w)), d);
        part = jj == (uint32_t)j ? d : part;
    }
    return part;
}

// lds: [16 waves][128] partial outputs, then the waves' maxima and sums.  q / knew / vnew: this layer's hand-off vectors
// (dim floats each); out: the attention output vector.
template <bool F16>
__device__ __forceinline__ void attend(const plan::Shape &sh, uint32_t head, uint32_t pos, Rsrc kc, Rsrc vc, Rsrc q, Rsrc knew, Rsrc vnew, Rsrc out,
                                       float *lds, Flow &f, uint64_t *tl, uint32_t wave) {
    using A = Attention<F16>;
    using P = typename A::P;
    float *sacc = lds, *smax = lds + PNW * 128, *ssum = smax + PNW;
    A at{sh, kc, vc, head, pos, wave, -FLT_MAX, 0.0f, {0, 0, 0, 0, 0, 0, 0, 0}};
    P pre[A::ATT_PRE], cur;
#pragma unroll
    for (int i = 0; i < A::ATT_PRE; ++i) {
        pre[i] = P{};
        if (i * plan::ATT_PASS < pos) at.request(pre[i], i * plan::ATT_PASS);
    }
    cur = P{};
    if (A::ATT_PRE * plan::ATT_PASS < pos) at.request(cur, A::ATT_PRE * plan::ATT_PASS);
    // The query: sixteen elements per lane, as soon as all of them are there.  Waves 0 and 1, whose threads merge, ask for
    // the newest key and value in the same rounds: the key is produced at about the same time as the query, the value
    // often is, and what is complete then costs no round trip after the passes.
    float qr[16];
    // (The newest key: lane (i, jj) = (lane % 8, lane / 8 % 4) asks for elements 16 i + 4 jj .. + 3 only, a quarter of what
    // it holds of the query, and the products are summed over 32 lanes.)
    const uint32_t kn_first = plan::att_k_elem(head, lane_id()) + 4u * ((lane_id() >> 3) & 3u);
    float snew_part = 0.0f;
    uint32_t vnw = FLOW_EMPTY;
    bool kv_hole = true;
    {
        const uint32_t first = plan::att_k_elem(head, lane_id());
        uint64_t deadline = 0;
        uint32_t rounds = 0;
        flow_watch(q, head * 128u + 127u, f);
        for (;;) {
            u32x4 v[4], kn = u32x4{FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY};
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = buf_load16<AUX_FLOW>(q, (first + 4u * j) * 4u);
            if (fresh(wave) < 2) {
                kn = buf_load16<AUX_FLOW>(knew, kn_first * 4u);
                vnw = __builtin_amdgcn_raw_buffer_load_b32(vnew, (int)((head * 128u + fresh(wave) * 64u + lane_id()) * 4u), 0, AUX_FLOW);
            }
            const bool hole = flow_empty(v[0]) || flow_empty(v[1]) || flow_empty(v[2]) || flow_empty(v[3]);
            if (!__any(hole) || f.dead) {
#pragma unroll
                for (int j = 0; j < 4; ++j) { qr[4 * j] = __uint_as_float(v[j].x); qr[4 * j + 1] = __uint_as_float(v[j].y); qr[4 * j + 2] = __uint_as_float(v[j].z); qr[4 * j + 3] = __uint_as_float(v[j].w); }
                kv_hole = __any(flow_empty(kn) || vnw == FLOW_EMPTY);
                if (!kv_hole) snew_part = att_new_score<F16>(qr, kn);
                break;
            }
            flow_backoff(f, deadline, rounds);
        }
    }
    stamp(tl, 1, wave);
#pragma unroll
    for (int i = 0; i < A::ATT_PRE; ++i)
        if (i * plan::ATT_PASS < pos) at.consume(pre[i], i * plan::ATT_PASS, qr);
    for (uint32_t tb = A::ATT_PRE * plan::ATT_PASS; tb < pos; tb += plan::ATT_PASS) {
        P nxt = P{};
        if (tb + plan::ATT_PASS < pos) at.request(nxt, tb + plan::ATT_PASS);
        at.consume(cur, tb, qr);
        cur = nxt;
    }
    // This wave's (maximum, sum, outputs): lanes 16 apart hold the same elements of different positions.  Two registers
    // are added across the halves of the wave with one exchange (lanes 0-31 keep the first's sum, lanes 32-63 the
    // second's), then the same across neighbouring rows: row r of s0 / s1 ends with element [0, 2, 1, 3][r] / that + 4.
    at.lsum = wave_total(at.lsum);
    const auto across_halves = [](float a, float b) {
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    };
    const auto across_rows = [](float a, float b) {
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    };
    const float s0 = across_rows(across_halves(at.o[0], at.o[1]), across_halves(at.o[2], at.o[3]));
    const float s1 = across_rows(across_halves(at.o[4], at.o[5]), across_halves(at.o[6], at.o[7]));
    const uint32_t lane = lane_id();
    {
        const uint32_t row = lane >> 4, e = ((row & 1u) << 1) | (row >> 1);
        sacc[wave * 128 + (lane & 15u) * 8 + e] = s0;
        sacc[wave * 128 + (lane & 15u) * 8 + e + 4] = s1;
    }
    if (lane == 0) { smax[wave] = at.m; ssum[wave] = at.lsum; }
    stamp(tl, 2, wave);
    // the newest position: its score like a cached one's (waves 0 and 1, whose threads merge), its value per element
    float snew = 0.0f, vn = 0.0f;
    if (wave < 2) {
        uint64_t deadline = 0;
        uint32_t rounds = 0;
        while (kv_hole) {                                         // (not complete in the round that brought the query)
            const u32x4 kn = buf_load16<AUX_FLOW>(knew, kn_first * 4u);
            vnw = __builtin_amdgcn_raw_buffer_load_b32(vnew, (int)((head * 128u + wave * 64u + lane) * 4u), 0, AUX_FLOW);
            kv_hole = __any(flow_empty(kn) || vnw == FLOW_EMPTY) && !f.dead;
            if (kv_hole) flow_backoff(f, deadline, rounds);
            else snew_part = att_new_score<F16>(qr, kn);
        }
        using C = attn::KV<F16>;                                // (what the cache row holds: rounded to its element type)
        float part = mq::sum8(snew_part);                        // over i, then over jj: the two half rows, then the neighbouring row
        part += mq::dpp<mq::DPP_MIRROR>(part);
        {
            const auto rr = __builtin_amdgcn_permlane16_swap(__float_as_uint(part), __float_as_uint(part), false, false);   // [row 0, row 0, row 2, row 2], [row 1, row 1, row 3, row 3]
            part = __uint_as_float(rr[0]) + __uint_as_float(rr[1]);
        }
        snew = part / sqrtf(128.0f);
        vn = C::round(__uint_as_float(vnw));
    }
    lds_barrier();
    if (wave < 2) {
        // Lane i of every row of 16 takes wave i's maximum and sum: one exponential per lane instead of sixteen per
        // thread; the factors then reach the threads as scalar operands.
        const uint32_t e = wave * 64u + lane;
        const float mw = smax[lane & 15u];
        float M = fmaxf(mw, mq::dpp<mq::DPP_XOR1>(mw));
        M = fmaxf(M, mq::dpp<mq::DPP_XOR2>(M)); M = fmaxf(M, mq::dpp<mq::DPP_HALF_MIRROR>(M)); M = fmaxf(M, mq::dpp<mq::DPP_MIRROR>(M));
        M = fmaxf(M, snew);
        const float fw = expf(mw - M);                          // a wave that saw no position has sum 0 and outputs 0
        float lw = ssum[lane & 15u] * fw;
        lw = mq::sum8(lw);
        lw += mq::dpp<mq::DPP_MIRROR>(lw);
        const float fn = expf(snew - M);
        float r = vn * fn;
        const float l = lw + fn;
        const int fb = __builtin_bit_cast(int, fw);
#pragma unroll
        for (int w = 0; w < PNW; ++w) r = fmaf(sacc[w * 128 + e], __builtin_bit_cast(float, __builtin_amdgcn_readlane(fb, w)), r);
        flow_put(out, head * 128u + e, r / l);
    }
}

__device__ __forceinline__ plan::Shape shape_of(const PersistentParams &p) {
    return plan::Shape{p.dim, p.hidden, p.n_heads, p.n_layers, p.vocab, p.seq_len, gridDim.x, p.qkv_units, p.gu_rows, p.rope_variant == SLAI_ROPE_NEOX ? 1u : 0u};
}

// A long context (plan::att_ahead): the head's attention walks the cached rows beyond the ones it asked for ahead at the
// rate one compute unit reads memory.  The seven workgroups of the head's units sit on the same die and wait for the
// attention's result anyway: their tile waves touch one word of every line of those rows, so that the attention finds
// them in the die's L2.
__device__ __forceinline__ void touch_far_rows(const plan::Shape &sh, uint32_t b, uint32_t pos, bool f16, uint32_t tile_waves, Rsrc kc, Rsrc vc, uint32_t wave_) {
    const uint32_t wave = fresh(wave_), n = plan::touch_count(pos, f16);
    if (wave >= tile_waves || n == 0) return;
    const uint32_t head = plan::qkv_head(sh, b), t = (b >> 3) % sh.qkv_units;
    uint32_t any = 0;
    for (uint32_t w = plan::touch_first(t, tile_waves, wave, lane_id()); w < n; w += plan::touch_stride(sh, tile_waves)) {
        const int off = (int)plan::touch_byte(sh, w, head, f16);
        any |= plan::touch_is_value(w, f16) ? __builtin_amdgcn_raw_buffer_load_b32(vc, off, 0, AUX_PLAIN) : __builtin_amdgcn_raw_buffer_load_b32(kc, off, 0, AUX_PLAIN);
    }
    asm volatile("" : : "v"(any));                                  // (the words are not used: the requests are the point)
}

// ---- the kernel ------------------------------------------------------------------------------------------------------------
// Workgroup roles: resident_plan.h (plan::qkv_unit, attention_head, gu_unit, proj_tiles, out_tiles).  The body exists
// twice, for the workgroups that run a head's attention in the first phase of a layer (ATTN) and for those that multiply
// a q / k / v unit there (or nothing): the attention needs nearly all registers, and only a body of its own shows the
// compiler that no unit requested ahead is ever alive across it.
template <bool F16, bool ATTN, bool FAR>
__device__ __forceinline__ void decode_token(const PersistentParams &p, float *smem, LdsWord *arrived, float (&rope_cs)[2][64], uint32_t (&layer_words)[2][sizeof(PersistentLayer) / 4],
                                             const uint32_t wave) {
    constexpr int LWORDS = sizeof(PersistentLayer) / 4;
    // Two sets of partial[2][16][64] | red[16], taken in turn by the phases of this workgroup: a wave that is done with a
    // phase goes on to the next one (there is one barrier per phase: before the reduction of a 64-row-unit phase, after
    // that of a 16-row-tile phase) while wave 0 may still be reducing the one before, but it cannot get further ahead than that.
    float *const lds_sets = smem;
    char *const lds = reinterpret_cast<char *>(smem);
#define PHASE_PARTIAL (lds_sets + plan::lds_set(phase & 1u) + plan::lds_partial())
#define PHASE_RED (lds_sets + plan::lds_set(phase & 1u) + plan::lds_red())
    const uint32_t b = blockIdx.x;
    Flow f{p.abort_flag, false};
    const plan::Shape sh = shape_of(p);
    const uint32_t dim = p.dim, hid = p.hidden, nh = p.n_heads;
    const uint32_t ncb = dim / 256, ncb_h = hid / 256, ng_o = ncb / 4, ng_d = (ncb_h + 3) / 4;
    float *slot = p.slots + plan::slot_of(sh, b);
    // time stamps: 16 per layer (4 per phase: entered, input there, multiplied, reduced), then 4 for the output matrix and the end
    uint64_t *trace = p.trace ? p.trace + plan::trace_row(sh, b) : nullptr;
    uint32_t phase = 0;                                            // phases this workgroup has run: parity picks the LDS set
    // Every workgroup has a role in every phase (plan::shape_ok: the grid is exactly the 16-row tiles of the projections
    // = seven q / k / v units and one attention per head = the units of gate / up), so the request for the next phase's
    // weights always has a place: right after the multiply of the phase before it.
    const plan::RowUnit qkv_u = ATTN ? plan::run_unit(0u, 0u, 1u) : plan::qkv_unit(sh, b);
    const plan::RowUnit gu_u = plan::gu_unit(sh, b);
    const uint32_t ntiles_out = plan::out_tiles(sh);
    const DevBuf wout = dev_buf(p.wout);
    const plan::Tiles16 wo_t = plan::wo_tiles(sh, b), down_t = plan::down_tiles(sh, b);

    const uint32_t pos = *p.pos_ptr;
    // The rotation of this lane's row of a q or k unit depends on the position only: cosine and sine are computed once
    // (rope.slang:36-39: the angle depends on (2 * i) mod head_size for both pairings; the frequencies come from a table
    // built once with the same powf) and kept in LDS, where reading them waits for no weights.
    if constexpr (!ATTN) {
        if (wave == 0 && qkv_u.seg != 0 && p.rope_variant >= 0) {
            const uint32_t lane = lane_id(), e = plan::unit_row(qkv_u, lane) & 127u;
            const uint32_t i = p.rope_variant == SLAI_ROPE_NEOX ? (e & 63u) : (e >> 1);
            const float theta = p.rope_theta ? p.rope_theta[i] : powf(p.rope_base, -(float)((2 * i) % 128u) / 128.0f);
            float sn, c;
            sincosf((float)pos * theta, &sn, &c);
            rope_cs[0][lane] = c; rope_cs[1][lane] = sn;
        }
    }

    Unit unit;                                                     // the weights requested ahead for this workgroup's next phase
    Req req;
    int unit_type = 0;                                             // its block format
    const auto qkv_matrix = [&](const uint32_t *lw) { return qkv_u.seg == 0 ? LAYER_BUF(lw, wv) : (qkv_u.seg == 1 ? LAYER_BUF(lw, wk) : LAYER_BUF(lw, wq)); };
    // Which weights a wave asks for next (a wave without a part in a 16-row-tile phase gets to the request after it at once).
    const auto ask_wo = [&](const uint32_t *lw) { const DevBuf W = LAYER_BUF(lw, wo); request16(unit, req, W, wo_t, ng_o, wave); unit_type = W.type; };
    const auto ask_gate_up = [&](const uint32_t *lw) { const DevBuf W = LAYER_BUF(lw, wgate); request64<true>(unit, req, W, LAYER_BUF(lw, wup), gu_u, ncb, wave); unit_type = W.type; };
    const auto ask_down = [&](const uint32_t *lw) { const DevBuf W = LAYER_BUF(lw, wdown); request16(unit, req, W, down_t, ng_d, wave); unit_type = W.type; };
    // what this workgroup multiplies after a layer: its q / k / v unit of the next one, or its first tile of the output matrix
    const auto ask_next = [&](const uint32_t *lw_next, bool last) {
        if (last) {
            if (b < ntiles_out) request64<false>(unit, req, wout, wout, plan::run_unit(0u, b * 64u, plan::umin(64u, p.vocab - b * 64u)), ncb, wave);
            unit_type = wout.type;
        } else if constexpr (!ATTN) {
            const DevBuf W = qkv_matrix(lw_next);
            request64<false>(unit, req, W, W, qkv_u, ncb, wave);
            unit_type = W.type;
        }
    };
    if constexpr (!ATTN) ask_next(layer_words[0], false);

    for (uint32_t l = 0; l < p.n_layers; ++l) {
        // this layer's description comes out of LDS entry by entry, as wave-uniform values, where it is used; the next
        // one's is requested now and parked in LDS after the first phase
        const uint32_t *lw = layer_words[l & 1u];
        const bool last = l + 1 == p.n_layers;
        uint32_t next_word = 0;
        if (wave == 0 && lane_id() < LWORDS && !last) next_word = reinterpret_cast<const uint32_t *>(p.layers + l + 1)[lane_id()];
        // Parked once wave 0 has waited for its memory requests anyway.  Nobody reads the slot it goes to any more (its
        // last reader was the gate / up phase of the layer before this one, two barriers ago), and a phase barrier lies
        // between this and its first reader.
        const auto park_next_layer = [&]() {
            if (wave == 0 && lane_id() < LWORDS && !last) layer_words[(l + 1) & 1u][lane_id()] = next_word;
        };
        uint64_t *tl = trace ? trace + 16 * l : nullptr;
        // the hand-off vectors of this layer, each behind a descriptor of its own size
        const Rsrc xa = make_rsrc(p.flow + plan::flow_xa(sh, l), dim * 4u), xb = make_rsrc(p.flow + plan::flow_xb(sh, l), dim * 4u);
        const Rsrc xm = make_rsrc(p.flow + plan::flow_xm(sh, l), dim * 4u), hb = make_rsrc(p.flow + plan::flow_hb(sh, l), hid * 4u);
        const Rsrc xnext = make_rsrc(p.flow + plan::flow_xa(sh, l + 1), dim * 4u);
        // ---- q / k / v, or the attention ------------------------------------------------------------------------------
        if constexpr (!ATTN) {
            const TileIn in{l == 0 ? make_rsrc(p.x, dim * 4u) : xa, l != 0, LAYER_BUF(lw, attn_norm).rs, dim, p.eps};
            stamp(tl, 0, wave);
            // the bias of this lane's row (zero from an empty descriptor when the model has none): asked for now, behind
            // this phase's weights -- after the next request it would wait for the next phase's
            const uint32_t row = plan::unit_row(qkv_u, lane_id());
            const DevBuf bias = qkv_u.seg == 0 ? LAYER_BUF(lw, bv) : (qkv_u.seg == 1 ? LAYER_BUF(lw, bk) : LAYER_BUF(lw, bq));
            float bias_v = 0.0f;
            if (fresh(wave) == 0) bias_v = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(bias.rs, (int)(row * 4u), 0, AUX_PLAIN));
            mult64_any<false>(unit_type, unit, req, ncb, in, true, slot, lds, PHASE_PARTIAL, PHASE_RED, f, tl, wave);
            park_next_layer();
            ask_wo(lw);
            const float o = finish64<false>(ncb, in, PHASE_PARTIAL, PHASE_RED, tl, wave);
            if (fresh(wave) == 0) {
                // RoPE (rope.slang:27-84) with the partner of the pair in a neighbouring lane, the row into the cache for the
                // tokens to come, and the value itself to this token's attention.  Stores only: none of this waits for the
                // weights just requested.
                const uint32_t lane = lane_id();
                float val = o + bias_v;
                if (qkv_u.seg != 0 && p.rope_variant >= 0) {
                    const bool neox = p.rope_variant == SLAI_ROPE_NEOX;
                    const float other = lane_xor(val, neox ? 32 : 1);
                    const bool first = neox ? lane < 32u : (lane & 1u) == 0;
                    const float c = rope_cs[0][lane], sn = rope_cs[1][lane];
                    val = first ? c * val - sn * other : sn * other + c * val;
                }
                if (lane < qkv_u.nrows) {
                    flow_put(make_rsrc(p.flow + plan::flow_qkv(sh, l, qkv_u.seg), dim * 4u), row, val);
                    if (qkv_u.seg != 2) {
                        const DevBuf cache = qkv_u.seg == 0 ? LAYER_BUF(lw, vcache) : LAYER_BUF(lw, kcache);
                        const uint32_t at = plan::cache_elem(sh, pos, row);
                        if constexpr (F16) __builtin_amdgcn_raw_buffer_store_b16(attn::f2h(val), cache.rs, (int)(at * 2u), 0, AUX_PLAIN);
                        else __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), cache.rs, (int)(at * 4u), 0, AUX_PLAIN);
                    }
                }
            }
            ++phase;
        } else {
            const uint32_t h = plan::attention_head(sh, b);
            stamp(tl, 0, wave);
            park_next_layer();
            attend<F16>(sh, h, pos, LAYER_BUF(lw, kcache).rs, LAYER_BUF(lw, vcache).rs, make_rsrc(p.flow + plan::flow_qkv(sh, l, 2), dim * 4u),
                        make_rsrc(p.flow + plan::flow_qkv(sh, l, 1), dim * 4u), make_rsrc(p.flow + plan::flow_qkv(sh, l, 0), dim * 4u), xb, PHASE_PARTIAL, f, tl, wave);
            stamp(tl, 3, wave);
            ++phase;
            // (only now: the attention needs the registers; these workgroups take no tile of the output projection)
            ask_gate_up(lw);
        }
        // ---- attention output projection into the residual (two tiles in each workgroup that multiplied q or k; the others pass) ---
        if constexpr (!ATTN) {
            uint64_t *tp = tl ? tl + 4 : nullptr;
            float residual;
            stamp(tp, 0, wave);
            // A long context: the head's attention walks the cached rows beyond the ones it asked for ahead at the rate one
            // compute unit reads memory.  The seven workgroups of the head's units sit on the same die and wait here anyway:
            // their tile waves touch one word of every line of those rows, so that the attention finds them in the die's L2.
            static_assert((Attention<F16>::ATT_PRE + 1) * plan::ATT_PASS == plan::att_ahead(F16), "what the attention requests before the query");
            if constexpr (FAR) {
                // (only in the kernel the host launches for long contexts: the short ones, which the throughput is quoted on,
                // should not carry this code and its registers)
                const DevBuf kc = LAYER_BUF(lw, kcache), vc = LAYER_BUF(lw, vcache);
                touch_far_rows(sh, b, pos, F16, ng_o, kc.rs, vc.rs, wave);
            }
            mult16_any(unit_type, unit, wo_t, ncb, ng_o, xb, l == 0 ? make_rsrc(p.x, dim * 4u) : xa, l != 0, residual, lds, PHASE_PARTIAL, arrived, f, tp, wave);
            const float o = finish16(wo_t, ng_o, PHASE_PARTIAL, arrived, f, tp, wave);               // (wave 0 only; the others go straight on)
            const uint32_t tid = wave * 64u + lane_id();
            if (tid < 16u * wo_t.n) flow_put(xm, plan::tiles16_row(wo_t, tid), residual + o);     // transformer.rs:352-355
            ask_gate_up(lw);                                        // (the waves without a part in the tiles: at once)
            lds_barrier();
            ++phase;
        }
        // ---- RMSNorm + gate / up + SiLU ---------------------------------------------------------------------------------
        {
            uint64_t *tp = tl ? tl + 8 : nullptr;
            const TileIn in{xm, true, LAYER_BUF(lw, ffn_norm).rs, dim, p.eps};
            stamp(tp, 0, wave);
            mult64_any<true>(unit_type, unit, req, ncb, in, true, slot, lds, PHASE_PARTIAL, PHASE_RED, f, tp, wave);
            ask_down(lw);
            const float o = finish64<true>(ncb, in, PHASE_PARTIAL, PHASE_RED, tp, wave);
            const uint32_t tid = wave * 64u + lane_id();
            if (tid < gu_u.nrows) flow_put(hb, gu_u.row0 + tid, o);
            ++phase;
        }
        // ---- down projection into the residual ----------------------------------------------------------------------------
        {
            uint64_t *tp = tl ? tl + 12 : nullptr;
            float residual;
            stamp(tp, 0, wave);
            residual = 0.0f;
            mult16_any(unit_type, unit, down_t, ncb_h, ng_d, hb, xm, true, residual, lds, PHASE_PARTIAL, arrived, f, tp, wave);
            const float o = finish16(down_t, ng_d, PHASE_PARTIAL, arrived, f, tp, wave);
            const uint32_t tid = wave * 64u + lane_id();
            if (tid < 16u * down_t.n) flow_put(xnext, plan::tiles16_row(down_t, tid), residual + o);    // transformer.rs:362-365
            ask_next(layer_words[(l + 1) & 1u], last);
            lds_barrier();
            ++phase;
        }
    }
    // ---- final RMSNorm and the output matrix: tiles b, b + grid, ... -------------------------------------------------------
    {
        const TileIn in{make_rsrc(p.flow + plan::flow_xa(sh, p.n_layers), dim * 4u), true, dev_buf(p.out_norm).rs, dim, p.eps};
        uint64_t *to = trace ? trace + 16 * p.n_layers : nullptr;
        bool first = true;
        // (the input is staged once: its sums of squares stay in this LDS set, and a barrier separates the tiles)
        for (uint32_t tile = b; tile < ntiles_out; tile += gridDim.x) {
            const plan::RowUnit u = plan::run_unit(0u, tile * 64u, plan::umin(64u, p.vocab - tile * 64u));
            uint64_t *tp = first ? to : nullptr;
            stamp(tp, 0, wave);
            mult64_any<false>(wout.type, unit, req, ncb, in, first, slot, lds, PHASE_PARTIAL, PHASE_RED, f, tp, wave);
            const uint32_t next = tile + gridDim.x;
            if (next < ntiles_out) request64<false>(unit, req, wout, wout, plan::run_unit(0u, next * 64u, plan::umin(64u, p.vocab - next * 64u)), ncb, wave);
            const float o = finish64<false>(ncb, in, PHASE_PARTIAL, PHASE_RED, tp, wave);
            const uint32_t tid = wave * 64u + lane_id();
            if (tid < u.nrows) p.logits[u.row0 + tid] = o;
            first = false;
            lds_barrier();                                         // partial[] is reused by the next tile
        }
        stamp(to, 4, wave);
    }
}

// The description of the current layer and of the next one is parked in LDS.  Read from memory at the moment of use, its
// lines (which the weight stream has long pushed out of L2) would cost a round trip to memory each, one after the other.
// FAR: the variant for positions beyond plan::att_ahead (touch_far_rows); the host picks it per token.
template <bool F16, bool FAR>
__global__ void __launch_bounds__(PNT) llama_decode_persistent_kernel(const PersistentParams p) {
    extern __shared__ __align__(16) float smem[];
    __shared__ float rope_cs[2][64];                               // cosine | sine of the rotation of wave 0's rows (q and k units)
    constexpr int LWORDS = sizeof(PersistentLayer) / 4;
    static_assert(LWORDS <= 64 && sizeof(PersistentLayer) == 14 * sizeof(ResidentBuf), "one thread per word; fourteen entries");
    __shared__ uint32_t layer_words[2][LWORDS];
    __shared__ uint32_t arrived_word;                              // the waves of a 16-row-tile phase count themselves in here (finish16)
    touch_kernel_arguments<sizeof(PersistentParams)>();
    // A launch after one in which a reader gave up does nothing: the host has not looked yet (it queues many tokens), and
    // every further token would only wait out the same time limits.
    if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
    if (threadIdx.x < LWORDS) layer_words[0][threadIdx.x] = reinterpret_cast<const uint32_t *>(p.layers)[threadIdx.x];
    if (threadIdx.x == 0) arrived_word = 0u;
    if (threadIdx.x < plan::MQ_ZERO_BYTES / 4) reinterpret_cast<uint32_t *>(smem)[plan::lds_mq_zero() / 4 + threadIdx.x] = 0u;   // the zeros of mfma_q4k.h
    __syncthreads();
    const plan::Shape sh = shape_of(p);
    const uint32_t wave = uniform_word(threadIdx.x >> 6);
    LdsWord *arrived = (LdsWord *)&arrived_word;
    if (plan::is_attention_workgroup(sh, blockIdx.x)) decode_token<F16, true, false>(p, smem, arrived, rope_cs, layer_words, wave);
    else decode_token<F16, false, FAR>(p, smem, arrived, rope_cs, layer_words, wave);
}

#undef PHASE_PARTIAL
#undef PHASE_RED

// Fills the hand-off buffers of a launch with FLOW_EMPTY (16 bytes per thread and step).
__global__ void flow_fill_kernel(u32x4 *buf, size_t n16) {
    const u32x4 e = {FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) buf[i] = e;
}

}  // namespace

size_t persistent_smem_bytes(const PersistentParams &p) {
    const plan::Shape s{p.dim, p.hidden, p.n_heads, p.n_layers, p.vocab, p.seq_len, 0, p.qkv_units, p.gu_rows, 0};
    return (size_t)plan::lds_floats(s) * sizeof(float);
}

// How many workgroups of the kernel the device keeps resident at once (0: it cannot run at all).
hipError_t persistent_capacity(const PersistentParams &p, int device, uint32_t *resident) {
    *resident = 0;
    const size_t smem = persistent_smem_bytes(p);
    const void *fn = p.kv_f16 ? (const void *)llama_decode_persistent_kernel<true, false> : (const void *)llama_decode_persistent_kernel<false, false>;
    const void *far = p.kv_f16 ? (const void *)llama_decode_persistent_kernel<true, true> : (const void *)llama_decode_persistent_kernel<false, true>;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e == hipSuccess) e = hipFuncSetAttribute(far, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
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

uint32_t resident_far_from(bool kv_f16) { return plan::att_ahead(kv_f16); }

hipError_t launch_flow_fill(hipStream_t s, void *buf, size_t bytes) {
    if (bytes % 16 || (uintptr_t)buf % 16) return hipErrorInvalidValue;
    flow_fill_kernel<<<64, 1024, 0, s>>>((u32x4 *)buf, bytes / 16);
    return hipGetLastError();
}

hipError_t launch_decode_persistent(hipStream_t s, const PersistentParams &p, uint32_t grid, bool far) {
    const plan::Shape sh{p.dim, p.hidden, p.n_heads, p.n_layers, p.vocab, p.seq_len, grid, p.qkv_units, p.gu_rows};
    if (!plan::shape_ok(sh)) return hipErrorInvalidValue;          // the index arithmetic of the kernel assumes these
    const size_t smem = persistent_smem_bytes(p);
    if (p.kv_f16) { if (far) llama_decode_persistent_kernel<true, true><<<grid, PNT, smem, s>>>(p); else llama_decode_persistent_kernel<true, false><<<grid, PNT, smem, s>>>(p); }
    else { if (far) llama_decode_persistent_kernel<false, true><<<grid, PNT, smem, s>>>(p); else llama_decode_persistent_kernel<false, false><<<grid, PNT, smem, s>>>(p); }
    return hipGetLastError();
}

}  // namespace slai
