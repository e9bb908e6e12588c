// Dequantisation-fused GEMV over 64-row tiles of the tiled weight layout (quant_tiled.h, ROWS = 64, KQ = 1)
// with wave-uniform activations, gfx950.
//
// Same contract as kernels_gemv.hip / kernels_gemv_tiled.hip (the reference's gemv_quant_*.slang shaders
// dispatched by crates/slai/src/ops/gemv_quant.rs:206-312).  A lane owns one row of a 64-row tile and a
// wave consumes one 256-column super-block at a time, so all 64 lanes multiply by the SAME activation:
// it is a scalar register operand of a plain v_fmac_f32 (full rate; a DPP-broadcast operand runs at half
// rate on this target).  The activations therefore have to be readable through the scalar data cache:
// the workgroup writes its normalised copy (and the per-16 sums the block formats need for their offset
// terms) to a private slot of a scratch buffer with ordinary vector stores, waits for them, and every
// wave then streams its 256 activations with s_load_dwordx8/16.  The slot is written before it is first
// read in a dispatch and the scalar cache starts every dispatch empty, so no cache maintenance is needed.
// When the kernel that produced the input already left such a copy (`prepared`: weighted activations followed
// by their sums of 16, see GEMV_EMIT in kernels_gemv_tiled.hip) the waves read that directly, nothing is staged
// and the only work left of the RMSNorm is the sum of squares, whose scale is applied in the epilogue.
//
// One workgroup = one tile = 64 complete output rows; wave w owns super-blocks w, w+NW, ...; partial
// sums meet in LDS once.  Segments of one launch may differ in block format (Q4_K q/k with a Q6_K v).
#include "common.h"
#include "attention_fast.h"
#include "device_util.h"
#include "gemv_operands.h"
#include "quant_tiled.h"

namespace slai {
namespace {

using namespace lanes;

// Stages of a unit requested ahead of the one being multiplied.  One is the measured optimum when every wave of every
// workgroup streams a unit of its own: with 2, 4 and 8 the gate/up launch took 12.6, 13.6 and 14.3 us against 12.3 (all
// 2752 units of the matrix are then requested at once, in no order the memory channels can follow).
constexpr int ROWTILE_LD = 1;

// The body for one block format.  `partial` = [DUAL?2:1][NW][64] floats, `red` = [NW] floats.
template <int T, bool DUAL, bool PREP>
__device__ __forceinline__ void tile_body(const GemvRowtileParams &p, const GemvRowtileSeg &seg, uint32_t tile, float *partial, float *red) {
    using F = Tiled<T>;
    const int tid = threadIdx.x, lane = tid & 63, NT = blockDim.x, NW = NT >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t unit_bytes = F::PT * 1024 + (F::TAIL ? 128 : 0);

    // ---- requests.  Loads retire in issue order.  With prepared activations nothing before the epilogue needs x, so
    // the weights go first; otherwise x is needed at once (the workgroup stages its copy) and goes first. ----------
    constexpr int XMAX = 4;                                   // float4 per thread: ncols <= 16 * blockDim
    float4 xv[XMAX], wv[XMAX];
    const bool norm = p.prologue == PRO_RMSNORM;
    auto request_x = [&]() {
#pragma unroll
        for (int j = 0; j < XMAX; ++j) {
            // every thread loads (clamped to the last float4) so that the requests are branch-free; `live` says whether
            // the value counts
            const uint32_t i = min((uint32_t)(j * NT + tid) * 4, p.ncols - 4);
            xv[j] = *(const float4 *)(p.x + i);
            if (!PREP) wv[j] = norm ? *(const float4 *)(p.norm_w + i) : make_float4(1.0f, 1.0f, 1.0f, 1.0f);
        }
    };
    typename F::Data d, e;
    uint16_t dt = 0, et = 0;
    uint32_t cb = wave;
    constexpr int NM = DUAL ? 2 : 1;
    UnitLoader<T, NM, ROWTILE_LD> ld;
    auto point = [&]() {                                      // aim the loader at super-block cb of this tile
        const size_t off = ((size_t)tile * p.ncb + cb) * unit_bytes;
        ld.unit[0] = seg.W + off + lane * 16; ld.tailp[0] = seg.W + off + (size_t)F::PT * 1024 + lane * 2; ld.d[0] = &d; ld.t[0] = &dt;
        if constexpr (DUAL) { ld.unit[1] = seg.W2 + off + lane * 16; ld.tailp[1] = seg.W2 + off + (size_t)F::PT * 1024 + lane * 2; ld.d[1] = &e; ld.t[1] = &et; }
    };
    auto request_w = [&]() {                                  // the pieces the first stages need; the rest follow inside the dot product
        if (cb < p.ncb) { point(); F::lead(ld); }
    };
    if constexpr (PREP) { request_w(); if (norm) request_x(); }
    else { request_x(); request_w(); }
    float old = 0.0f, bias = 0.0f;
    const uint32_t row = tile * 64 + tid;
    if (tid < 64 && row < seg.nrows) {
        if (seg.flags & GEMV_ACCUM) old = seg.out[row];
        if (seg.flags & GEMV_BIAS) bias = seg.bias[row];
    }

    float ss = 0.0f, scale = 1.0f;
    cfloat *xs;
    if constexpr (PREP) {
        xs = (cfloat *)(uintptr_t)p.prepared;
        // The copy was written by another kernel, possibly on another die: the first touch of each of its cache lines
        // goes to memory.  Touch the 17 lines of this wave's first super-block at once (one word each) so that those
        // misses overlap each other and the weight stream, instead of stalling the stages one after the other.
        if (cb < p.ncb) {
            typedef const uint32_t __attribute__((address_space(4))) cu32;
            cu32 *wx = (cu32 *)(xs + (size_t)cb * 256), *ws = (cu32 *)(xs + p.ncols + (size_t)cb * 16);
            uint32_t warm = ws[0];
#pragma unroll
            for (int i = 0; i < 16; ++i) warm |= wx[16 * i];
            asm volatile("" : : "s"(warm));
        }
    } else {
        // ---- the workgroup's own copy of the (weighted) activations and their sums of 16 ----------------------
        float *slot = p.scratch + (size_t)blockIdx.x * p.scratch_stride;
#pragma unroll
        for (int j = 0; j < XMAX; ++j) {
            const uint32_t i = (uint32_t)(j * NT + tid) * 4;
            if (i < p.ncols) {
                float4 v = xv[j];
                ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss);
                v.x *= wv[j].x; v.y *= wv[j].y; v.z *= wv[j].z; v.w *= wv[j].w;
                *(float4 *)(slot + i) = v;
                float s4 = (v.x + v.y) + (v.z + v.w);
                s4 += __shfl_xor(s4, 1, 64);
                s4 += __shfl_xor(s4, 2, 64);                  // lanes 4q..4q+3 hold 16 consecutive activations
                if ((lane & 3) == 0) slot[p.ncols + (i >> 4)] = s4;
            }
        }
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();  // also waits for this thread's stores (and, unavoidably, its weight loads) to complete
        // The slot is read through the constant address space, whose loads the compiler may move freely; hand it
        // the pointer only now, behind the barrier.
        uint64_t slot_bits = (uint64_t)(uintptr_t)slot;
        asm volatile("" : "+s"(slot_bits) : : "memory");
        xs = (cfloat *)slot_bits;
    }

    if constexpr (PREP) {
        if (norm) {                                           // the sum of squares (for the epilogue), while the first weights travel
#pragma unroll
            for (int j = 0; j < XMAX; ++j) {
                const float4 q = xv[j];
                const float live = (uint32_t)(j * NT + tid) * 4 < p.ncols ? 1.0f : 0.0f;
                ss = fmaf(live * q.x, q.x, ss); ss = fmaf(live * q.y, q.y, ss); ss = fmaf(live * q.z, q.z, ss); ss = fmaf(live * q.w, q.w, ss);
            }
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
        }
    }
    // ---- super-blocks of this wave -------------------------------------------------------------------
    float v = 0.0f, v2 = 0.0f;
    // At most four super-blocks per wave (ncols <= 16384 with 16 waves).  Straight-line code: inside a real loop the
    // compiler's scheduler requests all scalar loads of a super-block at once and runs out of registers.
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        if (cb < p.ncb) {
            ScalarX X{xs + (size_t)cb * 256, xs + p.ncols + (size_t)cb * 16};
            const typename F::Data *dp[NM];
            uint16_t tails[NM];
            float o2[NM];
            dp[0] = &d; tails[0] = dt;
            if constexpr (DUAL) { dp[1] = &e; tails[1] = et; }
            F::template dotn<NM>(dp, tails, X, o2, ld);       // gated pair: both matrices in lockstep, one pass over the activations
            v += o2[0];
            if constexpr (DUAL) v2 += o2[1];
            cb += NW;
            if (it < 3 && cb < p.ncb) { point(); F::lead(ld); }
        }
    }
    partial[wave * 64 + lane] = v;
    if constexpr (DUAL) partial[(NW + wave) * 64 + lane] = v2;
    lds_barrier();
    if (tid < 64 && row < seg.nrows) {                        // epilogue: one thread per output row
        if (p.prologue == PRO_RMSNORM) {
            float t = 0.0f;
            for (int w = 0; w < NW; ++w) t += red[w];
            // rms_norm.slang:60-66 computes (x * scale) * w; here the scale is applied to the finished dot product
            scale = 1.0f / sqrtf(t / (float)p.ncols + p.eps);
        }
        float o = 0.0f;
        for (int w = 0; w < NW; ++w) o += partial[w * 64 + tid];
        o *= scale;
        if constexpr (DUAL) {
            float up = 0.0f;
            for (int w = 0; w < NW; ++w) up += partial[(NW + w) * 64 + tid];
            up *= scale;
            o = up * (o / (1.0f + expf(-o)));                 // silu.slang:8-26
        }
        if (seg.flags & GEMV_BIAS) o += bias;
        if (seg.flags & GEMV_GELU) o = gelu_f(o);
        if (seg.flags & GEMV_ACCUM) o = old + o;
        seg.out[row] = o;
    }
}

// TT = block format of every segment, or 0 when the segments differ (the format then is a per-workgroup switch and
// the kernel needs the registers of its largest case).
template <int TT, bool DUAL, bool PREP>
__global__ void __launch_bounds__(1024) gemv_rowtile_kernel(const GemvRowtileParams p) {
    extern __shared__ float smem[];
    const int NW = blockDim.x >> 6;
    float *partial = smem;
    float *red = smem + (size_t)(DUAL ? 2 : 1) * NW * 64;
    touch_kernel_arguments<sizeof(GemvRowtileParams)>();
    // The segment is picked with selects over statically indexed fields: a dynamically indexed p.seg[s] would be
    // fetched in a second, dependent round trip.
    const uint32_t n0 = p.seg[0].ntiles, n1 = p.seg[1].ntiles;       // unused segments have ntiles = 0
    uint32_t tile = blockIdx.x;
    const int s = tile < n0 ? 0 : (tile - n0 < n1 ? 1 : 2);
    tile -= s == 0 ? 0u : (s == 1 ? n0 : n0 + n1);
    GemvRowtileSeg seg;
    seg.W = s == 0 ? p.seg[0].W : (s == 1 ? p.seg[1].W : p.seg[2].W);
    seg.W2 = s == 0 ? p.seg[0].W2 : (s == 1 ? p.seg[1].W2 : p.seg[2].W2);
    seg.type = s == 0 ? p.seg[0].type : (s == 1 ? p.seg[1].type : p.seg[2].type);
    seg.nrows = s == 0 ? p.seg[0].nrows : (s == 1 ? p.seg[1].nrows : p.seg[2].nrows);
    seg.out = s == 0 ? p.seg[0].out : (s == 1 ? p.seg[1].out : p.seg[2].out);
    seg.bias = s == 0 ? p.seg[0].bias : (s == 1 ? p.seg[1].bias : p.seg[2].bias);
    seg.flags = s == 0 ? p.seg[0].flags : (s == 1 ? p.seg[1].flags : p.seg[2].flags);
    if constexpr (TT != 0) {
        tile_body<TT, DUAL, PREP>(p, seg, tile, partial, red);
    } else {
        switch (seg.type) {                                    // uniform over the workgroup
        case T_Q4_K: tile_body<T_Q4_K, DUAL, PREP>(p, seg, tile, partial, red); break;
        case T_Q6_K: tile_body<T_Q6_K, DUAL, PREP>(p, seg, tile, partial, red); break;
        case T_Q5_K: if constexpr (!DUAL) tile_body<T_Q5_K, false, PREP>(p, seg, tile, partial, red); break;
        default: break;                                        // the launcher sends the other formats to their own kernels
        }
    }
}

// The same tiles for several input vectors (a chunk of prompt tokens; prepared input only).  Workgroup i runs on XCD
// i % 8, and workgroups are dispatched in index order: the bt.n workgroups of one tile get consecutive indices on ONE
// XCD, i = ((tile / 8) * bt.n + b) * 8 + tile % 8, so they run at the same time on neighbouring compute units, the
// first request for a piece of the tile brings it from memory and the others find it in that XCD's L2.
template <int TT, bool DUAL>
__global__ void __launch_bounds__(1024) gemv_rowtile_batch_kernel(const GemvRowtileParams p0, const GemvBatch bt, uint32_t total_tiles) {
    extern __shared__ float smem[];
    const int NW = blockDim.x >> 6;
    float *partial = smem;
    float *red = smem + (size_t)(DUAL ? 2 : 1) * NW * 64;
    touch_kernel_arguments<((sizeof(GemvRowtileParams) + 63) / 64 + 1) * 64>();
    const uint32_t i = blockIdx.x, j = i >> 3, b = j % bt.n;
    uint32_t tile = (j / bt.n) * 8 + (i & 7u);
    if (tile >= total_tiles) return;                             // (uniform) the tile count rounded up to the eight XCDs
    const uint32_t n0 = p0.seg[0].ntiles, n1 = p0.seg[1].ntiles;
    const int s = tile < n0 ? 0 : (tile - n0 < n1 ? 1 : 2);
    tile -= s == 0 ? 0u : (s == 1 ? n0 : n0 + n1);
    GemvRowtileSeg seg;
    seg.W = s == 0 ? p0.seg[0].W : (s == 1 ? p0.seg[1].W : p0.seg[2].W);
    seg.W2 = s == 0 ? p0.seg[0].W2 : (s == 1 ? p0.seg[1].W2 : p0.seg[2].W2);
    seg.type = s == 0 ? p0.seg[0].type : (s == 1 ? p0.seg[1].type : p0.seg[2].type);
    seg.nrows = s == 0 ? p0.seg[0].nrows : (s == 1 ? p0.seg[1].nrows : p0.seg[2].nrows);
    seg.out = s == 0 ? p0.seg[0].out : (s == 1 ? p0.seg[1].out : p0.seg[2].out);
    seg.bias = s == 0 ? p0.seg[0].bias : (s == 1 ? p0.seg[1].bias : p0.seg[2].bias);
    seg.flags = s == 0 ? p0.seg[0].flags : (s == 1 ? p0.seg[1].flags : p0.seg[2].flags);
    seg.out += (size_t)b * (s == 0 ? bt.out_stride[0] : (s == 1 ? bt.out_stride[1] : bt.out_stride[2]));
    GemvRowtileParams p = p0;
    p.x = p0.x + (size_t)b * bt.x_stride;
    p.prepared = p0.prepared + (size_t)b * bt.prepared_stride;
    if constexpr (TT != 0) {
        tile_body<TT, DUAL, true>(p, seg, tile, partial, red);
    } else {
        switch (seg.type) {                                    // uniform over the workgroup
        case T_Q4_K: tile_body<T_Q4_K, DUAL, true>(p, seg, tile, partial, red); break;
        case T_Q6_K: tile_body<T_Q6_K, DUAL, true>(p, seg, tile, partial, red); break;
        case T_Q5_K: if constexpr (!DUAL) tile_body<T_Q5_K, false, true>(p, seg, tile, partial, red); break;
        default: break;
        }
    }
}

// ---- q/k/v projections and attention in ONE launch ----------------------------------------------------------------
// For layers with as many kv heads as q heads, head size 128 and a context served by one workgroup per head.  The six
// 64-row tiles that make up a head's q, k and v (two each; segments in the order v, k, q) go to six workgroups of the
// SAME XCD: workgroup i runs on XCD i % 8, so head h = (i % 8) + 8 * ((i / 8) / 6) takes the workgroups i = (h % 8) +
// 8 * (6 * (h / 8) + t), t = 0..5.  Each writes its 64 results, waits until the stores have reached the XCD's L2
// (s_waitcnt vmcnt(0)) and bumps the head's counter with an atomic that executes in that L2.  The workgroup of the last
// tile (t = 5) then runs the attention of the head: it requests the cache rows first, spins on the counter until all six
// tiles are in, and reads q, k, v from L2.  Its five producers have smaller indices and are therefore dispatched before
// it, so it never waits for a workgroup that has no compute unit.  The spin is bounded: if the counter does not fill
// (it always has) the workgroup sets counters[timeout_slot] and goes on.
constexpr uint32_t HANDOFF_SPIN_LIMIT = 1u << 24;

template <bool F16, bool PREP>
__global__ void __launch_bounds__(1024) qkv_attention_kernel(const GemvRowtileParams p, const AttnLaunch a, uint32_t *counters, uint32_t timeout_slot) {
    extern __shared__ float smem[];
    const int NW = blockDim.x >> 6;
    float *partial = smem;
    float *red = smem + (size_t)NW * 64;
    touch_kernel_arguments<((sizeof(GemvRowtileParams) + 63) / 64 + (sizeof(AttnLaunch) + 63) / 64) * 64>();
    const uint32_t i = blockIdx.x, j = i >> 3, t = j % 6;
    const uint32_t h = (i & 7u) + 8u * (j / 6);
    const int s = (int)(t >> 1);
    const uint32_t tile = 2 * h + (t & 1u);
    GemvRowtileSeg seg;
    seg.W = s == 0 ? p.seg[0].W : (s == 1 ? p.seg[1].W : p.seg[2].W);
    seg.W2 = nullptr;
    seg.type = s == 0 ? p.seg[0].type : (s == 1 ? p.seg[1].type : p.seg[2].type);
    seg.nrows = s == 0 ? p.seg[0].nrows : (s == 1 ? p.seg[1].nrows : p.seg[2].nrows);
    seg.out = s == 0 ? p.seg[0].out : (s == 1 ? p.seg[1].out : p.seg[2].out);
    seg.bias = s == 0 ? p.seg[0].bias : (s == 1 ? p.seg[1].bias : p.seg[2].bias);
    seg.flags = s == 0 ? p.seg[0].flags : (s == 1 ? p.seg[1].flags : p.seg[2].flags);
    switch (seg.type) {                                        // uniform over the workgroup
    case T_Q4_K: tile_body<T_Q4_K, false, PREP>(p, seg, tile, partial, red); break;
    case T_Q6_K: tile_body<T_Q6_K, false, PREP>(p, seg, tile, partial, red); break;
    case T_Q5_K: tile_body<T_Q5_K, false, PREP>(p, seg, tile, partial, red); break;
    default: break;
    }
    uint32_t *counter = counters + (size_t)h * 32;             // one 128-byte line per head
    if (threadIdx.x < 64) {                                    // the wave that wrote the tile's results
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (threadIdx.x == 0) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (t != 5) return;
    attn::attn_fast_body<F16, 1024, 128, true, true, 8>(a, h, 0u, threadIdx.x, [&]() {
        if (threadIdx.x == 0) {
            uint32_t seen = 0, spins = 0;
            do {
                // a read-modify-write that returns the value: it executes in the L2 (the compiler would turn an
                // atomic add of 0 into a load, which may be served by this compute unit's own cache for ever)
                const uint32_t zero = 0;
                asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=&v"(seen) : "v"(counter), "v"(zero) : "memory");
                ++spins;
            } while (seen < 6u && spins < HANDOFF_SPIN_LIMIT);
            if (seen < 6u) counters[timeout_slot] = 1u;
            *counter = 0u;                                     // for the next launch; nobody else touches it any more
        }
        __syncthreads();
        asm volatile("" ::: "memory");
    });
}

template <int TT, bool DUAL>
hipError_t go(const GemvRowtileParams &p, uint32_t tiles, int NT, size_t smem, hipStream_t s, const GemvBatch *bt) {
    if (bt && bt->n > 1) {
        if (!p.prepared) return hipErrorInvalidValue;
        gemv_rowtile_batch_kernel<TT, DUAL><<<(tiles + 7) / 8 * 8 * bt->n, NT, smem, s>>>(p, *bt, tiles);
        return hipGetLastError();
    }
    if (p.prepared) gemv_rowtile_kernel<TT, DUAL, true><<<tiles, NT, smem, s>>>(p);
    else gemv_rowtile_kernel<TT, DUAL, false><<<tiles, NT, smem, s>>>(p);
    return hipGetLastError();
}

}  // namespace

size_t gemv_rowtile_scratch_floats(const GemvRowtileParams &p) {
    uint32_t tiles = 0;
    for (int i = 0; i < p.nseg; ++i) tiles += (p.seg[i].nrows + 63) / 64;
    return (size_t)tiles * (p.ncols + p.ncols / 16);
}

hipError_t launch_gemv_rowtile(slai_ctx *ctx, GemvRowtileParams p, const GemvBatch *bt) {
    if (p.ncb == 0 || p.ncols != p.ncb * 256) return hipErrorInvalidValue;
    int NW = (int)(p.ncb < 16 ? p.ncb : 16);
    if (p.ncols > 16u * 64u * NW) NW = (int)((p.ncols + 1023) / 1024);       // 4 float4 of x per thread at most
    if (NW > 16) return hipErrorInvalidValue;
    bool dual = false;
    uint32_t tiles = 0;
    for (int i = 0; i < p.nseg; ++i) {
        const int t = p.seg[i].type;
        if (!tiled_supported(t)) return hipErrorInvalidValue;
        p.seg[i].ntiles = (p.seg[i].nrows + 63) / 64;
        tiles += p.seg[i].ntiles;
        if (p.seg[i].flags & GEMV_SILU_GATE) dual = true;
    }
    for (int i = 0; i < p.nseg; ++i)
        if (dual != ((p.seg[i].flags & GEMV_SILU_GATE) != 0)) return hipErrorInvalidValue;
    p.scratch_stride = p.ncols + p.ncols / 16;
    const size_t smem = ((size_t)(dual ? 2 : 1) * NW * 64 + NW) * sizeof(float);
    int tt = p.seg[0].type;
    for (int i = 1; i < p.nseg; ++i)
        if (p.seg[i].type != tt) tt = 0;
    if (tt == 0) {
        for (int i = 0; i < p.nseg; ++i)
            if (p.seg[i].type == T_Q8_0 || p.seg[i].type == T_Q4_0 || (dual && p.seg[i].type == T_Q5_K))
                return hipErrorInvalidValue;                       // mixed launches: the K-quants only
    }
    const int NT = NW * 64;
    hipStream_t st = ctx->stream;
    switch (tt) {
    case T_Q4_K: return dual ? go<T_Q4_K, true>(p, tiles, NT, smem, st, bt) : go<T_Q4_K, false>(p, tiles, NT, smem, st, bt);
    case T_Q6_K: return dual ? go<T_Q6_K, true>(p, tiles, NT, smem, st, bt) : go<T_Q6_K, false>(p, tiles, NT, smem, st, bt);
    case T_Q8_0: return dual ? go<T_Q8_0, true>(p, tiles, NT, smem, st, bt) : go<T_Q8_0, false>(p, tiles, NT, smem, st, bt);
    case T_Q4_0: return dual ? go<T_Q4_0, true>(p, tiles, NT, smem, st, bt) : go<T_Q4_0, false>(p, tiles, NT, smem, st, bt);
    case T_Q5_K: return dual ? go<T_Q5_K, true>(p, tiles, NT, smem, st, bt) : go<T_Q5_K, false>(p, tiles, NT, smem, st, bt);
    default: return dual ? go<0, true>(p, tiles, NT, smem, st, bt) : go<0, false>(p, tiles, NT, smem, st, bt);
    }
}

hipError_t launch_qkv_attention(slai_ctx *ctx, GemvRowtileParams p, const AttnLaunch &a) {
    if (p.nseg != 3 || p.ncb == 0 || p.ncb > 16 || p.ncols != p.ncb * 256) return hipErrorInvalidValue;
    if (a.head_size != 128 || a.kv_mul != 1 || a.n_splits != 1 || a.n_heads % 8 || a.kv_dim % 8 || !a.knew || !a.vnew || !ctx->handoff_counters ||
        a.n_heads > ctx->handoff_heads)
        return hipErrorInvalidValue;
    for (int i = 0; i < 3; ++i) {
        const int t = p.seg[i].type;
        if ((t != T_Q4_K && t != T_Q6_K && t != T_Q5_K) || p.seg[i].nrows != a.n_heads * 128 || p.seg[i].W2 || (p.seg[i].flags & GEMV_SILU_GATE))
            return hipErrorInvalidValue;
        p.seg[i].ntiles = p.seg[i].nrows / 64;
    }
    // sixteen waves, one per super-block; the attention part uses all of them, eight lanes per position so that it fits
    // the 128 registers per lane a workgroup of this size leaves
    const int NW = 16;
    if (p.ncb != 16) return hipErrorInvalidValue;               // (other widths take the separate kernels)
    p.scratch_stride = p.ncols + p.ncols / 16;
    const size_t smem = ((size_t)NW * 64 + NW) * sizeof(float);
    const uint32_t grid = a.n_heads * 6;
    const int NT = NW * 64;
    uint32_t *c = ctx->handoff_counters;
    const uint32_t slot = ctx->handoff_heads * 32;
    if (a.kv_f16) {
        if (p.prepared) qkv_attention_kernel<true, true><<<grid, NT, smem, ctx->stream>>>(p, a, c, slot);
        else qkv_attention_kernel<true, false><<<grid, NT, smem, ctx->stream>>>(p, a, c, slot);
    } else {
        if (p.prepared) qkv_attention_kernel<false, true><<<grid, NT, smem, ctx->stream>>>(p, a, c, slot);
        else qkv_attention_kernel<false, false><<<grid, NT, smem, ctx->stream>>>(p, a, c, slot);
    }
    return hipGetLastError();
}

}  // namespace slai
