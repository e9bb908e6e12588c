// Row-per-lane dequantisation-fused GEMV over the tiled weight layout (quant_tiled.h), gfx950.
//
// Same contract as kernels_gemv.hip (the reference's gemv_quant_*.slang shaders dispatched by
// crates/slai/src/ops/gemv_quant.rs:206-312), restructured for the hardware:
//   * a lane owns one row of a 16/32/64-row tile and consumes whole 256-column super-blocks, so a
//     block header is decoded once per 256 weights and rows need no per-row shuffle reduction;
//   * each wave-wide load instruction reads 1024 contiguous bytes, 9-34 of them in flight per lane;
//   * the activations of a super-block sit in 16 registers of a 16-lane DPP row and enter the FMA
//     as a `row_newbcast` operand: no LDS traffic and no extra instructions for x;
//   * wave w of a workgroup owns column group w; the per-wave partial sums meet in LDS once.
// HBM-bound by design (packed weights are read exactly once); no MFMA.
#include "common.h"
#include "device_util.h"
#include "gemv_operands.h"
#include "quant_tiled.h"

namespace slai {
namespace {

using namespace lanes;

// One workgroup = `ngroups` waves; wave w owns column group w of every tile the workgroup visits.  The
// workgroup walks its tiles with a stride of the segment's workgroup count; the next tile's weights
// are requested before the current tile is consumed.
// `vec`: which input vector of a batched launch (0 otherwise) and its strides (see GemvBatch).
struct TiledVec { size_t x_off, emit_off, out0, out1, out2; };
template <int T, bool DUAL, int LD>
__device__ __forceinline__ void tiled_body(const GemvTiledParams &p, uint32_t blk, float *smem, const TiledVec vec) {
    using F = Tiled<T>;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, NW = blockDim.x >> 6;
    const int ROWS = 1 << p.rows_log2, KQ = 64 >> p.rows_log2;
    const int lane16 = lane & 15;
    const int kq = lane >> p.rows_log2;
    float *partial = smem;                                   // [DUAL?2:1][NW][64]
    float *red = smem + (size_t)(DUAL ? 2 : 1) * NW * 64;    // [NW]

    // the segment is picked with selects over statically indexed fields (no dependent fetches of the arguments)
    const uint32_t n0 = p.seg[0].nblocks, n1 = p.seg[1].nblocks;     // unused segments have nblocks = 0
    const int s = blk < n0 ? 0 : (blk - n0 < n1 ? 1 : 2);
    blk -= s == 0 ? 0u : (s == 1 ? n0 : n0 + n1);
    GemvTiledSeg seg;
    seg.W = s == 0 ? p.seg[0].W : (s == 1 ? p.seg[1].W : p.seg[2].W);
    seg.W2 = s == 0 ? p.seg[0].W2 : (s == 1 ? p.seg[1].W2 : p.seg[2].W2);
    seg.nrows = s == 0 ? p.seg[0].nrows : (s == 1 ? p.seg[1].nrows : p.seg[2].nrows);
    seg.nblocks = s == 0 ? n0 : (s == 1 ? n1 : p.seg[2].nblocks);
    seg.out = (s == 0 ? p.seg[0].out : (s == 1 ? p.seg[1].out : p.seg[2].out)) + (s == 0 ? vec.out0 : (s == 1 ? vec.out1 : vec.out2));
    seg.bias = s == 0 ? p.seg[0].bias : (s == 1 ? p.seg[1].bias : p.seg[2].bias);
    seg.flags = s == 0 ? p.seg[0].flags : (s == 1 ? p.seg[1].flags : p.seg[2].flags);
    const uint32_t ntiles = (seg.nrows + ROWS - 1) >> p.rows_log2;
    const uint32_t step = seg.nblocks;

    // ---- requests first: activations (small, cache resident), then the first tile's weights --------
    const uint32_t g = p.group0 + wave;                      // column group owned by this wave
    const uint32_t cb = g * KQ + kq;
    const bool valid = cb < p.ncb;
    const size_t xoff = (size_t)(valid ? cb : 0) * 256 + lane16;
    DevX X;
#pragma unroll
    for (int i = 0; i < 16; ++i) X.x[i] = p.x[vec.x_off + xoff + 16 * i];
    float nw[16], nb[16];
    if (p.prologue != PRO_NONE) {
#pragma unroll
        for (int i = 0; i < 16; ++i) nw[i] = p.norm_w[xoff + 16 * i];
        if (p.norm_b) {
#pragma unroll
            for (int i = 0; i < 16; ++i) nb[i] = p.norm_b[xoff + 16 * i];
        }
    }
    // One register set per matrix: the pieces of a unit are requested a stage ahead of their use inside the dot
    // product (UnitLoader), and the first pieces of the next tile before the current tile's reduction.
    constexpr int NM = DUAL ? 2 : 1;
    typename F::Data d, e;                                   // e: second matrix of a gated pair
    uint16_t dt = 0, et = 0;
    UnitLoader<T, NM, LD> ld;
    auto point = [&](uint32_t t) {
        const size_t off = ((size_t)t * p.ngroups + g) * p.unit_bytes;
        ld.unit[0] = seg.W + off + lane * 16; ld.tailp[0] = seg.W + off + (size_t)F::PT * 1024 + lane * 2; ld.d[0] = &d; ld.t[0] = &dt;
        if constexpr (DUAL) { ld.unit[1] = seg.W2 + off + lane * 16; ld.tailp[1] = seg.W2 + off + (size_t)F::PT * 1024 + lane * 2; ld.d[1] = &e; ld.t[1] = &et; }
    };
    // Loads are retired in issue order, so everything the epilogue reads from global memory (the value accumulated
    // into, the bias, the next norm's weight) is requested BEFORE the tile's weights; waiting for it then does not
    // wait for the weight stream.
    auto epi_request = [&](uint32_t t, float &old, float &bias, float &ew) {
        old = 0.0f; bias = 0.0f; ew = 0.0f;
        const uint32_t row = t * ROWS + tid;
        if (tid < ROWS && row < seg.nrows) {
            if (seg.flags & GEMV_ACCUM) old = seg.out[row];
            if (seg.flags & GEMV_BIAS) bias = seg.bias[row];
            if (seg.flags & GEMV_EMIT) ew = p.emit_w[row];
        }
    };
    uint32_t tile = blk;
    float old = 0.0f, bias = 0.0f, ew = 0.0f;
    if (tile < ntiles) { epi_request(tile, old, bias, ew); point(tile); F::lead(ld); }
#pragma unroll
    for (int i = 0; i < 16; ++i) X.x[i] = valid ? X.x[i] : 0.0f;

    if (p.prologue != PRO_NONE) {
        // every activation is held by ROWS/16 DPP rows; count it once
        const bool counted = valid && (lane & (ROWS - 1)) < 16;
        const float n = (float)p.ncols;
        float mean = 0.0f;
        if (p.prologue == PRO_LAYERNORM) {
            float sm = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) sm += X.x[i];
            sm = wave_sum(counted ? sm : 0.0f);
            if (lane == 0) red[wave] = sm;
            lds_barrier();
            float t = 0.0f;
            for (int w = 0; w < NW; ++w) t += red[w];
            mean = t / n;
            lds_barrier();
        }
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float c = valid ? X.x[i] - mean : 0.0f;
            X.x[i] = c;
            ss = fmaf(c, c, ss);
        }
        ss = wave_sum(counted ? ss : 0.0f);
        if (lane == 0) red[wave] = ss;
        lds_barrier();
        float t = 0.0f;
        for (int w = 0; w < NW; ++w) t += red[w];
        const float scale = 1.0f / sqrtf(t / n + p.eps);    // rms_norm.slang:60-66 / ops/layernorm.rs:104-111
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float v = (X.x[i] * scale) * nw[i];
            if (p.norm_b) v += nb[i];
            X.x[i] = valid ? v : 0.0f;
        }
    }
    if constexpr (T == T_Q6_K) {
#pragma unroll
        for (int i = 0; i < 16; ++i) X.s[i] = row16_sum(X.x[i]);
    } else {
        // Q4_K and Q8_0 only use sums over 32 consecutive activations: reduce pairs, keep the odd slots 0
#pragma unroll
        for (int i = 0; i < 16; i += 2) { X.s[i] = row16_sum(X.x[i] + X.x[i + 1]); X.s[i + 1] = 0.0f; }
    }

    // ---- tiles ------------------------------------------------------------------------------------------
    while (tile < ntiles) {
        const typename F::Data *dp[NM];
        uint16_t tails[NM];
        float o2[NM];
        dp[0] = &d; tails[0] = dt;
        if constexpr (DUAL) { dp[1] = &e; tails[1] = et; }
        F::template dotn<NM>(dp, tails, X, o2, ld);
        const uint32_t next = tile + step;
        const float old_c = old, bias_c = bias, ew_c = ew;
        if (next < ntiles) { epi_request(next, old, bias, ew); point(next); F::lead(ld); }
        float v = o2[0];
        for (int m = ROWS; m < 64; m <<= 1) v += __shfl_xor(v, m, 64);     // across the KQ super-blocks of the wave
        if (lane < ROWS) partial[wave * 64 + lane] = v;
        if constexpr (DUAL) {
            float v2 = o2[1];
            for (int m = ROWS; m < 64; m <<= 1) v2 += __shfl_xor(v2, m, 64);
            if (lane < ROWS) partial[(NW + wave) * 64 + lane] = v2;
        }
        lds_barrier();
        float ewv = 0.0f;
        if (tid < ROWS) {                                      // epilogue: one thread per output row
            const uint32_t row = tile * ROWS + tid;
            if (row < seg.nrows) {
                float o = 0.0f;
                for (int w = 0; w < NW; ++w) o += partial[w * 64 + tid];
                if constexpr (DUAL) {
                    float up = 0.0f;
                    for (int w = 0; w < NW; ++w) up += partial[(NW + w) * 64 + tid];
                    o = up * (o / (1.0f + expf(-o)));          // silu.slang:8-26
                }
                if (seg.flags & GEMV_BIAS) o += bias_c;
                if (seg.flags & GEMV_GELU) o = gelu_f(o);
                if (seg.flags & GEMV_ACCUM) o = old_c + o;
                seg.out[row] = o;
                ewv = ew_c * o;
                if (seg.flags & GEMV_EMIT) p.emit_out[vec.emit_off + row] = ewv;
            }
        }
        if ((seg.flags & GEMV_EMIT) && wave == 0) {            // wave-uniform: the sums of 16 consecutive weighted results
            const float s16 = row16_sum(ewv);                  // (0 in lanes without a row)
            const uint32_t row = tile * ROWS + lane;
            if (lane < ROWS && (lane & 15) == 0 && row < seg.nrows) p.emit_out[vec.emit_off + seg.nrows + (row >> 4)] = s16;
        }
        if (next < ntiles) lds_barrier();                      // partial[] is reused by the next tile
        tile = next;
    }
}

// Stages of weights a wave requests ahead.  Workgroups of up to four waves (narrow matrices: one wave per four
// super-blocks) have little in flight per compute unit and gain from four (+0.3 % on the 7B decode); wider ones lose
// with more than two, and so do the narrow ones with six or eight.
constexpr int lead_stages(int maxt) { return maxt <= 256 ? 4 : 2; }

template <int T, bool DUAL, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_tiled_kernel(const GemvTiledParams p) {
    extern __shared__ float smem[];
    touch_kernel_arguments<sizeof(GemvTiledParams)>();
    tiled_body<T, DUAL, lead_stages(MAXT)>(p, blockIdx.x, smem, TiledVec{0, 0, 0, 0, 0});
}

// The same for several input vectors (a chunk of prompt tokens).  Workgroup i runs on XCD i % 8 and workgroups are
// dispatched in index order: the bt.n workgroups that walk the same tiles get consecutive indices on ONE XCD,
// i = ((blk / 8) * bt.n + b) * 8 + blk % 8, so the first request for a piece of a tile brings it from memory and the
// others find it in that XCD's L2.
template <int T, bool DUAL, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_tiled_batch_kernel(const GemvTiledParams p, const GemvBatch bt, uint32_t total_blocks) {
    extern __shared__ float smem[];
    touch_kernel_arguments<((sizeof(GemvTiledParams) + 63) / 64 + 1) * 64>();
    const uint32_t i = blockIdx.x, j = i >> 3, b = j % bt.n;
    const uint32_t blk = (j / bt.n) * 8 + (i & 7u);
    if (blk >= total_blocks) return;                            // (uniform) the block count rounded up to the eight XCDs
    const TiledVec vec{(size_t)b * bt.x_stride, (size_t)b * bt.emit_stride,
                       (size_t)b * bt.out_stride[0], (size_t)b * bt.out_stride[1], (size_t)b * bt.out_stride[2]};
    tiled_body<T, DUAL, lead_stages(MAXT)>(p, blk, smem, vec);
}

template <int T, bool DUAL>
hipError_t go(hipStream_t s, const GemvTiledParams &p, dim3 grid, int NT, size_t smem, const GemvBatch *bt) {
    if (bt && bt->n > 1) {
        const uint32_t total = grid.x;
        const dim3 g((total + 7) / 8 * 8 * bt->n);
        if (NT <= 256) gemv_tiled_batch_kernel<T, DUAL, 256><<<g, NT, smem, s>>>(p, *bt, total);
        else if (NT <= 512) gemv_tiled_batch_kernel<T, DUAL, 512><<<g, NT, smem, s>>>(p, *bt, total);
        else if (NT <= 768) gemv_tiled_batch_kernel<T, DUAL, 768><<<g, NT, smem, s>>>(p, *bt, total);
        else gemv_tiled_batch_kernel<T, DUAL, 1024><<<g, NT, smem, s>>>(p, *bt, total);
        return hipGetLastError();
    }
    // the bound decides the register budget: 256/512 threads leave 256, 768 leave 168, 1024 leave 128 per lane
    if (NT <= 256) gemv_tiled_kernel<T, DUAL, 256><<<grid, NT, smem, s>>>(p);
    else if (NT <= 512) gemv_tiled_kernel<T, DUAL, 512><<<grid, NT, smem, s>>>(p);
    else if (NT <= 768) gemv_tiled_kernel<T, DUAL, 768><<<grid, NT, smem, s>>>(p);
    else gemv_tiled_kernel<T, DUAL, 1024><<<grid, NT, smem, s>>>(p);
    return hipGetLastError();
}

template <int T> hipError_t launch_t(slai_ctx *ctx, GemvTiledParams &p, const GemvBatch *bt) {
    if (p.launch_groups == 0) p.launch_groups = p.ngroups;
    if (p.ngroups == 0 || p.launch_groups > 16 || p.group0 + p.launch_groups > p.ngroups) return hipErrorInvalidValue;
    // a partial launch cannot normalise its input (that needs every column) or apply a non-linear epilogue
    if (p.launch_groups != p.ngroups && p.prologue != PRO_NONE) return hipErrorInvalidValue;
    for (int i = 0; i < p.nseg; ++i)
        if ((p.seg[i].flags & GEMV_EMIT) && (i != 0 || !p.emit_w || !p.emit_out || p.seg[i].nrows % 16 || (p.seg[i].flags & GEMV_SILU_GATE)))
            return hipErrorInvalidValue;
    const int NT = (int)p.launch_groups * 64;
    const uint32_t rows = 1u << p.rows_log2;
    bool dual = false;
    uint32_t total_tiles = 0;
    for (int i = 0; i < p.nseg; ++i) {
        total_tiles += (p.seg[i].nrows + rows - 1) / rows;
        if (p.seg[i].flags & GEMV_SILU_GATE) dual = true;
    }
    // workgroups: at most `gemv_max_wgs` in total (a small multiple of the CU count), shared between the
    // segments in proportion to their tile counts
    const uint32_t cap = (uint32_t)(ctx->gemv_max_wgs > 0 ? ctx->gemv_max_wgs : 512);
    uint32_t total = 0;
    for (int i = 0; i < p.nseg; ++i) {
        const uint32_t nt = (p.seg[i].nrows + rows - 1) / rows;
        uint32_t nb = total_tiles <= cap ? nt : (uint32_t)(((uint64_t)nt * cap + total_tiles - 1) / total_tiles);
        if (nb < 1) nb = 1;
        if (nb > nt) nb = nt;
        p.seg[i].nblocks = nb;
        total += nb;
    }
    const int NW = NT / 64;
    const size_t smem = ((size_t)(dual ? 2 : 1) * NW * 64 + NW) * sizeof(float);
    dim3 grid(total);
    if (dual) return go<T, true>(ctx->stream, p, grid, NT, smem, bt);
    return go<T, false>(ctx->stream, p, grid, NT, smem, bt);
}

}  // namespace

hipError_t launch_gemv_tiled(slai_ctx *ctx, int type, GemvTiledParams p, const GemvBatch *bt) {
    switch (type) {
    case T_Q4_K: return launch_t<T_Q4_K>(ctx, p, bt);
    case T_Q6_K: return launch_t<T_Q6_K>(ctx, p, bt);
    case T_Q8_0: return launch_t<T_Q8_0>(ctx, p, bt);
    case T_Q4_0: return launch_t<T_Q4_0>(ctx, p, bt);
    case T_Q5_K: return launch_t<T_Q5_K>(ctx, p, bt);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace slai
