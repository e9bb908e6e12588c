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
#include "quant_tiled.h"

namespace slai {
namespace {

__device__ __forceinline__ float gelu_f(float x) {
    const float GELU_COEF_A = 0.044715f, SQRT_2_OVER_PI = 0.7978846f;   // ops/unary.rs:81-85
    return 0.5f * x * (1.0f + tanhf(SQRT_2_OVER_PI * x * (1.0f + GELU_COEF_A * x * x)));
}

__device__ __forceinline__ float row16_sum(float v) {
    v += __shfl_xor(v, 1, 64); v += __shfl_xor(v, 2, 64); v += __shfl_xor(v, 4, 64); v += __shfl_xor(v, 8, 64);
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

struct DevX {
    float x[16];    // register i, lane j of the DPP row <-> x[cb*256 + 16*i + j]
    float s[16];    // s[i] = sum over the row of x[i]
    // acc += sum_b byte_b(w) * x[16*I + 4*W + b].  Lane k of every 16-lane row of register I is broadcast
    // to the row by the DPP operand (row_newbcast:k), so the activation costs no instruction of its own.
    // Written as assembly: the compiler forms DPP operands only on two-address encodings, which an FMA
    // does not have before register allocation, and it would otherwise hoist all 256 conversions of a
    // super-block ahead of the FMAs and run out of registers.
    template <int I, int W> __device__ __forceinline__ float fma4(uint32_t w, float acc) const {
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

template <int T> __device__ __forceinline__ void load_unit(const uint8_t *unit, int lane, typename Tiled<T>::Data &d, uint16_t &tail) {
    using F = Tiled<T>;
#pragma unroll
    for (int p = 0; p < F::PT; ++p) d.p[p] = ld128(unit + (size_t)p * 1024 + lane * 16);
    if constexpr (F::TAIL) tail = ld16(unit + (size_t)F::PT * 1024 + lane * 2);
    else tail = 0;
}

// NU = tiles per workgroup whose loads are issued before any arithmetic (2 matrices when DUAL).
template <int T, bool DUAL, int NU, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_tiled_kernel(const GemvTiledParams p) {
    using F = Tiled<T>;
    extern __shared__ float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, NW = blockDim.x >> 6;
    const int ROWS = 1 << p.rows_log2, KQ = 64 >> p.rows_log2;
    const int lane16 = lane & 15;
    const int kq = lane >> p.rows_log2;
    float *partial = smem;                                          // [NU][DUAL?2:1][NW][64]
    float *red = smem + (size_t)NU * (DUAL ? 2 : 1) * NW * 64;      // [NW]

    int s = 0;
    uint32_t blk = blockIdx.x;
    while (s < p.nseg - 1 && blk >= p.seg[s].nblocks) { blk -= p.seg[s].nblocks; ++s; }
    const GemvTiledSeg &seg = p.seg[s];
    const uint32_t ntiles = (seg.nrows + ROWS - 1) >> p.rows_log2;

    // ---- issue every weight load of this workgroup first: they do not depend on x ------------
    const uint32_t g = wave;                                        // column group owned by this wave
    typename F::Data d[NU];
    typename F::Data d2[DUAL ? NU : 1];
    uint16_t tail[NU], tail2[DUAL ? NU : 1];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const uint32_t tile = min(blk * NU + u, ntiles - 1);
        const size_t off = ((size_t)tile * p.ngroups + g) * p.unit_bytes;
        load_unit<T>(seg.W + off, lane, d[u], tail[u]);
        if constexpr (DUAL) load_unit<T>(seg.W2 + off, lane, d2[u], tail2[u]);
    }

    // ---- activations of this wave's super-blocks ---------------------------------------------------
    DevX X;
    const uint32_t cb = g * KQ + kq;
    const bool valid = cb < p.ncb;
    const float *xp = p.x + (size_t)(valid ? cb : 0) * 256 + lane16;
#pragma unroll
    for (int i = 0; i < 16; ++i) X.x[i] = valid ? xp[16 * i] : 0.0f;

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
            __syncthreads();
            float t = 0.0f;
            for (int w = 0; w < NW; ++w) t += red[w];
            mean = t / n;
            __syncthreads();
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
        __syncthreads();
        float t = 0.0f;
        for (int w = 0; w < NW; ++w) t += red[w];
        const float eps = p.eps_ptr ? *p.eps_ptr : p.eps;
        const float scale = 1.0f / sqrtf(t / n + eps);    // rms_norm.slang:60-66 / ops/layernorm.rs:104-111
        const float *wp = p.norm_w + (size_t)(valid ? cb : 0) * 256 + lane16;
        const float *bp = p.norm_b ? p.norm_b + (size_t)(valid ? cb : 0) * 256 + lane16 : nullptr;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float v = X.x[i] * scale;
            if (valid) { v = v * wp[16 * i]; if (bp) v += bp[16 * i]; }
            X.x[i] = v;
        }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) X.s[i] = row16_sum(X.x[i]);

    // ---- per-lane row dot products ------------------------------------------------------------------
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        float v = F::dot(d[u], tail[u], X);
        for (int m = ROWS; m < 64; m <<= 1) v += __shfl_xor(v, m, 64);     // across the KQ super-blocks of the wave
        if (lane < ROWS) partial[((u * (DUAL ? 2 : 1)) * NW + wave) * 64 + lane] = v;
        if constexpr (DUAL) {
            float v2 = F::dot(d2[u], tail2[u], X);
            for (int m = ROWS; m < 64; m <<= 1) v2 += __shfl_xor(v2, m, 64);
            if (lane < ROWS) partial[((u * 2 + 1) * NW + wave) * 64 + lane] = v2;
        }
    }
    __syncthreads();

    // ---- epilogue: one thread per output row ----------------------------------------------------------
    if (tid < NU * ROWS) {
        const int u = tid >> p.rows_log2, r = tid & (ROWS - 1);
        const uint32_t tile = blk * NU + u;
        const uint32_t row = tile * ROWS + r;
        if (tile < ntiles && row < seg.nrows) {
            float v = 0.0f;
            for (int w = 0; w < NW; ++w) v += partial[((u * (DUAL ? 2 : 1)) * NW + w) * 64 + r];
            if constexpr (DUAL) {
                float up = 0.0f;
                for (int w = 0; w < NW; ++w) up += partial[((u * 2 + 1) * NW + w) * 64 + r];
                v = up * (v / (1.0f + expf(-v)));          // silu.slang:8-26
            }
            if (seg.flags & GEMV_BIAS) v += seg.bias[row];
            if (seg.flags & GEMV_GELU) v = gelu_f(v);
            if (seg.flags & GEMV_ACCUM) v = seg.out[row] + v;
            seg.out[row] = v;
        }
    }
}

template <int T, bool DUAL, int NU>
hipError_t go(hipStream_t s, const GemvTiledParams &p, dim3 grid, int NT, size_t smem) {
    if (NT <= 256) gemv_tiled_kernel<T, DUAL, NU, 256><<<grid, NT, smem, s>>>(p);
    else if (NT <= 512) gemv_tiled_kernel<T, DUAL, NU, 512><<<grid, NT, smem, s>>>(p);
    else gemv_tiled_kernel<T, DUAL, NU, 1024><<<grid, NT, smem, s>>>(p);
    return hipGetLastError();
}

template <int T> hipError_t launch_t(slai_ctx *ctx, GemvTiledParams &p) {
    if (p.ngroups == 0 || p.ngroups > 16) return hipErrorInvalidValue;
    const int NT = (int)p.ngroups * 64;
    const uint32_t rows = 1u << p.rows_log2;
    bool dual = false;
    uint32_t total_tiles = 0;
    for (int i = 0; i < p.nseg; ++i) {
        total_tiles += (p.seg[i].nrows + rows - 1) / rows;
        if (p.seg[i].flags & GEMV_SILU_GATE) dual = true;
    }
    // two tiles per workgroup once there are plenty of tiles and registers allow it
    int NU = (!dual && NT <= 256 && total_tiles >= 1024 && ctx->gemv_tiles_per_wg >= 2) ? 2 : 1;
    if (T == T_Q8_0 && NT > 256) NU = 1;
    uint32_t total = 0;
    for (int i = 0; i < p.nseg; ++i) {
        const uint32_t nt = (p.seg[i].nrows + rows - 1) / rows;
        p.seg[i].nblocks = (nt + NU - 1) / NU;
        total += p.seg[i].nblocks;
    }
    const int NW = NT / 64;
    const size_t smem = ((size_t)NU * (dual ? 2 : 1) * NW * 64 + NW) * sizeof(float);
    dim3 grid(total);
    if (dual) return go<T, true, 1>(ctx->stream, p, grid, NT, smem);
    if (NU == 2) return go<T, false, 2>(ctx->stream, p, grid, NT, smem);
    return go<T, false, 1>(ctx->stream, p, grid, NT, smem);
}

}  // namespace

hipError_t launch_gemv_tiled(slai_ctx *ctx, int type, GemvTiledParams p) {
    switch (type) {
    case T_Q4_K: return launch_t<T_Q4_K>(ctx, p);
    case T_Q6_K: return launch_t<T_Q6_K>(ctx, p);
    case T_Q8_0: return launch_t<T_Q8_0>(ctx, p);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace slai
