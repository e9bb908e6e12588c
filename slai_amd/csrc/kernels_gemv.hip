// Dequantisation-fused GEMV for batch-1 decode on gfx950 (wave64).
//
// Replaces the reference's per-format GEMV shaders
// (crates/slai/shaders/slai/gemv_quant_{q8_0x2,q4_0x2,q4_k,q5_k,q6_kx2}.slang and stensor's f32
// Gemv, dispatched by crates/slai/src/ops/gemv_quant.rs:206-312): out[r] = sum_c deq(W[r,c]) * x[c].
//
// Design: the lanes of a workgroup partition the COLUMNS of a row into fixed 16-byte chunks
// (quant_formats.h), so each lane keeps its slice of the activation vector in registers for
// the whole kernel and streams its chunk of every row with aligned 128-bit loads; R rows are
// in flight per lane.  Nibble / 6-bit unpack happens in registers, accumulation is fp32, a
// wave reduce + one LDS pass across waves finishes a batch of rows.  The kernel is bound by
// HBM traffic of the packed weights; MFMA is not used (batch 1 is not a dense contraction).
//
// Fusions: RMSNorm / LayerNorm(+affine) of the input vector as a prologue (every workgroup
// recomputes the statistics from its register-resident x, which it needs anyway), bias,
// residual accumulate, SiLU-gate of two matrices, and GELU as epilogues.  Up to three
// matrices of the same format share one launch.
#include "common.h"
#include "device_util.h"
#include "quant_formats.h"

namespace slai {
namespace {

constexpr int R = 4;  // rows in flight per lane

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// Sum over the whole workgroup; every thread gets the result.  `red` has >= nwaves floats.
__device__ __forceinline__ float block_sum(float v, float *red, int wave, int lane, int nwaves) {
    v = wave_sum(v);
    __syncthreads();  // protect `red` from a previous use
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nwaves; ++w) t += red[w];
    return t;
}

__device__ __forceinline__ float gelu_f(float x) {
    // crates/slai/src/ops/unary.rs:81-85
    const float GELU_COEF_A = 0.044715f, SQRT_2_OVER_PI = 0.7978846f;
    return 0.5f * x * (1.0f + tanhf(SQRT_2_OVER_PI * x * (1.0f + GELU_COEF_A * x * x)));
}

template <int T, int K, bool DUAL, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_kernel(const GemvParams p) {
    touch_kernel_arguments<sizeof(GemvParams)>();
    using F = Chunk<T>;
    extern __shared__ float smem[];
    const int tid = threadIdx.x, NT = blockDim.x, lane = tid & 63, wave = tid >> 6, NW = NT >> 6;
    float *partial = smem;                       // [rows_per_wg][NW]
    float *red = smem + p.rows_per_wg * NW * (DUAL ? 2 : 1);  // [NW], behind both partial arrays

    // which matrix of the launch does this workgroup serve
    int s = 0;
    uint32_t blk = blockIdx.x;
    while (s < p.nseg - 1 && blk >= p.seg[s].nblocks) { blk -= p.seg[s].nblocks; ++s; }
    const GemvSeg &seg = p.seg[s];

    const uint32_t nchunks = F::nchunks(p.ncols);

    // ---- activation slice into registers --------------------------------------
    float x[K][F::E];
    float xs[K][F::NRUN];
    bool valid[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = tid + k * NT;
        valid[k] = c < nchunks;
#pragma unroll
        for (int r = 0; r < F::NRUN; ++r) {
            const float4 *src = reinterpret_cast<const float4 *>(p.x + F::run_col(valid[k] ? c : 0, r));
#pragma unroll
            for (int i = 0; i < F::RUNLEN / 4; ++i) {
                float4 v = valid[k] ? src[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                x[k][r * F::RUNLEN + 4 * i + 0] = v.x; x[k][r * F::RUNLEN + 4 * i + 1] = v.y;
                x[k][r * F::RUNLEN + 4 * i + 2] = v.z; x[k][r * F::RUNLEN + 4 * i + 3] = v.w;
            }
        }
    }

    // ---- prologue: normalise x in registers ---------------------------------------
    if (p.prologue != PRO_NONE) {
        const float eps = p.eps;
        const float n = (float)p.ncols;
        float mean = 0.0f;
        if (p.prologue == PRO_LAYERNORM) {
            float sm = 0.0f;
#pragma unroll
            for (int k = 0; k < K; ++k)
#pragma unroll
                for (int i = 0; i < F::E; ++i) sm += x[k][i];
            mean = block_sum(sm, red, wave, lane, NW) / n;
        }
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int i = 0; i < F::E; ++i) {
                float c = valid[k] ? x[k][i] - mean : 0.0f;
                x[k][i] = c;
                ss = fmaf(c, c, ss);
            }
        ss = block_sum(ss, red, wave, lane, NW);
        // rms_norm.slang:60-66 / ops/layernorm.rs:104-111: scale = 1/sqrt(mean_sq + eps)
        const float scale = 1.0f / sqrtf(ss / n + eps);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t c = valid[k] ? tid + k * NT : 0;
#pragma unroll
            for (int r = 0; r < F::NRUN; ++r) {
                const uint32_t col = F::run_col(c, r);
#pragma unroll
                for (int i = 0; i < F::RUNLEN; ++i) {
                    float v = x[k][r * F::RUNLEN + i] * scale;
                    if (valid[k]) {
                        v = v * p.norm_w[col + i];
                        if (p.norm_b) v += p.norm_b[col + i];
                    }
                    x[k][r * F::RUNLEN + i] = v;
                }
            }
        }
    }
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
        for (int r = 0; r < F::NRUN; ++r) {
            float t = 0.0f;
#pragma unroll
            for (int i = 0; i < F::RUNLEN; ++i) t += x[k][r * F::RUNLEN + i];
            xs[k][r] = t;
        }

    // ---- stream the rows -----------------------------------------------------------
    const uint32_t row0 = blk * p.rows_per_wg;
    const uint32_t last_row = seg.nrows - 1;
    for (uint32_t rb = 0; rb < p.rows_per_wg; rb += R) {
        typename F::Data d[R][K];
        typename F::Data d2[DUAL ? R : 1][DUAL ? K : 1];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t row = min(row0 + rb + r, last_row);
            const uint8_t *wr = seg.W + (size_t)row * seg.row_stride;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const uint32_t c = valid[k] ? tid + k * NT : 0;
                d[r][k] = F::load(wr, p.nb, c);
                if constexpr (DUAL) d2[r][k] = F::load(seg.W2 + (size_t)row * seg.row_stride, p.nb, c);
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float acc = 0.0f, acc2 = 0.0f;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const uint32_t c = valid[k] ? tid + k * NT : 0;
                float v = F::dot(d[r][k], c, x[k], xs[k]);
                acc += valid[k] ? v : 0.0f;
                if constexpr (DUAL) {
                    float v2 = F::dot(d2[r][k], c, x[k], xs[k]);
                    acc2 += valid[k] ? v2 : 0.0f;
                }
            }
            acc = wave_sum(acc);
            if constexpr (DUAL) acc2 = wave_sum(acc2);
            if (lane == 0) {
                partial[(rb + r) * NW + wave] = acc;
                if constexpr (DUAL) partial[(p.rows_per_wg + rb + r) * NW + wave] = acc2;
            }
        }
    }
    __syncthreads();

    // ---- epilogue ----------------------------------------------------------------
    if (tid < (int)p.rows_per_wg) {
        const uint32_t row = row0 + tid;
        if (row < seg.nrows) {
            float v = 0.0f;
            for (int w = 0; w < NW; ++w) v += partial[tid * NW + w];
            if constexpr (DUAL) {
                float u = 0.0f;
                for (int w = 0; w < NW; ++w) u += partial[(p.rows_per_wg + tid) * NW + w];
                // silu.slang:8-26: out = up * gate / (1 + exp(-gate))
                v = u * (v / (1.0f + expf(-v)));
            }
            if (seg.flags & GEMV_BIAS) v += seg.bias[row];
            if (seg.flags & GEMV_GELU) v = gelu_f(v);
            if (seg.flags & GEMV_ACCUM) v = seg.out[row] + v;
            seg.out[row] = v;
        }
    }
}

template <int T, bool DUAL>
hipError_t launch_k(slai_ctx *ctx, const GemvParams &p, int K, dim3 grid, int NT, size_t smem) {
    hipStream_t s = ctx->stream;
#define SLAI_GEMV_GO(KK)                                                                  \
    do {                                                                                  \
        if (NT <= 512) gemv_kernel<T, KK, DUAL, 512><<<grid, NT, smem, s>>>(p);           \
        else gemv_kernel<T, KK, DUAL, 1024><<<grid, NT, smem, s>>>(p);                    \
    } while (0)
    switch (K) {
    case 1: SLAI_GEMV_GO(1); break;
    case 2: SLAI_GEMV_GO(2); break;
    case 3: if constexpr (Chunk<T>::E <= 32) { SLAI_GEMV_GO(3); break; } return hipErrorInvalidValue;
    case 4: if constexpr (Chunk<T>::E <= 16) { SLAI_GEMV_GO(4); break; } return hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
    }
#undef SLAI_GEMV_GO
    return hipGetLastError();
}

template <int T> hipError_t launch_t(slai_ctx *ctx, GemvParams &p) {
    using F = Chunk<T>;
    const uint32_t nchunks = F::nchunks(p.ncols);
    const int maxk = F::E <= 16 ? 4 : (F::E <= 32 ? 3 : 2);
    int maxt = ctx->gemv_max_threads;
    if (maxt < 64) maxt = 64;
    if (maxt > 1024) maxt = 1024;
    int K = (int)((nchunks + maxt - 1) / maxt);
    if (K < 1) K = 1;
    if (K > maxk) {  // fall back to the widest workgroup before giving up
        K = (int)((nchunks + 1023) / 1024);
        if (K > maxk) return hipErrorInvalidValue;
    }
    int NT = (int)(((nchunks + K - 1) / K + 63) / 64) * 64;
    bool dual = false;
    uint32_t total = 0;
    uint32_t rpw = p.rows_per_wg ? p.rows_per_wg : 8;
    rpw = (rpw + R - 1) / R * R;
    if (rpw > 64) rpw = 64;
    p.rows_per_wg = rpw;
    for (int i = 0; i < p.nseg; ++i) {
        p.seg[i].nblocks = (p.seg[i].nrows + rpw - 1) / rpw;
        total += p.seg[i].nblocks;
        if (p.seg[i].flags & GEMV_SILU_GATE) dual = true;
    }
    const int NW = NT / 64;
    size_t smem = ((size_t)rpw * NW * (dual ? 2 : 1) + NW) * sizeof(float);
    dim3 grid(total);
    if (dual) return launch_k<T, true>(ctx, p, K, grid, NT, smem);
    return launch_k<T, false>(ctx, p, K, grid, NT, smem);
}

}  // namespace

bool gemv_supports(int type, uint32_t ncols) {
    switch (type) {
    case T_F32: return ncols % 4 == 0 && ncols / 4 <= 4096;
    case T_F16: return ncols % 8 == 0 && ncols / 8 <= 4096;
    case T_Q8_0: return ncols % 32 == 0 && ncols / 16 <= 4096;
    case T_Q4_0: case T_Q4_1: case T_Q5_0: case T_Q5_1: return ncols % 32 == 0 && ncols / 32 <= 3072;
    case T_Q8_K: return ncols % 256 == 0 && ncols / 16 <= 4096;
    case T_Q4_K: case T_Q5_K: return ncols % 256 == 0 && ncols / 32 <= 3072;
    case T_Q6_K: return ncols % 256 == 0 && ncols / 64 <= 2048;
    default: return false;
    }
}

hipError_t launch_gemv(slai_ctx *ctx, int type, GemvParams p) {
    if (!gemv_supports(type, p.ncols)) return hipErrorInvalidValue;
    switch (type) {
    case T_F32: return launch_t<T_F32>(ctx, p);
    case T_F16: return launch_t<T_F16>(ctx, p);
    case T_Q4_0: return launch_t<T_Q4_0>(ctx, p);
    case T_Q4_1: return launch_t<T_Q4_1>(ctx, p);
    case T_Q5_0: return launch_t<T_Q5_0>(ctx, p);
    case T_Q5_1: return launch_t<T_Q5_1>(ctx, p);
    case T_Q8_K: return launch_t<T_Q8_K>(ctx, p);
    case T_Q8_0: return launch_t<T_Q8_0>(ctx, p);
    case T_Q4_K: return launch_t<T_Q4_K>(ctx, p);
    case T_Q5_K: return launch_t<T_Q5_K>(ctx, p);
    case T_Q6_K: return launch_t<T_Q6_K>(ctx, p);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace slai
