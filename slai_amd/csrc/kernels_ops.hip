// Element-wise, normalisation, softmax, f32 matmul and argmax kernels of the decode path.
// Each kernel names the reference shader / CPU routine whose result it reproduces.
#include "common.h"
#include "device_util.h"
#include <float.h>
#include <hip/hip_fp16.h>

namespace slai {
namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}
// blockDim.x must be a multiple of 64, <= 1024; red has 16 floats
__device__ __forceinline__ float block_sum(float v, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; ++w) t += red[w];
    return t;
}
__device__ __forceinline__ float block_max(float v, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int w = 1; w < nw; ++w) t = fmaxf(t, red[w]);
    return t;
}

// rms_norm.slang:48-67 / models/llama2/cpu.rs:340-348: out = (v * 1/sqrt(mean(v^2)+eps)) * w
__global__ void rms_norm_kernel(VecView out, VecView v, VecView w, const float *eps_ptr, float eps) {
    __shared__ float red[16];
    float ss = 0.0f;
    for (uint32_t i = threadIdx.x; i < v.n; i += blockDim.x) { float a = v.p[(size_t)i * v.stride]; ss = fmaf(a, a, ss); }
    ss = block_sum(ss, red);
    const float e = eps_ptr ? *eps_ptr : eps;
    const float rms = 1.0f / sqrtf(ss / (float)v.n + e);
    for (uint32_t i = threadIdx.x; i < v.n; i += blockDim.x)
        out.p[(size_t)i * out.stride] = (v.p[(size_t)i * v.stride] * rms) * w.p[(size_t)i * w.stride];
}

// layernorm.slang:19-81 / ops/layernorm.rs:104-111 (no affine)
__global__ void layernorm_kernel(VecView out, VecView v, float eps) {
    __shared__ float red[16];
    float sm = 0.0f;
    for (uint32_t i = threadIdx.x; i < v.n; i += blockDim.x) sm += v.p[(size_t)i * v.stride];
    const float mean = block_sum(sm, red) / (float)v.n;
    float ss = 0.0f;
    for (uint32_t i = threadIdx.x; i < v.n; i += blockDim.x) { float c = v.p[(size_t)i * v.stride] - mean; ss = fmaf(c, c, ss); }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)v.n + eps);
    for (uint32_t i = threadIdx.x; i < v.n; i += blockDim.x)
        out.p[(size_t)i * out.stride] = (v.p[(size_t)i * v.stride] - mean) * scale;
}

// stensor OpAssign Add / Mul / Copy (context.rs:428-469,660-672)
template <int OP>   // 0 add, 1 mul, 2 copy (a <- b; a is not read)
__global__ void binop_kernel(VecView a, VecView b) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += gridDim.x * blockDim.x) {
        float *pa = a.p + (size_t)i * a.stride;
        const float vb = b.p[(size_t)i * b.stride];
        if constexpr (OP == 0) *pa = *pa + vb;
        else if constexpr (OP == 1) *pa = *pa * vb;
        else *pa = vb;
    }
}

// The norm-weighted copy of x that the 64-row-tile GEMV reads through the scalar cache: out[i] = x[i] * w[i] for
// i < n, followed by the n/16 sums of 16 consecutive products.  n is a multiple of 16.
__global__ void prepare_kernel(float *out, const float *x, const float *w, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;      // grid covers n exactly (n % 64 == 0 not required)
    float v = 0.0f;
    if (i < n) { v = x[i] * w[i]; out[i] = v; }
    float s = v;
    s += __shfl_xor(s, 1, 64); s += __shfl_xor(s, 2, 64); s += __shfl_xor(s, 4, 64); s += __shfl_xor(s, 8, 64);
    if (i < n && (i & 15) == 0) out[n + (i >> 4)] = s;
}

// silu.slang:11-27: a = b * a / (1 + exp(-a))
__global__ void silu_kernel(VecView a, VecView b) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += gridDim.x * blockDim.x) {
        float *pa = a.p + (size_t)i * a.stride;
        const float l = *pa, r = b.p[(size_t)i * b.stride];
        *pa = r * (l / (1.0f + expf(-1.0f * l)));
    }
}

// the same over gate and up given as `nparts` partial sums each
// (n, part: multiples of four, 16-byte aligned; ntokens < 32: a quad-major matrix of which only the first ntokens token
// slots are in use.  split_flag: write each group of four as f16 heads and remainders, the
// form the prompt-chunk GEMM reads on the half-precision matrix cores, and report values beyond the f16 range.)
__global__ void silu_parts_kernel(float4 *a, const float4 *b, uint32_t n4, uint32_t nparts, uint32_t part4, int *split_flag, uint32_t ntokens) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += gridDim.x * blockDim.x) {
        if ((i & 31u) >= ntokens) continue;                    // quad-major: group i belongs to token slot i % 32; unused slots hold stale values
        float4 l = make_float4(0.0f, 0.0f, 0.0f, 0.0f), r = l;
        for (uint32_t s = 0; s < nparts; ++s) {
            const float4 la = a[i + (size_t)s * part4], rb = b[i + (size_t)s * part4];
            l.x += la.x; l.y += la.y; l.z += la.z; l.w += la.w;
            r.x += rb.x; r.y += rb.y; r.z += rb.z; r.w += rb.w;
        }
        const float4 o = make_float4(r.x * (l.x / (1.0f + expf(-1.0f * l.x))), r.y * (l.y / (1.0f + expf(-1.0f * l.y))),
                                     r.z * (l.z / (1.0f + expf(-1.0f * l.z))), r.w * (l.w / (1.0f + expf(-1.0f * l.w))));
        if (split_flag) {
            if (split_overflows(o)) *split_flag = 3;            // 3: a gated hidden value
            a[i] = split_quad(o);
        } else {
            a[i] = o;
        }
    }
}

// ops/unary.rs:81-85 (UnaryOp::Gelu) over a quad-major matrix (groups of four columns, 32 token slots of which the
// first ntokens are in use), in place; with split_flag written as f16 heads and remainders like silu_parts_kernel does
__global__ void gelu_quads_kernel(float4 *a, uint32_t n4, uint32_t ntokens, int *split_flag) {
    const float GELU_COEF_A = 0.044715f, SQRT_2_OVER_PI = 0.7978846f;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += gridDim.x * blockDim.x) {
        if ((i & 31u) >= ntokens) continue;
        const float4 x = a[i];
        const float4 o = make_float4(0.5f * x.x * (1.0f + tanhf(SQRT_2_OVER_PI * x.x * (1.0f + GELU_COEF_A * x.x * x.x))),
                                     0.5f * x.y * (1.0f + tanhf(SQRT_2_OVER_PI * x.y * (1.0f + GELU_COEF_A * x.y * x.y))),
                                     0.5f * x.z * (1.0f + tanhf(SQRT_2_OVER_PI * x.z * (1.0f + GELU_COEF_A * x.z * x.z))),
                                     0.5f * x.w * (1.0f + tanhf(SQRT_2_OVER_PI * x.w * (1.0f + GELU_COEF_A * x.w * x.w))));
        if (split_flag) {
            if (split_overflows(o)) *split_flag = 3;            // 3: a hidden value
            a[i] = split_quad(o);
        } else {
            a[i] = o;
        }
    }
}

// ops/unary.rs:81-85 (UnaryOp::Gelu)
__global__ void gelu_kernel(VecView a) {
    const float GELU_COEF_A = 0.044715f, SQRT_2_OVER_PI = 0.7978846f;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += gridDim.x * blockDim.x) {
        float *pa = a.p + (size_t)i * a.stride;
        const float x = *pa;
        *pa = 0.5f * x * (1.0f + tanhf(SQRT_2_OVER_PI * x * (1.0f + GELU_COEF_A * x * x)));
    }
}

// rope.slang:27-84; one thread per rotated pair
__global__ void rope_kernel(int variant, const slai_rope_config *cfg, VecView q, VecView k) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (2 * i >= q.n) return;
    const uint32_t hs = cfg->head_size;
    const float head_dim = (float)((i * 2) % hs);
    const float theta = powf(cfg->base_freq, -head_dim / (float)hs);
    const float m_theta = (float)cfg->pos * theta;
    const float c = cosf(m_theta), s = sinf(m_theta);
    uint32_t i0, i1;
    if (variant == SLAI_ROPE_ORIGINAL) { i0 = 2 * i; i1 = 2 * i + 1; }
    else { const uint32_t head_id = (i * 2) / hs; i0 = i + head_id * hs / 2; i1 = i0 + hs / 2; }
    float x = q.p[(size_t)i0 * q.stride], y = q.p[(size_t)i1 * q.stride];
    q.p[(size_t)i0 * q.stride] = c * x - s * y;
    q.p[(size_t)i1 * q.stride] = s * x + c * y;
    if (i * 2 < cfg->kv_dim) {
        x = k.p[(size_t)i0 * k.stride]; y = k.p[(size_t)i1 * k.stride];
        k.p[(size_t)i0 * k.stride] = c * x - s * y;
        k.p[(size_t)i1 * k.stride] = s * x + c * y;
    }
}

// batched_multiquery_attention.slang:18-32
__global__ void attn_mask_kernel(const slai_attn_params *params, float *attn, uint32_t nthreads) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nthreads) return;
    const uint32_t nonzero_len = params->pos + 1u, aligned_len = (params->pos + 1u + 3u) / 4u * 4u;
    if (i % aligned_len < nonzero_len) attn[i] /= sqrtf((float)params->head_size);
    else attn[i] = 0.0f;
}

// softmax.slang:26-96: one workgroup per column (j,k,l); max, exp, sum, divide
__global__ void softmax_cols_kernel(View4 m) {
    __shared__ float red[16];
    const uint32_t j = blockIdx.x, k = blockIdx.y, l = blockIdx.z;
    float *col = m.p + (size_t)j * m.stride[1] + (size_t)k * m.stride[2] + (size_t)l * m.stride[3];
    const uint32_t n = m.size[0], st = m.stride[0];
    float mx = -1.0e38f;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) mx = fmaxf(mx, col[(size_t)i * st]);
    mx = block_max(mx, red);
    float den = 0.0f;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float e = expf(col[(size_t)i * st] - mx);
        den += e;
        col[(size_t)i * st] = e;
    }
    den = block_sum(den, red);
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) col[(size_t)i * st] = col[(size_t)i * st] / den;
}

// stensor f32 Gemv with view shapes (context.rs:298-317): out(i,j,k,l) = sum_c A'(i,c,k,l) B'(c,j,k,l),
// A' = A or A^T, B' = B or B^T; a batch dimension of size 1 broadcasts.  One wave per output element.
__global__ void matmul_f32_kernel(View4 out, View4 a, View4 b, int a_mode, int b_mode, uint32_t inner) {
    const uint32_t lane = threadIdx.x & 63;
    const size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const size_t total = (size_t)out.size[0] * out.size[1] * out.size[2] * out.size[3];
    if (wave >= total) return;
    uint32_t i = (uint32_t)(wave % out.size[0]);
    size_t rest = wave / out.size[0];
    uint32_t j = (uint32_t)(rest % out.size[1]); rest /= out.size[1];
    uint32_t k = (uint32_t)(rest % out.size[2]);
    uint32_t l = (uint32_t)(rest / out.size[2]);
    const uint32_t ka = a.size[2] == 1 ? 0 : k, la = a.size[3] == 1 ? 0 : l;
    const uint32_t kb = b.size[2] == 1 ? 0 : k, lb = b.size[3] == 1 ? 0 : l;
    const float *pa = a.p + (size_t)ka * a.stride[2] + (size_t)la * a.stride[3];
    const float *pb = b.p + (size_t)kb * b.stride[2] + (size_t)lb * b.stride[3];
    const size_t a_i = a_mode == SLAI_MODE_N ? a.stride[0] : a.stride[1], a_c = a_mode == SLAI_MODE_N ? a.stride[1] : a.stride[0];
    const size_t b_c = b_mode == SLAI_MODE_N ? b.stride[0] : b.stride[1], b_j = b_mode == SLAI_MODE_N ? b.stride[1] : b.stride[0];
    float acc = 0.0f;
    for (uint32_t c = lane; c < inner; c += 64) acc = fmaf(pa[i * a_i + c * a_c], pb[c * b_c + j * b_j], acc);
    acc = wave_sum(acc);
    if (lane == 0)
        out.p[(size_t)i * out.stride[0] + (size_t)j * out.stride[1] + (size_t)k * out.stride[2] + (size_t)l * out.stride[3]] = acc;
}

// models/sampler.rs:55-57 (nalgebra imax: first strict maximum) + the forced-token rule of
// slai-chat/src/sampler.rs:100-105 and the loop bookkeeping of chat_llama2.rs:105-158, on the device.
__global__ void argmax_kernel(const float *v, uint32_t n, int *out_index, DecodeState *st, const int *prompt,
                              int *out_tokens) {
    __shared__ float bv[16];
    __shared__ uint32_t bi[16];
    float best = -FLT_MAX;
    uint32_t besti = 0xffffffffu;
    // ascending indices per thread, strict comparison: the first maximum is kept (nalgebra `imax`).  16-byte loads,
    // eight of them in flight per thread.
    auto take = [&](float x, uint32_t i) { if (besti == 0xffffffffu || x > best) { best = x; besti = i; } };
    const uint32_t n4 = ((uintptr_t)v % 16 == 0) ? n / 4 : 0;
    const float4 *v4 = reinterpret_cast<const float4 *>(v);
    for (uint32_t i = threadIdx.x; i < n4; i += 8 * blockDim.x) {
        float4 r[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const uint32_t j = i + u * blockDim.x;
            r[u] = v4[j < n4 ? j : i];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const uint32_t j = i + u * blockDim.x;
            if (j < n4) { take(r[u].x, 4 * j); take(r[u].y, 4 * j + 1); take(r[u].z, 4 * j + 2); take(r[u].w, 4 * j + 3); }
        }
    }
    for (uint32_t i = 4 * n4 + threadIdx.x; i < n; i += blockDim.x) take(v[i], i);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ob = __shfl_xor(best, m, 64);
        const uint32_t oi = __shfl_xor(besti, m, 64);
        if (oi != 0xffffffffu && (besti == 0xffffffffu || ob > best || (ob == best && oi < besti))) { best = ob; besti = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    if (lane == 0) { bv[wave] = best; bi[wave] = besti; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < nw; ++w)
            if (bi[w] != 0xffffffffu && (besti == 0xffffffffu || bv[w] > best || (bv[w] == best && bi[w] < besti))) { best = bv[w]; besti = bi[w]; }
        int next = (int)besti;
        if (out_index) *out_index = next;
        if (st) {
            const int pos = st->pos;
            if (pos < st->n_prompt - 1) next = prompt[pos + 1];
            out_tokens[st->step] = next;
            st->token = next;
            st->pos = pos + 1;
            st->step = st->step + 1;
        }
    }
}

// f32 -> cache element type (f16 round-to-nearest-even, or a plain copy)
__global__ void store_kv_kernel(const float *src, void *dst, uint32_t n, int f16) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    if (f16) reinterpret_cast<__half *>(dst)[i] = __float2half_rn(src[i]);
    else reinterpret_cast<float *>(dst)[i] = src[i];
}

// which XCD each workgroup of a launch runs on (hardware id register)
__global__ void xcd_of_workgroup_kernel(uint32_t *out) {
    uint32_t v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    if (threadIdx.x == 0) out[blockIdx.x] = v & 0xfu;
}

inline uint32_t grid_for(uint32_t n, uint32_t block) { uint32_t g = (n + block - 1) / block; return g ? (g > 4096 ? 4096 : g) : 1; }

}  // namespace

hipError_t launch_xcd_of_workgroup(hipStream_t s, uint32_t *out, uint32_t n_workgroups) {
    xcd_of_workgroup_kernel<<<n_workgroups, 64, 0, s>>>(out);
    return hipGetLastError();
}
hipError_t launch_store_kv(hipStream_t s, const float *src, void *dst, uint32_t n, int f16) {
    store_kv_kernel<<<(n + 255) / 256, 256, 0, s>>>(src, dst, n, f16);
    return hipGetLastError();
}
hipError_t launch_rms_norm(hipStream_t s, VecView out, VecView v, VecView w, const float *eps_ptr, float eps) {
    rms_norm_kernel<<<1, v.n >= 2048 ? 1024 : 256, 0, s>>>(out, v, w, eps_ptr, eps);
    return hipGetLastError();
}
hipError_t launch_layernorm(hipStream_t s, VecView out, VecView v, float eps) {
    layernorm_kernel<<<1, v.n >= 2048 ? 1024 : 256, 0, s>>>(out, v, eps);
    return hipGetLastError();
}
hipError_t launch_binop(hipStream_t s, int op, VecView a, VecView b) {
    const dim3 grid = grid_for(a.n, 256);
    if (op == 0) binop_kernel<0><<<grid, 256, 0, s>>>(a, b);
    else if (op == 1) binop_kernel<1><<<grid, 256, 0, s>>>(a, b);
    else binop_kernel<2><<<grid, 256, 0, s>>>(a, b);
    return hipGetLastError();
}
hipError_t launch_prepare(hipStream_t s, float *out, const float *x, const float *w, uint32_t n) {
    prepare_kernel<<<(n + 255) / 256, 256, 0, s>>>(out, x, w, n);
    return hipGetLastError();
}
hipError_t launch_silu(hipStream_t s, VecView a, VecView b) {
    silu_kernel<<<grid_for(a.n, 256), 256, 0, s>>>(a, b);
    return hipGetLastError();
}
hipError_t launch_silu_parts(hipStream_t s, float *a, const float *b, uint32_t n, uint32_t nparts, uint32_t part, int *split_flag, uint32_t ntokens) {
    if (n % 4 || part % 4 || (((uintptr_t)a | (uintptr_t)b) & 15)) return hipErrorInvalidValue;
    silu_parts_kernel<<<grid_for(n / 4, 256), 256, 0, s>>>((float4 *)a, (const float4 *)b, n / 4, nparts, part / 4, split_flag, ntokens);
    return hipGetLastError();
}
hipError_t launch_gelu_quads(hipStream_t s, float *a, uint32_t n, uint32_t ntokens, int *split_flag) {
    if (n % 4 || ((uintptr_t)a & 15) || ntokens == 0 || ntokens > 32) return hipErrorInvalidValue;
    gelu_quads_kernel<<<grid_for(n / 4, 256), 256, 0, s>>>((float4 *)a, n / 4, ntokens, split_flag);
    return hipGetLastError();
}
hipError_t launch_gelu(hipStream_t s, VecView a) {
    gelu_kernel<<<grid_for(a.n, 256), 256, 0, s>>>(a);
    return hipGetLastError();
}
hipError_t launch_rope(hipStream_t s, int variant, const slai_rope_config *cfg_dev, VecView q, VecView k) {
    rope_kernel<<<(q.n / 2 + 255) / 256, 256, 0, s>>>(variant, cfg_dev, q, k);
    return hipGetLastError();
}
hipError_t launch_attn_mask(hipStream_t s, const slai_attn_params *params_dev, float *attn, uint32_t nthreads) {
    if (!nthreads) return hipSuccess;
    attn_mask_kernel<<<(nthreads + 255) / 256, 256, 0, s>>>(params_dev, attn, nthreads);
    return hipGetLastError();
}
hipError_t launch_softmax_cols(hipStream_t s, View4 m) {
    dim3 grid(m.size[1], m.size[2], m.size[3]);
    softmax_cols_kernel<<<grid, 256, 0, s>>>(m);
    return hipGetLastError();
}
hipError_t launch_matmul_f32(hipStream_t s, View4 out, View4 a, View4 b, int a_mode, int b_mode) {
    const uint32_t inner = a_mode == SLAI_MODE_N ? a.size[1] : a.size[0];
    const size_t total = (size_t)out.size[0] * out.size[1] * out.size[2] * out.size[3];
    if (!total) return hipSuccess;
    const size_t blocks = (total * 64 + 255) / 256;
    matmul_f32_kernel<<<(uint32_t)blocks, 256, 0, s>>>(out, a, b, a_mode, b_mode, inner);
    return hipGetLastError();
}
hipError_t launch_argmax(hipStream_t s, const float *v, uint32_t n, int *out_index, DecodeState *decode, const int *prompt,
                         int *out_tokens) {
    argmax_kernel<<<1, 1024, 0, s>>>(v, n, out_index, decode, prompt, out_tokens);
    return hipGetLastError();
}

}  // namespace slai
