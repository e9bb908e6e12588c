// KV-cache attention for single-token decode: QK^T, softmax, .V in one kernel, split over the
// sequence (flash-decoding) with a small combine kernel when more than one split is used.
//
// Reproduces `BatchedMultiqueryAttention` (crates/slai/src/ops/batched_multiquery_attention.rs:32-156,
// CPU form models/llama2/cpu.rs:488-539): per query head h (kv head h / kv_mul)
//   s_t = q_h . K[t]_h / sqrt(head_size), t <= pos;  p = softmax(s);  out_h = sum_t p_t V[t]_h
// which the reference issues as four launches (gemv, mask/scale, softmax, gemv) with the score
// matrix round-tripping through memory.  Exactly pos+1 positions are read (the reference rounds
// up to a multiple of 4 and reads uninitialised cache columns).
//
// Cache layout is the reference's: [kv_dim x seq_len] column-major, i.e. one position = kv_dim
// contiguous values (transformer.rs:87-106), f32 or f16.
//
// In the model path the kernel also performs RoPE (rope.slang:27-84) on q and on the fresh key
// and writes the fresh key/value into the cache, so Q/K/V leave the projection GEMV exactly once.
#include "common.h"
#include <cstdlib>
#include "device_util.h"
#include "attention_fast.h"
#include "quant_formats.h"
#include <float.h>
#include <mutex>

// Scratch of slai_attention_static (the entry point that allocates nothing): the per-split partial results of the
// split attention kernel.  Every GPU the library runs on holds its own copy of the array, at its own address, until the
// process ends; in host code the name is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t SLAI_ATTENTION_STATIC_FLOATS = 512 * 1024;     // 2 MiB
static __device__ __align__(256) float scratch[SLAI_ATTENTION_STATIC_FLOATS];

namespace slai {
namespace {

constexpr int ATT_THREADS = 256;
constexpr int MAX_HS = 256;

using namespace attn;

// grid = (n_heads, n_splits), block = ATT_THREADS.  Dynamic LDS: scores for one split.
template <bool F16>
__global__ void __launch_bounds__(ATT_THREADS) attn_kernel(AttnLaunch a, uint32_t max_split_len) {
    touch_kernel_arguments<sizeof(AttnLaunch) + 8>();
    using C = KV<F16>;
    using CT = typename C::T;
    extern __shared__ float sscore[];             // [max_split_len]
    __shared__ float sq[MAX_HS], sk[MAX_HS], sv[MAX_HS];
    __shared__ float sred[ATT_THREADS / 64];
    __shared__ float sacc[ATT_THREADS * 2];  // cross-group reduction of the output

    const uint32_t h = blockIdx.x, split = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t hs = a.head_size, kvh = h / a.kv_mul;
    const uint32_t pos = *a.pos_ptr;
    const uint32_t T = pos + 1;
    const uint32_t chunk = (T + a.n_splits - 1) / a.n_splits;
    const uint32_t t0 = split * chunk;
    const uint32_t t1 = min(T, t0 + chunk);
    CT *kc = reinterpret_cast<CT *>(a.kcache), *vc = reinterpret_cast<CT *>(a.vcache);
    const size_t hoff = (size_t)kvh * hs;
    const bool fresh = a.knew != nullptr;
    const bool own_new = fresh && t0 <= pos && pos < t1;   // this split covers the current position

    // ---- q (and the fresh k/v) into LDS, with bias and RoPE when fused -----------------------
    if (tid < hs / 2) {
        const uint32_t i = tid;   // pair index inside the head
        uint32_t e0, e1;
        if (a.rope_variant == SLAI_ROPE_NEOX) { e0 = i; e1 = i + hs / 2; } else { e0 = 2 * i; e1 = 2 * i + 1; }
        float q0 = a.q[(size_t)h * hs + e0], q1 = a.q[(size_t)h * hs + e1];
        if (fresh) {
            if (a.qbias) { q0 += a.qbias[(size_t)h * hs + e0]; q1 += a.qbias[(size_t)h * hs + e1]; }
            const bool rot = a.rope_variant >= 0;   // GPT-2 has learned positions: no rotation
            float c = 1.0f, s = 0.0f;
            if (rot) {
                // rope.slang:36-39: the angle depends on (2*i) mod head_size for both variants
                const float head_dim = (float)((2 * i) % hs);
                const float theta = powf(a.rope_base, -head_dim / (float)hs);
                const float m_theta = (float)pos * theta;
                c = cosf(m_theta); s = sinf(m_theta);
                const float r0 = c * q0 - s * q1, r1 = s * q0 + c * q1;
                q0 = r0; q1 = r1;
            }
            if (own_new) {
                float k0 = a.knew[hoff + e0], k1 = a.knew[hoff + e1];
                float v0 = a.vnew[hoff + e0], v1 = a.vnew[hoff + e1];
                if (a.kbias) { k0 += a.kbias[hoff + e0]; k1 += a.kbias[hoff + e1]; }
                if (a.vbias) { v0 += a.vbias[hoff + e0]; v1 += a.vbias[hoff + e1]; }
                if (rot) {
                    const float kr0 = c * k0 - s * k1, kr1 = s * k0 + c * k1;
                    k0 = kr0; k1 = kr1;
                }
                sk[e0] = C::round(k0); sk[e1] = C::round(k1);
                sv[e0] = C::round(v0); sv[e1] = C::round(v1);
                // several query heads share a kv head: the first of the group writes the cache
                if (h % a.kv_mul == 0) {
                    CT *kd = kc + (size_t)pos * a.kv_dim + hoff, *vd = vc + (size_t)pos * a.kv_dim + hoff;
                    C::store(kd + e0, k0); C::store(kd + e1, k1);
                    C::store(vd + e0, v0); C::store(vd + e1, v1);
                }
            }
        }
        sq[e0] = q0; sq[e1] = q1;
    }
    __syncthreads();

    // ---- scores: one wave per position, lanes over element pairs ----------------------------------
    const float inv_sqrt = sqrtf((float)hs);
    float lmax = -FLT_MAX;
    for (uint32_t t = t0 + wave; t < t1; t += ATT_THREADS / 64) {
        float part = 0.0f;
        const bool use_new = own_new && t == pos;
        for (uint32_t e = 2 * lane; e < hs; e += 128) {
            float2 kv;
            if (use_new) kv = make_float2(sk[e], sk[e + 1]);
            else kv = C::load2(kc + (size_t)t * a.kv_dim + hoff + e);
            part = fmaf(sq[e], kv.x, part);
            part = fmaf(sq[e + 1], kv.y, part);
        }
        part = wave_sum(part);
        const float sc = part / inv_sqrt;       // cpu.rs:521 `score /= sqrt(head_size)`
        if (lane == 0) sscore[t - t0] = sc;
        lmax = fmaxf(lmax, sc);
    }
    // block max
    if (lane == 0) sred[wave] = lmax;
    __syncthreads();
    float m = sred[0];
#pragma unroll
    for (int w = 1; w < ATT_THREADS / 64; ++w) m = fmaxf(m, sred[w]);
    __syncthreads();

    // ---- exp and sum ------------------------------------------------------------------------------
    float lsum = 0.0f;
    for (uint32_t t = t0 + tid; t < t1; t += ATT_THREADS) {
        const float e = expf(sscore[t - t0] - m);
        sscore[t - t0] = e;
        lsum += e;
    }
    lsum = wave_sum(lsum);
    if (lane == 0) sred[wave] = lsum;
    __syncthreads();
    float l = 0.0f;
#pragma unroll
    for (int w = 0; w < ATT_THREADS / 64; ++w) l += sred[w];

    // ---- weighted sum of values: thread = (position group g, element pair i) ------------------------
    const uint32_t pairs = hs / 2;
    const uint32_t groups = ATT_THREADS / pairs ? ATT_THREADS / pairs : 1;
    const uint32_t g = tid / pairs, i2 = tid % pairs;
    float o0 = 0.0f, o1 = 0.0f;
    if (g < groups && pairs <= ATT_THREADS) {
        for (uint32_t t = t0 + g; t < t1; t += groups) {
            const float p = sscore[t - t0];
            float2 vv;
            if (own_new && t == pos) vv = make_float2(sv[2 * i2], sv[2 * i2 + 1]);
            else vv = C::load2(vc + (size_t)t * a.kv_dim + hoff + 2 * i2);
            o0 = fmaf(p, vv.x, o0);
            o1 = fmaf(p, vv.y, o1);
        }
    }
    sacc[2 * tid] = o0; sacc[2 * tid + 1] = o1;
    __syncthreads();
    if (tid < pairs) {
        float r0 = 0.0f, r1 = 0.0f;
        for (uint32_t gg = 0; gg < groups; ++gg) { r0 += sacc[2 * (gg * pairs + tid)]; r1 += sacc[2 * (gg * pairs + tid) + 1]; }
        if (a.n_splits == 1) {
            a.out[(size_t)h * hs + 2 * tid] = r0 / l;
            a.out[(size_t)h * hs + 2 * tid + 1] = r1 / l;
        } else {
            float *po = a.scratch + ((size_t)h * a.n_splits + split) * (hs + 2);
            po[2 * tid] = r0; po[2 * tid + 1] = r1;
            if (tid == 0) { po[hs] = (t1 > t0) ? m : -FLT_MAX; po[hs + 1] = (t1 > t0) ? l : 0.0f; }
        }
    }
}

// ---- the fast form (attention_fast.h) as a kernel of its own: grid = (n_heads, n_splits), block = NT
// Grouped-query models (`grouped`: a one-dimensional grid): the kv_mul query heads of a kv head read the same cache rows
// (batched_multiquery_attention.rs:48-98 serves them from one product).  Workgroup b of a launch runs on die b mod 8, and
// a die's workgroups share its L2, so the workgroups of one (kv head, split) are given indices 8 apart: they run at the
// same time on one die, the rows come from memory once, and the other kv_mul - 1 workgroups find them in that L2.
//   b = (key mod 8) + 8 * (j + kv_mul * (key / 8)),  key = kv head + n_kv_heads * split,  j = query head within the group
__device__ __forceinline__ void combine_head(const float *scratch, float *out, uint32_t hs, uint32_t n_splits, uint32_t h, uint32_t tid, uint32_t nthreads, float *sw);

template <bool F16, int NT, int HS, bool SINGLE>
__global__ void __launch_bounds__(NT) attn_fast_kernel(AttnLaunch a, uint32_t max_split_len, uint32_t grouped) {
    touch_kernel_arguments<sizeof(AttnLaunch) + 8>();
    uint32_t h = blockIdx.x, split = SINGLE ? 0u : blockIdx.y;
    if (grouped) {
        const uint32_t b = blockIdx.x, slot = b >> 3, j = slot % a.kv_mul, key = (b & 7u) + 8u * (slot / a.kv_mul);
        const uint32_t n_kv = a.n_heads / a.kv_mul;
        if (key >= n_kv * a.n_splits) return;                    // (the grid is rounded up to whole dies)
        h = (key % n_kv) * a.kv_mul + j;
        split = key / n_kv;
    }
    // (the split form on a model without grouped queries reads every cached row exactly once: non-temporal requests)
    if (!SINGLE && F16 && a.kv_mul == 1) attn_fast_body<F16, NT, HS, SINGLE, false, 4, false, true>(a, h, split, threadIdx.x, []() {});
    else attn_fast_body<F16, NT, HS, SINGLE, false>(a, h, split, threadIdx.x, []() {});
    if constexpr (!SINGLE) {
        // The last of a head's splits merges them: every workgroup waits until its partial result is in the die's L2
        // (all splits of the head run on this die: the launcher has checked), then counts itself in with an atomic that
        // executes there and returns the count; the one that completes it finds every partial result in that L2.
        if (a.combine_counters) {
            __shared__ uint32_t last;
            __shared__ float sw[64];
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (threadIdx.x == 0) {
                uint32_t *counter = a.combine_counters + (size_t)h * 32;
                uint32_t seen;
                const uint32_t one = 1;
                asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=&v"(seen) : "v"(counter), "v"(one) : "memory");
                last = seen + 1 == a.n_splits ? 1u : 0u;
                if (last) *counter = 0u;                               // for the next launch; nobody else touches it any more
            }
            __syncthreads();
            if (last) combine_head(a.scratch, a.out, HS, a.n_splits, h, threadIdx.x, NT, sw);
        }
    }
}
// the size of that grid
static uint32_t grouped_grid(const AttnLaunch &a) {
    const uint32_t keys = (a.n_heads / a.kv_mul) * a.n_splits;
    return 8u * a.kv_mul * ((keys + 7u) / 8u);
}

// A chunk of tokens whose keys and values are already in the caches: grid = (n_heads, tokens), whole context in one
// workgroup; token b reads q + b * q_stride and its position pos_ptr[b], and writes out + b * out_stride or, with
// out_quads, column b of the quad-major matrix `out` ([columns / 4][32 tokens][4], the prompt-chunk GEMM's input; with
// split_flag as f16 head + remainder pairs).
template <bool F16, int HS>
__global__ void __launch_bounds__(512) attn_fast_batch_kernel(AttnLaunch a0, uint32_t q_stride, uint32_t out_stride, uint32_t out_quads, int *split_flag) {
    touch_kernel_arguments<sizeof(AttnLaunch) + 24>();
    AttnLaunch a = a0;
    const uint32_t b = blockIdx.y;
    a.q = a0.q + (size_t)b * q_stride;
    a.out = out_quads ? a0.out : a0.out + (size_t)b * out_stride;
    a.pos_ptr = a0.pos_ptr + b;
    a.knew = nullptr; a.vnew = nullptr;
    attn_fast_body<F16, 512, HS, true, false>(a, blockIdx.x, 0u, threadIdx.x, []() {}, out_quads ? b : 0xffffffffu, out_quads ? split_flag : nullptr);
}

// The bias / RoPE / cache-write part of attn_fast_body for a chunk of tokens, as a launch of its own: a token's
// attention reads the rows of the earlier tokens of its chunk, so all rows are written before any attention starts.
// grid = (n_heads, tokens), block = head_size / 2 (one rotation pair per thread; rope.slang:27-84).
template <bool F16>
__global__ void rope_store_batch_kernel(AttnLaunch a, float *q, const float *k, const float *v, uint32_t q_stride, uint32_t kv_stride,
                                        uint32_t nparts, uint32_t q_part, uint32_t kv_part) {
    using C = KV<F16>;
    using CT = typename C::T;
    const uint32_t h = blockIdx.x, b = blockIdx.y, i = threadIdx.x, HS = a.head_size;
    const uint32_t kvh = h / a.kv_mul;
    const uint32_t pos = a.pos_ptr[b];
    const size_t hoff = (size_t)kvh * HS;
    uint32_t e0, e1;
    if (a.rope_variant == SLAI_ROPE_NEOX) { e0 = i; e1 = i + HS / 2; } else { e0 = 2 * i; e1 = 2 * i + 1; }
    float *qb = q + (size_t)b * q_stride + (size_t)h * HS;
    const float *kb = k + (size_t)b * kv_stride + hoff, *vb = v + (size_t)b * kv_stride + hoff;
    float q0 = qb[e0], q1 = qb[e1];
    float k0 = kb[e0], k1 = kb[e1], v0 = vb[e0], v1 = vb[e1];
    for (uint32_t s = 1; s < nparts; ++s) {                      // partial results of a projection split over its columns
        q0 += qb[(size_t)s * q_part + e0]; q1 += qb[(size_t)s * q_part + e1];
        k0 += kb[(size_t)s * kv_part + e0]; k1 += kb[(size_t)s * kv_part + e1];
        v0 += vb[(size_t)s * kv_part + e0]; v1 += vb[(size_t)s * kv_part + e1];
    }
    if (a.qbias) { q0 += a.qbias[(size_t)h * HS + e0]; q1 += a.qbias[(size_t)h * HS + e1]; }
    if (a.kbias) { k0 += a.kbias[hoff + e0]; k1 += a.kbias[hoff + e1]; }
    if (a.vbias) { v0 += a.vbias[hoff + e0]; v1 += a.vbias[hoff + e1]; }
    if (a.rope_variant >= 0) {
        const float theta = a.rope_theta ? a.rope_theta[i] : powf(a.rope_base, -(float)((2 * i) % HS) / (float)HS);
        const float m_theta = (float)pos * theta;
        float c, sn;
        sincosf(m_theta, &sn, &c);
        const float r0 = c * q0 - sn * q1, r1 = sn * q0 + c * q1;
        q0 = r0; q1 = r1;
        const float kr0 = c * k0 - sn * k1, kr1 = sn * k0 + c * k1;
        k0 = kr0; k1 = kr1;
    }
    qb[e0] = q0; qb[e1] = q1;
    if (h % a.kv_mul == 0) {                                   // several query heads share a kv head: the first of the group writes
        CT *kc = reinterpret_cast<CT *>(a.kcache), *vc = reinterpret_cast<CT *>(a.vcache);
        CT *kd = kc + (size_t)pos * a.kv_dim + hoff, *vd = vc + (size_t)pos * a.kv_dim + hoff;
        C::store(kd + e0, k0); C::store(kd + e1, k1);
        C::store(vd + e0, v0); C::store(vd + e1, v1);
    }
}

__global__ void rope_theta_kernel(float *out, uint32_t hs, float base) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < hs / 2) out[i] = powf(base, -(float)((2 * i) % hs) / (float)hs);      // rope.slang:36-38
}

// grid = n_heads, block = 128: merge the per-split (max, sum, unnormalised output) triples.
// n_splits <= 64: one lane per split computes its weight exp(m_s - M) / L, then every thread
// accumulates its output elements with independent loads.
__device__ __forceinline__ void combine_head(const float *scratch, float *out, uint32_t hs, uint32_t n_splits, uint32_t h, uint32_t tid, uint32_t nthreads, float *sw /* [64], LDS */) {
    const float *base = scratch + (size_t)h * n_splits * (hs + 2);
    if (tid < 64) {
        const bool on = tid < n_splits;
        const float ms = on ? base[(size_t)tid * (hs + 2) + hs] : -FLT_MAX;
        const float ls = on ? base[(size_t)tid * (hs + 2) + hs + 1] : 0.0f;
        const float M = wave_max(ms);
        const float w = ls > 0.0f ? expf(ms - M) : 0.0f;
        const float L = wave_sum(w * ls);
        sw[tid] = w / L;
    }
    __syncthreads();
    for (uint32_t e = tid; e < hs; e += nthreads) {
        float acc = 0.0f;
#pragma unroll 8
        for (uint32_t s = 0; s < n_splits; ++s) acc = fmaf(sw[s], base[(size_t)s * (hs + 2) + e], acc);
        out[(size_t)h * hs + e] = acc;
    }
}
__global__ void __launch_bounds__(128) attn_combine_kernel(const float *scratch, float *out, uint32_t hs, uint32_t n_splits) {
    __shared__ float sw[64];
    combine_head(scratch, out, hs, n_splits, blockIdx.x, threadIdx.x, blockDim.x, sw);
}

}  // namespace

hipError_t launch_rope_theta(hipStream_t s, float *out, uint32_t head_size, float base) {
    rope_theta_kernel<<<(head_size / 2 + 63) / 64, 64, 0, s>>>(out, head_size, base);
    return hipGetLastError();
}

size_t attention_scratch_floats(uint32_t n_heads, uint32_t head_size, uint32_t n_splits) {
    return n_splits > 1 ? (size_t)n_heads * n_splits * (head_size + 2) : 0;
}

hipError_t launch_attention(hipStream_t s, const AttnLaunch &a_in) {
    AttnLaunch a = a_in;
    {
        // The splits of a head merge themselves only in the fast form, and only when all of them run on one die: workgroup
        // (head, split) of the two-dimensional grid has index head + n_heads * split, a (kv head, split) key of the grouped
        // grid lands on die (kv head + n_kv_heads * split) mod 8.
        const bool fast_form = (a.head_size == 64 || a.head_size == 128) && a.kv_dim % 8 == 0;
        static const bool on_die_env = [] { const char *e = getenv("SLAI_GQA_ON_DIE"); return !(e && e[0] == '0'); }();
        const bool grouped_form = fast_form && on_die_env && a.kv_mul > 1 && a.n_heads % a.kv_mul == 0;
        const uint32_t per_die = grouped_form ? a.n_heads / a.kv_mul : a.n_heads;
        if (a.n_splits <= 1 || !fast_form || per_die % 8 != 0) a.combine_counters = nullptr;
    }
    if (a.head_size > MAX_HS || a.head_size % 2 || a.head_size / 2 > ATT_THREADS || a.n_splits == 0 || a.n_splits > 64) return hipErrorInvalidValue;
    const uint32_t max_split_len = (a.seq_len + a.n_splits - 1) / a.n_splits;
    const bool fast = (a.head_size == 64 || a.head_size == 128) && a.kv_dim % 8 == 0;
    // (SLAI_GQA_ON_DIE=0: one workgroup per (query head, split) in plain order, for comparisons)
    static const bool on_die = [] { const char *e = getenv("SLAI_GQA_ON_DIE"); return !(e && e[0] == '0'); }();
    const uint32_t grouped = fast && on_die && a.kv_mul > 1 && a.n_heads % a.kv_mul == 0 ? 1u : 0u;
    dim3 grid(grouped ? grouped_grid(a) : a.n_heads, grouped ? 1u : a.n_splits);
    const size_t smem = fast ? 0 : (size_t)max_split_len * sizeof(float);   // the general kernel keeps its scores in LDS
    if (smem > 48 * 1024) return hipErrorInvalidValue;
    if (fast && a.n_splits == 1) {
        if (a.head_size == 128) { if (a.kv_f16) attn_fast_kernel<true, 512, 128, true><<<grid, 512, smem, s>>>(a, max_split_len, grouped); else attn_fast_kernel<false, 512, 128, true><<<grid, 512, smem, s>>>(a, max_split_len, grouped); }
        else { if (a.kv_f16) attn_fast_kernel<true, 512, 64, true><<<grid, 512, smem, s>>>(a, max_split_len, grouped); else attn_fast_kernel<false, 512, 64, true><<<grid, 512, smem, s>>>(a, max_split_len, grouped); }
    } else if (fast) {
        if (a.head_size == 128) { if (a.kv_f16) attn_fast_kernel<true, 256, 128, false><<<grid, 256, smem, s>>>(a, max_split_len, grouped); else attn_fast_kernel<false, 256, 128, false><<<grid, 256, smem, s>>>(a, max_split_len, grouped); }
        else { if (a.kv_f16) attn_fast_kernel<true, 256, 64, false><<<grid, 256, smem, s>>>(a, max_split_len, grouped); else attn_fast_kernel<false, 256, 64, false><<<grid, 256, smem, s>>>(a, max_split_len, grouped); }
    } else if (a.kv_f16) attn_kernel<true><<<grid, ATT_THREADS, smem, s>>>(a, max_split_len);
    else attn_kernel<false><<<grid, ATT_THREADS, smem, s>>>(a, max_split_len);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (a.n_splits > 1 && !a.combine_counters) {
        attn_combine_kernel<<<a.n_heads, 128, 0, s>>>(a.scratch, a.out, a.head_size, a.n_splits);
        e = hipGetLastError();
    }
    return e;
}

namespace {
constexpr int STATIC_MAX_DEVICES = 64;
float *static_scratch_ptr[STATIC_MAX_DEVICES];      // device d's address of `scratch`; set by attention_static_setup
std::mutex static_scratch_mutex;
}  // namespace

hipError_t attention_static_setup(int device) {
    if (device < 0 || device >= STATIC_MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(static_scratch_mutex);
    if (static_scratch_ptr[device]) return hipSuccess;
    float *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!ptr) return hipErrorInvalidSymbol;
    static_scratch_ptr[device] = ptr;
    return hipSuccess;
}

hipError_t launch_attention_batch(hipStream_t s, const AttnLaunch &a, uint32_t n, uint32_t q_stride, uint32_t out_stride, bool out_quads, int *split_flag) {
    if ((a.head_size != 64 && a.head_size != 128) || a.kv_dim % 8 || a.knew || a.vnew || n == 0 || n > 65535 || (out_quads && n > 32)) return hipErrorInvalidValue;
    const uint32_t oq = out_quads ? 1u : 0u;
    dim3 grid(a.n_heads, n);
    if (a.head_size == 128) {
        if (a.kv_f16) attn_fast_batch_kernel<true, 128><<<grid, 512, 0, s>>>(a, q_stride, out_stride, oq, split_flag);
        else attn_fast_batch_kernel<false, 128><<<grid, 512, 0, s>>>(a, q_stride, out_stride, oq, split_flag);
    } else {
        if (a.kv_f16) attn_fast_batch_kernel<true, 64><<<grid, 512, 0, s>>>(a, q_stride, out_stride, oq, split_flag);
        else attn_fast_batch_kernel<false, 64><<<grid, 512, 0, s>>>(a, q_stride, out_stride, oq, split_flag);
    }
    return hipGetLastError();
}

hipError_t launch_rope_store_batch(hipStream_t s, const AttnLaunch &a, float *q, const float *k, const float *v, uint32_t n, uint32_t q_stride, uint32_t kv_stride,
                                   uint32_t nparts, uint32_t q_part, uint32_t kv_part) {
    if (a.head_size % 2 || a.head_size / 2 > 1024 || n == 0 || n > 65535 || a.kv_mul == 0 || nparts == 0) return hipErrorInvalidValue;
    dim3 grid(a.n_heads, n);
    if (a.kv_f16) rope_store_batch_kernel<true><<<grid, a.head_size / 2, 0, s>>>(a, q, k, v, q_stride, kv_stride, nparts, q_part, kv_part);
    else rope_store_batch_kernel<false><<<grid, a.head_size / 2, 0, s>>>(a, q, k, v, q_stride, kv_stride, nparts, q_part, kv_part);
    return hipGetLastError();
}

}  // namespace slai

// slai_attention for callers that must not allocate (code under graph capture, tight serving loops): the same kernels
// with the split partials in this device's copy of the static array.  No hipMalloc / hipFree on any path; shapes whose
// partials do not fit are refused.  Calls on one GPU share the array, so calls that overlap in time (two contexts, two
// streams) race; nothing in it has to start at zero: every partial the combine pass reads is written by the same call.
SLAI_EXPORT int slai_attention_static(slai_ctx *ctx, const slai_attn_params *params, const slai_buffer *params_gpu, slai_view q,
                                      slai_view key_cache, slai_view value_cache, slai_view att, slai_view xb) {
    using namespace slai;
    (void)att;
    AttnLaunch a{};
    if (int rc = attention_describe(ctx, "slai_attention_static", params, params_gpu, q, key_cache, value_cache, xb, &a)) return rc;
    const size_t need = attention_scratch_floats(a.n_heads, a.head_size, a.n_splits);
    if (need > SLAI_ATTENTION_STATIC_FLOATS)
        return set_error(ctx, SLAI_E_SHAPE, "slai_attention_static: n_heads * splits * (head_size + 2) = " + std::to_string(need) + " floats of partial results exceed the static scratch of " +
                                            std::to_string(SLAI_ATTENTION_STATIC_FLOATS) + " floats; use slai_attention");
    float *ptr = ctx->device >= 0 && ctx->device < STATIC_MAX_DEVICES ? static_scratch_ptr[ctx->device] : nullptr;
    if (!ptr) return set_error(ctx, SLAI_E_STATE, "slai_attention_static: the static scratch of this device was not set up");
    a.scratch = ptr;
    hipError_t e = launch_attention(ctx->stream, a);
    if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, "slai_attention_static: unsupported head size or context length");
    SLAI_HIP_TRY(ctx, e);
    return SLAI_OK;
}
