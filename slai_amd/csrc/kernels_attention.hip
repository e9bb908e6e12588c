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
#include "device_util.h"
#include "quant_formats.h"
#include <float.h>

namespace slai {
namespace {

constexpr int ATT_THREADS = 256;
constexpr int MAX_HS = 256;

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

// binary16 <-> binary32 with the hardware converters (round to nearest even, subnormals kept): one instruction per
// value instead of the bit-level routine the weight decoders share with the host.  Finite values convert identically.
__device__ __forceinline__ float h2f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f2h(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

template <bool F16> struct KV;
template <> struct KV<true> {
    using T = uint16_t;
    __device__ static float2 load2(const T *p) { uint32_t w = *reinterpret_cast<const uint32_t *>(p); return make_float2(h2f((uint16_t)(w & 0xffffu)), h2f((uint16_t)(w >> 16))); }
    __device__ static float round(float v) { return h2f(f2h(v)); }
    __device__ static void store(T *p, float v) { *p = f2h(v); }
};
template <> struct KV<false> {
    using T = float;
    __device__ static float2 load2(const T *p) { return *reinterpret_cast<const float2 *>(p); }
    __device__ static float round(float v) { return v; }
    __device__ static void store(T *p, float v) { *p = v; }
};

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

// ---- the same computation for head sizes 64 and 128, organised around 16-byte loads with many of them in flight:
// scores with 4 lanes per position (each lane a contiguous quarter of the head), values with one lane per 8
// elements.  Every wave runs a softmax of its own over the positions it owns (running max and rescaling), so the
// only workgroup barriers are the one after q is rotated and the one before the waves are merged.  NT = 512 serves
// one workgroup per head over the whole context (no combine pass; short contexts: measured faster than 256 or 1024
// threads), NT = 256 the split form.
template <bool F16> struct Vec8;
template <> struct Vec8<true> {   // 8 f16 = 16 bytes
    struct Raw { uint4 w; };
    __device__ static Raw load_raw(const uint16_t *p) { return Raw{*reinterpret_cast<const uint4 *>(p)}; }
    __device__ static void decode(const Raw &r, float (&o)[8]) {
        const uint32_t u[4] = {r.w.x, r.w.y, r.w.z, r.w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[2 * i] = h2f((uint16_t)(u[i] & 0xffffu)); o[2 * i + 1] = h2f((uint16_t)(u[i] >> 16)); }
    }
    __device__ static void load(const uint16_t *p, float (&o)[8]) {
        const uint4 w = *reinterpret_cast<const uint4 *>(p);
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[2 * i] = h2f((uint16_t)(u[i] & 0xffffu)); o[2 * i + 1] = h2f((uint16_t)(u[i] >> 16)); }
    }
};
template <> struct Vec8<false> {  // 8 f32 = 32 bytes
    struct Raw { float4 a, b; };
    __device__ static Raw load_raw(const float *p) { return Raw{*reinterpret_cast<const float4 *>(p), *reinterpret_cast<const float4 *>(p + 4)}; }
    __device__ static void decode(const Raw &r, float (&o)[8]) {
        o[0] = r.a.x; o[1] = r.a.y; o[2] = r.a.z; o[3] = r.a.w; o[4] = r.b.x; o[5] = r.b.y; o[6] = r.b.z; o[7] = r.b.w;
    }
    __device__ static void load(const float *p, float (&o)[8]) {
        const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
};

template <bool F16, int NT, int HS, bool SINGLE>
__global__ void __launch_bounds__(NT) attn_fast_kernel(AttnLaunch a, uint32_t max_split_len) {
    touch_kernel_arguments<sizeof(AttnLaunch) + 8>();
    using C = KV<F16>;
    using CT = typename C::T;
    constexpr int NW = NT / 64;
    constexpr int EPL = HS / 4;                   // elements per lane in the score phase
    constexpr int LPP = HS / 8;                   // lanes per position in the value phase
    __shared__ float sq[HS], sk[HS], sv[HS];
    __shared__ float sred[NW], sred2[NW];
    __shared__ float sacc[NW][LPP * 8];           // per-wave partial outputs (= HS floats per wave)

    const uint32_t h = blockIdx.x, split = SINGLE ? 0 : blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t kvh = h / a.kv_mul;
    // SINGLE: one workgroup per head covers the whole context
    const uint32_t pos = *a.pos_ptr;
    const uint32_t T = pos + 1;
    const uint32_t chunk = SINGLE ? T : (T + a.n_splits - 1) / a.n_splits;
    const uint32_t t0 = SINGLE ? 0 : split * chunk;
    const uint32_t t1 = SINGLE ? T : min(T, t0 + chunk);
    CT *kc = reinterpret_cast<CT *>(a.kcache), *vc = reinterpret_cast<CT *>(a.vcache);
    const size_t hoff = (size_t)kvh * HS;
    const bool fresh = a.knew != nullptr;
    const bool own_new = SINGLE ? fresh : (fresh && t0 <= pos && pos < t1);

    // ---- requests first: the query pair of this thread (with the fresh key / value and the RoPE frequency), then the
    // first pass of keys and values.  Nothing below depends on anything but the position. ----------------------------
    uint32_t e0 = 0, e1 = 1;
    float q0 = 0.0f, q1 = 0.0f, k0 = 0.0f, k1 = 0.0f, v0 = 0.0f, v1 = 0.0f, theta = 0.0f;
    const bool rot = fresh && a.rope_variant >= 0;             // GPT-2 has learned positions: no rotation
    if (tid < HS / 2) {
        const uint32_t i = tid;
        if (a.rope_variant == SLAI_ROPE_NEOX) { e0 = i; e1 = i + HS / 2; } else { e0 = 2 * i; e1 = 2 * i + 1; }
        q0 = a.q[(size_t)h * HS + e0]; q1 = a.q[(size_t)h * HS + e1];
        if (fresh) {
            if (a.qbias) { q0 += a.qbias[(size_t)h * HS + e0]; q1 += a.qbias[(size_t)h * HS + e1]; }
            if (rot && a.rope_theta) theta = a.rope_theta[i];
            if (own_new) {
                k0 = a.knew[hoff + e0]; k1 = a.knew[hoff + e1];
                v0 = a.vnew[hoff + e0]; v1 = a.vnew[hoff + e1];
                if (a.kbias) { k0 += a.kbias[hoff + e0]; k1 += a.kbias[hoff + e1]; }
                if (a.vbias) { v0 += a.vbias[hoff + e0]; v1 += a.vbias[hoff + e1]; }
            }
        }
    }
    // ---- the first pass of keys and values is requested before anything else is computed: they depend on nothing
    // but the position, and their latency then overlaps the q load and the RoPE.  A pass is NT/4 positions; wave w
    // owns positions 16w..16w+15 of it for both the scores (4 lanes per position) and the values (LPP lanes per
    // position, PW positions per sub-pass), so nothing but the final merge crosses waves. -----------------------
    constexpr int PW = 64 / LPP;                  // positions per value sub-pass of a wave
    constexpr int NU = 16 / PW;                   // value sub-passes per pass
    const uint32_t sub = tid & 3;
    const uint32_t wpos = wave * 16;
    const uint32_t vgl = lane / LPP, ve = (lane % LPP) * 8;
    typename Vec8<F16>::Raw kv0[EPL / 8], vv0[NU];            // kept undecoded: fewer registers while they wait
    {
        const uint32_t t = t0 + tid / 4;
        // the fresh row comes from LDS later; lanes without a position read a valid address and are masked
        const uint32_t tc = (t < t1 && !(own_new && t == pos)) ? t : t0;
        const CT *kp = kc + (size_t)tc * a.kv_dim + hoff + sub * EPL;
#pragma unroll
        for (int j = 0; j < EPL / 8; ++j) kv0[j] = Vec8<F16>::load_raw(kp + 8 * j);
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const uint32_t tv = t0 + wpos + u * PW + vgl;
            const uint32_t tvc = (tv < t1 && !(own_new && tv == pos)) ? tv : t0;
            vv0[u] = Vec8<F16>::load_raw(vc + (size_t)tvc * a.kv_dim + hoff + ve);
        }
    }

    // ---- q (and the fresh k/v) into LDS, rotated (rope.slang:27-84) ------------------------------------------------
    if (tid < HS / 2) {
        if (fresh) {
            if (rot) {
                // rope.slang:36-39: the angle depends on (2*i) mod head_size for both variants; the frequencies
                // base^(-(2i mod hs)/hs) come from a table built once with the same powf
                if (!a.rope_theta) theta = powf(a.rope_base, -(float)((2 * tid) % HS) / (float)HS);
                const float m_theta = (float)pos * theta;
                float c, sn;
                sincosf(m_theta, &sn, &c);
                const float r0 = c * q0 - sn * q1, r1 = sn * q0 + c * q1;
                q0 = r0; q1 = r1;
                const float kr0 = c * k0 - sn * k1, kr1 = sn * k0 + c * k1;
                k0 = kr0; k1 = kr1;
            }
            if (own_new) {
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

    // ---- per wave, pass by pass: scores of 16 positions, running softmax (max m, sum, rescaled outputs), then the
    // weighted values of the same 16 positions.  The next pass's keys and values are requested before the current
    // pass is used. -----------------------------------------------------------------------------------------------
    float qr[EPL];
#pragma unroll
    for (int j = 0; j < EPL; ++j) qr[j] = sq[sub * EPL + j];
    const float root = sqrtf((float)HS);
    float m = -FLT_MAX, lsum = 0.0f;
    float o[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t tb = t0; tb < t1; tb += NT / 4) {           // uniform trip count: the shuffles below need whole waves
        const uint32_t t = tb + tid / 4;
        const bool live = t < t1;
        const bool use_new = own_new && live && t == pos;    // its cache row is being written by this very launch
        typename Vec8<F16>::Raw nxt[EPL / 8] = {}, nxtv[NU] = {};
        if (tb + NT / 4 < t1) {                               // (uniform) there is a next pass
            const uint32_t tn = t + NT / 4;
            const uint32_t tnc = (tn < t1 && !(own_new && tn == pos)) ? tn : t0;
            const CT *kp = kc + (size_t)tnc * a.kv_dim + hoff + sub * EPL;
#pragma unroll
            for (int j = 0; j < EPL / 8; ++j) nxt[j] = Vec8<F16>::load_raw(kp + 8 * j);
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const uint32_t tv = tb + NT / 4 + wpos + u * PW + vgl;
                const uint32_t tvc = (tv < t1 && !(own_new && tv == pos)) ? tv : t0;
                nxtv[u] = Vec8<F16>::load_raw(vc + (size_t)tvc * a.kv_dim + hoff + ve);
            }
        }
        float kv[EPL];
#pragma unroll
        for (int j = 0; j < EPL / 8; ++j) {
            float tmp[8];
            Vec8<F16>::decode(kv0[j], tmp);
#pragma unroll
            for (int q = 0; q < 8; ++q) kv[8 * j + q] = tmp[q];
        }
        if (use_new) {
#pragma unroll
            for (int j = 0; j < EPL; ++j) kv[j] = sk[sub * EPL + j];
        }
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) part = fmaf(qr[j], kv[j], part);
        part += __shfl_xor(part, 1, 64);
        part += __shfl_xor(part, 2, 64);
        const float sc = live ? part / root : -FLT_MAX;      // cpu.rs:521 `score /= sqrt(head_size)`
        const float mn = fmaxf(m, wave_max(sc));
        const float resc = expf(m - mn);                     // 0 on the first live pass, 1 while nothing was live
        const float pr = live ? expf(sc - mn) : 0.0f;
        lsum = fmaf(lsum, resc, sub == 0 ? pr : 0.0f);
#pragma unroll
        for (int q = 0; q < 8; ++q) o[q] *= resc;
        m = mn;
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const uint32_t tv = tb + wpos + u * PW + vgl;
            const float pw = __shfl(pr, 4 * (u * PW + vgl), 64);      // 0 for positions past the end
            float vv[8];
            Vec8<F16>::decode(vv0[u], vv);
            if (own_new && tv == pos) {
#pragma unroll
                for (int q = 0; q < 8; ++q) vv[q] = sv[ve + q];
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) o[q] = fmaf(pw, vv[q], o[q]);
        }
#pragma unroll
        for (int j = 0; j < EPL / 8; ++j) kv0[j] = nxt[j];
#pragma unroll
        for (int u = 0; u < NU; ++u) vv0[u] = nxtv[u];
    }
    lsum = wave_sum(lsum);
    // lanes of a wave that hold the same elements: PW position groups per wave
#pragma unroll
    for (int msk = LPP; msk < 64; msk <<= 1) {
#pragma unroll
        for (int q = 0; q < 8; ++q) o[q] += __shfl_xor(o[q], msk, 64);
    }
    if (lane < LPP) {
#pragma unroll
        for (int q = 0; q < 8; ++q) sacc[wave][lane * 8 + q] = o[q];
    }
    if (lane == 0) { sred[wave] = m; sred2[wave] = lsum; }
    __syncthreads();
    // ---- merge the waves: each holds (max, sum, outputs) over its own positions ------------------------------------
    if (tid < HS) {
        float M = sred[0];
#pragma unroll
        for (int w = 1; w < NW; ++w) M = fmaxf(M, sred[w]);
        float r = 0.0f, l = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float f = expf(sred[w] - M);               // a wave that saw no position has sum 0 and outputs 0
            r = fmaf(sacc[w][tid], f, r);
            l = fmaf(sred2[w], f, l);
        }
        if (a.n_splits == 1) {
            a.out[(size_t)h * HS + tid] = r / l;
        } else {
            float *po = a.scratch + ((size_t)h * a.n_splits + split) * (HS + 2);
            po[tid] = r;
            if (tid == 0) { po[HS] = (t1 > t0) ? M : -FLT_MAX; po[HS + 1] = (t1 > t0) ? l : 0.0f; }
        }
    }
}

__global__ void rope_theta_kernel(float *out, uint32_t hs, float base) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < hs / 2) out[i] = powf(base, -(float)((2 * i) % hs) / (float)hs);      // rope.slang:36-38
}

// grid = n_heads, block = 128: merge the per-split (max, sum, unnormalised output) triples.
// n_splits <= 64: one lane per split computes its weight exp(m_s - M) / L, then every thread
// accumulates its output elements with independent loads.
__global__ void __launch_bounds__(128) attn_combine_kernel(const float *scratch, float *out, uint32_t hs, uint32_t n_splits) {
    __shared__ float sw[64];
    const uint32_t h = blockIdx.x, tid = threadIdx.x;
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
    for (uint32_t e = tid; e < hs; e += blockDim.x) {
        float acc = 0.0f;
#pragma unroll 8
        for (uint32_t s = 0; s < n_splits; ++s) acc = fmaf(sw[s], base[(size_t)s * (hs + 2) + e], acc);
        out[(size_t)h * hs + e] = acc;
    }
}

}  // namespace

hipError_t launch_rope_theta(hipStream_t s, float *out, uint32_t head_size, float base) {
    rope_theta_kernel<<<(head_size / 2 + 63) / 64, 64, 0, s>>>(out, head_size, base);
    return hipGetLastError();
}

size_t attention_scratch_floats(uint32_t n_heads, uint32_t head_size, uint32_t n_splits) {
    return n_splits > 1 ? (size_t)n_heads * n_splits * (head_size + 2) : 0;
}

hipError_t launch_attention(hipStream_t s, const AttnLaunch &a) {
    if (a.head_size > MAX_HS || a.head_size % 2 || a.head_size / 2 > ATT_THREADS || a.n_splits == 0 || a.n_splits > 64) return hipErrorInvalidValue;
    const uint32_t max_split_len = (a.seq_len + a.n_splits - 1) / a.n_splits;
    dim3 grid(a.n_heads, a.n_splits);
    const bool fast = (a.head_size == 64 || a.head_size == 128) && a.kv_dim % 8 == 0;
    const size_t smem = fast ? 0 : (size_t)max_split_len * sizeof(float);   // the general kernel keeps its scores in LDS
    if (smem > 48 * 1024) return hipErrorInvalidValue;
    if (fast && a.n_splits == 1) {
        if (a.head_size == 128) { if (a.kv_f16) attn_fast_kernel<true, 512, 128, true><<<grid, 512, smem, s>>>(a, max_split_len); else attn_fast_kernel<false, 512, 128, true><<<grid, 512, smem, s>>>(a, max_split_len); }
        else { if (a.kv_f16) attn_fast_kernel<true, 512, 64, true><<<grid, 512, smem, s>>>(a, max_split_len); else attn_fast_kernel<false, 512, 64, true><<<grid, 512, smem, s>>>(a, max_split_len); }
    } else if (fast) {
        if (a.head_size == 128) { if (a.kv_f16) attn_fast_kernel<true, 256, 128, false><<<grid, 256, smem, s>>>(a, max_split_len); else attn_fast_kernel<false, 256, 128, false><<<grid, 256, smem, s>>>(a, max_split_len); }
        else { if (a.kv_f16) attn_fast_kernel<true, 256, 64, false><<<grid, 256, smem, s>>>(a, max_split_len); else attn_fast_kernel<false, 256, 64, false><<<grid, 256, smem, s>>>(a, max_split_len); }
    } else if (a.kv_f16) attn_kernel<true><<<grid, ATT_THREADS, smem, s>>>(a, max_split_len);
    else attn_kernel<false><<<grid, ATT_THREADS, smem, s>>>(a, max_split_len);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (a.n_splits > 1) {
        attn_combine_kernel<<<a.n_heads, 128, 0, s>>>(a.scratch, a.out, a.head_size, a.n_splits);
        e = hipGetLastError();
    }
    return e;
}

}  // namespace slai
