// Single-token attention for head sizes 64 and 128 as a device function, shared by the stand-alone attention kernel
// and the launch that also computes q, k and v (see kernels_attention.hip for the contract and the reference lines).
#pragma once
#include "common.h"
#include "device_util.h"
#include <float.h>

namespace slai {
namespace attn {

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

// ---- the same computation for head sizes 64 and 128, built on 16-byte loads with many of them in flight:
// scores with 4 lanes per position (each lane a contiguous quarter of the head), values with one lane per 8
// elements.  Every wave runs a softmax of its own over the positions it owns (running max and rescaling), so the
// only workgroup barriers are the one after q is rotated and the one before the waves are merged.  NT = 512 serves
// one workgroup per head over the whole context (no combine pass; short contexts: measured faster than 256 or 1024
// threads), NT = 256 the split form.
template <bool F16> struct Vec8;
template <> struct Vec8<true> {   // 8 f16 = 16 bytes
    struct Raw { uint4 w; };
    // STREAM: with the non-temporal hint -- for rows that this launch reads exactly once and whose line one request covers
    template <bool STREAM = false> __device__ static Raw load_raw(const uint16_t *p) {
        if constexpr (STREAM) {
            typedef uint32_t words4 __attribute__((ext_vector_type(4)));
            const words4 v = __builtin_nontemporal_load(reinterpret_cast<const words4 *>(p));
            Raw r; r.w.x = v.x; r.w.y = v.y; r.w.z = v.z; r.w.w = v.w;
            return r;
        } else {
            return Raw{*reinterpret_cast<const uint4 *>(p)};
        }
    }
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
    template <bool STREAM = false> __device__ static Raw load_raw(const float *p) { return Raw{*reinterpret_cast<const float4 *>(p), *reinterpret_cast<const float4 *>(p + 4)}; }   // (two requests per line: never streamed)
    __device__ static void decode(const Raw &r, float (&o)[8]) {
        o[0] = r.a.x; o[1] = r.a.y; o[2] = r.a.z; o[3] = r.a.w; o[4] = r.b.x; o[5] = r.b.y; o[6] = r.b.z; o[7] = r.b.w;
    }
    __device__ static void load(const float *p, float (&o)[8]) {
        const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
};

// `h`, `split`: head and split of the calling workgroup; `tid`: 0 .. NT-1 (the first NT threads of the workgroup; any
// others must have left the kernel).  `wait_inputs()` is called once, by every thread, before q / knew / vnew are read:
// a launch in which this workgroup's inputs are produced by other workgroups of the same launch blocks there (FUSED:
// the requests for the cache, which depend on nothing but the position, then go first).  `quad_token` (single-split
// form only): write the result as that token's column of a quad-major matrix instead of a plain vector; with
// `split_flag` as f16 head + remainder pairs (split_quad's layout), *split_flag set when a value is beyond f16.
// STREAM: the cached rows are requested with the non-temporal hint (f16 rows of a launch that reads each of them once:
// the split form on a model with as many kv heads as query heads; 19.75 -> 19.1 us per layer at position 4047).
// FLOW: q / knew / vnew were written by other workgroups of this very launch and the result is read by others again:
// they are read and written with the coherent accesses of device_util.h (no cache of this compute unit may serve them).
template <bool F16, int NT, int HS, bool SINGLE, bool FUSED, int KL = 4, bool FLOW = false, bool STREAM = false, class Wait>
__device__ __forceinline__ void attn_fast_body(const AttnLaunch &a, uint32_t h, uint32_t split, uint32_t tid, Wait &&wait_inputs,
                                               uint32_t quad_token = 0xffffffffu, int *split_flag = nullptr) {
    using C = KV<F16>;
    using CT = typename C::T;
    constexpr int NW = NT / 64;
    // KL lanes share a position in the score phase (4, or 8 where registers are scarce: half as many elements per lane)
    constexpr int EPL = HS / KL;                  // elements per lane in the score phase: piece jj (eight of them) is elements
                                                  // 8 KL jj + 8 sub .. + 7, so that the KL lanes of a position ask for 16 KL contiguous
                                                  // bytes (of an f16 cache) in one request, not for 16 bytes each at a stride of 2 EPL
    constexpr int PPW = 64 / KL;                  // positions a wave owns per pass
    constexpr int LPP = HS / 8;                   // lanes per position in the value phase
    __shared__ float sq[HS], sk[HS], sv[HS];
    __shared__ float sred[NW], sred2[NW];
    __shared__ float sacc[NW][LPP * 8];           // per-wave partial outputs (= HS floats per wave)

    const uint32_t lane = tid & 63, wave = tid >> 6;
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
    auto load_inputs = [&]() {
        if (tid < HS / 2) {
            const uint32_t i = tid;
            if (a.rope_variant == SLAI_ROPE_NEOX) { e0 = i; e1 = i + HS / 2; } else { e0 = 2 * i; e1 = 2 * i + 1; }
            if constexpr (FLOW) { q0 = flow_load(a.q + (size_t)h * HS + e0); q1 = flow_load(a.q + (size_t)h * HS + e1); }
            else { q0 = a.q[(size_t)h * HS + e0]; q1 = a.q[(size_t)h * HS + e1]; }
            if (fresh) {
                if (a.qbias) { q0 += a.qbias[(size_t)h * HS + e0]; q1 += a.qbias[(size_t)h * HS + e1]; }
                if (rot && a.rope_theta) theta = a.rope_theta[i];
                if (own_new) {
                    if constexpr (FLOW) {
                        k0 = flow_load(a.knew + hoff + e0); k1 = flow_load(a.knew + hoff + e1);
                        v0 = flow_load(a.vnew + hoff + e0); v1 = flow_load(a.vnew + hoff + e1);
                    } else {
                        k0 = a.knew[hoff + e0]; k1 = a.knew[hoff + e1];
                        v0 = a.vnew[hoff + e0]; v1 = a.vnew[hoff + e1];
                    }
                    if (a.kbias) { k0 += a.kbias[hoff + e0]; k1 += a.kbias[hoff + e1]; }
                    if (a.vbias) { v0 += a.vbias[hoff + e0]; v1 += a.vbias[hoff + e1]; }
                }
            }
        }
    };
    if constexpr (!FUSED) { wait_inputs(); load_inputs(); }
    // ---- the first pass of keys and values is requested before anything else is computed: they depend on nothing
    // but the position, and their latency then overlaps the q load and the RoPE.  A pass is NT/KL positions; wave w
    // owns PPW consecutive ones for both the scores (KL lanes per position) and the values (LPP lanes per
    // position, PW positions per sub-pass), so nothing but the final merge crosses waves. -----------------------
    constexpr int PW = 64 / LPP;                  // positions per value sub-pass of a wave
    constexpr int NU = PPW / PW;                  // value sub-passes per pass
    const uint32_t sub = tid & (KL - 1);
    const uint32_t wpos = wave * PPW;
    const uint32_t vgl = lane / LPP, ve = (lane % LPP) * 8;
    typename Vec8<F16>::Raw kv0[EPL / 8], vv0[NU];            // kept undecoded: fewer registers while they wait
    {
        const uint32_t t = t0 + tid / KL;
        // the fresh row comes from LDS later; lanes without a position read a valid address and are masked
        const uint32_t tc = (t < t1 && !(own_new && t == pos)) ? t : min(t0, pos);
        const CT *kp = kc + (size_t)tc * a.kv_dim + hoff + sub * 8;
#pragma unroll
        for (int j = 0; j < EPL / 8; ++j) kv0[j] = Vec8<F16>::template load_raw<STREAM>(kp + 8 * KL * j);
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const uint32_t tv = t0 + wpos + u * PW + vgl;
            const uint32_t tvc = (tv < t1 && !(own_new && tv == pos)) ? tv : min(t0, pos);
            vv0[u] = Vec8<F16>::template load_raw<STREAM>(vc + (size_t)tvc * a.kv_dim + hoff + ve);
        }
    }

    if constexpr (FUSED) { wait_inputs(); load_inputs(); }

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
    for (int j = 0; j < EPL; ++j) qr[j] = sq[(j / 8) * 8 * KL + sub * 8 + (j % 8)];
    const float root = sqrtf((float)HS);
    float m = -FLT_MAX, lsum = 0.0f;
    float o[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t tb = t0; tb < t1; tb += NT / KL) {           // uniform trip count: the shuffles below need whole waves
        const uint32_t t = tb + tid / KL;
        const bool live = t < t1;
        const bool use_new = own_new && live && t == pos;    // its cache row is being written by this very launch
        typename Vec8<F16>::Raw nxt[EPL / 8] = {}, nxtv[NU] = {};
        if (tb + NT / KL < t1) {                               // (uniform) there is a next pass
            const uint32_t tn = t + NT / KL;
            const uint32_t tnc = (tn < t1 && !(own_new && tn == pos)) ? tn : min(t0, pos);
            const CT *kp = kc + (size_t)tnc * a.kv_dim + hoff + sub * 8;
#pragma unroll
            for (int j = 0; j < EPL / 8; ++j) nxt[j] = Vec8<F16>::template load_raw<STREAM>(kp + 8 * KL * j);
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const uint32_t tv = tb + NT / KL + wpos + u * PW + vgl;
                const uint32_t tvc = (tv < t1 && !(own_new && tv == pos)) ? tv : min(t0, pos);
                nxtv[u] = Vec8<F16>::template load_raw<STREAM>(vc + (size_t)tvc * a.kv_dim + hoff + ve);
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
            for (int j = 0; j < EPL; ++j) kv[j] = sk[(j / 8) * 8 * KL + sub * 8 + (j % 8)];
        }
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) part = fmaf(qr[j], kv[j], part);
        part += __shfl_xor(part, 1, 64);
        part += __shfl_xor(part, 2, 64);
        if constexpr (KL == 8) part += __shfl_xor(part, 4, 64);
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
            const float pw = __shfl(pr, KL * (u * PW + vgl), 64);      // 0 for positions past the end
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
            const uint32_t e = h * HS + tid;
            // (a chunk of prompt tokens: token `quad_token` of a [columns / 4][32 tokens][4] matrix)
            if (quad_token != 0xffffffffu) {
                float *slot = a.out + ((size_t)(e >> 2) * 32 + quad_token) * 4;
                if (split_flag) {
                    const float v = r / l;
                    uint32_t hd, rm;
                    split_pair_f16(v, 0.0f, hd, rm);
                    if (!(fabsf(v) < 65504.0f)) *split_flag = 2;
                    uint16_t *s16 = reinterpret_cast<uint16_t *>(slot);
                    s16[e & 3u] = (uint16_t)hd;
                    s16[4 + (e & 3u)] = (uint16_t)rm;
                } else {
                    slot[e & 3u] = r / l;
                }
            } else if constexpr (FLOW) {
                flow_store(a.out + e, r / l);
            } else {
                a.out[e] = r / l;
            }
        } else {
            float *po = a.scratch + ((size_t)h * a.n_splits + split) * (HS + 2);
            po[tid] = r;
            if (tid == 0) { po[HS] = (t1 > t0) ? M : -FLT_MAX; po[HS + 1] = (t1 > t0) ? l : 0.0f; }
        }
    }
}


}  // namespace attn
}  // namespace slai
