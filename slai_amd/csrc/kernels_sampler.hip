// Temperature / top-p sampling on the device: crates/slai/src/models/sampler.rs:33-131 with the random draw
// (`coin`) supplied by the caller or derived from (seed, position), plus the forced-token rule and loop
// bookkeeping the greedy kernel applies (crates/slai-chat/src/sampler.rs:100-105, chat_llama2.rs:105-158).
//
// One workgroup of 1024 threads.  Wave w owns the contiguous slice [w*seg, (w+1)*seg) of the vocabulary and walks
// it 64 consecutive entries at a time, so loads are coalesced and index order (which the cumulative distribution
// and the order among equal probabilities depend on) is wave order, then iteration order, then lane order.
//
// The reference sorts the candidates by descending probability and walks the sorted list twice (once up to the
// nucleus mass `topp`, once up to coin * mass).  Here both walks are one primitive, `crossing(target)`: the first
// sorted position whose running mass exceeds `target`.  It is found without sorting, by fixing the probability's
// bit pattern four bits at a time (probabilities are non-negative floats, so their bits order like they do): each
// pass bins the candidates that match the bits fixed so far by their next four bits, reduces the 16 (mass, count)
// pairs over the workgroup in a fixed order, and walks the bins from the largest down.  Equal probabilities keep
// index order, as the reference's stable sort does.  Sums are taken in a different order than the reference's
// sequential ones, so results can differ from it when `coin` falls within rounding distance of a boundary.
#include "common.h"
#include "device_util.h"

#include <cfloat>

namespace slai {
namespace {

constexpr int NT = 1024, NW = NT / 64;
constexpr int CACHE = 32;                       // probabilities of a thread's first CACHE entries stay in registers

struct Shared {
    float f[NW][16];
    uint32_t u[NW][16];
    float totf[16];
    uint32_t totu[16];
    float red[NW];
    uint32_t redu[NW];
    uint32_t result;
};

__device__ __forceinline__ float wsum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}
__device__ __forceinline__ float wmax(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}
// 16 values per lane -> their 16 totals over the wave with 17 exchanges instead of 96: every step halves the values
// a lane is responsible for.  Afterwards a[0] of lane L holds the total of value 8*b5 + 4*b4 + 2*b3 + b2 (bits of L).
template <class X> __device__ __forceinline__ void wave_reduce16(X (&a)[16], uint32_t lane) {
#pragma unroll
    for (int half = 8, m = 32; half >= 1; half >>= 1, m >>= 1) {
        const bool up = lane & m;
#pragma unroll
        for (int k = 0; k < half; ++k) {
            const X keep = up ? a[k + half] : a[k];
            const X send = up ? a[k] : a[k + half];
            a[k] = keep + __shfl_xor(send, m, 64);
        }
    }
    a[0] += __shfl_xor(a[0], 2, 64);
    a[0] += __shfl_xor(a[0], 1, 64);
}

struct Dist {                                   // what defines the distribution: p_i = exp(v_i / T - xm) / S
    const float *v; uint32_t n; float T, xm, S;
    uint32_t seg, base;                         // slice length (a multiple of 64) and this thread's first index
    uint32_t iters;                             // 64-entry steps per slice
    float pc[CACHE];
    __device__ __forceinline__ uint32_t index(uint32_t k) const { return base + 64 * k; }
    __device__ __forceinline__ float raw(uint32_t k) const {          // sampler.rs:39-42 + softmax.rs:46-59
        const uint32_t i = index(k);
        return i < n ? expf(v[i] / T - xm) : 0.0f;
    }
    __device__ __forceinline__ float prob_uncached(uint32_t k) const { return raw(k) / S; }
};

// body(p, i) for every step of the thread's slice: p from the registers for the first CACHE steps, recomputed beyond
template <class F> __device__ __forceinline__ void for_each_prob(const Dist &D, F &&body) {
#pragma unroll
    for (uint32_t k = 0; k < CACHE; ++k)
        if (k < D.iters) body(D.pc[k], D.index(k));
    for (uint32_t k = CACHE; k < D.iters; ++k) body(D.prob_uncached(k), D.index(k));
}

struct Cross { uint32_t key, j, position; float cum; };

// First position of the descending, index-stable order of the candidates (p >= cutoff) at which the running mass
// exceeds `target`; when it never does, the last position.  `cum` is the running mass there (sampler.rs:108-118).
__device__ __forceinline__ Cross crossing(const Dist &D, float cutoff, float target, Shared &sh) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t prefix = 0, cnt_above = 0, ties = 0;
    float mass_above = 0.0f;
    for (int shift = 28; shift >= 0; shift -= 4) {
        float m[16];
        uint32_t c[16];
#pragma unroll
        for (int d = 0; d < 16; ++d) { m[d] = 0.0f; c[d] = 0; }
        const uint32_t himask = shift == 28 ? 0u : (0xffffffffu << (shift + 4));
        for_each_prob(D, [&](float p, uint32_t i) {
            const uint32_t key = __float_as_uint(p);
            const bool on = i < D.n && p >= cutoff && (key & himask) == prefix;
            if (__ballot(on)) {                                 // whole waves skip entries that left the search
                const uint32_t dg = (key >> shift) & 15u;
#pragma unroll
                for (int d = 0; d < 16; ++d) { const bool hit = on && dg == (uint32_t)d; m[d] += hit ? p : 0.0f; c[d] += hit ? 1u : 0u; }
            }
        });
        wave_reduce16(m, lane);
        wave_reduce16(c, lane);
        if ((lane & 3) == 0) {
            const uint32_t idx = ((lane >> 5) & 1) * 8 + ((lane >> 4) & 1) * 4 + ((lane >> 3) & 1) * 2 + ((lane >> 2) & 1);
            sh.f[wave][idx] = m[0]; sh.u[wave][idx] = c[0];
        }
        __syncthreads();
        if (threadIdx.x < 16) { float t = 0.0f; for (int w = 0; w < NW; ++w) t += sh.f[w][threadIdx.x]; sh.totf[threadIdx.x] = t; }
        else if (threadIdx.x < 32) { uint32_t t = 0; for (int w = 0; w < NW; ++w) t += sh.u[w][threadIdx.x - 16]; sh.totu[threadIdx.x - 16] = t; }
        __syncthreads();
        // every thread walks the 16 bins the same way
        int sel = -1, lowest = 0;
        float acc = mass_above; uint32_t cacc = cnt_above;
        for (int d = 15; d >= 0; --d) {
            if (!sh.totu[d]) continue;
            lowest = d;
            if (sel < 0) {
                if (acc + sh.totf[d] > target) sel = d;
                else { acc += sh.totf[d]; cacc += sh.totu[d]; }
            }
        }
        if (sel < 0) {                                          // no bin crosses: continue in the smallest one
            sel = lowest; acc = mass_above; cacc = cnt_above;
            for (int d = 15; d > lowest; --d) if (sh.totu[d]) { acc += sh.totf[d]; cacc += sh.totu[d]; }
        }
        mass_above = acc; cnt_above = cacc; prefix |= (uint32_t)sel << shift; ties = sh.totu[sel];
        // no barrier here: the totals are rewritten only after the next pass's first barrier, which every thread
        // reaches after this walk
    }
    Cross r;
    r.key = prefix;
    const float pv = __uint_as_float(prefix);
    float cc = mass_above; uint32_t j = ties;
    for (uint32_t t = 1; t <= ties; ++t) { cc += pv; if (cc > target) { j = t; break; } }
    r.j = j; r.cum = cc; r.position = cnt_above + j - 1;
    return r;
}

// index of the j-th (1-based, index order) candidate whose probability has the bits `key`
__device__ __forceinline__ uint32_t locate(const Dist &D, float cutoff, uint32_t key, uint32_t j, Shared &sh) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t mine = 0;
    for_each_prob(D, [&](float p, uint32_t i) { mine += (i < D.n && p >= cutoff && __float_as_uint(p) == key) ? 1u : 0u; });
    uint32_t wtot = mine;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) wtot += __shfl_xor(wtot, m, 64);
    if (lane == 0) sh.redu[wave] = wtot;
    if (threadIdx.x == 0) sh.result = 0xffffffffu;
    __syncthreads();
    uint32_t before = 0;
    for (uint32_t w = 0; w < wave; ++w) before += sh.redu[w];
    if (j > before && j <= before + wtot) {                     // (wave-uniform) the wanted entry is in this slice
        uint32_t seen = before;
        bool done = false;
        for_each_prob(D, [&](float p, uint32_t i) {
            if (!done) {
                const bool on = i < D.n && p >= cutoff && __float_as_uint(p) == key;
                const unsigned long long mask = __ballot(on);
                const uint32_t cnt = (uint32_t)__popcll(mask);
                if (j <= seen + cnt) {
                    unsigned long long mm = mask;
                    for (uint32_t s = seen + 1; s < j; ++s) mm &= mm - 1;          // drop the lower set bits
                    const uint32_t hit_lane = (uint32_t)__ffsll((long long)mm) - 1;
                    if (lane == hit_lane) sh.result = i;
                    done = true;
                }
                seen += cnt;
            }
        });
    }
    __syncthreads();
    const uint32_t r = sh.result;
    __syncthreads();
    return r;
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

__global__ void __launch_bounds__(NT) sample_kernel(const float *v, uint32_t n, float temperature, float topp, float coin_arg,
                                                    int *out_index, DecodeState *st, const int *prompt, int *out_tokens) {
    __shared__ Shared sh;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float coin = coin_arg;
    if (st) {                                                   // the decode loop: parameters and counter live in device memory
        temperature = st->temperature; topp = st->topp;
        const uint64_t seed = ((uint64_t)st->seed_hi << 32) | st->seed_lo;
        coin = (float)(splitmix64(seed + (uint64_t)(uint32_t)st->pos) >> 40) * (1.0f / 16777216.0f);
    }
    Dist D;
    D.v = v; D.n = n; D.T = temperature;
    D.seg = ((n + NW - 1) / NW + 63) / 64 * 64;
    D.base = wave * D.seg + lane;
    D.iters = D.seg / 64;
    // ---- max (of v / T: division by a positive T is monotonic, so it is max(v) / T) and first index of the maximum
    float best = -FLT_MAX; uint32_t besti = 0xffffffffu;
    for (uint32_t k = 0; k < D.iters; ++k) {
        const uint32_t i = D.index(k);
        if (i < n) { const float x = v[i]; if (besti == 0xffffffffu || x > best) { best = x; besti = i; } }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ob = __shfl_xor(best, m, 64);
        const uint32_t oi = __shfl_xor(besti, m, 64);
        if (oi != 0xffffffffu && (besti == 0xffffffffu || ob > best || (ob == best && oi < besti))) { best = ob; besti = oi; }
    }
    if (lane == 0) { sh.red[wave] = best; sh.redu[wave] = besti; }
    __syncthreads();
    best = sh.red[0]; besti = sh.redu[0];
    for (int w = 1; w < NW; ++w)
        if (sh.redu[w] != 0xffffffffu && (besti == 0xffffffffu || sh.red[w] > best || (sh.red[w] == best && sh.redu[w] < besti))) { best = sh.red[w]; besti = sh.redu[w]; }
    __syncthreads();
    uint32_t chosen;
    if (temperature == 0.0f) {
        chosen = besti;                                         // sampler.rs:34-36: greedy
    } else {
        D.xm = best / temperature;
        // ---- normaliser
        float part = 0.0f;
        for (uint32_t k = 0; k < D.iters; ++k) part += D.raw(k);
        part = wsum(part);
        if (lane == 0) sh.red[wave] = part;
        __syncthreads();
        float S = 0.0f;
        for (int w = 0; w < NW; ++w) S += sh.red[w];
        __syncthreads();
        D.S = S;
#pragma unroll
        for (uint32_t k = 0; k < CACHE; ++k) D.pc[k] = k < D.iters ? D.prob_uncached(k) : 0.0f;
        if (topp <= 0.0f || topp >= 1.0f) {
            // ---- sampler.rs:63-78 `sample_mult`: the first index whose cumulative probability exceeds the coin
            float tot = 0.0f;
            for_each_prob(D, [&](float p, uint32_t) { tot += wsum(p); });
            if (lane == 0) sh.red[wave] = tot;
            if (threadIdx.x == 0) sh.result = n - 1;           // rounding may leave the total below the coin
            __syncthreads();
            float cdf = 0.0f;
            for (uint32_t w = 0; w < wave; ++w) cdf += sh.red[w];
            uint32_t found = 0xffffffffu;
            for_each_prob(D, [&](float p, uint32_t i) {
                if (found == 0xffffffffu) {
                    float inc = p;
#pragma unroll
                    for (int d = 1; d < 64; d <<= 1) { const float o = __shfl_up(inc, d, 64); if (lane >= (uint32_t)d) inc += o; }
                    const bool hit = i < n && coin < cdf + inc;
                    const unsigned long long mask = __ballot(hit);
                    if (mask) found = __shfl(i, __ffsll((long long)mask) - 1, 64);
                    cdf += __shfl(inc, 63, 64);
                }
            });
            if (lane == 0 && found != 0xffffffffu) atomicMin(&sh.result, found);
            __syncthreads();
            chosen = sh.result;
        } else {
            // ---- sampler.rs:85-131 `sample_topp`
            const float cutoff = (1.0f - topp) / ((float)n - 1.0f);
            const Cross nucleus = crossing(D, cutoff, topp, sh);
            const float r = coin * nucleus.cum;
            Cross pick = crossing(D, cutoff, r, sh);
            if (pick.position > nucleus.position) pick = nucleus;     // rounding: stay inside the nucleus (:130)
            chosen = locate(D, cutoff, pick.key, pick.j, sh);
            if (chosen == 0xffffffffu) chosen = besti;          // not reachable with finite logits; keeps the id valid
        }
    }
    if (threadIdx.x == 0) {
        int next = (int)chosen;
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

}  // namespace

hipError_t launch_sample(hipStream_t s, const float *v, uint32_t n, float temperature, float topp, float coin, int *out_index,
                         DecodeState *decode, const int *prompt, int *out_tokens) {
    sample_kernel<<<1, NT, 0, s>>>(v, n, temperature, topp, coin, out_index, decode, prompt, out_tokens);
    return hipGetLastError();
}

}  // namespace slai
