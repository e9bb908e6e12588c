// Temperature / top-p sampling on the device: crates/slai/src/models/sampler.rs:33-131 with the random draw
// (`coin`) supplied by the caller or derived from (seed, position), plus the forced-token rule and loop
// bookkeeping the greedy kernel applies (crates/slai-chat/src/sampler.rs:100-105, chat_llama2.rs:105-158).
//
// One workgroup of 1024 threads.  Wave w owns the contiguous slice [w*slice, (w+1)*slice) of the vocabulary and
// walks it 64 consecutive entries at a time, so loads are coalesced and index order (which the cumulative
// distribution and the order among equal probabilities depend on) is wave order, then iteration order, then lane
// order.  The probabilities are written once to a scratch vector (n floats, L2-resident) and re-read by the passes.
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
constexpr int UNROLL = 16;                      // scratch entries a thread requests before it uses the first

struct Shared {
    float f[NW][16];
    uint32_t u[NW][16];
    float totf[16];
    uint32_t totu[16];
    float red[NW];
    uint32_t redu[NW];
    uint32_t result;
    // a bin of at most 64 entries, gathered and ordered by one wave
    uint32_t gcount;
    float gp[64], sp[64];
    uint32_t gi[64], si[64];
    uint32_t res_key, res_idx, res_pos; float res_cum;
};

__device__ __forceinline__ float wsum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}
// 16 values per lane -> their 16 totals over the wave with 17 exchanges instead of 96: every step halves the values
// a lane is responsible for.  Afterwards a[0] of lane L holds the total of value 8*b5 + 4*b4 + 2*b3 + b2 (bits of L).
template <int HALF, int M, class X> __device__ __forceinline__ void halve(X (&a)[16], uint32_t lane) {
    const bool up = lane & M;
#pragma unroll
    for (int k = 0; k < HALF; ++k) {
        const X keep = up ? a[k + HALF] : a[k];
        const X send = up ? a[k] : a[k + HALF];
        a[k] = keep + __shfl_xor(send, M, 64);
    }
}
template <class X> __device__ __forceinline__ void wave_reduce16(X (&a)[16], uint32_t lane) {
    halve<8, 32>(a, lane); halve<4, 16>(a, lane); halve<2, 8>(a, lane); halve<1, 4>(a, lane);
    a[0] += __shfl_xor(a[0], 2, 64);
    a[0] += __shfl_xor(a[0], 1, 64);
}

// The distribution: probabilities (softmax of v / T, sampler.rs:39-42 with softmax.rs:46-59) of the entries this
// thread owns, index(k) = wave * slice + 64 * k + lane.  R > 0: the slice is 64 * R entries and they stay in registers
// (vocabularies up to 16 * 64 * R); R == 0: they are written once to a scratch vector and re-read by every pass (a
// single compute unit re-reads slowly: this is the fallback for larger vocabularies).  A thread only ever reads
// back the scratch entries it wrote itself.
template <int R> struct Dist {
    float r[R > 0 ? R : 1];
    const float *p; uint32_t n;
    uint32_t kmax;                              // bits of the largest probability, 1 / (sum of the exponentials)
    uint32_t base;                              // this thread's first index: wave * slice + lane
    uint32_t iters;                             // 64-entry steps per slice (R, or a multiple of UNROLL)
    __device__ __forceinline__ uint32_t index(uint32_t k) const { return base + 64 * k; }
};

// body(p, i) for every entry of the thread's slice, in increasing i
template <int R, class F> __device__ __forceinline__ void for_each_prob(const Dist<R> &D, F &&body) {
    if constexpr (R > 0) {
#pragma unroll
        for (int k = 0; k < R; ++k) body(D.r[k], D.index(k));
    } else {
        for (uint32_t k0 = 0; k0 < D.iters; k0 += UNROLL) {
            float v[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) { const uint32_t i = D.index(k0 + u); v[u] = i < D.n ? D.p[i] : 0.0f; }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) body(v[u], D.index(k0 + u));
        }
    }
}

// `index` is the entry itself when the search ended in a bin small enough to order directly; 0xffffffff otherwise:
// then the entry is the j-th (index order) of those whose probability has the bits `key`
struct Cross { uint32_t key, j, position, index; float cum; };

// First position of the descending, index-stable order of the candidates (p >= cutoff) at which the running mass
// exceeds `target`; when it never does, the last position.  `cum` is the running mass there (sampler.rs:108-118).
template <int R> __device__ __forceinline__ Cross crossing(const Dist<R> &D, float cutoff, float target, Shared &sh) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t prefix = 0, cnt_above = 0, ties = 0;
    float mass_above = 0.0f;
    // every candidate's bits lie between those of the cutoff and of the largest probability: the four-bit groups the
    // two share need no pass
    int start = 28;
    {
        const uint32_t lo = __float_as_uint(cutoff), hi = D.kmax;
        if (hi >= lo) {
            const uint32_t x = lo ^ hi;
            start = x ? ((31 - __clz((int)x)) / 4) * 4 : 0;
            prefix = start < 28 ? hi & (0xffffffffu << (start + 4)) : 0u;
        }
    }
    for (int shift = start; shift >= 0; shift -= 4) {
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
        if (ties >= 1 && ties <= 64 && shift > 0) {
            // ---- few entries left: gather them, let one wave put them in the sampler's order (probability descending,
            // then index) and add them up in that order
            const uint32_t mask = 0xffffffffu << shift;
            if (threadIdx.x == 0) sh.gcount = 0;
            __syncthreads();
            for_each_prob(D, [&](float p, uint32_t i) {
                if (i < D.n && p >= cutoff && (__float_as_uint(p) & mask) == prefix) {
                    const uint32_t slot = atomicAdd(&sh.gcount, 1u);
                    if (slot < 64) { sh.gp[slot] = p; sh.gi[slot] = i; }
                }
            });
            __syncthreads();
            if (wave == 0) {
                const uint32_t cnt = ties;
                const bool live = lane < cnt;
                const float mp = live ? sh.gp[lane] : 0.0f;
                const uint32_t mi = live ? sh.gi[lane] : 0xffffffffu;
                uint32_t rank = 0;
                for (uint32_t q = 0; q < cnt; ++q) {
                    const float op = sh.gp[q]; const uint32_t oi = sh.gi[q];
                    rank += (op > mp || (op == mp && oi < mi)) ? 1u : 0u;
                }
                if (live) { sh.sp[rank] = mp; sh.si[rank] = mi; }
                // (one wave: its LDS writes are complete before its next LDS reads are issued)
                float run = live ? sh.sp[lane] : 0.0f;
#pragma unroll
                for (int d = 1; d < 64; d <<= 1) { const float o = __shfl_up(run, d, 64); if (lane >= (uint32_t)d) run += o; }
                run += mass_above;
                const unsigned long long over = __ballot(live && run > target);
                const uint32_t at = over ? (uint32_t)__ffsll((long long)over) - 1 : cnt - 1;   // never crossed: the last one
                if (lane == at) { sh.res_key = __float_as_uint(sh.sp[at]); sh.res_idx = sh.si[at]; sh.res_pos = cnt_above + at; sh.res_cum = run; }
            }
            __syncthreads();
            Cross r;
            r.key = sh.res_key; r.index = sh.res_idx; r.position = sh.res_pos; r.cum = sh.res_cum; r.j = 0;
            __syncthreads();
            return r;
        }
    }
    Cross r;
    r.key = prefix; r.index = 0xffffffffu;
    const float pv = __uint_as_float(prefix);
    float cc = mass_above; uint32_t j = ties;
    for (uint32_t t = 1; t <= ties; ++t) { cc += pv; if (cc > target) { j = t; break; } }
    r.j = j; r.cum = cc; r.position = cnt_above + j - 1;
    return r;
}

// index of the j-th (1-based, index order) candidate whose probability has the bits `key`
template <int R> __device__ __forceinline__ uint32_t locate(const Dist<R> &D, float cutoff, uint32_t key, uint32_t j, Shared &sh) {
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

// sampler.rs:63-78 `sample_mult` on registers: the first index whose cumulative probability exceeds the coin.  Row sums
// (one per 64-entry step) of all waves are scanned by the first 16 * R threads; the wave that owns the crossing row
// then scans that row alone.
template <int R> __device__ __forceinline__ uint32_t sample_mult_rows(const Dist<R> &D, float coin, uint32_t fallback, Shared &sh, float *rows /* [NW * R] */,
                                                                     float *incl /* [NW * R] */) {
    static_assert(R == 32, "two 16-value reductions cover the rows");
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float a[16], b[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) { a[k] = D.r[k]; b[k] = D.r[16 + k]; }
    wave_reduce16(a, lane);
    wave_reduce16(b, lane);
    if ((lane & 3) == 0) {
        const uint32_t idx = ((lane >> 5) & 1) * 8 + ((lane >> 4) & 1) * 4 + ((lane >> 3) & 1) * 2 + ((lane >> 2) & 1);
        rows[wave * R + idx] = a[0]; rows[wave * R + 16 + idx] = b[0];
    }
    if (threadIdx.x == 0) sh.result = 0xffffffffu;
    __syncthreads();
    // inclusive scan of the NW * R row sums in index order (row t belongs to wave t / R, step t % R)
    const uint32_t t = threadIdx.x;
    float inc = t < NW * R ? rows[t] : 0.0f;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) { const float o = __shfl_up(inc, d, 64); if (lane >= (uint32_t)d) inc += o; }
    if (lane == 63) sh.red[wave] = inc;
    __syncthreads();
    float before = 0.0f;
    for (uint32_t w = 0; w < wave; ++w) before += sh.red[w];
    inc += before;
    if (t < NW * R) incl[t] = inc;
    const unsigned long long hits = __ballot(t < NW * R && coin < inc);
    if (lane == 0 && hits) atomicMin(&sh.result, (t & ~63u) + (uint32_t)__ffsll((long long)hits) - 1);
    __syncthreads();
    const uint32_t row = sh.result;                           // first row whose running total exceeds the coin
    __syncthreads();
    if (row == 0xffffffffu) return fallback;                  // rounding left the total below the coin (:77)
    if (wave == row / R) {
        const uint32_t k = row % R;
        float x = 0.0f;
#pragma unroll
        for (int q = 0; q < R; ++q) x = k == (uint32_t)q ? D.r[q] : x;
        const float start = row ? incl[row - 1] : 0.0f;
        float run = x;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) { const float o = __shfl_up(run, d, 64); if (lane >= (uint32_t)d) run += o; }
        const uint32_t i = D.index(k);
        const unsigned long long mask = __ballot(i < D.n && coin < start + run);
        const unsigned long long valid = __ballot(i < D.n);
        // the row total said the crossing is here; if the finer sums disagree, it is the row's last entry
        const uint32_t at = mask ? (uint32_t)__ffsll((long long)mask) - 1 : 63u - (uint32_t)__clzll((long long)valid);
        if (lane == at) sh.result = i;
    }
    __syncthreads();
    const uint32_t r = sh.result;
    __syncthreads();
    return r;
}

template <int R>
__global__ void __launch_bounds__(NT) sample_kernel(const float *__restrict__ v, uint32_t n, float temperature, float topp, float coin_arg,
                                                    float *pbuf, int *out_index, DecodeState *st, const int *prompt, int *out_tokens) {
    __shared__ Shared sh;
    __shared__ float rows[R > 0 ? NW * R : 1], rows_incl[R > 0 ? NW * R : 1];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float coin = coin_arg;
    if (st) {                                                   // the decode loop: parameters and counter live in device memory
        temperature = st->temperature; topp = st->topp;
        const uint64_t seed = ((uint64_t)st->seed_hi << 32) | st->seed_lo;
        coin = (float)(splitmix64(seed + (uint64_t)(uint32_t)st->pos) >> 40) * (1.0f / 16777216.0f);
    }
    const uint32_t slice = R > 0 ? 64u * R : ((n + NW - 1) / NW + 64 * UNROLL - 1) / (64 * UNROLL) * (64 * UNROLL);
    Dist<R> D;
    D.p = pbuf; D.n = n;
    D.base = wave * slice + lane;
    D.iters = slice / 64;
    // ---- max (of v / T: division by a positive T is monotonic, so it is max(v) / T) and first index of the maximum
    float best = -FLT_MAX; uint32_t besti = 0xffffffffu;
    if constexpr (R > 0) {
#pragma unroll
        for (int k = 0; k < R; ++k) { const uint32_t i = D.index(k); D.r[k] = v[i < n ? i : 0]; }
#pragma unroll
        for (int k = 0; k < R; ++k) {
            const uint32_t i = D.index(k);
            if (i < n && (besti == 0xffffffffu || D.r[k] > best)) { best = D.r[k]; besti = i; }
        }
    } else {
        for (uint32_t k0 = 0; k0 < D.iters; k0 += UNROLL) {
            float x[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) { const uint32_t i = D.index(k0 + u); x[u] = v[i < n ? i : 0]; }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const uint32_t i = D.index(k0 + u);
                if (i < n && (besti == 0xffffffffu || x[u] > best)) { best = x[u]; besti = i; }
            }
        }
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
        // ---- exp(v / T - max), their sum, then the probabilities (in the registers, or in the scratch)
        const float xm = best / temperature;
        float part = 0.0f;
        if constexpr (R > 0) {
#pragma unroll
            for (int k = 0; k < R; ++k) { D.r[k] = D.index(k) < n ? expf(D.r[k] / temperature - xm) : 0.0f; part += D.r[k]; }
        } else {
            for (uint32_t k0 = 0; k0 < D.iters; k0 += UNROLL) {
                float x[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) { const uint32_t i = D.index(k0 + u); x[u] = v[i < n ? i : 0]; }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const uint32_t i = D.index(k0 + u);
                    if (i < n) { const float e = expf(x[u] / temperature - xm); pbuf[i] = e; part += e; }
                }
            }
        }
        part = wsum(part);
        if (lane == 0) sh.red[wave] = part;
        __syncthreads();
        float S = 0.0f;
        for (int w = 0; w < NW; ++w) S += sh.red[w];
        __syncthreads();
        D.kmax = __float_as_uint(1.0f / S);                 // the maximum's exponential is exp(0) = 1
        const float cutoff_all = (1.0f - topp) / ((float)n - 1.0f);     // sampler.rs:93 (only meaningful with top-p)
        uint32_t candidates = 0;
        if constexpr (R > 0) {
#pragma unroll
            for (int k = 0; k < R; ++k) D.r[k] = D.r[k] / S;
        } else {
            for (uint32_t k0 = 0; k0 < D.iters; k0 += UNROLL) {
                float e[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) { const uint32_t i = D.index(k0 + u); e[u] = i < n ? pbuf[i] : 0.0f; }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const uint32_t i = D.index(k0 + u);
                    const float pv = e[u] / S;
                    if (i < n) pbuf[i] = pv;
                    candidates += (uint32_t)__popcll(__ballot(i < n && pv >= cutoff_all));   // (wave-uniform) for the top-p search
                }
            }
        }
        if (topp <= 0.0f || topp >= 1.0f) {
            if constexpr (R > 0) {
                chosen = sample_mult_rows(D, coin, n - 1, sh, rows, rows_incl);
            } else {
            // ---- sampler.rs:63-78 `sample_mult`: the first index whose cumulative probability exceeds the coin
            float tot = 0.0f;
            for_each_prob(D, [&](float p, uint32_t) { tot += p; });
            tot = wsum(tot);
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
            }
        } else {
            // ---- sampler.rs:85-131 `sample_topp`
            const float cutoff = (1.0f - topp) / ((float)n - 1.0f);
            if constexpr (R == 0) {
                // A large vocabulary: the candidates (p >= cutoff, sampler.rs:93-103) are first packed, in index order,
                // behind the probabilities in the scratch; when at most 32768 are left (any distribution a model
                // produces in practice) the search runs over them in registers instead of re-reading the whole
                // vocabulary in every pass.
                float *cp = pbuf + (size_t)NW * slice;                         // packed probabilities
                uint32_t *ci = reinterpret_cast<uint32_t *>(cp + (size_t)NW * slice);   // and their vocabulary indices
                if (lane == 0) sh.redu[wave] = candidates;                     // counted while the probabilities were written
                __syncthreads();
                uint32_t at = 0, n0 = 0;
                for (uint32_t w = 0; w < NW; ++w) { if (w < wave) at += sh.redu[w]; n0 += sh.redu[w]; }
                __syncthreads();
                if (n0 <= NW * 64 * 32) {
                    for_each_prob(D, [&](float p, uint32_t i) {
                        const bool on = i < n && p >= cutoff;
                        const unsigned long long mask = __ballot(on);
                        if (on) {
                            const uint32_t pos = at + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
                            cp[pos] = p; ci[pos] = i;
                        }
                        at += (uint32_t)__popcll(mask);
                    });
                    __syncthreads();                                           // other waves read what this one packed
                    Dist<32> C;
                    C.p = cp; C.n = n0; C.kmax = D.kmax;
                    C.base = wave * (64u * 32u) + lane; C.iters = 32;
#pragma unroll
                    for (int k = 0; k < 32; ++k) { const uint32_t i = C.index(k); C.r[k] = i < n0 ? cp[i] : 0.0f; }
                    const Cross nucleus = crossing(C, cutoff, topp, sh);
                    const float r = coin * nucleus.cum;
                    Cross pick = crossing(C, cutoff, r, sh);
                    if (pick.position > nucleus.position) pick = nucleus;
                    uint32_t slot = pick.index != 0xffffffffu ? pick.index : locate(C, cutoff, pick.key, pick.j, sh);
                    chosen = slot < n0 ? ci[slot] : besti;
                    goto picked;
                }
            }
            const Cross nucleus = crossing(D, cutoff, topp, sh);
            const float r = coin * nucleus.cum;
            Cross pick = crossing(D, cutoff, r, sh);
            if (pick.position > nucleus.position) pick = nucleus;     // rounding: stay inside the nucleus (:130)
            chosen = pick.index != 0xffffffffu ? pick.index : locate(D, cutoff, pick.key, pick.j, sh);
            if (chosen == 0xffffffffu) chosen = besti;          // not reachable with finite logits; keeps the id valid
        }
    }
picked:
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

// floats of scratch a launch over n logits needs: none below 32769, else the probabilities and the packed candidates
// (probabilities + indices), each padded to the slices of the 16 waves
size_t sample_scratch_floats(uint32_t n) {
    if (n <= NW * 64 * 32) return 1;
    const size_t slice = ((size_t)(n + NW - 1) / NW + 64 * UNROLL - 1) / (64 * UNROLL) * (64 * UNROLL);
    return 3 * NW * slice;
}

hipError_t launch_sample(hipStream_t s, const float *v, uint32_t n, float temperature, float topp, float coin, float *scratch, int *out_index,
                         DecodeState *decode, const int *prompt, int *out_tokens) {
    if (n <= NW * 64 * 32) sample_kernel<32><<<1, NT, 0, s>>>(v, n, temperature, topp, coin, scratch, out_index, decode, prompt, out_tokens);
    else sample_kernel<0><<<1, NT, 0, s>>>(v, n, temperature, topp, coin, scratch, out_index, decode, prompt, out_tokens);
    return hipGetLastError();
}

}  // namespace slai
