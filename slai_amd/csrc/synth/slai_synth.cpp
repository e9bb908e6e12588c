// slai_synth -- synthetic-model support: a deterministic normal generator and
// fp32 -> GGUF block quantizers (Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, Q8_K, Q4_K, Q5_K, Q6_K, F16).
//
// The reference has no quantizer (crates/slai/src/quantization.rs only dequantizes),
// so these follow ggml's public `quantize_row_*_ref` algorithms.  They are INPUT
// GENERATORS: the same bytes are handed to the device library and to whatever checks
// it, so their fidelity to ggml cannot affect parity (it is not pinned against ggml).
// Host-only code; nothing here runs on the decode path.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#include <algorithm>
#ifdef _OPENMP
#include <omp.h>
#endif

#define SYN_API extern "C" __attribute__((visibility("default")))

namespace {

int g_threads = 0;  // 0 = OpenMP default

inline uint16_t f32_to_f16(float f) {
    uint32_t x; std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, e = (x >> 23) & 0xffu, m = x & 0x7fffffu;
    if (e == 0xff) return (uint16_t)(sign | 0x7c00u | (m ? (0x200u | (m >> 13)) : 0));
    int ne = (int)e - 127 + 15;
    if (ne >= 31) return (uint16_t)(sign | 0x7c00u);
    if (ne <= 0) {
        if (ne < -10) return (uint16_t)sign;
        m |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - ne), hm = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t hm = m >> 13, rem = m & 0x1fffu, out = sign | ((uint32_t)ne << 10) | hm;
    if (rem > 0x1000u || (rem == 0x1000u && (hm & 1u))) out++;
    return (uint16_t)out;
}
inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff, x;
    if (e == 0) {
        if (!m) x = sign;
        else { float v = std::ldexp((float)m, -24); std::memcpy(&x, &v, 4); x |= sign; }
    } else if (e == 31) x = sign | 0x7f800000u | (m << 13);
    else x = sign | ((e + 112) << 23) | (m << 13);
    float f; std::memcpy(&f, &x, 4); return f;
}

inline int nearest_int(float fval) {
    float val = fval + 12582912.f;
    int i; std::memcpy(&i, &val, 4);
    return (i & 0x007fffff) - 0x00400000;
}

// ---- Q8_0 / Q4_0 ---------------------------------------------------------
void quantize_row_q8_0(const float *x, uint8_t *y, size_t k) {
    for (size_t i = 0; i < k / 32; ++i, y += 34) {
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) amax = std::max(amax, std::fabs(x[i * 32 + j]));
        float d = amax / 127.0f, id = d ? 1.0f / d : 0.0f;
        uint16_t dh = f32_to_f16(d); std::memcpy(y, &dh, 2);
        for (int j = 0; j < 32; ++j) ((int8_t *)y)[2 + j] = (int8_t)std::roundf(x[i * 32 + j] * id);
    }
}
void quantize_row_q4_0(const float *x, uint8_t *y, size_t k) {
    for (size_t i = 0; i < k / 32; ++i, y += 18) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < 32; ++j) { float v = x[i * 32 + j]; if (amax < std::fabs(v)) { amax = std::fabs(v); max = v; } }
        float d = max / -8.0f, id = d ? 1.0f / d : 0.0f;
        uint16_t dh = f32_to_f16(d); std::memcpy(y, &dh, 2);
        for (int j = 0; j < 16; ++j) {
            float x0 = x[i * 32 + j] * id, x1 = x[i * 32 + 16 + j] * id;
            uint8_t xi0 = (uint8_t)std::min(15, (int)(int8_t)(x0 + 8.5f));
            uint8_t xi1 = (uint8_t)std::min(15, (int)(int8_t)(x1 + 8.5f));
            y[2 + j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}

// ---- Q4_1 / Q5_0 / Q5_1 / Q8_K (ggml's quantize_row_*_ref) --------------------
void quantize_row_q4_1(const float *x, uint8_t *y, size_t k) {
    for (size_t i = 0; i < k / 32; ++i, y += 20) {
        float mn = x[i * 32], mx = x[i * 32];
        for (int j = 1; j < 32; ++j) { mn = std::min(mn, x[i * 32 + j]); mx = std::max(mx, x[i * 32 + j]); }
        float d = (mx - mn) / 15.0f, id = d ? 1.0f / d : 0.0f;
        uint16_t dh = f32_to_f16(d), mh = f32_to_f16(mn);
        std::memcpy(y, &dh, 2); std::memcpy(y + 2, &mh, 2);
        for (int j = 0; j < 16; ++j) {
            float x0 = (x[i * 32 + j] - mn) * id, x1 = (x[i * 32 + 16 + j] - mn) * id;
            uint8_t xi0 = (uint8_t)std::min(15, (int)(int8_t)(x0 + 0.5f)), xi1 = (uint8_t)std::min(15, (int)(int8_t)(x1 + 0.5f));
            y[4 + j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}
void quantize_row_q5_0(const float *x, uint8_t *y, size_t k) {
    for (size_t i = 0; i < k / 32; ++i, y += 22) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < 32; ++j) { float v = x[i * 32 + j]; if (amax < std::fabs(v)) { amax = std::fabs(v); max = v; } }
        float d = max / -16.0f, id = d ? 1.0f / d : 0.0f;
        uint16_t dh = f32_to_f16(d); std::memcpy(y, &dh, 2);
        uint32_t qh = 0;
        for (int j = 0; j < 16; ++j) {
            float x0 = x[i * 32 + j] * id, x1 = x[i * 32 + 16 + j] * id;
            uint8_t xi0 = (uint8_t)std::min(31, (int)(int8_t)(x0 + 16.5f)), xi1 = (uint8_t)std::min(31, (int)(int8_t)(x1 + 16.5f));
            y[6 + j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (uint32_t)((xi0 & 0x10u) >> 4) << (j + 0);
            qh |= (uint32_t)((xi1 & 0x10u) >> 4) << (j + 16);
        }
        std::memcpy(y + 2, &qh, 4);
    }
}
void quantize_row_q5_1(const float *x, uint8_t *y, size_t k) {
    for (size_t i = 0; i < k / 32; ++i, y += 24) {
        float mn = x[i * 32], mx = x[i * 32];
        for (int j = 1; j < 32; ++j) { mn = std::min(mn, x[i * 32 + j]); mx = std::max(mx, x[i * 32 + j]); }
        float d = (mx - mn) / 31.0f, id = d ? 1.0f / d : 0.0f;
        uint16_t dh = f32_to_f16(d), mh = f32_to_f16(mn);
        std::memcpy(y, &dh, 2); std::memcpy(y + 2, &mh, 2);
        uint32_t qh = 0;
        for (int j = 0; j < 16; ++j) {
            float x0 = (x[i * 32 + j] - mn) * id, x1 = (x[i * 32 + 16 + j] - mn) * id;
            uint8_t xi0 = (uint8_t)(x0 + 0.5f), xi1 = (uint8_t)(x1 + 0.5f);
            y[8 + j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (uint32_t)((xi0 & 0x10u) >> 4) << (j + 0);
            qh |= (uint32_t)((xi1 & 0x10u) >> 4) << (j + 16);
        }
        std::memcpy(y + 4, &qh, 4);
    }
}
void quantize_row_q8_k(const float *x, uint8_t *y, size_t k) {
    for (size_t i = 0; i < k / 256; ++i, y += 292) {
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < 256; ++j) { float ax = std::fabs(x[i * 256 + j]); if (ax > amax) { amax = ax; max = x[i * 256 + j]; } }
        int8_t *qs = (int8_t *)(y + 4);
        int16_t bsums[16];
        if (!amax) { std::memset(y, 0, 292); continue; }
        const float iscale = -127.0f / max;
        for (int j = 0; j < 256; ++j) {
            int v = (int)std::nearbyintf(iscale * x[i * 256 + j]);
            qs[j] = (int8_t)std::min(127, v);
        }
        for (int j = 0; j < 16; ++j) { int sum = 0; for (int l = 0; l < 16; ++l) sum += qs[j * 16 + l]; bsums[j] = (int16_t)sum; }
        const float d = 1.0f / iscale;
        std::memcpy(y, &d, 4); std::memcpy(y + 260, bsums, 32);
    }
}

// ---- K-quants --------------------------------------------------------------
float make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *L, float *the_min,
                       uint8_t *Laux, float rmin, float rdelta, int nstep) {
    float min = x[0], max = x[0], sum_w = weights[0], sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        float w = weights[i]; sum_w += w; sum_x += w * x[i];
    }
    if (min > 0) min = 0;
    if (max == min) { for (int i = 0; i < n; ++i) L[i] = 0; *the_min = -min; return 0.f; }
    float iscale = nmax / (max - min), scale = 1 / iscale, best_mad = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * (x[i] - min));
        L[i] = (uint8_t)std::max(0, std::min(nmax, l));
        float diff = scale * L[i] + min - x[i];
        best_mad += weights[i] * diff * diff;
    }
    if (nstep < 1) { *the_min = -min; return scale; }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (max - min);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * (x[i] - min));
            l = std::max(0, std::min(nmax, l));
            Laux[i] = (uint8_t)l;
            float w = weights[i];
            sum_l += w * l; sum_l2 += w * l * l; sum_xl += w * l * x[i];
        }
        float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) { this_min = 0; this_scale = sum_xl / sum_l2; }
            float mad = 0;
            for (int i = 0; i < n; ++i) {
                float diff = this_scale * Laux[i] + this_min - x[i];
                mad += weights[i] * diff * diff;
            }
            if (mad < best_mad) {
                for (int i = 0; i < n; ++i) L[i] = Laux[i];
                best_mad = mad; scale = this_scale; min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

inline void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) { *d = q[j] & 63; *m = q[j + 4] & 63; }
    else { *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4)); *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4)); }
}

// Shared front half of Q4_K / Q5_K: sub-block scales/mins, 6-bit packing, d/dmin,
// and the final per-element levels L[256].  `scales12` is zero-initialised here.
void kquant_levels(const float *x, int nmax, float rmin, int nstep, uint8_t *scales12, uint16_t *d_out,
                   uint16_t *dmin_out, uint8_t *L) {
    uint8_t Laux[32]; float weights[32], mins[8], scales[8];
    float max_scale = 0, max_min = 0;
    for (int j = 0; j < 8; ++j) {
        float sum_x2 = 0;
        for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
        float av_x = std::sqrt(sum_x2 / 32);
        for (int l = 0; l < 32; ++l) weights[l] = av_x + std::fabs(x[32 * j + l]);
        scales[j] = make_qkx2_quants(32, nmax, x + 32 * j, weights, L + 32 * j, &mins[j], Laux, rmin, 0.1f, nstep);
        if (scales[j] > max_scale) max_scale = scales[j];
        if (mins[j] > max_min) max_min = mins[j];
    }
    float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    std::memset(scales12, 0, 12);
    for (int j = 0; j < 8; ++j) {
        uint8_t ls = (uint8_t)std::min(63, nearest_int(inv_scale * scales[j]));
        uint8_t lm = (uint8_t)std::min(63, nearest_int(inv_min * mins[j]));
        if (j < 4) { scales12[j] = ls; scales12[j + 4] = lm; }
        else {
            scales12[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            scales12[j - 4] |= (uint8_t)((ls >> 4) << 6);
            scales12[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    *d_out = f32_to_f16(max_scale / 63.f);
    *dmin_out = f32_to_f16(max_min / 63.f);
    float df = f16_to_f32(*d_out), dminf = f16_to_f32(*dmin_out);
    uint8_t sc, m;
    for (int j = 0; j < 8; ++j) {
        get_scale_min_k4(j, scales12, &sc, &m);
        float d = df * sc;
        if (!d) continue;
        float dm = dminf * m;
        for (int ii = 0; ii < 32; ++ii) {
            int l = nearest_int((x[32 * j + ii] + dm) / d);
            L[32 * j + ii] = (uint8_t)std::max(0, std::min(nmax, l));
        }
    }
}

void quantize_row_q4_k(const float *x, uint8_t *y, size_t k) {
    uint8_t L[256];
    for (size_t i = 0; i < k / 256; ++i, x += 256, y += 144) {
        uint16_t d, dmin;
        kquant_levels(x, 15, -1.f, 20, y + 4, &d, &dmin, L);
        std::memcpy(y, &d, 2); std::memcpy(y + 2, &dmin, 2);
        uint8_t *q = y + 16;
        for (int j = 0; j < 256; j += 64, q += 32)
            for (int l = 0; l < 32; ++l) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
    }
}
void quantize_row_q5_k(const float *x, uint8_t *y, size_t k) {
    uint8_t L[256];
    for (size_t i = 0; i < k / 256; ++i, x += 256, y += 176) {
        uint16_t d, dmin;
        kquant_levels(x, 31, -0.5f, 15, y + 4, &d, &dmin, L);
        std::memcpy(y, &d, 2); std::memcpy(y + 2, &dmin, 2);
        uint8_t *qh = y + 16, *ql = y + 48;
        std::memset(qh, 0, 32);
        uint8_t m1 = 1, m2 = 2;
        for (int n = 0; n < 256; n += 64, ql += 32) {
            for (int j = 0; j < 32; ++j) {
                int l1 = L[n + j]; if (l1 > 15) { l1 -= 16; qh[j] |= m1; }
                int l2 = L[n + j + 32]; if (l2 > 15) { l2 -= 16; qh[j] |= m2; }
                ql[j] = (uint8_t)(l1 | (l2 << 4));
            }
            m1 <<= 2; m2 <<= 2;
        }
    }
}

const float GROUP_MAX_EPS = 1e-15f;
float make_qx_quants(int n, int nmax, const float *x, int8_t *L) {  // rmse_type 1, no weights
    float max = 0, amax = 0;
    for (int i = 0; i < n; ++i) { float ax = std::fabs(x[i]); if (ax > amax) { amax = ax; max = x[i]; } }
    if (amax < GROUP_MAX_EPS) { for (int i = 0; i < n; ++i) L[i] = 0; return 0.f; }
    float iscale = -nmax / max, sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; ++i) {
        int l = std::max(-nmax, std::min(nmax - 1, nearest_int(iscale * x[i])));
        L[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        sumlx += w * x[i] * l; suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.0f, best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / max;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; ++i) {
            int l = std::max(-nmax, std::min(nmax - 1, nearest_int(iscale * x[i])));
            float w = x[i] * x[i];
            sumlx += w * x[i] * l; suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; ++i) {
                int l = nearest_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + std::max(-nmax, std::min(nmax - 1, l)));
            }
            scale = sumlx / suml2; best = scale * sumlx;
        }
    }
    return scale;
}
void quantize_row_q6_k(const float *x, uint8_t *y, size_t k) {
    int8_t L[256]; float scales[16];
    for (size_t i = 0; i < k / 256; ++i, x += 256, y += 210) {
        float max_scale = 0, max_abs_scale = 0;
        for (int ib = 0; ib < 16; ++ib) {
            float scale = make_qx_quants(16, 32, x + 16 * ib, L + 16 * ib);
            scales[ib] = scale;
            float a = std::fabs(scale);
            if (a > max_abs_scale) { max_abs_scale = a; max_scale = scale; }
        }
        if (max_abs_scale < GROUP_MAX_EPS) { std::memset(y, 0, 210); continue; }
        float iscale = -128.f / max_scale;
        uint16_t dh = f32_to_f16(1 / iscale); std::memcpy(y + 208, &dh, 2);
        int8_t *sc = (int8_t *)(y + 192);
        for (int ib = 0; ib < 16; ++ib) sc[ib] = (int8_t)std::min(127, nearest_int(iscale * scales[ib]));
        float df = f16_to_f32(dh);
        for (int j = 0; j < 16; ++j) {
            float d = df * sc[j];
            if (!d) continue;
            for (int ii = 0; ii < 16; ++ii) {
                int l = std::max(-32, std::min(31, nearest_int(x[16 * j + ii] / d)));
                L[16 * j + ii] = (int8_t)(l + 32);
            }
        }
        uint8_t *ql = y, *qh = y + 128;
        for (int j = 0; j < 256; j += 128, ql += 64, qh += 32) {
            for (int l = 0; l < 32; ++l) {
                uint8_t q1 = L[j + l] & 0xF, q2 = L[j + l + 32] & 0xF, q3 = L[j + l + 64] & 0xF, q4 = L[j + l + 96] & 0xF;
                ql[l] = (uint8_t)(q1 | (q3 << 4));
                ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
                qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) | ((L[j + l + 64] >> 4) << 4) | ((L[j + l + 96] >> 4) << 6));
            }
        }
    }
}

size_t row_bytes(int type, size_t ncols) {
    switch (type) {
    case 0: return ncols * 4;
    case 1: return ncols * 2;
    case 2: return ncols / 32 * 18;
    case 3: return ncols / 32 * 20;
    case 6: return ncols / 32 * 22;
    case 7: return ncols / 32 * 24;
    case 15: return ncols / 256 * 292;
    case 8: return ncols / 32 * 34;
    case 12: return ncols / 256 * 144;
    case 13: return ncols / 256 * 176;
    case 14: return ncols / 256 * 210;
    default: return 0;
    }
}
int block_elems(int type) { return type <= 1 ? 1 : (type == 2 || type == 8) ? 32 : 256; }

void quantize_row(int type, const float *x, uint8_t *y, size_t k) {
    switch (type) {
    case 0: std::memcpy(y, x, k * 4); break;
    case 1: for (size_t i = 0; i < k; ++i) { uint16_t h = f32_to_f16(x[i]); std::memcpy(y + 2 * i, &h, 2); } break;
    case 2: quantize_row_q4_0(x, y, k); break;
    case 3: quantize_row_q4_1(x, y, k); break;
    case 6: quantize_row_q5_0(x, y, k); break;
    case 7: quantize_row_q5_1(x, y, k); break;
    case 15: quantize_row_q8_k(x, y, k); break;
    case 8: quantize_row_q8_0(x, y, k); break;
    case 12: quantize_row_q4_k(x, y, k); break;
    case 13: quantize_row_q5_k(x, y, k); break;
    case 14: quantize_row_q6_k(x, y, k); break;
    }
}

// ---- counter-based normal generator ----------------------------------------
inline uint64_t splitmix64(uint64_t &s) {
    uint64_t z = (s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
// Values [first, first+n) of the stream `seed`; value i depends only on (seed, i/2),
// so any partition over threads gives the same array.
void normal_fill(uint64_t seed, size_t first, size_t n, float std, float *out) {
    size_t i = first, end = first + n;
    while (i < end) {
        size_t pair = i / 2;
        uint64_t s = seed * 0xd1342543de82ef95ull + pair * 0x2545f4914f6cdd1dull + 0x632be59bd9b4e019ull;
        uint64_t r = splitmix64(s);
        float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);  // (0,1]
        float u2 = (float)(uint32_t)((r >> 8) & 0xffffffu) * (1.0f / 16777216.0f);
        float rad = std::sqrt(-2.0f * std::log(u1)) * std;
        float ang = 6.28318530717958647692f * u2;
        float z0 = rad * std::cos(ang), z1 = rad * std::sin(ang);
        if ((i & 1) == 0) { out[i - first] = z0; ++i; if (i < end) { out[i - first] = z1; ++i; } }
        else { out[i - first] = z1; ++i; }
    }
}

}  // namespace

SYN_API void slai_synth_set_threads(int n) { g_threads = n; }

SYN_API size_t slai_synth_row_bytes(int type, size_t ncols) { return row_bytes(type, ncols); }

/// out[i] = std * N(0,1) for stream `seed`, i in [0, n).
SYN_API void slai_synth_normal(uint64_t seed, float std, float *out, size_t n) {
    const size_t chunk = 1 << 16;
    size_t nchunks = (n + chunk - 1) / chunk;
#pragma omp parallel for schedule(dynamic) num_threads(g_threads > 0 ? g_threads : omp_get_max_threads())
    for (size_t c = 0; c < nchunks; ++c) {
        size_t b = c * chunk, e = std::min(n, b + chunk);
        normal_fill(seed, b, e - b, std, out + b);
    }
}

/// Quantizes a row-major [nrows x ncols] fp32 matrix into GGUF blocks of `type`
/// (ggml type tag).  Returns bytes written, 0 if the type or shape is unsupported.
SYN_API size_t slai_synth_quantize(int type, const float *x, size_t nrows, size_t ncols, void *out) {
    size_t rb = row_bytes(type, ncols);
    if (!rb || ncols % (size_t)block_elems(type)) return 0;
#pragma omp parallel for schedule(dynamic, 8) num_threads(g_threads > 0 ? g_threads : omp_get_max_threads())
    for (size_t r = 0; r < nrows; ++r) quantize_row(type, x + r * ncols, (uint8_t *)out + r * rb, ncols);
    return rb * nrows;
}

/// Fused generate + quantize: the matrix is std*N(0,1) from stream `seed` (element
/// (r,c) is value r*ncols+c of the stream), never materialised in full.
SYN_API size_t slai_synth_normal_quantized(uint64_t seed, float std, int type, size_t nrows, size_t ncols, void *out) {
    size_t rb = row_bytes(type, ncols);
    if (!rb || ncols % (size_t)block_elems(type)) return 0;
#pragma omp parallel num_threads(g_threads > 0 ? g_threads : omp_get_max_threads())
    {
        std::vector<float> row(ncols);
#pragma omp for schedule(dynamic, 8)
        for (size_t r = 0; r < nrows; ++r) {
            normal_fill(seed, r * ncols, ncols, std, row.data());
            quantize_row(type, row.data(), (uint8_t *)out + r * rb, ncols);
        }
    }
    return rb * nrows;
}

SYN_API uint16_t slai_synth_f32_to_f16(float f) { return f32_to_f16(f); }
