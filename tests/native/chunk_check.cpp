// Host build of the device-side layout/decoder header, for CPU tests of its index math.
// Compiled by tests/test_chunks_host.py with g++ -ffp-contract=off.
#include "quant_formats.h"
#include "quant_tiled.h"
#include <vector>

using namespace slai;

extern "C" {

size_t cc_row_stride(int t, uint32_t ncols) { return device_row_stride(t, ncols); }

// verbatim GGUF rows -> device layout
void cc_repack(int t, const uint8_t *src, uint32_t nrows, uint32_t ncols, uint8_t *dst) {
    uint32_t nb = ncols / block_elems(t);
    size_t rs = device_row_stride(t, ncols), gs = gguf_row_bytes(t, ncols);
    for (uint32_t r = 0; r < nrows; ++r)
        for (uint32_t b = 0; b < nb; ++b)
            repack_block(t, src + r * gs + (size_t)b * block_bytes(t), dst + r * rs, nb, b);
}

void cc_dequant(int t, const uint8_t *dev, uint32_t nrows, uint32_t ncols, float *out) {
    uint32_t nb = ncols / block_elems(t);
    size_t rs = device_row_stride(t, ncols);
    for (uint32_t r = 0; r < nrows; ++r)
        for (uint32_t c = 0; c < ncols; ++c) out[(size_t)r * ncols + c] = dequant_elem(t, dev + r * rs, nb, c);
}

}  // extern "C"

template <int T> static void gemv_t(const uint8_t *dev, uint32_t nrows, uint32_t ncols, const float *xv, float *out) {
    using F = Chunk<T>;
    uint32_t nb = ncols / block_elems(T), nc = F::nchunks(ncols);
    size_t rs = device_row_stride(T, ncols);
    for (uint32_t r = 0; r < nrows; ++r) {
        double acc = 0;
        for (uint32_t c = 0; c < nc; ++c) {
            float x[F::E], xs[F::NRUN];
            for (int q = 0; q < F::NRUN; ++q) {
                xs[q] = 0;
                for (int i = 0; i < F::RUNLEN; ++i) { x[q * F::RUNLEN + i] = xv[F::run_col(c, q) + i]; xs[q] += x[q * F::RUNLEN + i]; }
            }
            typename F::Data d = F::load(dev + r * rs, nb, c);
            acc += (double)F::dot(d, c, x, xs);
        }
        out[r] = (float)acc;
    }
}

// returns the number of columns covered exactly once by the chunk->column map (must equal ncols)
template <int T> static uint32_t cover_t(uint32_t ncols) {
    using F = Chunk<T>;
    std::vector<int> seen(ncols, 0);
    for (uint32_t c = 0; c < F::nchunks(ncols); ++c)
        for (int q = 0; q < F::NRUN; ++q)
            for (int i = 0; i < F::RUNLEN; ++i) { uint32_t col = F::run_col(c, q) + i; if (col < ncols) seen[col]++; }
    uint32_t ok = 0;
    for (uint32_t c = 0; c < ncols; ++c) ok += seen[c] == 1;
    return ok;
}

extern "C" {

int cc_gemv(int t, const uint8_t *dev, uint32_t nrows, uint32_t ncols, const float *x, float *out) {
    switch (t) {
    case T_F32: gemv_t<T_F32>(dev, nrows, ncols, x, out); break;
    case T_F16: gemv_t<T_F16>(dev, nrows, ncols, x, out); break;
    case T_Q4_0: gemv_t<T_Q4_0>(dev, nrows, ncols, x, out); break;
    case T_Q4_1: gemv_t<T_Q4_1>(dev, nrows, ncols, x, out); break;
    case T_Q5_0: gemv_t<T_Q5_0>(dev, nrows, ncols, x, out); break;
    case T_Q5_1: gemv_t<T_Q5_1>(dev, nrows, ncols, x, out); break;
    case T_Q8_K: gemv_t<T_Q8_K>(dev, nrows, ncols, x, out); break;
    case T_Q8_0: gemv_t<T_Q8_0>(dev, nrows, ncols, x, out); break;
    case T_Q4_K: gemv_t<T_Q4_K>(dev, nrows, ncols, x, out); break;
    case T_Q5_K: gemv_t<T_Q5_K>(dev, nrows, ncols, x, out); break;
    case T_Q6_K: gemv_t<T_Q6_K>(dev, nrows, ncols, x, out); break;
    default: return -1;
    }
    return 0;
}
uint32_t cc_cover(int t, uint32_t ncols) {
    switch (t) {
    case T_F32: return cover_t<T_F32>(ncols);
    case T_F16: return cover_t<T_F16>(ncols);
    case T_Q4_0: return cover_t<T_Q4_0>(ncols);
    case T_Q4_1: return cover_t<T_Q4_1>(ncols);
    case T_Q5_0: return cover_t<T_Q5_0>(ncols);
    case T_Q5_1: return cover_t<T_Q5_1>(ncols);
    case T_Q8_K: return cover_t<T_Q8_K>(ncols);
    case T_Q8_0: return cover_t<T_Q8_0>(ncols);
    case T_Q4_K: return cover_t<T_Q4_K>(ncols);
    case T_Q5_K: return cover_t<T_Q5_K>(ncols);
    case T_Q6_K: return cover_t<T_Q6_K>(ncols);
    default: return 0;
    }
}
uint16_t cc_encode_f16(float f) { return encode_f16(f); }
float cc_decode_f16(uint16_t h) { return decode_f16(h); }
}

// ---- tiled layout ---------------------------------------------------------------------------
struct HostX {
    const float *xb;   // the 256 activations of one cblock
    template <int I1, int I2> struct St {};
    template <int I1, int I2> St<I1, I2> stage() const { return {}; }
    template <int SLOT, int W, int I1, int I2> float fma4(St<I1, I2>, uint32_t w, float acc) const {
        const int I = SLOT ? I2 : I1;
        for (int b = 0; b < 4; ++b) acc = fmaf((float)((w >> (8 * b)) & 0xffu), xb[16 * I + 4 * W + b], acc);
        return acc;
    }
    float sum16(int i) const { float t = 0; for (int k = 0; k < 16; ++k) t += xb[16 * i + k]; return t; }
};

template <int T> static void tiled_gemv_t(const TiledGeom &g, const uint8_t *dev, const float *xv, float *out) {
    using F = Tiled<T>;
    const uint32_t rows = 1u << g.rows_log2, kqn = 64u >> g.rows_log2;
    std::vector<float> xz(256, 0.0f);
    for (uint32_t row = 0; row < g.nrows; ++row) {
        double acc = 0;
        for (uint32_t cb = 0; cb < g.ngroups * kqn; ++cb) {
            const uint32_t t = row >> g.rows_log2, r = row & (rows - 1), grp = cb / kqn, kq = cb % kqn, lane = kq * rows + r;
            const uint8_t *unit = dev + ((size_t)t * g.ngroups + grp) * g.unit_bytes;
            typename F::Data d;
            for (int p = 0; p < F::PT; ++p) memcpy(&d.p[p], unit + (size_t)p * 1024 + lane * 16, 16);
            uint16_t tail = 0;
            if (F::TAIL) memcpy(&tail, unit + (size_t)F::PT * 1024 + lane * 2, 2);
            HostX x{cb < g.ncb ? xv + (size_t)cb * 256 : xz.data()};
            acc += (double)F::dot(d, tail, x);
        }
        out[row] = (float)acc;
    }
}

extern "C" {
size_t cc_tiled_bytes(int t, uint32_t nrows, uint32_t ncols) { return tiled_bytes(tiled_geom(t, nrows, ncols)); }
uint32_t cc_tiled_rows_log2(int t, uint32_t nrows, uint32_t ncols) { return tiled_geom(t, nrows, ncols).rows_log2; }
void cc_tiled_repack(int t, const uint8_t *src, uint32_t nrows, uint32_t ncols, uint8_t *dst) {
    TiledGeom g = tiled_geom(t, nrows, ncols);
    uint32_t nb = ncols / block_elems(t);
    size_t gs = gguf_row_bytes(t, ncols);
    for (uint32_t r = 0; r < nrows; ++r)
        for (uint32_t b = 0; b < nb; ++b) tiled_repack_block(g, src + r * gs + (size_t)b * block_bytes(t), dst, r, b);
}
void cc_tiled_dequant(int t, const uint8_t *dev, uint32_t nrows, uint32_t ncols, float *out) {
    TiledGeom g = tiled_geom(t, nrows, ncols);
    for (uint32_t r = 0; r < nrows; ++r)
        for (uint32_t c = 0; c < ncols; ++c) out[(size_t)r * ncols + c] = tiled_dequant_elem(g, dev, r, c);
}
int cc_tiled_gemv(int t, const uint8_t *dev, uint32_t nrows, uint32_t ncols, const float *x, float *out) {
    TiledGeom g = tiled_geom(t, nrows, ncols);
    switch (t) {
    case T_Q4_K: tiled_gemv_t<T_Q4_K>(g, dev, x, out); break;
    case T_Q6_K: tiled_gemv_t<T_Q6_K>(g, dev, x, out); break;
    case T_Q8_0: tiled_gemv_t<T_Q8_0>(g, dev, x, out); break;
    case T_Q4_0: tiled_gemv_t<T_Q4_0>(g, dev, x, out); break;
    case T_Q5_K: tiled_gemv_t<T_Q5_K>(g, dev, x, out); break;
    default: return -1;
    }
    return 0;
}
}
