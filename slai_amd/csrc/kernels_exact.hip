// Kernels whose results must be bit-identical to the reference's CPU dequantizers
// (crates/slai/src/quantization.rs, crates/slai/src/gguf.rs:116-131): device-layout repack,
// row dequantisation and the embedding-row gather.  This translation unit is compiled with
// -ffp-contract=off so that `d * q - m` stays two roundings.
#include "common.h"
#include "quant_formats.h"
#include "quant_tiled.h"

namespace slai {

QMatDev qmat_dev(const slai_qmat *m) {
    QMatDev d{};
    if (!m) return d;
    d.type = m->type; d.tiled = m->tiled ? 1 : 0; d.dptr = m->dptr; d.row_stride = m->row_stride; d.nb = m->nb;
    d.nrows = m->nrows; d.ncols = m->ncols; d.rows_log2 = m->rows_log2; d.ncb = m->ncb; d.ngroups = m->ngroups;
    d.ntiles = m->ntiles; d.unit_bytes = m->unit_bytes;
    return d;
}

namespace {

__device__ __forceinline__ TiledGeom geom_of(const QMatDev &m) {
    TiledGeom g;
    g.type = m.type; g.nrows = m.nrows; g.ncols = m.ncols; g.rows_log2 = m.rows_log2; g.ncb = m.ncb; g.ngroups = m.ngroups;
    g.ntiles = m.ntiles; g.pieces = tiled_pieces(m.type); g.unit_bytes = m.unit_bytes;
    return g;
}
__device__ __forceinline__ float qmat_elem(const QMatDev &m, uint32_t row, uint32_t col) {
    if (m.tiled) return tiled_dequant_elem(geom_of(m), m.dptr, row, col);
    return dequant_elem(m.type, m.dptr + (size_t)row * m.row_stride, m.nb, col);
}

__global__ void repack_kernel(QMatDev m, uint8_t *dst, const uint8_t *src, size_t gguf_row, int bb) {
    const size_t total = (size_t)m.nrows * m.nb;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const uint32_t r = (uint32_t)(i / m.nb), b = (uint32_t)(i % m.nb);
        const uint8_t *blk = src + (size_t)r * gguf_row + (size_t)b * bb;
        if (m.tiled) tiled_repack_block(geom_of(m), blk, dst, r, b);
        else repack_block(m.type, blk, dst + (size_t)r * m.row_stride, m.nb, b);
    }
}

// f32 / f16 rows: plain copy with the padded device stride
__global__ void copy_rows_kernel(const uint8_t *src, uint8_t *dst, uint32_t nrows, size_t gguf_row, size_t dev_row) {
    const size_t words = gguf_row / 2;  // rows are multiples of 2 bytes
    const size_t total = (size_t)nrows * words;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / words, w = i % words;
        reinterpret_cast<uint16_t *>(dst + r * dev_row)[w] = reinterpret_cast<const uint16_t *>(src + r * gguf_row)[w];
    }
}

__global__ void dequant_rows_kernel(QMatDev m, uint32_t row0, uint32_t nrows, float *out, size_t out_stride) {
    const size_t total = (size_t)nrows * m.ncols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const uint32_t r = (uint32_t)(i / m.ncols), c = (uint32_t)(i % m.ncols);
        out[(size_t)r * out_stride + c] = qmat_elem(m, row0 + r, c);
    }
}

__global__ void embed_kernel(QMatDev a, const int *row_a, QMatDev b, const int *row_b, int has_b, uint32_t ncols, float *out) {
    const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= ncols) return;
    float v = qmat_elem(a, (uint32_t)*row_a, c);
    // gpt2/cpu.rs:227-228: token embedding first, then += position embedding
    if (has_b) v = v + qmat_elem(b, (uint32_t)*row_b, c);
    out[c] = v;
}

// one embedding row per token of a chunk: grid = (columns / 256, tokens)
__global__ void embed_rows_kernel(QMatDev a, const int *rows, QMatDev pm, const int *positions, int has_pos, uint32_t ncols, float *out, uint32_t out_stride) {
    const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (c >= ncols) return;
    float v = qmat_elem(a, (uint32_t)rows[b], c);
    if (has_pos) v = v + qmat_elem(pm, (uint32_t)positions[b], c);     // gpt2/cpu.rs:227-228
    out[(size_t)b * out_stride + c] = v;
}

}  // namespace

hipError_t launch_repack(hipStream_t s, const slai_qmat *m, const uint8_t *src) {
    const size_t gr = gguf_row_bytes(m->type, m->ncols);
    if (!m->tiled && (m->type == T_F32 || m->type == T_F16)) {
        if (gr == m->row_stride) return hipMemcpyAsync(m->dptr, src, gr * m->nrows, hipMemcpyDeviceToDevice, s);
        copy_rows_kernel<<<1024, 256, 0, s>>>(src, m->dptr, m->nrows, gr, m->row_stride);
    } else {
        repack_kernel<<<2048, 256, 0, s>>>(qmat_dev(m), m->dptr, src, gr, block_bytes(m->type));
    }
    return hipGetLastError();
}

hipError_t launch_dequant_rows(hipStream_t s, const slai_qmat *m, uint32_t row0, uint32_t nrows, float *out, size_t out_stride) {
    size_t total = (size_t)nrows * m->ncols;
    uint32_t grid = (uint32_t)((total + 255) / 256);
    if (grid > 65536) grid = 65536;
    if (grid == 0) return hipSuccess;
    dequant_rows_kernel<<<grid, 256, 0, s>>>(qmat_dev(m), row0, nrows, out, out_stride);
    return hipGetLastError();
}

hipError_t launch_embed(hipStream_t s, const slai_qmat *a, const int *row_a, const slai_qmat *b, const int *row_b, uint32_t ncols, float *out) {
    embed_kernel<<<(ncols + 255) / 256, 256, 0, s>>>(qmat_dev(a), row_a, qmat_dev(b), row_b, b ? 1 : 0, ncols, out);
    return hipGetLastError();
}

hipError_t launch_embed_rows(hipStream_t s, const slai_qmat *m, const int *tokens, uint32_t n, uint32_t ncols, float *out, uint32_t out_stride,
                             const slai_qmat *pos_m, const int *positions) {
    if (n == 0 || n > 65535 || (pos_m && !positions)) return hipErrorInvalidValue;
    embed_rows_kernel<<<dim3((ncols + 255) / 256, n), 256, 0, s>>>(qmat_dev(m), tokens, qmat_dev(pos_m), positions, pos_m ? 1 : 0, ncols, out, out_stride);
    return hipGetLastError();
}

}  // namespace slai
