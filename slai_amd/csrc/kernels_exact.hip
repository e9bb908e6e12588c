// Kernels whose results must be bit-identical to the reference's CPU dequantizers
// (crates/slai/src/quantization.rs, crates/slai/src/gguf.rs:116-131): device-layout repack,
// row dequantisation and the embedding-row gather.  This translation unit is compiled with
// -ffp-contract=off so that `d * q - m` stays two roundings.
#include "common.h"
#include "quant_formats.h"

namespace slai {
namespace {

__global__ void repack_kernel(int type, const uint8_t *src, uint8_t *dst, uint32_t nrows, uint32_t nb, size_t gguf_row,
                              size_t dev_row, int bb) {
    const size_t total = (size_t)nrows * nb;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const uint32_t r = (uint32_t)(i / nb), b = (uint32_t)(i % nb);
        repack_block(type, src + (size_t)r * gguf_row + (size_t)b * bb, dst + (size_t)r * dev_row, nb, b);
    }
}

// f32 / f16 rows: plain byte copy with the padded device stride
__global__ void copy_rows_kernel(const uint8_t *src, uint8_t *dst, uint32_t nrows, size_t gguf_row, size_t dev_row) {
    const size_t words = gguf_row / 2;  // rows are multiples of 2 bytes
    const size_t total = (size_t)nrows * words;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / words, w = i % words;
        reinterpret_cast<uint16_t *>(dst + r * dev_row)[w] = reinterpret_cast<const uint16_t *>(src + r * gguf_row)[w];
    }
}

__global__ void dequant_rows_kernel(int type, const uint8_t *dev, size_t row_stride, uint32_t nb, uint32_t row0,
                                    uint32_t nrows, uint32_t ncols, float *out, size_t out_stride) {
    const size_t total = (size_t)nrows * ncols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const uint32_t r = (uint32_t)(i / ncols), c = (uint32_t)(i % ncols);
        out[(size_t)r * out_stride + c] = dequant_elem(type, dev + (size_t)(row0 + r) * row_stride, nb, c);
    }
}

__global__ void embed_kernel(int type_a, const uint8_t *a, size_t stride_a, uint32_t nb_a, const int *row_a, int type_b,
                             const uint8_t *b, size_t stride_b, uint32_t nb_b, const int *row_b, uint32_t ncols,
                             float *out) {
    const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= ncols) return;
    float v = dequant_elem(type_a, a + (size_t)(*row_a) * stride_a, nb_a, c);
    // gpt2/cpu.rs:227-228: token embedding first, then += position embedding
    if (b) v = v + dequant_elem(type_b, b + (size_t)(*row_b) * stride_b, nb_b, c);
    out[c] = v;
}

}  // namespace

hipError_t launch_repack(hipStream_t s, int type, const uint8_t *src, uint8_t *dst, uint32_t nrows, uint32_t ncols) {
    const uint32_t nb = ncols / block_elems(type);
    const size_t gr = gguf_row_bytes(type, ncols), dr = device_row_stride(type, ncols);
    if (type == T_F32 || type == T_F16) {
        if (gr == dr) return hipMemcpyAsync(dst, src, gr * nrows, hipMemcpyDeviceToDevice, s);
        copy_rows_kernel<<<1024, 256, 0, s>>>(src, dst, nrows, gr, dr);
    } else {
        repack_kernel<<<2048, 256, 0, s>>>(type, src, dst, nrows, nb, gr, dr, block_bytes(type));
    }
    return hipGetLastError();
}

hipError_t launch_dequant_rows(hipStream_t s, int type, const uint8_t *dev, size_t row_stride, uint32_t nb, uint32_t row0,
                               uint32_t nrows, uint32_t ncols, float *out, size_t out_stride) {
    size_t total = (size_t)nrows * ncols;
    uint32_t grid = (uint32_t)((total + 255) / 256);
    if (grid > 65536) grid = 65536;
    if (grid == 0) return hipSuccess;
    dequant_rows_kernel<<<grid, 256, 0, s>>>(type, dev, row_stride, nb, row0, nrows, ncols, out, out_stride);
    return hipGetLastError();
}

hipError_t launch_embed(hipStream_t s, int type_a, const uint8_t *a, size_t stride_a, uint32_t nb_a, const int *row_a,
                        int type_b, const uint8_t *b, size_t stride_b, uint32_t nb_b, const int *row_b, uint32_t ncols,
                        float *out) {
    embed_kernel<<<(ncols + 255) / 256, 256, 0, s>>>(type_a, a, stride_a, nb_a, row_a, type_b, b, stride_b, nb_b, row_b,
                                                      ncols, out);
    return hipGetLastError();
}

}  // namespace slai
