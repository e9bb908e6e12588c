// Host-side mirror of the reference's op facade and tensor helpers:
// `LlmContext` (crates/slai/src/context.rs:69-96 and the op methods :205-501,:565-570,:660-672,:760-797)
// and the `GpuTensor` constructors / sub-views the decode path uses
// (crates/slai/src/models/llama2/transformer.rs:54-137,329-330).  Same method names and argument order
// (out-parameter first); every method forwards to the C ABI of include/slai_hip.h.
#pragma once
#include "slai_hip.h"

namespace slai {

// GpuTensor<f32>: an owned buffer plus its [nrows, ncols] shape (column-major like stensor's default).
struct GpuTensor {
    slai_buffer *buf = nullptr;
    uint32_t nrows = 0, ncols = 1;
    int dtype = SLAI_DT_F32;

    static int vector(slai_ctx *ctx, uint32_t n, uint32_t usage, GpuTensor *out, int dtype = SLAI_DT_F32) {
        return matrix(ctx, n, 1, usage, out, dtype);
    }
    static int matrix(slai_ctx *ctx, uint32_t nrows, uint32_t ncols, uint32_t usage, GpuTensor *out, int dtype = SLAI_DT_F32) {
        out->nrows = nrows; out->ncols = ncols; out->dtype = dtype;
        size_t esz = dtype == SLAI_DT_F16 ? 2 : (dtype == SLAI_DT_U8 ? 1 : 4);
        return slai_buffer_create(ctx, (size_t)nrows * ncols * esz, dtype, usage, &out->buf);
    }
    // `GpuTensor::vector(backend, data, usage)`: allocate and upload
    static int vector_from(slai_ctx *ctx, const float *data, uint32_t n, uint32_t usage, GpuTensor *out) {
        int rc = vector(ctx, n, usage, out);
        if (rc) return rc;
        return slai_write_buffer(ctx, out->buf, 0, data, (size_t)n * 4);
    }
    void destroy(slai_ctx *ctx) { if (buf) slai_buffer_destroy(ctx, buf); buf = nullptr; }

    slai_view view() const {
        slai_view v{buf, 0, {nrows, ncols, 1, 1}, {1, nrows, nrows * ncols, nrows * ncols}};
        return v;
    }
    // `.column(i)` (transformer.rs:329-330): one contiguous column of a column-major matrix
    slai_view column(uint32_t i) const {
        slai_view v{buf, (uint64_t)i * nrows, {nrows, 1, 1, 1}, {1, nrows, nrows, nrows}};
        return v;
    }
    // `.rows(start, n)` of a vector
    slai_view rows(uint32_t start, uint32_t n) const {
        slai_view v{buf, start, {n, 1, 1, 1}, {1, n, n, n}};
        return v;
    }
};

class LlmContext {
public:
    explicit LlmContext(slai_ctx *c) : ctx(c) {}
    slai_ctx *ctx;

    int begin_submission() { return slai_begin_submission(ctx); }                              // context.rs:79-88
    int submit() { return slai_submit(ctx); }                                                  // context.rs:90-95
    int rms_norm_assign(const slai_buffer *config, slai_view out, slai_view value, slai_view weight) {   // :230-246
        return slai_rms_norm_assign(ctx, config, out, value, weight);
    }
    int layernorm_assign(slai_view out, slai_view value, float eps) { return slai_layernorm_assign(ctx, out, value, eps); }  // :205-217
    int matmul_quant_assign(slai_view out, const slai_qmat *a, slai_view b) { return slai_matmul_quant_assign(ctx, out, a, b); }  // :355-369
    int matmul_assign(slai_view out, slai_view a, slai_view b, int a_mode, int b_mode) {      // :298-317
        return slai_matmul_assign(ctx, out, a, b, a_mode, b_mode);
    }
    int add_assign(slai_view in_out_a, slai_view b) { return slai_add_assign(ctx, in_out_a, b); }      // :428-441
    int mul_assign(slai_view in_out_a, slai_view b) { return slai_mul_assign(ctx, in_out_a, b); }      // :456-469
    int copy(slai_view in, slai_view out) { return slai_copy(ctx, in, out); }                          // :660-672
    int rope(int variant, const slai_buffer *config, slai_view in_out_q, slai_view in_out_k) {         // :471-487
        return slai_rope(ctx, variant, config, in_out_q, in_out_k);
    }
    int silu(slai_view in_out_h1, slai_view in_h2) { return slai_silu(ctx, in_out_h1, in_h2); }         // :489-501
    int gelu_inplace(slai_view x) { return slai_gelu_inplace(ctx, x); }                                 // :565-570
    int attn_mask(const slai_attn_params *params, const slai_buffer *params_gpu, slai_buffer *attn) {  // :760-785
        return slai_attn_mask(ctx, params, params_gpu, attn);
    }
    int softmax_cols(slai_view in_out_mat) { return slai_softmax_cols(ctx, in_out_mat); }               // :787-797
};

}  // namespace slai
