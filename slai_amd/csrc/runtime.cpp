// C-ABI runtime of libslai_hip: context, buffers, quantized matrices, the LlmContext op
// facade (crates/slai/src/context.rs) and HIP-graph capture.  Declarations and the reference
// interfaces they replace are in include/slai_hip.h.
#include "common.h"
#include "quant_formats.h"
#include "quant_tiled.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace slai {

int set_error(slai_ctx *ctx, int code, const std::string &msg) {
    if (ctx) ctx->err = msg;
    return code;
}
int hip_fail(slai_ctx *ctx, hipError_t e, const char *what) {
    return set_error(ctx, SLAI_E_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

static int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}

static bool view_is_vector(const slai_view &v) { return v.size[1] == 1 && v.size[2] == 1 && v.size[3] == 1; }
static uint32_t view_len(const slai_view &v) { return v.size[0] * v.size[1] * v.size[2] * v.size[3]; }

// A view used as a flat vector: either a genuine vector, or any contiguous tensor.
static bool as_vec(const slai_view &v, VecView *out) {
    if (!v.buf || v.buf->dtype != SLAI_DT_F32) return false;
    uint32_t n = view_len(v), stride;
    if (view_is_vector(v)) stride = v.stride[0] ? v.stride[0] : 1;
    else {
        // contiguous column-major or row-major block
        bool cm = v.stride[0] == 1 && (v.size[1] == 1 || v.stride[1] == v.size[0]);
        bool rm = v.stride[1] == 1 && (v.size[0] == 1 || v.stride[0] == v.size[1]);
        if (!(cm || rm) || v.size[2] != 1 || v.size[3] != 1) return false;
        stride = 1;
    }
    if (n == 0) return false;
    size_t last = v.offset + (size_t)(n - 1) * stride;
    if ((last + 1) * sizeof(float) > v.buf->bytes) return false;
    out->p = reinterpret_cast<float *>(v.buf->dptr) + v.offset;
    out->n = n;
    out->stride = stride;
    return true;
}

static bool as_view4(const slai_view &v, View4 *out) {
    if (!v.buf || v.buf->dtype != SLAI_DT_F32) return false;
    size_t last = v.offset;
    for (int d = 0; d < 4; ++d) {
        if (v.size[d] == 0) return false;
        last += (size_t)(v.size[d] - 1) * v.stride[d];
    }
    if ((last + 1) * sizeof(float) > v.buf->bytes) return false;
    out->p = reinterpret_cast<float *>(v.buf->dptr) + v.offset;
    for (int d = 0; d < 4; ++d) { out->size[d] = v.size[d]; out->stride[d] = v.stride[d]; }
    return true;
}

}  // namespace slai

using namespace slai;

// ---- context ------------------------------------------------------------------
SLAI_EXPORT int slai_ctx_create(int device, slai_ctx **out) {
    if (!out) return SLAI_E_ARG;
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) return SLAI_E_HIP;
    if (hipSetDevice(device) != hipSuccess) return SLAI_E_HIP;
    if (attention_static_setup(device) != hipSuccess) return SLAI_E_HIP;   // (this device's address of the static attention scratch)
    slai_ctx *ctx = new slai_ctx();
    ctx->device = device;
    if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) { delete ctx; return SLAI_E_HIP; }
    ctx->gemv_rows_per_wg = env_int("SLAI_GEMV_ROWS_PER_WG", 8);
    ctx->gemv_max_threads = env_int("SLAI_GEMV_MAX_THREADS", 512);
    ctx->attn_splits = env_int("SLAI_ATTN_SPLITS", 0);
    ctx->use_graph = env_int("SLAI_NO_GRAPH", 0) == 0;
    ctx->prompt_gemm = env_int("SLAI_PROMPT_GEMM", 1) != 0;
    ctx->prompt_split_f16 = env_int("SLAI_PROMPT_SPLIT_F16", 1);
    if (hipMalloc((void **)&ctx->split_flag, sizeof(int)) != hipSuccess || hipMemset(ctx->split_flag, 0, sizeof(int)) != hipSuccess) {
        (void)hipStreamDestroy(ctx->stream); delete ctx; return SLAI_E_HIP;
    }
    ctx->gemv_max_wgs = env_int("SLAI_GEMV_MAX_WGS", 512);
    ctx->tiled_layout = env_int("SLAI_TILED", 1) != 0;
    ctx->rowtile_gemv = env_int("SLAI_ROWTILE", 1) != 0;
    ctx->fuse_qkv_attention = env_int("SLAI_FUSE_QKV_ATTN", 1) != 0;
    ctx->persistent = env_int("SLAI_PERSISTENT", 1) != 0;
    ctx->resident_max_pos = (uint32_t)std::max(0, env_int("SLAI_RESIDENT_MAX_POS", 2048));
    *out = ctx;
    return SLAI_OK;
}

static void buffer_free(slai_buffer *b) {
    if (b->dptr) (void)hipFree(b->dptr);
    if (b->host_staging) (void)hipHostFree(b->host_staging);
    delete b;
}

SLAI_EXPORT void slai_ctx_destroy(slai_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->attn_scratch) (void)hipFree(ctx->attn_scratch);
    if (ctx->gemv_scratch) (void)hipFree(ctx->gemv_scratch);
    if (ctx->split_flag) (void)hipFree(ctx->split_flag);
    if (ctx->sampler_scratch) (void)hipFree(ctx->sampler_scratch);
    if (ctx->handoff_counters) (void)hipFree(ctx->handoff_counters);
    for (void *p : ctx->retired_scratch) (void)hipFree(p);
    for (slai_buffer *b : ctx->retired_buffers) buffer_free(b);
    if (ctx->timer0) (void)hipEventDestroy(ctx->timer0);
    if (ctx->timer1) (void)hipEventDestroy(ctx->timer1);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

SLAI_EXPORT const char *slai_last_error(slai_ctx *ctx) { return ctx ? ctx->err.c_str() : "null context"; }
SLAI_EXPORT void *slai_ctx_stream(slai_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

// context.rs:79-95.  The reference records launches into an encoder and hands it to the queue on submit; here every
// launch goes to the context's stream at once, so the pair only keeps the reference's state rules: beginning while a
// submission is open submits it first, submitting with none open does nothing.  Both are legal inside a graph capture.
SLAI_EXPORT int slai_begin_submission(slai_ctx *ctx) {
    if (!ctx) return SLAI_E_ARG;
    if (ctx->submission_open) slai_submit(ctx);
    ctx->submission_open = true;
    return SLAI_OK;
}
SLAI_EXPORT int slai_submit(slai_ctx *ctx) {
    if (!ctx) return SLAI_E_ARG;
    ctx->submission_open = false;
    return SLAI_OK;
}
SLAI_EXPORT int slai_synchronize(slai_ctx *ctx) {
    if (!ctx) return SLAI_E_ARG;
    SLAI_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return SLAI_OK;
}

// ---- buffers --------------------------------------------------------------------
SLAI_EXPORT int slai_buffer_create(slai_ctx *ctx, size_t bytes, int dtype, uint32_t usage, slai_buffer **out) {
    if (!ctx || !out) return SLAI_E_ARG;
    *out = nullptr;
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "slai_buffer_create during graph capture");
    if (dtype < SLAI_DT_F32 || dtype > SLAI_DT_I32) return set_error(ctx, SLAI_E_ARG, "bad dtype");
    slai_buffer *b = new slai_buffer();
    b->bytes = bytes; b->dtype = dtype; b->usage = usage;
    size_t alloc = bytes ? bytes : 16;
    hipError_t e = hipMalloc(&b->dptr, alloc);
    if (e == hipSuccess) e = hipMemsetAsync(b->dptr, 0, alloc, ctx->stream);
    if (e == hipSuccess && (usage & SLAI_USAGE_MAP_READ)) e = hipHostMalloc(&b->host_staging, alloc, hipHostMallocDefault);
    if (e != hipSuccess) {
        if (b->dptr) (void)hipFree(b->dptr);
        delete b;
        return hip_fail(ctx, e, "slai_buffer_create");
    }
    *out = b;
    return SLAI_OK;
}

SLAI_EXPORT void slai_buffer_destroy(slai_ctx *ctx, slai_buffer *b) {
    if (!b) return;
    if (b->idle_in_cache) {
        // its cache still lists it and would hand the freed memory to the next get_or_insert: the cache frees it (clear / destroy)
        if (ctx) set_error(ctx, SLAI_E_STATE, "slai_buffer_destroy: the buffer sits idle in a tensor cache; clear or destroy the cache instead");
        return;
    }
    if (ctx && ctx->capturing) {
        // no synchronisation and no free inside a capture: the buffer is kept until the context goes
        ctx->retired_buffers.push_back(b);
        return;
    }
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    buffer_free(b);
}
SLAI_EXPORT size_t slai_buffer_size(const slai_buffer *b) { return b ? b->bytes : 0; }
SLAI_EXPORT void *slai_buffer_device_ptr(const slai_buffer *b) { return b ? b->dptr : nullptr; }

SLAI_EXPORT int slai_write_buffer(slai_ctx *ctx, slai_buffer *b, size_t offset, const void *src, size_t bytes) {
    if (!ctx || !b || (!src && bytes)) return SLAI_E_ARG;
    if (offset + bytes > b->bytes) return set_error(ctx, SLAI_E_SHAPE, "slai_write_buffer: out of range");
    if (!bytes) return SLAI_OK;
    SLAI_HIP_TRY(ctx, hipMemcpyAsync((char *)b->dptr + offset, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    // pageable source: the copy must have consumed `src` before the caller reuses it
    SLAI_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return SLAI_OK;
}

SLAI_EXPORT int slai_read_buffer(slai_ctx *ctx, const slai_buffer *b, size_t offset, void *dst, size_t bytes) {
    if (!ctx || !b || (!dst && bytes)) return SLAI_E_ARG;
    if (offset + bytes > b->bytes) return set_error(ctx, SLAI_E_SHAPE, "slai_read_buffer: out of range");
    if (!bytes) return SLAI_OK;
    if (b->host_staging) {
        SLAI_HIP_TRY(ctx, hipMemcpyAsync((char *)b->host_staging + offset, (const char *)b->dptr + offset, bytes,
                                         hipMemcpyDeviceToHost, ctx->stream));
        SLAI_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        memcpy(dst, (const char *)b->host_staging + offset, bytes);
    } else {
        SLAI_HIP_TRY(ctx, hipMemcpyAsync(dst, (const char *)b->dptr + offset, bytes, hipMemcpyDeviceToHost, ctx->stream));
        SLAI_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    }
    return SLAI_OK;
}

SLAI_EXPORT int slai_copy_buffer(slai_ctx *ctx, slai_buffer *dst, size_t dst_offset, const slai_buffer *src,
                                 size_t src_offset, size_t bytes) {
    if (!ctx || !dst || !src) return SLAI_E_ARG;
    if (dst_offset + bytes > dst->bytes || src_offset + bytes > src->bytes)
        return set_error(ctx, SLAI_E_SHAPE, "slai_copy_buffer: out of range");
    if (!bytes) return SLAI_OK;
    SLAI_HIP_TRY(ctx, hipMemcpyAsync((char *)dst->dptr + dst_offset, (const char *)src->dptr + src_offset, bytes,
                                     hipMemcpyDeviceToDevice, ctx->stream));
    return SLAI_OK;
}

// ---- temporaries (crates/slai/src/tensor_cache.rs) ---------------------------------------------
SLAI_EXPORT int slai_tensor_cache_create(slai_ctx *ctx, slai_tensor_cache **out) {
    if (!ctx || !out) return SLAI_E_ARG;
    *out = new slai_tensor_cache();
    return SLAI_OK;
}
// `TensorCache::clear` (tensor_cache.rs:195-197): idle tensors are freed; those handed out stay with their holders.
// A tensor that was handed out while a graph was being captured may be named by that graph for as long as the graph
// lives, so its memory is not freed here: it is retired and goes with the context (as grown scratch blocks do).
static void cache_release(slai_ctx *ctx, slai_tensor_cache *c, bool may_free) {
    bool synced = false;
    for (auto &kv : c->tensors)
        for (slai_buffer *b : kv.second) {
            b->idle_in_cache = false;
            if (!may_free || b->captured) { ctx->retired_buffers.push_back(b); continue; }
            if (!synced) { (void)hipStreamSynchronize(ctx->stream); synced = true; }
            buffer_free(b);
        }
    c->tensors.clear();
}
SLAI_EXPORT int slai_tensor_cache_clear(slai_ctx *ctx, slai_tensor_cache *c) {
    if (!ctx || !c) return SLAI_E_ARG;
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "slai_tensor_cache_clear during graph capture");
    cache_release(ctx, c, true);
    return SLAI_OK;
}
// Inside a capture nothing is synchronised or freed and the capture goes on: the idle tensors are retired.
SLAI_EXPORT void slai_tensor_cache_destroy(slai_ctx *ctx, slai_tensor_cache *c) {
    if (!c) return;
    if (ctx) cache_release(ctx, c, !ctx->capturing);
    delete c;
}
// `TensorCache::get_or_insert` (tensor_cache.rs:162-188) with the insert closure of context.rs:107-127: an idle tensor of
// this element type, shape and usage if the cache has one (its contents are whatever its last holder left), a new
// zero-filled buffer otherwise.  A hit allocates nothing and is legal during graph capture; a miss is not.
SLAI_EXPORT int slai_tensor_cache_get_or_insert(slai_ctx *ctx, slai_tensor_cache *c, int dtype, const uint32_t shape[4], uint32_t usage, slai_buffer **out) {
    if (!ctx || !c || !shape || !out) return SLAI_E_ARG;
    *out = nullptr;
    if (dtype < SLAI_DT_F32 || dtype > SLAI_DT_I32) return set_error(ctx, SLAI_E_ARG, "bad dtype");
    slai_tensor_key key{dtype, {shape[0], shape[1], shape[2], shape[3]}, usage};
    auto it = c->tensors.find(key);
    if (it != c->tensors.end() && !it->second.empty()) {
        *out = it->second.back();
        it->second.pop_back();
        (*out)->idle_in_cache = false;
        if (ctx->capturing) (*out)->captured = true;
        return SLAI_OK;
    }
    static const size_t esz[] = {4, 2, 1, 4};
    uint64_t n = 1;
    for (int i = 0; i < 4; ++i) {
        if (shape[i] == 0) return set_error(ctx, SLAI_E_SHAPE, "slai_tensor_cache_get_or_insert: a dimension of size zero");
        n *= shape[i];
        if (n > (uint64_t)1 << 40) return set_error(ctx, SLAI_E_SHAPE, "slai_tensor_cache_get_or_insert: shape too large");
    }
    slai_buffer *b = nullptr;
    if (int rc = slai_buffer_create(ctx, (size_t)n * esz[dtype], dtype, usage, &b)) return rc;
    for (int i = 0; i < 4; ++i) b->shape[i] = shape[i];
    *out = b;
    return SLAI_OK;
}
// What dropping a `CachedTensor` does (tensor_cache.rs:118-124, `reclaim` :199-203): the buffer goes back to the cache
// under the key it was handed out with.  Buffers that did not come from a cache are refused.
SLAI_EXPORT int slai_tensor_cache_reclaim(slai_ctx *ctx, slai_tensor_cache *c, slai_buffer *b) {
    if (!ctx || !c || !b) return SLAI_E_ARG;
    if (!b->shape[0]) return set_error(ctx, SLAI_E_ARG, "slai_tensor_cache_reclaim: not a cached tensor");
    // (the reference cannot give a tensor back twice: dropping its handle is what gives it back)
    if (b->idle_in_cache) return set_error(ctx, SLAI_E_STATE, "slai_tensor_cache_reclaim: this tensor is already back in its cache");
    b->idle_in_cache = true;
    slai_tensor_key key{b->dtype, {b->shape[0], b->shape[1], b->shape[2], b->shape[3]}, b->usage};
    c->tensors[key].push_back(b);
    return SLAI_OK;
}
SLAI_EXPORT size_t slai_tensor_cache_idle(const slai_tensor_cache *c) {
    size_t n = 0;
    if (c) for (const auto &kv : c->tensors) n += kv.second.size();
    return n;
}

// ---- quantized matrices ---------------------------------------------------------
// Upper bound of |w| over a matrix in GGUF block order, from the block scales alone: |d| * 63 * 15 + |dmin| * 63 (Q4_K;
// 31 for Q5_K), |d| * 128 * 32 (Q6_K), |d| * 128 (Q8_0), |d| * 8 (Q4_0).  binary16 magnitudes order like their bit
// patterns, so the scan compares integers and converts once.
static float weight_bound(int t, size_t nblocks, const uint8_t *packed) {
    size_t stride, d_off;
    switch (t) {
    case T_Q4_K: stride = 144; d_off = 0; break;
    case T_Q5_K: stride = 176; d_off = 0; break;
    case T_Q6_K: stride = 210; d_off = 208; break;
    case T_Q8_0: stride = 34; d_off = 0; break;
    case T_Q4_0: stride = 18; d_off = 0; break;
    default: return INFINITY;
    }
    const bool has_min = t == T_Q4_K || t == T_Q5_K;
    uint16_t dmax = 0, mmax = 0;
    for (size_t b = 0; b < nblocks; ++b) {
        const uint8_t *p = packed + b * stride + d_off;
        dmax = std::max<uint16_t>(dmax, (uint16_t)((p[0] | (p[1] << 8)) & 0x7fff));
        if (has_min) mmax = std::max<uint16_t>(mmax, (uint16_t)((p[2] | (p[3] << 8)) & 0x7fff));
    }
    if (dmax >= 0x7c00 || mmax >= 0x7c00) return INFINITY;    // an infinite or NaN scale
    const float d = decode_f16(dmax), dm = decode_f16(mmax);
    switch (t) {
    case T_Q4_K: return d * 63.0f * 15.0f + dm * 63.0f;
    case T_Q5_K: return d * 63.0f * 31.0f + dm * 63.0f;
    case T_Q6_K: return d * 128.0f * 32.0f;
    case T_Q8_0: return d * 128.0f;
    default: return d * 8.0f;
    }
}

SLAI_EXPORT int slai_qmat_create(slai_ctx *ctx, uint32_t ggml_type, uint32_t nrows, uint32_t ncols, const void *packed,
                                 slai_qmat **out) {
    return slai_qmat_create_layout(ctx, ggml_type, nrows, ncols, packed, SLAI_LAYOUT_AUTO, out);
}

SLAI_EXPORT int slai_qmat_create_layout(slai_ctx *ctx, uint32_t ggml_type, uint32_t nrows, uint32_t ncols, const void *packed,
                                        int layout, slai_qmat **out) {
    if (!ctx || !out || !packed) return SLAI_E_ARG;
    *out = nullptr;
    if (layout < SLAI_LAYOUT_AUTO || layout > SLAI_LAYOUT_TILE64) return set_error(ctx, SLAI_E_ARG, "slai_qmat_create: unknown layout");
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "slai_qmat_create during graph capture");
    const int t = (int)ggml_type;
    const int be = block_elems(t);
    if (!be) return set_error(ctx, SLAI_E_TYPE, "slai_qmat_create: unsupported ggml type " + std::to_string(ggml_type));
    if (nrows == 0 || ncols == 0 || ncols % be) return set_error(ctx, SLAI_E_SHAPE, "slai_qmat_create: ncols must be a multiple of the block length");
    slai_qmat *m = new slai_qmat();
    m->type = t; m->nrows = nrows; m->ncols = ncols; m->nb = ncols / be;
    m->row_stride = device_row_stride(t, ncols);
    m->bytes = m->row_stride * nrows;
    if (ctx->tiled_layout && layout != SLAI_LAYOUT_ROWS && tiled_supported(t) && ncols % 256 == 0) {
        // 64-row tiles (wave-uniform GEMV) pay off when there are enough tiles to occupy the device, or when the
        // caller launches several such matrices together and says so
        const uint32_t ncb = ncols / 256;
        bool tile64 = layout == SLAI_LAYOUT_TILE64 || (layout == SLAI_LAYOUT_AUTO && nrows >= 8192 && nrows % 64 == 0 && ncb <= 16);
        if (!ctx->rowtile_gemv || ncb > 64) tile64 = false;
        const TiledGeom g = tiled_geom(t, nrows, ncols, tile64 ? 6u : 0u);
        // more than 16 column groups (over 16384 columns in 16-row tiles): only on request, the GEMV then takes several
        // launches and supports neither a normalisation prologue nor a non-linear epilogue
        if (g.ngroups <= 16 || tile64 || (layout == SLAI_LAYOUT_TILE16 && g.ngroups <= 64)) {
            m->tiled = true; m->rows_log2 = g.rows_log2; m->ncb = g.ncb; m->ngroups = g.ngroups; m->ntiles = g.ntiles;
            m->unit_bytes = g.unit_bytes; m->bytes = tiled_bytes(g);
        }
    }
    const size_t src_bytes = gguf_row_bytes(t, ncols) * nrows;
    uint8_t *staging = nullptr;
    hipError_t e = hipMalloc((void **)&m->dptr, m->bytes);
    const bool verbatim = !m->tiled && (t == T_Q4_K || t == T_Q5_K || ((t == T_F32 || t == T_F16) && gguf_row_bytes(t, ncols) == m->row_stride));
    if (e == hipSuccess) {
        if (verbatim) {
            e = hipMemcpyAsync(m->dptr, packed, src_bytes, hipMemcpyHostToDevice, ctx->stream);
        } else {
            e = hipMalloc((void **)&staging, src_bytes);
            if (e == hipSuccess) e = hipMemsetAsync(m->dptr, 0, m->bytes, ctx->stream);
            if (e == hipSuccess) e = hipMemcpyAsync(staging, packed, src_bytes, hipMemcpyHostToDevice, ctx->stream);
            if (e == hipSuccess) e = launch_repack(ctx->stream, m, staging);
        }
    }
    // (while the copies run) the bound the prompt pass needs to choose between the f16 and the fp32 matrix instructions
    if (e == hipSuccess && m->tiled) m->wbound = weight_bound(t, (size_t)nrows * m->nb, (const uint8_t *)packed);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (staging) (void)hipFree(staging);
    if (e != hipSuccess) {
        if (m->dptr) (void)hipFree(m->dptr);
        delete m;
        return hip_fail(ctx, e, "slai_qmat_create");
    }
    *out = m;
    return SLAI_OK;
}

SLAI_EXPORT void slai_qmat_destroy(slai_ctx *ctx, slai_qmat *m) {
    if (!m) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (m->dptr) (void)hipFree(m->dptr);
    delete m;
}
SLAI_EXPORT int slai_qmat_shape(const slai_qmat *m, uint32_t *nrows, uint32_t *ncols, uint32_t *ggml_type) {
    if (!m) return SLAI_E_ARG;
    if (nrows) *nrows = m->nrows;
    if (ncols) *ncols = m->ncols;
    if (ggml_type) *ggml_type = (uint32_t)m->type;
    return SLAI_OK;
}
SLAI_EXPORT size_t slai_qmat_device_bytes(const slai_qmat *m) { return m ? m->bytes : 0; }

SLAI_EXPORT int slai_qmat_dequantize(slai_ctx *ctx, const slai_qmat *m, uint32_t row0, uint32_t nrows, slai_view out) {
    if (!ctx || !m || !out.buf) return SLAI_E_ARG;
    if (row0 + nrows > m->nrows) return set_error(ctx, SLAI_E_SHAPE, "slai_qmat_dequantize: row range");
    if (out.buf->dtype != SLAI_DT_F32) return set_error(ctx, SLAI_E_TYPE, "slai_qmat_dequantize: out must be f32");
    if (out.size[0] != nrows || out.size[1] != m->ncols || out.stride[1] != 1 || out.stride[0] < m->ncols)
        return set_error(ctx, SLAI_E_SHAPE, "slai_qmat_dequantize: out must be a row-major [nrows x ncols] view");
    if (nrows == 0) return SLAI_OK;
    size_t last = out.offset + (size_t)(nrows - 1) * out.stride[0] + m->ncols;
    if (last * sizeof(float) > out.buf->bytes) return set_error(ctx, SLAI_E_SHAPE, "slai_qmat_dequantize: out too small");
    SLAI_HIP_TRY(ctx, launch_dequant_rows(ctx->stream, m, row0, nrows, (float *)out.buf->dptr + out.offset, out.stride[0]));
    return SLAI_OK;
}

// ---- GEMV dispatch over the two weight layouts ------------------------------------------------
namespace slai {
bool gemv_can_emit(const slai_qmat *m) { return m && m->tiled && m->rows_log2 != 6 && m->ngroups <= 64 && m->nrows % 16 == 0; }
bool gemv_is_rowtile(const slai_ctx *ctx, const slai_qmat *m) {
    return ctx->rowtile_gemv && m && m->tiled && m->rows_log2 == 6 && m->ncb <= 64;
}

bool gemv_gated_is_rowtile(const slai_ctx *ctx, const slai_qmat *gate, const slai_qmat *up) {
    return gemv_is_rowtile(ctx, gate) && gemv_is_rowtile(ctx, up) && gate->type == up->type;
}

// Grows one of the context's scratch blocks.  The block it replaces stays allocated until the context goes: graphs
// captured earlier (a model's decode graph) and launches already queued keep using the old address, which still holds
// as much as they were built for.  Growth is at least twofold, so the retired blocks together stay below the live one.
int scratch_grow(slai_ctx *ctx, float **block, size_t *have, size_t floats, const char *what) {
    if (floats <= *have) return SLAI_OK;
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, std::string(what) + " must be reserved before graph capture");
    floats = std::max(floats, 2 * *have);
    float *fresh = nullptr;
    SLAI_HIP_TRY(ctx, hipMalloc((void **)&fresh, floats * sizeof(float)));
    if (*block) ctx->retired_scratch.push_back(*block);
    *block = fresh; *have = floats;
    return SLAI_OK;
}

int gemv_scratch_reserve(slai_ctx *ctx, size_t floats) {
    return scratch_grow(ctx, &ctx->gemv_scratch, &ctx->gemv_scratch_floats, floats, "GEMV scratch");
}

bool qkv_attention_fusable(const slai_ctx *ctx, const slai_qmat *v, const slai_qmat *k, const slai_qmat *q, const AttnLaunch &a) {
    if (!ctx->fuse_qkv_attention || !ctx->handoff_counters || a.n_heads > ctx->handoff_heads) return false;
    if (a.head_size != 128 || a.kv_mul != 1 || a.n_splits != 1 || a.n_heads % 8 || a.kv_dim % 8 || !a.knew || !a.vnew) return false;
    for (const slai_qmat *m : {v, k, q}) {
        if (!gemv_is_rowtile(ctx, m) || m->ncb != 16 || m->nrows != a.n_heads * 128u) return false;
        if (m->type != T_Q4_K && m->type != T_Q6_K && m->type != T_Q5_K) return false;
    }
    return true;
}
// Allocated once per context and never moved (captured graphs hold the address): models with more heads than the
// first reservation allows simply keep separate launches.
int handoff_reserve(slai_ctx *ctx, uint32_t n_heads) {
    if (ctx->handoff_counters) return SLAI_OK;
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "hand-off counters must be reserved before graph capture");
    if (n_heads < 256) n_heads = 256;
    const size_t bytes = ((size_t)n_heads * 32 + 32) * sizeof(uint32_t);
    SLAI_HIP_TRY(ctx, hipMalloc((void **)&ctx->handoff_counters, bytes));
    // The hand-off relies on workgroup i running on XCD i mod 8 (workgroups with equal i mod 8 then share an L2):
    // look before relying on it, and keep separate launches on a device that places workgroups differently.
    uint32_t where[256];
    SLAI_HIP_TRY(ctx, launch_xcd_of_workgroup(ctx->stream, ctx->handoff_counters, 256));
    SLAI_HIP_TRY(ctx, hipMemcpyAsync(where, ctx->handoff_counters, sizeof where, hipMemcpyDeviceToHost, ctx->stream));
    SLAI_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    for (uint32_t i = 8; i < 256; ++i)
        if (where[i] != where[i % 8]) ctx->fuse_qkv_attention = false;
    SLAI_HIP_TRY(ctx, hipMemsetAsync(ctx->handoff_counters, 0, bytes, ctx->stream));
    SLAI_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    ctx->handoff_heads = n_heads;
    return SLAI_OK;
}
int handoff_check(slai_ctx *ctx) {
    if (!ctx->handoff_counters) return SLAI_OK;
    uint32_t flag = 0;
    SLAI_HIP_TRY(ctx, hipMemcpy(&flag, ctx->handoff_counters + (size_t)ctx->handoff_heads * 32, sizeof flag, hipMemcpyDeviceToHost));
    if (flag) {
        // reported once: the slot is cleared so that later, healthy calls are not failed for an old time-out, and so are
        // the per-head counters, which a launch that gave up may have left anywhere
        (void)hipMemset(ctx->handoff_counters, 0, ((size_t)ctx->handoff_heads * 32 + 32) * sizeof(uint32_t));
        return set_error(ctx, SLAI_E_HIP, "q/k/v -> attention hand-off timed out inside a launch; results are invalid");
    }
    return SLAI_OK;
}

int sampler_scratch_reserve(slai_ctx *ctx, size_t floats) {
    return scratch_grow(ctx, &ctx->sampler_scratch, &ctx->sampler_scratch_floats, floats, "sampler scratch");
}

int step_mark(slai_ctx *ctx, const char *name) {
    if (!ctx->step_marks) return SLAI_OK;
    hipEvent_t e;
    SLAI_HIP_TRY(ctx, hipEventCreate(&e));
    ctx->step_marks->emplace_back(name, e);
    SLAI_HIP_TRY(ctx, hipEventRecord(e, ctx->stream));
    return SLAI_OK;
}

static int gemv_call_impl(slai_ctx *ctx, const GemvCall &c, const char *who, const AttnLaunch *fused_attn);
int gemv_call(slai_ctx *ctx, const GemvCall &c, const char *who, const AttnLaunch *fused_attn) {
    if (ctx->only_step && strcmp(ctx->only_step, who) != 0) return SLAI_OK;
    if (int rc = gemv_call_impl(ctx, c, who, fused_attn)) return rc;
    return step_mark(ctx, who);
}

static int gemv_call_impl(slai_ctx *ctx, const GemvCall &c, const char *who, const AttnLaunch *fused_attn) {
    const slai_qmat *m0 = c.m[0];
    if (!m0 || c.nseg < 1 || c.nseg > 3) return set_error(ctx, SLAI_E_ARG, std::string(who) + ": bad GEMV call");
    // 64-row tiles: wave-uniform activations, formats may differ between the segments
    bool rowtile = ctx->rowtile_gemv && (c.prologue == PRO_NONE || (c.prologue == PRO_RMSNORM && !c.norm_b));
    for (int i = 0; i < c.nseg && rowtile; ++i) {
        const slai_qmat *m = c.m[i], *m2 = c.m2[i];
        rowtile = m && m->tiled && m->rows_log2 == 6 && m->ncols == m0->ncols && m->ncb <= 64 &&
                  (!m2 || (m2->tiled && m2->rows_log2 == 6 && m2->type == m->type && m2->ncols == m->ncols && m2->nrows == m->nrows)) &&
                  (((c.flags[i] & GEMV_SILU_GATE) != 0) == (m2 != nullptr)) &&
                  (((c.flags[i] ^ c.flags[0]) & GEMV_SILU_GATE) == 0);
    }
    for (int i = 1; i < c.nseg && rowtile; ++i)
        if (c.m[i]->type != m0->type && (c.m[i]->type == T_Q8_0 || m0->type == T_Q8_0 || c.m[i]->type == T_Q4_0 || m0->type == T_Q4_0)) rowtile = false;
    if (c.flags[0] & GEMV_EMIT) {
        if (rowtile || !gemv_can_emit(m0) || !c.emit_w || !c.emit_out) return set_error(ctx, SLAI_E_ARG, std::string(who) + ": this GEMV cannot emit a prepared copy");
    }
    if (c.prepared && !rowtile) return set_error(ctx, SLAI_E_ARG, std::string(who) + ": prepared activations need 64-row tiles");
    const GemvBatch *batch = c.batch.n > 1 ? &c.batch : nullptr;
    if (batch && (fused_attn || (rowtile && !c.prepared) || (!rowtile && !m0->tiled)))
        return set_error(ctx, SLAI_E_ARG, std::string(who) + ": several input vectors need prepared input (64-row tiles) or 16-row tiles");
    if (rowtile) {
        GemvRowtileParams p;
        p.nseg = c.nseg; p.ncols = m0->ncols; p.ncb = m0->ncb; p.x = c.x; p.prologue = c.prologue; p.norm_w = c.norm_w; p.eps = c.eps;
        p.prepared = c.prepared;
        for (int i = 0; i < c.nseg; ++i) {
            p.seg[i].W = c.m[i]->dptr; p.seg[i].W2 = c.m2[i] ? c.m2[i]->dptr : nullptr; p.seg[i].type = c.m[i]->type;
            p.seg[i].nrows = c.m[i]->nrows; p.seg[i].out = c.out[i]; p.seg[i].bias = c.bias[i]; p.seg[i].flags = c.flags[i];
        }
        if (!p.prepared) {
            int rc = gemv_scratch_reserve(ctx, gemv_rowtile_scratch_floats(p));
            if (rc) return rc;
            p.scratch = ctx->gemv_scratch;
        }
        hipError_t e = fused_attn ? launch_qkv_attention(ctx, p, *fused_attn) : launch_gemv_rowtile(ctx, p, batch);
        if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": unsupported shape for the row-tile GEMV");
        if (e != hipSuccess) return hip_fail(ctx, e, who);
        return SLAI_OK;
    }
    if (fused_attn) return set_error(ctx, SLAI_E_ARG, std::string(who) + ": attention can only join a 64-row-tile launch");
    for (int i = 0; i < c.nseg; ++i) {
        const slai_qmat *m = c.m[i], *m2 = c.m2[i];
        if (!m || m->type != m0->type || m->ncols != m0->ncols || m->tiled != m0->tiled ||
            (m->tiled && (m->rows_log2 != m0->rows_log2 || m->ngroups > 64)))
            return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": matrices of one launch must share format, width and layout");
        if (m2 && (m2->type != m->type || m2->ncols != m->ncols || m2->nrows != m->nrows || m2->tiled != m->tiled ||
                   (m->tiled && m2->rows_log2 != m->rows_log2)))
            return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": gate and up must share format, shape and layout");
        if ((c.flags[i] & GEMV_SILU_GATE) && !m2) return set_error(ctx, SLAI_E_ARG, std::string(who) + ": gated GEMV without a second matrix");
    }
    hipError_t e;
    if (m0->tiled) {
        GemvTiledParams p;
        p.nseg = c.nseg; p.ncols = m0->ncols; p.ncb = m0->ncb; p.ngroups = m0->ngroups; p.rows_log2 = m0->rows_log2;
        p.unit_bytes = m0->unit_bytes; p.x = c.x; p.prologue = c.prologue; p.norm_w = c.norm_w; p.norm_b = c.norm_b;
        p.eps = c.eps; p.emit_w = c.emit_w; p.emit_out = c.emit_out;
        for (int i = 0; i < c.nseg; ++i) {
            p.seg[i].W = c.m[i]->dptr; p.seg[i].W2 = c.m2[i] ? c.m2[i]->dptr : nullptr; p.seg[i].nrows = c.m[i]->nrows;
            p.seg[i].out = c.out[i]; p.seg[i].bias = c.bias[i]; p.seg[i].flags = c.flags[i];
        }
        if (m0->ngroups <= 16) {
            e = launch_gemv_tiled(ctx, m0->type, p, batch);
        } else {
            // wide matrix: balanced slices of at most 16 column groups, one launch each; the first writes (or adds to
            // the residual), the others accumulate, the last one emits
            if (c.prologue != PRO_NONE) return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": no normalisation prologue over more than 16384 columns in 16-row tiles");
            for (int i = 0; i < c.nseg; ++i)
                if (c.flags[i] & (GEMV_GELU | GEMV_SILU_GATE)) return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": no non-linear epilogue over more than 16384 columns in 16-row tiles");
            const uint32_t nchunks = (m0->ngroups + 15) / 16, per = (m0->ngroups + nchunks - 1) / nchunks;
            e = hipSuccess;
            for (uint32_t k = 0; k < nchunks && e == hipSuccess; ++k) {
                GemvTiledParams q = p;
                q.group0 = k * per;
                q.launch_groups = std::min(per, m0->ngroups - q.group0);
                for (int i = 0; i < c.nseg; ++i) {
                    if (k > 0) { q.seg[i].flags = (q.seg[i].flags | GEMV_ACCUM) & ~GEMV_BIAS; }
                    if (k + 1 < nchunks) q.seg[i].flags &= ~GEMV_EMIT;
                }
                e = launch_gemv_tiled(ctx, m0->type, q, batch);
            }
        }
    } else {
        if (!gemv_supports(m0->type, m0->ncols)) return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": unsupported column count for this format");
        GemvParams p;
        p.nseg = c.nseg; p.ncols = m0->ncols; p.nb = m0->nb; p.x = c.x; p.prologue = c.prologue; p.norm_w = c.norm_w;
        p.norm_b = c.norm_b; p.eps = c.eps; p.rows_per_wg = ctx->gemv_rows_per_wg;
        for (int i = 0; i < c.nseg; ++i) {
            p.seg[i].W = c.m[i]->dptr; p.seg[i].W2 = c.m2[i] ? c.m2[i]->dptr : nullptr; p.seg[i].row_stride = c.m[i]->row_stride;
            p.seg[i].nrows = c.m[i]->nrows; p.seg[i].out = c.out[i]; p.seg[i].bias = c.bias[i]; p.seg[i].flags = c.flags[i];
        }
        e = launch_gemv(ctx, m0->type, p);
    }
    if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": unsupported shape for this format");
    if (e != hipSuccess) return hip_fail(ctx, e, who);
    return SLAI_OK;
}
}  // namespace slai

// ---- ops ---------------------------------------------------------------------------
#define NEED_VEC(view, name, vv)                                                                           \
    VecView vv;                                                                                            \
    if (!as_vec(view, &vv)) return set_error(ctx, SLAI_E_SHAPE, std::string(__func__) + ": bad view '" name "'")

SLAI_EXPORT int slai_rms_norm_assign(slai_ctx *ctx, const slai_buffer *config, slai_view out, slai_view value, slai_view weight) {
    if (!ctx || !config) return SLAI_E_ARG;
    if (config->bytes < sizeof(slai_rms_norm_config)) return set_error(ctx, SLAI_E_SHAPE, "slai_rms_norm_assign: config buffer too small");
    NEED_VEC(out, "out", vo); NEED_VEC(value, "value", vv); NEED_VEC(weight, "weight", vw);
    if (vo.n != vv.n || vw.n != vv.n) return set_error(ctx, SLAI_E_SHAPE, "slai_rms_norm_assign: length mismatch");
    SLAI_HIP_TRY(ctx, launch_rms_norm(ctx->stream, vo, vv, vw, (const float *)config->dptr, 0.0f));
    return SLAI_OK;
}

SLAI_EXPORT int slai_layernorm_assign(slai_ctx *ctx, slai_view out, slai_view value, float eps) {
    if (!ctx) return SLAI_E_ARG;
    NEED_VEC(out, "out", vo); NEED_VEC(value, "value", vv);
    if (vo.n != vv.n) return set_error(ctx, SLAI_E_SHAPE, "slai_layernorm_assign: length mismatch");
    SLAI_HIP_TRY(ctx, launch_layernorm(ctx->stream, vo, vv, eps));
    return SLAI_OK;
}

SLAI_EXPORT int slai_matmul_quant_assign(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view v) {
    if (!ctx || !m) return SLAI_E_ARG;
    NEED_VEC(out, "out", vo); NEED_VEC(v, "v", vv);
    if (vo.n != m->nrows || vv.n != m->ncols) return set_error(ctx, SLAI_E_SHAPE, "slai_matmul_quant_assign: dimension mismatch");
    if (vo.stride != 1 || vv.stride != 1 || (v.offset % 4) != 0)
        return set_error(ctx, SLAI_E_SHAPE, "slai_matmul_quant_assign: vectors must be contiguous, input offset a multiple of 4");
    GemvCall c;
    c.m[0] = m; c.out[0] = vo.p; c.x = vv.p;
    return gemv_call(ctx, c, "slai_matmul_quant_assign");
}

// Several vectors through one quantised matrix on the matrix cores (kernels_gemm_chunk.hip): out[:, t] (+)= m * x[:, t]
// for the ntokens <= 32 columns of two contiguous column-major matrices.  The operator under the chunked prompt pass of
// the models, exposed for tests and callers with their own layer loop; the reference only has the one-vector product
// (context.rs:355-399).
SLAI_EXPORT int slai_matmul_quant_columns(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view x, int accumulate) {
    if (!ctx || !m) return SLAI_E_ARG;
    const char *fn = "slai_matmul_quant_columns";
    if (!out.buf || !x.buf || out.buf->dtype != SLAI_DT_F32 || x.buf->dtype != SLAI_DT_F32) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": f32 views needed");
    const uint32_t nt = x.size[1];
    if (nt == 0 || nt > 32 || out.size[1] != nt || x.size[0] != m->ncols || out.size[0] != m->nrows || x.size[2] != 1 || x.size[3] != 1 ||
        out.size[2] != 1 || out.size[3] != 1)
        return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": out must be nrows x n, x ncols x n, n <= 32");
    if (x.stride[0] != 1 || out.stride[0] != 1 || (nt > 1 && (x.stride[1] != m->ncols || out.stride[1] != m->nrows)) || x.offset % 4)
        return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": contiguous column-major matrices needed, input offset a multiple of 4");
    if ((x.offset + (size_t)nt * m->ncols) * 4 > x.buf->bytes || (out.offset + (size_t)nt * m->nrows) * 4 > out.buf->bytes)
        return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": view beyond its buffer");
    if (!gemm_chunk_supports(m)) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": the matrix has no tiled layout");
    // the kernels read the activations quad-major with 32 token slots; the GEMV scratch holds that copy
    if (int rc = gemv_scratch_reserve(ctx, (size_t)32 * m->ncols)) return rc;
    const float *xp = reinterpret_cast<const float *>(x.buf->dptr) + x.offset;
    float *op = reinterpret_cast<float *>(out.buf->dptr) + out.offset;
    // (SLAI_PROMPT_SPLIT_F16=2, for kernel tests: the f16 form, whose range the caller then has to keep)
    SLAI_HIP_TRY(ctx, launch_rows_to_quads(ctx->stream, ctx->gemv_scratch, xp, m->ncols, nt, m->ncols, ctx->prompt_split_f16 == 2 && m->wbound < 255.0f ? ctx->split_flag : nullptr));
    GemmChunkParams p;
    p.nseg = 1; p.ncols = m->ncols; p.ncb = m->ncb; p.ngroups = m->ngroups; p.rows_log2 = m->rows_log2;
    p.x = ctx->gemv_scratch; p.ntokens = nt; p.split_f16 = ctx->prompt_split_f16 == 2 && m->wbound < 255.0f;
    p.seg[0].W = m->dptr; p.seg[0].type = m->type; p.seg[0].nrows = m->nrows; p.seg[0].out = op; p.seg[0].out_stride = m->nrows;
    p.seg[0].flags = accumulate ? GEMV_ACCUM : 0;
    hipError_t e = launch_gemm_chunk(ctx, p);
    if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": unsupported shape");
    if (e != hipSuccess) return hip_fail(ctx, e, fn);
    return SLAI_OK;
}

// `prepared` (optional): the slai_rms_norm_prepare form of (x, norm weight); `emit_w` / `emit_out` (optional): leave
// that form of (result, emit_w) in emit_out.
static int fused_gemv(slai_ctx *ctx, const char *fn, slai_view out, const slai_qmat *m, const slai_qmat *m2, slai_view v,
                      const slai_view *norm_weight, float eps, uint32_t flags, const slai_view *prepared = nullptr,
                      const slai_view *emit_w = nullptr, const slai_view *emit_out = nullptr, bool plain_prepared = false) {
    if (!ctx || !m) return SLAI_E_ARG;
    VecView vo, vv, vw{nullptr, 0, 1};
    if (!as_vec(out, &vo) || !as_vec(v, &vv)) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": bad view");
    if (norm_weight && (!as_vec(*norm_weight, &vw) || vw.n != m->ncols || vw.stride != 1))
        return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": bad norm weight");
    if (vo.n != m->nrows || vv.n != m->ncols || vo.stride != 1 || vv.stride != 1 || (v.offset % 4) != 0)
        return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": dimension mismatch or non-contiguous vectors");
    if (m2 && (m2->type != m->type || m2->nrows != m->nrows || m2->ncols != m->ncols))
        return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": gate and up must share format and shape");
    GemvCall c;
    c.m[0] = m; c.m2[0] = m2; c.out[0] = vo.p; c.flags[0] = flags; c.x = vv.p;
    if (norm_weight) { c.prologue = PRO_RMSNORM; c.norm_w = vw.p; c.eps = eps; }
    if (prepared) {
        VecView vp;
        if (!as_vec(*prepared, &vp) || vp.stride != 1 || vp.n < m->ncols + m->ncols / 16 || (prepared->offset % 16) != 0)
            return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": prepared activations must be ncols + ncols/16 contiguous floats, 64-byte aligned");
        if (!gemv_is_rowtile(ctx, m)) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": prepared activations need a matrix in the TILE64 layout");
        c.prologue = plain_prepared ? PRO_NONE : PRO_RMSNORM; c.eps = eps; c.prepared = vp.p;
    }
    if (emit_w) {
        VecView ve, vq;
        if (!emit_out || !as_vec(*emit_w, &ve) || !as_vec(*emit_out, &vq) || ve.stride != 1 || vq.stride != 1 || ve.n != m->nrows ||
            vq.n < m->nrows + m->nrows / 16 || (emit_out->offset % 16) != 0)
            return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": bad next-norm weight or prepared output");
        if (!gemv_can_emit(m)) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": this matrix layout cannot emit prepared activations");
        c.flags[0] |= GEMV_EMIT; c.emit_w = ve.p; c.emit_out = vq.p;
    }
    return gemv_call(ctx, c, fn);
}

SLAI_EXPORT int slai_rms_norm_prepare(slai_ctx *ctx, slai_view out_prepared, slai_view x, slai_view norm_weight) {
    if (!ctx) return SLAI_E_ARG;
    VecView vo, vx, vw;
    if (!as_vec(out_prepared, &vo) || !as_vec(x, &vx) || !as_vec(norm_weight, &vw)) return set_error(ctx, SLAI_E_SHAPE, "slai_rms_norm_prepare: bad view");
    if (vx.n % 16 || vw.n != vx.n || vo.n < vx.n + vx.n / 16 || vo.stride != 1 || vx.stride != 1 || vw.stride != 1 || (out_prepared.offset % 16) != 0)
        return set_error(ctx, SLAI_E_SHAPE, "slai_rms_norm_prepare: need n % 16 == 0 and n + n/16 contiguous output floats, 64-byte aligned");
    SLAI_HIP_TRY(ctx, launch_prepare(ctx->stream, vo.p, vx.p, vw.p, vx.n));
    return SLAI_OK;
}
SLAI_EXPORT int slai_matmul_quant_assign_prepared(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view prepared) {
    if (!m) return SLAI_E_ARG;
    slai_view v = prepared;                       // the first ncols floats of the prepared form are the vector itself
    v.size[0] = m->ncols; v.size[1] = v.size[2] = v.size[3] = 1; v.stride[0] = 1;
    return fused_gemv(ctx, "slai_matmul_quant_assign_prepared", out, m, nullptr, v, nullptr, 0.0f, 0, &prepared, nullptr, nullptr, true);
}
SLAI_EXPORT int slai_rms_norm_matmul_quant_assign_prepared(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view x, slai_view prepared,
                                                           float eps) {
    return fused_gemv(ctx, "slai_rms_norm_matmul_quant_assign_prepared", out, m, nullptr, x, nullptr, eps, 0, &prepared);
}
SLAI_EXPORT int slai_ffn_gate_up_silu_prepared(slai_ctx *ctx, slai_view out_hb, const slai_qmat *gate, const slai_qmat *up, slai_view x,
                                               slai_view prepared, float eps) {
    if (!up) return SLAI_E_ARG;
    return fused_gemv(ctx, "slai_ffn_gate_up_silu_prepared", out_hb, gate, up, x, nullptr, eps, GEMV_SILU_GATE, &prepared);
}
SLAI_EXPORT int slai_matmul_quant_add_assign_emit(slai_ctx *ctx, slai_view in_out_x, const slai_qmat *m, slai_view v, slai_view next_norm_weight,
                                                  slai_view out_prepared) {
    return fused_gemv(ctx, "slai_matmul_quant_add_assign_emit", in_out_x, m, nullptr, v, nullptr, 0.0f, GEMV_ACCUM, nullptr, &next_norm_weight,
                      &out_prepared);
}

SLAI_EXPORT int slai_rms_norm_matmul_quant_assign(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view x, slai_view norm_weight,
                                                  float eps) {
    return fused_gemv(ctx, "slai_rms_norm_matmul_quant_assign", out, m, nullptr, x, &norm_weight, eps, 0);
}
SLAI_EXPORT int slai_ffn_gate_up_silu(slai_ctx *ctx, slai_view out_hb, const slai_qmat *gate, const slai_qmat *up, slai_view x,
                                      slai_view norm_weight, float eps) {
    if (!up) return SLAI_E_ARG;
    return fused_gemv(ctx, "slai_ffn_gate_up_silu", out_hb, gate, up, x, &norm_weight, eps, GEMV_SILU_GATE);
}
SLAI_EXPORT int slai_matmul_quant_add_assign(slai_ctx *ctx, slai_view in_out_x, const slai_qmat *m, slai_view v) {
    return fused_gemv(ctx, "slai_matmul_quant_add_assign", in_out_x, m, nullptr, v, nullptr, 0.0f, GEMV_ACCUM);
}

SLAI_EXPORT int slai_matmul_assign(slai_ctx *ctx, slai_view out, slai_view a, slai_view b, int a_mode, int b_mode) {
    if (!ctx) return SLAI_E_ARG;
    View4 vo, va, vb;
    if (!as_view4(out, &vo) || !as_view4(a, &va) || !as_view4(b, &vb)) return set_error(ctx, SLAI_E_SHAPE, "slai_matmul_assign: bad view");
    const uint32_t m = a_mode == SLAI_MODE_N ? va.size[0] : va.size[1], inner = a_mode == SLAI_MODE_N ? va.size[1] : va.size[0];
    const uint32_t inner_b = b_mode == SLAI_MODE_N ? vb.size[0] : vb.size[1], n = b_mode == SLAI_MODE_N ? vb.size[1] : vb.size[0];
    if (inner != inner_b || vo.size[0] != m || vo.size[1] != n) return set_error(ctx, SLAI_E_SHAPE, "slai_matmul_assign: dimension mismatch");
    for (int d = 2; d < 4; ++d)
        if ((va.size[d] != 1 && va.size[d] != vo.size[d]) || (vb.size[d] != 1 && vb.size[d] != vo.size[d]))
            return set_error(ctx, SLAI_E_SHAPE, "slai_matmul_assign: batch dimension mismatch");
    SLAI_HIP_TRY(ctx, launch_matmul_f32(ctx->stream, vo, va, vb, a_mode, b_mode));
    return SLAI_OK;
}

static int binop(slai_ctx *ctx, int op, slai_view a, slai_view b, const char *fn) {
    if (!ctx) return SLAI_E_ARG;
    VecView va, vb;
    if (!as_vec(a, &va) || !as_vec(b, &vb) || va.n != vb.n) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": bad views or length mismatch");
    SLAI_HIP_TRY(ctx, launch_binop(ctx->stream, op, va, vb));
    return SLAI_OK;
}
SLAI_EXPORT int slai_add_assign(slai_ctx *ctx, slai_view a, slai_view b) { return binop(ctx, 0, a, b, "slai_add_assign"); }
SLAI_EXPORT int slai_mul_assign(slai_ctx *ctx, slai_view a, slai_view b) { return binop(ctx, 1, a, b, "slai_mul_assign"); }
SLAI_EXPORT int slai_copy(slai_ctx *ctx, slai_view in, slai_view out) { return binop(ctx, 2, out, in, "slai_copy"); }

SLAI_EXPORT int slai_rope(slai_ctx *ctx, int variant, const slai_buffer *config, slai_view in_out_q, slai_view in_out_k) {
    if (!ctx || !config) return SLAI_E_ARG;
    if (config->bytes < sizeof(slai_rope_config)) return set_error(ctx, SLAI_E_SHAPE, "slai_rope: config buffer too small");
    if (variant != SLAI_ROPE_ORIGINAL && variant != SLAI_ROPE_NEOX) return set_error(ctx, SLAI_E_ARG, "slai_rope: bad variant");
    NEED_VEC(in_out_q, "q", vq); NEED_VEC(in_out_k, "k", vk);
    // ops/rope.rs:58-64
    if (vq.n % 2 || vk.n % 2 || vq.n < vk.n) return set_error(ctx, SLAI_E_SHAPE, "slai_rope: q and k must have even lengths with len(q) >= len(k)");
    SLAI_HIP_TRY(ctx, launch_rope(ctx->stream, variant, (const slai_rope_config *)config->dptr, vq, vk));
    return SLAI_OK;
}

SLAI_EXPORT int slai_silu(slai_ctx *ctx, slai_view h1, slai_view h2) {
    if (!ctx) return SLAI_E_ARG;
    NEED_VEC(h1, "h1", va); NEED_VEC(h2, "h2", vb);
    if (va.n != vb.n) return set_error(ctx, SLAI_E_SHAPE, "slai_silu: length mismatch");
    SLAI_HIP_TRY(ctx, launch_silu(ctx->stream, va, vb));
    return SLAI_OK;
}

SLAI_EXPORT int slai_gelu_inplace(slai_ctx *ctx, slai_view x) {
    if (!ctx) return SLAI_E_ARG;
    NEED_VEC(x, "x", va);
    SLAI_HIP_TRY(ctx, launch_gelu(ctx->stream, va));
    return SLAI_OK;
}

SLAI_EXPORT int slai_attn_mask(slai_ctx *ctx, const slai_attn_params *params, const slai_buffer *params_gpu, slai_buffer *attn) {
    if (!ctx || !params || !params_gpu || !attn) return SLAI_E_ARG;
    if (params_gpu->bytes < sizeof(slai_attn_params)) return set_error(ctx, SLAI_E_SHAPE, "slai_attn_mask: params buffer too small");
    const uint32_t rounded_pos = (params->pos + 1 + 3) / 4 * 4;          // context.rs:773
    const size_t n = (size_t)params->n_heads * rounded_pos;             // context.rs:783
    if (n * sizeof(float) > attn->bytes) return set_error(ctx, SLAI_E_SHAPE, "slai_attn_mask: attn buffer too small");
    SLAI_HIP_TRY(ctx, launch_attn_mask(ctx->stream, (const slai_attn_params *)params_gpu->dptr, (float *)attn->dptr, (uint32_t)n));
    return SLAI_OK;
}

SLAI_EXPORT int slai_softmax_cols(slai_ctx *ctx, slai_view m) {
    if (!ctx) return SLAI_E_ARG;
    View4 v;
    if (!as_view4(m, &v)) return set_error(ctx, SLAI_E_SHAPE, "slai_softmax_cols: bad view");
    if (v.size[2] > 65535 || v.size[3] > 65535) return set_error(ctx, SLAI_E_SHAPE, "slai_softmax_cols: batch too large");
    SLAI_HIP_TRY(ctx, launch_softmax_cols(ctx->stream, v));
    return SLAI_OK;
}

namespace slai {
uint32_t pick_attn_splits(const slai_ctx *ctx, uint32_t n_heads, uint32_t seq_len) {
    if (ctx->attn_splits > 0) return (uint32_t)ctx->attn_splits;
    // short contexts: one workgroup per head walks the whole context, no combine pass
    if (seq_len <= 1024) return 1;
    // enough workgroups to cover the chip, at least ~32 positions per split at full context
    uint32_t s = (512 + n_heads - 1) / n_heads;
    uint32_t cap = seq_len / 32 ? seq_len / 32 : 1;
    if (s > cap) s = cap;
    if (s > 32) s = 32;
    return s ? s : 1;
}
int ensure_attn_scratch(slai_ctx *ctx, size_t floats) {
    return scratch_grow(ctx, &ctx->attn_scratch, &ctx->attn_scratch_floats, floats, "attention scratch");
}
}  // namespace slai

namespace slai {
// Checks the arguments of slai_attention and fills everything of the launch but the scratch block and the number of
// splits' buffer; allocates nothing.
int attention_describe(slai_ctx *ctx, const char *fn, const slai_attn_params *params, const slai_buffer *params_gpu, slai_view q, slai_view key_cache,
                       slai_view value_cache, slai_view xb, AttnLaunch *out) {
    if (!ctx || !params || !params_gpu || !key_cache.buf || !value_cache.buf) return SLAI_E_ARG;
    if (params_gpu->bytes < sizeof(slai_attn_params)) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": params buffer too small");
    VecView vq, vx;
    if (!as_vec(q, &vq)) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": bad view 'q'");
    if (!as_vec(xb, &vx)) return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": bad view 'xb'");
    const uint32_t hs = params->head_size, nh = params->n_heads;
    if (!params->kv_mul || nh % params->kv_mul || vq.n != nh * hs || vx.n != nh * hs || vq.stride != 1 || vx.stride != 1 ||
        params->kv_dim != nh / params->kv_mul * hs || params->pos >= params->seq_len)
        return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": inconsistent parameters");
    const int kdt = key_cache.buf->dtype;
    if (kdt != value_cache.buf->dtype || (kdt != SLAI_DT_F32 && kdt != SLAI_DT_F16)) return set_error(ctx, SLAI_E_TYPE, std::string(fn) + ": caches must both be f32 or f16");
    const size_t esz = kdt == SLAI_DT_F16 ? 2 : 4;
    for (const slai_view *c : {&key_cache, &value_cache}) {
        if (c->size[0] != params->kv_dim || c->size[1] != params->seq_len || c->stride[0] != 1 || c->stride[1] != params->kv_dim ||
            (c->offset + (size_t)params->kv_dim * params->seq_len) * esz > c->buf->bytes || (c->offset % 2))
            return set_error(ctx, SLAI_E_SHAPE, std::string(fn) + ": caches must be [kv_dim x seq_len] column-major");
    }
    AttnLaunch a{};
    a.q = vq.p;
    a.kcache = (char *)key_cache.buf->dptr + key_cache.offset * esz;
    a.vcache = (char *)value_cache.buf->dptr + value_cache.offset * esz;
    a.kv_f16 = kdt == SLAI_DT_F16;
    a.n_heads = nh; a.kv_mul = params->kv_mul; a.head_size = hs; a.kv_dim = params->kv_dim; a.seq_len = params->seq_len;
    a.pos_ptr = &((const slai_attn_params *)params_gpu->dptr)->pos;
    a.rope_variant = SLAI_ROPE_ORIGINAL; a.rope_base = 0.0f;
    a.out = vx.p;
    a.n_splits = pick_attn_splits(ctx, nh, params->seq_len);
    *out = a;
    return SLAI_OK;
}
}  // namespace slai

SLAI_EXPORT int slai_attention(slai_ctx *ctx, const slai_attn_params *params, const slai_buffer *params_gpu, slai_view q,
                               slai_view key_cache, slai_view value_cache, slai_view att, slai_view xb) {
    (void)att;
    AttnLaunch a{};
    if (int rc = attention_describe(ctx, "slai_attention", params, params_gpu, q, key_cache, value_cache, xb, &a)) return rc;
    int rc = ensure_attn_scratch(ctx, attention_scratch_floats(a.n_heads, a.head_size, a.n_splits));
    if (rc) return rc;
    a.scratch = ctx->attn_scratch;
    hipError_t e = launch_attention(ctx->stream, a);
    if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, "slai_attention: unsupported head size or context length");
    SLAI_HIP_TRY(ctx, e);
    return SLAI_OK;
}

SLAI_EXPORT int slai_argmax(slai_ctx *ctx, slai_view logits, slai_buffer *out_index) {
    if (!ctx || !out_index) return SLAI_E_ARG;
    NEED_VEC(logits, "logits", vl);
    if (vl.stride != 1 || out_index->dtype != SLAI_DT_I32 || out_index->bytes < 4) return set_error(ctx, SLAI_E_SHAPE, "slai_argmax: contiguous logits and an I32 output are required");
    SLAI_HIP_TRY(ctx, launch_argmax(ctx->stream, vl.p, vl.n, (int *)out_index->dptr, nullptr, nullptr, nullptr));
    return SLAI_OK;
}

// models/sampler.rs:33-53 `Sampler::sample`, with the draw passed in.  The logits are left as they are (the reference
// overwrites them with the probabilities).
SLAI_EXPORT int slai_sample(slai_ctx *ctx, slai_view logits, float temperature, float topp, float coin, slai_buffer *out_index) {
    if (!ctx || !out_index) return SLAI_E_ARG;
    NEED_VEC(logits, "logits", vl);
    if (vl.stride != 1 || out_index->dtype != SLAI_DT_I32 || out_index->bytes < 4) return set_error(ctx, SLAI_E_SHAPE, "slai_sample: contiguous logits and an I32 output are required");
    if (!(temperature >= 0.0f) || !(coin >= 0.0f && coin < 1.0f)) return set_error(ctx, SLAI_E_ARG, "slai_sample: temperature must be >= 0 and the draw in [0, 1)");
    if (int rc = sampler_scratch_reserve(ctx, sample_scratch_floats(vl.n))) return rc;
    SLAI_HIP_TRY(ctx, launch_sample(ctx->stream, vl.p, vl.n, temperature, topp, coin, ctx->sampler_scratch, (int *)out_index->dptr, nullptr, nullptr,
                                    nullptr));
    return SLAI_OK;
}
// The draw the device loop uses at position `pos`: the top 24 bits of splitmix64(seed + pos), scaled to [0, 1)
SLAI_EXPORT float slai_sampler_coin(uint64_t seed, uint32_t pos) {
    uint64_t x = seed + (uint64_t)pos;
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x ^= x >> 31;
    return (float)(x >> 40) * (1.0f / 16777216.0f);
}

// ---- timing ---------------------------------------------------------------------------
SLAI_EXPORT int slai_timer_begin(slai_ctx *ctx) {
    if (!ctx) return SLAI_E_ARG;
    if (!ctx->timer0) {
        SLAI_HIP_TRY(ctx, hipEventCreate(&ctx->timer0));
        SLAI_HIP_TRY(ctx, hipEventCreate(&ctx->timer1));
    }
    SLAI_HIP_TRY(ctx, hipEventRecord(ctx->timer0, ctx->stream));
    return SLAI_OK;
}
SLAI_EXPORT int slai_timer_end(slai_ctx *ctx, float *elapsed_ms) {
    if (!ctx || !elapsed_ms) return SLAI_E_ARG;
    if (!ctx->timer0) return set_error(ctx, SLAI_E_STATE, "slai_timer_end without slai_timer_begin");
    SLAI_HIP_TRY(ctx, hipEventRecord(ctx->timer1, ctx->stream));
    SLAI_HIP_TRY(ctx, hipEventSynchronize(ctx->timer1));
    SLAI_HIP_TRY(ctx, hipEventElapsedTime(elapsed_ms, ctx->timer0, ctx->timer1));
    return SLAI_OK;
}

// ---- graphs ---------------------------------------------------------------------------
SLAI_EXPORT int slai_graph_begin_capture(slai_ctx *ctx) {
    if (!ctx) return SLAI_E_ARG;
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "capture already in progress");
    SLAI_HIP_TRY(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return SLAI_OK;
}
SLAI_EXPORT int slai_graph_end_capture(slai_ctx *ctx, slai_graph **out) {
    if (!ctx || !out) return SLAI_E_ARG;
    if (!ctx->capturing) return set_error(ctx, SLAI_E_STATE, "no capture in progress");
    ctx->capturing = false;
    slai_graph *g = new slai_graph();
    hipError_t e = hipStreamEndCapture(ctx->stream, &g->graph);
    if (e == hipSuccess) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        if (g->graph) (void)hipGraphDestroy(g->graph);
        delete g;
        return hip_fail(ctx, e, "slai_graph_end_capture");
    }
    *out = g;
    return SLAI_OK;
}
SLAI_EXPORT int slai_graph_launch(slai_ctx *ctx, slai_graph *g) {
    if (!ctx || !g) return SLAI_E_ARG;
    SLAI_HIP_TRY(ctx, hipGraphLaunch(g->exec, ctx->stream));
    return SLAI_OK;
}
SLAI_EXPORT void slai_graph_destroy(slai_ctx *ctx, slai_graph *g) {
    if (!g) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
}
