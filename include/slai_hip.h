/*
 * slai_hip.h -- C ABI of libslai_hip.so, the MI355X (gfx950) implementation of slai's
 * per-token decode path.
 *
 * Every entry point names the reference interface it stands in for
 * (paths relative to the dimforge/slai tree).  All functions return 0 on success or a
 * negative SLAI_E_* code; slai_last_error() gives the message (the reference's
 * `Result<(), B::Error>`).  Shape violations return SLAI_E_SHAPE instead of panicking.
 *
 * A context owns one HIP stream; every launch goes to it.  A context is not thread
 * safe (the reference serialises forwards with three RwLock write guards,
 * crates/slai-chat/src/chat_llama2.rs:170-172); distinct contexts are independent.
 */
#ifndef SLAI_HIP_H
#define SLAI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SLAI_OK 0
#define SLAI_E_HIP (-1)       /* a HIP runtime call failed */
#define SLAI_E_SHAPE (-2)     /* dimension / stride / alignment mismatch */
#define SLAI_E_TYPE (-3)      /* unsupported ggml type tag */
#define SLAI_E_ARG (-4)       /* null or out-of-range argument */
#define SLAI_E_PARSE (-5)     /* malformed GGUF */
#define SLAI_E_MISSING (-6)   /* missing tensor / metadata key */
#define SLAI_E_STATE (-7)     /* call not valid in the current state */
#define SLAI_E_IO (-8)        /* a file could not be opened or mapped */

typedef struct slai_ctx slai_ctx;
typedef struct slai_buffer slai_buffer;
typedef struct slai_qmat slai_qmat;
typedef struct slai_graph slai_graph;
typedef struct slai_tensor_cache slai_tensor_cache;
typedef struct slai_tokenizer slai_tokenizer;
typedef struct slai_gguf slai_gguf;
typedef struct slai_llama2 slai_llama2;
typedef struct slai_gpt2 slai_gpt2;

/* stensor `GpuTensorView` = buffer slice + `ViewShape{size, strides, offset}` (used
 * throughout crates/slai/src/context.rs).  Offsets and strides are in ELEMENTS of
 * the buffer's scalar type; element (i,j,k,l) lives at
 * offset + i*stride[0] + j*stride[1] + k*stride[2] + l*stride[3].
 * size = [nrows, ncols, nmats, ncubes]. */
typedef struct {
    slai_buffer *buf;
    uint64_t offset;
    uint32_t size[4];
    uint32_t stride[4];
} slai_view;

/* crates/slai/src/ops/rms_norm.rs:15-21 */
typedef struct { float nudge_factor; uint32_t _padding[3]; } slai_rms_norm_config;
/* crates/slai/src/ops/rope.rs:24-33 */
typedef struct { uint32_t head_size, kv_dim, pos; float base_freq; } slai_rope_config;
/* crates/slai/src/ops/batched_multiquery_attention.rs:17-29 */
typedef struct { uint32_t seq_len, kv_dim, kv_mul, n_heads, head_size, pos; uint32_t _padding[2]; } slai_attn_params;

/* wgpu BufferUsages bits accepted by the constructors (crates/slai/src/models/llama2/transformer.rs:49-137);
 * only MAP_READ changes behaviour (pinned host staging for slai_read_buffer). */
#define SLAI_USAGE_MAP_READ 0x1u
#define SLAI_USAGE_COPY_SRC 0x4u
#define SLAI_USAGE_COPY_DST 0x8u
#define SLAI_USAGE_UNIFORM 0x40u
#define SLAI_USAGE_STORAGE 0x80u

/* Buffer scalar types. */
#define SLAI_DT_F32 0
#define SLAI_DT_F16 1
#define SLAI_DT_U8 2
#define SLAI_DT_I32 3

/* crates/slai/src/ops/rope.rs:8-14 `RoPEVariant` */
#define SLAI_ROPE_ORIGINAL 0
#define SLAI_ROPE_NEOX 1
/* stensor `MatrixMode` N / T (crates/slai/src/context.rs:298-317) */
#define SLAI_MODE_N 0
#define SLAI_MODE_T 1

/* ---- context / backend -------------------------------------------------
 * slang_hal `Backend` + `LlmOps::new` (crates/slai/src/context.rs:48-66): creating the
 * context loads the one code object that holds every kernel. */
int slai_ctx_create(int device, slai_ctx **out);
void slai_ctx_destroy(slai_ctx *ctx);
const char *slai_last_error(slai_ctx *ctx);
/* The HIP stream every launch of this context goes to (as a `hipStream_t`). */
void *slai_ctx_stream(slai_ctx *ctx);

/* `LlmContext::begin_submission` / `submit` (crates/slai/src/context.rs:79-95) and
 * `Backend::synchronize` (crates/slai-chat/src/chat_llama2.rs:219). */
int slai_begin_submission(slai_ctx *ctx);
int slai_submit(slai_ctx *ctx);
int slai_synchronize(slai_ctx *ctx);

/* ---- buffers ------------------------------------------------------------
 * `GpuTensor::{vector,matrix,scalar}(_uninit)` allocations
 * (crates/slai/src/models/llama2/transformer.rs:54-137); buffers are zero-filled. */
int slai_buffer_create(slai_ctx *ctx, size_t bytes, int dtype, uint32_t usage, slai_buffer **out);
void slai_buffer_destroy(slai_ctx *ctx, slai_buffer *buf);
size_t slai_buffer_size(const slai_buffer *buf);
void *slai_buffer_device_ptr(const slai_buffer *buf);
/* `TensorCache` (crates/slai/src/tensor_cache.rs:126-204), the pool of temporaries behind `LlmContext`
 * (context.rs:69-76,107-127): idle buffers keyed by element type, shape[4] and usage.
 *   get_or_insert (:162-188)  an idle buffer with this key (contents as its last holder left them) or a new zero-filled
 *                             one; a hit allocates nothing and is legal during graph capture, a miss is SLAI_E_STATE there
 *   reclaim (:118-124,199-203, what dropping a `CachedTensor` does)  back into the pool under its key
 *   clear (:195-197; the chat calls it once per token, chat_llama2.rs:174)  frees the idle buffers; SLAI_E_STATE during
 *                             a capture.  A buffer that was handed out while a graph was being captured may be named by that
 *                             graph, so clear / destroy keep its memory until the context is destroyed (the pool forgets it)
 *   destroy                   clear + the cache itself; inside a capture nothing is synchronised or freed (the idle buffers
 *                             are kept until the context is destroyed) and the capture goes on
 *   idle  number of buffers in the pool.
 * slai_buffer_destroy refuses (message in slai_last_error, nothing freed) a buffer that sits idle in a cache, and inside a
 * capture keeps the buffer's memory until the context is destroyed.
 * The models of this library do not use it: `Llama2State` preallocates every activation (transformer.rs:47-140). */
int slai_tensor_cache_create(slai_ctx *ctx, slai_tensor_cache **out);
void slai_tensor_cache_destroy(slai_ctx *ctx, slai_tensor_cache *cache);
int slai_tensor_cache_get_or_insert(slai_ctx *ctx, slai_tensor_cache *cache, int dtype, const uint32_t shape[4], uint32_t usage,
                                    slai_buffer **out);
int slai_tensor_cache_reclaim(slai_ctx *ctx, slai_tensor_cache *cache, slai_buffer *buf);
int slai_tensor_cache_clear(slai_ctx *ctx, slai_tensor_cache *cache);
size_t slai_tensor_cache_idle(const slai_tensor_cache *cache);
/* `Backend::write_buffer` (crates/slai-chat/src/chat_llama2.rs:180-185); byte offsets. */
int slai_write_buffer(slai_ctx *ctx, slai_buffer *buf, size_t offset, const void *src, size_t bytes);
/* `Backend::read_buffer` (crates/slai-chat/src/chat_llama2.rs:225-227); synchronises. */
int slai_read_buffer(slai_ctx *ctx, const slai_buffer *buf, size_t offset, void *dst, size_t bytes);
/* `GpuTensor::copy_from_view` (crates/slai-chat/src/chat_llama2.rs:186-188,207). */
int slai_copy_buffer(slai_ctx *ctx, slai_buffer *dst, size_t dst_offset, const slai_buffer *src,
                     size_t src_offset, size_t bytes);

/* ---- quantized matrices ---------------------------------------------------
 * `GpuQuantMatrix` (crates/slai/src/quantized_matrix.rs:11-22) built by
 * `GgufTensorData::to_gpu_matrix` (crates/slai/src/gguf.rs:133-194).  `packed` holds
 * nrows rows of verbatim GGUF blocks (ggml type tag as in gguf.rs:75-107:
 * 0 F32, 1 F16, 2 Q4_0, 8 Q8_0, 12 Q4_K, 13 Q5_K, 14 Q6_K).  Any block count is
 * accepted (no pairing constraint), F16 stays 16-bit. */
int slai_qmat_create(slai_ctx *ctx, uint32_t ggml_type, uint32_t nrows, uint32_t ncols, const void *packed,
                     slai_qmat **out);
/* The same with the device layout chosen by the caller.  Layouts are private regroupings of the packed GGUF
 * bytes; every layout serves every op, they differ in speed.  AUTO picks by shape; ROWS keeps rows contiguous;
 * TILE16 / TILE64 regroup 16..64-row tiles for the row-per-lane GEMVs (TILE64: matrices that are launched
 * together over the same input and jointly have many rows, e.g. q/k/v or gate/up). */
#define SLAI_LAYOUT_AUTO 0
#define SLAI_LAYOUT_ROWS 1
#define SLAI_LAYOUT_TILE16 2
#define SLAI_LAYOUT_TILE64 3
int slai_qmat_create_layout(slai_ctx *ctx, uint32_t ggml_type, uint32_t nrows, uint32_t ncols, const void *packed,
                            int layout, slai_qmat **out);
void slai_qmat_destroy(slai_ctx *ctx, slai_qmat *m);
/* `GpuQuantMatrix::shape` (quantized_matrix.rs:72-86): [nrows, ncols] in elements, and the type tag. */
int slai_qmat_shape(const slai_qmat *m, uint32_t *nrows, uint32_t *ncols, uint32_t *ggml_type);
/* Bytes the matrix occupies in device memory. */
size_t slai_qmat_device_bytes(const slai_qmat *m);
/* `GgufTensorData::dequantize` (crates/slai/src/gguf.rs:116-131, block math
 * crates/slai/src/quantization.rs) evaluated on the device from the device layout:
 * rows [row0, row0+nrows) to a dense row-major f32 view.  Bit-exact. */
int slai_qmat_dequantize(slai_ctx *ctx, const slai_qmat *m, uint32_t row0, uint32_t nrows, slai_view out);

/* ---- ops: the `LlmContext` facade (crates/slai/src/context.rs) -------------
 * Out-parameter first, then inputs, as in the reference. */
/* context.rs:230-246 -> ops/rms_norm.rs:35-66, shader rms_norm.slang:48-67 */
int slai_rms_norm_assign(slai_ctx *ctx, const slai_buffer *config, slai_view out, slai_view value, slai_view weight);
/* context.rs:205-217 -> ops/layernorm.rs:60-98 (rows of a vector = one group), no affine;
 * eps is explicit (the shader hard-codes 1e-6, the CPU path 1e-5: layernorm.slang:6, ops/layernorm.rs:105). */
int slai_layernorm_assign(slai_ctx *ctx, slai_view out, slai_view value, float eps);
/* context.rs:355-369 -> ops/gemv_quant.rs:206-312: out = m * v */
int slai_matmul_quant_assign(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view v);
/* context.rs:298-317 (stensor f32 Gemv): out = op(a) * op(b), batched over dims 2,3 */
int slai_matmul_assign(slai_ctx *ctx, slai_view out, slai_view a, slai_view b, int a_mode, int b_mode);
/* context.rs:428-441 / 456-469 / 660-672 (stensor OpAssign Add / Mul / Copy) */
int slai_add_assign(slai_ctx *ctx, slai_view in_out_a, slai_view b);
int slai_mul_assign(slai_ctx *ctx, slai_view in_out_a, slai_view b);
int slai_copy(slai_ctx *ctx, slai_view in, slai_view out);
/* context.rs:471-487 -> ops/rope.rs:45-85, rope.slang:27-84 */
int slai_rope(slai_ctx *ctx, int variant, const slai_buffer *config, slai_view in_out_q, slai_view in_out_k);
/* context.rs:489-501 -> ops/silu.rs:24-48, silu.slang:11-27 */
int slai_silu(slai_ctx *ctx, slai_view in_out_h1, slai_view in_h2);
/* context.rs:565-570 -> ops/unary.rs:159-223 (UnaryOp::Gelu), unary.slang:67-74 */
int slai_gelu_inplace(slai_ctx *ctx, slai_view x);
/* context.rs:760-785, batched_multiquery_attention.slang:18-32 */
int slai_attn_mask(slai_ctx *ctx, const slai_attn_params *params, const slai_buffer *params_gpu, slai_buffer *attn);
/* context.rs:787-797 -> ops/softmax.rs:22-40, softmax.slang:26-96 */
int slai_softmax_cols(slai_ctx *ctx, slai_view in_out_mat);
/* `BatchedMultiqueryAttention::launch` (ops/batched_multiquery_attention.rs:32-100): one fused
 * kernel pair (QK^T, softmax, .V with split-K) instead of the reference's four launches.
 * Caches are [kv_dim x seq_len] column-major, f32 or f16 by the buffer's dtype.  `att` is
 * accepted for signature parity and not written. */
int slai_attention(slai_ctx *ctx, const slai_attn_params *params, const slai_buffer *params_gpu, slai_view q,
                   slai_view key_cache, slai_view value_cache, slai_view att, slai_view xb);
/* slai_attention without any allocation.  It has no counterpart in the reference: it is for callers that cannot call
 * hipMalloc -- code under HIP graph capture, tight serving loops, harnesses that forbid allocation.  Same arguments,
 * kernels and results as slai_attention; the per-split partial results live in a static device array of
 * 524288 floats (2 MiB, held by every GPU the library runs on until the process ends), so n_heads * splits *
 * (head_size + 2) must not exceed that (SLAI_E_SHAPE otherwise; 32 heads of 128 at any context need 66560).  All calls on
 * one GPU share the array: calls that overlap in time on one GPU race. */
int slai_attention_static(slai_ctx *ctx, const slai_attn_params *params, const slai_buffer *params_gpu, slai_view q,
                          slai_view key_cache, slai_view value_cache, slai_view att, slai_view xb);
/* `Sampler::sample_argmax` (crates/slai/src/models/sampler.rs:55-57; first strict maximum),
 * on the device; out_index is a 1-element I32 buffer. */
int slai_argmax(slai_ctx *ctx, slai_view logits, slai_buffer *out_index);
/* `Sampler::sample` (models/sampler.rs:33-53): temperature 0 is the arg-max; otherwise softmax of
 * logits / temperature, then `sample_mult` (:63-78) when topp is outside (0, 1), else `sample_topp`
 * (:85-131).  `coin` in [0, 1) is the draw the reference takes from `rand::random()`.  The logits are
 * not modified.  Sums run in a different order than the reference's sequential ones: the result can
 * differ from it when `coin` lies within rounding distance of a boundary of the cumulative distribution. */
int slai_sample(slai_ctx *ctx, slai_view logits, float temperature, float topp, float coin, slai_buffer *out_index);
/* the draw the device-side loops use at position `pos`: top 24 bits of splitmix64(seed + pos) / 2^24 */
float slai_sampler_coin(uint64_t seed, uint32_t pos);

/* ---- fused forms of the call sequences `Llama2::launch` issues (no single reference counterpart;
 * each replaces the listed context.rs calls with one kernel, same results up to summation order) */
/* rms_norm_assign(xb, x, w) + matmul_quant_assign(out, m, xb)   (transformer.rs:327-334, 368-375) */
int slai_rms_norm_matmul_quant_assign(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view x, slai_view norm_weight,
                                      float eps);
/* rms_norm_assign + matmul_quant_assign(hb, gate) + matmul_quant_assign(hb2, up) + silu(hb, hb2)
 * (transformer.rs:356-361); gate and up must share a format */
int slai_ffn_gate_up_silu(slai_ctx *ctx, slai_view out_hb, const slai_qmat *gate, const slai_qmat *up, slai_view x,
                          slai_view norm_weight, float eps);
/* matmul_quant_assign(xb2, m, v) + add_assign(x, xb2)   (transformer.rs:352-355, 362-365) */
int slai_matmul_quant_add_assign(slai_ctx *ctx, slai_view in_out_x, const slai_qmat *m, slai_view v);
/* "Prepared" activations: for an input x and the weight w of the RMSNorm that follows it, the n products x[i]*w[i]
 * followed by the n/16 sums of 16 consecutive products (n + n/16 contiguous floats, 64-byte aligned, n % 16 == 0).
 * A GEMV over a TILE64 matrix that is handed this form reads its activations directly and only derives the norm's
 * scale from x; it equals slai_rms_norm_assign + slai_matmul_quant_assign.  slai_rms_norm_prepare builds the form
 * from x; slai_matmul_quant_add_assign_emit is slai_matmul_quant_add_assign that also leaves the form of its result
 * (with the weight of the norm that comes next) for the GEMV after it, so that no separate pass is needed. */
int slai_rms_norm_prepare(slai_ctx *ctx, slai_view out_prepared, slai_view x, slai_view norm_weight);
/* out = m . v for v in prepared form built with a weight of all ones (no norm): slai_matmul_quant_assign for TILE64 */
/* Up to 32 vectors through one quantised matrix in one pass over it, on the fp32 matrix cores: out[:, t] = m * x[:, t]
 * (accumulate != 0: +=) for contiguous column-major `out` (nrows x n) and `x` (ncols x n), n <= 32.  The operator under
 * slai_llama2_prefill; matrices in a tiled layout only (SLAI_E_SHAPE otherwise).  No counterpart in the reference, whose
 * `matmul_quant` (context.rs:355-399) takes one vector. */
int slai_matmul_quant_columns(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view x, int accumulate);
int slai_matmul_quant_assign_prepared(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view prepared);
int slai_rms_norm_matmul_quant_assign_prepared(slai_ctx *ctx, slai_view out, const slai_qmat *m, slai_view x, slai_view prepared,
                                               float eps);
int slai_ffn_gate_up_silu_prepared(slai_ctx *ctx, slai_view out_hb, const slai_qmat *gate, const slai_qmat *up, slai_view x,
                                   slai_view prepared, float eps);
int slai_matmul_quant_add_assign_emit(slai_ctx *ctx, slai_view in_out_x, const slai_qmat *m, slai_view v, slai_view next_norm_weight,
                                      slai_view out_prepared);

/* ---- GPU timing on the context's stream with HIP events: the role of the GPU timestamp
 * queries bracketing a pass in crates/slai-bench/src/main.rs:198,223-241.  slai_timer_end
 * synchronises and returns the milliseconds since the matching slai_timer_begin. */
int slai_timer_begin(slai_ctx *ctx);
int slai_timer_end(slai_ctx *ctx, float *elapsed_ms);

/* ---- HIP graph capture of a submission (no reference counterpart: the reference
 * re-encodes ~550 dispatches per token, crates/slai-chat/src/chat_llama2.rs:179-230) */
int slai_graph_begin_capture(slai_ctx *ctx);
int slai_graph_end_capture(slai_ctx *ctx, slai_graph **out);
int slai_graph_launch(slai_ctx *ctx, slai_graph *g);
void slai_graph_destroy(slai_ctx *ctx, slai_graph *g);

/* ---- GGUF (crates/slai/src/gguf.rs) -----------------------------------------
 * `Gguf::from_bytes` (gguf.rs:504-524).  The bytes must outlive the handle. */
int slai_gguf_parse(const void *bytes, size_t len, slai_gguf **out, char *err, size_t err_len);
/* The same over a read-only mapping of a file, which the handle owns (the headless chat maps the model file and
 * parses the mapping: crates/slai-chat/src/cli.rs:43-57); tensors are uploaded straight from the mapping. */
int slai_gguf_open_file(const char *path, slai_gguf **out, char *err, size_t err_len);
void slai_gguf_free(slai_gguf *g);
uint32_t slai_gguf_version(const slai_gguf *g);
uint64_t slai_gguf_tensor_count(const slai_gguf *g);
uint64_t slai_gguf_metadata_count(const slai_gguf *g);
uint64_t slai_gguf_data_start(const slai_gguf *g);
/* tensor i: name, dims [nrows, ncols, nmats, ncubes] (gguf.rs:579-581), ggml type, absolute offset */
int slai_gguf_tensor_info(const slai_gguf *g, uint64_t i, const char **name, uint64_t dims[4], uint32_t *ggml_type,
                          uint64_t *offset);
int slai_gguf_find_tensor(const slai_gguf *g, const char *name, uint64_t *index);
/* metadata lookups (gguf.rs:283-331 `unwrap_u32`, `as_f32`, `as_string`, `unwrap_array_len`) */
int slai_gguf_meta_u32(const slai_gguf *g, const char *key, uint32_t *out);
int slai_gguf_meta_f32(const slai_gguf *g, const char *key, float *out);
int slai_gguf_meta_str(const slai_gguf *g, const char *key, const char **out);
int slai_gguf_meta_array_len(const slai_gguf *g, const char *key, uint64_t *out);
/* `metadata_debug_strings` (gguf.rs:686-695): entry i of slai_gguf_metadata_count(), keys in sorted order, as
 * "key = Type(value)" or "key = array[len]" */
int slai_gguf_meta_describe(const slai_gguf *g, uint64_t i, char *out, size_t out_len);
/* `as_string_array` (gguf.rs:316-322): pointers into the file bytes (not NUL-terminated) and lengths of the first
 * `capacity` elements; `count` receives the number of elements.  `as_f32_array` (gguf.rs:324-330) likewise. */
int slai_gguf_meta_array_str(const slai_gguf *g, const char *key, const char **ptrs, uint64_t *lens, uint64_t capacity,
                             uint64_t *count);
int slai_gguf_meta_array_f32(const slai_gguf *g, const char *key, float *out, uint64_t capacity, uint64_t *count);
/* `GgufTensor::to_gpu_matrix` (gguf.rs:357-366) */
int slai_gguf_tensor_to_qmat(slai_ctx *ctx, const slai_gguf *g, const char *name, slai_qmat **out);
int slai_gguf_tensor_to_qmat_layout(slai_ctx *ctx, const slai_gguf *g, const char *name, int layout, slai_qmat **out);

/* ---- Llama-2 / Qwen2 model assembly ------------------------------------------
 * `ChatLlama2::from_gguf_with_model_type` (crates/slai-chat/src/chat_llama2.rs:39-62):
 * `Llama2Config::from_gguf_with_model_type` (models/llama2/cpu.rs:79-109),
 * `Llama2Weights::from_gguf` (models/llama2/transformer.rs:202-297),
 * `Llama2State::new` (transformer.rs:47-140). */
#define SLAI_MODEL_LLAMA 0
#define SLAI_MODEL_QWEN2 1
#define SLAI_KV_F32 0   /* the reference's cache type (transformer.rs:87-106) */
#define SLAI_KV_F16 1
typedef struct {
    uint32_t dim, hidden_dim, n_layers, n_q_heads, n_kv_heads, vocab_size, seq_len;
    float rope_base_freq, rms_norm_eps;
} slai_llama2_config;   /* models/llama2/cpu.rs:46-67 */

int slai_llama2_from_gguf(slai_ctx *ctx, const slai_gguf *g, int model_type, int kv_dtype, slai_llama2 **out);
/* Host-only check of everything slai_llama2_from_gguf reads: hyper-parameters, then presence, block format and shape of
 * every tensor against them (the kernels index norm vectors and biases by the model's widths).  Replaces the `unwrap()`s
 * and shape asserts of `Llama2Weights::from_gguf` (transformer.rs:202-297) with an error code and message; needs no
 * device.  slai_llama2_from_gguf runs it first and uploads nothing when it fails. */
int slai_llama2_check_gguf(const slai_gguf *g, int model_type, char *err, size_t err_len);
void slai_llama2_destroy(slai_llama2 *m);
int slai_llama2_get_config(const slai_llama2 *m, slai_llama2_config *out);
/* Bytes of packed weights resident in device memory (roofline denominator). */
size_t slai_llama2_weight_bytes(const slai_llama2 *m);
/* `ChatLlama2::forward_logits` (chat_llama2.rs:163-240): one position through
 * `Llama2::launch` (transformer.rs:316-381); logits (vocab floats) copied to `logits_out` when
 * not NULL.  fused = 0 issues the reference's op sequence one kernel per op; fused = 1 uses the
 * fused kernels (norm-in-GEMV, gate/up+SiLU, residual epilogues, RoPE-in-attention). */
int slai_llama2_forward_logits(slai_llama2 *m, uint32_t pos, uint32_t token, int fused, float *logits_out);
/* The per-token loop of `ChatLlama2::forward` (chat_llama2.rs:105-158) with greedy sampling and
 * the forced-token rule (crates/slai-chat/src/sampler.rs:100-105): runs positions
 * start_pos .. start_pos+n_steps-1 entirely on the device (one captured graph replayed per
 * token, argmax and token feedback on the device); out_tokens[i] = token chosen after step i.
 * elapsed_ms (optional) = stream time of the n_steps replays measured with HIP events. */
int slai_llama2_generate(slai_llama2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos,
                         uint32_t n_steps, int32_t *out_tokens, float *elapsed_ms);
/* The same loop with `Sampler::new(vocab, temperature, topp).sample()` run on the device (the chat
 * samples every generated token with 0.7 / 0.95: crates/slai-chat/src/sampler.rs:100-108), so no
 * logits cross the bus.  Draws are slai_sampler_coin(seed, pos). */
int slai_llama2_generate_sampled(slai_llama2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos,
                                 uint32_t n_steps, float temperature, float topp, uint64_t seed, int32_t *out_tokens,
                                 float *elapsed_ms);
/* Prompt tokens in chunks.  The reference feeds a prompt one token per forward pass and discards the logits of every
 * prompt position but the last (chat_llama2.rs:105-158 with the forced-token rule, slai-chat/src/sampler.rs:100-105);
 * this fills the caches for positions start_pos .. start_pos+n_tokens-1 with `chunk` tokens per pass over the
 * weights and computes no logits (chunk: 0 = the path's default, 1 = token by token, at most 64).  Generation then
 * continues with slai_llama2_generate(prompt, n_prompt, n_prompt - 1, ...).  slai_llama2_prefill_supported() says which
 * path a model takes: 2 = matrix-core GEMM over the dequantised tiles (every format with a tiled layout), at most
 * 32 tokens per pass: on the half-precision units with every weight and activation split into an f16 head and an f16
 * remainder (about 22 bits of each, fp32 accumulation), repeated with fp32 MFMA when an activation turns out to be beyond
 * the f16 range (slai_llama2_prefill_fp32_repeats counts those calls), in fp32 MFMA from the start when the context was
 * created with SLAI_PROMPT_SPLIT_F16=0 or when the block scales of a layer matrix allow a weight of 255 or more in
 * magnitude (the pair form holds 256 * w in f16; trained models are orders of magnitude below); 1 = the GEMV kernels with one workgroup per token and tile sharing the weights through L2 (the
 * same layouts when the context was created with SLAI_PROMPT_GEMM=0); 0 = layouts without chunked kernels, run token by
 * token with the same result. */
int slai_llama2_prefill(slai_llama2 *m, const int32_t *tokens, uint32_t n_tokens, uint32_t start_pos, uint32_t chunk,
                        float *elapsed_ms);
int slai_llama2_prefill_supported(const slai_llama2 *m);
uint32_t slai_llama2_prefill_fp32_repeats(const slai_llama2 *m);
/* Which form the per-token loop of this model takes: 0 = one launch per step of `Llama2::launch` (transformer.rs:316-381;
 * four to five per layer), 1 = the whole layer stack and the output matrix in one resident launch per token (widths of
 * 1024 .. 4096 in steps of 1024, as many cache heads as query heads of size 128, Q4_K / Q5_K / Q6_K mixes, gate / up in
 * Q4_K; a context created with SLAI_PERSISTENT=0 in the environment never takes it).  The form is chosen per token: a model
 * of form 1 takes the resident launch at positions below SLAI_RESIDENT_MAX_POS (environment, default 2048) and one launch
 * per step beyond, with the same caches and loop state.  Results are the same to within summation order. */
int slai_llama2_decode_form(const slai_llama2 *m);
/* Measurement aid without a reference counterpart (profilers see the resident launch as one kernel): runs one token at
 * (pos, token) with in-kernel time stamps and returns them, n_workgroups x stamps_per_workgroup 64-bit ticks of the
 * constant 100 MHz clock; per workgroup 16 per layer -- 4 per phase (q/k/v + attention, output projection, gate/up, down
 * projection): entered, input staged, multiplied, reduced -- then 8 for the output matrix.  Zero = phase not taken. */
int slai_llama2_trace_token(slai_llama2 *m, uint32_t pos, uint32_t token, uint64_t *out, size_t capacity, uint32_t *n_workgroups,
                            uint32_t *stamps_per_workgroup);
/* Measurement aid without a reference counterpart (the reference times whole forwards, slai-bench/src/main.rs:184-247):
 * one token at (pos, token) through the launch-per-step form, launched from the host `reps` times with an event after
 * every launch.  Returns, per step name in order of first appearance (`names`: newline separated, e.g. "llama2 qkv +
 * attention"), the mean time from the end of the launch before it to the end of the step's launch in microseconds, and
 * how many times the step occurs per token.  The intervals include the event markers (a few microseconds each), so their
 * sum is above the time of a token replayed from a graph; `alone_us` is each step's launches alone, one per layer back to
 * back with events only before the first and after the last: the figure to set against a profiler's kernel duration.
 * SLAI_E_STATE for a model that takes the resident launch. */
int slai_llama2_time_steps(slai_llama2 *m, uint32_t pos, uint32_t token, uint32_t reps, char *names, size_t names_len, float *mean_us,
                           float *alone_us, uint32_t *per_token, uint32_t capacity, uint32_t *n_steps);
/* Device access for set-up and inspection: layer l's caches ([kv_dim x seq_len]) and the state vectors. */
int slai_llama2_kv_buffers(slai_llama2 *m, uint32_t layer, slai_buffer **key_cache, slai_buffer **value_cache);
int slai_llama2_logits_buffer(slai_llama2 *m, slai_buffer **logits);

/* ---- GPT-2 model assembly (crates/slai/src/models/gpt2/cpu.rs:19-48,113-217,224-383) */
typedef struct { uint32_t n_vocab, n_seq, n_embd, n_head, n_layer, ff_len, attn_b; } slai_gpt2_params;
int slai_gpt2_from_gguf(slai_ctx *ctx, const slai_gguf *g, int kv_dtype, slai_gpt2 **out);
/* The same host-only check for a GPT-2 file (`Gpt2Model::from_gguf`, gpt2/cpu.rs:118-190, unwraps instead). */
int slai_gpt2_check_gguf(const slai_gguf *g, char *err, size_t err_len);
void slai_gpt2_destroy(slai_gpt2 *m);
int slai_gpt2_get_params(const slai_gpt2 *m, slai_gpt2_params *out);
size_t slai_gpt2_weight_bytes(const slai_gpt2 *m);
int slai_gpt2_forward_logits(slai_gpt2 *m, uint32_t pos, uint32_t token, float *logits_out);
int slai_gpt2_generate(slai_gpt2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos,
                       uint32_t n_steps, int32_t *out_tokens, float *elapsed_ms);
int slai_gpt2_generate_sampled(slai_gpt2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos,
                               uint32_t n_steps, float temperature, float topp, uint64_t seed, int32_t *out_tokens,
                               float *elapsed_ms);
/* slai_llama2_prefill for GPT-2 (gpt2/cpu.rs:225-383 for a chunk of tokens; no counterpart in the reference): 32 tokens
 * per pass over the weights on the matrix cores where every layer matrix has a tiled layout
 * (slai_gpt2_prefill_supported() == 2; f16 head + remainder pairs with the fp32 repeat of slai_llama2_prefill, counted by
 * slai_gpt2_prefill_fp32_repeats), token by token with the same result otherwise (0). */
int slai_gpt2_prefill(slai_gpt2 *m, const int32_t *tokens, uint32_t n_tokens, uint32_t start_pos, uint32_t chunk,
                      float *elapsed_ms);
int slai_gpt2_prefill_supported(const slai_gpt2 *m);
uint32_t slai_gpt2_prefill_fp32_repeats(const slai_gpt2 *m);

/* ---- Tokenizers (host only) ---------------------------------------------------
 * `AnyTokenizer` (crates/slai-chat/src/llm.rs:100-164) over `LlamaTokenizer`
 * (crates/slai/src/models/llama2/tokenizer.rs:23-179) and `Gpt2Tokenizer`
 * (crates/slai/src/models/gpt2/tokenizer.rs:55-216), read from the GGUF metadata keys
 * tokenizer.ggml.{model,tokens,scores,merges,bos_token_id,eos_token_id,unknown_token_id}.
 * Where the reference panics (text that needs a byte-fallback id outside the vocabulary, a
 * `<...>` span that is not a token, a merge line with fewer than two fields) these return an
 * error; slai_tokenizer_last_error() gives the message. */
#define SLAI_TOKENIZER_AUTO (-1)  /* by `tokenizer.ggml.model`, llm.rs:106-118 */
#define SLAI_TOKENIZER_LLAMA 0
#define SLAI_TOKENIZER_GPT2 1
int slai_tokenizer_from_gguf(const slai_gguf *g, int kind, slai_tokenizer **out, char *err, size_t err_len);
void slai_tokenizer_free(slai_tokenizer *t);
int slai_tokenizer_kind(const slai_tokenizer *t);
uint32_t slai_tokenizer_bos(const slai_tokenizer *t);
uint32_t slai_tokenizer_eos(const slai_tokenizer *t);
uint32_t slai_tokenizer_unk(const slai_tokenizer *t); /* UINT32_MAX for GPT-2 */
uint32_t slai_tokenizer_vocab_size(const slai_tokenizer *t);
const char *slai_tokenizer_last_error(const slai_tokenizer *t);
/* bytes (not NUL-terminated) and length of a vocabulary entry: `bos_str` / `eos_str` */
int slai_tokenizer_token_str(const slai_tokenizer *t, uint32_t id, const char **ptr, size_t *len);
/* `encode(text, bos, eos)`; the GPT-2 tokenizer ignores the two flags (llm.rs:156-162).  `count`
 * receives the number of ids even when `capacity` is too small (SLAI_E_SHAPE). */
int slai_tokenizer_encode(slai_tokenizer *t, const char *text, size_t text_len, int bos, int eos, int32_t *out,
                          size_t capacity, size_t *count);
/* `decode(prev_token, token)` (llm.rs:149-154) over a run: Llama decodes token i with token i-1
 * (`prev_token` for the first) as predecessor; GPT-2 decodes the run as a whole. */
int slai_tokenizer_decode(slai_tokenizer *t, const int32_t *tokens, size_t n, int32_t prev_token, char *out,
                          size_t capacity, size_t *len);

#ifdef __cplusplus
}
#endif
#endif /* SLAI_HIP_H */
