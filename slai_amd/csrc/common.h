// Internal definitions shared by the runtime and the kernel launchers of libslai_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "slai_hip.h"

#define SLAI_EXPORT extern "C" __attribute__((visibility("default")))

struct slai_buffer {
    void *dptr = nullptr;
    size_t bytes = 0;
    int dtype = SLAI_DT_F32;
    uint32_t usage = 0;
    void *host_staging = nullptr;  // pinned, when created with SLAI_USAGE_MAP_READ
    uint32_t shape[4] = {0, 0, 0, 0};  // set for buffers handed out by a slai_tensor_cache (its key)
    bool idle_in_cache = false;        // back in its cache and not handed out: a second reclaim is an error
    bool captured = false;             // handed out by its cache during a graph capture: a graph may name it, so it is never freed before the context
};

struct slai_qmat {
    int type = 0;
    uint32_t nrows = 0, ncols = 0, nb = 0;  // nb = GGUF blocks per row
    // row layout (quant_formats.h): bytes between rows.  Unused when `tiled`.
    size_t row_stride = 0;
    // tiled layout (quant_tiled.h)
    bool tiled = false;
    uint32_t rows_log2 = 0, ncb = 0, ngroups = 0, ntiles = 0, unit_bytes = 0;
    uint8_t *dptr = nullptr;
    size_t bytes = 0;
    // tiled layouts: an upper bound of |w| over the matrix, from its block headers (the prompt pass takes the f16 matrix
    // cores only where 256 * |w| fits f16)
    float wbound = 0.0f;
};

// `TensorCache` (crates/slai/src/tensor_cache.rs:126-204): idle temporaries keyed by element type, shape and usage.
struct slai_tensor_key {
    int dtype; uint32_t shape[4]; uint32_t usage;
    bool operator<(const slai_tensor_key &o) const {
        if (dtype != o.dtype) return dtype < o.dtype;
        for (int i = 0; i < 4; ++i) if (shape[i] != o.shape[i]) return shape[i] < o.shape[i];
        return usage < o.usage;
    }
};
struct slai_tensor_cache {
    std::map<slai_tensor_key, std::vector<slai_buffer *>> tensors;
};

struct slai_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

struct slai_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::string err;
    bool capturing = false;
    bool submission_open = false;   // between slai_begin_submission and slai_submit
    // attention split-K partials (grown on demand, never inside a capture)
    float *attn_scratch = nullptr;
    size_t attn_scratch_floats = 0;
    // per-workgroup activation slots of the row-tile GEMV (grown on demand, never inside a capture)
    float *gemv_scratch = nullptr;
    size_t gemv_scratch_floats = 0;
    float *sampler_scratch = nullptr;   // probabilities of the device sampler (one float per vocabulary entry)
    size_t sampler_scratch_floats = 0;
    uint32_t *handoff_counters = nullptr;   // q/k/v + attention in one launch: one 128-byte line per head, then a timeout flag
    uint32_t handoff_heads = 0;
    bool fuse_qkv_attention = true;     // SLAI_FUSE_QKV_ATTN=0: always separate launches
    int prompt_split_f16 = 1;           // SLAI_PROMPT_SPLIT_F16: 0 = prompt-chunk GEMMs in fp32 MFMA, 1 = the models' on the f16 matrix cores (f16 head + remainder), 2 = slai_matmul_quant_columns too
    int *split_flag = nullptr;          // device word the kernels that write split activations set when a value is beyond f16
    bool prompt_gemm = true;            // SLAI_PROMPT_GEMM=0: prompt chunks never take the matrix-core kernels
    // tuning knobs (environment overridable, see runtime.cpp)
    int gemv_rows_per_wg = 8;
    int gemv_max_threads = 1024;
    int gemv_max_wgs = 512;     // workgroups per tiled GEMV launch (SLAI_GEMV_MAX_WGS)
    bool tiled_layout = true;   // SLAI_TILED=0 keeps every matrix in the row layout
    bool rowtile_gemv = true;   // SLAI_ROWTILE=0: no 64-row tiles / wave-uniform GEMV
    int attn_splits = 0;  // 0 = automatic
    // Scratch blocks that a larger one has replaced.  Captured graphs (and launches already queued) hold the old
    // addresses, so a block is only freed with the context.
    std::vector<void *> retired_scratch;
    std::vector<slai_buffer *> retired_buffers;   // cached tensors a captured graph may name, and buffers destroyed inside a capture
    hipEvent_t timer0 = nullptr, timer1 = nullptr;
    // the one-launch-per-token form of the Llama-2 layer stack where a model's shapes allow it (SLAI_PERSISTENT=0 switches it off)
    bool persistent = true;
    uint32_t resident_max_pos = 2048;   // tokens at positions below this take the resident launch (where the model has one): SLAI_RESIDENT_MAX_POS
    // When set, every launch of a decode step is followed by an event recorded under the step's name
    // (slai_llama2_time_steps); null otherwise.
    std::vector<std::pair<const char *, hipEvent_t>> *step_marks = nullptr;
    const char *only_step = nullptr;         // when set, launches of decode steps with another name are skipped (step timing)
    bool use_graph = true;  // SLAI_NO_GRAPH=1 replays the token sequence eagerly (profilers that cannot trace graph launches)
};

namespace slai {

int set_error(slai_ctx *ctx, int code, const std::string &msg);
int hip_fail(slai_ctx *ctx, hipError_t e, const char *what);

#define SLAI_HIP_TRY(ctx, call)                                         \
    do {                                                                \
        hipError_t e__ = (call);                                        \
        if (e__ != hipSuccess) return ::slai::hip_fail(ctx, e__, #call); \
    } while (0)

// ---- GEMV -------------------------------------------------------------------
enum : uint32_t {
    GEMV_BIAS = 1u,      // val += bias[row]
    GEMV_ACCUM = 2u,     // out[row] += val
    GEMV_SILU_GATE = 4u, // dual: val = up * gate/(1+exp(-gate))   (W = gate, W2 = up)
    GEMV_GELU = 8u,      // val = gelu(val)
    GEMV_EMIT = 16u,     // also write the weighted copy of the result for the next row-tile GEMV (tiled kernel only)
    GEMM_OUT_QUADS = 32u, // prompt-chunk GEMM only: write the result quad-major (the layout its input has)
};
enum : int { PRO_NONE = 0, PRO_RMSNORM = 1, PRO_LAYERNORM = 2 };

struct GemvSeg {
    const uint8_t *W = nullptr;
    const uint8_t *W2 = nullptr;
    size_t row_stride = 0;
    uint32_t nrows = 0;
    uint32_t nblocks = 0;  // filled by the launcher
    float *out = nullptr;
    const float *bias = nullptr;
    uint32_t flags = 0;
};
struct GemvParams {
    GemvSeg seg[3];
    int nseg = 1;
    uint32_t ncols = 0, nb = 0;
    const float *x = nullptr;
    int prologue = PRO_NONE;
    const float *norm_w = nullptr, *norm_b = nullptr;
    float eps = 0.0f;
    uint32_t rows_per_wg = 8;
};
// All segments share the ggml type `type`, the input x and the prologue.
hipError_t launch_gemv(slai_ctx *ctx, int type, GemvParams p);
bool gemv_supports(int type, uint32_t ncols);

// GEMV over the tiled layout (kernels_gemv_tiled.hip); all segments share type and column geometry.
// Several input vectors through one launch (a chunk of prompt tokens): vector b reads x + b * x_stride (and prepared + b *
// prepared_stride), writes segment i to out + b * out_stride[i] and its emitted copy to emit_out + b * emit_stride (strides
// in floats).  The workgroups that read the same weights run next to each other on one XCD, so the weights come from
// memory once per launch and from that XCD's L2 for the other vectors.  n = 1: a plain launch.
struct GemvBatch {
    uint32_t n = 1;
    uint32_t x_stride = 0, prepared_stride = 0, emit_stride = 0;
    uint32_t out_stride[3] = {0, 0, 0};
};

struct GemvTiledSeg {
    const uint8_t *W = nullptr;
    const uint8_t *W2 = nullptr;
    uint32_t nrows = 0;
    uint32_t nblocks = 0;  // filled by the launcher
    float *out = nullptr;
    const float *bias = nullptr;
    uint32_t flags = 0;
};
struct GemvTiledParams {
    GemvTiledSeg seg[3];
    int nseg = 1;
    uint32_t ncols = 0, ncb = 0, ngroups = 0, rows_log2 = 4, unit_bytes = 0;
    // A workgroup has one wave per column group, at most 16: wider matrices take several launches, each over the
    // groups [group0, group0 + launch_groups) and all but the first accumulating into the output.
    uint32_t group0 = 0, launch_groups = 0;   // launch_groups = 0: all of them
    const float *x = nullptr;
    int prologue = PRO_NONE;
    const float *norm_w = nullptr, *norm_b = nullptr;
    float eps = 0.0f;
    const float *emit_w = nullptr;    // GEMV_EMIT (segment 0): weights of the next norm
    float *emit_out = nullptr;        // [nrows + nrows/16]
};
hipError_t launch_gemv_tiled(slai_ctx *ctx, int type, GemvTiledParams p, const GemvBatch *batch = nullptr);

// GEMV over 64-row tiles with wave-uniform activations (kernels_gemv_rowtile.hip).  Segments share the
// input, the prologue and the column count; their block formats may differ.
struct GemvRowtileSeg {
    const uint8_t *W = nullptr;
    const uint8_t *W2 = nullptr;
    int type = 0;
    uint32_t nrows = 0;
    uint32_t ntiles = 0;   // filled by the launcher
    float *out = nullptr;
    const float *bias = nullptr;
    uint32_t flags = 0;
};
struct GemvRowtileParams {
    GemvRowtileSeg seg[3];
    int nseg = 1;
    uint32_t ncols = 0, ncb = 0;
    const float *x = nullptr;
    int prologue = PRO_NONE;          // PRO_NONE or PRO_RMSNORM
    const float *norm_w = nullptr;
    float eps = 0.0f;
    // When set: the weighted activations followed by their ncols/16 sums of 16, left by the kernel that produced x
    // (GEMV_EMIT); x itself is then only read for the RMSNorm sum of squares.
    const float *prepared = nullptr;
    float *scratch = nullptr;         // one slot of ncols + ncols/16 floats per workgroup (= per tile); unused with `prepared`
    uint32_t scratch_stride = 0;      // filled by the launcher
};
size_t gemv_rowtile_scratch_floats(const GemvRowtileParams &p);
// With a batch of more than one vector the input must come `prepared`.
hipError_t launch_gemv_rowtile(slai_ctx *ctx, GemvRowtileParams p, const GemvBatch *batch = nullptr);

// A chunk of up to 32 input vectors ("prompt tokens") through up to three matrices on the matrix cores
// (kernels_gemm_chunk.hip): out[t][r] = sum_c deq(W[r][c]) * x[t][c] (+ bias[r]) (+ the old out[t][r]).  The input is
// "quad-major": the float4 of columns c .. c + 3 of token t at x + ((c / 4) * 32 + t) * 4 (32 token slots whatever
// ntokens is); the output is row-major (token t at out + t * out_stride) or, with GEMM_OUT_QUADS, quad-major as well.
// K-quants in 64-row tiles (any number of segments, formats may differ) or in 16- / 32-row tiles (one segment; more than
// 16 column groups take several launches).
struct GemmChunkSeg {
    const uint8_t *W = nullptr;
    int type = 0;
    uint32_t nrows = 0;
    uint32_t ntiles = 0;   // filled by the launcher
    float *out = nullptr;
    const float *bias = nullptr;
    uint32_t flags = 0;    // GEMV_BIAS, GEMV_ACCUM, GEMM_OUT_QUADS
    uint32_t out_stride = 0;
    uint32_t part_stride = 0;   // ksplit > 1: floats between the partial results
};
struct GemmChunkParams {
    GemmChunkSeg seg[3];
    int nseg = 1;
    uint32_t ncols = 0, ncb = 0, ngroups = 0, rows_log2 = 6;
    uint32_t group0 = 0;        // 16- / 32-row tiles: first column group of this launch (set by the launcher)
    const float *x = nullptr;   // quad-major, 16-byte aligned
    uint32_t ntokens = 0;
    // 64-row tiles only.  ksplit > 1: the columns are cut into ksplit ranges of whole super-blocks, each computed by a
    // workgroup of its own (tile counts rarely divide the compute units evenly; smaller units do); range s writes its
    // partial result to out + s * part_stride and the reader adds them up.  No bias, no accumulation then.
    uint32_t ksplit = 1;
    // weights and activations as f16 head + remainder pairs on the half-precision matrix cores (about 22 bits of each;
    // |x| < 65504, |w| < 255) instead of fp32 MFMA; x must then hold the split form (split_flag of the kernels that write it).
    bool split_f16 = false;
};
bool gemm_chunk_supports(const slai_qmat *m);
hipError_t launch_gemm_chunk(slai_ctx *ctx, GemmChunkParams p);
// quad-major out = RMSNorm of the `ntokens` row-major vectors of n floats at x + t * x_stride
hipError_t launch_rms_norm_quads(hipStream_t s, float *out, const float *x, const float *w, uint32_t n, uint32_t ntokens, uint32_t x_stride, float eps, int *split_flag = nullptr);
// the same with LayerNorm (mean-centred, * g + b)
hipError_t launch_layernorm_quads(hipStream_t s, float *out, const float *x, const float *g, const float *b, uint32_t n, uint32_t ntokens, uint32_t x_stride, float eps,
                                  int *split_flag = nullptr);
// quad-major copy of row-major vectors
hipError_t launch_rows_to_quads(hipStream_t s, float *out, const float *x, uint32_t n, uint32_t ntokens, uint32_t x_stride, int *split_flag = nullptr);

// One GEMV launch over up to three matrices of one format and layout: out[i] = epilogue(m[i] . prologue(x)).
struct GemvCall {
    const slai_qmat *m[3] = {nullptr, nullptr, nullptr};
    const slai_qmat *m2[3] = {nullptr, nullptr, nullptr};   // second matrix of a SiLU-gated pair
    float *out[3] = {nullptr, nullptr, nullptr};
    const float *bias[3] = {nullptr, nullptr, nullptr};
    uint32_t flags[3] = {0, 0, 0};
    int nseg = 1;
    const float *x = nullptr;
    int prologue = PRO_NONE;
    const float *norm_w = nullptr, *norm_b = nullptr;
    float eps = 0.0f;
    // Producer side (segment 0 only, needs GEMV_EMIT in flags[0]): besides out[0], write emit_out[row] = out[row] *
    // emit_w[row] and, behind the nrows products, the nrows/16 sums of 16 consecutive products.
    const float *emit_w = nullptr;
    float *emit_out = nullptr;
    // Consumer side: such a copy of norm_w-weighted x (see GemvRowtileParams::prepared); nullptr = none.
    const float *prepared = nullptr;
    GemvBatch batch;   // more than one input vector (64-row-tile launches with prepared input and 16-row-tile launches only)
};
// True when gemv_call would honour GEMV_EMIT for this matrix as segment 0.
bool gemv_can_emit(const slai_qmat *m);
// True when gemv_call takes the 64-row-tile path for this matrix (and so can use `prepared`).
bool gemv_is_rowtile(const slai_ctx *ctx, const slai_qmat *m);
// The same for a SiLU-gated pair launched together (a gated Q8_0 pair needs too many registers there).
bool gemv_gated_is_rowtile(const slai_ctx *ctx, const slai_qmat *gate, const slai_qmat *up);
// Returns SLAI_OK or an error code with the message set on ctx.
// `fused_attn`: also run this attention in the same launch (see launch_qkv_attention; the caller has checked
// qkv_attention_fusable).
struct AttnLaunch;
int gemv_call(slai_ctx *ctx, const GemvCall &c, const char *who, const AttnLaunch *fused_attn = nullptr);
int step_mark(slai_ctx *ctx, const char *name);        // records an event under `name` when step timing is on
bool qkv_attention_fusable(const slai_ctx *ctx, const slai_qmat *v, const slai_qmat *k, const slai_qmat *q, const AttnLaunch &a);
int handoff_reserve(slai_ctx *ctx, uint32_t n_heads);   // not during graph capture
int handoff_check(slai_ctx *ctx);                        // after a synchronize: error if a hand-off ever timed out
// Makes sure the row-tile GEMV's scratch holds `floats` floats (call outside graph capture).
int gemv_scratch_reserve(slai_ctx *ctx, size_t floats);
int sampler_scratch_reserve(slai_ctx *ctx, size_t floats);   // grows the sampler's scratch; not during graph capture

// ---- dequantisation / repack ---------------------------------------------------
// Device-side description of a quantized matrix in either layout.
struct QMatDev {
    int type; int tiled;
    const uint8_t *dptr;
    size_t row_stride; uint32_t nb;                                   // row layout
    uint32_t nrows, ncols, rows_log2, ncb, ngroups, ntiles, unit_bytes;   // tiled layout
};
QMatDev qmat_dev(const slai_qmat *m);
hipError_t launch_repack(hipStream_t s, const slai_qmat *m, const uint8_t *src_gguf_rows);
// rows [row0,row0+nrows) to f32, out[r*out_stride + c]
hipError_t launch_dequant_rows(hipStream_t s, const slai_qmat *m, uint32_t row0, uint32_t nrows, float *out, size_t out_stride);
// out[c] = deq(A[row_a][c]) (+ deq(B[row_b][c]) when B != null); row indices read from device memory
hipError_t launch_embed(hipStream_t s, const slai_qmat *a, const int *row_a, const slai_qmat *b, const int *row_b, uint32_t ncols, float *out);

// ---- element-wise / normalisation ops -------------------------------------------------
struct VecView { float *p; uint32_t n; uint32_t stride; };  // element i at p[i*stride]
// out[i] = id of the XCD workgroup i of a launch of n_workgroups runs on
hipError_t launch_xcd_of_workgroup(hipStream_t s, uint32_t *out, uint32_t n_workgroups);
hipError_t launch_rms_norm(hipStream_t s, VecView out, VecView v, VecView w, const float *eps_ptr, float eps);
hipError_t launch_layernorm(hipStream_t s, VecView out, VecView v, float eps);
hipError_t launch_binop(hipStream_t s, int op /*0 add,1 mul,2 copy(a<-b)*/, VecView a, VecView b);
hipError_t launch_silu(hipStream_t s, VecView a, VecView b);
// out[i] = x[i]*w[i] (i < n), out[n + j] = sum of products 16j..16j+15; n % 16 == 0
hipError_t launch_prepare(hipStream_t s, float *out, const float *x, const float *w, uint32_t n);
hipError_t launch_gelu(hipStream_t s, VecView a);
// GELU over the first ntokens token slots of a quad-major matrix of n floats, in place (split_flag: see launch_silu_parts)
hipError_t launch_gelu_quads(hipStream_t s, float *a, uint32_t n, uint32_t ntokens, int *split_flag = nullptr);
hipError_t launch_rope(hipStream_t s, int variant, const slai_rope_config *cfg_dev, VecView q, VecView k);
hipError_t launch_attn_mask(hipStream_t s, const slai_attn_params *params_dev, float *attn, uint32_t nthreads);
struct View4 { float *p; uint32_t size[4]; uint32_t stride[4]; };
hipError_t launch_softmax_cols(hipStream_t s, View4 m);
hipError_t launch_matmul_f32(hipStream_t s, View4 out, View4 a, View4 b, int a_mode, int b_mode);
// first strict maximum over n floats -> *out_index.  When `decode` is set the kernel also applies the
// forced-token rule and advances the device-side decode state (see DecodeState).
struct DecodeState {      // lives in device memory; the whole greedy loop runs without the host
    int pos;              // position of the token being processed
    int token;            // token fed at `pos`
    int n_prompt;         // prompt length (forced tokens while pos < n_prompt-1)
    int step;             // index into out_tokens
    // sampling (ignored by the greedy kernel): models/sampler.rs `Sampler { temperature, topp }`; the draw for
    // position pos is the top 24 bits of splitmix64(seed + pos), scaled to [0, 1)
    float temperature, topp;
    uint32_t seed_lo, seed_hi;
};
hipError_t launch_argmax(hipStream_t s, const float *v, uint32_t n, int *out_index, DecodeState *decode,
                         const int *prompt, int *out_tokens);
// models/sampler.rs:33-53 `Sampler::sample` with the draw `coin` in [0, 1) given (or, with `decode`, derived from the
// state's seed and position; temperature and topp then come from the state as well)
// `scratch`: sample_scratch_floats(n) floats of device memory
size_t sample_scratch_floats(uint32_t n);
hipError_t launch_sample(hipStream_t s, const float *v, uint32_t n, float temperature, float topp, float coin, float *scratch, int *out_index,
                         DecodeState *decode, const int *prompt, int *out_tokens);

// ---- attention ---------------------------------------------------------------------
struct AttnLaunch {
    const float *q;          // [n_heads*head_size] (pre-RoPE when rope != -1)
    void *kcache, *vcache;   // [seq_len][kv_dim] (position major), f32 or f16
    int kv_f16;
    uint32_t n_heads, kv_mul, head_size, kv_dim, seq_len;
    const uint32_t *pos_ptr; // device; the attended range is [0, *pos_ptr]
    // fused RoPE + cache write of the current position (model path): the fresh k/v columns
    const float *knew, *vnew;  // null: caches already hold position pos and q is already rotated
    const float *qbias, *kbias, *vbias;  // optional (Qwen2), added before RoPE
    int rope_variant; float rope_base;
    const float *rope_theta;   // optional: head_size/2 frequencies base^(-(2i mod hs)/hs), i = pair index (device)
    float *out;              // [n_heads*head_size]
    float *scratch;          // n_heads*n_splits*(head_size+2) floats when n_splits > 1
    uint32_t n_splits;
    // When set (n_splits > 1, fast form only): one zeroed 128-byte line of counters per head.  The workgroup of a head's
    // split that finishes last merges the head's partial results itself and no combine launch follows.  Only for callers
    // who have verified that workgroup i of a launch runs on die i mod 8 (slai_ctx::fuse_qkv_attention): the partial
    // results of a head's splits then meet in that die's L2.
    uint32_t *combine_counters;
};
hipError_t launch_attention(hipStream_t s, const AttnLaunch &a);
// A chunk of `n` consecutive tokens whose keys and values are already in the caches: token b attends from q + b * q_stride
// over positions [0, pos_ptr[b]] into out + b * out_stride (out_quads: into column b of the quad-major matrix `out`,
// n <= 32); knew / vnew must be null.  One workgroup per head and token.
hipError_t launch_attention_batch(hipStream_t s, const AttnLaunch &a, uint32_t n, uint32_t q_stride, uint32_t out_stride, bool out_quads = false,
                                  int *split_flag = nullptr);
// out[b] = embedding row tokens[b] (dequantised), b < n
// (+ row positions[b] of `pos_m` when that is given: learned position embeddings)
hipError_t launch_embed_rows(hipStream_t s, const slai_qmat *m, const int *tokens, uint32_t n, uint32_t ncols, float *out, uint32_t out_stride,
                             const slai_qmat *pos_m = nullptr, const int *positions = nullptr);
// The step before it: for token b (position pos_ptr[b]) add the biases, rotate q + b * q_stride in place and write the
// rotated key k + b * kv_stride and the value v + b * kv_stride to row pos_ptr[b] of the caches.  Uses the q / cache /
// bias / rope fields of `a`.
// q, k, v may come as `nparts` partial results to be added first (q + i * q_part, k / v + i * kv_part, i < nparts); the
// rotated q is written to part 0.
hipError_t launch_rope_store_batch(hipStream_t s, const AttnLaunch &a, float *q, const float *k, const float *v, uint32_t n, uint32_t q_stride, uint32_t kv_stride,
                                   uint32_t nparts = 1, uint32_t q_part = 0, uint32_t kv_part = 0);
// a[i] = silu(sum_s a[i + s * part]) * sum_s b[i + s * part], i < n (silu.slang:11-27 over partial results)
hipError_t launch_silu_parts(hipStream_t s, float *a, const float *b, uint32_t n, uint32_t nparts, uint32_t part, int *split_flag = nullptr, uint32_t ntokens = 32);
// q/k/v GEMV (three segments in the order v, k, q) and the attention over their results in one launch
hipError_t launch_qkv_attention(slai_ctx *ctx, GemvRowtileParams p, const AttnLaunch &a);
// out[i] = powf(base, -((2*i) % head_size) / head_size), i < head_size/2
hipError_t launch_rope_theta(hipStream_t s, float *out, uint32_t head_size, float base);
size_t attention_scratch_floats(uint32_t n_heads, uint32_t head_size, uint32_t n_splits);
// slai_attention's argument checks; fills the launch except for the scratch block (allocates nothing)
int attention_describe(slai_ctx *ctx, const char *fn, const slai_attn_params *params, const slai_buffer *params_gpu, slai_view q, slai_view key_cache,
                       slai_view value_cache, slai_view xb, AttnLaunch *out);
// Looks up, once per device and with that device current, where this device keeps the static scratch array of
// slai_attention_static (called by slai_ctx_create).
hipError_t attention_static_setup(int device);


// ---- the whole layer stack of a Llama-2 token in one resident launch (kernels_decode_persistent.hip) ----------------------
// A matrix, vector or cache as the kernel sees it: address and size in bytes.  Every access of the kernel to it goes
// through a buffer descriptor built from the pair, so the hardware checks it against the size.
struct ResidentBuf { const void *ptr; uint32_t bytes; uint32_t type; };   // type: block format of a weight matrix, else 0
struct PersistentLayer {                 // one per layer, in device memory (16 bytes per entry)
    ResidentBuf wq, wk, wv;              // 64-row tiles; K-quant formats
    ResidentBuf wo;                      // 16-row tiles, Q4_K or Q6_K
    ResidentBuf wgate, wup;              // 64-row tiles, both Q4_K
    ResidentBuf wdown;                   // 16-row tiles, Q4_K or Q6_K
    ResidentBuf attn_norm, ffn_norm;     // dim floats
    ResidentBuf bq, bk, bv;              // optional biases (ptr null: none)
    ResidentBuf kcache, vcache;          // [seq_len][dim]
};
struct PersistentParams {
    const PersistentLayer *layers;
    uint32_t n_layers, dim, hidden, n_heads, seq_len, vocab;
    uint32_t qkv_units, gu_rows;         // the decomposition (resident_plan.h: plan::Shape)
    float eps;
    int rope_variant; float rope_base; const float *rope_theta;
    int kv_f16;
    ResidentBuf wout; ResidentBuf out_norm;     // output matrix (64-row tiles) and the final norm
    const float *x;                      // the embedding row of the token (written by the launch before this one)
    float *logits;
    const uint32_t *pos_ptr;
    // hand-off buffers, filled with FLOW_EMPTY before every launch (layout: resident_plan.h, plan::flow_*): the vectors that
    // cross workgroups, q and the newest k and v among them
    float *flow;
    float *slots;                        // per-workgroup staging of the normalised input of a 64-row-unit phase
    uint32_t *abort_flag;                // set when a reader gave up
    uint64_t *trace;                     // optional: per workgroup 16 * n_layers + 8 time stamps (100 MHz clock); null = none
};
size_t persistent_smem_bytes(const PersistentParams &p);
hipError_t persistent_capacity(const PersistentParams &p, int device, uint32_t *resident);
hipError_t launch_flow_fill(hipStream_t s, void *buf, size_t bytes);
// far: the variant for a position beyond resident_far_from(kv_f16), whose unit workgroups touch the far cache rows into L2
hipError_t launch_decode_persistent(hipStream_t s, const PersistentParams &p, uint32_t grid, bool far);
uint32_t resident_far_from(bool kv_f16);

}  // namespace slai
