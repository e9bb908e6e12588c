// Llama-2 / Qwen2 and GPT-2 model assembly on top of the op facade.
//
// Mirrors crates/slai/src/models/llama2/transformer.rs (`Llama2State` :16-140, `Llama2Weights` :179-297,
// `Llama2::launch` :316-381), models/llama2/cpu.rs (`Llama2Config` :46-143), the per-token driver
// crates/slai-chat/src/chat_llama2.rs:64-240 and, for GPT-2, models/gpt2/cpu.rs:19-48,113-217,224-383.
#include "common.h"
#include "host_gguf.h"
#include "llm_context.h"
#include "quant_formats.h"
#include "resident_plan.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>

namespace slai {
uint32_t pick_attn_splits(const slai_ctx *ctx, uint32_t n_heads, uint32_t seq_len);
int ensure_attn_scratch(slai_ctx *ctx, size_t floats);
hipError_t launch_store_kv(hipStream_t s, const float *src, void *dst, uint32_t n, int f16);
}  // namespace slai

using namespace slai;

#define TRY(call) do { int rc__ = (call); if (rc__) return rc__; } while (0)

namespace {
const uint32_t STORAGE = SLAI_USAGE_STORAGE, UNIFORM = SLAI_USAGE_UNIFORM, COPY_DST = SLAI_USAGE_COPY_DST,
               COPY_SRC = SLAI_USAGE_COPY_SRC, MAP_READ = SLAI_USAGE_MAP_READ;

// `gguf.tensors[name].data().as_f32().unwrap()` + `GpuTensor::vector` (transformer.rs:250-263)
// The kernels index these vectors by the model's widths, so a tensor of any other length is refused here, before
// anything is launched (`expected` elements: the width the readers assume).
int f32_vector_from_gguf(slai_ctx *ctx, const Gguf &g, const std::string &name, bool required, uint32_t expected, GpuTensor *out) {
    const GgufTensorInfo *t = g.find(name);
    if (!t) return required ? set_error(ctx, SLAI_E_MISSING, "missing tensor '" + name + "'") : SLAI_OK;
    if (t->type != 0) return set_error(ctx, SLAI_E_TYPE, "tensor '" + name + "' must be F32");
    uint64_t n = 1;
    for (int d = 0; d < 4; ++d) {
        if (t->dims[d] == 0 || t->dims[d] > UINT32_MAX || (n *= t->dims[d]) > UINT32_MAX) { n = 0; break; }
    }
    if (n != expected)
        return set_error(ctx, SLAI_E_SHAPE, "tensor '" + name + "' has " + std::to_string(n) + " elements, the model needs " + std::to_string(expected));
    return GpuTensor::vector_from(ctx, reinterpret_cast<const float *>(g.bytes + t->offset), (uint32_t)n, STORAGE, out);
}
int qmat_from_gguf(slai_ctx *ctx, const slai_gguf *g, const std::string &name, slai_qmat **out, int layout = SLAI_LAYOUT_AUTO) {
    return slai_gguf_tensor_to_qmat_layout(ctx, g, name.c_str(), layout, out);
}
int meta_u32(slai_ctx *ctx, const Gguf &g, const std::string &key, uint32_t *out) {
    const GgufMetaValue *v = g.meta(key);
    if (!v) return set_error(ctx, SLAI_E_MISSING, "missing metadata key '" + key + "'");
    if (v->type != 4) return set_error(ctx, SLAI_E_TYPE, "unwrap: unexpected GGUF attribute type for '" + key + "'");
    *out = (uint32_t)v->u;
    return SLAI_OK;
}

// Host-only shape checks of a model file, run before anything is uploaded or launched: the kernels index weights and
// vectors by the model's widths, so a tensor of any other shape must never reach them.  `err` receives the message.
int check_matrix(const Gguf &g, const std::string &name, bool required, uint64_t nrows, uint64_t ncols, std::string &err) {
    const GgufTensorInfo *t = g.find(name);
    if (!t) { if (!required) return SLAI_OK; err = "missing tensor '" + name + "'"; return SLAI_E_MISSING; }
    const int be = block_elems((int)t->type);
    if (!be) { err = "tensor '" + name + "' has ggml type " + std::to_string(t->type) + " which has no device kernel"; return SLAI_E_TYPE; }
    if (t->dims[2] != 1 || t->dims[3] != 1 || t->dims[0] != nrows || t->dims[1] != ncols) {
        err = "tensor '" + name + "' is " + std::to_string(t->dims[0]) + " x " + std::to_string(t->dims[1]) + ", the model needs " + std::to_string(nrows) + " x " + std::to_string(ncols);
        return SLAI_E_SHAPE;
    }
    if (ncols % be) { err = "tensor '" + name + "': row length is not a multiple of the block length"; return SLAI_E_SHAPE; }
    if (t->offset > g.len || gguf_row_bytes((int)t->type, (uint32_t)ncols) * nrows > g.len - t->offset) { err = "tensor '" + name + "' runs past the end of the file"; return SLAI_E_PARSE; }
    return SLAI_OK;
}
int check_vector(const Gguf &g, const std::string &name, bool required, uint64_t n, std::string &err) {
    const GgufTensorInfo *t = g.find(name);
    if (!t) { if (!required) return SLAI_OK; err = "missing tensor '" + name + "'"; return SLAI_E_MISSING; }
    if (t->type != 0) { err = "tensor '" + name + "' must be F32"; return SLAI_E_TYPE; }
    uint64_t have = 1;
    for (int d = 0; d < 4; ++d) {
        if (t->dims[d] == 0 || t->dims[d] > UINT32_MAX || (have *= t->dims[d]) > UINT32_MAX) { have = 0; break; }
    }
    if (have != n) { err = "tensor '" + name + "' has " + std::to_string(have) + " elements, the model needs " + std::to_string(n); return SLAI_E_SHAPE; }
    if (t->offset > g.len || n * 4 > g.len - t->offset) { err = "tensor '" + name + "' runs past the end of the file"; return SLAI_E_PARSE; }
    return SLAI_OK;
}

// Two matrices over the same input can share a GEMV launch: any formats in 64-row tiles, otherwise one format and layout.
bool same_launch(const slai_qmat *a, const slai_qmat *b) {
    if (a->tiled && b->tiled && a->rows_log2 == 6 && b->rows_log2 == 6 && (a->type == b->type || (a->type != T_Q8_0 && b->type != T_Q8_0 && a->type != T_Q4_0 && b->type != T_Q4_0)))
        return true;
    return a->type == b->type && a->tiled == b->tiled && (!a->tiled || a->rows_log2 == b->rows_log2);
}

struct DeviceLoop {           // device-resident state of the greedy loop
    slai_buffer *state = nullptr;       // DecodeState
    slai_buffer *prompt = nullptr;      // int32[capacity]
    slai_buffer *out_tokens = nullptr;  // int32[capacity]
    uint32_t capacity = 0;
    slai_graph *graph[3][2] = {{nullptr, nullptr}, {nullptr, nullptr}, {nullptr, nullptr}};   // one token, [launch form][greedy pick | temperature / top-p pick]
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
};
int loop_init(slai_ctx *ctx, DeviceLoop &L, uint32_t capacity) {
    L.capacity = capacity;
    TRY(slai_buffer_create(ctx, sizeof(DecodeState), SLAI_DT_I32, STORAGE | COPY_DST, &L.state));
    TRY(slai_buffer_create(ctx, (size_t)capacity * 4, SLAI_DT_I32, STORAGE | COPY_DST, &L.prompt));
    TRY(slai_buffer_create(ctx, (size_t)capacity * 4, SLAI_DT_I32, STORAGE | COPY_SRC, &L.out_tokens));
    SLAI_HIP_TRY(ctx, hipEventCreate(&L.ev0));
    SLAI_HIP_TRY(ctx, hipEventCreate(&L.ev1));
    return SLAI_OK;
}
void loop_destroy(slai_ctx *ctx, DeviceLoop &L) {
    for (auto &form : L.graph)
        for (slai_graph *g : form)
            if (g) slai_graph_destroy(ctx, g);
    if (L.state) slai_buffer_destroy(ctx, L.state);
    if (L.prompt) slai_buffer_destroy(ctx, L.prompt);
    if (L.out_tokens) slai_buffer_destroy(ctx, L.out_tokens);
    if (L.ev0) (void)hipEventDestroy(L.ev0);
    if (L.ev1) (void)hipEventDestroy(L.ev1);
}
}  // namespace

// =================================================================================================
// Llama-2
// =================================================================================================
struct Llama2LayerWeights {          // transformer.rs:179-192
    GpuTensor attn_norm;
    slai_qmat *attn_k = nullptr, *attn_q = nullptr, *attn_v = nullptr;
    GpuTensor attn_k_bias, attn_q_bias, attn_v_bias;   // optional
    slai_qmat *ffn_down = nullptr, *ffn_gate = nullptr;
    GpuTensor ffn_norm;
    slai_qmat *ffn_up = nullptr, *attn_output = nullptr;
};
struct Llama2Weights {               // transformer.rs:194-199
    std::vector<Llama2LayerWeights> layers;
    slai_qmat *token_embd = nullptr;   // kept packed; one row is dequantised on the device per token
    slai_qmat *output = nullptr;       // aliases token_embd when the file has no output.weight
    GpuTensor output_norm;
};
struct Llama2State {                 // transformer.rs:16-44
    GpuTensor x, xb, xb2, hb, hb2, q, att, logits;
    GpuTensor kcol, vcol;            // fresh K/V of the current position (fused path, and staging for f16 caches)
    GpuTensor rope_theta;            // fused path: head_size/2 RoPE frequencies
    GpuTensor xw;                    // fused path: norm-weighted copy of x (+ dim/16 sums of 16) left by the producer of x
    std::vector<GpuTensor> key_cache, value_cache;
    slai_buffer *rope_config = nullptr, *rms_norm_config = nullptr, *attn_params = nullptr;
};

// Activations of a chunk of prompt tokens that go through the layers together (one row per token), and the
// positions 0, 1, 2, ... as device words (token b of a chunk at pos0 reads its position from positions + pos0 + b).
struct PromptChunkState {
    uint32_t rows = 0;
    GpuTensor x, xw, xb, q, k, v, hb;
    GpuTensor xn, hb2;                 // matrix-core path: normalised activations, the up projection
    slai_buffer *positions = nullptr;
    slai_buffer *tokens = nullptr;     // int32[seq_len]
};

struct slai_llama2 {
    slai_ctx *ctx = nullptr;
    int model_type = SLAI_MODEL_LLAMA;
    int kv_dtype = SLAI_KV_F32;
    slai_llama2_config config{};
    Llama2Weights weights;
    Llama2State state;
    DeviceLoop loop;
    size_t weight_bytes = 0;
    uint32_t attn_splits = 1;

    uint32_t kv_dim() const { return config.dim * config.n_kv_heads / config.n_q_heads; }
    uint32_t head_size() const { return config.dim / config.n_q_heads; }
    int rope_variant() const { return model_type == SLAI_MODEL_QWEN2 ? SLAI_ROPE_NEOX : SLAI_ROPE_ORIGINAL; }  // llama2/mod.rs:27-32

    int load(const slai_gguf *g);
    int launch(LlmContext &ctxt, const slai_attn_params &attn_params, uint32_t pos);   // transformer.rs:316-381
    int enqueue_fused(int sampler, int form = 0);   // sampler 0: stop at the logits, 1: greedy pick + loop state, 2: temperature / top-p pick + loop state; form 1: the resident launch
    int form_at(uint32_t pos) const;               // the launch form of the token at `pos`

    // The layer stack as ONE resident launch per token (kernels_decode_persistent.hip), for the models it covers.
    struct {
        bool ready = false;
        mutable const char *why_not = nullptr;   // set when the context asked for the form and the model does not take it
        uint32_t grid = 0;
        PersistentParams params{};
        slai_buffer *layers = nullptr, *flow = nullptr, *slots = nullptr;
        size_t flow_bytes = 0;
    } persistent;
    bool persistent_supported() const;
    int persistent_setup();
    int enqueue_persistent(int sampler, bool far);

    // Prompt tokens in chunks: every weight matrix is read once per chunk instead of once per token.
    PromptChunkState chunk;
    bool chunk_supported() const;        // per-token workgroups over shared weights (any tiled format)
    bool chunk_gemm_supported() const;   // matrix cores (K-quants)
    int chunk_reserve(uint32_t rows);
    int enqueue_chunk(uint32_t pos0, uint32_t n, const int *tokens_dev);   // fills the caches for positions pos0 .. pos0 + n - 1
    bool chunk_split_ok() const;         // every layer matrix small enough for the f16 head + remainder form (256 * |w| within f16)
    uint32_t prefill_fp32_repeats = 0;   // prefill calls repeated in fp32 because an activation was beyond the f16 range
    int enqueue_chunk_gemm(uint32_t pos0, uint32_t n, const int *tokens_dev, bool split_f16);   // the same on the matrix cores, n <= 32
    // q / k / v given as nparts partial sums, 32 rows apart; out_quads: the result goes to xn, quad-major, instead of xb
    int chunk_attention(uint32_t l, uint32_t pos0, uint32_t n, uint32_t nparts = 1, bool out_quads = false, int *split_flag = nullptr);
};

// models/llama2/cpu.rs:79-109
static int llama2_config_from_gguf(slai_ctx *ctx, const Gguf &g, int model_type, slai_llama2_config *c) {
    const std::string m = model_type == SLAI_MODEL_QWEN2 ? "qwen2" : "llama";   // llama2/mod.rs:19-25
    TRY(meta_u32(ctx, g, m + ".embedding_length", &c->dim));
    TRY(meta_u32(ctx, g, m + ".feed_forward_length", &c->hidden_dim));
    TRY(meta_u32(ctx, g, m + ".block_count", &c->n_layers));
    TRY(meta_u32(ctx, g, m + ".attention.head_count", &c->n_q_heads));
    TRY(meta_u32(ctx, g, m + ".attention.head_count_kv", &c->n_kv_heads));
    TRY(meta_u32(ctx, g, m + ".context_length", &c->seq_len));
    const GgufMetaValue *tok = g.meta("tokenizer.ggml.tokens");
    if (!tok) return set_error(ctx, SLAI_E_MISSING, "missing metadata key 'tokenizer.ggml.tokens'");
    if (tok->type != 9) return set_error(ctx, SLAI_E_TYPE, "unwrap: unexpected GGUF attribute type for 'tokenizer.ggml.tokens'");
    c->vocab_size = (uint32_t)tok->arr_len;
    const GgufMetaValue *fb = g.meta(m + ".rope.freq_base");
    if (fb && fb->type != 6) return set_error(ctx, SLAI_E_TYPE, "unwrap: unexpected GGUF attribute type for rope.freq_base");
    c->rope_base_freq = fb ? (float)fb->f : 10000.0f;
    const GgufMetaValue *ep = g.meta(m + ".attention.layer_norm_rms_epsilon");
    if (ep && ep->type != 6) return set_error(ctx, SLAI_E_TYPE, "unwrap: unexpected GGUF attribute type for layer_norm_rms_epsilon");
    c->rms_norm_eps = ep ? (float)ep->f : 1.0e-6f;
    if (!c->dim || !c->n_q_heads || !c->n_kv_heads || c->dim % c->n_q_heads || c->n_q_heads % c->n_kv_heads || !c->seq_len || !c->vocab_size)
        return set_error(ctx, SLAI_E_SHAPE, "inconsistent model hyper-parameters");
    return SLAI_OK;
}

// Everything `load` is going to read, checked on the host alone: hyper-parameters, then the presence, block format and
// shape of every tensor (`Llama2Weights::from_gguf`, transformer.rs:202-297, unwraps and asserts where this returns a code).
static int llama2_check_gguf(const Gguf &g, int model_type, slai_llama2_config *cfg, std::string &err) {
    slai_ctx scratch_ctx;                                  // (only carries the message of the config reader)
    if (int rc = llama2_config_from_gguf(&scratch_ctx, g, model_type, cfg)) { err = scratch_ctx.err; return rc; }
    const slai_llama2_config &c = *cfg;
    const uint64_t dim = c.dim, kvd = (uint64_t)c.dim * c.n_kv_heads / c.n_q_heads, hid = c.hidden_dim, hs = c.dim / c.n_q_heads;
    if (hs % 2 || hs > 256) { err = "head size must be even and <= 256"; return SLAI_E_SHAPE; }
    if (!hid || !c.n_layers) { err = "inconsistent model hyper-parameters"; return SLAI_E_SHAPE; }
    for (uint32_t l = 0; l < c.n_layers; ++l) {
        const std::string p = "blk." + std::to_string(l) + ".";
        const struct { const char *name; bool required; uint64_t r, k; } mats[] = {
            {"attn_q.weight", true, dim, dim}, {"attn_k.weight", true, kvd, dim}, {"attn_v.weight", true, kvd, dim}, {"attn_output.weight", true, dim, dim},
            {"ffn_down.weight", true, dim, hid}, {"ffn_gate.weight", true, hid, dim}, {"ffn_up.weight", true, hid, dim}};
        for (const auto &m : mats)
            if (int rc = check_matrix(g, p + m.name, m.required, m.r, m.k, err)) return rc;
        const struct { const char *name; bool required; uint64_t n; } vecs[] = {
            {"attn_q.bias", false, dim}, {"attn_k.bias", false, kvd}, {"attn_v.bias", false, kvd}, {"ffn_norm.weight", true, dim}, {"attn_norm.weight", true, dim}};
        for (const auto &v : vecs)
            if (int rc = check_vector(g, p + v.name, v.required, v.n, err)) return rc;
    }
    if (int rc = check_matrix(g, "token_embd.weight", true, c.vocab_size, dim, err)) return rc;
    if (int rc = check_matrix(g, "output.weight", false, c.vocab_size, dim, err)) return rc;
    return check_vector(g, "output_norm.weight", true, dim, err);
}

static int copy_message(int rc, const std::string &msg, char *err, size_t err_len) {
    if (err && err_len) { const size_t n = std::min(msg.size(), err_len - 1); memcpy(err, msg.data(), n); err[n] = 0; }
    return rc;
}

SLAI_EXPORT int slai_llama2_check_gguf(const slai_gguf *g, int model_type, char *err, size_t err_len) {
    if (!g || (model_type != SLAI_MODEL_LLAMA && model_type != SLAI_MODEL_QWEN2)) return copy_message(SLAI_E_ARG, "slai_llama2_check_gguf: bad argument", err, err_len);
    slai_llama2_config cfg{};
    std::string msg;
    const int rc = llama2_check_gguf(g->g, model_type, &cfg, msg);
    return copy_message(rc, msg, err, err_len);
}

int slai_llama2::load(const slai_gguf *gg) {
    const Gguf &g = gg->g;
    {   // nothing is uploaded or launched for a file whose tensors do not fit the hyper-parameters
        std::string msg;
        if (int rc = llama2_check_gguf(g, model_type, &config, msg)) return set_error(ctx, rc, msg);
    }
    const uint32_t dim = config.dim, kvd = kv_dim();
    if (head_size() % 2 || head_size() > 256) return set_error(ctx, SLAI_E_SHAPE, "head size must be even and <= 256");
    // ---- Llama2Weights::from_gguf (transformer.rs:202-297)
    weights.layers.resize(config.n_layers);
    for (uint32_t l = 0; l < config.n_layers; ++l) {
        Llama2LayerWeights &w = weights.layers[l];
        const std::string p = "blk." + std::to_string(l) + ".";
        TRY(qmat_from_gguf(ctx, gg, p + "attn_q.weight", &w.attn_q, SLAI_LAYOUT_TILE64));
        TRY(qmat_from_gguf(ctx, gg, p + "attn_k.weight", &w.attn_k, SLAI_LAYOUT_TILE64));
        TRY(qmat_from_gguf(ctx, gg, p + "attn_v.weight", &w.attn_v, SLAI_LAYOUT_TILE64));
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_q.bias", false, dim, &w.attn_q_bias));
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_k.bias", false, kvd, &w.attn_k_bias));
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_v.bias", false, kvd, &w.attn_v_bias));
        TRY(qmat_from_gguf(ctx, gg, p + "attn_output.weight", &w.attn_output));
        // (explicit 16-row tiles: a feed-forward width beyond 16384 then still gets the tiled layout, in column slices)
        TRY(qmat_from_gguf(ctx, gg, p + "ffn_down.weight", &w.ffn_down, SLAI_LAYOUT_TILE16));
        TRY(qmat_from_gguf(ctx, gg, p + "ffn_gate.weight", &w.ffn_gate, SLAI_LAYOUT_TILE64));
        TRY(qmat_from_gguf(ctx, gg, p + "ffn_up.weight", &w.ffn_up, SLAI_LAYOUT_TILE64));
        TRY(f32_vector_from_gguf(ctx, g, p + "ffn_norm.weight", true, dim, &w.ffn_norm));
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_norm.weight", true, dim, &w.attn_norm));
        struct { slai_qmat *m; uint32_t r, c; } chk[] = {{w.attn_q, dim, dim}, {w.attn_k, kvd, dim}, {w.attn_v, kvd, dim},
            {w.attn_output, dim, dim}, {w.ffn_down, dim, config.hidden_dim}, {w.ffn_gate, config.hidden_dim, dim}, {w.ffn_up, config.hidden_dim, dim}};
        for (auto &c : chk)
            if (c.m->nrows != c.r || c.m->ncols != c.c) return set_error(ctx, SLAI_E_SHAPE, "layer " + std::to_string(l) + ": weight shape does not match the config");
        for (slai_qmat *m : {w.attn_q, w.attn_k, w.attn_v, w.attn_output, w.ffn_down, w.ffn_gate, w.ffn_up}) weight_bytes += m->bytes;
        weight_bytes += 2 * (size_t)dim * 4;
    }
    TRY(qmat_from_gguf(ctx, gg, "token_embd.weight", &weights.token_embd, SLAI_LAYOUT_TILE64));
    if (g.find("output.weight")) TRY(qmat_from_gguf(ctx, gg, "output.weight", &weights.output, SLAI_LAYOUT_TILE64));
    else weights.output = weights.token_embd;                                       // transformer.rs:279-285
    TRY(f32_vector_from_gguf(ctx, g, "output_norm.weight", true, dim, &weights.output_norm));
    if (weights.token_embd->nrows != config.vocab_size || weights.token_embd->ncols != dim || weights.output->nrows != config.vocab_size ||
        weights.output->ncols != dim)
        return set_error(ctx, SLAI_E_SHAPE, "embedding / output shape does not match the config");
    weight_bytes += weights.output->bytes + (size_t)dim * 4;

    {   // activation slots of the 64-row-tile GEMV: the largest launch is q/k/v together, gate/up, or the output matrix
        const uint32_t t64 = std::max(std::max((dim + 63) / 64 + 2 * ((kvd + 63) / 64), (config.hidden_dim + 63) / 64), (config.vocab_size + 63) / 64);
        TRY(gemv_scratch_reserve(ctx, (size_t)t64 * (dim + dim / 16 + 16)));
        TRY(handoff_reserve(ctx, config.n_q_heads));
    }
    // ---- Llama2State::new (transformer.rs:47-140); buffers are zero-initialised
    Llama2State &s = state;
    TRY(GpuTensor::vector(ctx, dim, STORAGE | COPY_DST | COPY_SRC, &s.x));
    TRY(GpuTensor::vector(ctx, dim, STORAGE | COPY_SRC, &s.xb));
    TRY(GpuTensor::vector(ctx, dim, STORAGE, &s.xb2));
    TRY(GpuTensor::vector(ctx, config.hidden_dim, STORAGE, &s.hb));
    TRY(GpuTensor::vector(ctx, config.hidden_dim, STORAGE, &s.hb2));
    TRY(GpuTensor::vector(ctx, dim, STORAGE | COPY_SRC, &s.q));
    TRY(GpuTensor::vector(ctx, kvd, STORAGE, &s.kcol));
    TRY(GpuTensor::vector(ctx, dim + dim / 16 + 16, STORAGE, &s.xw));
    TRY(GpuTensor::vector(ctx, head_size() / 2, STORAGE, &s.rope_theta));
    SLAI_HIP_TRY(ctx, launch_rope_theta(ctx->stream, (float *)s.rope_theta.buf->dptr, head_size(), config.rope_base_freq));
    TRY(GpuTensor::vector(ctx, kvd, STORAGE, &s.vcol));
    const int cdt = kv_dtype == SLAI_KV_F16 ? SLAI_DT_F16 : SLAI_DT_F32;
    s.key_cache.resize(config.n_layers); s.value_cache.resize(config.n_layers);
    for (uint32_t l = 0; l < config.n_layers; ++l) {
        TRY(GpuTensor::matrix(ctx, kvd, config.seq_len, STORAGE, &s.key_cache[l], cdt));
        TRY(GpuTensor::matrix(ctx, kvd, config.seq_len, STORAGE, &s.value_cache[l], cdt));
    }
    TRY(GpuTensor::matrix(ctx, config.seq_len, config.n_q_heads, STORAGE, &s.att));
    TRY(GpuTensor::vector(ctx, config.vocab_size, STORAGE | COPY_SRC | MAP_READ, &s.logits));
    TRY(slai_buffer_create(ctx, sizeof(slai_rope_config), SLAI_DT_U8, UNIFORM | COPY_DST, &s.rope_config));
    TRY(slai_buffer_create(ctx, sizeof(slai_rms_norm_config), SLAI_DT_U8, UNIFORM | COPY_DST, &s.rms_norm_config));
    TRY(slai_buffer_create(ctx, sizeof(slai_attn_params), SLAI_DT_U8, UNIFORM | COPY_DST, &s.attn_params));

    attn_splits = pick_attn_splits(ctx, config.n_q_heads, config.seq_len);
    TRY(ensure_attn_scratch(ctx, attention_scratch_floats(config.n_q_heads, head_size(), attn_splits)));
    TRY(loop_init(ctx, loop, config.seq_len + 1));
    TRY(persistent_setup());
    // (said only to a caller who asked for the form by name: most models simply have other shapes)
    const char *asked = getenv("SLAI_PERSISTENT");
    if (asked && ctx->persistent && !persistent.ready)
        fprintf(stderr, "slai: SLAI_PERSISTENT=%s, but this model keeps one launch per step: %s\n", asked, persistent.why_not ? persistent.why_not : "unknown");
    return slai_synchronize(ctx);
}

// The resident launch covers the shapes of the headline configuration and its smaller relatives: as many cache heads as
// query heads of size 128, a width of 1024 .. 4096 in steps of 1024, q / k / v, gate / up and the output matrix in 64-row
// tiles of K-quants (gate and up both Q4_K), the two projections into the residual in 16-row tiles of Q4_K or Q6_K.
// Everything else keeps the launch-per-step form, and so do the tokens of these models beyond the position up to which
// one workgroup per head walks the cache fast enough (form_at).
bool slai_llama2::persistent_supported() const {
    const uint32_t dim = config.dim, hid = config.hidden_dim, nh = config.n_q_heads;
    if (!ctx->persistent) return false;
    const auto no = [&](const char *why) { persistent.why_not = why; return false; };
    if (!ctx->fuse_qkv_attention) return no("workgroups are not placed on the dies round robin (or SLAI_FUSE_QKV_ATTN=0)");
    if (!ctx->rowtile_gemv || !ctx->handoff_counters || nh > ctx->handoff_heads) return no("64-row tiles or the hand-off counters are switched off");
    if (config.n_kv_heads != nh || head_size() != 128 || nh % 8 || dim % 1024 || dim > 4096 || hid % 256 || hid / 256 > 64)
        return no("shape: needs as many cache heads as query heads of size 128 (a multiple of 8), a width of 1024 .. 4096, an FFN width in super-blocks");
    const auto kquant = [](int t) { return t == T_Q4_K || t == T_Q5_K || t == T_Q6_K; };
    const auto proj = [&](const slai_qmat *m, uint32_t cols) {
        return m->tiled && m->rows_log2 == 4 && (m->type == T_Q4_K || m->type == T_Q6_K) && m->ncb == cols / 256 && m->ngroups == (cols / 256 + 3) / 4 && m->ngroups <= 16;
    };
    for (const Llama2LayerWeights &w : weights.layers) {
        for (const slai_qmat *m : {w.attn_q, w.attn_k, w.attn_v})
            if (!gemv_is_rowtile(ctx, m) || !kquant(m->type) || m->ncb != dim / 256) return no("q / k / v are not K-quants in 64-row tiles");
        if (!gemv_is_rowtile(ctx, w.ffn_gate) || !gemv_is_rowtile(ctx, w.ffn_up) || w.ffn_gate->type != T_Q4_K || w.ffn_up->type != T_Q4_K)
            return no("gate / up are not Q4_K in 64-row tiles");
        if (!proj(w.attn_output, dim) || !proj(w.ffn_down, hid)) return no("the projections into the residual are not Q4_K / Q6_K in 16-row tiles");
    }
    if (!(gemv_is_rowtile(ctx, weights.output) && kquant(weights.output->type) && weights.output->ncb == dim / 256)) return no("the output matrix is not a K-quant in 64-row tiles");
    return true;
}

// Leaves persistent.ready set when the model takes the resident launch; otherwise persistent.why_not says why not (when
// the context asked for the form at all).
int slai_llama2::persistent_setup() {
    if (!persistent_supported()) return SLAI_OK;
    const auto no = [&](const char *why) { persistent.why_not = why; return SLAI_OK; };
    const uint32_t dim = config.dim, hid = config.hidden_dim, nh = config.n_q_heads, nl = config.n_layers;
    PersistentParams &p = persistent.params;
    p.n_layers = nl; p.dim = dim; p.hidden = hid; p.n_heads = nh; p.seq_len = config.seq_len; p.vocab = config.vocab_size;
    p.eps = config.rms_norm_eps; p.rope_variant = rope_variant(); p.rope_base = config.rope_base_freq;
    p.rope_theta = (const float *)state.rope_theta.buf->dptr;
    p.kv_f16 = kv_dtype == SLAI_KV_F16;
    // every matrix, vector and cache goes to the kernel with its size: the kernel reads them through buffer descriptors
    bool fits = true;
    const auto mat = [&](const slai_qmat *m) { if (m->bytes > 0xffffffffull) fits = false; return ResidentBuf{m->dptr, (uint32_t)m->bytes, (uint32_t)m->type}; };
    const auto vec = [&](const GpuTensor &t) { return t.buf ? ResidentBuf{t.buf->dptr, (uint32_t)t.buf->bytes, 0u} : ResidentBuf{nullptr, 0u, 0u}; };
    p.wout = mat(weights.output); p.out_norm = vec(weights.output_norm);
    p.x = (const float *)state.x.buf->dptr; p.logits = (float *)state.logits.buf->dptr;
    p.pos_ptr = (const uint32_t *)&((DecodeState *)loop.state->dptr)->pos;
    p.abort_flag = ctx->handoff_counters + (size_t)ctx->handoff_heads * 32;
    // the device must keep the whole grid resident: every compute unit one workgroup, and enough of them for every role
    uint32_t resident = 0;
    p.qkv_units = 6; p.gu_rows = 64;                                  // (the occupancy query only needs the widths)
    if (persistent_capacity(p, ctx->device, &resident) != hipSuccess) return no("the occupancy query for the kernel failed");
    hipDeviceProp_t prop;
    SLAI_HIP_TRY(ctx, hipGetDeviceProperties(&prop, ctx->device));
    const plan::Shape sh = plan::make_shape(dim, hid, nh, nl, config.vocab_size, config.seq_len, rope_variant() == SLAI_ROPE_NEOX ? 1u : 0u);
    const uint32_t grid = sh.grid;                                    // one workgroup per compute unit at most, all resident
    if (grid > std::min(resident, (uint32_t)prop.multiProcessorCount)) return no("the device keeps too few workgroups of the kernel resident for this shape");
    if (!plan::shape_ok(sh)) return no("shape: the FFN width does not spread evenly over one workgroup per 16 rows of the model width");
    p.qkv_units = sh.qkv_units; p.gu_rows = sh.gu_rows;
    std::vector<PersistentLayer> host(nl);
    for (uint32_t l = 0; l < nl; ++l) {
        const Llama2LayerWeights &w = weights.layers[l];
        PersistentLayer &d = host[l];
        d.wq = mat(w.attn_q); d.wk = mat(w.attn_k); d.wv = mat(w.attn_v); d.wo = mat(w.attn_output);
        d.wgate = mat(w.ffn_gate); d.wup = mat(w.ffn_up); d.wdown = mat(w.ffn_down);
        d.attn_norm = vec(w.attn_norm); d.ffn_norm = vec(w.ffn_norm);
        d.bq = vec(w.attn_q_bias); d.bk = vec(w.attn_k_bias); d.bv = vec(w.attn_v_bias);
        d.kcache = vec(state.key_cache[l]); d.vcache = vec(state.value_cache[l]);
    }
    if (!fits) return no("a matrix beyond 4 GiB");
    TRY(slai_buffer_create(ctx, host.size() * sizeof(PersistentLayer), SLAI_DT_U8, STORAGE | COPY_DST, &persistent.layers));
    TRY(slai_write_buffer(ctx, persistent.layers, 0, host.data(), host.size() * sizeof(PersistentLayer)));
    persistent.flow_bytes = (size_t)plan::flow_floats(sh) * sizeof(float);
    TRY(slai_buffer_create(ctx, persistent.flow_bytes, SLAI_DT_F32, STORAGE, &persistent.flow));
    TRY(slai_buffer_create(ctx, (size_t)plan::slot_floats(sh) * sizeof(float), SLAI_DT_F32, STORAGE, &persistent.slots));
    p.layers = (const PersistentLayer *)persistent.layers->dptr;
    p.flow = (float *)persistent.flow->dptr;
    p.slots = (float *)persistent.slots->dptr;
    persistent.grid = grid;
    persistent.ready = true;
    return SLAI_OK;
}

// embedding row | hand-off buffers emptied | the layer stack and the output matrix | pick
int slai_llama2::enqueue_persistent(int sampler, bool far) {
    Llama2State &s = state;
    DecodeState *ds = (DecodeState *)loop.state->dptr;
    SLAI_HIP_TRY(ctx, launch_embed(ctx->stream, weights.token_embd, &ds->token, nullptr, nullptr, config.dim, (float *)s.x.buf->dptr));
    TRY(step_mark(ctx, "embedding row"));
    SLAI_HIP_TRY(ctx, launch_flow_fill(ctx->stream, persistent.flow->dptr, persistent.flow_bytes));
    TRY(step_mark(ctx, "hand-off buffers emptied"));
    SLAI_HIP_TRY(ctx, launch_decode_persistent(ctx->stream, persistent.params, persistent.grid, far));
    TRY(step_mark(ctx, "llama2 resident token"));
    if (sampler == 1)
        SLAI_HIP_TRY(ctx, launch_argmax(ctx->stream, (const float *)s.logits.buf->dptr, config.vocab_size, nullptr, ds,
                                        (const int *)loop.prompt->dptr, (int *)loop.out_tokens->dptr));
    else if (sampler == 2)
        SLAI_HIP_TRY(ctx, launch_sample(ctx->stream, (const float *)s.logits.buf->dptr, config.vocab_size, 0.0f, 0.0f, 0.0f, ctx->sampler_scratch, nullptr, ds,
                                        (const int *)loop.prompt->dptr, (int *)loop.out_tokens->dptr));
    return SLAI_OK;
}

// `Llama2::launch` (transformer.rs:316-381), one kernel per op in the reference's order.
int slai_llama2::launch(LlmContext &ctxt, const slai_attn_params &attn_params, uint32_t pos) {
    Llama2State &s = state;
    const bool f16 = kv_dtype == SLAI_KV_F16;
    for (uint32_t l = 0; l < config.n_layers; ++l) {
        const Llama2LayerWeights &wl = weights.layers[l];
        TRY(ctxt.rms_norm_assign(s.rms_norm_config, s.xb.view(), s.x.view(), wl.attn_norm.view()));             // :327
        // :329-334 -- the GEMVs write straight into the cache column; an f16 cache goes through kcol/vcol
        slai_view k_cache = f16 ? s.kcol.view() : s.key_cache[l].column(pos);
        slai_view v_cache = f16 ? s.vcol.view() : s.value_cache[l].column(pos);
        TRY(ctxt.matmul_quant_assign(s.q.view(), wl.attn_q, s.xb.view()));
        TRY(ctxt.matmul_quant_assign(k_cache, wl.attn_k, s.xb.view()));
        TRY(ctxt.matmul_quant_assign(v_cache, wl.attn_v, s.xb.view()));
        if (wl.attn_q_bias.buf) TRY(ctxt.add_assign(s.q.view(), wl.attn_q_bias.view()));                        // :336-344
        if (wl.attn_k_bias.buf) TRY(ctxt.add_assign(k_cache, wl.attn_k_bias.view()));
        if (wl.attn_v_bias.buf) TRY(ctxt.add_assign(v_cache, wl.attn_v_bias.view()));
        TRY(ctxt.rope(rope_variant(), s.rope_config, s.q.view(), k_cache));                                      // :346-347
        if (f16) {
            const size_t off = (size_t)pos * kv_dim() * 2;
            SLAI_HIP_TRY(ctx, launch_store_kv(ctx->stream, (const float *)s.kcol.buf->dptr, (char *)s.key_cache[l].buf->dptr + off, kv_dim(), 1));
            SLAI_HIP_TRY(ctx, launch_store_kv(ctx->stream, (const float *)s.vcol.buf->dptr, (char *)s.value_cache[l].buf->dptr + off, kv_dim(), 1));
        }
        TRY(slai_attention(ctx, &attn_params, s.attn_params, s.q.view(), s.key_cache[l].view(), s.value_cache[l].view(),
                           s.att.view(), s.xb.view()));                                                          // :350, :383-400
        TRY(ctxt.matmul_quant_assign(s.xb2.view(), wl.attn_output, s.xb.view()));                                // :352
        TRY(ctxt.add_assign(s.x.view(), s.xb2.view()));                                                          // :355
        TRY(ctxt.rms_norm_assign(s.rms_norm_config, s.xb.view(), s.x.view(), wl.ffn_norm.view()));               // :356
        TRY(ctxt.matmul_quant_assign(s.hb.view(), wl.ffn_gate, s.xb.view()));                                    // :359
        TRY(ctxt.matmul_quant_assign(s.hb2.view(), wl.ffn_up, s.xb.view()));                                     // :360
        TRY(ctxt.silu(s.hb.view(), s.hb2.view()));                                                               // :361
        TRY(ctxt.matmul_quant_assign(s.xb2.view(), wl.ffn_down, s.hb.view()));                                   // :362
        TRY(ctxt.add_assign(s.x.view(), s.xb2.view()));                                                          // :365
    }
    TRY(ctxt.rms_norm_assign(s.rms_norm_config, s.xb.view(), s.x.view(), weights.output_norm.view()));           // :368-373
    TRY(ctxt.matmul_quant_assign(s.logits.view(), weights.output, s.xb.view()));                                 // :375
    return SLAI_OK;
}

// The same computation as `launch`, as fused kernels whose per-token scalars (position, token) live
// in device memory, so the sequence can be captured once and replayed for every token:
//   embedding-row gather | per layer: [RMSNorm+QKV GEMV] [RoPE+cache write+attention] [Wo GEMV+residual]
//   [RMSNorm+gate/up GEMV+SiLU] [down GEMV+residual] | [RMSNorm+logits GEMV] [argmax + loop state]
// The resident launch walks a head's cached positions with one workgroup, at the rate one compute unit reads memory;
// the launch-per-step form spreads them over the device.  Up to ctx->resident_max_pos positions the resident launch is
// the faster one, beyond it the steps are: the form is chosen per token (both keep the same caches and loop state).
// (Forms: 0 one launch per step, 1 the resident launch, 2 the resident launch whose unit workgroups also bring the cache
// rows beyond the ones the attention asks for ahead into the die's L2 -- a kernel of its own, so that the short contexts do
// not carry that code.)
int slai_llama2::form_at(uint32_t pos) const {
    if (!persistent.ready || pos >= ctx->resident_max_pos) return 0;
    return pos > resident_far_from(kv_dtype == SLAI_KV_F16) ? 2 : 1;
}

int slai_llama2::enqueue_fused(int sampler, int form) {
    if (form != 0) return persistent.ready ? enqueue_persistent(sampler, form == 2) : set_error(ctx, SLAI_E_STATE, "this model does not take the resident launch");
    Llama2State &s = state;
    DecodeState *ds = (DecodeState *)loop.state->dptr;
    float *x = (float *)s.x.buf->dptr, *xb = (float *)s.xb.buf->dptr, *hb = (float *)s.hb.buf->dptr, *hb2 = (float *)s.hb2.buf->dptr;
    float *q = (float *)s.q.buf->dptr, *kcol = (float *)s.kcol.buf->dptr, *vcol = (float *)s.vcol.buf->dptr;
    const uint32_t dim = config.dim, kvd = kv_dim();
    const auto wanted = [&](const char *name) { return !ctx->only_step || strcmp(ctx->only_step, name) == 0; };
    if (wanted("embedding row")) {
        SLAI_HIP_TRY(ctx, launch_embed(ctx->stream, weights.token_embd, &ds->token, nullptr, nullptr, dim, x));
        TRY(step_mark(ctx, "embedding row"));
    }
    // When the GEMV that writes x can leave a norm-weighted copy for the 64-row-tile GEMV that reads it next, that
    // consumer skips its own staging of the activations.
    float *xw = (float *)s.xw.buf->dptr;
    const float *prepared = nullptr;                           // valid copy for the next consumer of x, or none
    for (uint32_t l = 0; l < config.n_layers; ++l) {
        const Llama2LayerWeights &wl = weights.layers[l];
        // ---- bias + RoPE + cache write + attention (described first: it may join the q/k/v launch)
        AttnLaunch a{};
        a.q = q; a.kcache = s.key_cache[l].buf->dptr; a.vcache = s.value_cache[l].buf->dptr;
        a.kv_f16 = kv_dtype == SLAI_KV_F16;
        a.n_heads = config.n_q_heads; a.kv_mul = config.n_q_heads / config.n_kv_heads; a.head_size = head_size();
        a.kv_dim = kvd; a.seq_len = config.seq_len;
        a.pos_ptr = (const uint32_t *)&ds->pos;
        a.knew = kcol; a.vnew = vcol;
        a.qbias = wl.attn_q_bias.buf ? (const float *)wl.attn_q_bias.buf->dptr : nullptr;
        a.kbias = wl.attn_k_bias.buf ? (const float *)wl.attn_k_bias.buf->dptr : nullptr;
        a.vbias = wl.attn_v_bias.buf ? (const float *)wl.attn_v_bias.buf->dptr : nullptr;
        a.rope_variant = rope_variant(); a.rope_base = config.rope_base_freq;
        a.rope_theta = (const float *)s.rope_theta.buf->dptr;
        a.out = xb; a.scratch = ctx->attn_scratch; a.n_splits = attn_splits;
        // (split attention: the last split of a head merges them, where the placement of workgroups on the dies was verified)
        if (ctx->fuse_qkv_attention && ctx->handoff_counters && a.n_heads <= ctx->handoff_heads) a.combine_counters = ctx->handoff_counters;
        bool attention_done = false;
        // ---- RMSNorm + Q/K/V projections: matrices of one format and layout share a launch
        {
            // V first: in the usual mixes it has the widest format, so its workgroups should be dispatched earliest
            const slai_qmat *mats[3] = {wl.attn_v, wl.attn_k, wl.attn_q};
            float *outs[3] = {vcol, kcol, q};
            bool done[3] = {false, false, false};
            for (int i = 0; i < 3; ++i) {
                if (done[i]) continue;
                GemvCall c;
                c.nseg = 0; c.x = x;
                c.prologue = PRO_RMSNORM; c.norm_w = (const float *)wl.attn_norm.buf->dptr; c.eps = config.rms_norm_eps;
                if (gemv_is_rowtile(ctx, mats[i])) c.prepared = prepared;
                for (int j = i; j < 3; ++j) {
                    if (done[j] || !same_launch(mats[i], mats[j])) continue;
                    c.m[c.nseg] = mats[j]; c.out[c.nseg] = outs[j]; ++c.nseg;
                    done[j] = true;
                }
                // all three in one launch of 64-row tiles, one workgroup per head for the attention: one launch does both
                if (c.nseg == 3 && qkv_attention_fusable(ctx, mats[0], mats[1], mats[2], a)) {
                    TRY(gemv_call(ctx, c, "llama2 qkv + attention", &a));
                    attention_done = true;
                } else {
                    TRY(gemv_call(ctx, c, "llama2 qkv"));
                }
            }
        }
        if (!attention_done && wanted("llama2 attention")) {
            hipError_t e = launch_attention(ctx->stream, a);
            if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, "attention: unsupported head size or context length");
            SLAI_HIP_TRY(ctx, e);
            TRY(step_mark(ctx, "llama2 attention"));
        }
        // ---- attention output projection, residual in the epilogue
        {
            GemvCall c;
            c.m[0] = wl.attn_output; c.out[0] = x; c.flags[0] = GEMV_ACCUM; c.x = xb;
            prepared = nullptr;
            const bool gated_launch = wl.ffn_gate->type == wl.ffn_up->type && wl.ffn_gate->tiled == wl.ffn_up->tiled && wl.ffn_gate->rows_log2 == wl.ffn_up->rows_log2;
            const bool ffn_takes_prepared = gated_launch ? gemv_gated_is_rowtile(ctx, wl.ffn_gate, wl.ffn_up)
                                                         : (gemv_is_rowtile(ctx, wl.ffn_gate) && gemv_is_rowtile(ctx, wl.ffn_up));
            if (gemv_can_emit(wl.attn_output) && ffn_takes_prepared) {
                c.flags[0] |= GEMV_EMIT; c.emit_w = (const float *)wl.ffn_norm.buf->dptr; c.emit_out = xw;
                prepared = xw;
            }
            TRY(gemv_call(ctx, c, "llama2 attn_output"));
        }
        // ---- RMSNorm + gate/up + SiLU
        if (wl.ffn_gate->type == wl.ffn_up->type && wl.ffn_gate->tiled == wl.ffn_up->tiled && wl.ffn_gate->rows_log2 == wl.ffn_up->rows_log2) {
            GemvCall c;
            c.m[0] = wl.ffn_gate; c.m2[0] = wl.ffn_up; c.out[0] = hb; c.flags[0] = GEMV_SILU_GATE; c.x = x;
            c.prologue = PRO_RMSNORM; c.norm_w = (const float *)wl.ffn_norm.buf->dptr; c.eps = config.rms_norm_eps;
            c.prepared = prepared;
            TRY(gemv_call(ctx, c, "llama2 ffn gate/up"));
        } else {
            const slai_qmat *mats[2] = {wl.ffn_gate, wl.ffn_up};
            float *outs[2] = {hb, hb2};
            for (int i = 0; i < 2; ++i) {
                GemvCall c;
                c.m[0] = mats[i]; c.out[0] = outs[i]; c.x = x;
                c.prologue = PRO_RMSNORM; c.norm_w = (const float *)wl.ffn_norm.buf->dptr; c.eps = config.rms_norm_eps;
                c.prepared = prepared;
                TRY(gemv_call(ctx, c, "llama2 ffn gate/up"));
            }
            if (wanted("llama2 silu")) {
                SLAI_HIP_TRY(ctx, launch_silu(ctx->stream, VecView{hb, config.hidden_dim, 1}, VecView{hb2, config.hidden_dim, 1}));
                TRY(step_mark(ctx, "llama2 silu"));
            }
        }
        // ---- down projection, residual in the epilogue
        {
            GemvCall c;
            c.m[0] = wl.ffn_down; c.out[0] = x; c.flags[0] = GEMV_ACCUM; c.x = hb;
            // the next reader of x: the next layer's q/k/v (all three must take the prepared copy) or the output matrix
            const bool last = l + 1 == config.n_layers;
            bool next_ok = gemv_can_emit(wl.ffn_down);
            if (last) next_ok = next_ok && gemv_is_rowtile(ctx, weights.output);
            else {
                const Llama2LayerWeights &wn = weights.layers[l + 1];
                next_ok = next_ok && gemv_is_rowtile(ctx, wn.attn_q) && gemv_is_rowtile(ctx, wn.attn_k) && gemv_is_rowtile(ctx, wn.attn_v);
            }
            prepared = nullptr;
            if (next_ok) {
                const GpuTensor &nw = last ? weights.output_norm : weights.layers[l + 1].attn_norm;
                c.flags[0] |= GEMV_EMIT; c.emit_w = (const float *)nw.buf->dptr; c.emit_out = xw;
                prepared = xw;
            }
            TRY(gemv_call(ctx, c, "llama2 ffn_down"));
        }
    }
    {
        GemvCall c;
        c.m[0] = weights.output; c.out[0] = (float *)s.logits.buf->dptr; c.x = x;
        c.prologue = PRO_RMSNORM; c.norm_w = (const float *)weights.output_norm.buf->dptr; c.eps = config.rms_norm_eps;
        c.prepared = prepared;
        TRY(gemv_call(ctx, c, "llama2 output"));
    }
    if (sampler == 1)
        SLAI_HIP_TRY(ctx, launch_argmax(ctx->stream, (const float *)s.logits.buf->dptr, config.vocab_size, nullptr, ds,
                                        (const int *)loop.prompt->dptr, (int *)loop.out_tokens->dptr));
    else if (sampler == 2)
        SLAI_HIP_TRY(ctx, launch_sample(ctx->stream, (const float *)s.logits.buf->dptr, config.vocab_size, 0.0f, 0.0f, 0.0f, ctx->sampler_scratch, nullptr, ds,
                                        (const int *)loop.prompt->dptr, (int *)loop.out_tokens->dptr));
    return SLAI_OK;
}

// The chunked path covers the layouts the loader picks for models whose widths are multiples of 256: q/k/v and the
// gate/up pair in 64-row tiles (they take the norm-weighted copy of x the previous launch leaves), attention output and
// down projection in 16- or 32-row tiles (they leave it).
bool slai_llama2::chunk_supported() const {
    const uint32_t hs = head_size();
    if ((hs != 64 && hs != 128) || kv_dim() % 8 || config.dim % 16) return false;
    for (const Llama2LayerWeights &w : weights.layers) {
        for (const slai_qmat *m : {w.attn_q, w.attn_k, w.attn_v})
            if (!gemv_is_rowtile(ctx, m)) return false;
        if (!gemv_gated_is_rowtile(ctx, w.ffn_gate, w.ffn_up)) return false;
        if (!gemv_can_emit(w.attn_output) || !gemv_can_emit(w.ffn_down)) return false;
    }
    return true;
}

int slai_llama2::chunk_reserve(uint32_t rows) {
    PromptChunkState &c = chunk;
    if (rows < 32) rows = 32;                                   // the quad-major buffers always have 32 token slots
    if (rows <= c.rows) return SLAI_OK;
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "prompt chunk buffers must be reserved before graph capture");
    TRY(slai_synchronize(ctx));
    for (GpuTensor *t : {&c.x, &c.xw, &c.xb, &c.q, &c.k, &c.v, &c.hb, &c.xn, &c.hb2}) t->destroy(ctx);
    c.rows = 0;
    const uint32_t dim = config.dim, kvd = kv_dim();
    TRY(GpuTensor::matrix(ctx, dim, rows, STORAGE, &c.x));
    TRY(GpuTensor::matrix(ctx, dim + dim / 16, rows, STORAGE, &c.xw));
    TRY(GpuTensor::matrix(ctx, dim, rows, STORAGE, &c.xb));
    // (room for the partial results of a projection split four ways over its columns, see GemmChunkParams::ksplit)
    TRY(GpuTensor::matrix(ctx, dim, 4 * rows, STORAGE, &c.q));
    TRY(GpuTensor::matrix(ctx, kvd, 4 * rows, STORAGE, &c.k));
    TRY(GpuTensor::matrix(ctx, kvd, 4 * rows, STORAGE, &c.v));
    TRY(GpuTensor::matrix(ctx, config.hidden_dim, 4 * rows, STORAGE, &c.hb));
    TRY(GpuTensor::matrix(ctx, dim, rows, STORAGE, &c.xn));
    TRY(GpuTensor::matrix(ctx, config.hidden_dim, 4 * rows, STORAGE, &c.hb2));
    if (!c.positions) {
        TRY(slai_buffer_create(ctx, (size_t)config.seq_len * 4, SLAI_DT_I32, STORAGE | COPY_DST, &c.positions));
        TRY(slai_buffer_create(ctx, (size_t)config.seq_len * 4, SLAI_DT_I32, STORAGE | COPY_DST, &c.tokens));
        std::vector<uint32_t> iota(config.seq_len);
        for (uint32_t i = 0; i < config.seq_len; ++i) iota[i] = i;
        TRY(slai_write_buffer(ctx, c.positions, 0, iota.data(), iota.size() * 4));
    }
    c.rows = rows;
    return SLAI_OK;
}

// The layer loop of enqueue_fused for n tokens at once.  Token b of the chunk lives in row b of every activation
// matrix; the GEMV launches take all rows (GemvBatch), bias + RoPE + cache write run for all rows before the attention
// of any row (a token attends to the earlier tokens of its chunk), and the logits are not computed.
int slai_llama2::enqueue_chunk(uint32_t pos0, uint32_t n, const int *tokens_dev) {
    PromptChunkState &pc = chunk;
    if (n == 0 || n > pc.rows || pos0 + n > config.seq_len) return set_error(ctx, SLAI_E_ARG, "prompt chunk out of range");
    const uint32_t dim = config.dim, kvd = kv_dim(), hid = config.hidden_dim, xws = dim + dim / 16;
    float *x = (float *)pc.x.buf->dptr, *xw = (float *)pc.xw.buf->dptr, *xb = (float *)pc.xb.buf->dptr, *q = (float *)pc.q.buf->dptr;
    float *k = (float *)pc.k.buf->dptr, *v = (float *)pc.v.buf->dptr, *hb = (float *)pc.hb.buf->dptr;
    for (uint32_t b = 0; b < n; ++b) {
        SLAI_HIP_TRY(ctx, launch_embed(ctx->stream, weights.token_embd, tokens_dev + b, nullptr, nullptr, dim, x + (size_t)b * dim));
        SLAI_HIP_TRY(ctx, launch_prepare(ctx->stream, xw + (size_t)b * xws, x + (size_t)b * dim, (const float *)weights.layers[0].attn_norm.buf->dptr, dim));
    }
    for (uint32_t l = 0; l < config.n_layers; ++l) {
        const Llama2LayerWeights &wl = weights.layers[l];
        {   // ---- RMSNorm + q/k/v
            const slai_qmat *mats[3] = {wl.attn_v, wl.attn_k, wl.attn_q};
            float *outs[3] = {v, k, q};
            const uint32_t strides[3] = {kvd, kvd, dim};
            bool done[3] = {false, false, false};
            for (int i = 0; i < 3; ++i) {
                if (done[i]) continue;
                GemvCall c;
                c.nseg = 0; c.x = x; c.prepared = xw;
                c.prologue = PRO_RMSNORM; c.norm_w = (const float *)wl.attn_norm.buf->dptr; c.eps = config.rms_norm_eps;
                c.batch.n = n; c.batch.x_stride = dim; c.batch.prepared_stride = xws;
                for (int j = i; j < 3; ++j) {
                    if (done[j] || !same_launch(mats[i], mats[j])) continue;
                    c.m[c.nseg] = mats[j]; c.out[c.nseg] = outs[j]; c.batch.out_stride[c.nseg] = strides[j]; ++c.nseg;
                    done[j] = true;
                }
                TRY(gemv_call(ctx, c, "llama2 qkv (prompt chunk)"));
            }
        }
        TRY(chunk_attention(l, pos0, n));
        {   // ---- attention output, residual, copy for the feed-forward norm
            GemvCall c;
            c.m[0] = wl.attn_output; c.out[0] = x; c.flags[0] = GEMV_ACCUM | GEMV_EMIT; c.x = xb;
            c.emit_w = (const float *)wl.ffn_norm.buf->dptr; c.emit_out = xw;
            c.batch.n = n; c.batch.x_stride = dim; c.batch.out_stride[0] = dim; c.batch.emit_stride = xws;
            TRY(gemv_call(ctx, c, "llama2 attn_output (prompt chunk)"));
        }
        {   // ---- RMSNorm + gate/up + SiLU
            GemvCall c;
            c.m[0] = wl.ffn_gate; c.m2[0] = wl.ffn_up; c.out[0] = hb; c.flags[0] = GEMV_SILU_GATE; c.x = x; c.prepared = xw;
            c.prologue = PRO_RMSNORM; c.norm_w = (const float *)wl.ffn_norm.buf->dptr; c.eps = config.rms_norm_eps;
            c.batch.n = n; c.batch.x_stride = dim; c.batch.prepared_stride = xws; c.batch.out_stride[0] = hid;
            TRY(gemv_call(ctx, c, "llama2 ffn gate/up (prompt chunk)"));
        }
        {   // ---- down projection, residual, copy for the next layer's norm (nothing reads it after the last layer)
            GemvCall c;
            c.m[0] = wl.ffn_down; c.out[0] = x; c.flags[0] = GEMV_ACCUM; c.x = hb;
            if (l + 1 < config.n_layers) {
                c.flags[0] |= GEMV_EMIT; c.emit_w = (const float *)weights.layers[l + 1].attn_norm.buf->dptr; c.emit_out = xw;
            }
            c.batch.n = n; c.batch.x_stride = hid; c.batch.out_stride[0] = dim; c.batch.emit_stride = xws;
            TRY(gemv_call(ctx, c, "llama2 ffn_down (prompt chunk)"));
        }
    }
    return SLAI_OK;
}

// Bias + RoPE + cache write for the n tokens of a chunk (their q / k / v are in the chunk's matrices), then their
// attention into the chunk's xb.
int slai_llama2::chunk_attention(uint32_t l, uint32_t pos0, uint32_t n, uint32_t nparts, bool out_quads, int *split_flag) {
    PromptChunkState &pc = chunk;
    Llama2State &s = state;
    const Llama2LayerWeights &wl = weights.layers[l];
    const uint32_t dim = config.dim, kvd = kv_dim();
    float *q = (float *)pc.q.buf->dptr;
    AttnLaunch a{};
    a.q = q; a.kcache = s.key_cache[l].buf->dptr; a.vcache = s.value_cache[l].buf->dptr;
    a.kv_f16 = kv_dtype == SLAI_KV_F16;
    a.n_heads = config.n_q_heads; a.kv_mul = config.n_q_heads / config.n_kv_heads; a.head_size = head_size();
    a.kv_dim = kvd; a.seq_len = config.seq_len;
    a.pos_ptr = (const uint32_t *)pc.positions->dptr + pos0;
    a.qbias = wl.attn_q_bias.buf ? (const float *)wl.attn_q_bias.buf->dptr : nullptr;
    a.kbias = wl.attn_k_bias.buf ? (const float *)wl.attn_k_bias.buf->dptr : nullptr;
    a.vbias = wl.attn_v_bias.buf ? (const float *)wl.attn_v_bias.buf->dptr : nullptr;
    a.rope_variant = rope_variant(); a.rope_base = config.rope_base_freq;
    a.rope_theta = (const float *)s.rope_theta.buf->dptr;
    a.out = out_quads ? (float *)pc.xn.buf->dptr : (float *)pc.xb.buf->dptr; a.scratch = nullptr; a.n_splits = 1;
    SLAI_HIP_TRY(ctx, launch_rope_store_batch(ctx->stream, a, q, (const float *)pc.k.buf->dptr, (const float *)pc.v.buf->dptr, n, dim, kvd, nparts, 32 * dim, 32 * kvd));
    SLAI_HIP_TRY(ctx, launch_attention_batch(ctx->stream, a, n, dim, dim, out_quads, split_flag));
    return SLAI_OK;
}

bool slai_llama2::chunk_gemm_supported() const {
    const uint32_t hs = head_size();
    if ((hs != 64 && hs != 128) || kv_dim() % 8 || config.dim % 4 || config.hidden_dim % 4) return false;
    for (const Llama2LayerWeights &w : weights.layers)
        for (const slai_qmat *m : {w.attn_q, w.attn_k, w.attn_v, w.attn_output, w.ffn_gate, w.ffn_up, w.ffn_down})
            if (!gemm_chunk_supports(m)) return false;
    return true;
}

namespace {
// Into how many column ranges a launch over 64-row-tile matrices is cut (GemmChunkParams::ksplit): tile counts such as
// 192 or 344 do not divide 256 compute units evenly, two or four times as many smaller units nearly do; four ranges
// while that stays within about four workgroups per compute unit, else two (measured on the 7B shapes).
uint32_t chunk_ksplit(int nmat, const slai_qmat *const *mats) {
    uint32_t tiles = 0;
    for (int i = 0; i < nmat; ++i) {
        if (mats[i]->rows_log2 != 6) return 1;
        tiles += (mats[i]->nrows + 63) / 64;
    }
    if (mats[0]->ncb < 8) return 1;
    return tiles * 4 <= 1024 ? 4 : 2;
}

// matrices (with the same input) through the matrix-core kernel: 64-row-tile matrices share a launch
int gemm_chunk_call(slai_ctx *ctx, int nmat, const slai_qmat *const *mats, float *const *outs, const uint32_t *out_strides, uint32_t flags,
                    const float *xq, uint32_t ntokens, const char *who, uint32_t ksplit = 1, bool split_f16 = false) {
    bool done[3] = {false, false, false};
    for (int i = 0; i < nmat; ++i) {
        if (done[i]) continue;
        GemmChunkParams p;
        p.nseg = 0; p.ncols = mats[i]->ncols; p.ncb = mats[i]->ncb; p.ngroups = mats[i]->ngroups; p.rows_log2 = mats[i]->rows_log2;
        p.x = xq; p.ntokens = ntokens; p.ksplit = ksplit; p.split_f16 = split_f16;
        for (int j = i; j < nmat; ++j) {
            // (one launch: 64-row tiles of the same width, and of the same format unless both are K-quants)
            const auto kquant = [](int t) { return t == T_Q4_K || t == T_Q5_K || t == T_Q6_K; };
            if (done[j] || (j != i && (mats[j]->rows_log2 != 6 || mats[i]->rows_log2 != 6 || mats[j]->ncols != mats[i]->ncols ||
                                       (mats[j]->type != mats[i]->type && !(kquant(mats[j]->type) && kquant(mats[i]->type)))))) continue;
            GemmChunkSeg &sg = p.seg[p.nseg++];
            sg.W = mats[j]->dptr; sg.type = mats[j]->type; sg.nrows = mats[j]->nrows; sg.out = outs[j]; sg.out_stride = out_strides[j]; sg.flags = flags;
            sg.part_stride = 32 * out_strides[j];
            done[j] = true;
        }
        hipError_t e = launch_gemm_chunk(ctx, p);
        if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": unsupported shape for the prompt-chunk GEMM");
        if (e != hipSuccess) return hip_fail(ctx, e, who);
    }
    return SLAI_OK;
}
}  // namespace

// The layer loop for a chunk of up to 32 tokens with every projection on the matrix cores (kernels_gemm_chunk.hip):
bool slai_llama2::chunk_split_ok() const {
    for (const Llama2LayerWeights &wl : weights.layers)
        for (const slai_qmat *m : {wl.attn_q, wl.attn_k, wl.attn_v, wl.attn_output, wl.ffn_gate, wl.ffn_up, wl.ffn_down})
            if (!(m->wbound < 255.0f)) return false;
    return true;
}

// RMSNorm of all rows, q/k/v, bias + RoPE + cache write, attention, output projection into the residual, RMSNorm,
// gate and up, SiLU, down projection into the residual (transformer.rs:316-381 per token).
// split_f16: the GEMMs on the half-precision matrix cores, their inputs written as f16 heads and remainders by the kernels
// before them (which set *ctx->split_flag when a value does not fit: the caller then repeats the pass without).
int slai_llama2::enqueue_chunk_gemm(uint32_t pos0, uint32_t n, const int *tokens_dev, bool split_f16) {
    PromptChunkState &pc = chunk;
    int *const sf = split_f16 ? ctx->split_flag : nullptr;
    if (n == 0 || n > 32 || n > pc.rows || pos0 + n > config.seq_len) return set_error(ctx, SLAI_E_ARG, "prompt chunk out of range");
    const uint32_t dim = config.dim, kvd = kv_dim(), hid = config.hidden_dim;
    float *x = (float *)pc.x.buf->dptr, *xn = (float *)pc.xn.buf->dptr, *q = (float *)pc.q.buf->dptr;
    float *k = (float *)pc.k.buf->dptr, *v = (float *)pc.v.buf->dptr, *hb = (float *)pc.hb.buf->dptr, *hb2 = (float *)pc.hb2.buf->dptr;
    SLAI_HIP_TRY(ctx, launch_embed_rows(ctx->stream, weights.token_embd, tokens_dev, n, dim, x, dim));
    // xn (the normalised rows, then the attention output) and hb, hb2 are quad-major with 32 token slots: the layout the
    // GEMM kernels read.
    // q/k/v and gate/up are cut into column ranges when every matrix involved has 64-row tiles (chunk_ksplit).
    for (uint32_t l = 0; l < config.n_layers; ++l) {
        const Llama2LayerWeights &wl = weights.layers[l];
        SLAI_HIP_TRY(ctx, launch_rms_norm_quads(ctx->stream, xn, x, (const float *)wl.attn_norm.buf->dptr, dim, n, dim, config.rms_norm_eps, sf));
        {
            const slai_qmat *mats[3] = {wl.attn_v, wl.attn_k, wl.attn_q};
            float *outs[3] = {v, k, q};
            const uint32_t strides[3] = {kvd, kvd, dim};
            const uint32_t ks = chunk_ksplit(3, mats);
            TRY(gemm_chunk_call(ctx, 3, mats, outs, strides, 0, xn, n, "llama2 qkv (prompt chunk)", ks, split_f16));
            TRY(chunk_attention(l, pos0, n, ks, true, sf));   // straight into xn, quad-major (as f16 pairs for the f16 form)
        }
        {
            const slai_qmat *mats[1] = {wl.attn_output};
            float *outs[1] = {x};
            const uint32_t strides[1] = {dim};
            TRY(gemm_chunk_call(ctx, 1, mats, outs, strides, GEMV_ACCUM, xn, n, "llama2 attn_output (prompt chunk)", 1, split_f16));
        }
        SLAI_HIP_TRY(ctx, launch_rms_norm_quads(ctx->stream, xn, x, (const float *)wl.ffn_norm.buf->dptr, dim, n, dim, config.rms_norm_eps, sf));
        {
            const slai_qmat *mats[2] = {wl.ffn_gate, wl.ffn_up};
            float *outs[2] = {hb, hb2};
            const uint32_t strides[2] = {hid, hid};
            const uint32_t ks = chunk_ksplit(2, mats);
            TRY(gemm_chunk_call(ctx, 2, mats, outs, strides, GEMM_OUT_QUADS, xn, n, "llama2 ffn gate/up (prompt chunk)", ks, split_f16));
            // element-wise over the token slots in use (those past the chunk hold stale values)
            SLAI_HIP_TRY(ctx, launch_silu_parts(ctx->stream, hb, hb2, 32 * hid, ks, 32 * hid, sf, n));
        }
        {
            const slai_qmat *mats[1] = {wl.ffn_down};
            float *outs[1] = {x};
            const uint32_t strides[1] = {dim};
            TRY(gemm_chunk_call(ctx, 1, mats, outs, strides, GEMV_ACCUM, hb, n, "llama2 ffn_down (prompt chunk)", 1, split_f16));
        }
    }
    return SLAI_OK;
}

SLAI_EXPORT int slai_llama2_from_gguf(slai_ctx *ctx, const slai_gguf *g, int model_type, int kv_dtype, slai_llama2 **out) {
    if (!ctx || !g || !out) return SLAI_E_ARG;
    *out = nullptr;
    if ((model_type != SLAI_MODEL_LLAMA && model_type != SLAI_MODEL_QWEN2) || (kv_dtype != SLAI_KV_F32 && kv_dtype != SLAI_KV_F16))
        return set_error(ctx, SLAI_E_ARG, "slai_llama2_from_gguf: bad model type or kv dtype");
    std::unique_ptr<slai_llama2> m(new slai_llama2());
    m->ctx = ctx; m->model_type = model_type; m->kv_dtype = kv_dtype;
    int rc = m->load(g);
    if (rc) { std::string keep = ctx->err; slai_llama2_destroy(m.release()); ctx->err = keep; return rc; }
    *out = m.release();
    return SLAI_OK;
}

SLAI_EXPORT void slai_llama2_destroy(slai_llama2 *m) {
    if (!m) return;
    slai_ctx *ctx = m->ctx;
    slai_synchronize(ctx);
    loop_destroy(ctx, m->loop);
    for (auto &w : m->weights.layers) {
        for (slai_qmat *q : {w.attn_k, w.attn_q, w.attn_v, w.ffn_down, w.ffn_gate, w.ffn_up, w.attn_output}) slai_qmat_destroy(ctx, q);
        for (GpuTensor *t : {&w.attn_norm, &w.attn_k_bias, &w.attn_q_bias, &w.attn_v_bias, &w.ffn_norm}) t->destroy(ctx);
    }
    if (m->weights.output != m->weights.token_embd) slai_qmat_destroy(ctx, m->weights.output);
    slai_qmat_destroy(ctx, m->weights.token_embd);
    m->weights.output_norm.destroy(ctx);
    Llama2State &s = m->state;
    for (GpuTensor *t : {&s.x, &s.xb, &s.xb2, &s.hb, &s.hb2, &s.q, &s.att, &s.logits, &s.kcol, &s.vcol, &s.xw, &s.rope_theta}) t->destroy(ctx);
    for (auto &t : s.key_cache) t.destroy(ctx);
    for (auto &t : s.value_cache) t.destroy(ctx);
    for (slai_buffer *b : {s.rope_config, s.rms_norm_config, s.attn_params}) if (b) slai_buffer_destroy(ctx, b);
    for (slai_buffer *b : {m->persistent.layers, m->persistent.flow, m->persistent.slots}) if (b) slai_buffer_destroy(ctx, b);
    PromptChunkState &pc = m->chunk;
    for (GpuTensor *t : {&pc.x, &pc.xw, &pc.xb, &pc.q, &pc.k, &pc.v, &pc.hb, &pc.xn, &pc.hb2}) t->destroy(ctx);
    for (slai_buffer *b : {pc.positions, pc.tokens}) if (b) slai_buffer_destroy(ctx, b);
    delete m;
}

SLAI_EXPORT int slai_llama2_decode_form(const slai_llama2 *m) { return m && m->persistent.ready ? 1 : 0; }

// One token at (pos, token) through the resident launch with its time stamps switched on: per workgroup 16 stamps per
// layer (four per phase: entered, input staged, multiplied, reduced) and 8 for the output matrix, in ticks of the
// constant 100 MHz clock.  The caches are left as any forward pass at that position leaves them.
SLAI_EXPORT int slai_llama2_trace_token(slai_llama2 *m, uint32_t pos, uint32_t token, uint64_t *out, size_t capacity, uint32_t *n_workgroups,
                                        uint32_t *stamps_per_workgroup) {
    if (!m || !out || !n_workgroups || !stamps_per_workgroup) return SLAI_E_ARG;
    slai_ctx *ctx = m->ctx;
    if (!m->persistent.ready) return set_error(ctx, SLAI_E_STATE, "slai_llama2_trace_token: this model does not take the resident launch");
    if (pos >= m->config.seq_len || token >= m->config.vocab_size) return set_error(ctx, SLAI_E_ARG, "slai_llama2_trace_token: position or token out of range");
    const uint32_t stride = 16 * m->config.n_layers + 8, grid = m->persistent.grid;
    const size_t n = (size_t)grid * stride;
    if (capacity < n) return set_error(ctx, SLAI_E_SHAPE, "slai_llama2_trace_token: need room for " + std::to_string(n) + " stamps");
    slai_buffer *buf = nullptr;
    TRY(slai_buffer_create(ctx, n * 8, SLAI_DT_U8, STORAGE | COPY_SRC, &buf));
    DecodeState ds{(int)pos, (int)token, 0, 0};
    int rc = slai_write_buffer(ctx, m->loop.state, 0, &ds, sizeof ds);
    m->persistent.params.trace = (uint64_t *)buf->dptr;
    if (!rc) rc = m->enqueue_persistent(0, pos > resident_far_from(m->kv_dtype == SLAI_KV_F16));
    m->persistent.params.trace = nullptr;
    if (!rc) rc = slai_synchronize(ctx);
    if (!rc) rc = handoff_check(ctx);
    if (!rc) rc = slai_read_buffer(ctx, buf, 0, out, n * 8);
    slai_buffer_destroy(ctx, buf);
    *n_workgroups = grid; *stamps_per_workgroup = stride;
    return rc;
}

// One token, launched from the host `reps` times at the same position, with an event after every launch (the resident
// form: the embedding row, the emptying of the hand-off buffers and the one launch of the layer stack): mean time from the end of the launch before to the end of each launch, by step name in order of
// first appearance (`names`: newline separated), and how often the step occurs per token.
SLAI_EXPORT int slai_llama2_time_steps(slai_llama2 *m, uint32_t pos, uint32_t token, uint32_t reps, char *names, size_t names_len, float *mean_us,
                                       float *alone_us, uint32_t *per_token, uint32_t capacity, uint32_t *n_steps) {
    if (!m || !names || !mean_us || !alone_us || !per_token || !n_steps || reps == 0) return SLAI_E_ARG;
    slai_ctx *ctx = m->ctx;
    if (pos >= m->config.seq_len || token >= m->config.vocab_size) return set_error(ctx, SLAI_E_ARG, "slai_llama2_time_steps: position or token out of range");
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "slai_llama2_time_steps: not during graph capture");
    DecodeState ds{(int)pos, (int)token, 0, 0};
    TRY(slai_write_buffer(ctx, m->loop.state, 0, &ds, sizeof ds));
    const auto enqueue = [&]() { return m->enqueue_fused(0, m->persistent.ready ? (pos > resident_far_from(m->kv_dtype == SLAI_KV_F16) ? 2 : 1) : 0); };
    TRY(enqueue());                                             // untimed: sizes scratch, warms the caches
    TRY(slai_synchronize(ctx));
    std::vector<std::pair<const char *, hipEvent_t>> marks;
    marks.reserve((size_t)reps * (5 * m->config.n_layers + 4));
    ctx->step_marks = &marks;
    int rc = SLAI_OK;
    for (uint32_t r = 0; r < reps && !rc; ++r) {
        rc = step_mark(ctx, nullptr);                           // where the token starts
        if (!rc) rc = enqueue();
    }
    ctx->step_marks = nullptr;
    if (!rc) rc = slai_synchronize(ctx);
    if (!rc) rc = handoff_check(ctx);
    std::vector<const char *> order;
    std::vector<double> total;
    std::vector<uint32_t> count;
    for (size_t i = 1; i < marks.size() && !rc; ++i) {
        if (!marks[i].first) continue;                          // a token's start: nothing was launched before it
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, marks[i - 1].second, marks[i].second) != hipSuccess) { rc = set_error(ctx, SLAI_E_HIP, "slai_llama2_time_steps: event time"); break; }
        size_t k = 0;
        while (k < order.size() && strcmp(order[k], marks[i].first) != 0) ++k;
        if (k == order.size()) { order.push_back(marks[i].first); total.push_back(0.0); count.push_back(0); }
        total[k] += ms; ++count[k];
    }
    for (auto &mk : marks) (void)hipEventDestroy(mk.second);
    if (rc) return rc;
    if (order.size() > capacity) return set_error(ctx, SLAI_E_SHAPE, "slai_llama2_time_steps: more steps than room for them");
    std::string joined;
    for (size_t k = 0; k < order.size(); ++k) {
        mean_us[k] = (float)(total[k] * 1000.0 / count[k]);
        per_token[k] = count[k] / reps;
        joined += order[k];
        joined += '\n';
    }
    if (joined.size() + 1 > names_len) return set_error(ctx, SLAI_E_SHAPE, "slai_llama2_time_steps: the names do not fit");
    memcpy(names, joined.c_str(), joined.size() + 1);
    *n_steps = (uint32_t)order.size();
    // each step alone: only its launches (one per layer: every layer's own weights, so nothing stays cached from launch to
    // launch), back to back, an event before the first and after the last
    hipEvent_t e0, e1;
    SLAI_HIP_TRY(ctx, hipEventCreate(&e0));
    SLAI_HIP_TRY(ctx, hipEventCreate(&e1));
    for (size_t k = 0; k < order.size() && !rc; ++k) {
        if (m->persistent.ready) { alone_us[k] = mean_us[k]; continue; }     // (a resident launch needs the buffers emptied before it: never alone)
        ctx->only_step = order[k];
        rc = m->enqueue_fused(0, 0);                            // untimed
        if (!rc && hipEventRecord(e0, ctx->stream) != hipSuccess) rc = SLAI_E_HIP;
        for (uint32_t r = 0; r < reps && !rc; ++r) rc = m->enqueue_fused(0, 0);
        if (!rc && hipEventRecord(e1, ctx->stream) != hipSuccess) rc = SLAI_E_HIP;
        ctx->only_step = nullptr;
        if (!rc) rc = slai_synchronize(ctx);
        float ms = 0.0f;
        if (!rc && hipEventElapsedTime(&ms, e0, e1) != hipSuccess) rc = SLAI_E_HIP;
        alone_us[k] = ms * 1000.0f / (float)(reps * (per_token[k] ? per_token[k] : 1));
    }
    ctx->only_step = nullptr;
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    if (rc == SLAI_E_HIP) return set_error(ctx, SLAI_E_HIP, "slai_llama2_time_steps: event");
    if (rc) return rc;
    // leave the state a whole forward at this position leaves
    TRY(enqueue());
    TRY(slai_synchronize(ctx));
    return handoff_check(ctx);
}

SLAI_EXPORT int slai_llama2_get_config(const slai_llama2 *m, slai_llama2_config *out) {
    if (!m || !out) return SLAI_E_ARG;
    *out = m->config;
    return SLAI_OK;
}
SLAI_EXPORT size_t slai_llama2_weight_bytes(const slai_llama2 *m) { return m ? m->weight_bytes : 0; }

// `Llama2Config::derived_configs` (models/llama2/cpu.rs:111-143)
static void derived_configs(const slai_llama2 *m, uint32_t pos, slai_rope_config *rope, slai_rms_norm_config *rms, slai_attn_params *attn) {
    const slai_llama2_config &c = m->config;
    *rope = slai_rope_config{m->head_size(), m->kv_dim(), pos, c.rope_base_freq};
    *rms = slai_rms_norm_config{c.rms_norm_eps, {0, 0, 0}};
    *attn = slai_attn_params{c.seq_len, m->kv_dim(), c.n_q_heads / c.n_kv_heads, c.n_q_heads, m->head_size(), pos, {0, 0}};
}

SLAI_EXPORT int slai_llama2_forward_logits(slai_llama2 *m, uint32_t pos, uint32_t token, int fused, float *logits_out) {
    if (!m) return SLAI_E_ARG;
    slai_ctx *ctx = m->ctx;
    if (pos >= m->config.seq_len || token >= m->config.vocab_size) return set_error(ctx, SLAI_E_ARG, "slai_llama2_forward_logits: position or token out of range");
    Llama2State &s = m->state;
    if (!fused) {
        // chat_llama2.rs:176-189: per-token uniforms, then the embedding column into x
        slai_rope_config rope; slai_rms_norm_config rms; slai_attn_params attn;
        derived_configs(m, pos, &rope, &rms, &attn);
        TRY(slai_write_buffer(ctx, s.rope_config, 0, &rope, sizeof rope));
        TRY(slai_write_buffer(ctx, s.rms_norm_config, 0, &rms, sizeof rms));
        TRY(slai_write_buffer(ctx, s.attn_params, 0, &attn, sizeof attn));
        const slai_qmat *te = m->weights.token_embd;
        TRY(slai_qmat_dequantize(ctx, te, token, 1, slai_view{s.x.buf, 0, {1, m->config.dim, 1, 1}, {m->config.dim, 1, m->config.dim, m->config.dim}}));
        LlmContext ctxt(ctx);
        TRY(ctxt.begin_submission());                                   // :199
        TRY(m->launch(ctxt, attn, pos));                                 // :200-207
        TRY(ctxt.submit());                                              // :218
    } else {
        DecodeState ds{(int)pos, (int)token, 0, 0};
        TRY(slai_write_buffer(ctx, m->loop.state, 0, &ds, sizeof ds));
        TRY(m->enqueue_fused(0, m->form_at(pos)));
    }
    TRY(slai_synchronize(ctx));                                          // :219
    TRY(handoff_check(ctx));
    if (logits_out) TRY(slai_read_buffer(ctx, s.logits.buf, 0, logits_out, (size_t)m->config.vocab_size * 4));   // :225-227
    return SLAI_OK;
}

// `sampling`: null for the greedy loop, else temperature / top-p / seed of the device sampler
struct SamplingParams { float temperature, topp; uint64_t seed; };
template <class Model>
static int generate_impl(Model *m, slai_ctx *ctx, DeviceLoop &L, uint32_t seq_len, uint32_t vocab, const int32_t *prompt, uint32_t n_prompt,
                         uint32_t start_pos, uint32_t n_steps, int32_t *out_tokens, float *elapsed_ms, const SamplingParams *sampling = nullptr) {
    if (sampling && !(sampling->temperature >= 0.0f)) return set_error(ctx, SLAI_E_ARG, "generate: the temperature must not be negative");
    const int mode = sampling ? 2 : 1;
    if (sampling) TRY(sampler_scratch_reserve(ctx, sample_scratch_floats(vocab)));
    if (!prompt || !out_tokens || n_prompt == 0 || start_pos >= n_prompt) return set_error(ctx, SLAI_E_ARG, "generate: bad prompt / start position");
    if (n_steps == 0) return SLAI_OK;
    if (start_pos + n_steps > seq_len) return set_error(ctx, SLAI_E_SHAPE, "generate: would run past the context length");
    if (n_prompt > L.capacity || n_steps > L.capacity) return set_error(ctx, SLAI_E_SHAPE, "generate: prompt longer than the context length");
    for (uint32_t i = 0; i < n_prompt; ++i)
        if (prompt[i] < 0 || (uint32_t)prompt[i] >= vocab) return set_error(ctx, SLAI_E_ARG, "generate: prompt token out of range");
    DecodeState ds{(int)start_pos, prompt[start_pos], (int)n_prompt, 0, 0.0f, 0.0f, 0, 0};     // chat_llama2.rs:105
    if (sampling) { ds.temperature = sampling->temperature; ds.topp = sampling->topp; ds.seed_lo = (uint32_t)sampling->seed; ds.seed_hi = (uint32_t)(sampling->seed >> 32); }
    TRY(slai_write_buffer(ctx, L.state, 0, &ds, sizeof ds));
    TRY(slai_write_buffer(ctx, L.prompt, 0, prompt, (size_t)n_prompt * 4));
    if (!ctx->use_graph) {
        SLAI_HIP_TRY(ctx, hipEventRecord(L.ev0, ctx->stream));
        for (uint32_t i = 0; i < n_steps; ++i) TRY(m->enqueue_fused(mode, m->form_at(start_pos + i)));
        SLAI_HIP_TRY(ctx, hipEventRecord(L.ev1, ctx->stream));
        TRY(slai_synchronize(ctx));
        TRY(handoff_check(ctx));
        if (elapsed_ms) SLAI_HIP_TRY(ctx, hipEventElapsedTime(elapsed_ms, L.ev0, L.ev1));
        return slai_read_buffer(ctx, L.out_tokens, 0, out_tokens, (size_t)n_steps * 4);
    }
    // one captured token per launch form the run needs (the form depends on the position: Model::form_at)
    for (uint32_t i = 0; i < n_steps; ++i) {
        slai_graph *&graph = L.graph[m->form_at(start_pos + i)][sampling ? 1 : 0];
        if (graph) continue;
        TRY(slai_graph_begin_capture(ctx));
        int rc = m->enqueue_fused(mode, m->form_at(start_pos + i));
        slai_graph *g = nullptr;
        int rc2 = slai_graph_end_capture(ctx, &g);
        if (rc) { if (g) slai_graph_destroy(ctx, g); return rc; }
        if (rc2) return rc2;
        graph = g;
    }
    SLAI_HIP_TRY(ctx, hipEventRecord(L.ev0, ctx->stream));
    for (uint32_t i = 0; i < n_steps; ++i) TRY(slai_graph_launch(ctx, L.graph[m->form_at(start_pos + i)][sampling ? 1 : 0]));   // chat_llama2.rs:109 loop
    SLAI_HIP_TRY(ctx, hipEventRecord(L.ev1, ctx->stream));
    TRY(slai_synchronize(ctx));
    TRY(handoff_check(ctx));
    if (elapsed_ms) SLAI_HIP_TRY(ctx, hipEventElapsedTime(elapsed_ms, L.ev0, L.ev1));
    return slai_read_buffer(ctx, L.out_tokens, 0, out_tokens, (size_t)n_steps * 4);
}

SLAI_EXPORT int slai_llama2_generate(slai_llama2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos, uint32_t n_steps,
                                     int32_t *out_tokens, float *elapsed_ms) {
    if (!m) return SLAI_E_ARG;
    return generate_impl(m, m->ctx, m->loop, m->config.seq_len, m->config.vocab_size, prompt, n_prompt, start_pos, n_steps, out_tokens, elapsed_ms);
}

// The same loop with `Sampler::new(vocab, temperature, topp).sample(logits)` (models/sampler.rs:33-53; the chat uses
// 0.7 / 0.95, slai-chat/src/sampler.rs:107) on the device instead of a logits readback per token.  The draw for
// position pos is slai_sampler_coin(seed, pos).
SLAI_EXPORT int slai_llama2_generate_sampled(slai_llama2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos, uint32_t n_steps,
                                             float temperature, float topp, uint64_t seed, int32_t *out_tokens, float *elapsed_ms) {
    if (!m) return SLAI_E_ARG;
    const SamplingParams sp{temperature, topp, seed};
    return generate_impl(m, m->ctx, m->loop, m->config.seq_len, m->config.vocab_size, prompt, n_prompt, start_pos, n_steps, out_tokens, elapsed_ms, &sp);
}

// 0: the ordinary loop, 1: per-token workgroups over shared weights, 2: matrix cores
SLAI_EXPORT int slai_llama2_prefill_supported(const slai_llama2 *m) {
    if (!m) return 0;
    if (m->ctx->prompt_gemm && m->chunk_gemm_supported()) return 2;
    return m->chunk_supported() ? 1 : 0;
}

// The prompt loop of chat_llama2.rs:105-158 feeds the prompt one token per forward pass and throws the logits of all but
// the last away.  This runs positions start_pos .. start_pos + n_tokens - 1 through the layers `chunk` tokens at a time
// and computes no logits; afterwards the caches are what the token-by-token loop would have left, and generation
// continues with slai_llama2_generate(prompt, n_prompt, start_pos = n_prompt - 1, ...).
SLAI_EXPORT int slai_llama2_prefill(slai_llama2 *m, const int32_t *tokens, uint32_t n_tokens, uint32_t start_pos, uint32_t chunk, float *elapsed_ms) {
    if (!m) return SLAI_E_ARG;
    slai_ctx *ctx = m->ctx;
    if (elapsed_ms) *elapsed_ms = 0.0f;
    if (n_tokens == 0) return SLAI_OK;
    if (!tokens) return set_error(ctx, SLAI_E_ARG, "slai_llama2_prefill: no tokens");
    if ((uint64_t)start_pos + n_tokens > m->config.seq_len) return set_error(ctx, SLAI_E_SHAPE, "slai_llama2_prefill: would run past the context length");
    for (uint32_t i = 0; i < n_tokens; ++i)
        if (tokens[i] < 0 || (uint32_t)tokens[i] >= m->config.vocab_size) return set_error(ctx, SLAI_E_ARG, "slai_llama2_prefill: token out of range");
    if (chunk > 64) return set_error(ctx, SLAI_E_ARG, "slai_llama2_prefill: at most 64 tokens per chunk");
    // K-quants in the tiled layouts: matrix cores, 32 tokens per pass; other tiled formats: one workgroup per token and
    // tile over shared weights; anything else: the ordinary loop
    const bool gemm = ctx->prompt_gemm && m->chunk_gemm_supported();
    const bool shared = !gemm && m->chunk_supported();
    if (chunk == 0) chunk = gemm ? 32 : 16;
    if (chunk == 1 || (!gemm && !shared)) {
        // one token per pass, picks discarded
        std::vector<int32_t> prompt((size_t)start_pos + n_tokens, 0), picks(n_tokens);
        std::copy(tokens, tokens + n_tokens, prompt.begin() + start_pos);
        return generate_impl(m, ctx, m->loop, m->config.seq_len, m->config.vocab_size, prompt.data(), (uint32_t)prompt.size(), start_pos, n_tokens,
                             picks.data(), elapsed_ms);
    }
    if (gemm && chunk > 32) chunk = 32;
    TRY(m->chunk_reserve(chunk));
    TRY(slai_write_buffer(ctx, m->chunk.tokens, 0, tokens, (size_t)n_tokens * 4));
    const int *tokens_dev = (const int *)m->chunk.tokens->dptr;
    SLAI_HIP_TRY(ctx, hipEventRecord(m->loop.ev0, ctx->stream));
    // The matrix-core pass runs on the half-precision units with split activations; if one of them turns out to be
    // beyond the f16 range the whole pass is repeated in fp32 (it only writes the caches, so that is safe).
    bool split = gemm && ctx->prompt_split_f16 != 0 && ctx->split_flag && m->chunk_split_ok();
    for (;;) {
        if (split) SLAI_HIP_TRY(ctx, hipMemsetAsync(ctx->split_flag, 0, sizeof(int), ctx->stream));
        for (uint32_t i = 0; i < n_tokens; i += chunk) {
            const uint32_t n = std::min(chunk, n_tokens - i);
            if (gemm) TRY(m->enqueue_chunk_gemm(start_pos + i, n, tokens_dev + i, split));
            else TRY(m->enqueue_chunk(start_pos + i, n, tokens_dev + i));
        }
        SLAI_HIP_TRY(ctx, hipEventRecord(m->loop.ev1, ctx->stream));
        TRY(slai_synchronize(ctx));
        if (!split) break;
        int beyond = 0;
        SLAI_HIP_TRY(ctx, hipMemcpy(&beyond, ctx->split_flag, sizeof(int), hipMemcpyDeviceToHost));
        if (!beyond) break;
        ++m->prefill_fp32_repeats;
        split = false;
    }
    if (elapsed_ms) SLAI_HIP_TRY(ctx, hipEventElapsedTime(elapsed_ms, m->loop.ev0, m->loop.ev1));
    return SLAI_OK;
}

SLAI_EXPORT uint32_t slai_llama2_prefill_fp32_repeats(const slai_llama2 *m) { return m ? m->prefill_fp32_repeats : 0; }

SLAI_EXPORT int slai_llama2_kv_buffers(slai_llama2 *m, uint32_t layer, slai_buffer **key_cache, slai_buffer **value_cache) {
    if (!m || layer >= m->config.n_layers) return SLAI_E_ARG;
    if (key_cache) *key_cache = m->state.key_cache[layer].buf;
    if (value_cache) *value_cache = m->state.value_cache[layer].buf;
    return SLAI_OK;
}
SLAI_EXPORT int slai_llama2_logits_buffer(slai_llama2 *m, slai_buffer **logits) {
    if (!m || !logits) return SLAI_E_ARG;
    *logits = m->state.logits.buf;
    return SLAI_OK;
}

// =================================================================================================
// GPT-2 (models/gpt2/cpu.rs)
// =================================================================================================
struct Gpt2Layer {                   // gpt2/cpu.rs:67-89
    GpuTensor ln_1_g, ln_1_b, ln_2_g, ln_2_b;
    slai_qmat *c_attn_attn_w = nullptr; GpuTensor c_attn_attn_b;
    slai_qmat *c_attn_proj_w = nullptr; GpuTensor c_attn_proj_b;
    GpuTensor key_cache, value_cache;
    slai_qmat *c_mlp_fc_w = nullptr; GpuTensor c_mlp_fc_b;
    slai_qmat *c_mlp_proj_w = nullptr; GpuTensor c_mlp_proj_b;
};

struct slai_gpt2 {
    slai_ctx *ctx = nullptr;
    int kv_dtype = SLAI_KV_F32;
    slai_gpt2_params params{};
    std::vector<Gpt2Layer> layers;
    GpuTensor ln_f_g, ln_f_b;
    slai_qmat *wte = nullptr, *wpe = nullptr;   // lm_head is wte (gpt2/cpu.rs:196-197)
    GpuTensor layer_input, curr_768, curr_2304, curr_3072, curr_vocab;   // gpt2/cpu.rs:102-110
    DeviceLoop loop;
    size_t weight_bytes = 0;
    uint32_t attn_splits = 1;

    int load(const slai_gguf *g);
    int enqueue_fused(int sampler, int form = 0);   // 0: stop at the logits, 1: greedy pick + loop state, 2: temperature / top-p pick + loop state (one form only)
    int form_at(uint32_t) const { return 0; }

    // Prompt tokens in chunks of up to 32 on the matrix cores (see slai_llama2::enqueue_chunk_gemm); row-major x and qkv,
    // quad-major xn (normalised rows, then the attention output) and h.
    struct { GpuTensor x, xn, qkv, h; slai_buffer *positions = nullptr, *tokens = nullptr; bool ready = false; } chunk;
    bool chunk_gemm_supported() const;
    int chunk_reserve();
    bool chunk_split_ok() const;
    uint32_t prefill_fp32_repeats = 0;
    int enqueue_chunk_gemm(uint32_t pos0, uint32_t n, const int *tokens_dev, bool split_f16);
};

// Gpt2Params::from_gguf (gpt2/cpu.rs:37-48)
static int gpt2_params_from_gguf(slai_ctx *ctx, const Gguf &g, slai_gpt2_params *out) {
    slai_gpt2_params &params = *out;
    const GgufMetaValue *tok = g.meta("tokenizer.ggml.tokens");
    if (!tok) return set_error(ctx, SLAI_E_MISSING, "missing metadata key 'tokenizer.ggml.tokens'");
    if (tok->type != 9) return set_error(ctx, SLAI_E_TYPE, "unwrap: unexpected GGUF attribute type for 'tokenizer.ggml.tokens'");
    params.n_vocab = (uint32_t)tok->arr_len;
    TRY(meta_u32(ctx, g, "gpt2.context_length", &params.n_seq));
    TRY(meta_u32(ctx, g, "gpt2.embedding_length", &params.n_embd));
    TRY(meta_u32(ctx, g, "gpt2.attention.head_count", &params.n_head));
    TRY(meta_u32(ctx, g, "gpt2.block_count", &params.n_layer));
    TRY(meta_u32(ctx, g, "gpt2.feed_forward_length", &params.ff_len));
    // The reference reads attn_b from dimensions()[0] of a 1-D bias, which is 1 after the dim swap
    // (gpt2/cpu.rs:46 + gguf.rs:581); the forward needs 3*n_embd (:252-270).
    params.attn_b = 3 * params.n_embd;
    const uint32_t E = params.n_embd;
    if (!E || !params.n_head || E % params.n_head || (E / params.n_head) % 2 || E / params.n_head > 256 || !params.ff_len || !params.n_seq || !params.n_vocab)
        return set_error(ctx, SLAI_E_SHAPE, "inconsistent GPT-2 hyper-parameters");
    return SLAI_OK;
}

// The host-only check of a GPT-2 file (see llama2_check_gguf): gpt2/cpu.rs:118-190 unwraps where this returns a code.
static int gpt2_check_gguf(const Gguf &g, slai_gpt2_params *params, std::string &err) {
    slai_ctx scratch_ctx;
    if (int rc = gpt2_params_from_gguf(&scratch_ctx, g, params)) { err = scratch_ctx.err; return rc; }
    const uint64_t E = params->n_embd, F = params->ff_len;
    for (uint32_t l = 0; l < params->n_layer; ++l) {
        const std::string p = "blk." + std::to_string(l) + ".";
        const struct { const char *name; uint64_t r, k; } mats[] = {
            {"attn_qkv.weight", 3 * E, E}, {"attn_output.weight", E, E}, {"ffn_up.weight", F, E}, {"ffn_down.weight", E, F}};
        for (const auto &m : mats)
            if (int rc = check_matrix(g, p + m.name, true, m.r, m.k, err)) return rc;
        const struct { const char *name; uint64_t n; } vecs[] = {
            {"attn_norm.weight", E}, {"attn_norm.bias", E}, {"ffn_norm.weight", E}, {"ffn_norm.bias", E}, {"attn_qkv.bias", 3 * E},
            {"attn_output.bias", E}, {"ffn_up.bias", F}, {"ffn_down.bias", E}};
        for (const auto &v : vecs)
            if (int rc = check_vector(g, p + v.name, true, v.n, err)) return rc;
    }
    if (int rc = check_vector(g, "output_norm.weight", true, E, err)) return rc;
    if (int rc = check_vector(g, "output_norm.bias", true, E, err)) return rc;
    if (int rc = check_matrix(g, "token_embd.weight", true, params->n_vocab, E, err)) return rc;
    const GgufTensorInfo *wpe = g.find("position_embd.weight");
    if (!wpe) { err = "missing tensor 'position_embd.weight'"; return SLAI_E_MISSING; }
    if (wpe->dims[0] < params->n_seq) { err = "embedding shapes do not match the parameters"; return SLAI_E_SHAPE; }
    return check_matrix(g, "position_embd.weight", true, wpe->dims[0], E, err);
}

SLAI_EXPORT int slai_gpt2_check_gguf(const slai_gguf *g, char *err, size_t err_len) {
    if (!g) return copy_message(SLAI_E_ARG, "slai_gpt2_check_gguf: bad argument", err, err_len);
    slai_gpt2_params params{};
    std::string msg;
    const int rc = gpt2_check_gguf(g->g, &params, msg);
    return copy_message(rc, msg, err, err_len);
}

int slai_gpt2::load(const slai_gguf *gg) {
    const Gguf &g = gg->g;
    {
        std::string msg;
        if (int rc = gpt2_check_gguf(g, &params, msg)) return set_error(ctx, rc, msg);
    }
    const uint32_t E = params.n_embd;
    const int cdt = kv_dtype == SLAI_KV_F16 ? SLAI_DT_F16 : SLAI_DT_F32;
    layers.resize(params.n_layer);
    for (uint32_t l = 0; l < params.n_layer; ++l) {       // gpt2/cpu.rs:118-179
        Gpt2Layer &w = layers[l];
        const std::string p = "blk." + std::to_string(l) + ".";
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_norm.weight", true, E, &w.ln_1_g));
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_norm.bias", true, E, &w.ln_1_b));
        TRY(f32_vector_from_gguf(ctx, g, p + "ffn_norm.weight", true, E, &w.ln_2_g));
        TRY(f32_vector_from_gguf(ctx, g, p + "ffn_norm.bias", true, E, &w.ln_2_b));
        TRY(qmat_from_gguf(ctx, gg, p + "attn_qkv.weight", &w.c_attn_attn_w));
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_qkv.bias", true, 3 * E, &w.c_attn_attn_b));
        TRY(qmat_from_gguf(ctx, gg, p + "attn_output.weight", &w.c_attn_proj_w));
        TRY(f32_vector_from_gguf(ctx, g, p + "attn_output.bias", true, E, &w.c_attn_proj_b));
        TRY(qmat_from_gguf(ctx, gg, p + "ffn_up.weight", &w.c_mlp_fc_w));
        TRY(f32_vector_from_gguf(ctx, g, p + "ffn_up.bias", true, params.ff_len, &w.c_mlp_fc_b));
        TRY(qmat_from_gguf(ctx, gg, p + "ffn_down.weight", &w.c_mlp_proj_w));
        TRY(f32_vector_from_gguf(ctx, g, p + "ffn_down.bias", true, E, &w.c_mlp_proj_b));
        struct { slai_qmat *m; uint32_t r, c; } chk[] = {{w.c_attn_attn_w, 3 * E, E}, {w.c_attn_proj_w, E, E}, {w.c_mlp_fc_w, params.ff_len, E}, {w.c_mlp_proj_w, E, params.ff_len}};
        for (auto &c : chk)
            if (c.m->nrows != c.r || c.m->ncols != c.c) return set_error(ctx, SLAI_E_SHAPE, "layer " + std::to_string(l) + ": weight shape does not match the parameters");
        TRY(GpuTensor::matrix(ctx, E, params.n_seq, STORAGE, &w.key_cache, cdt));
        TRY(GpuTensor::matrix(ctx, E, params.n_seq, STORAGE, &w.value_cache, cdt));
        for (slai_qmat *m : {w.c_attn_attn_w, w.c_attn_proj_w, w.c_mlp_fc_w, w.c_mlp_proj_w}) {
            weight_bytes += m->bytes;
            // activation slots of the 64-row-tile GEMV (one launch per matrix here); must exist before a graph is captured
            if (gemv_is_rowtile(ctx, m)) TRY(gemv_scratch_reserve(ctx, (size_t)((m->nrows + 63) / 64) * (m->ncols + m->ncols / 16)));
        }
        weight_bytes += (size_t)(4 * E + 3 * E + E + params.ff_len + E) * 4;
    }
    TRY(f32_vector_from_gguf(ctx, g, "output_norm.weight", true, E, &ln_f_g));
    TRY(f32_vector_from_gguf(ctx, g, "output_norm.bias", true, E, &ln_f_b));
    TRY(qmat_from_gguf(ctx, gg, "token_embd.weight", &wte));
    TRY(qmat_from_gguf(ctx, gg, "position_embd.weight", &wpe));
    if (gemv_is_rowtile(ctx, wte)) TRY(gemv_scratch_reserve(ctx, (size_t)((wte->nrows + 63) / 64) * (wte->ncols + wte->ncols / 16)));
    if (wte->nrows != params.n_vocab || wte->ncols != E || wpe->ncols != E || wpe->nrows < params.n_seq)
        return set_error(ctx, SLAI_E_SHAPE, "embedding shapes do not match the parameters");
    weight_bytes += wte->bytes + 2 * (size_t)E * 4;
    TRY(GpuTensor::vector(ctx, E, STORAGE, &layer_input));
    TRY(GpuTensor::vector(ctx, E, STORAGE, &curr_768));
    TRY(GpuTensor::vector(ctx, params.attn_b, STORAGE, &curr_2304));
    TRY(GpuTensor::vector(ctx, params.ff_len, STORAGE, &curr_3072));
    TRY(GpuTensor::vector(ctx, params.n_vocab, STORAGE | COPY_SRC | MAP_READ, &curr_vocab));
    attn_splits = pick_attn_splits(ctx, params.n_head, params.n_seq);
    TRY(ensure_attn_scratch(ctx, attention_scratch_floats(params.n_head, E / params.n_head, attn_splits)));
    TRY(loop_init(ctx, loop, params.n_seq + 1));
    return slai_synchronize(ctx);
}

// gpt2/cpu.rs:224-383 as fused kernels (LayerNorm eps 1e-5: ops/layernorm.rs:105)
int slai_gpt2::enqueue_fused(int sampler, int) {
    DecodeState *ds = (DecodeState *)loop.state->dptr;
    const uint32_t E = params.n_embd;
    float *x = (float *)layer_input.buf->dptr, *att_out = (float *)curr_768.buf->dptr, *qkv = (float *)curr_2304.buf->dptr,
          *h = (float *)curr_3072.buf->dptr, *logits = (float *)curr_vocab.buf->dptr;
    const float eps = 1.0e-5f;
    // :227-228 wte[:,tok] + wpe[:,pos]
    SLAI_HIP_TRY(ctx, launch_embed(ctx->stream, wte, &ds->token, wpe, &ds->pos, E, x));
    for (uint32_t l = 0; l < params.n_layer; ++l) {
        Gpt2Layer &w = layers[l];
        {   // :235-255 LayerNorm*g+b, qkv GEMV + bias
            GemvCall c;
            c.m[0] = w.c_attn_attn_w; c.out[0] = qkv; c.bias[0] = (const float *)w.c_attn_attn_b.buf->dptr; c.flags[0] = GEMV_BIAS; c.x = x;
            c.prologue = PRO_LAYERNORM; c.norm_w = (const float *)w.ln_1_g.buf->dptr; c.norm_b = (const float *)w.ln_1_b.buf->dptr; c.eps = eps;
            TRY(gemv_call(ctx, c, "gpt2 qkv"));
        }
        {   // :263-290 split q/k/v, cache write, attention with kv_mul = 1
            AttnLaunch a{};
            a.q = qkv; a.knew = qkv + E; a.vnew = qkv + 2 * E;
            a.kcache = w.key_cache.buf->dptr; a.vcache = w.value_cache.buf->dptr; a.kv_f16 = kv_dtype == SLAI_KV_F16;
            a.n_heads = params.n_head; a.kv_mul = 1; a.head_size = E / params.n_head; a.kv_dim = E; a.seq_len = params.n_seq;
            a.pos_ptr = (const uint32_t *)&ds->pos;
            a.rope_variant = -1; a.rope_base = 0.0f;
            a.out = att_out; a.scratch = ctx->attn_scratch; a.n_splits = attn_splits;
            hipError_t e = launch_attention(ctx->stream, a);
            if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, "attention: unsupported head size or context length");
            SLAI_HIP_TRY(ctx, e);
        }
        {   // :302-312 projection + bias + residual
            GemvCall c;
            c.m[0] = w.c_attn_proj_w; c.out[0] = x; c.bias[0] = (const float *)w.c_attn_proj_b.buf->dptr; c.flags[0] = GEMV_BIAS | GEMV_ACCUM; c.x = att_out;
            TRY(gemv_call(ctx, c, "gpt2 attn proj"));
        }
        {   // :318-343 LayerNorm*g+b, fc GEMV + bias, GELU
            GemvCall c;
            c.m[0] = w.c_mlp_fc_w; c.out[0] = h; c.bias[0] = (const float *)w.c_mlp_fc_b.buf->dptr; c.flags[0] = GEMV_BIAS | GEMV_GELU; c.x = x;
            c.prologue = PRO_LAYERNORM; c.norm_w = (const float *)w.ln_2_g.buf->dptr; c.norm_b = (const float *)w.ln_2_b.buf->dptr; c.eps = eps;
            TRY(gemv_call(ctx, c, "gpt2 mlp fc"));
        }
        {   // :353-360 projection + bias + residual
            GemvCall c;
            c.m[0] = w.c_mlp_proj_w; c.out[0] = x; c.bias[0] = (const float *)w.c_mlp_proj_b.buf->dptr; c.flags[0] = GEMV_BIAS | GEMV_ACCUM; c.x = h;
            TRY(gemv_call(ctx, c, "gpt2 mlp proj"));
        }
    }
    {   // :366-379 final LayerNorm*g+b, lm_head = wte
        GemvCall c;
        c.m[0] = wte; c.out[0] = logits; c.x = x;
        c.prologue = PRO_LAYERNORM; c.norm_w = (const float *)ln_f_g.buf->dptr; c.norm_b = (const float *)ln_f_b.buf->dptr; c.eps = eps;
        TRY(gemv_call(ctx, c, "gpt2 lm_head"));
    }
    if (sampler == 1)
        SLAI_HIP_TRY(ctx, launch_argmax(ctx->stream, logits, params.n_vocab, nullptr, ds, (const int *)loop.prompt->dptr, (int *)loop.out_tokens->dptr));
    else if (sampler == 2)
        SLAI_HIP_TRY(ctx, launch_sample(ctx->stream, logits, params.n_vocab, 0.0f, 0.0f, 0.0f, ctx->sampler_scratch, nullptr, ds, (const int *)loop.prompt->dptr,
                                        (int *)loop.out_tokens->dptr));
    return SLAI_OK;
}

bool slai_gpt2::chunk_gemm_supported() const {
    const uint32_t hs = params.n_embd / params.n_head;
    if ((hs != 64 && hs != 128) || params.n_embd % 8 || params.n_embd > 16384) return false;
    for (const Gpt2Layer &w : layers)
        for (const slai_qmat *m : {w.c_attn_attn_w, w.c_attn_proj_w, w.c_mlp_fc_w, w.c_mlp_proj_w})
            if (!gemm_chunk_supports(m)) return false;
    return true;
}

int slai_gpt2::chunk_reserve() {
    if (chunk.ready) return SLAI_OK;
    if (ctx->capturing) return set_error(ctx, SLAI_E_STATE, "prompt chunk buffers must be reserved before graph capture");
    const uint32_t E = params.n_embd;
    TRY(GpuTensor::matrix(ctx, E, 32, STORAGE, &chunk.x));
    TRY(GpuTensor::matrix(ctx, E, 32, STORAGE, &chunk.xn));
    TRY(GpuTensor::matrix(ctx, 3 * E, 32, STORAGE, &chunk.qkv));
    TRY(GpuTensor::matrix(ctx, params.ff_len, 32, STORAGE, &chunk.h));
    TRY(slai_buffer_create(ctx, (size_t)params.n_seq * 4, SLAI_DT_I32, STORAGE | COPY_DST, &chunk.positions));
    TRY(slai_buffer_create(ctx, (size_t)params.n_seq * 4, SLAI_DT_I32, STORAGE | COPY_DST, &chunk.tokens));
    std::vector<uint32_t> iota(params.n_seq);
    for (uint32_t i = 0; i < params.n_seq; ++i) iota[i] = i;
    TRY(slai_write_buffer(ctx, chunk.positions, 0, iota.data(), iota.size() * 4));
    chunk.ready = true;
    return SLAI_OK;
}

// gpt2/cpu.rs:225-383 for n <= 32 tokens at once, every projection on the matrix cores: embeddings, then per layer
// LayerNorm, qkv + bias, cache write, attention, projection + bias into the residual, LayerNorm, fc + bias, GELU,
// projection + bias into the residual.  No logits.
bool slai_gpt2::chunk_split_ok() const {
    for (const Gpt2Layer &w : layers)
        for (const slai_qmat *m : {w.c_attn_attn_w, w.c_attn_proj_w, w.c_mlp_fc_w, w.c_mlp_proj_w})
            if (!(m->wbound < 255.0f)) return false;
    return true;
}

int slai_gpt2::enqueue_chunk_gemm(uint32_t pos0, uint32_t n, const int *tokens_dev, bool split_f16) {
    if (n == 0 || n > 32 || pos0 + n > params.n_seq) return set_error(ctx, SLAI_E_ARG, "prompt chunk out of range");
    const uint32_t E = params.n_embd, F = params.ff_len;
    float *x = (float *)chunk.x.buf->dptr, *xn = (float *)chunk.xn.buf->dptr, *qkv = (float *)chunk.qkv.buf->dptr, *h = (float *)chunk.h.buf->dptr;
    const int *positions = (const int *)chunk.positions->dptr + pos0;
    const float eps = 1.0e-5f;
    int *const sf = split_f16 ? ctx->split_flag : nullptr;     // see slai_llama2::enqueue_chunk_gemm
    SLAI_HIP_TRY(ctx, launch_embed_rows(ctx->stream, wte, tokens_dev, n, E, x, E, wpe, positions));
    const auto gemm = [&](const slai_qmat *m, const float *bias, float *out, uint32_t out_stride, uint32_t flags, const float *xq, const char *who) -> int {
        GemmChunkParams p;
        p.nseg = 1; p.ncols = m->ncols; p.ncb = m->ncb; p.ngroups = m->ngroups; p.rows_log2 = m->rows_log2;
        p.x = xq; p.ntokens = n; p.split_f16 = split_f16;
        p.seg[0].W = m->dptr; p.seg[0].type = m->type; p.seg[0].nrows = m->nrows; p.seg[0].out = out; p.seg[0].out_stride = out_stride;
        p.seg[0].bias = bias; p.seg[0].flags = flags;
        hipError_t e = launch_gemm_chunk(ctx, p);
        if (e == hipErrorInvalidValue) return set_error(ctx, SLAI_E_SHAPE, std::string(who) + ": unsupported shape for the prompt-chunk GEMM");
        if (e != hipSuccess) return hip_fail(ctx, e, who);
        return SLAI_OK;
    };
    for (uint32_t l = 0; l < params.n_layer; ++l) {
        Gpt2Layer &w = layers[l];
        SLAI_HIP_TRY(ctx, launch_layernorm_quads(ctx->stream, xn, x, (const float *)w.ln_1_g.buf->dptr, (const float *)w.ln_1_b.buf->dptr, E, n, E, eps, sf));
        TRY(gemm(w.c_attn_attn_w, (const float *)w.c_attn_attn_b.buf->dptr, qkv, 3 * E, GEMV_BIAS, xn, "gpt2 qkv (prompt chunk)"));
        AttnLaunch a{};
        a.q = qkv; a.kcache = w.key_cache.buf->dptr; a.vcache = w.value_cache.buf->dptr; a.kv_f16 = kv_dtype == SLAI_KV_F16;
        a.n_heads = params.n_head; a.kv_mul = 1; a.head_size = E / params.n_head; a.kv_dim = E; a.seq_len = params.n_seq;
        a.pos_ptr = (const uint32_t *)positions;
        a.rope_variant = -1; a.rope_base = 0.0f;
        a.out = xn; a.scratch = nullptr; a.n_splits = 1;
        // keys and values of all tokens into the caches first (no rotation: learned positions), then the attention of each
        SLAI_HIP_TRY(ctx, launch_rope_store_batch(ctx->stream, a, qkv, qkv + E, qkv + 2 * E, n, 3 * E, 3 * E));
        SLAI_HIP_TRY(ctx, launch_attention_batch(ctx->stream, a, n, 3 * E, E, true, sf));
        TRY(gemm(w.c_attn_proj_w, (const float *)w.c_attn_proj_b.buf->dptr, x, E, GEMV_BIAS | GEMV_ACCUM, xn, "gpt2 attn proj (prompt chunk)"));
        SLAI_HIP_TRY(ctx, launch_layernorm_quads(ctx->stream, xn, x, (const float *)w.ln_2_g.buf->dptr, (const float *)w.ln_2_b.buf->dptr, E, n, E, eps, sf));
        TRY(gemm(w.c_mlp_fc_w, (const float *)w.c_mlp_fc_b.buf->dptr, h, F, GEMV_BIAS | GEMM_OUT_QUADS, xn, "gpt2 mlp fc (prompt chunk)"));
        SLAI_HIP_TRY(ctx, launch_gelu_quads(ctx->stream, h, 32 * F, n, sf));
        TRY(gemm(w.c_mlp_proj_w, (const float *)w.c_mlp_proj_b.buf->dptr, x, E, GEMV_BIAS | GEMV_ACCUM, h, "gpt2 mlp proj (prompt chunk)"));
    }
    return SLAI_OK;
}

SLAI_EXPORT int slai_gpt2_from_gguf(slai_ctx *ctx, const slai_gguf *g, int kv_dtype, slai_gpt2 **out) {
    if (!ctx || !g || !out) return SLAI_E_ARG;
    *out = nullptr;
    if (kv_dtype != SLAI_KV_F32 && kv_dtype != SLAI_KV_F16) return set_error(ctx, SLAI_E_ARG, "slai_gpt2_from_gguf: bad kv dtype");
    std::unique_ptr<slai_gpt2> m(new slai_gpt2());
    m->ctx = ctx; m->kv_dtype = kv_dtype;
    int rc = m->load(g);
    if (rc) { std::string keep = ctx->err; slai_gpt2_destroy(m.release()); ctx->err = keep; return rc; }
    *out = m.release();
    return SLAI_OK;
}

SLAI_EXPORT void slai_gpt2_destroy(slai_gpt2 *m) {
    if (!m) return;
    slai_ctx *ctx = m->ctx;
    slai_synchronize(ctx);
    loop_destroy(ctx, m->loop);
    for (auto &w : m->layers) {
        for (slai_qmat *q : {w.c_attn_attn_w, w.c_attn_proj_w, w.c_mlp_fc_w, w.c_mlp_proj_w}) slai_qmat_destroy(ctx, q);
        for (GpuTensor *t : {&w.ln_1_g, &w.ln_1_b, &w.ln_2_g, &w.ln_2_b, &w.c_attn_attn_b, &w.c_attn_proj_b, &w.key_cache, &w.value_cache,
                             &w.c_mlp_fc_b, &w.c_mlp_proj_b}) t->destroy(ctx);
    }
    slai_qmat_destroy(ctx, m->wte); slai_qmat_destroy(ctx, m->wpe);
    for (GpuTensor *t : {&m->ln_f_g, &m->ln_f_b, &m->layer_input, &m->curr_768, &m->curr_2304, &m->curr_3072, &m->curr_vocab}) t->destroy(ctx);
    for (GpuTensor *t : {&m->chunk.x, &m->chunk.xn, &m->chunk.qkv, &m->chunk.h}) t->destroy(ctx);
    for (slai_buffer *b : {m->chunk.positions, m->chunk.tokens}) if (b) slai_buffer_destroy(ctx, b);
    delete m;
}

SLAI_EXPORT int slai_gpt2_get_params(const slai_gpt2 *m, slai_gpt2_params *out) {
    if (!m || !out) return SLAI_E_ARG;
    *out = m->params;
    return SLAI_OK;
}
SLAI_EXPORT size_t slai_gpt2_weight_bytes(const slai_gpt2 *m) { return m ? m->weight_bytes : 0; }

SLAI_EXPORT int slai_gpt2_forward_logits(slai_gpt2 *m, uint32_t pos, uint32_t token, float *logits_out) {
    if (!m) return SLAI_E_ARG;
    slai_ctx *ctx = m->ctx;
    if (pos >= m->params.n_seq || token >= m->params.n_vocab) return set_error(ctx, SLAI_E_ARG, "slai_gpt2_forward_logits: position or token out of range");
    DecodeState ds{(int)pos, (int)token, 0, 0};
    TRY(slai_write_buffer(ctx, m->loop.state, 0, &ds, sizeof ds));
    TRY(m->enqueue_fused(false));
    TRY(slai_synchronize(ctx));
    if (logits_out) TRY(slai_read_buffer(ctx, m->curr_vocab.buf, 0, logits_out, (size_t)m->params.n_vocab * 4));
    return SLAI_OK;
}

SLAI_EXPORT int slai_gpt2_generate(slai_gpt2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos, uint32_t n_steps,
                                   int32_t *out_tokens, float *elapsed_ms) {
    if (!m) return SLAI_E_ARG;
    return generate_impl(m, m->ctx, m->loop, m->params.n_seq, m->params.n_vocab, prompt, n_prompt, start_pos, n_steps, out_tokens, elapsed_ms);
}
SLAI_EXPORT int slai_gpt2_generate_sampled(slai_gpt2 *m, const int32_t *prompt, uint32_t n_prompt, uint32_t start_pos, uint32_t n_steps,
                                           float temperature, float topp, uint64_t seed, int32_t *out_tokens, float *elapsed_ms) {
    if (!m) return SLAI_E_ARG;
    const SamplingParams sp{temperature, topp, seed};
    return generate_impl(m, m->ctx, m->loop, m->params.n_seq, m->params.n_vocab, prompt, n_prompt, start_pos, n_steps, out_tokens, elapsed_ms, &sp);
}

// 0: the ordinary loop, 2: matrix cores (see slai_llama2_prefill_supported)
SLAI_EXPORT int slai_gpt2_prefill_supported(const slai_gpt2 *m) { return m && m->ctx->prompt_gemm && m->chunk_gemm_supported() ? 2 : 0; }

// slai_llama2_prefill for GPT-2: fills the caches for positions start_pos .. start_pos + n_tokens - 1, 32 tokens per pass
// over the weights where every layer matrix has a tiled layout, token by token otherwise; no logits.
SLAI_EXPORT int slai_gpt2_prefill(slai_gpt2 *m, const int32_t *tokens, uint32_t n_tokens, uint32_t start_pos, uint32_t chunk, float *elapsed_ms) {
    if (!m) return SLAI_E_ARG;
    slai_ctx *ctx = m->ctx;
    if (elapsed_ms) *elapsed_ms = 0.0f;
    if (n_tokens == 0) return SLAI_OK;
    if (!tokens) return set_error(ctx, SLAI_E_ARG, "slai_gpt2_prefill: no tokens");
    if ((uint64_t)start_pos + n_tokens > m->params.n_seq) return set_error(ctx, SLAI_E_SHAPE, "slai_gpt2_prefill: would run past the context length");
    for (uint32_t i = 0; i < n_tokens; ++i)
        if (tokens[i] < 0 || (uint32_t)tokens[i] >= m->params.n_vocab) return set_error(ctx, SLAI_E_ARG, "slai_gpt2_prefill: token out of range");
    if (chunk > 64) return set_error(ctx, SLAI_E_ARG, "slai_gpt2_prefill: at most 64 tokens per chunk");
    const bool gemm = ctx->prompt_gemm && m->chunk_gemm_supported();
    if (chunk == 0) chunk = 32;
    if (chunk == 1 || !gemm) {
        std::vector<int32_t> prompt((size_t)start_pos + n_tokens, 0), picks(n_tokens);
        std::copy(tokens, tokens + n_tokens, prompt.begin() + start_pos);
        return generate_impl(m, ctx, m->loop, m->params.n_seq, m->params.n_vocab, prompt.data(), (uint32_t)prompt.size(), start_pos, n_tokens, picks.data(),
                             elapsed_ms);
    }
    if (chunk > 32) chunk = 32;
    TRY(m->chunk_reserve());
    TRY(slai_write_buffer(ctx, m->chunk.tokens, 0, tokens, (size_t)n_tokens * 4));
    const int *tokens_dev = (const int *)m->chunk.tokens->dptr;
    SLAI_HIP_TRY(ctx, hipEventRecord(m->loop.ev0, ctx->stream));
    // on the half-precision matrix cores first, repeated in fp32 when an activation was beyond f16 (see slai_llama2_prefill)
    bool split = ctx->prompt_split_f16 != 0 && ctx->split_flag && m->chunk_split_ok();
    for (;;) {
        if (split) SLAI_HIP_TRY(ctx, hipMemsetAsync(ctx->split_flag, 0, sizeof(int), ctx->stream));
        for (uint32_t i = 0; i < n_tokens; i += chunk) TRY(m->enqueue_chunk_gemm(start_pos + i, std::min(chunk, n_tokens - i), tokens_dev + i, split));
        SLAI_HIP_TRY(ctx, hipEventRecord(m->loop.ev1, ctx->stream));
        TRY(slai_synchronize(ctx));
        if (!split) break;
        int beyond = 0;
        SLAI_HIP_TRY(ctx, hipMemcpy(&beyond, ctx->split_flag, sizeof(int), hipMemcpyDeviceToHost));
        if (!beyond) break;
        ++m->prefill_fp32_repeats;
        split = false;
    }
    if (elapsed_ms) SLAI_HIP_TRY(ctx, hipEventElapsedTime(elapsed_ms, m->loop.ev0, m->loop.ev1));
    return SLAI_OK;
}

SLAI_EXPORT uint32_t slai_gpt2_prefill_fp32_repeats(const slai_gpt2 *m) { return m ? m->prefill_fp32_repeats : 0; }
