// Who does what, and where every access lands, in the resident decode kernel (kernels_decode_persistent.hip): the roles
// of the workgroups in each phase of a layer, the byte offsets of the weights a lane requests, the pieces of a hand-off
// vector a lane takes, the rows of the hand-off buffers and of the caches, the blocks of LDS, the per-workgroup slots and
// trace rows.
//
// Everything here is plain integer arithmetic that compiles for the device and for the host: the kernel forms its
// addresses with these functions and nothing else, and a host program (tests/native/resident_bounds.cpp) walks every
// (workgroup, wave, lane, layer) of a launch through the same functions and checks each access against the allocation
// the loader makes for it.
#pragma once
#include "quant_tiled.h"

namespace slai {

// A 64-bit value from two 32-bit words.  The words are taken as unsigned on purpose: the lane-broadcast builtins return
// `int`, and an int with bit 31 set, widened on its way into a 64-bit "or", fills the upper word with ones -- a pointer
// rebuilt that way is wrong for every address whose lower word is 0x80000000 or above.
SLAI_HD constexpr uint64_t join_words(uint32_t lo, uint32_t hi) { return ((uint64_t)hi << 32) | (uint64_t)lo; }
static_assert(join_words(0x80000000u, 0x7fu) == 0x0000007f80000000ull, "the lower word must not be sign-extended");
static_assert(join_words((uint32_t)(int)0xffffffffu, 0u) == 0x00000000ffffffffull, "an int -1 as lower word stays 32 bits wide");

namespace plan {

constexpr uint32_t WG_THREADS = 1024, WG_WAVES = 16;

struct Shape {
    uint32_t dim, hidden, n_heads, n_layers, vocab, seq_len;
    uint32_t grid;            // workgroups of the launch (all resident)
    uint32_t qkv_units;       // units per head in the q / k / v phase: 7 (v in three, k and q in two each)
    uint32_t gu_rows;         // rows per unit of the gate / up phase, at most 64
    uint32_t neox;            // rotary pairs are (i, i + 64) of a head (NeoX) instead of (2i, 2i + 1)
};

SLAI_HD uint32_t umin(uint32_t a, uint32_t b) { return a < b ? a : b; }
SLAI_HD uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// The decomposition of a model: the grid is the number of 16-row tiles of the two projections into the residual (dim / 16
// = 8 per head), which is also seven q / k / v units (v in three, k and q in two each) plus the attention workgroup of
// every head, and the gate / up rows are spread evenly over it -- every workgroup has a role in every phase of a layer.
SLAI_HD Shape make_shape(uint32_t dim, uint32_t hidden, uint32_t n_heads, uint32_t n_layers, uint32_t vocab, uint32_t seq_len, uint32_t neox = 0) {
    Shape s{dim, hidden, n_heads, n_layers, vocab, seq_len, dim / 16u, 7u, 64u, neox};
    s.gu_rows = s.grid ? umin(64u, umax(1u, (hidden + s.grid - 1) / s.grid)) : 0u;
    return s;
}

// ---- supported shapes: what the kernel's index arithmetic assumes -------------------------------------------------------
SLAI_HD bool shape_ok(const Shape &s) {
    if (s.n_heads == 0 || s.n_heads % 8 || s.dim != s.n_heads * 128) return false;            // heads of 128, eight dies
    if (s.dim % 1024 || s.dim > 4096) return false;                                            // one wave per super-block of the input; two tiles of the output projection side by side
    if (s.hidden % 256 || s.hidden / 256 > 64) return false;                                   // sixteen waves x four super-blocks in the down projection
    if (s.grid != s.dim / 16 || s.qkv_units != 7 || (s.qkv_units + 1) * s.n_heads != s.grid) return false;   // a role for every workgroup in the first two phases
    if (s.gu_rows == 0 || s.gu_rows > 64 || (s.hidden + s.gu_rows - 1) / s.gu_rows != s.grid) return false;  // ... and in gate / up
    if (s.seq_len == 0 || s.seq_len > 65536 || s.n_layers == 0 || s.vocab == 0) return false;     // (a cache stays far below 4 GiB: cache_elem)
    return true;
}

// ---- hand-off buffers: one allocation of flow_floats() floats ------------------------------------------------------------
// xa [(n_layers + 1) x dim]: the input of layer l (row 0 unused: layer 0 reads the embedding row); row n_layers feeds
// the output matrix.  xb, xm [n_layers x dim]: attention output, residual after the attention.  hb [n_layers x hidden].
SLAI_HD uint64_t flow_floats(const Shape &s) { return (uint64_t)(6 * s.n_layers + 1) * s.dim + (uint64_t)s.n_layers * s.hidden; }
SLAI_HD uint64_t flow_xa(const Shape &s, uint32_t l) { return (uint64_t)l * s.dim; }
SLAI_HD uint64_t flow_xb(const Shape &s, uint32_t l) { return (uint64_t)(s.n_layers + 1) * s.dim + (uint64_t)l * s.dim; }
SLAI_HD uint64_t flow_xm(const Shape &s, uint32_t l) { return (uint64_t)(2 * s.n_layers + 1) * s.dim + (uint64_t)l * s.dim; }
// the rotated query, and the newest key (rotated) and value as the attention of this very token reads them (seg: 0 v, 1 k, 2 q)
SLAI_HD uint64_t flow_qkv(const Shape &s, uint32_t l, uint32_t seg) { return (uint64_t)((3 + seg) * s.n_layers + 1) * s.dim + (uint64_t)l * s.dim; }
SLAI_HD uint64_t flow_hb(const Shape &s, uint32_t l) { return (uint64_t)(6 * s.n_layers + 1) * s.dim + (uint64_t)l * s.hidden; }

// ---- per-workgroup slot (the staged input of a 64-row-unit phase, read back with scalar loads) ---------------------------
SLAI_HD uint32_t slot_stride(const Shape &s) { return s.dim + s.dim / 16 + 16; }             // floats
SLAI_HD uint64_t slot_floats(const Shape &s) { return (uint64_t)s.grid * slot_stride(s); }
SLAI_HD uint64_t slot_of(const Shape &s, uint32_t b) { return (uint64_t)b * slot_stride(s); }
// a multiplying wave reads 256 activations and 16 sums of its super-block from the slot
SLAI_HD uint32_t slot_x(uint32_t cb) { return cb * 256; }
SLAI_HD uint32_t slot_sums(const Shape &s, uint32_t cb) { return s.dim + cb * 16; }

// ---- dynamic LDS of a workgroup, in floats: two sets of partial[2][16][64] | red[16], used by its phases in turn -----------
SLAI_HD uint32_t lds_partial() { return 0; }
SLAI_HD uint32_t lds_red() { return 2 * WG_WAVES * 64; }
SLAI_HD uint32_t lds_set(uint32_t parity) { return parity * (lds_red() + 2 * WG_WAVES); }
// ... then, for the Q4_K phases on the matrix cores (mfma_q4k.h): a block of zeros, and per wave the staged activations
// of up to four super-blocks and room for the accumulators of two matrices on their way to the lanes that own the rows
constexpr uint32_t MQ_SB_BYTES = 1024 + 80, MQ_ZERO_BYTES = MQ_SB_BYTES, MQ_CS_BYTES = 1024;   // (zeros: a whole staged super-block of them)
constexpr uint32_t MQ_WAVE_BYTES = 4 * MQ_SB_BYTES + 4 * MQ_CS_BYTES;   // (two accumulator blocks per matrix of a gated pair)
SLAI_HD uint32_t lds_mq_zero() { return 2 * (lds_red() + 2 * WG_WAVES) * 4; }                          // bytes from here on
SLAI_HD uint32_t lds_mq_wave(uint32_t wave) { return lds_mq_zero() + MQ_ZERO_BYTES + wave * MQ_WAVE_BYTES; }
SLAI_HD uint32_t lds_mq_sb(uint32_t wave, uint32_t k) { return lds_mq_wave(wave) + k * MQ_SB_BYTES; }
SLAI_HD uint32_t lds_mq_cs(uint32_t wave) { return lds_mq_wave(wave) + 4 * MQ_SB_BYTES; }
SLAI_HD uint32_t lds_bytes(const Shape &) { return lds_mq_wave(WG_WAVES); }
SLAI_HD uint32_t lds_floats(const Shape &s) { return lds_bytes(s) / 4; }

// ---- the attention of a head over the cached positions: eight lanes per position for the scores (sixteen elements
// each), sixteen lanes per position for the values (eight elements each: the two positions the row of 16 lanes scored);
// a pass is 128 positions, eight per wave ---------------------------------------------------------------------------------
constexpr uint32_t ATT_PASS = 128;
SLAI_HD uint32_t att_k_pos(uint32_t tb, uint32_t wave, uint32_t lane) { return tb + wave * 8 + lane / 8; }
SLAI_HD uint32_t att_k_elem(uint32_t head, uint32_t lane) { return head * 128 + (lane & 7u) * 16; }
SLAI_HD uint32_t att_v_pos(uint32_t tb, uint32_t wave, uint32_t u, uint32_t lane) { return tb + wave * 8 + 2 * (lane / 16) + u; }
SLAI_HD uint32_t att_v_elem(uint32_t head, uint32_t lane) { return head * 128 + (lane & 15u) * 8; }
// element e of position t of a cache [seq_len x dim] (times the element size: below 4 GiB, shape_ok bounds seq_len and dim)
SLAI_HD uint32_t cache_elem(const Shape &s, uint32_t t, uint32_t e) { return t * s.dim + e; }
// The attention asks for the first att_ahead() cached positions before the query exists; the rows beyond them it walks at
// the rate one compute unit reads memory.  The workgroups of the head's q / k / v units (same die) therefore touch one
// word of every 128-byte line of those rows while they wait for the attention's result, so that the attention finds them
// in the die's L2.  Touch number w of a head: row att_ahead + w / (2 lines_per_row), key | value, line w % lines_per_row.
SLAI_HD constexpr uint32_t att_ahead(bool f16) { return (f16 ? 4u : 2u) * ATT_PASS; }
SLAI_HD uint32_t touch_lines_per_row(uint32_t elem_bytes) { return 128u * elem_bytes / 128u; }
SLAI_HD uint32_t touch_count(uint32_t pos, bool f16) { const uint32_t a = att_ahead(f16); return pos > a ? (pos - a) * 2u * touch_lines_per_row(f16 ? 2u : 4u) : 0u; }
SLAI_HD uint32_t touch_row(uint32_t w, bool f16) { return att_ahead(f16) + w / (2u * touch_lines_per_row(f16 ? 2u : 4u)); }
SLAI_HD bool touch_is_value(uint32_t w, bool f16) { return (w / touch_lines_per_row(f16 ? 2u : 4u)) & 1u; }
SLAI_HD uint32_t touch_byte(const Shape &s, uint32_t w, uint32_t head, bool f16) {
    const uint32_t es = f16 ? 2u : 4u;
    return cache_elem(s, touch_row(w, f16), head * 128u) * es + (w % touch_lines_per_row(es)) * 128u;
}
// touches are dealt to the tile waves of the head's unit workgroups: worker (unit t, wave, lane) starts at its index and strides
SLAI_HD uint32_t touch_first(uint32_t t, uint32_t tile_waves, uint32_t wave, uint32_t lane) { return (t * tile_waves + wave) * 64u + lane; }
SLAI_HD uint32_t touch_stride(const Shape &s, uint32_t tile_waves) { return s.qkv_units * tile_waves * 64u; }
// the control block: one 128-byte line per head (counters of the launches that hand q / k / v over per step), then the
// flag of a wait that gave up
SLAI_HD uint32_t counter_word(uint32_t head, uint32_t which = 0) { return head * 32 + which; }

// ---- time stamps: per workgroup 16 per layer (four per phase) and 8 for the output matrix -------------------------------
SLAI_HD uint32_t trace_stride(const Shape &s) { return 16 * s.n_layers + 8; }
SLAI_HD uint64_t trace_row(const Shape &s, uint32_t b) { return (uint64_t)b * trace_stride(s); }

// ---- roles ----------------------------------------------------------------------------------------------------------------
// A unit of a 64-row-unit phase: up to 64 rows of matrix `seg`; lane i of every wave owns row unit_row(u, i) (lanes past
// nrows repeat the last row and their results are dropped); wave w owns super-block w.  The rows are one run
// [row0, row0 + nrows), or two: lanes below `split` take row0 + i, the others row1 + (i - split).
struct RowUnit { uint32_t seg, row0, nrows, split, row1; };
SLAI_HD RowUnit run_unit(uint32_t seg, uint32_t row0, uint32_t nrows) { return RowUnit{seg, row0, nrows, nrows, 0u}; }
SLAI_HD uint32_t unit_row(const RowUnit &u, uint32_t lane) {
    const uint32_t i = umin(lane, u.nrows - 1);
    return i < u.split ? u.row0 + i : u.row1 + (i - u.split);
}

// q / k / v (segments 0: v, 1: k, 2: q): workgroup i < 7 * n_heads takes unit (i / 8) % 7 of head (i % 8) + 8 * (i / 56),
// so that all units of a head, and the head's attention workgroup qkv_workgroups + head, run on die i % 8 (their hand-off
// goes through that die's L2).  v is cut into three runs of rows.  q and k are cut in two halves that hold complete rotary
// pairs, because the workgroup that multiplies a unit also rotates it: rows 0..63 / 64..127 of the head for adjacent
// pairs, rows {0..31, 64..95} / {32..63, 96..127} for NeoX pairs -- the partner of lane i is lane i ^ 1, or i ^ 32.
SLAI_HD uint32_t qkv_workgroups(const Shape &s) { return s.qkv_units * s.n_heads; }
SLAI_HD uint32_t qkv_head(const Shape &s, uint32_t b) { return (b & 7u) + 8u * ((b >> 3) / s.qkv_units); }
SLAI_HD RowUnit qkv_unit(const Shape &s, uint32_t b) {
    const uint32_t t = (b >> 3) % s.qkv_units, head = qkv_head(s, b);
    const uint32_t nv = s.qkv_units - 4;                      // units of v: 3; k and q two each
    if (t < nv) {
        const uint32_t lo = 128u * t / nv, hi = 128u * (t + 1) / nv;
        return run_unit(0u, head * 128u + lo, hi - lo);
    }
    const uint32_t seg = t < nv + 2 ? 1u : 2u, part = (t - nv) & 1u;
    if (s.neox) return RowUnit{seg, head * 128u + 32u * part, 64u, 32u, head * 128u + 64u + 32u * part};
    return run_unit(seg, head * 128u + 64u * part, 64u);
}
SLAI_HD bool is_attention_workgroup(const Shape &s, uint32_t b) { return b >= qkv_workgroups(s) && b < qkv_workgroups(s) + s.n_heads; }
SLAI_HD uint32_t attention_head(const Shape &s, uint32_t b) { return b - qkv_workgroups(s); }

// gate / up: workgroup b < gu_units takes rows [b * gu_rows, ...) of both matrices
SLAI_HD uint32_t gu_units(const Shape &s) { return (s.hidden + s.gu_rows - 1) / s.gu_rows; }
SLAI_HD RowUnit gu_unit(const Shape &s, uint32_t b) { return run_unit(0u, b * s.gu_rows, umin(s.gu_rows, s.hidden - b * s.gu_rows)); }

// The two projections into the residual, in 16-row tiles (dim / 16 of them = the grid).  Down projection: workgroup b
// takes tile b.  Attention output projection: the workgroups of a head's q and k units take two tiles each, side by side
// on other waves -- their own, b, and the one of a workgroup that takes none: the head's three v units (which end last in
// the phase before and have asked for all their gate / up weights by then: their polls for the attention's result would
// return behind those) and the head's attention workgroup (which has just finished and holds no weights).
struct Tiles16 { uint32_t n, tile0, tile1; };      // (two named fields: an indexed pair would live in memory on the device)
SLAI_HD uint32_t tiles16_tile(const Tiles16 &t, uint32_t k) { return k == 0 ? t.tile0 : t.tile1; }
SLAI_HD uint32_t proj_tiles(const Shape &s) { return s.dim / 16; }
SLAI_HD Tiles16 down_tiles(const Shape &, uint32_t b) { return Tiles16{1u, b, b}; }
SLAI_HD bool takes_wo_tiles(const Shape &s, uint32_t b) { return b < qkv_workgroups(s) && (b >> 3) % s.qkv_units >= s.qkv_units - 4; }
SLAI_HD Tiles16 wo_tiles(const Shape &s, uint32_t b) {
    if (!takes_wo_tiles(s, b)) return Tiles16{0u, 0u, 0u};
    const uint32_t t = (b >> 3) % s.qkv_units, nv = s.qkv_units - 4, j = t - nv;       // j: which of the head's four q / k units
    return Tiles16{2u, b, j < nv ? b - 8u * (t - j) : qkv_workgroups(s) + qkv_head(s, b)};    // + v unit j's tile, or the attention's
}
// the row thread i < 16 * t.n of the workgroup finishes
SLAI_HD uint32_t tiles16_row(const Tiles16 &t, uint32_t i) { return 16u * tiles16_tile(t, (i >> 4) & 1u) + (i & 15u); }

// output matrix: 64-row tiles b, b + grid, ...
SLAI_HD uint32_t out_tiles(const Shape &s) { return (s.vocab + 63) / 64; }

// ---- weights: byte offsets inside one matrix, all below 2^32 (checked at load time) --------------------------------------
// 64-row tiles (quant_tiled.h, ROWS = 64, KQ = 1): the 16 bytes of piece P of (row, super-block cb) sit at
// tile64_piece0 + P * 1024, the 2-byte tail (Q6_K) at tile64_tail.
SLAI_HD uint32_t tile64_piece0(uint32_t row, uint32_t cb, uint32_t ncb, uint32_t unit_bytes) { return ((row >> 6) * ncb + cb) * unit_bytes + (row & 63u) * 16u; }
SLAI_HD uint32_t tile64_tail(uint32_t row, uint32_t cb, uint32_t ncb, uint32_t unit_bytes, uint32_t pieces) {
    return ((row >> 6) * ncb + cb) * unit_bytes + pieces * 1024u + (row & 63u) * 2u;
}
// 16-row tiles (ROWS = 16, KQ = 4): lane = 16 * kq + row; column group g of tile t
SLAI_HD uint32_t tile16_piece0(uint32_t tile, uint32_t g, uint32_t ngroups, uint32_t unit_bytes, uint32_t lane) { return (tile * ngroups + g) * unit_bytes + lane * 16u; }
SLAI_HD uint32_t tile16_tail(uint32_t tile, uint32_t g, uint32_t ngroups, uint32_t unit_bytes, uint32_t pieces, uint32_t lane) {
    return (tile * ngroups + g) * unit_bytes + pieces * 1024u + lane * 2u;
}
SLAI_HD uint32_t unit_bytes_of(int type) { return tiled_pieces(type) * 1024u + tiled_tail(type); }

// ---- the input of a 64-row-unit phase: wave w (< ncb) fetches the 256 values of super-block w, 16 bytes per lane, and ------
// leaves them (weighted) and their sums of 16 in its part of the workgroup's slot
SLAI_HD uint32_t wave_piece(uint32_t wave, uint32_t lane) { return wave * 64u + lane; }          // index of a 16-byte piece (4 floats)

// ---- the input of a 16-row-tile phase: lane (kq, j) of wave g holds x[cb * 256 + 16 i + j], i < 16, cb = 4 g + kq ---------
SLAI_HD uint32_t tile16_cb(uint32_t wave, uint32_t lane) { return wave * 4u + (lane >> 4); }
// first float of the lane's sixteen (lanes whose super-block does not exist read super-block 0 and drop it)
SLAI_HD uint32_t tile16_x0(uint32_t wave, uint32_t lane, uint32_t ncb) { const uint32_t cb = tile16_cb(wave, lane); return (cb < ncb ? cb : 0u) * 256u + (lane & 15u); }

// the same input for the matrix cores: wave g takes super-block 4 g + k (k < 4) as 64 pieces of 16 bytes, one per lane
SLAI_HD uint32_t tile16_sb(uint32_t wave, uint32_t k) { return wave * 4u + k; }
SLAI_HD uint32_t tile16_piece(uint32_t wave, uint32_t k, uint32_t lane) { return tile16_sb(wave, k) * 64u + lane; }

}  // namespace plan
}  // namespace slai
