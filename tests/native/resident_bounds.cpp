// Host walk of every address the resident decode kernel (slai_amd/csrc/kernels_decode_persistent.hip) forms, through
// the same functions the kernel calls (slai_amd/csrc/resident_plan.h), against the sizes of the allocations the loader
// makes (`slai_llama2::persistent_setup`, slai_qmat_create_layout).  Compiled by tests/test_resident_plan.py with g++.
//
// rb_audit walks, for every workgroup, wave and lane of a launch and every layer:
//   * the weight pieces and tails a lane requests in each phase, against the matrix's bytes;
//   * the piece of a hand-off vector a lane fetches, against the vector, and the words it writes into the workgroup's
//     slot, against the slot; what the wave reads back from there;
//   * the rows a workgroup writes into the hand-off vectors, q / k / v, the logits; counters, trace rows, the layer table;
//   * coverage: every output row of every matrix is produced exactly once per layer and every piece of an input vector is
//     staged exactly once per workgroup and phase;
//   * the 64-bit addresses: each buffer gets a fake base whose lower word lies below or above 0x80000000; the address is
//     rebuilt from its two words the way the kernel does and every access must fall inside [base, base + bytes).
// With `sign_extending_join` the lower word is widened as a signed int (the defect an earlier form of the kernel had):
// the audit must then report violations for bases at or above 0x80000000 in the lower word.
#include "quant_formats.h"
#include "quant_tiled.h"
#include "resident_plan.h"

#include <cstdio>
#include <string>
#include <vector>

using namespace slai;

namespace {

struct Region { const char *name; uint64_t base, bytes; };

struct Audit {
    bool sign_ext = false;
    uint64_t violations = 0, checks = 0;
    std::string first;
    uint64_t rebuilt(uint64_t base) const {
        const uint32_t lo = (uint32_t)base, hi = (uint32_t)(base >> 32);
        if (sign_ext) return ((uint64_t)hi << 32) | (uint64_t)(int64_t)(int32_t)lo;     // what `(uint64_t)readfirstlane(lo)` did
        return join_words(lo, hi);
    }
    // an access of `size` bytes at byte offset `off` of region r
    void touch(const Region &r, uint64_t off, uint64_t size, const char *what, uint32_t b, uint32_t wave, uint32_t lane, uint32_t layer) {
        ++checks;
        const uint64_t addr = rebuilt(r.base) + off;
        if (off + size > r.bytes || addr < r.base || addr + size > r.base + r.bytes) {
            if (!violations++) {
                char msg[320];
                snprintf(msg, sizeof msg, "%s: %s offset %llu + %llu beyond %llu bytes (address %#llx, base %#llx) at workgroup %u wave %u lane %u layer %u",
                         r.name, what, (unsigned long long)off, (unsigned long long)size, (unsigned long long)r.bytes, (unsigned long long)addr,
                         (unsigned long long)r.base, b, wave, lane, layer);
                first = msg;
            }
        }
    }
    void fail(const std::string &msg) { if (!violations++) first = msg; }
};

size_t matrix_bytes(int type, uint32_t nrows, uint32_t ncols, uint32_t rows_log2) { return tiled_bytes(tiled_geom(type, nrows, ncols, rows_log2)); }

// the weight requests of one lane for a unit of a 64-row-tile matrix
void walk_tile64(Audit &a, const Region &w, int type, const plan::RowUnit &u, uint32_t ncb, uint32_t b, uint32_t layer, std::vector<uint32_t> *row_count) {
    const uint32_t ub = plan::unit_bytes_of(type), pt = tiled_pieces(type);
    for (uint32_t wave = 0; wave < plan::WG_WAVES; ++wave) {
        if (wave >= ncb) continue;
        for (uint32_t lane = 0; lane < 64; ++lane) {
            const uint32_t row = plan::unit_row(u, lane);
            const uint32_t voff = plan::tile64_piece0(row, wave, ncb, ub);
            for (uint32_t p = 0; p < pt; ++p) a.touch(w, (uint64_t)voff + p * 1024u, 16, "weight piece", b, wave, lane, layer);
            if (tiled_tail(type)) a.touch(w, plan::tile64_tail(row, wave, ncb, ub, pt), 2, "weight tail", b, wave, lane, layer);
        }
    }
    if (row_count)
        for (uint32_t i = 0; i < u.nrows; ++i) {
            if (plan::unit_row(u, i) >= row_count->size()) { a.fail("a unit names a row past its matrix"); return; }
            ++(*row_count)[plan::unit_row(u, i)];
        }
}

// the input of a 64-row-unit phase: wave w < ncb fetches piece w * 64 + lane of the n-vector and of the norm weights,
// leaves the weighted values and their sums of 16 in the workgroup's slot, and reads its part of the slot back
void walk_stage64(Audit &a, const plan::Shape &s, const Region &x, const Region &norm, const Region &slots, uint32_t n, uint32_t ncb, uint32_t b, uint32_t layer) {
    std::vector<uint32_t> seen(n / 4, 0);
    const uint64_t slot0 = plan::slot_of(s, b) * 4;
    for (uint32_t wave = 0; wave < plan::WG_WAVES && wave < ncb; ++wave) {
        for (uint32_t lane = 0; lane < 64; ++lane) {
            const uint32_t piece = plan::wave_piece(wave, lane);
            a.touch(norm, (uint64_t)piece * 16, 16, "norm weights", b, wave, lane, layer);
            a.touch(x, (uint64_t)piece * 16, 16, "input piece", b, wave, lane, layer);
            a.touch(slots, slot0 + (uint64_t)piece * 16, 16, "slot values", b, wave, lane, layer);
            if ((lane & 3) == 0) a.touch(slots, slot0 + ((uint64_t)n + (piece >> 2)) * 4, 4, "slot sums", b, wave, lane, layer);
            if (piece < seen.size()) ++seen[piece];
            // what the wave reads back must be what the wave wrote
            if (piece * 4 < plan::slot_x(wave) || piece * 4 + 4 > plan::slot_x(wave) + 256) a.fail("a wave stages values outside the part of the slot it reads");
        }
        a.touch(slots, slot0 + (uint64_t)plan::slot_x(wave) * 4, 256 * 4, "slot read (activations)", b, wave, 0, layer);
        a.touch(slots, slot0 + ((uint64_t)n + wave * 16) * 4, 16 * 4, "slot read (sums)", b, wave, 0, layer);
        if (plan::slot_x(wave) + 256 > n) a.fail("a multiplying wave reads activations past the input");
    }
    for (uint32_t i = 0; i < seen.size(); ++i)
        if (seen[i] != 1) { a.fail("64-row-unit phase: a piece of the input is staged " + std::to_string(seen[i]) + " times"); break; }
    if ((uint64_t)n + n / 16 > plan::slot_stride(s)) a.fail("the slot is smaller than the staged input");
    if (ncb > plan::WG_WAVES) a.fail("more super-blocks than waves");
}

// a 16-row tile phase: the weights of the multiplying waves (tile k of the workgroup on waves k * ngroups ..), the sixteen
// floats of the n-vector each of their lanes takes, the residual values and the rows written; `rows` counts the latter
void walk_tile16(Audit &a, const Region &w, int type, const plan::Tiles16 &t, uint32_t ncb, uint32_t ngroups, const Region &x, uint32_t n, const Region &res,
                 const Region &out, std::vector<uint32_t> &rows, uint32_t b, uint32_t layer) {
    const uint32_t ub = plan::unit_bytes_of(type), pt = tiled_pieces(type);
    if (t.n > 2 || ngroups * t.n > plan::WG_WAVES) { a.fail("more column groups than waves"); return; }
    for (uint32_t k = 0; k < t.n; ++k) {
        std::vector<uint32_t> seen(n, 0), pieces_seen(n + 1024, 0);
        for (uint32_t wave = k * ngroups; wave < (k + 1) * ngroups; ++wave) {
            const uint32_t g = wave % ngroups;
            if (wave / ngroups != k) a.fail("wave to tile mapping");
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t voff = plan::tile16_piece0(plan::tiles16_tile(t, k), g, ngroups, ub, lane);
                for (uint32_t p = 0; p < pt; ++p) a.touch(w, (uint64_t)voff + p * 1024u, 16, "weight piece (16-row tile)", b, wave, lane, layer);
                if (tiled_tail(type)) a.touch(w, plan::tile16_tail(plan::tiles16_tile(t, k), g, ngroups, ub, pt, lane), 2, "weight tail (16-row tile)", b, wave, lane, layer);
                // the same input as the matrix cores take it: the lane's 16-byte piece of each of the wave's super-blocks
                for (uint32_t kk = 0; kk < 4; ++kk)
                    if (plan::tile16_sb(g, kk) < ncb) {
                        a.touch(x, (uint64_t)plan::tile16_piece(g, kk, lane) * 16, 16, "input piece (16-row tile)", b, wave, lane, layer);
                        if (plan::tile16_sb(g, kk) != plan::tile16_cb(g, kk * 16)) a.fail("the staged super-blocks are not those of the lanes");
                        for (uint32_t e = 0; e < 4; ++e) ++pieces_seen[plan::tile16_piece(g, kk, lane) * 4 + e];
                    }
                const uint32_t x0 = plan::tile16_x0(g, lane, ncb);
                const bool valid = plan::tile16_cb(g, lane) < ncb;
                for (uint32_t i = 0; i < 16; ++i) {
                    a.touch(x, ((uint64_t)x0 + 16 * i) * 4, 4, "input value (16-row tile)", b, wave, lane, layer);
                    if (valid && x0 + 16 * i < n && lane < 16 * (64 / 16)) ++seen[x0 + 16 * i];
                }
                a.touch(out, 0, 0, "", b, wave, lane, layer);
            }
        }
        // every value of the input reaches the 16-lane row that multiplies its super-block exactly once per tile
        for (uint32_t i = 0; i < n; ++i)
            if (pieces_seen[i] != 1) { a.fail("16-row-tile phase: input value " + std::to_string(i) + " is staged " + std::to_string(pieces_seen[i]) + " times"); break; }
        for (uint32_t i = 0; i < n; ++i)
            if (seen[i] != 1) { a.fail("16-row-tile phase: input value " + std::to_string(i) + " is taken " + std::to_string(seen[i]) + " times"); break; }
    }
    for (uint32_t i = 0; i < 16 * t.n; ++i) {                   // thread i of the workgroup: residual in, row out
        const uint32_t row = plan::tiles16_row(t, i);
        a.touch(res, (uint64_t)row * 4, 4, "residual load", b, 0, i, layer);
        a.touch(out, (uint64_t)row * 4, 4, "projection store", b, 0, i, layer);
        if (row < rows.size()) ++rows[row];
    }
}

}  // namespace

extern "C" {

// types: block formats of q, k, v, attention output, gate/up, down, output matrix.  handoff_heads: lines of the counter
// block (the runtime reserves max(n_heads, 256)).  high_bases: fake addresses with bit 31 of the lower word set.
// Returns the number of violations; `msg` receives the first one, `checked` the number of accesses looked at.
unsigned long long rb_audit(uint32_t dim, uint32_t hidden, uint32_t n_heads, uint32_t n_layers, uint32_t vocab, uint32_t seq_len, uint32_t grid,
                            int tq, int tk, int tv, int to, int tg, int td, int tout, uint32_t handoff_heads, int kv_bytes, int high_bases,
                            int sign_extending_join, int neox, char *msg, size_t msg_len, unsigned long long *checked) {
    Audit a;
    a.sign_ext = sign_extending_join != 0;
    plan::Shape s = plan::make_shape(dim, hidden, n_heads, n_layers, vocab, seq_len, neox ? 1u : 0u);
    if (grid) s.grid = grid;                                  // (a grid other than the plan's own must be refused)
    grid = s.grid;
    if (!plan::shape_ok(s)) a.fail("plan::shape_ok refuses the shape");
    else {
        // fake placement: 4 GiB apart, lower word 0x10000000 or 0x90000000 (+ a region-specific stagger)
        uint64_t next = high_bases ? 0x0000007f90000000ull : 0x0000007f10000000ull;
        const auto place = [&](const char *name, uint64_t bytes) { Region r{name, next, bytes}; next += 0x100000000ull + 0x01000000ull; return r; };
        const uint32_t ncb = dim / 256, ncb_h = hidden / 256, ng_o = ncb / 4, ng_d = (ncb_h + 3) / 4;
        const Region wq = place("wq", matrix_bytes(tq, dim, dim, 6)), wk = place("wk", matrix_bytes(tk, dim, dim, 6)), wv = place("wv", matrix_bytes(tv, dim, dim, 6));
        const Region wo = place("wo", matrix_bytes(to, dim, dim, 4)), wg = place("wgate", matrix_bytes(tg, hidden, dim, 6)), wu = place("wup", matrix_bytes(tg, hidden, dim, 6));
        const Region wd = place("wdown", matrix_bytes(td, dim, hidden, 4)), wout = place("wout", matrix_bytes(tout, vocab, dim, 6));
        const Region norm = place("norm vector", (uint64_t)dim * 4), xemb = place("embedding row", (uint64_t)dim * 4);
        const Region flow = place("hand-off buffers", plan::flow_floats(s) * 4), slots = place("slots", plan::slot_floats(s) * 4);
        const Region bias = place("bias vector", (uint64_t)dim * 4), logits = place("logits", (uint64_t)vocab * 4);
        const Region counters = place("counters", ((uint64_t)handoff_heads * 32 + 32) * 4);
        const Region trace = place("trace", (uint64_t)grid * plan::trace_stride(s) * 8);
        const Region layers = place("layer table", (uint64_t)n_layers * 14 * 16);
        const Region cache = place("cache", (uint64_t)seq_len * dim * kv_bytes);
        if ((wd.bytes | wout.bytes | wg.bytes) > 0xffffffffull) a.fail("a matrix beyond 4 GiB");
        // the four tile16 checks below assume what the loader checks: 16-row tiles with ceil(ncb / 4) groups
        if (tiled_geom(to, dim, dim, 4).ngroups != ng_o || tiled_geom(td, dim, hidden, 4).ngroups != ng_d) a.fail("group count of a projection differs from the kernel's");
        for (uint32_t l = 0; l < n_layers && a.violations < 8; ++l) {
            std::vector<uint32_t> rows_q(dim, 0), rows_k(dim, 0), rows_v(dim, 0), rows_h(hidden, 0), rows_o(dim, 0), rows_d(dim, 0);
            std::vector<uint32_t> heads_attended(n_heads, 0), units_of_head(n_heads, 0);
            std::vector<std::vector<uint32_t>> touched(n_heads, std::vector<uint32_t>(plan::touch_count(seq_len - 1, kv_bytes == 2), 0));
            // a hand-off vector of this layer as a region of its own size, placed inside the allocation
            const auto vec = [&](const char *name, uint64_t first_float, uint64_t n) {
                a.touch(flow, first_float * 4, n * 4, "hand-off row", 0, 0, 0, l);
                return Region{name, flow.base + first_float * 4, n * 4};
            };
            const Region xa = vec("xa", plan::flow_xa(s, l), dim), xb = vec("xb", plan::flow_xb(s, l), dim), xm = vec("xm", plan::flow_xm(s, l), dim);
            const Region hb = vec("hb", plan::flow_hb(s, l), hidden), xnext = vec("xa (next)", plan::flow_xa(s, l + 1), dim);
            const Region vnew = vec("newest value", plan::flow_qkv(s, l, 0), dim), knew = vec("newest key", plan::flow_qkv(s, l, 1), dim), qvec = vec("query", plan::flow_qkv(s, l, 2), dim);
            for (uint32_t b = 0; b < grid; ++b) {
                for (uint32_t tid = 0; tid < 14 * 4 && l + 1 < n_layers; ++tid) a.touch(layers, ((uint64_t)(l + 1) * 14 * 4 + tid) * 4, 4, "layer table word", b, 0, tid, l);
                for (uint32_t ph = 0; ph < 4; ++ph)
                    for (uint32_t k = 0; k < 4; ++k) a.touch(trace, (plan::trace_row(s, b) + 16 * l + 4 * ph + k) * 8, 8, "time stamp", b, 0, 0, l);
                if (b < plan::qkv_workgroups(s)) {
                    const plan::RowUnit u = plan::qkv_unit(s, b);
                    const uint32_t h = plan::qkv_head(s, b);
                    if (u.nrows == 0 || u.nrows > 64 || h >= n_heads || b % 8 != h % 8) { a.fail("q / k / v role"); continue; }
                    if (plan::unit_row(u, 0) / 128 != h || plan::unit_row(u, u.nrows - 1) / 128 != h) a.fail("a q / k / v unit leaves its head");
                    ++units_of_head[h];
                    walk_tile64(a, u.seg == 0 ? wv : (u.seg == 1 ? wk : wq), u.seg == 0 ? tv : (u.seg == 1 ? tk : tq), u, ncb, b, l, u.seg == 0 ? &rows_v : (u.seg == 1 ? &rows_k : &rows_q));
                    walk_stage64(a, s, l == 0 ? xemb : xa, norm, slots, dim, ncb, b, l);
                    // wave 0: lane t adds the bias of its row, rotates with a partner lane of the same unit, and stores
                    const Region &hand = u.seg == 0 ? vnew : (u.seg == 1 ? knew : qvec);
                    for (uint32_t t = 0; t < 64; ++t) {
                        const uint32_t row = plan::unit_row(u, t);
                        a.touch(bias, (uint64_t)row * 4, 4, "bias load", b, 0, t, l);
                        if (t >= u.nrows) continue;
                        a.touch(hand, (uint64_t)row * 4, 4, "q / k / v store", b, 0, t, l);
                        if (u.seg != 2) a.touch(cache, (uint64_t)plan::cache_elem(s, seq_len - 1, row) * kv_bytes, kv_bytes, "cache row store", b, 0, t, l);
                        if (u.seg != 0) {
                            // the partner of a rotary pair: element e ^ 1 (adjacent pairs) or e ^ 64 (NeoX) of the head, held
                            // by lane t ^ 1 or t ^ 32 of the same unit
                            const uint32_t partner = plan::unit_row(u, s.neox ? t ^ 32u : t ^ 1u);
                            if (partner != (s.neox ? row ^ 64u : row ^ 1u) || (s.neox ? t ^ 32u : t ^ 1u) >= u.nrows) a.fail("a rotary pair is split over units");
                        }
                    }
                    // the far cache rows of the head, touched into the die's L2 by the tile waves of its unit workgroups: every
                    // 128-byte line of every row beyond what the attention asks for ahead, of key and value, exactly once
                    {
                        const bool f16 = kv_bytes == 2;
                        const uint32_t T = seq_len - 1, n = plan::touch_count(T, f16), t = (b >> 3) % s.qkv_units;
                        for (uint32_t wave = 0; wave < ng_o; ++wave)
                            for (uint32_t lane = 0; lane < 64; ++lane)
                                for (uint32_t w = plan::touch_first(t, ng_o, wave, lane); w < n; w += plan::touch_stride(s, ng_o)) {
                                    const uint32_t byte = plan::touch_byte(s, w, h, f16);
                                    a.touch(cache, byte, 4, "cache line touched", b, wave, lane, l);
                                    const uint32_t row = plan::touch_row(w, f16), in_row = byte - plan::cache_elem(s, row, h * 128) * kv_bytes;
                                    if (row < plan::att_ahead(f16) || row >= T || byte % 128 != 0 || in_row >= 128 * kv_bytes) a.fail("a touch outside the head's far cache rows");
                                    ++touched[h][(size_t)w];
                                }
                    }
                } else if (plan::is_attention_workgroup(s, b)) {
                    const uint32_t h = plan::attention_head(s, b);
                    if (h >= n_heads || b % 8 != h % 8) { a.fail("attention role"); continue; }
                    ++heads_attended[h];
                    // cached positions: every pass of the deepest context, every wave and lane; per position, each element of
                    // the head's key once (eight lanes of sixteen) and of its value once (sixteen lanes of eight)
                    const uint32_t T = seq_len - 1;
                    std::vector<uint32_t> kseen((size_t)T * 128, 0), vseen((size_t)T * 128, 0);
                    for (uint32_t tb = 0; tb < T; tb += plan::ATT_PASS)
                        for (uint32_t wave = 0; wave < plan::WG_WAVES; ++wave)
                            for (uint32_t lane = 0; lane < 64; ++lane) {
                                const uint32_t t = plan::att_k_pos(tb, wave, lane), e = plan::att_k_elem(h, lane);
                                a.touch(cache, (uint64_t)plan::cache_elem(s, t < T ? t : 0, e) * kv_bytes, 16 * kv_bytes, "cached key", b, wave, lane, l);
                                if (e / 128 != h || e % 16) a.fail("key elements of another head");
                                if (t < T) for (uint32_t i = 0; i < 16; ++i) ++kseen[(size_t)t * 128 + e % 128 + i];
                                for (uint32_t uu = 0; uu < 2; ++uu) {
                                    const uint32_t tv = plan::att_v_pos(tb, wave, uu, lane), ev = plan::att_v_elem(h, lane);
                                    a.touch(cache, (uint64_t)plan::cache_elem(s, tv < T ? tv : 0, ev) * kv_bytes, 8 * kv_bytes, "cached value", b, wave, lane, l);
                                    if (ev / 128 != h) a.fail("value elements of another head");
                                    if (tv < T) for (uint32_t i = 0; i < 8; ++i) ++vseen[(size_t)tv * 128 + ev % 128 + i];
                                    // the weight of that position comes from the half of the lane's own row of 16 that scored it
                                    if (plan::att_k_pos(tb, wave, 16 * (lane / 16) + 8 * uu) != tv) a.fail("value lane takes the weight of another position");
                                }
                            }
                    for (size_t i = 0; i < kseen.size(); ++i)
                        if (kseen[i] != 1 || vseen[i] != 1) { a.fail("attention: an element of a cached position is read " + std::to_string(kseen[i]) + " / " + std::to_string(vseen[i]) + " times"); break; }
                    for (uint32_t lane = 0; lane < 64; ++lane) {
                        a.touch(qvec, (uint64_t)plan::att_k_elem(h, lane) * 4, 64, "query", b, 0, lane, l);
                        a.touch(knew, (uint64_t)plan::att_k_elem(h, lane) * 4, 64, "newest key", b, 0, lane, l);
                    }
                    for (uint32_t t = 0; t < 128; ++t) {
                        a.touch(vnew, ((uint64_t)h * 128 + t) * 4, 4, "newest value", b, t / 64, t % 64, l);
                        a.touch(xb, ((uint64_t)h * 128 + t) * 4, 4, "attention output", b, t / 64, t % 64, l);
                    }
                }
                a.touch(counters, (uint64_t)handoff_heads * 32 * 4, 4, "abort flag", b, 0, 0, l);
                {
                    const plan::Tiles16 wt = plan::wo_tiles(s, b), dt = plan::down_tiles(s, b);
if (plan::takes_wo_tiles(s, b) != (wt.n == 2) || (wt.n != 0 && wt.n != 2)) a.fail("the workgroups of the q and k units take two tiles of the output projection each, the others none");
                    walk_tile16(a, wo, to, wt, ncb, ng_o, xb, dim, l == 0 ? xemb : xa, xm, rows_o, b, l);
                    walk_tile16(a, wd, td, dt, ncb_h, ng_d, hb, hidden, xm, xnext, rows_d, b, l);
                }
                if (b < plan::gu_units(s)) {
                    const plan::RowUnit u = plan::gu_unit(s, b);
                    if (u.nrows == 0 || u.nrows > 64) { a.fail("gate / up role"); continue; }
                    walk_tile64(a, wg, tg, u, ncb, b, l, &rows_h);
                    walk_tile64(a, wu, tg, u, ncb, b, l, nullptr);
                    walk_stage64(a, s, xm, norm, slots, dim, ncb, b, l);
                    for (uint32_t t = 0; t < u.nrows; ++t) a.touch(hb, (uint64_t)(u.row0 + t) * 4, 4, "hb store", b, 0, t, l);
                }
            }
            for (uint32_t h = 0; h < n_heads; ++h)
                for (size_t w = 0; w < touched[h].size(); ++w)
                    if (touched[h][w] != 1) { a.fail("far cache rows of head " + std::to_string(h) + ": line " + std::to_string(w) + " is touched " + std::to_string(touched[h][w]) + " times"); h = n_heads; break; }
            const auto once = [&](const std::vector<uint32_t> &v, const char *what) {
                for (size_t i = 0; i < v.size(); ++i)
                    if (v[i] != 1) { a.fail(std::string(what) + ": row " + std::to_string(i) + " is produced " + std::to_string(v[i]) + " times in layer " + std::to_string(l)); return; }
            };
            once(rows_q, "q"); once(rows_k, "k"); once(rows_v, "v"); once(rows_h, "gate / up"); once(rows_o, "attention output projection"); once(rows_d, "down projection");
            once(heads_attended, "attention");
            for (uint32_t h = 0; h < n_heads; ++h)
                if (units_of_head[h] != s.qkv_units) a.fail("a head's counter would not reach its target");
        }
        // the output matrix
        std::vector<uint32_t> rows_l(vocab, 0);
        const Region xlast{"xa (last)", flow.base + plan::flow_xa(s, n_layers) * 4, (uint64_t)dim * 4};
        for (uint32_t b = 0; b < grid && a.violations < 8; ++b) {
            bool first = true;
            for (uint32_t tile = b; tile < plan::out_tiles(s); tile += grid) {
                const plan::RowUnit u = plan::run_unit(0u, tile * 64u, plan::umin(64u, vocab - tile * 64u));
                walk_tile64(a, wout, tout, u, ncb, b, n_layers, &rows_l);
                if (first) walk_stage64(a, s, xlast, norm, slots, dim, ncb, b, n_layers);
                first = false;
                for (uint32_t t = 0; t < u.nrows; ++t) a.touch(logits, (uint64_t)(u.row0 + t) * 4, 4, "logits store", b, 0, t, n_layers);
            }
            for (uint32_t k = 0; k < 5; ++k) a.touch(trace, (plan::trace_row(s, b) + 16 * n_layers + k) * 8, 8, "time stamp (output)", b, 0, 0, n_layers);
        }
        for (size_t i = 0; i < rows_l.size(); ++i)
            if (rows_l[i] != 1) { a.fail("logits: row " + std::to_string(i) + " is produced " + std::to_string(rows_l[i]) + " times"); break; }
    }
    if (msg && msg_len) snprintf(msg, msg_len, "%s", a.first.c_str());
    if (checked) *checked = a.checks;
    return a.violations;
}

// the decomposition plan::make_shape picks: grid, rows per gate / up unit, number of gate / up units
void rb_shape(uint32_t dim, uint32_t hidden, uint32_t n_heads, uint32_t grid, uint32_t *qkv_units /* receives the grid */, uint32_t *gu_rows, uint32_t *gu_units) {
    const plan::Shape s = plan::make_shape(dim, hidden, n_heads, 1, 64, 64);
    (void)grid;
    *qkv_units = s.grid; *gu_rows = s.gu_rows; *gu_units = plan::gu_units(s);
}

}  // extern "C"
