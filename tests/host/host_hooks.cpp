// Host-side test hooks: expose the host/device helper code of diffulex_amd/csrc to the
// CPU test-suite (compiled with the host compiler only; nothing here runs on a GPU).
#include <cstdint>
#include <vector>

#include "../../diffulex_amd/csrc/fp8_e4m3.h"
#include "../../diffulex_amd/csrc/partition.h"

extern "C" {

void hook_quantise_e4m3(const float* x, float scale, uint8_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = dfx::quantise_e4m3(x[i], scale);
}

void hook_e4m3_to_f32(const uint8_t* codes, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = dfx::e4m3fn_to_f32(codes[i]);
}

void hook_bf16_round(const float* x, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = dfx::f32_to_bf16_bits(x[i]);
}

int hook_effective_workgroups(int64_t total_units, int64_t n_items, int max_tiles, int n_wg) {
    return dfx::effective_workgroups(total_units, n_items, max_tiles, n_wg);
}

// Replays the persistent kernel's walk over its unit range on the host.  For workgroup w it
// appends one record per segment: {w, kv_head, seq, row_tile, tile0, tile1, complete, slot}.
// ctx/q_len/new_len: per-sequence lengths.  Returns the number of records (<= cap).
int64_t hook_walk_segments_masked(const int* ctx, const int* q_len, const int* new_len, int num_seqs, int h_kv,
                                  int group, int rows_per_tile, int n_wg, int block_causal, int dbs, int64_t* rec,
                                  int64_t cap);

int64_t hook_walk_segments(const int* ctx, const int* q_len, const int* new_len, int num_seqs, int h_kv, int group,
                           int rows_per_tile, int n_wg, int64_t* rec, int64_t cap) {
    return hook_walk_segments_masked(ctx, q_len, new_len, num_seqs, h_kv, group, rows_per_tile, n_wg, 0, 0, rec, cap);
}

// Every unit of one sequence in order: out[3 * u + {0, 1, 2}] = row tile, tile inside the item,
// tiles of the item.  Returns the number of units (<= cap entries are written).
int hook_enumerate_units(int ctx, int q_len, int new_len, int group, int rows_per_tile, int block_causal, int dbs,
                         int* out, int cap) {
    using namespace dfx;
    const SeqShape sh = make_seq_shape(ctx, q_len, new_len, group, rows_per_tile, block_causal != 0, dbs);
    for (int u = 0; u < sh.units && u < cap; ++u) locate_unit(sh, u, out[3 * u], out[3 * u + 1], out[3 * u + 2]);
    return sh.units;
}

int64_t hook_walk_segments_masked(const int* ctx, const int* q_len, const int* new_len, int num_seqs, int h_kv,
                                  int group, int rows_per_tile, int n_wg, int block_causal, int dbs, int64_t* rec,
                                  int64_t cap) {
    using namespace dfx;
    std::vector<SeqShape> sh(num_seqs);
    std::vector<int> prefix(num_seqs + 1, 0);
    for (int s = 0; s < num_seqs; ++s) {
        sh[s] = make_seq_shape(ctx[s], q_len[s], new_len[s], group, rows_per_tile, block_causal != 0, dbs);
        prefix[s + 1] = prefix[s] + sh[s].units;
    }
    const int per_head = prefix[num_seqs];
    const int64_t total = static_cast<int64_t>(per_head) * h_kv;
    int64_t n = 0;
    if (total == 0) return 0;
    for (int w = 0; w < n_wg; ++w) {
        const int64_t begin = wg_first_unit(w, total, n_wg), end = wg_first_unit(w + 1, total, n_wg);
        const WgSplit split = make_wg_split(total, n_wg);
        if (split.first(w) != begin || split.first(w + 1) != end) return -1;  // the two forms of the cut agree
        if (begin >= end) continue;
        int kvh = static_cast<int>(begin / per_head);
        const int rem = static_cast<int>(begin - static_cast<int64_t>(kvh) * per_head);
        int s = 0;
        while (!(prefix[s] <= rem && rem < prefix[s + 1])) ++s;
        int u = rem - prefix[s];
        int64_t pos = begin;
        while (pos < end) {
            int rt, tile0, n_tiles;
            locate_unit(sh[s], u, rt, tile0, n_tiles);
            const int64_t seg_end = pos + (n_tiles - tile0) < end ? pos + (n_tiles - tile0) : end;
            const int tile1 = tile0 + static_cast<int>(seg_end - pos);
            const bool complete = tile0 == 0 && tile1 == n_tiles;
            if (n < cap) {
                int64_t* r = rec + n * 8;
                r[0] = w; r[1] = kvh; r[2] = s; r[3] = rt; r[4] = tile0; r[5] = tile1; r[6] = complete;
                r[7] = partial_slot(w, pos, begin);
            }
            ++n;
            u += tile1 - tile0;
            pos = seg_end;
            if (pos >= end) break;
            if (u == sh[s].units) {
                u = 0;
                do {
                    if (++s == num_seqs) { s = 0; ++kvh; }
                } while (prefix[s + 1] == prefix[s]);
            }
        }
    }
    return n;
}

// What the workgroups that own pieces of item (kv_head, seq, row_tile) derive when they finish
// their piece: the slots of all pieces.  Returns the number of slots written (0: the item was
// not cut), -1 if the item is empty, -2 if the walk from some owner disagrees with wg_of_unit.
int hook_combine_slots(const int* ctx, const int* q_len, const int* new_len, int num_seqs, int h_kv, int group,
                       int rows_per_tile, int n_wg, int kvh, int s, int rt, int* slots, int cap) {
    using namespace dfx;
    int before = 0, all = 0;
    SeqShape mine{};
    for (int i = 0; i < num_seqs; ++i) {
        const SeqShape sh = make_seq_shape(ctx[i], q_len[i], new_len[i], group, rows_per_tile);
        if (i < s) before += sh.units;
        if (i == s) mine = sh;
        all += sh.units;
    }
    if (rt >= mine.n_row_tiles || mine.n_tiles == 0) return -1;
    const int64_t total = static_cast<int64_t>(all) * h_kv;
    const int64_t item_begin = static_cast<int64_t>(kvh) * all + before + static_cast<int64_t>(rt) * mine.n_tiles;
    const int64_t item_end = item_begin + mine.n_tiles;
    const int wa = wg_of_unit(item_begin, total, n_wg), wb = wg_of_unit(item_end - 1, total, n_wg);
    const WgSplit split = make_wg_split(total, n_wg);
    for (int me = wa; me <= wb; ++me) {
        if (split.first(me) >= split.first(me + 1)) continue;  // owns nothing
        int xa, xb;
        owners_of_units(split, me, item_begin, item_end - 1, xa, xb);
        if (xa != wa || xb != wb) return -2;
    }
    if (wa == wb) return 0;
    int n = 0;
    for (int w = wa; w <= wb; ++w) {
        const int64_t ws = wg_first_unit(w, total, n_wg), we = wg_first_unit(w + 1, total, n_wg);
        if (ws >= we) continue;
        const int64_t pb = ws > item_begin ? ws : item_begin;
        if (n < cap) slots[n] = partial_slot(w, pb, ws);
        ++n;
    }
    return n;
}

// The capacity sweep of a launch plan over one KV head (partition.h): n_w + 1 cut points into out
// (out[0] = 0, out[n_w] = the head's units); returns whether the last workgroup's share fits.
int hook_sweep_head(const int* prefix, int num_seqs, int n_w, int cap2, int* out) {
    using namespace dfx;
    out[0] = 0;
    const bool ok = sweep_head(prefix, num_seqs, n_w, cap2, out + 1, 1);
    out[n_w] = prefix[num_seqs];
    return ok ? 1 : 0;
}

// owners_of_units with a table of cut points (a plan's bounds): the first and last workgroup whose
// range meets units [first_unit, last_unit], walking from `me`.
void hook_owners_with_bounds(const int* bounds, int n_wg, int me, long long first_unit, long long last_unit, int* wa, int* wb) {
    using namespace dfx;
    WgSplit sp = make_wg_split(bounds[n_wg], n_wg);
    sp.bounds = bounds;
    owners_of_units(sp, me, first_unit, last_unit, *wa, *wb);
}
}
