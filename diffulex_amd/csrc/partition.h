// Work partition of the paged-attention kernel, shared by the device code and by
// host-side tests (plain C++, no HIP dependency).
//
// Work is measured in "units": one unit is one KV tile (kTileTokens tokens of one KV head of
// one sequence) processed for one row tile of that sequence's queries.  Sequence s owns
//     units(s) = n_tiles(s) * n_row_tiles(s)
// consecutive units (row-tile major) -- fewer under the block-causal mask, where a row tile owns
// no fresh tile that none of its queries can see -- the sequences follow each other, and the whole list is
// repeated for every KV head.  The linear unit space [0, total) is cut into n_wg equal
// ranges, one per participating workgroup; wherever a cut falls inside a (sequence, head, row
// tile) item the sides produce partial results, which the workgroup that finishes its piece
// last merges.
#pragma once

#include <stdint.h>

#ifndef DFX_HD
#define DFX_HD inline
#endif

namespace dfx {

constexpr int kTileTokens = 64;

DFX_HD int ceil_div(int a, int b) { return (a + b - 1) / b; }

struct SeqShape {
    int ctx;        // cached tokens
    int q_len;      // query rows of the sequence
    int new_len;    // fresh K/V rows
    int n_ctx_tiles;
    int n_tiles;    // KV tiles: context tiles then fresh tiles (never mixed in one tile)
    int n_row_tiles;
    int units;
    // Block-causal mask with row tiles that do not straddle query heads (rph > 0): row tile k of a
    // head holds queries k * RT .. (k + 1) * RT - 1, which see no fresh token from (k + 1) * RT on,
    // so that row tile owns only its context tiles and its first min(n_new_tiles, (k + 1) * step)
    // fresh tiles.  rph == 0: every row tile owns all n_tiles.
    int rph;        // row tiles per query head, or 0
    int step;       // fresh tiles that become visible per row tile (RT / kTileTokens)
    int n_new_tiles;
    int ramp;       // row tiles of a head that see fewer than n_new_tiles fresh tiles
};

// Units of the first k row tiles of one query head (rph > 0).
DFX_HD int units_before_row_tile(const SeqShape& s, int k) {
    const int kr = k < s.ramp ? k : s.ramp;  // the ramp: step, 2 * step, ... fresh tiles
    return k * s.n_ctx_tiles + s.step * (kr * (kr + 1) / 2) + (k - kr) * s.n_new_tiles;
}

// KV tiles row tile rt of the sequence owns.
DFX_HD int tiles_of_row_tile(const SeqShape& s, int rt) {
    if (s.rph == 0) return s.n_tiles;
    const int k = rt % s.rph;
    return s.n_ctx_tiles + (k < s.ramp ? (k + 1) * s.step : s.n_new_tiles);
}

DFX_HD SeqShape make_seq_shape(int ctx, int q_len, int new_len, int group, int rows_per_tile,
                               bool block_causal = false, int dbs = 0) {
    SeqShape s;
    s.ctx = ctx > 0 ? ctx : 0;
    s.q_len = q_len > 0 ? q_len : 0;
    s.new_len = new_len > 0 ? new_len : 0;
    s.n_ctx_tiles = ceil_div(s.ctx, kTileTokens);
    s.n_new_tiles = ceil_div(s.new_len, kTileTokens);
    s.n_tiles = s.n_ctx_tiles + s.n_new_tiles;
    s.n_row_tiles = ceil_div(group * s.q_len, rows_per_tile);
    s.units = s.n_tiles * s.n_row_tiles;
    s.rph = 0;
    s.step = rows_per_tile / kTileTokens;
    s.ramp = 0;
    if (block_causal && dbs > 0 && s.q_len > 0 && s.q_len % rows_per_tile == 0 && rows_per_tile % dbs == 0 &&
        rows_per_tile % kTileTokens == 0) {
        s.rph = s.q_len / rows_per_tile;
        // row tile k sees (k + 1) * step fresh tiles while that is fewer than all of them
        const int full_from = ceil_div(s.n_new_tiles, s.step) - 1;  // first k that sees every fresh tile
        s.ramp = full_from < 0 ? 0 : (full_from < s.rph ? full_from : s.rph);
        s.units = group * units_before_row_tile(s, s.rph);
    }
    return s;
}

// Unit u of a sequence (0 <= u < units) -> its row tile, its tile inside that row tile's item and
// the number of tiles of that item.
DFX_HD void locate_unit(const SeqShape& s, int u, int& rt, int& tile, int& item_tiles) {
    if (s.rph == 0) {
        rt = u / s.n_tiles;
        tile = u - rt * s.n_tiles;
        item_tiles = s.n_tiles;
        return;
    }
    const int per_head = units_before_row_tile(s, s.rph);
    const int g = u / per_head;
    const int v = u - g * per_head;
    int lo = 0, hi = s.rph - 1;  // the largest k with units_before_row_tile(k) <= v
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (units_before_row_tile(s, mid) <= v) lo = mid;
        else hi = mid - 1;
    }
    rt = g * s.rph + lo;
    tile = v - units_before_row_tile(s, lo);
    item_tiles = tiles_of_row_tile(s, rt);
}

// How many of the n_wg workgroups of the launch take part.  Cutting an item into p pieces costs
// log2(p) rounds of a pairwise merge on top of the pieces' own tiles, so a workgroup should own at
// least about sqrt(tiles of the longest item) units (the best of 0.35 .. 2 times that, measured
// for batches of 1 .. 32 at 2K .. 32K), but there is never a reason to use fewer workgroups than
// there are items.  Small batches with long contexts are the case this matters for.  Integer
// arithmetic only: every workgroup (and the host-side tests) must arrive at the same number.
DFX_HD int effective_workgroups(int64_t total_units, int64_t n_items, int max_tiles, int n_wg) {
    int r = 0;  // floor(sqrt(max_tiles))
    while (static_cast<int64_t>(r + 1) * (r + 1) <= static_cast<int64_t>(max_tiles)) ++r;
    const int min_units = r > 4 ? r : 4;
    int64_t n = (total_units + min_units - 1) / min_units;
    if (n < n_items) n = n_items;
    if (n > n_wg) n = n_wg;
    return n < 1 ? 1 : static_cast<int>(n);
}

// First unit of workgroup w (w == n_wg gives total).
DFX_HD int64_t wg_first_unit(int w, int64_t total, int n_wg) { return (static_cast<int64_t>(w) * total) / n_wg; }

// The workgroup whose range contains unit u: the largest w with wg_first_unit(w) <= u.
DFX_HD int wg_of_unit(int64_t u, int64_t total, int n_wg) {
    return static_cast<int>(((u + 1) * n_wg - 1) / total);
}

// The same cut points without a 64-bit division at every use: with total = q * n_wg + r,
// floor(w * total / n_wg) = w * q + floor(w * r / n_wg), and w * r fits 32 bits (n_wg < 65536).
// `bounds`, if not null: the cut points come from a table instead (bounds[w] = first unit of workgroup
// w, bounds[n_wg] = total; strictly increasing), as a launch plan may place them (plan.h); q and r
// still describe the total.
struct WgSplit {
    int64_t q;
    uint32_t r;
    int n_wg;
    const int32_t* bounds;
    DFX_HD int64_t first(int w) const {
        if (bounds != nullptr) return bounds[w];
        return static_cast<int64_t>(w) * q + (static_cast<uint32_t>(w) * r) / static_cast<uint32_t>(n_wg);
    }
};

DFX_HD WgSplit make_wg_split(int64_t total, int n_wg) {
    WgSplit sp;
    sp.q = total / n_wg;
    sp.r = static_cast<uint32_t>(total - sp.q * n_wg);
    sp.n_wg = n_wg;
    sp.bounds = nullptr;
    return sp;
}

// The workgroups wa..wb whose ranges meet units [first_unit, last_unit] (wa = wg_of_unit(first_unit),
// wb = wg_of_unit(last_unit)), found by walking from a workgroup `me` that owns one of those units.
DFX_HD void owners_of_units(const WgSplit& sp, int me, int64_t first_unit, int64_t last_unit, int& wa, int& wb) {
    wa = me;
    while (sp.first(wa) > first_unit) --wa;
    wb = me;
    while (wb + 1 < sp.n_wg && sp.first(wb + 1) <= last_unit) ++wb;
}

// The cut points of one KV head by a sweep over its sequences (plan.h: mode 2 of a launch plan).
// Per workgroup, measured at the headline shape (timers in the attention kernel, least squares over
// the workgroups of a launch): 12.8 µs + 1.31 µs per unit + 5.0 µs per whole item + 6.7 µs if its
// range begins inside an item + 10.0 µs if it ends inside one (rms error 1.0 µs) -- a cut costs
// two workgroups as much as thirteen tiles.  In half units: a unit 2, a whole item kSweepWhole, a range
// that begins inside an item kSweepBegins, one that ends inside an item kSweepEnds.  With a capacity
// per workgroup the sweep gives every workgroup in turn what fits: the rest of the item the one
// before it cut, whole items while they fit, and a piece of the next item if a piece of at least
// kSweepMinPiece units fits and leaves at least as much (5: shorter pieces measured worse; the
// other constants within a third of these measure the same to 1 %, halved they lose 3-20 %).  It
// succeeds if the last workgroup's share fits as well.  `out`, if not null, receives the n_w - 1
// inner cut points (in units of the head), out_stride numbers apart.
constexpr int kSweepWhole = 8, kSweepBegins = 10, kSweepEnds = 15, kSweepMinPiece = 5;
DFX_HD bool sweep_head(const int* __restrict__ prefix, int num_seqs, int n_w, int cap2, int* __restrict__ out, int out_stride) {
    // One lane walks; 64 lanes walk for 64 capacities, so the walk is one flat loop whose every turn
    // either finishes the item under the cursor or closes a workgroup's range, written with selects
    // rather than nested branches (lanes that disagree on a branch run both sides one after the
    // other).  The item under the cursor is kept in registers (lo, hi: its first unit and the one
    // behind its last) and the beginning of the one after next is read a turn ahead.
    const int per_head = prefix[num_seqs];
    int pos = 0, i = 0, w = 0;
    int lo = 0, hi = prefix[1], next = num_seqs > 1 ? prefix[2] : per_head;
    int budget = cap2;
    bool fresh = true;  // the workgroup has taken nothing yet
    auto advance = [&] {
        ++i;
        lo = hi;
        hi = next;
        next = i + 2 <= num_seqs ? prefix[i + 2] : per_head;
    };
    while (w + 1 < n_w && i < num_seqs) {
        const int rest = hi - pos;          // units of the item from the cursor on (0: a sequence without units)
        const bool mid = lo < pos;          // the workgroup before has cut this item
        budget -= (fresh && mid) ? kSweepBegins : 0;
        const int need = rest > 0 ? 2 * rest + (mid ? 0 : kSweepWhole) : 0;
        if (need <= budget) {               // the rest of the item fits
            budget -= need;
            pos = hi;
            fresh = fresh && rest <= 0;
            advance();
            continue;
        }
        // it does not: a piece of it, if a piece of at least kSweepMinPiece units fits and leaves as much
        // (an item that was cut already is cut again wherever the capacity ends), and the range is closed
        const int room = (budget - kSweepEnds) / 2;
        const int again = room < 1 ? 1 : (room > rest ? rest : room);
        const int first = room < kSweepMinPiece ? 0
                          : (rest - room >= kSweepMinPiece ? room : (rest - kSweepMinPiece >= kSweepMinPiece ? rest - kSweepMinPiece : 0));
        pos += (fresh && mid) ? again : first;
        if (out != nullptr) out[w * out_stride] = pos;  // cut point w + 1
        ++w;
        budget = cap2;
        fresh = true;
    }
    if (out != nullptr)
        for (; w + 1 < n_w; ++w) out[w * out_stride] = pos;  // (workgroups without units: every sequence is taken)
    // the last workgroup takes what is left
    int used2 = 0;
    while (i < num_seqs) {
        const int rest = hi - pos;
        if (rest > 0) {
            used2 += 2 * rest + (lo < pos ? kSweepBegins : kSweepWhole);
            pos = hi;
        }
        advance();
    }
    return used2 <= cap2;
}

// ---- pairing partition (built by the plan kernel; never computed inside the attention kernels) ----
//
// When there are at most as many items as workgroups, equal ranges of the linear unit space cut
// nearly every item in two: every workgroup then stores one piece and merges another, each a
// round trip through memory on its critical path.  The pairing partition gives every item a home
// workgroup instead and only moves what must move: items are sorted by length, the k-th longest
// is paired with the k-th shortest (workgroups without an item count as empty items), and a long
// item donates its first d tiles to its partner, which processes them FIRST (its stored state is
// in memory long before the owner of the rest comes to merge) and then its own item.  A pair is
// only cut if its long item exceeds the launch's critical length M, the smallest value every pair
// can meet; cost constants below are in tiles (measured: a stored piece costs its workgroup about
// 1.5 tiles' time, a merged one 3, a second item's query rows and output 1.5).
constexpr int kPairCostMerge = 3;   // on the side that keeps the item's end
constexpr int kPairCostDonee = 3;   // on the side that takes the donated tiles: store + second item
constexpr int kPairSlack = 6;       // accept the pairing while M <= ceil(total / n_wg) + this
constexpr int kMaxPairItems = 1024;

// Critical length of one pair (l >= s tiles): uncut, or cut as evenly as the costs allow.
DFX_HD int pair_critical_length(int l, int s) {
    const int cut = (l + s + kPairCostMerge + kPairCostDonee + 1) / 2;
    return l < cut ? l : cut;
}

// Tiles the long item of a pair donates so that its owner meets M (0: the pair is not cut).
DFX_HD int pair_donation(int l, int s, int M) {
    (void)s;
    if (l <= M) return 0;
    int d = l + kPairCostMerge - M;       // owner: l - d + merge <= M
    if (d > l - 1) d = l - 1;             // the owner keeps at least the item's last tile
    return d < 1 ? 1 : d;
}

// A workgroup writes at most two partial results: slot 2w for a piece that starts at the
// first unit of its range, slot 2w+1 for a piece that starts later (it then necessarily
// runs to the end of the range).
DFX_HD int partial_slot(int w, int64_t piece_begin, int64_t wg_begin) {
    return 2 * w + (piece_begin != wg_begin ? 1 : 0);
}

}  // namespace dfx
