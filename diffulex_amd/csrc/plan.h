// The launch plan of the streaming paged-attention kernels, built once per decoding step and read
// by the attention launch of every layer (the lengths, block tables and strides are the same for
// all of them; only the q / k / v / cache base pointers change).
//
// Layout of the plan buffer:
//   PlanHeader                                  64 bytes
//   int32 prefix[num_seqs + 1]                  exclusive prefix of the sequences' units (per KV head)
//   int32 bounds[n_wg + 1]                      mode 2: first unit of every workgroup's range
//   WgWork work[n_wg]                           what every workgroup does (partition.h: linear ranges
//                                               of the unit space, or the pairing partition), and the
//                                               item of its first unit
//   int32 order[num_seqs]                       header.reordered: the sequence at every position of the
//                                               unit space (prefix[] then runs over positions)
//   BandDesc first[n_wg][kPlanFirst][NW]        the band descriptors of every workgroup's first units
//   UnitDesc units[capacity]                    one per unit, in each workgroup's processing order
//   BandDesc bands[capacity * NW]               one per unit and wave
// Two kernels fill it: paged_attn_plan_kernel (one workgroup: prefix, partition) and
// paged_attn_plan_fill_kernel (one workgroup per attention workgroup: the descriptors).  A plan
// whose header does not carry the magic number, or whose unit capacity was too small for the
// batch, is ignored by the attention kernels, which then plan for themselves.
#pragma once

#include "attn_stream.h"

namespace dfx {

struct PlanArgs {
    uint8_t* buf;
    int64_t capacity;   // unit descriptors
    int n_wg;           // workgroups of the attention launch
    int waves;          // waves per attention workgroup
    uint32_t signature;
    int allow_pairing;
    int equal_ranges;   // cut the unit space into equal ranges, as the attention kernels do without a plan
    int batch_order;    // keep the sequences in the batch's order in the unit space
};

// Where the plan cuts the linear unit space (mode 2): ranges of equal COST, a unit costing 2 and
// every sequence whose units begin in the range kPlanSeqCost more (a workgroup opens and closes an
// item there: query rows, first scores alone, rows written or a partial result through memory --
// time it cannot spend on tiles; equal ranges of units leave the workgroups with several short
// items behind), and a cut point within kPlanSnap units of such a beginning moved onto it (a piece
// of a few tiles costs two workgroups a partial result through memory for less work than that
// takes).  Both values are measured, not derived (MI355X, 64 sequences x 4 KV heads of 8-32 tiles
// on 256 workgroups: 0 / 0: 67.6 µs, 3 / 2: 65.9, 6 / 3: 65.2, 8 / 4: 65.2-65.8, 8 / 6: 69.7, 8 / 0:
// 73.5).  Only where a workgroup's range holds at most two items on average: with more, shorter
// items every cut point is near a beginning, the ranges become whole numbers of items, and that
// costs more than the cuts (800 items of 6 tiles: 77 µs against 70 with equal ranges; 400 items of
// 12 tiles: 58 against 63).
constexpr int kPlanSeqCost = 8;
constexpr int kPlanSnap = 4;
constexpr int kPlanMaxItemsPerWg = 2;
constexpr int kPlanMinUnitsPerWg = 8;  // below this the ranges stay equal
// LDS of paged_attn_plan_kernel, in ints: unit prefix and item prefix over the sequences, the sort keys
// and unit bases of the pairing partition (the cut points of the other partitions), scratch, then the
// unit prefix over the positions of the second order of the sequences, that order, and the cut points the
// sweep's candidates leave behind.
constexpr int kPlanCutsRoom = 8192;
constexpr int kPlanKernelLdsBytes = (2 * (kMaxSeqs + 1) + 2 * kMaxPairItems + 64 + (kMaxPairItems + 64) + kMaxPairItems + kPlanCutsRoom) * 4;

// Linear position of item y (0 <= y < items of the sequence) inside the sequence's units, and its tiles.
DFX_HD void item_of_sequence(const SeqShape& sh, int rt, int& offset, int& tiles) {
    tiles = tiles_of_row_tile(sh, rt);
    if (sh.rph == 0) {
        offset = rt * sh.n_tiles;
    } else {
        const int g = rt / sh.rph, k = rt - g * sh.rph;
        offset = g * units_before_row_tile(sh, sh.rph) + units_before_row_tile(sh, k);
    }
}

// Descending bitonic sort of n (a power of two) keys in LDS by all threads of the workgroup.
DFX_D void bitonic_sort_desc(uint32_t* keys, int n) {
    for (int k = 2; k <= n; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < n; i += blockDim.x) {
                const int ixj = i ^ j;
                if (ixj > i) {
                    const uint32_t x = keys[i], y = keys[ixj];
                    const bool up = (i & k) == 0;  // this pair sorts descending
                    if (up ? x < y : x > y) {
                        keys[i] = y;
                        keys[ixj] = x;
                    }
                }
            }
            __syncthreads();
        }
}

// Phase one, one workgroup of 512 threads: the unit prefix, the partition and every workgroup's work.
template <int RT>
__global__ void __launch_bounds__(512) paged_attn_plan_kernel(const KArgs a, const PlanArgs pa) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int* prefix = reinterpret_cast<int*>(smem);                         // [kMaxSeqs + 1]
    int* iprefix = prefix + kMaxSeqs + 1;                               // [kMaxSeqs + 1] items before a sequence
    uint32_t* keys = reinterpret_cast<uint32_t*>(iprefix + kMaxSeqs + 1);  // [kMaxPairItems]
    int* ubase = reinterpret_cast<int*>(keys + kMaxPairItems);          // [kMaxPairItems]
    int* misc = ubase + kMaxPairItems;                                  // [64]
    int* pprefix = misc + 64;                                           // [kMaxPairItems + 64]
    int* order2 = pprefix + kMaxPairItems + 64;                         // [kMaxPairItems]
    int* cuts = order2 + kMaxPairItems;                                 // [kPlanCutsRoom]
    PlanHeader* hdr = reinterpret_cast<PlanHeader*>(pa.buf);
    const PlanLayout lay = plan_layout(a.num_seqs, pa.n_wg, pa.capacity, pa.waves);
    int* g_prefix = reinterpret_cast<int*>(pa.buf + lay.prefix_off);
    WgWork* work = reinterpret_cast<WgWork*>(pa.buf + lay.work_off);
    const int tid = threadIdx.x;

    const UnitSummary summary = build_unit_prefix<RT>(a, prefix, misc);
    const int per_head = summary.per_head;
    const int64_t total = static_cast<int64_t>(per_head) * a.h_kv;
    const int64_t n_items = static_cast<int64_t>(summary.items) * a.h_kv;
    const int n_active = total == 0 ? 0
                         : a.fixed_wg ? a.n_wg
                                      : effective_workgroups(total, n_items, summary.max_tiles, a.n_wg);

    // items before each sequence (row tiles of sequences that have units)
    {
        int carry = 0;
        for (int base = 0; base < a.num_seqs; base += blockDim.x) {
            const int sq = base + tid;
            int r = 0;
            if (sq < a.num_seqs) {
                const SeqShape shp = load_seq_shape(a, sq, RT);
                r = shp.units > 0 ? shp.n_row_tiles : 0;
            }
            int tot;
            const int incl = block_inclusive_scan(r, misc, tot);
            if (sq < a.num_seqs) iprefix[sq + 1] = carry + incl;
            carry += tot;
        }
        if (tid == 0) iprefix[0] = 0;
        __syncthreads();
    }
    const int items_per_head = summary.items;

    // item x (KV head minor: the heads of one (sequence, row tile) are neighbours, and stay
    // neighbours in the sorted list, being equally long) -> its first unit and its tiles
    auto locate_item = [&](int x, int64_t& begin, int& tiles) {
        const int y = x / a.h_kv, kvh = x - y * a.h_kv;
        (void)items_per_head;
        int lo = 0, hi = a.num_seqs;  // the sequence with iprefix[s] <= y < iprefix[s + 1]
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (iprefix[mid + 1] <= y) lo = mid + 1;
            else hi = mid;
        }
        const SeqShape shp = load_seq_shape(a, lo, RT);
        int off;
        item_of_sequence(shp, y - iprefix[lo], off, tiles);
        begin = static_cast<int64_t>(kvh) * per_head + prefix[lo] + off;
    };

    // ---- pairing partition, if it applies --------------------------------------------------------
    const int m = n_active;
    bool pairing = pa.allow_pairing && total > 0 && n_items <= m && m <= kMaxPairItems && total >= m;
    bool placed = false;  // cut points placed by cost (mode 2)
    bool reordered = false;  // the sweep found the second order of the sequences better
    int critical = 0;
    if (pairing) {  // (uniform: every thread takes the same branch)
        int n_sort = 1;
        while (n_sort < m) n_sort <<= 1;
        for (int x = tid; x < n_sort; x += blockDim.x) {
            uint32_t key = 0;  // empty entry: sorts last
            if (x < n_items) {
                int64_t begin;
                int tiles;
                locate_item(x, begin, tiles);
                key = (static_cast<uint32_t>(tiles) << 10) | static_cast<uint32_t>(kMaxPairItems - 1 - x);
                if (tiles >= (1 << 21)) key = 0xffffffffu;  // (cannot be keyed: forces the fallback below)
            }
            keys[x] = key;
        }
        __syncthreads();
        bitonic_sort_desc(keys, n_sort);
        // the launch's critical length: the worst pair (k-th longest with k-th shortest)
        int worst = 0;
        for (int k = tid; 2 * k < m; k += blockDim.x) {
            const int l = static_cast<int>(keys[k] >> 10), s = static_cast<int>(keys[m - 1 - k] >> 10);
            const int c = (2 * k == m - 1) ? l : pair_critical_length(l, s);
            worst = max(worst, c);
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) worst = max(worst, __shfl_xor(worst, d));
        if ((tid & 63) == 0) misc[32 + (tid >> 6)] = worst;
        __syncthreads();
        for (int w = 0; w < static_cast<int>(blockDim.x >> 6); ++w) critical = max(critical, misc[32 + w]);
        __syncthreads();
        const int even = static_cast<int>((total + m - 1) / m);
        pairing = critical <= even + kPairSlack && keys[0] != 0xffffffffu;
    }

    if (pairing) {
        // unit counts per workgroup, then their exclusive prefix
        int carry = 0;
        for (int base = 0; base < m; base += blockDim.x) {
            const int k = base + tid;
            int count = 0;
            if (k < m) {
                const int kp = m - 1 - k;
                const int mine = static_cast<int>(keys[k] >> 10), other = static_cast<int>(keys[kp] >> 10);
                if (k < kp) count = mine - pair_donation(mine, other, critical);
                else if (k > kp) count = mine + pair_donation(other, mine, critical);
                else count = mine;
            }
            int tot;
            const int incl = block_inclusive_scan(count, misc, tot);
            if (k < m) ubase[k] = carry + incl - count;
            carry += tot;
        }
        __syncthreads();
        // Which workgroup gets which entry of the sorted list.  The KV heads of one sequence are
        // equally long, hence neighbours in the list, and read the same token rows of the cache at
        // the same time: they go to workgroups whose numbers differ by a multiple of m / h_kv (of 8,
        // the number of XCDs, at the usual sizes), i.e. onto the same XCD, behind the same L2 and TLB
        // -- where the equal ranges of the linear unit space put them too.
        const int heads = (a.h_kv > 0 && m % a.h_kv == 0) ? a.h_kv : 1;
        auto workgroup_of = [&](int entry) { return (entry % heads) * (m / heads) + entry / heads; };
        for (int k = tid; k < pa.n_wg; k += blockDim.x) {
            WgWork w;
            w.a0 = w.a1 = w.b0 = w.b1 = 0;
            w.partner = -1;
            w.ubase = 0;
            w.q0 = w.q_len = w.kvh = w.rt = 0;  // (the fill kernel enters them)
            w.pad[0] = w.pad[1] = 0;
            if (k >= m) {
                work[k] = w;
                continue;
            }
            {
                const int kp = m - 1 - k;
                const int mine = static_cast<int>(keys[k] >> 10), other = static_cast<int>(keys[kp] >> 10);
                int64_t my_begin = 0, other_begin = 0;
                int t;
                if (mine > 0) locate_item(kMaxPairItems - 1 - static_cast<int>(keys[k] & 1023u), my_begin, t);
                if (other > 0) locate_item(kMaxPairItems - 1 - static_cast<int>(keys[kp] & 1023u), other_begin, t);
                if (k < kp) {  // the long item's owner keeps its end
                    const int d = pair_donation(mine, other, critical);
                    w.a0 = my_begin + d;
                    w.a1 = my_begin + mine;
                    if (d > 0) w.partner = workgroup_of(kp);
                } else if (k > kp) {  // the partner: donated tiles first, then its own item
                    const int d = pair_donation(other, mine, critical);
                    w.a0 = other_begin;
                    w.a1 = other_begin + d;
                    w.b0 = my_begin;
                    w.b1 = my_begin + mine;
                    if (d > 0) w.partner = workgroup_of(kp);
                } else {
                    w.a0 = my_begin;
                    w.a1 = my_begin + mine;
                }
                w.ubase = ubase[k];
            }
            work[workgroup_of(k)] = w;
        }
    } else {
        const WgSplit split = make_wg_split(total > 0 ? total : 1, n_active > 0 ? n_active : 1);
        int32_t* g_bounds = reinterpret_cast<int32_t*>(pa.buf + lay.bounds_off);
        int* bounds = reinterpret_cast<int*>(keys);  // [n_wg + 1] (the pairing partition's arrays are free here)
        static_assert(kMaxPairItems + kMaxPairItems >= 1025, "room for the cut points of up to 1024 workgroups");
        placed = !pa.equal_ranges && n_active > 1 && n_active <= 1024 && total >= static_cast<int64_t>(kPlanMinUnitsPerWg) * n_active &&
                 n_items <= static_cast<int64_t>(kPlanMaxItemsPerWg) * n_active && total < (1ll << 30);
        // the sweep, where the workgroups divide evenly among the KV heads (whose sequences are the same):
        // 64 capacities, from the mean load (no cuts) upwards in steps of 1 %, one per lane; the smallest
        // that succeeds gives the cut points, which every KV head then uses.
        //
        // The sweep takes the sequences in the order they have in the unit space, and what it can do
        // depends on that order: a long sequence must be cut, and what is left of it fills a workgroup
        // only together with a short neighbour.  So the unit space may list the sequences in another
        // order than the batch does (the attention kernels never see the difference: their descriptors
        // name the sequence).  A second order is swept next to the batch's own -- the k-th longest
        // sequence followed by the k-th shortest, whose units add up to about two workgroups' shares: one
        // cut per pair at most -- and the order whose smallest capacity is lower is taken (measured at 64
        // sequences x 4 KV heads of 8-32 tiles on 256 workgroups: 27 cut items per head and the last
        // workgroup done after 58 us in the batch's order, 16 and 54 in the second).
        bool swept = false;
        const int n_w = a.h_kv > 0 ? n_active / a.h_kv : 0;
        if (placed && blockDim.x == 512 && n_w >= 2 && n_w * a.h_kv == n_active && n_w <= 1023) {  // (uniform)
            int nonempty = 0;
            for (int sq = tid; sq < a.num_seqs; sq += blockDim.x) nonempty += prefix[sq + 1] > prefix[sq];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) nonempty += __shfl_xor(nonempty, d);
            if ((tid & 63) == 0) misc[40 + (tid >> 6)] = nonempty;
            __syncthreads();
            nonempty = 0;
            for (int w = 0; w < static_cast<int>(blockDim.x >> 6); ++w) nonempty += misc[40 + w];
            const int base2 = (2 * per_head + kSweepWhole * nonempty + n_w - 1) / n_w;
            const bool two = !pa.batch_order && a.num_seqs >= 3 && a.num_seqs <= kMaxPairItems && per_head < (1 << 20);
            if (two) {  // (uniform)
                int n_sort = 1;
                while (n_sort < a.num_seqs) n_sort <<= 1;
                for (int x = tid; x < n_sort; x += blockDim.x)  // (a key of 0 sorts behind every sequence)
                    keys[x] = x < a.num_seqs ? (static_cast<uint32_t>(prefix[x + 1] - prefix[x]) << 11) | static_cast<uint32_t>(kMaxPairItems - x) : 0u;
                __syncthreads();
                bitonic_sort_desc(keys, n_sort);
                for (int p = tid; p < a.num_seqs; p += blockDim.x) {
                    const int k = p >> 1;
                    const int e = (p & 1) ? a.num_seqs - 1 - k : k;  // even positions: the longest ones, odd positions: the shortest
                    order2[p] = kMaxPairItems - static_cast<int>(keys[e] & 2047u);
                }
                __syncthreads();
                int carry = 0;
                for (int base = 0; base < a.num_seqs; base += blockDim.x) {
                    const int p = base + tid;
                    int u = 0;
                    if (p < a.num_seqs) u = prefix[order2[p] + 1] - prefix[order2[p]];
                    int tot;
                    const int incl = block_inclusive_scan(u, misc, tot);
                    if (p < a.num_seqs) pprefix[p + 1] = carry + incl;
                    carry += tot;
                }
                if (tid == 0) pprefix[0] = 0;
                __syncthreads();
            }
            // every lane keeps the n_w - 1 inner cut points of its capacity (lane-minor, so that the lanes'
            // stores do not collide) as long as they fit; otherwise the best capacity is swept again
            const int n_cand = two ? 128 : 64;
            const bool keep = n_cand * (n_w - 1) <= kPlanCutsRoom;
            // (8 capacities per wave and order: lanes of one wave that walk at different speeds wait for each
            // other; the kernel runs with 8 waves, the second order's candidates in waves 4 to 7; every flag
            // is written)
            int* fits = ubase + 64;  // [128]
            {
                const int per_wave = n_cand / 8;
                const int cand = (tid >> 6) * per_wave + (tid & 63);
                if ((tid & 63) < per_wave) {
                    const int step = cand & 63;
                    const bool ok = sweep_head((cand >> 6) ? pprefix : prefix, a.num_seqs, n_w, base2 + base2 * step / 100,
                                               keep ? cuts + cand : nullptr, n_cand);
                    fits[cand] = ok ? 1 : 0;
                }
            }
            __syncthreads();
            if (tid < 64) {
                const uint64_t votes0 = __ballot(fits[tid] != 0);
                const uint64_t votes1 = __ballot(two && fits[64 + tid] != 0);
                const int best0 = votes0 != 0 ? __builtin_ctzll(votes0) : 64;
                const int best1 = votes1 != 0 ? __builtin_ctzll(votes1) : 64;
                if (tid == 0) {
                    // (kept in misc: the cut points written below reach into ubase[0] when n_active == 1024)
                    const bool second = best1 < best0;
                    const int best = second ? best1 : best0;
                    misc[48] = best;
                    misc[49] = second ? 1 : 0;
                    if (best < 64 && !keep) sweep_head(second ? pprefix : prefix, a.num_seqs, n_w, base2 + base2 * best / 100, cuts, 1);
                }
            }
            __syncthreads();
            swept = misc[48] < 64;
            reordered = swept && misc[49] != 0;
            if (swept) {
                const int cand = misc[48] + (reordered ? 64 : 0);
                for (int k = tid; k <= n_active; k += blockDim.x) {
                    const int kvh = k / n_w, w = k - kvh * n_w;  // (k == n_active: the end of the last head)
                    bounds[k] = kvh * per_head + (w == 0 ? 0 : cuts[keep ? (w - 1) * n_cand + cand : w - 1]);
                }
            }
            __syncthreads();
        }
        if (placed && !swept) {  // (uniform)
            // Cost of the units before unit x: 2 x + kPlanSeqCost * (sequences that begin at or before x).
            // Sequence j of the launch (KV head major) begins at unit start(j); the cost there:
            const int n_seq_heads = a.h_kv * a.num_seqs;
            auto start = [&](int j) {  // j == n_seq_heads: total
                const int kvh = j / a.num_seqs;
                return static_cast<int64_t>(kvh) * per_head + prefix[j - kvh * a.num_seqs];
            };
            auto cost_at = [&](int j) { return 2 * start(j) + static_cast<int64_t>(kPlanSeqCost) * j; };
            const int64_t cost_total = cost_at(n_seq_heads);
            for (int k = tid; k <= n_active; k += blockDim.x) {
                int64_t x = k == 0 ? 0 : total;
                if (k > 0 && k < n_active) {
                    const int64_t target = cost_total * k / n_active;
                    int lo = 0, hi = n_seq_heads;  // the first sequence whose beginning costs at least the target
                    while (lo < hi) {
                        const int mid = (lo + hi) >> 1;
                        if (cost_at(mid) < target) lo = mid + 1;
                        else hi = mid;
                    }
                    x = 0;
                    if (lo > 0) {
                        // inside the sequence before it the cost grows by 2 per unit: the first unit that reaches the target
                        const int64_t below = start(lo - 1), above = start(lo);
                        x = (target - static_cast<int64_t>(kPlanSeqCost) * (lo - 1) + 1) >> 1;
                        x = x > above ? above : x;
                        if (x - below <= kPlanSnap && below > 0) x = below;
                        else if (above - x <= kPlanSnap && above < total) x = above;
                    }
                }
                bounds[k] = static_cast<int>(x);
            }
            __syncthreads();
        }
        if (placed) {
            // every workgroup that takes part must own a unit (a cut item's pieces are counted by their
            // owners' numbers), except that the sweep may leave workgroups without any where a sequence
            // begins (no item reaches across such a point): if not, equal ranges
            int bad = 0;
            for (int k = tid; k < n_active; k += blockDim.x) bad |= swept ? bounds[k] > bounds[k + 1] : bounds[k] >= bounds[k + 1];
            if (tid == 0) misc[32] = 0;
            __syncthreads();
            if (bad) misc[32] = 1;
            __syncthreads();
            placed = misc[32] == 0;
        }
        reordered = reordered && placed;
        for (int k = tid; k < pa.n_wg; k += blockDim.x) {
            WgWork w;
            w.a0 = w.a1 = w.b0 = w.b1 = 0;
            w.partner = -1;
            w.ubase = 0;
            w.q0 = w.q_len = w.kvh = w.rt = 0;  // (the fill kernel enters them)
            w.pad[0] = w.pad[1] = 0;
            if (k < n_active && total > 0) {
                w.a0 = placed ? bounds[k] : split.first(k);
                w.a1 = placed ? bounds[k + 1] : split.first(k + 1);
                w.ubase = static_cast<int32_t>(w.a0);
            }
            work[k] = w;
        }
        if (placed)
            for (int k = tid; k <= n_active; k += blockDim.x) g_bounds[k] = bounds[k];
    }
    // the unit prefix over the positions of the unit space, and who is where
    {
        int32_t* g_order = reinterpret_cast<int32_t*>(pa.buf + lay.order_off);
        for (int s = tid; s <= a.num_seqs; s += blockDim.x) g_prefix[s] = reordered ? pprefix[s] : prefix[s];
        for (int s = tid; s < a.num_seqs; s += blockDim.x) g_order[s] = reordered ? order2[s] : s;
    }
    if (tid == 0) {
        PlanHeader h;
        h.magic = total <= pa.capacity ? kPlanMagic : 0u;  // too small a buffer: the kernels plan for themselves
        h.signature = pa.signature;
        h.n_active = n_active;
        h.mode = pairing ? 1 : (placed ? 2 : 0);
        h.per_head = per_head;
        h.total_units = static_cast<int32_t>(total);
        h.capacity = static_cast<int32_t>(pa.capacity);
        h.critical = critical;
        h.reordered = reordered ? 1 : 0;
        for (int i = 0; i < 7; ++i) h.pad[i] = 0;
        *hdr = h;
    }
}

// Phase two, one workgroup per attention workgroup: the unit and band descriptors of its work.
template <int HD, int NB, int NW, bool COMPACT, int KVB, bool DISTINCT = false>
__global__ void __launch_bounds__(64 * NW) paged_attn_plan_fill_kernel(const KArgs a, const PlanArgs pa) {
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    using C = StreamCfg<HD, NB, NW, COMPACT, KVB>;
    StreamAttn<HD, NB, NW, COMPACT, KVB, false, DISTINCT> at(a, smem);
    const PlanHeader* hdr = reinterpret_cast<const PlanHeader*>(pa.buf);
    if (hdr->magic != kPlanMagic) return;
    const PlanLayout lay = plan_layout(a.num_seqs, pa.n_wg, pa.capacity, NW);
    const int* g_prefix = reinterpret_cast<const int*>(pa.buf + lay.prefix_off);
    const WgWork w = reinterpret_cast<const WgWork*>(pa.buf + lay.work_off)[blockIdx.x];
    UnitDesc* g_units = reinterpret_cast<UnitDesc*>(pa.buf + lay.units_off);
    BandDesc* g_bands = reinterpret_cast<BandDesc*>(pa.buf + lay.bands_off);
    for (int s = threadIdx.x; s <= a.num_seqs; s += blockDim.x) at.prefix[s] = g_prefix[s];
    at.per_head = hdr->per_head;
    if (hdr->reordered) at.order = reinterpret_cast<const int32_t*>(pa.buf + lay.order_off);
    __syncthreads();
    int64_t done = w.ubase;
    at.rel_base = w.a0;
    bool first_chunk = true;
    for (int seg = 0; seg < 2; ++seg) {
        at.begin = seg == 0 ? w.a0 : w.b0;
        at.end = seg == 0 ? w.a1 : w.b1;
        for (int64_t chunk = at.begin; chunk < at.end; chunk += C::kPlanUnits) {
            const int n = static_cast<int>(min(static_cast<int64_t>(C::kPlanUnits), at.end - chunk));
            at.plan_units(chunk, n, seg == 0 ? w.partner : -1, seg);
            __syncthreads();
            if (first_chunk && static_cast<int>(threadIdx.x) < min(n, kPlanFirst) * NW) {
                // the first units' band descriptors once more, where the attention kernel finds them with its entry
                BandDesc* g_first = reinterpret_cast<BandDesc*>(pa.buf + lay.first_off) + static_cast<int64_t>(blockIdx.x) * kPlanFirst * NW;
                g_first[threadIdx.x] = at.bands[threadIdx.x];
            }
            if (first_chunk && threadIdx.x == 0) {
                // the first unit's item, for the attention kernel to request its query rows early
                WgWork* mine = reinterpret_cast<WgWork*>(pa.buf + lay.work_off) + blockIdx.x;
                const UnitDesc d = at.units[0];
                mine->q0 = d.q0;
                mine->q_len = d.q_len;
                mine->kvh = d.kvh;
                mine->rt = d.rt;
            }
            first_chunk = false;
            // descriptors are multiples of 16 bytes: copy as such
            const u32x4* su = reinterpret_cast<const u32x4*>(at.units);
            u32x4* du = reinterpret_cast<u32x4*>(g_units + done);
            for (int i = threadIdx.x; i < n * 3; i += blockDim.x) du[i] = su[i];
            const u32x4* sb = reinterpret_cast<const u32x4*>(at.bands);
            u32x4* db = reinterpret_cast<u32x4*>(g_bands + done * NW);
            for (int i = threadIdx.x; i < n * NW; i += blockDim.x) db[i] = sb[i];
            done += n;
            __syncthreads();
        }
    }
}

}  // namespace dfx
