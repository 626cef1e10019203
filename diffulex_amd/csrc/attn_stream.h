// Streaming tile path of the paged-attention kernels (page_size a multiple of 16; bf16 KV, or
// FP8-E4M3 KV with head_dim 128: see the second kernel below).
//
// K/V tiles go HBM -> LDS directly (global_load_lds_dwordx4, 16 bytes per lane, never through
// registers) into a ring of kStages stages, so several tiles are in flight per compute unit
// while the matrix cores work on an older one.  The ring runs over the workgroup's whole unit
// range: tiles of the next (sequence, head) item are already on their way while the current
// item is finished.
//
// Everything data dependent about a unit (which sequence / head / tile it is, where its rows
// start in memory, whether it opens or closes an item) is worked out ahead of time by all
// lanes in parallel and kept in a small LDS table, kPlanUnits units at a time.  The tile loop
// itself reads that table and issues nothing to memory but the asynchronous tile loads, so
// their in-order completion counter can be waited on exactly.
//
// LDS tile layout: the swizzled row-major layout of attn_tile.h.  A direct-to-LDS load writes
// lane i's 16 bytes at wave_base + 16*i, so the swizzle is applied on the global side: lane i
// fetches the chunk that belongs at position i.
//
// The asynchronous loads are issued from inline assembly and waited for with explicit
// s_waitcnt vmcnt(n): the compiler does not model them, so it neither drains them at every
// barrier nor before every LDS read.  vmcnt retires in order, so waits the compiler adds for
// its own loads/stores can only be stricter than needed, never too weak.
#pragma once

#include "attn_tile.h"

namespace dfx {

// One unit of the plan: wave-uniform facts (UnitDesc) and the start of each wave's band of
// rows of the tile in memory (BandDesc; 64 / waves rows per band).
struct UnitDesc {
    int32_t s, kvh, rt, q0;
    int32_t q_len, base, limit, flags;
    int32_t partner, run;  // partner: pairing partition, the workgroup with the other piece of this item (else -1);
                           // run: units from this one to the end of this workgroup's piece of the item
    int32_t item_rel;    // first unit of the item, relative to the workgroup's first unit
    int32_t n_tiles;     // KV tiles of the item
};
static_assert(sizeof(UnitDesc) == 48, "UnitDesc is read as three 16-byte LDS words");
struct BandDesc {
    int64_t off;   // byte offset of the band's first row from the K base pointer (the V base too, for cached rows)
    int32_t last;  // last valid row of the band; later rows re-read it
    int32_t is_ctx;  // 1: cached rows; fresh rows: -(1 + index of the band's first row in k_new / v_new), from
                     // which the V offset follows where v_new has another token stride than k_new
};
// ---- the launch plan (plan.h builds it; layout of the buffer described there) ----------------------
constexpr uint32_t kPlanMagic = 0x44465850u;  // "DFXP"

struct PlanHeader {
    uint32_t magic;      // kPlanMagic once both kernels have run; 0: unusable
    uint32_t signature;  // of the launch configuration the plan was made for
    int32_t n_active;    // workgroups that take part
    int32_t mode;        // 0: equal linear ranges, 1: pairing partition, 2: linear ranges cut at the plan's bounds table
    int32_t per_head;    // units per KV head
    int32_t total_units;
    int32_t capacity;    // unit descriptors the buffer has room for
    int32_t critical;    // pairing: the critical length M (tiles), for diagnostics
    int32_t reordered;   // 1: the unit space lists the sequences in the order of the plan's order table
    int32_t pad[7];
};
static_assert(sizeof(PlanHeader) == 64, "header is one 64-byte line");

struct WgWork {
    int64_t a0, a1, b0, b1;  // linear unit ranges [a0, a1) then [b0, b1), each inside one item under pairing
    int32_t partner;         // pairing: the workgroup holding the other piece of the shared item, or -1
    int32_t ubase;           // index of the workgroup's first unit descriptor
    // of the workgroup's first unit (copied from its descriptor): what it takes to request the
    // query rows of the first item before the descriptors have been read
    int32_t q0, q_len, kvh, rt;
    int32_t pad[2];
};
static_assert(sizeof(WgWork) == 64, "four 16-byte words");

// Band descriptors of the first kPlanFirst units of every workgroup, a second time and by themselves:
// a workgroup reads those of its own waves with its plan entry, in one trip to memory, and starts its
// first tile loads from them while the descriptor tables are still on their way.
constexpr int kPlanFirst = 4;

struct PlanLayout {
    int64_t prefix_off, bounds_off, work_off, order_off, first_off, units_off, bands_off, bytes;
};
DFX_HD PlanLayout plan_layout(int num_seqs, int n_wg, int64_t capacity, int waves) {
    PlanLayout l;
    l.prefix_off = sizeof(PlanHeader);
    l.bounds_off = (l.prefix_off + (static_cast<int64_t>(num_seqs) + 1) * 4 + 63) / 64 * 64;
    l.work_off = (l.bounds_off + (static_cast<int64_t>(n_wg) + 1) * 4 + 63) / 64 * 64;
    l.order_off = (l.work_off + static_cast<int64_t>(n_wg) * sizeof(WgWork) + 63) / 64 * 64;
    l.first_off = (l.order_off + static_cast<int64_t>(num_seqs) * 4 + 63) / 64 * 64;
    l.units_off = l.first_off + static_cast<int64_t>(n_wg) * kPlanFirst * waves * static_cast<int64_t>(sizeof(BandDesc));
    l.bands_off = l.units_off + capacity * static_cast<int64_t>(sizeof(UnitDesc));
    l.bytes = l.bands_off + capacity * waves * static_cast<int64_t>(sizeof(BandDesc));
    return l;
}

// UnitDesc::flags: bits 8..15 a bit per band of rows whose page is missing (holes); bits 16..21, set by
// mark_plain_steps() only, the number of consecutive plain steps that begin with this unit
// kUnitFreshStart: the item's first tile of fresh rows, or the first tile of the workgroup's piece of the item
// where that is a later one of them (where the fresh rows' rotary embedding is the launch's, the workgroup
// rotates the item's fresh K rows when it meets this unit)
enum : int32_t { kUnitCtx = 1, kUnitFirst = 2, kUnitLast = 4, kUnitComplete = 8, kUnitFreshStart = 16, kUnitHoleShift = 8, kUnitPlainShift = 16 };
DFX_HD uint32_t unit_holes(int flags) { return (static_cast<uint32_t>(flags) >> kUnitHoleShift) & 0xffu; }

// COMPACT: a configuration small enough (2 stages, short plan, at most kCompactMaxSeqs sequences)
// for two workgroups to share a compute unit.  Items with at most 128 rows run with four waves,
// one per SIMD, which then does nothing while its wave waits for LDS, for the issue of a load or
// at the barrier; a second, independent workgroup on the same SIMDs fills those gaps.
constexpr int kCompactMaxSeqs = 1023;

//
// KVB: bytes per cache element.  With FP8 codes (KVB == 1) a ring stage holds the tile as stored,
// and each wave widens the rows it loaded itself into one of two bf16 tiles in the layout of
// attn_tile.h one step before the matrix instructions read them (see the FP8 kernel below).
template <int HD, int NB, int NW, bool COMPACT = false, int KVB = 2>
struct StreamCfg : Shape<HD, NB, NW> {
    using S = Shape<HD, NB, NW>;
    static constexpr int ROWB = HD * KVB;             // bytes per token row as loaded
    static constexpr int CPR = ROWB / 16;             // 16-byte chunks per row
    static constexpr int RPI = 1024 / ROWB;           // rows one wave-wide load covers
    static constexpr int MAT_BYTES = S::TN * ROWB;    // K (or V) tile
    static constexpr int STAGE_BYTES = 2 * MAT_BYTES;
    static constexpr int kStages = COMPACT ? 2 : 4;
    static constexpr int IPW = MAT_BYTES / 1024 / NW;  // loads per wave per matrix per tile
    static constexpr int LOADS_PER_UNIT = 2 * IPW;
    static constexpr int ROWS_PER_WAVE = IPW * RPI;        // 16 (4 waves) or 8 (8 waves)
    // units described (and then streamed) at a time: the tile loop drains and refills its ring at the end of
    // every table (≈ 5 µs), so as many as the LDS of a compute unit has room for beside the tiles
    static constexpr int kPlanUnits = COMPACT ? 32 : (NW == 8 ? 88 : 128);
    static constexpr int PREFIX_BYTES = COMPACT ? (kCompactMaxSeqs + 1) * 4 : S::PREFIX_BYTES;
    static constexpr int UNIT_TABLE_BYTES = kPlanUnits * static_cast<int>(sizeof(UnitDesc));
    static constexpr int BAND_TABLE_BYTES = kPlanUnits * NW * static_cast<int>(sizeof(BandDesc));
    static constexpr int UNIT_TABLE_OFF = PREFIX_BYTES + S::MISC_BYTES;
    static constexpr int BAND_TABLE_OFF = UNIT_TABLE_OFF + UNIT_TABLE_BYTES;
    static constexpr int STAGES_OFF = (BAND_TABLE_OFF + BAND_TABLE_BYTES + 255) / 256 * 256;  // tiles start at a multiple of 256
    static constexpr int WIDE_OFF = STAGES_OFF + kStages * STAGE_BYTES;
    static constexpr int WIDE_BYTES = 2 * TileLayout<HD>::MAT_BYTES;  // widened K tile, widened V tile
    static constexpr int LDS_BYTES = WIDE_OFF + (KVB == 1 ? 2 * WIDE_BYTES : 0);
    static_assert(KVB == 2 || (KVB == 1 && !COMPACT), "bf16 or FP8 codes");
    static_assert(ROWS_PER_WAVE * NW == S::TN && IPW >= 1, "the waves' row bands tile the 64 rows");
    static_assert(LDS_BYTES <= (COMPACT ? 80 : 160) * 1024, "LDS budget of a gfx950 compute unit");

    // FP8 stages are read back by the lanes that loaded them, in load order: no swizzle needed
    DFX_HD static int swizzle(int row) { return KVB == 2 ? TileLayout<HD>::swizzle(row) : 0; }
};

// One wave-wide 16-byte-per-lane direct-to-LDS load from base + voff; lane i's data lands at
// lds_wave_base + 16*i.  base and lds_wave_base must be wave-uniform.
DFX_D void async_load16(const void* base, uint32_t voff, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                 :
                 : "v"(voff), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base))
                 : "memory", "m0");
}

// The float at p (wave-uniform, not written during the launch), read into a scalar register.
DFX_D float scalar_load(const float* p) {
    float x;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(x) : "s"(p) : "memory");
    return x;
}

template <int N>
DFX_D void wait_async_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// DISTINCT: the cache is in the distinct layout (K [pages, H, HD / 8, page, 8], V [pages, H, HD, page]; pages of
// a multiple of 64 tokens, so that a tile lies in one page).  A stage then holds the K tile chunk-major and the
// V tile d-major (attn_tile.h), both filled by the same direct-to-LDS loads: a wave takes two chunk columns of K
// (1 KiB contiguous each) and 16 rows of V^T (128 contiguous bytes each).  The descriptors are per tile, the
// same for every wave: BandDesc::off = KV head << 52 | page << 20 | first token's place in the page,
// BandDesc::last = the tile's last valid token.  Fresh rows, row-major in memory: K is gathered into the chunk-major tile by the
// loads themselves (a lane per token), V lands row-major and is transposed inside LDS before its step
// (transpose_fresh_v).
template <int HD, int NB, int NW, bool COMPACT = false, int KVB = 2, bool HIDDEN = false, bool DISTINCT = false>
struct StreamAttn : TileMath<HD, NB, NW, HIDDEN> {
    static_assert(!DISTINCT || (KVB == 2 && !COMPACT && NW == 8 && HD == 128), "distinct layout: bf16, 8 waves, head_dim 128");
    using Base = TileMath<HD, NB, NW, HIDDEN>;
    using C = StreamCfg<HD, NB, NW, COMPACT, KVB>;
    using L = TileLayout<HD>;
    using Base::a;
    using Base::col;
    using Base::half;
    using Base::lane;
    using Base::o;
    using Base::qf;
    using Base::tid;
    using Base::wave;

    uint8_t* lds;
    int* prefix;
    int* misc;
    UnitDesc* units;
    BandDesc* bands;
    uint32_t stages_lds;  // LDS byte address of stage 0
    int wave_s;           // the wave's number as a wave-uniform value (a scalar register from the start)
    int64_t begin, end;
    int64_t rel_base;  // what UnitDesc::item_rel is relative to: the first unit of the workgroup's work
    int per_head;
    // plan kernels only: the sequence at every position of the unit space (prefix[] is over positions), or
    // null where the sequences follow each other in their own order
    const int32_t* order = nullptr;
    float k_mul, v_inv;  // FP8: the current item's K scale and the reciprocal of its V scale
    // Units described at a time.  The 8-wave kernel on a cache of codes raises it where a plan has done the
    // planning: the unit prefix over the sequences, a tenth of the LDS, is then not needed, and the tables
    // take its place -- at its benchmark shape a workgroup's 170 units then fit one table instead of two,
    // and every table's end costs it a drained pipeline and a prologue of three widened matrices.
    static constexpr bool kGrowTables = KVB == 1 && NW == 8 && !COMPACT;
    int chunk_cap = C::kPlanUnits;

    DFX_D StreamAttn(const KArgs& args, uint8_t* smem)
        : Base(args), lds(smem), prefix(reinterpret_cast<int*>(smem)),
          misc(reinterpret_cast<int*>(smem + C::PREFIX_BYTES)),
          units(reinterpret_cast<UnitDesc*>(smem + C::UNIT_TABLE_OFF)),
          bands(reinterpret_cast<BandDesc*>(smem + C::BAND_TABLE_OFF)),
          stages_lds(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem)) + C::STAGES_OFF),
          wave_s(uniform(static_cast<int>(threadIdx.x >> 6))) {
        if constexpr (DISTINCT) {  // the lane's operand offsets in a chunk-major K tile and a d-major V tile (attn_tile.h)
            this->k_lane = static_cast<uint32_t>(half * Base::CHUNK_COL_BYTES + Base::swap_quads(col) * 16);
            this->v_lane = static_cast<uint32_t>(Base::vt_chunk_offset(col, half));
        }
    }

    // ---- planning --------------------------------------------------------------------------
    // Describe units [first, first + count) in the plan table (entry i is unit first + i); one
    // lane per (unit, wave).
    // [begin, end) is the range of the linear unit space the workgroup is working on (all of its
    // units, or one of its two ranges under the pairing partition, whose `partner` then holds the
    // other piece of a cut item).
    DFX_D void plan_units(int64_t first, int count, int partner = -1, int seg = 0) const {
        (void)seg;
        // (the thread's number worked out here: what depends on it is then not computed ahead of the
        // caller's chunk loop and, where registers are few, kept in scratch meanwhile)
        for (int idx = thread_number_here(wave_s); idx < count * NW; idx += C::THREADS) {
            const int64_t pos = first + idx / NW;
            const int w = idx % NW;
            const int slot_in_ring = idx / NW;
            const int kv_head = static_cast<int>(pos / per_head);
            const int rem = static_cast<int>(pos - static_cast<int64_t>(kv_head) * per_head);
            int lo = 0, hi = a.num_seqs;  // the position with prefix[p] <= rem < prefix[p + 1]
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (prefix[mid + 1] <= rem) lo = mid + 1;
                else hi = mid;
            }
            const int sq = order != nullptr ? order[lo] : lo;
            const SeqShape shp = load_seq_shape(a, sq, C::RT);
            const int u = rem - prefix[lo];
            int rt, tile, item_tiles;
            locate_unit(shp, u, rt, tile, item_tiles);
            const bool is_ctx = tile < shp.n_ctx_tiles;
            const int base = (is_ctx ? tile : tile - shp.n_ctx_tiles) * C::TN;
            const int limit = is_ctx ? shp.ctx : shp.new_len;
            // the piece of the item this workgroup owns
            const int64_t before = pos - begin, after = end - pos;
            const int tile0 = before >= tile ? 0 : tile - static_cast<int>(before);
            const int tile1 = after >= item_tiles - tile ? item_tiles : tile + static_cast<int>(after);
            if (w == 0) {
                UnitDesc d;
                d.s = sq;
                d.kvh = kv_head;
                d.rt = rt;
                d.q0 = a.cu_q[sq];
                d.q_len = shp.q_len;
                d.base = base;
                d.limit = limit;
                d.flags = (is_ctx ? kUnitCtx : 0) | (tile == tile0 ? kUnitFirst : 0) |
                          (tile == tile1 - 1 ? kUnitLast : 0) |
                          (tile0 == 0 && tile1 == item_tiles ? kUnitComplete : 0) |
                          (!is_ctx && (tile == shp.n_ctx_tiles || tile == tile0) ? kUnitFreshStart : 0);
                d.partner = partner;
                d.run = tile1 - tile;
                d.item_rel = static_cast<int>(pos - tile - rel_base);
                d.n_tiles = item_tiles;
                units[slot_in_ring] = d;
            }
            // Rows past the end re-read the last valid rows (finite data; their scores are masked).
            int band = base + w * C::ROWS_PER_WAVE;
            const bool past_end = band >= limit;
            if (past_end) band = ((limit - 1) / C::ROWS_PER_WAVE) * C::ROWS_PER_WAVE;
            BandDesc b;
            bool hole = false;  // the band's page has no valid block-table entry: its tokens are skipped
            if constexpr (DISTINCT) {
                // one descriptor per tile, repeated for every wave
                if (is_ctx) {
                    const int p = a.page_shift >= 0 ? (base >> a.page_shift) : (base / a.page_size);
                    int64_t page = p < a.max_pages ? a.block_tables[static_cast<int64_t>(sq) * a.bt_stride + p] : -1;
                    hole = page < 0 || page >= a.n_pages;
                    page = page < 0 ? 0 : (page >= a.n_pages ? a.n_pages - 1 : page);
                    b.off = (static_cast<int64_t>(kv_head) << 52) | (page << 20) | static_cast<int64_t>(base - p * a.page_size);
                } else {
                    b.off = ((static_cast<int64_t>(a.cu_new[sq]) + base) * a.kn_st + kv_head * a.kn_sh) * 2;
                }
                b.last = limit - 1 - base;
                b.is_ctx = is_ctx ? 1 : -(1 + a.cu_new[sq] + base);
            } else if (is_ctx) {
                const int p = a.page_shift >= 0 ? (band >> a.page_shift) : (band / a.page_size);
                int64_t page = p < a.max_pages ? a.block_tables[static_cast<int64_t>(sq) * a.bt_stride + p] : -1;
                hole = !past_end && (page < 0 || page >= a.n_pages);
                page = page < 0 ? 0 : (page >= a.n_pages ? a.n_pages - 1 : page);
                b.off = (page * a.c_sp + static_cast<int64_t>(band - p * a.page_size) * a.c_st + kv_head * a.c_sh) * KVB;
            } else {
                b.off = ((static_cast<int64_t>(a.cu_new[sq]) + band) * a.kn_st + kv_head * a.kn_sh) * 2;
            }
            if constexpr (!DISTINCT) {
                b.last = limit - 1 - band;
                b.is_ctx = is_ctx ? 1 : -(1 + a.cu_new[sq] + band);
            }
            bands[slot_in_ring * NW + w] = b;
            // the NW lanes of a unit are neighbours in a wave: its holes as a bit per band
            const uint64_t votes = __ballot(hole);
            const int holes = static_cast<int>((votes >> ((threadIdx.x & 63) & ~(NW - 1))) & ((1u << NW) - 1));
            if (w == 0 && holes != 0) units[slot_in_ring].flags |= holes << kUnitHoleShift;
        }
    }

    // ---- loads -----------------------------------------------------------------------------
    // Start the loads of planned unit `rel` (this wave's band of K and V rows) into its ring stage.
    DFX_D void issue_unit(int rel) const { issue_unit_desc(bands[rel * NW + wave], rel); }
    // The same from a band descriptor the caller holds (wave-uniform or not: it is made uniform here).
    DFX_D void issue_unit_desc(const BandDesc& b, int rel) const {
        const int last = uniform(b.last);
        const int tag = uniform(b.is_ctx);
        const bool is_ctx = tag > 0;
        const int64_t off = (static_cast<int64_t>(uniform(static_cast<int>(b.off >> 32))) << 32) |
                            static_cast<uint32_t>(uniform(static_cast<int>(b.off)));
        if constexpr (DISTINCT) {
            const uint32_t dst = stages_lds + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES;
            const uint32_t tok = static_cast<uint32_t>(min(lane, last));  // tokens past the end re-read the last valid one
            if (is_ctx) {
                const int64_t kvh = static_cast<int64_t>(static_cast<uint64_t>(off) >> 52);
                const int64_t page = (off >> 20) & 0xffffffffll;
                const int64_t in_page = off & 0xfffff;
                const uint8_t* kb = a.k_cache + (page * a.kd_sp + kvh * a.kd_sh + in_page * 8) * 2;
                const uint8_t* vb = a.v_cache + (page * a.vd_sp + kvh * a.vd_sh + in_page) * 2;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int c = wave_s * 2 + j;  // chunk column: a lane per token
                    async_load16(kb + static_cast<int64_t>(c) * a.kd_sc * 2, tok * 16, dst + c * Base::CHUNK_COL_BYTES);
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    // 8 rows of V^T: 8 lanes per row, the chunk at position p of row d holds tokens 8 * (p ^ swizzle(d)) ..;
                    // chunks past the end re-read the last one with a valid token (clear_v_tail zeroes what is not)
                    const int d = wave * 16 + j * 8 + (lane >> 3);
                    const int tc = min((lane & 7) ^ ((d >> 1) & 7), last >> 3);
                    async_load16(vb, static_cast<uint32_t>(d) * static_cast<uint32_t>(a.vd_sd * 2) + tc * 16,
                                 dst + C::MAT_BYTES + (wave * 16 + j * 8) * (C::TN * 2));
                }
            } else {
                const uint8_t* kb = reinterpret_cast<const uint8_t*>(a.k_new) + off;
                const uint8_t* vb = reinterpret_cast<const uint8_t*>(a.v_new) + off + static_cast<int64_t>(-1 - tag) * a.v_fresh_delta;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int c = wave_s * 2 + j;
                    async_load16(kb + c * 16, tok * static_cast<uint32_t>(a.kn_st * 2), dst + c * Base::CHUNK_COL_BYTES);
                }
#pragma unroll
                for (int j = 0; j < C::IPW; ++j) {  // row-major, as a unified-layout stage holds it
                    const int r = wave * C::ROWS_PER_WAVE + j * C::RPI + lane / C::CPR;
                    const int chunk = (lane % C::CPR) ^ C::swizzle(r);
                    async_load16(vb, static_cast<uint32_t>(min(r, last)) * static_cast<uint32_t>(a.vn_st * 2) + chunk * 16,
                                 dst + C::MAT_BYTES + wave * (C::IPW * 1024) + j * 1024);
                }
            }
            return;
        }
        if constexpr (HIDDEN && NW == 8 && KVB == 2) {
            // the common case, a full band of cached rows: offsets precomputed per lane, no vector arithmetic
            if (is_ctx && last >= C::ROWS_PER_WAVE - 1) {
                const int dst = uniform(static_cast<int>(stages_lds + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES + wave * (C::IPW * 1024)));
                if constexpr (HD == 128) pipe_issue_band(a.k_cache + off, a.v_cache + off, dst);
                else pipe64_issue_band(a.k_cache + off, a.v_cache + off, dst);
                return;
            }
        }
        const uint8_t* kbase = (is_ctx ? a.k_cache : reinterpret_cast<const uint8_t*>(a.k_new)) + off;
        // fresh V rows may lie further apart than fresh K rows (V a slice of a projection, K rotated
        // into a buffer of its own): same head offset, another token stride
        const uint8_t* vbase = is_ctx ? a.v_cache + off
                                      : reinterpret_cast<const uint8_t*>(a.v_new) + off + static_cast<int64_t>(-1 - tag) * a.v_fresh_delta;
        const uint32_t row_stride = static_cast<uint32_t>(is_ctx ? a.c_st * KVB : a.kn_st * 2);
        const uint32_t row_stride_v = static_cast<uint32_t>(is_ctx ? a.c_st * KVB : a.vn_st * 2);
        const uint32_t dst = stages_lds + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES + wave * (C::IPW * 1024);
#pragma unroll
        for (int j = 0; j < C::IPW; ++j) {
            const int r = j * C::RPI + lane / C::CPR;  // row inside the band
            const int lds_row = wave * C::ROWS_PER_WAVE + r;
            const int chunk = (lane % C::CPR) ^ C::swizzle(lds_row);
            const uint32_t rl = static_cast<uint32_t>(min(r, last));
            uint32_t voff = rl * row_stride + chunk * 16;
            uint32_t voff_v = rl * row_stride_v + chunk * 16;
            // Fresh rows are bf16 and are fetched by widen_unit() itself; the loads are issued all
            // the same (every lane re-reads the band's first bytes) so that every unit advances
            // the completion counter by the same amount.
            if (KVB == 1 && !is_ctx) voff = voff_v = 0;
            async_load16(kbase, voff, dst + j * 1024);
            async_load16(vbase, voff_v, dst + C::MAT_BYTES + j * 1024);
        }
    }

    // FP8 only: bring unit `rel` into bf16 tile (rel & 1).  A wave widens the rows it loaded itself,
    // so it only has to wait for its own loads; fresh rows (bf16 in memory) are copied from
    // global memory here, once per item.
    DFX_D uint8_t* wide_tile(int rel) const { return lds + C::WIDE_OFF + (rel & 1) * C::WIDE_BYTES; }
    DFX_D void widen_unit(int rel) const {
        const BandDesc b = bands[rel * NW + wave];
        const int tag = uniform(b.is_ctx);
        const bool is_ctx = tag > 0;
        uint8_t* kt = wide_tile(rel);
        uint8_t* vt = kt + L::MAT_BYTES;
        const uint8_t* raw = lds + C::STAGES_OFF + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES + wave * (C::IPW * 1024) + lane * 16;
        if (is_ctx) {
#pragma unroll
            for (int j = 0; j < C::IPW; ++j) {
                const int row = wave * C::ROWS_PER_WAVE + j * C::RPI + lane / C::CPR;
                const int cc = lane % C::CPR;
                const u32x4 kc = *reinterpret_cast<const u32x4*>(raw + j * 1024);
                const u32x4 vc = *reinterpret_cast<const u32x4*>(raw + C::MAT_BYTES + j * 1024);
                u32x4 lo, hi;
                widen16(kc, lo, hi);
                *reinterpret_cast<u32x4*>(kt + L::chunk_offset(row, 2 * cc)) = lo;
                *reinterpret_cast<u32x4*>(kt + L::chunk_offset(row, 2 * cc + 1)) = hi;
                widen16(vc, lo, hi);
                *reinterpret_cast<u32x4*>(vt + L::chunk_offset(row, 2 * cc)) = lo;
                *reinterpret_cast<u32x4*>(vt + L::chunk_offset(row, 2 * cc + 1)) = hi;
            }
        } else {
            const int last = uniform(b.last);
            const int64_t off = (static_cast<int64_t>(uniform(static_cast<int>(b.off >> 32))) << 32) |
                                static_cast<uint32_t>(uniform(static_cast<int>(b.off)));
            const uint8_t* kbase = reinterpret_cast<const uint8_t*>(a.k_new) + off;
            const uint8_t* vbase = reinterpret_cast<const uint8_t*>(a.v_new) + off + static_cast<int64_t>(-1 - tag) * a.v_fresh_delta;
#pragma unroll
            for (int j = 0; j < C::IPW; ++j) {
                const int r = j * C::RPI + lane / C::CPR;
                const int row = wave * C::ROWS_PER_WAVE + r;
                const int cc = lane % C::CPR;
                const int64_t voff = static_cast<int64_t>(min(r, last)) * a.kn_st * 2 + cc * 32;
                const int64_t voff_v = static_cast<int64_t>(min(r, last)) * a.vn_st * 2 + cc * 32;
                const u32x4 k0 = *reinterpret_cast<const u32x4*>(kbase + voff);
                const u32x4 k1 = *reinterpret_cast<const u32x4*>(kbase + voff + 16);
                const u32x4 v0 = *reinterpret_cast<const u32x4*>(vbase + voff_v);
                const u32x4 v1 = *reinterpret_cast<const u32x4*>(vbase + voff_v + 16);
                // Wait here, inside the branch: a wait the compiler places where the two branches
                // meet again would drain the asynchronous loads in every step.
                __builtin_amdgcn_s_waitcnt(0x0f70);
                *reinterpret_cast<u32x4*>(kt + L::chunk_offset(row, 2 * cc)) = k0;
                *reinterpret_cast<u32x4*>(kt + L::chunk_offset(row, 2 * cc + 1)) = k1;
                *reinterpret_cast<u32x4*>(vt + L::chunk_offset(row, 2 * cc)) = v0;
                *reinterpret_cast<u32x4*>(vt + L::chunk_offset(row, 2 * cc + 1)) = v1;
            }
        }
    }

    // FP8, pipelined kernel.  Its step works on the K tile of one unit and the V tile of the unit
    // before, so the widened K tiles and the widened V tiles are kept apart, two of each, and a
    // unit's two halves are widened a step apart (K first).  Fresh rows are copied as they are: the
    // kernel folds the scales that tell them from cached rows into its softmax constants.
    DFX_D uint8_t* wide_k(int rel) const { return lds + C::WIDE_OFF + (rel & 1) * L::MAT_BYTES; }
    DFX_D uint8_t* wide_v(int rel) const { return lds + C::WIDE_OFF + 2 * L::MAT_BYTES + (rel & 1) * L::MAT_BYTES; }
    // CTX_ONLY: the caller knows the band to be one of cached rows.
    template <bool IS_V, bool CTX_ONLY = false>
    DFX_D void widen_matrix(int rel) const {
        int tag = 1;
        if constexpr (!CTX_ONLY) tag = uniform(bands[rel * NW + wave_s].is_ctx);
        uint8_t* dst = IS_V ? wide_v(rel) : wide_k(rel);
        // (the lane's number worked out here: see thread_number_here())
        const int ln = thread_number_here(0);
        const int cc = ln % C::CPR;
        if (CTX_ONLY || tag > 0) {
            const uint8_t* raw = lds + C::STAGES_OFF + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES +
                                 (IS_V ? C::MAT_BYTES : 0) + wave_s * (C::IPW * 1024) + ln * 16;
#pragma unroll
            for (int j = 0; j < C::IPW; ++j) {
                const int row = wave_s * C::ROWS_PER_WAVE + j * C::RPI + ln / C::CPR;
                const u32x4 codes = *reinterpret_cast<const u32x4*>(raw + j * 1024);
                u32x4 lo, hi;
                widen16(codes, lo, hi);
                *reinterpret_cast<u32x4*>(dst + L::chunk_offset(row, 2 * cc)) = lo;
                *reinterpret_cast<u32x4*>(dst + L::chunk_offset(row, 2 * cc + 1)) = hi;
            }
        } else {
            const BandDesc b = bands[rel * NW + wave_s];
            const int last = uniform(b.last);
            const int64_t off = (static_cast<int64_t>(uniform(static_cast<int>(b.off >> 32))) << 32) |
                                static_cast<uint32_t>(uniform(static_cast<int>(b.off)));
            const uint8_t* base = IS_V ? reinterpret_cast<const uint8_t*>(a.v_new) + off + static_cast<int64_t>(-1 - tag) * a.v_fresh_delta
                                       : reinterpret_cast<const uint8_t*>(a.k_new) + off;
            const int64_t stride = (IS_V ? a.vn_st : a.kn_st) * 2;
#pragma unroll
            for (int j = 0; j < C::IPW; ++j) {
                const int r = j * C::RPI + ln / C::CPR;
                const int row = wave_s * C::ROWS_PER_WAVE + r;
                const int64_t voff = static_cast<int64_t>(min(r, last)) * stride + cc * 32;
                const u32x4 x0 = *reinterpret_cast<const u32x4*>(base + voff);
                const u32x4 x1 = *reinterpret_cast<const u32x4*>(base + voff + 16);
                // Wait here, inside the branch: a wait the compiler places where the two branches
                // meet again would drain the asynchronous loads in every step.
                __builtin_amdgcn_s_waitcnt(0x0f70);
                *reinterpret_cast<u32x4*>(dst + L::chunk_offset(row, 2 * cc)) = x0;
                *reinterpret_cast<u32x4*>(dst + L::chunk_offset(row, 2 * cc + 1)) = x1;
            }
        }
    }

    // Make the compiler wait for the query loads here, once per item.  Left to itself it puts the
    // wait before their first use inside the tile loop, where it also drains the asynchronous tile
    // loads issued since, in every iteration.
    DFX_D void touch_queries() const {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb)
#pragma unroll
            for (int slab = 0; slab < C::NSLAB; ++slab) asm volatile("" : : "v"(qf[qb][slab]));
    }

    // Adopt the item of unit d as the current one and fetch its query rows.  With wait == false
    // the caller calls touch_queries() itself before the tile loop.
    DFX_D void begin_item(const UnitDesc& d, bool wait = true) {
        this->s = uniform(d.s);
        this->kvh = uniform(d.kvh);
        this->q0 = uniform(d.q0);
        this->sh.q_len = uniform(d.q_len);
        if (KVB == 1) {
            k_mul = a.k_scale[this->kvh];
            this->out_mul = a.v_scale[this->kvh];
            v_inv = 1.0f / this->out_mul;
        }
        this->load_queries(uniform(d.rt));
        if (wait) touch_queries();
    }

    // Pipelined kernel.  The query rows of an item go straight into the Q operand registers
    // (attn_pipe_gen.h), which no matrix instruction reads during the last step of the item before:
    // request_queries(d) may be called from there on, adopt_item(d) once that item is finished and
    // the loads have been waited for.
    DFX_D void request_queries(const UnitDesc& d) const {
        static_assert(HIDDEN, "pipelined kernel only");
        const int q_len = uniform(d.q_len);
        const int r = this->row_of(uniform(d.rt), 0);
        const bool valid = r < a.group * q_len;
        const int g = valid ? r / q_len : 0;
        const int i = valid ? r - g * q_len : 0;
        // (lanes without a row read row 0 of the item: finite data whose results are never stored; a row
        // beyond the rows q has -- offsets rewritten in place after the plan was made -- reads row 0 of q)
        int row = uniform(d.q0) + i;
        row = row < a.n_q ? row : 0;
        const uint16_t* qp = a.q + row * a.q_st + (uniform(d.kvh) * a.group + g) * a.q_sh + half * 8;
        if constexpr (HD == 128) pipe_issue_queries(qp);
        else pipe64_issue_queries(qp);
    }
    DFX_D void adopt_item(const UnitDesc& d) {
        this->s = uniform(d.s);
        this->kvh = uniform(d.kvh);
        this->q0 = uniform(d.q0);
        this->sh.q_len = uniform(d.q_len);
        if (KVB == 1) {
            // read through the scalar cache into scalar registers: as vector loads the compiler keeps them
            // in vector registers, spills those, and waits for every tile load in flight at each reload
            k_mul = scalar_load(a.k_scale + this->kvh);
            this->out_mul = scalar_load(a.v_scale + this->kvh);
            v_inv = __builtin_bit_cast(float, uniform(__builtin_bit_cast(int, 1.0f / this->out_mul)));
        }
        this->reset_accumulators();
    }
    // ---- rotary embedding inside the launch (KArgs::rope_table) ---------------------------------------
    DFX_D int64_t rope_position(int64_t token) const {
        int64_t pos = a.rope_pos_i64 ? static_cast<const int64_t*>(a.rope_pos)[token]
                                     : static_cast<int64_t>(static_cast<const int32_t*>(a.rope_pos)[token]);
        // (outside the table: a caller error, clamped as dfx_rope_kv_store clamps it)
        return pos < 0 ? 0 : (pos >= a.rope_max_pos ? a.rope_max_pos - 1 : pos);
    }
    // The query rows of item d are rotated in the Q operand registers once they have landed: the position
    // of the lane's row first (a load of its own, which the caller lets travel with other work), then the
    // request for its angles, then pipe_rope_queries().
    DFX_D int64_t rope_query_position(const UnitDesc& d) const {
        static_assert(HIDDEN && HD == 128, "pipelined kernels");
        const int q_len = uniform(d.q_len);
        const int r = this->row_of(uniform(d.rt), 0);
        const int i = r < a.group * q_len ? r % q_len : 0;
        int row = uniform(d.q0) + i;
        row = row < a.n_q ? row : 0;
        return rope_position(row);
    }
    DFX_D void request_rope_angles(int64_t pos) const {
        int h = half;  // (opaque: the lane's share of the address is then not worked out at the kernel's entry and kept in scratch)
        asm volatile("" : "+v"(h));
        pipe_issue_rope_angles(a.rope_table + pos * HD + h * 8);
    }
    DFX_D void rope_queries(const UnitDesc& d) const {
        request_rope_angles(rope_query_position(d));
        pipe_rope_queries();
    }
    // The fresh K rows of one sequence, KV head kv_head: rotated from k_src into k_new and, with the fused
    // store, into their cache slots together with the V rows (what dfx_rope_kv_store does in a launch of its
    // own, bit for bit).  All threads of the workgroup; a lane takes a pair of 16-byte chunks (c, c + 8) of
    // a row.  Several workgroups (the row tiles of one sequence and head) may do the same rows: they write
    // the same bytes.
    // The rows are n0 .. n1 - 1 of k_src / k_new / v_new.
    template <bool FP8>
    DFX_D void rope_fresh_rows(int64_t n0, int64_t n1, int kv_head) const {
        static_assert(HIDDEN && HD == 128, "pipelined kernels");
        const int64_t n_slots = a.n_pages * a.page_size;
        for (int64_t idx = thread_number_here(wave_s); idx < (n1 - n0) * 8; idx += C::THREADS) {
            const int64_t t = n0 + (idx >> 3);
            const int c = static_cast<int>(idx & 7);
            // The slot first: its load travels with that of the position, and with a two-byte cache the V chunks
            // then travel with the K chunks and the angles (two trips to memory instead of four).
            int64_t slot = -1;
            if (a.store_slots != nullptr)
                slot = a.store_slots_i64 ? static_cast<const int64_t*>(a.store_slots)[t]
                                         : static_cast<int64_t>(static_cast<const int32_t*>(a.store_slots)[t]);
            const int64_t pos = rope_position(t);
            const bool stored = slot >= 0 && slot < n_slots;
            const int64_t page = a.page_shift >= 0 ? (slot >> a.page_shift) : slot / a.page_size;
            const int64_t e = page * a.c_sp + (slot - page * a.page_size) * a.c_st + kv_head * a.c_sh + c * 8;  // elements
            const uint16_t* vp = a.v_new + t * a.vn_st + kv_head * a.vn_sh + c * 8;
            uint8_t* kc = const_cast<uint8_t*>(a.k_cache);
            uint8_t* vc = const_cast<uint8_t*>(a.v_cache);
            uint32_t lo[4], hi[4];
            const uint16_t* ksrc = a.k_src + t * a.ks_st + kv_head * a.ks_sh + c * 8;
            if (!FP8 && stored) pipe_rope_row_with_v(ksrc, a.rope_table + pos * HD + c * 8, vp, vc + e * 2, lo, hi);
            else pipe_rope_row(ksrc, a.rope_table + pos * HD + c * 8, lo, hi);
            const u32x4 o1 = {lo[0], lo[1], lo[2], lo[3]}, o2 = {hi[0], hi[1], hi[2], hi[3]};
            uint16_t* dst = const_cast<uint16_t*>(a.k_new) + t * a.kn_st + kv_head * a.kn_sh + c * 8;
            *reinterpret_cast<u32x4*>(dst) = o1;
            *reinterpret_cast<u32x4*>(dst + HD / 2) = o2;
            if (!stored) continue;
            if constexpr (FP8) {
                const u32x4 v1 = *reinterpret_cast<const u32x4*>(vp), v2 = *reinterpret_cast<const u32x4*>(vp + HD / 2);
                const float ks = a.k_scale[kv_head], vs = a.v_scale[kv_head];
                *reinterpret_cast<u32x2*>(kc + e) = quantise8(o1, ks);
                *reinterpret_cast<u32x2*>(kc + e + HD / 2) = quantise8(o2, ks);
                *reinterpret_cast<u32x2*>(vc + e) = quantise8(v1, vs);
                *reinterpret_cast<u32x2*>(vc + e + HD / 2) = quantise8(v2, vs);
            } else {
                *reinterpret_cast<u32x4*>(kc + e * 2) = o1;
                *reinterpret_cast<u32x4*>(kc + e * 2 + HD) = o2;
            }
        }
    }
    // The same for every item whose fresh tiles begin among the n_units units in the tables (kUnitFreshStart),
    // before any of those tiles is requested.  Every thread of the workgroup; the tables are complete.
    // Returns whether any row was written: the caller then waits for its stores (vmcnt(0)) and lets the
    // workgroup meet at a barrier before a tile load asks for the rows.
    template <bool FP8>
    DFX_D bool rope_fresh_rows_of_chunk(int n_units) const {
        const int t = thread_number_here(wave_s);
        const bool starts = t < n_units && (units[t].flags & kUnitFreshStart) != 0;
        const uint64_t votes = __ballot(starts);
        constexpr int kBallots = kGrowTables ? 4 : 2;  // waves whose ballots cover a table
        if (wave_s < kBallots && t == wave_s * 64) {
            misc[20 + 2 * wave_s] = static_cast<int>(votes);
            misc[21 + 2 * wave_s] = static_cast<int>(votes >> 32);
        }
        __syncthreads();
        static_assert(C::kPlanUnits <= 128 && NW >= kBallots, "the ballots cover a table");
        bool any = false;
        for (int w = 0; w < kBallots; ++w) {
            uint64_t m = (static_cast<uint64_t>(static_cast<uint32_t>(uniform(misc[21 + 2 * w]))) << 32) |
                         static_cast<uint32_t>(uniform(misc[20 + 2 * w]));
            while (m != 0) {
                const int r = w * 64 + __builtin_ctzll(m);
                m &= m - 1;
                // (the sequence's fresh rows from the descriptors: the first band of a fresh tile names its first row,
                // the unit the tile's place among the fresh rows and their number -- no trip to the offsets array)
                const int64_t n0 = -1 - static_cast<int64_t>(uniform(bands[r * NW].is_ctx)) - uniform(units[r].base);
                rope_fresh_rows<FP8>(n0, n0 + uniform(units[r].limit), uniform(units[r].kvh));
                any = true;
            }
        }
        return any;
    }

    // ---- distinct layout: what the loads cannot do ---------------------------------------------------
    // The V half of the stage of a fresh tile holds the rows as they lie in memory (row-major, swizzled as a
    // unified-layout tile); the step reads d-major.  Transposed in place through registers: every thread
    // takes two 16-byte chunks (8 values of one token), all read, barrier, all write two bytes at a time.
    // Every thread of the workgroup; the tile has landed (barrier behind the wait); ends with a barrier.
    DFX_D void transpose_fresh_v(int rel) const {
        static_assert(!DISTINCT || C::THREADS * 2 == C::TN * L::CPR, "two chunks per thread");
        uint8_t* vt = lds + C::STAGES_OFF + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES + C::MAT_BYTES;
        const int t = thread_number_here(wave_s);
        u32x4 x[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = t + C::THREADS * i;
            x[i] = *reinterpret_cast<const u32x4*>(vt + L::chunk_offset(idx / L::CPR, idx % L::CPR));
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = t + C::THREADS * i;
            const int row = idx / L::CPR, cc = idx % L::CPR;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t w = x[i][j >> 1];
                *reinterpret_cast<uint16_t*>(vt + Base::vt_chunk_offset(cc * 8 + j, row >> 3) + (row & 7) * 2) =
                    static_cast<uint16_t>((j & 1) ? (w >> 16) : w);
            }
        }
        __syncthreads();
    }
    // A tile of cached rows that ends before its 64th token: the V^T rows hold whatever the page holds behind
    // the sequence's end (the chunk with the last valid token) or copies of that chunk (the ones after it), and
    // a probability of zero does not make a NaN or an infinity harmless.  Zeroes the tokens from n_valid on.
    // Every thread of the workgroup; the tile has landed; ends with a barrier.
    DFX_D void clear_v_tail(int rel, int n_valid) const {
        uint8_t* vt = lds + C::STAGES_OFF + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES + C::MAT_BYTES;
        const int t = thread_number_here(wave_s);
#pragma unroll
        for (int i = 0; i < HD * 8 / C::THREADS; ++i) {
            const int idx = t + C::THREADS * i;
            const int d = idx >> 3, tc = idx & 7;
            const int keep = n_valid - tc * 8;  // tokens of this chunk to keep
            if (keep >= 8) continue;
            u32x4* p = reinterpret_cast<u32x4*>(vt + Base::vt_chunk_offset(d, tc));
            u32x4 v = {0, 0, 0, 0};
            if (keep > 0) {
                v = *p;
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] &= (2 * k < keep ? 0x0000ffffu : 0u) | (2 * k + 1 < keep ? 0xffff0000u : 0u);
            }
            *p = v;
        }
        __syncthreads();
    }

    // First key position the lane's query row does not see under the block-causal mask (fresh tiles
    // only).  Worked out where a tile needs it, once or twice per item, rather than kept per item: a
    // value that lives through the tile loop takes one of the few registers the compiler has there.
    DFX_D int visible_limit(const UnitDesc& d) const {
        const int q_len = uniform(d.q_len);
        const int r = this->row_of(uniform(d.rt), 0);
        const int i = r < a.group * q_len ? r % q_len : 0;
        // (the divisor made opaque here: its reciprocal, worked out once ahead of the tile loop, would be
        // kept in scratch, and the reload waits for every tile load in flight)
        int dbs = a.dbs;
        asm volatile("" : "+s"(dbs));
        return (i / dbs + 1) * dbs;
    }
    // Under the block-causal mask: the fresh key position up to which every query row of row tile rt of
    // an item with q_len query positions sees everything.  The tile's rows are (head of the group, query
    // position) pairs, position minor: within one head the first row has the lowest position, across
    // heads position 0 is among them.
    DFX_D int clear_limit(int rt, int q_len) const {
        const int r_lo = rt * C::RT;
        const int r_hi = min(r_lo + C::RT, a.group * q_len) - 1;
        const int g_lo = r_lo / q_len;
        const int first_pos = g_lo == r_hi / q_len ? r_lo - g_lo * q_len : 0;
        int dbs = a.dbs;
        asm volatile("" : "+s"(dbs));
        return (first_pos / dbs + 1) * dbs;
    }
    // The same for the 32 rows of this wave alone (row_of(rt, 0) over its lanes), which is what decides whether
    // the wave masks a tile: never below clear_limit() of the whole tile.  Negative (minus the limit) if the
    // wave's rows do not all see the same keys -- with a diffusion block of 32 positions or a multiple and
    // items that begin on a block boundary they do: every lane's visible_limit() is this value then, a tile
    // is masked with one threshold for the wave, and the waves of a row tile that spans several blocks each
    // mask only the tile their own block ends in.  A wave without rows: never masks.
    DFX_D int wave_clear_limit(int rt, int q_len) const {
        const int n_rows = a.group * q_len;
        const int r_lo = rt * C::RT + wave * 32;
        if (r_lo >= n_rows) return 0x7fffffff;
        const int g_lo = r_lo / q_len;
        const int p_lo = r_lo - g_lo * q_len;
        const int p_hi = p_lo + min(31, n_rows - 1 - r_lo);  // in the head of the first row, if it is below q_len
        int dbs = a.dbs;
        asm volatile("" : "+s"(dbs));
        if (p_hi >= q_len) return -dbs;  // several heads: position 0 is among the rows
        const int clear = (p_lo / dbs + 1) * dbs;
        return p_hi < clear ? clear : -clear;
    }
    // Both at once, waiting for every outstanding load of the wave.
    DFX_D void begin_item_hidden(const UnitDesc& d) {
        request_queries(d);
        wait_async_loads<0>();
        adopt_item(d);
    }

    DFX_D TileInfo tile_info_of(int rel) const {
        const UnitDesc u = units[rel];
        TileInfo t;
        t.base = uniform(u.base);
        t.limit = uniform(u.limit);
        t.is_ctx = (uniform(u.flags) & kUnitCtx) != 0;
        t.holes = unit_holes(uniform(u.flags));
        t.c_tile = a.c;
        t.v_mul = 1.0f;
        return t;
    }

    // Close the item whose last unit of this workgroup's piece is planned unit `last_rel`.
    // Returns 0 (the run goes on in the next plan), 1 (rows written), 2 (piece stored), 3 (pieces merged).
    DFX_D int finish_run(int last_rel, const WgSplit& split) {
        const UnitDesc e = units[last_rel];
        if (!(uniform(e.flags) & kUnitLast)) return 0;
        this->outputs_ready();
        float l_tot[NB];
        this->row_sums(l_tot);
        if (uniform(e.flags) & kUnitComplete) {
            this->store_output(uniform(e.rt), l_tot);
            return 1;
        }
        return finish_cut_item(*this, uniform(e.rt), rel_base + uniform(e.item_rel), uniform(e.n_tiles), split,
                               uniform(e.partner), l_tot, misc + kMaxWaves + 1, rel_base) ? 3 : 2;
    }

    // Step r of the pipelined loop (softmax and O^T of unit r, S^T of unit r + 1, tile loads of unit
    // r + 3; r + 5 with a ring of codes) is "plain" if it needs none of the loop's case distinctions:
    // unit r + 1 follows in the same run and needs no mask, and the unit to fetch is in the table with
    // every wave's band a full band of cached rows.  Writes into the flags of every unit r the number of consecutive plain steps
    // from step r on (kUnitPlainShift).  One wave, one lane per unit; the table is complete
    // (barrier) and nobody else writes flags now; readers come behind a later barrier.
    static constexpr int kPlainAhead = KVB == 1 ? C::kStages + 1 : C::kStages - 1;  // step r fetches unit r + kPlainAhead
    // fresh_bands: the kernel's plain steps fetch bands of fresh rows (a launch without a cache) instead of cached ones.
    DFX_D void mark_plain_steps(int n_units, bool fresh_bands = false) const {
        if (wave_s != NW - 1) return;
        const int lane_here = thread_number_here(0);
        // 64 units at a time, the last ones first: a stretch that reaches the end of its 64 goes on with
        // the count of the unit behind it
        int next_count = 0;
        for (int first = ((n_units - 1) / 64) * 64; first >= 0; first -= 64) {
            const int r = first + lane_here;
            bool plain = false;
            int flags = 0;
            if (r + kPlainAhead < n_units) {
                bool full = true;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const BandDesc& b = bands[(r + kPlainAhead) * NW + w];
                    full = full && (b.is_ctx > 0) != fresh_bands && b.last >= (DISTINCT ? C::TN : C::ROWS_PER_WAVE) - 1;
                }
                flags = units[r].flags;
                const UnitDesc& nxt = units[r + 1];
                bool masked = nxt.base + C::TN > nxt.limit || unit_holes(nxt.flags) != 0;
                if (!(nxt.flags & kUnitCtx) && a.mask_mode == DFX_MASK_BLOCK_CAUSAL)
                    masked = masked || nxt.base + C::TN > clear_limit(nxt.rt, nxt.q_len);
                plain = full && !(flags & kUnitLast) && !masked;
                // distinct layout: the step's own tile must need nothing done to its V^T rows first (a fresh tile is
                // transposed, one that ends early or lies on a missing page is cleared: the general step does that)
                if (DISTINCT) plain = plain && (flags & kUnitCtx) != 0 && units[r].base + C::TN <= units[r].limit && unit_holes(flags) == 0;
                // codes: the step also widens K of unit r + 2 and V of unit r + 1, and a plain one only knows cached rows
                if (KVB == 1) plain = plain && (flags & nxt.flags & units[r + 2].flags & kUnitCtx) != 0;
            }
            const uint64_t votes = __ballot(plain);
            const uint64_t not_plain = ~(votes >> lane_here);  // bit j: step r + j is not plain (bits past 63 - lane: set)
            int count = __builtin_ctzll(not_plain);
            if (count == 64 - lane_here) count += next_count;  // (the stretch runs into the next 64)
            if (plain) units[r].flags = flags | (count << kUnitPlainShift);  // (at most kPlanUnits: the flags' top bits are free)
            next_count = (votes & 1) ? uniform(count) : 0;     // lane 0 holds the first unit of these 64
        }
    }
    // ---- the workgroup's work -----------------------------------------------------------------
    // Calls body(n_units) for every chunk of the workgroup's units, with the chunk's descriptors in
    // the LDS tables and begin / end set to the range of the unit space the chunk belongs to.  The
    // descriptors come from the plan buffer if the launch has a valid one; otherwise the workgroup
    // works out its equal share of the unit space and its descriptors itself.
    WgSplit split;
    template <typename Body>
    DFX_D void for_each_chunk(Body&& body) {
        for_each_chunk(body, [](const WgWork&) {});
    }
    // on_work(w): called as soon as a plan has told what the workgroup does (w: uniform values),
    // before its descriptors are fetched, if it has anything to do.
    template <typename Body, typename OnWork>
    DFX_D void for_each_chunk(Body&& body, OnWork&& on_work) {
        const PlanHeader* hdr = reinterpret_cast<const PlanHeader*>(a.plan);
        bool planned = false;
        WgWork w;
        w.a0 = w.a1 = w.b0 = w.b1 = 0;
        w.partner = -1;
        w.ubase = 0;
        int64_t total = 0;
        int n_active = 0, plan_mode = 0;
        const UnitDesc* g_units = nullptr;
        const BandDesc* g_bands = nullptr;
        if (hdr != nullptr) {
            // One trip to memory: the header and this workgroup's entry together (the host has told
            // where the tables start; a header that says otherwise makes the plan unusable).
            const PlanLayout lay = plan_layout(a.num_seqs, a.n_wg, a.plan_capacity, NW);
            const u32x4* gh = reinterpret_cast<const u32x4*>(hdr);
            const u32x4* gw = reinterpret_cast<const u32x4*>(reinterpret_cast<const WgWork*>(a.plan + lay.work_off) + blockIdx.x);
            const u32x4 h0 = gh[0], h1 = gh[1];
            const u32x4 g0 = gw[0], g1 = gw[1], g2 = gw[2], g3 = gw[3];
            auto u = [](uint32_t v) { return uniform(static_cast<int>(v)); };
            auto u64 = [&](uint32_t lo, uint32_t hi) { return (static_cast<int64_t>(u(hi)) << 32) | static_cast<uint32_t>(u(lo)); };
            planned = u(h0[0]) == static_cast<int>(kPlanMagic) && u(h0[1]) == static_cast<int>(a.plan_signature) &&
                      u(h1[2]) == a.plan_capacity;
            if (planned) {
                n_active = u(h0[2]);
                plan_mode = u(h0[3]);
                per_head = u(h1[0]);
                total = u(h1[1]);
                if (total == 0) return;
                w.a0 = u64(g0[0], g0[1]);
                w.a1 = u64(g0[2], g0[3]);
                w.b0 = u64(g1[0], g1[1]);
                w.b1 = u64(g1[2], g1[3]);
                w.partner = u(g2[0]);
                w.ubase = u(g2[1]);
                w.q0 = u(g2[2]);
                w.q_len = u(g2[3]);
                w.kvh = u(g3[0]);
                w.rt = u(g3[1]);
                g_units = reinterpret_cast<const UnitDesc*>(a.plan + lay.units_off);
                g_bands = reinterpret_cast<const BandDesc*>(a.plan + lay.bands_off);
                if (w.a1 + w.b1 > w.a0 + w.b0) on_work(w);
            }
        }
        if (!planned) {
            const UnitSummary summary = build_unit_prefix<C::RT>(a, prefix, misc);
            per_head = summary.per_head;
            total = static_cast<int64_t>(per_head) * a.h_kv;
            if (total == 0) return;
            n_active = a.fixed_wg ? a.n_wg
                                  : effective_workgroups(total, static_cast<int64_t>(summary.items) * a.h_kv,
                                                         summary.max_tiles, a.n_wg);
        }
        split = make_wg_split(total, n_active);
        if (planned && plan_mode == 2) {
            // the plan has placed the cut points itself: its table, for the owners of a cut item's pieces,
            // into the space the unit prefix takes when the kernel plans (visible behind the barriers
            // of the first chunk; first read when a run ends)
            const int32_t* g_bounds = reinterpret_cast<const int32_t*>(a.plan + plan_layout(a.num_seqs, a.n_wg, a.plan_capacity, NW).bounds_off);
            for (int i = thread_number_here(wave_s); i <= n_active; i += C::THREADS) prefix[i] = g_bounds[i];
            split.bounds = prefix;
        }
        if constexpr (kGrowTables) {
            if (planned) {
                // [cut points][scratch][unit table][band table] up to where the stages begin
                const int bounds_bytes = plan_mode == 2 ? ((n_active + 1) * 4 + 255) & ~255 : 0;
                const int per_unit = static_cast<int>(sizeof(UnitDesc)) + NW * static_cast<int>(sizeof(BandDesc));
                const int cap = (C::STAGES_OFF - bounds_bytes - C::S::MISC_BYTES) / per_unit;
                if (cap > C::kPlanUnits) {
                    chunk_cap = min(cap, 256);  // (a thread per unit where the fresh rows' beginnings are looked for)
                    misc = reinterpret_cast<int*>(lds + bounds_bytes);
                    units = reinterpret_cast<UnitDesc*>(lds + bounds_bytes + C::S::MISC_BYTES);
                    bands = reinterpret_cast<BandDesc*>(reinterpret_cast<uint8_t*>(units) + chunk_cap * static_cast<int>(sizeof(UnitDesc)));
                }
            }
        }
        if (!planned && static_cast<int>(blockIdx.x) < n_active) {
            w.a0 = split.first(blockIdx.x);
            w.a1 = split.first(blockIdx.x + 1);
        }
        rel_base = w.a0;
        // With a plan the descriptors of both ranges follow each other in its unit list: one list here
        // too, so that tiles of the second range are already on their way while the first is finished.
        const int64_t n_total = (w.a1 - w.a0) + (planned ? w.b1 - w.b0 : 0);
        begin = w.a0;
        end = planned ? w.a0 + n_total : w.a1;  // (with a plan only the length matters from here on)
        for (int64_t done = 0; done < n_total; done += chunk_cap) {
            const int n_units = static_cast<int>(min(static_cast<int64_t>(chunk_cap), n_total - done));
            __syncthreads();  // every wave is done with the previous descriptors and their stages
            if (planned) {
                // descriptors are multiples of 16 bytes: copied as such.  The lane's addresses are worked
                // out here: computed ahead of the chunk loop they end up in scratch, and every reload is
                // a trip to memory in front of the first tile.
                const int t = thread_number_here(wave_s);
                const u32x4* su = reinterpret_cast<const u32x4*>(g_units + w.ubase + done);
                u32x4* du = reinterpret_cast<u32x4*>(units);
                const u32x4* sb = reinterpret_cast<const u32x4*>(g_bands + (w.ubase + done) * NW);
                u32x4* db = reinterpret_cast<u32x4*>(bands);
                for (int i = t; i < n_units * 3; i += C::THREADS) du[i] = su[i];
                for (int i = t; i < n_units * NW; i += C::THREADS) db[i] = sb[i];
            } else {
                plan_units(begin + done, n_units);
            }
            __syncthreads();
            body(n_units);
        }
    }

    // Planned start of the pipelined kernel: one trip to memory (scalar loads of the plan's header,
    // the workgroup's entry and the band descriptors of its waves' first units), after which every
    // wave requests, in this order, its share of the descriptor tables (straight into LDS, as the
    // tiles travel), the query rows of the first item and the tiles of the ring fill.  The tables are
    // then the oldest loads in flight and are waited for alone.  body(n_units, prefilled): prefilled
    // units have been requested together with the first item's query rows (0: nothing has, the
    // classic start; later chunks of a long range; launches without a usable plan).
    static constexpr int kPrefill = 2;  // units requested with the first item's query rows
    bool queries_requested = false;     // ... which the planned start has requested (the first chunk's body resets it)
    template <typename Body>
    DFX_D void for_each_chunk_prefetched(Body&& body) {
        static_assert(HIDDEN && KVB == 2 && C::kPlanUnits * NW <= 2 * C::THREADS, "table shares below");
        constexpr int QL = C::S::NSLAB, UL = C::LOADS_PER_UNIT;  // loads of a lane's query row, of a wave's share of a unit
        bool planned = false;
        int64_t n_total = 0, n_first = 0, ubase = 0;
        int n_active = 0, plan_mode = 0, prefilled = 0;
        const UnitDesc* g_units = nullptr;
        const BandDesc* g_bands = nullptr;
        if (a.plan != nullptr) {
            // All of it in one trip: five scalar loads issued together.  (The host has told where the
            // tables start and checked that the buffer holds them: they may be read before the header has
            // said whether the plan is this launch's.)
            const PlanLayout lay = plan_layout(a.num_seqs, a.n_wg, a.plan_capacity, NW);
            const uint8_t* hp = a.plan;
            const uint8_t* ep = a.plan + lay.work_off + static_cast<int64_t>(blockIdx.x) * sizeof(WgWork);
            const uint8_t* fp = a.plan + lay.first_off + (static_cast<int64_t>(blockIdx.x) * kPlanFirst * NW + wave_s) * sizeof(BandDesc);
            typedef uint32_t words8 __attribute__((ext_vector_type(8)));
            typedef uint32_t words16 __attribute__((ext_vector_type(16)));
            words8 h;
            words16 e;
            u32x4 f[kPrefill];
            static_assert(NW * sizeof(BandDesc) == 0x80 && sizeof(WgWork) == 64 && kPlanFirst >= kPrefill && kPrefill == 2, "the loads below");
            asm volatile("s_load_dwordx8 %0, %4, 0x0\n\ts_load_dwordx16 %1, %5, 0x0\n\ts_load_dwordx4 %2, %6, 0x0\n\t"
                         "s_load_dwordx4 %3, %6, 0x80\n\ts_waitcnt lgkmcnt(0)"
                         : "=&s"(h), "=&s"(e), "=&s"(f[0]), "=&s"(f[1])
                         : "s"(hp), "s"(ep), "s"(fp)
                         : "memory");
            planned = (h[0] == kPlanMagic) & (h[1] == a.plan_signature) & (static_cast<int32_t>(h[6]) == a.plan_capacity);
            if (planned) {
                n_active = static_cast<int>(h[2]);
                plan_mode = static_cast<int>(h[3]);
                per_head = static_cast<int>(h[4]);
                const int64_t total = static_cast<int>(h[5]);
                if (total == 0) return;
                auto i64 = [&](int i) { return static_cast<int64_t>((static_cast<uint64_t>(e[i + 1]) << 32) | e[i]); };
                const int64_t a0 = i64(0);
                n_first = i64(2) - a0;
                n_total = n_first + (i64(6) - i64(4));
                ubase = static_cast<int32_t>(e[9]);
                if (n_total <= 0) return;
                split = make_wg_split(total, n_active);
                if (plan_mode == 2) split.bounds = prefix;
                rel_base = begin = a0;
                end = a0 + n_total;
                g_units = reinterpret_cast<const UnitDesc*>(a.plan + lay.units_off) + ubase;
                g_bands = reinterpret_cast<const BandDesc*>(a.plan + lay.bands_off) + ubase * NW;
                const int n_units = static_cast<int>(min(static_cast<int64_t>(C::kPlanUnits), n_total));
                {
                    const int t = thread_number_here(wave_s);
                    const uint32_t share = static_cast<uint32_t>(wave_s) * 1024;
                    if (t < n_units * 3) async_load16(g_units, t * 16, lds_of(units) + share);
                    if (t < n_units * NW) async_load16(g_bands, t * 16, lds_of(bands) + share);
                    if (t + C::THREADS < n_units * NW)
                        async_load16(reinterpret_cast<const uint8_t*>(g_bands) + C::THREADS * 16, t * 16, lds_of(bands) + C::THREADS * 16 + share);
                    // the plan's cut points, for the owners of a cut item's pieces (first read when a run ends)
                    if (plan_mode == 2 && t * 4 <= n_active) async_load16(a.plan + lay.bounds_off, t * 16, lds_of(prefix) + share);
                }
                UnitDesc d;
                d.q0 = static_cast<int32_t>(e[10]);
                d.q_len = static_cast<int32_t>(e[11]);
                d.kvh = static_cast<int32_t>(e[12]);
                d.rt = static_cast<int32_t>(e[13]);
                request_queries(d);
                // Two units, not the ring's three: with the third behind them the query rows land later, and
                // the launch came out no faster than without any of this (paired runs, 64 sequences x 4 KV heads
                // of 8-32 tiles: one unit -0.2 us, two -0.4, three +0.4 against the copy of the tables through
                // registers).  (The plan repeats the first units of the workgroup's first range only.)
                prefilled = static_cast<int>(min(static_cast<int64_t>(min(n_units, kPrefill)), n_first > 0 ? n_first : n_total));
                // (with the rotary embedding inside the launch a tile of fresh rows waits for their rotation)
                if (a.rope_table != nullptr) prefilled = static_cast<int32_t>(f[0][3]) <= 0 ? 0 : (prefilled == 2 && static_cast<int32_t>(f[1][3]) <= 0 ? 1 : prefilled);
                queries_requested = true;
#pragma unroll
                for (int u = 0; u < kPrefill; ++u) {
                    if (u < prefilled) {
                        BandDesc b;
                        b.off = static_cast<int64_t>((static_cast<uint64_t>(f[u][1]) << 32) | f[u][0]);
                        b.last = static_cast<int32_t>(f[u][2]);
                        b.is_ctx = static_cast<int32_t>(f[u][3]);
                        issue_unit_desc(b, u);
                    }
                }
                // the tables are this wave's oldest loads: 8 of query rows and 4 per unit are younger
                static_assert(kPrefill == 2, "wait counts");
                if (prefilled == 2) wait_async_loads<QL + 2 * UL>();
                else if (prefilled == 1) wait_async_loads<QL + UL>();
                else wait_async_loads<QL>();
            }
        }
        if (!planned) {
            const UnitSummary summary = build_unit_prefix<C::RT>(a, prefix, misc);
            per_head = summary.per_head;
            const int64_t total = static_cast<int64_t>(per_head) * a.h_kv;
            if (total == 0) return;
            n_active = a.fixed_wg ? a.n_wg
                                  : effective_workgroups(total, static_cast<int64_t>(summary.items) * a.h_kv, summary.max_tiles, a.n_wg);
            split = make_wg_split(total, n_active);
            if (static_cast<int>(blockIdx.x) >= n_active) return;
            rel_base = begin = split.first(blockIdx.x);
            end = split.first(blockIdx.x + 1);
            n_total = end - begin;
        }
        for (int64_t done = 0; done < n_total; done += C::kPlanUnits) {
            const int n_units = static_cast<int>(min(static_cast<int64_t>(C::kPlanUnits), n_total - done));
            const bool prefetched = planned && done == 0;
            if (!prefetched) {
                __syncthreads();  // every wave is done with the previous descriptors and their stages
                if (planned) {
                    const int t = thread_number_here(wave_s);
                    const u32x4* su = reinterpret_cast<const u32x4*>(g_units + done);
                    u32x4* du = reinterpret_cast<u32x4*>(units);
                    const u32x4* sb = reinterpret_cast<const u32x4*>(g_bands + done * NW);
                    u32x4* db = reinterpret_cast<u32x4*>(bands);
                    for (int i = t; i < n_units * 3; i += C::THREADS) du[i] = su[i];
                    for (int i = t; i < n_units * NW; i += C::THREADS) db[i] = sb[i];
                } else {
                    plan_units(begin + done, n_units);
                }
            }
            __syncthreads();
            body(n_units, prefetched ? prefilled : 0);
        }
    }
    DFX_D static uint32_t lds_of(const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); }

    // Wait until at most `younger` units' loads of this wave are outstanding (younger <= 2).
    DFX_D static void wait_younger(int younger) {
        if (younger >= 2) wait_async_loads<2 * C::LOADS_PER_UNIT>();
        else if (younger == 1) wait_async_loads<C::LOADS_PER_UNIT>();
        else wait_async_loads<0>();
    }
};

template <int HD, int NB, int NW, bool COMPACT, bool DISTINCT = false>
__global__ void __launch_bounds__(64 * NW, COMPACT ? 2 : 1) paged_attn_stream_kernel(const KArgs a) {
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    using C = StreamCfg<HD, NB, NW, COMPACT>;
    StreamAttn<HD, NB, NW, COMPACT, 2, false, DISTINCT> at(a, smem);
    // The fused cache store comes first, while next to nothing is live in registers: anywhere
    // later its address arithmetic would push values of the tile loop out of their registers.
    if constexpr (!DISTINCT) store_fresh_rows<HD, false>(a);
    at.for_each_chunk([&](int n_units) {
        const WgSplit& split = at.split;
        // An item that opens with this plan: its query rows are requested ahead of the ring fill,
        // so that their (cold) latency runs concurrently with that of the first tiles.
        const bool opens = (uniform(at.units[0].flags) & kUnitFirst) != 0;
        if (opens) at.begin_item(at.units[0], false);
        int issued = 0;  // ring fill: kStages - 1 units in flight
        for (; issued < C::kStages - 1 && issued < n_units; ++issued) at.issue_unit(issued);
        at.touch_queries();  // unconditional: the compiler must see no path into the tile loop with these loads pending

        int rel = 0;
        while (rel < n_units) {
            // a run of units of one item: all of this workgroup's piece of it, or up to the end of the plan
            const UnitDesc d = at.units[rel];
            const int flags = uniform(d.flags);
            const int run_end = min(rel + uniform(d.run), n_units);
            if ((flags & kUnitFirst) && rel != 0) at.begin_item(d);
            for (; rel < run_end; ++rel) {
                // the unit must have landed: only younger units may still be outstanding
                at.wait_younger(issued - rel - 1);
                __builtin_amdgcn_s_barrier();
                // every wave has finished the previous unit: its stage may be overwritten
                if (issued < n_units) at.issue_unit(issued++);

                const UnitDesc u = at.units[rel];
                TileInfo t;
                t.base = uniform(u.base);
                t.limit = uniform(u.limit);
                t.is_ctx = (uniform(u.flags) & kUnitCtx) != 0;
                t.holes = unit_holes(uniform(u.flags));
                t.c_tile = a.c;
                t.v_mul = 1.0f;
                const uint8_t* k_tile = smem + C::STAGES_OFF + (static_cast<unsigned>(rel) % C::kStages) * C::STAGE_BYTES;
                if constexpr (DISTINCT) {  // (once or twice per item)
                    if (!t.is_ctx) at.transpose_fresh_v(rel);
                    else if (t.holes != 0) at.clear_v_tail(rel, 0);  // (a page without a table entry: page 0 was read in its place)
                    else if (t.base + C::TN > t.limit) at.clear_v_tail(rel, t.limit - t.base);
                }
                if (at.wave < a.busy_waves) {  // waves whose 32 rows exist in no item of this launch only fetch
                    f32x16 sc[2][NB];
                    bf16x8 pb[NB][2][2];
                    if constexpr (DISTINCT) {
                        at.scores_chunk_major(k_tile, sc);
                        at.template softmax_tile<false, C::ROWS_PER_WAVE, true>(sc, t, pb, [&] { at.outputs_ready(); });
                        at.accumulate_dmajor(k_tile + C::MAT_BYTES, pb);
                    } else {
                        at.scores(k_tile, sc);
                        at.template softmax_tile<false, C::ROWS_PER_WAVE>(sc, t, pb, [&] { at.outputs_ready(); });
                        at.accumulate(k_tile + C::MAT_BYTES, pb);
                    }
                } else {
                    at.outputs_untouched();
                }
            }
            at.finish_run(rel - 1, split);
        }
    });
}

// FP8-E4M3 context cache (fresh K/V stay bf16).  The ring stages hold the codes as stored; in
// step `rel` a wave first widens its own rows of unit rel + 1 into the bf16 tile the matrix
// instructions of the previous step have just released, then computes unit rel from the other
// bf16 tile.  The ring needs no barrier (a stage's band is written and read by one wave only);
// the one barrier per step orders the two bf16 tiles.
// NB query blocks per wave: 1 with head_dim 128 (8 waves for up to 256 rows); with head_dim 64 a
// 64-token tile of codes is 4 KiB, one load instruction each for 4 waves, so 4 waves take 1 or 2.
template <int HD, int NB, int NW>
__global__ void __launch_bounds__(64 * NW, 1) paged_attn_stream_fp8_kernel(const KArgs a) {
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    using C = StreamCfg<HD, NB, NW, false, 1>;
    StreamAttn<HD, NB, NW, false, 1> at(a, smem);
    store_fresh_rows<HD, true>(a);  // first, as in the bf16 kernel
    at.for_each_chunk([&](int n_units) {
        const WgSplit& split = at.split;
        const bool opens = (uniform(at.units[0].flags) & kUnitFirst) != 0;
        if (opens) at.begin_item(at.units[0], false);  // query rows ahead of the ring fill, as in the bf16 kernel
        int issued = 0;
        for (; issued < C::kStages - 1 && issued < n_units; ++issued) at.issue_unit(issued);
        at.touch_queries();  // unconditional: the compiler must see no path into the tile loop with these loads pending
        at.wait_younger(issued - 1);
        at.widen_unit(0);

        int rel = 0;
        while (rel < n_units) {
            const UnitDesc d = at.units[rel];
            const int flags = uniform(d.flags);
            const int run_end = min(rel + uniform(d.run), n_units);
            if ((flags & kUnitFirst) && rel != 0) at.begin_item(d);
            for (; rel < run_end; ++rel) {
                // stage (rel + 3) % 4 held unit rel - 1, which this wave widened a step ago
                if (issued < n_units) at.issue_unit(issued++);
                if (rel + 1 < n_units) at.wait_younger(issued - rel - 2);
                // every wave has widened its rows of unit rel and is done computing unit rel - 1
                __builtin_amdgcn_s_barrier();
                if (rel + 1 < n_units) at.widen_unit(rel + 1);

                const UnitDesc u = at.units[rel];
                TileInfo t;
                t.base = uniform(u.base);
                t.limit = uniform(u.limit);
                t.is_ctx = (uniform(u.flags) & kUnitCtx) != 0;
                t.holes = unit_holes(uniform(u.flags));
                t.c_tile = t.is_ctx ? a.c * at.k_mul : a.c;
                t.v_mul = t.is_ctx ? 1.0f : at.v_inv;
                const uint8_t* k_tile = at.wide_tile(rel);
                if (at.wave < a.busy_waves) {
                    f32x16 sc[2][NB];
                    at.scores(k_tile, sc);
                    bf16x8 pb[NB][2][2];
                    at.template softmax_tile<true, C::ROWS_PER_WAVE>(sc, t, pb, [&] { at.outputs_ready(); });
                    at.accumulate(k_tile + TileLayout<HD>::MAT_BYTES, pb);
                } else {
                    at.outputs_untouched();
                }
            }
            at.finish_run(rel - 1, split);
        }
    });
}

// The bf16 streaming kernel with the software-pipelined tile step of attn_pipe_gen.h (head_dim
// 128, 4-stage ring).  One step of its loop computes S^T of unit r + 1 and the softmax and O^T of
// unit r, so the ring holds the K tile of the next unit and the V tile of the current one.
//
// amdgpu_num_vgpr(32): the compiler allocates v0..v31 and a0..a31 only; the registers above hold
// the matrix state of the generated blocks, which the compiler never sees.
//
// PREFILL: the variant for launches without a cache.  Every tile
// is one of fresh rows there, and its plain steps fetch full bands of those the way the other variant's
// fetch bands of cached rows (which keeps its fresh tiles, one or two per item, on the general step).
// The blocks of attn_pipe_gen.h for the tile layout of the kernel's cache and its head_dim.
template <bool DISTINCT, int HD = 128>
struct PipeBlocks {
    static_assert(HD == 128 || (HD == 64 && !DISTINCT), "families of blocks generated");
#define DFX_PIPE_BLOCK(name, params, args)                     \
    DFX_D static void name params {                            \
        if constexpr (DISTINCT) pipe_d_##name args;            \
        else if constexpr (HD == 64) pipe64_##name args;       \
        else pipe_##name args;                                 \
    }
#define pipe64_mask_a_8 pipe_mask_a_8
#define pipe64_mask_a_16 pipe_mask_a_16
#define pipe64_mask_b_8 pipe_mask_b_8
#define pipe64_mask_b_16 pipe_mask_b_16
    DFX_PIPE_BLOCK(first_scores, (uint32_t k, float& mx), (k, mx))
    DFX_PIPE_BLOCK(mask_a_8, (int thr, uint32_t holes, float& mx), (thr, holes, mx))
    DFX_PIPE_BLOCK(mask_a_16, (int thr, uint32_t holes, float& mx), (thr, holes, mx))
    DFX_PIPE_BLOCK(mask_b_8, (int thr, uint32_t holes, float& mx), (thr, holes, mx))
    DFX_PIPE_BLOCK(mask_b_16, (int thr, uint32_t holes, float& mx), (thr, holes, mx))
    DFX_PIPE_BLOCK(step_ab_x, (uint32_t k, uint32_t v, float c, float nm, float& l), (k, v, c, nm, l))
    DFX_PIPE_BLOCK(step_ab_y, (float c, float nm, float& l, float& mx), (c, nm, l, mx))
    DFX_PIPE_BLOCK(step_ba_x, (uint32_t k, uint32_t v, float c, float nm, float& l), (k, v, c, nm, l))
    DFX_PIPE_BLOCK(step_ba_y, (float c, float nm, float& l, float& mx), (c, nm, l, mx))
    DFX_PIPE_BLOCK(last_a_x, (uint32_t v, float c, float nm, float& l), (v, c, nm, l))
    DFX_PIPE_BLOCK(last_a_y, (float c, float nm, float& l), (c, nm, l))
    DFX_PIPE_BLOCK(last_b_x, (uint32_t v, float c, float nm, float& l), (v, c, nm, l))
    DFX_PIPE_BLOCK(last_b_y, (float c, float nm, float& l), (c, nm, l))
    DFX_D static void rescale_outputs(float alpha) {
        if constexpr (HD == 64) pipe64_rescale_outputs(alpha);
        else pipe_rescale_outputs(alpha);
    }
#undef pipe64_mask_a_8
#undef pipe64_mask_a_16
#undef pipe64_mask_b_8
#undef pipe64_mask_b_16
#undef DFX_PIPE_BLOCK
};

// DISTINCT: the cache is in the distinct layout (StreamAttn): the blocks read a chunk-major K tile and a d-major V
// tile, a full tile of cached rows is fetched by pipe_d_issue_band, and the general step first does to its own
// tile's V^T rows what the loads could not (transpose_fresh_v, clear_v_tail); no store, no rotary embedding.
// HD: 128, or 64 (unified layout, launches with a cache or without: the blocks pipe64_*; a wave fetches its 8 rows of
// a tile with one load per matrix; no rotary embedding inside the launch).
template <int NW, bool PREFILL = false, bool DISTINCT = false, int HD = 128>
__global__ void __launch_bounds__(64 * NW, 1) __attribute__((amdgpu_num_vgpr(32)))
paged_attn_pipe_kernel(const KArgs a) {
    static_assert(!(PREFILL && DISTINCT), "a launch without a cache has no cache layout");
    static_assert(HD == 128 || !(PREFILL || DISTINCT), "head_dim 64: one kernel");
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    using C = StreamCfg<HD, 1, NW, false>;
    using SA = StreamAttn<HD, 1, NW, false, 2, true, DISTINCT>;
    using PB = PipeBlocks<DISTINCT, HD>;
    SA at(a, smem);
    pipe_reserve();
    if constexpr (DISTINCT) {
        // a lane per token of a chunk column of K; 8 lanes per row of V^T, the wave's rows 16 w + lane / 8 and 8 further
        uint32_t v[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int d = at.wave * 16 + j * 8 + (at.lane >> 3);
            v[j] = static_cast<uint32_t>(d) * static_cast<uint32_t>(a.vd_sd * 2) + ((at.lane & 7) ^ ((d >> 1) & 7)) * 16;
        }
        pipe_d_set_load_offsets(at.lane * 16, v[0], v[1]);
    } else if constexpr (HD == 64) {
        const int r = at.lane / C::CPR;  // one load covers the wave's 8 rows
        const int chunk = (at.lane % C::CPR) ^ C::swizzle(at.wave * C::ROWS_PER_WAVE + r);
        pipe64_set_load_offsets(static_cast<uint32_t>(r) * static_cast<uint32_t>(a.c_st * 2) + chunk * 16);
    } else {
        uint32_t o[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int r = j * C::RPI + at.lane / C::CPR;
            const int chunk = (at.lane % C::CPR) ^ C::swizzle(at.wave * C::ROWS_PER_WAVE + r);
            o[j] = static_cast<uint32_t>(r) * static_cast<uint32_t>(a.c_st * 2) + chunk * 16;
        }
        pipe_set_load_offsets(o[0], o[1]);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int r = j * C::RPI + at.lane / C::CPR;
            const int chunk = (at.lane % C::CPR) ^ C::swizzle(at.wave * C::ROWS_PER_WAVE + r);
            o[j] = static_cast<uint32_t>(r) * static_cast<uint32_t>(a.kn_st * 2) + chunk * 16;
        }
        if constexpr (PREFILL) {
            pipe_set_fresh_offsets(o[0], o[1]);
            // (no cache: the registers of the cached rows' offsets take those of the fresh V rows)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int r = j * C::RPI + at.lane / C::CPR;
                const int chunk = (at.lane % C::CPR) ^ C::swizzle(at.wave * C::ROWS_PER_WAVE + r);
                o[j] = static_cast<uint32_t>(r) * static_cast<uint32_t>(a.vn_st * 2) + chunk * 16;
            }
            pipe_set_load_offsets(o[0], o[1]);
        }
    }
    const bool rope = !PREFILL && !DISTINCT && HD == 128 && a.rope_table != nullptr;  // (with it the store travels with the rotation of the fresh K rows)
    if constexpr (!DISTINCT) {
        if (!rope) store_fresh_rows<HD, false, 1>(a);
    }
    const bool busy = at.wave < a.busy_waves;  // waves whose 32 rows exist in no item of this launch only fetch
    constexpr int kHoleRows = C::ROWS_PER_WAVE;
    static_assert(kHoleRows == 8 || kHoleRows == 16, "mask blocks of attn_pipe_gen.h");
    // With a plan the query rows of the workgroup's first item and the tiles of the ring fill are
    // requested as soon as its entry of the plan has been read (for_each_chunk_prefetched: `prefilled`
    // units are on their way then, behind the query rows).
    at.for_each_chunk_prefetched([&](int n_units, int prefilled) {
        const WgSplit& split = at.split;
        // An item that opens with this chunk: its query rows first.  Requested behind the ring fill,
        // the wait for them would also wait for every tile of the fill.
        const bool opens = (uniform(at.units[0].flags) & kUnitFirst) != 0;
        if (opens && !at.queries_requested) at.request_queries(at.units[0]);
        at.queries_requested = false;
        // The rotary embedding inside the launch: the fresh K rows of the items that end in this chunk, and the
        // angles of the first item's query rows, requested behind the stores of those rows so that the two
        // trips to memory run together.
        bool rotate_first = false;
        if constexpr (!PREFILL && !DISTINCT && HD == 128) {
            if (rope) {
                int64_t pos = 0;
                if (opens) pos = at.rope_query_position(at.units[0]);
                const bool any = at.template rope_fresh_rows_of_chunk<false>(n_units);
                if (opens) at.request_rope_angles(pos);
                rotate_first = opens;
                if (any) {
                    wait_async_loads<0>();  // this thread's rows are in memory ...
                    __syncthreads();        // ... and so are everybody's, before a tile load asks for them
                }
            }
        }
        // While the query rows are on their way: the marks of the plain steps.  They are first read
        // behind the barrier of the first run's first step; they only add bits to the flags that
        // nobody looks at before.  (Not behind the ring fill: a spilled register reloaded here would
        // wait for every tile of it.)
        at.mark_plain_steps(n_units, PREFILL);
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the marks are written before this wave reaches that barrier
        if (opens) {
            // the query rows: everything in flight, or everything but the tiles requested behind them
            if (prefilled == 0) wait_async_loads<0>();
            else if (prefilled == 1) wait_async_loads<C::LOADS_PER_UNIT>();
            else wait_async_loads<2 * C::LOADS_PER_UNIT>();
            if constexpr (HD == 128) {
                if (rotate_first) pipe_rope_queries();
            }
            at.adopt_item(at.units[0]);
        }
        // The wave's loads of unit u.  Without a cache every band is one of fresh rows, and a full one is fetched by
        // the block the plain steps use (offsets per lane worked out once) instead of the general code.
        auto issue_unit = [&](int u) {
            if constexpr (PREFILL) {
                const BandDesc& b = at.bands[u * NW + at.wave];
                const int tag = uniform(b.is_ctx);
                if (tag <= 0 && uniform(b.last) >= C::ROWS_PER_WAVE - 1) {
                    const int64_t off = (static_cast<int64_t>(uniform(static_cast<int>(b.off >> 32))) << 32) |
                                        static_cast<uint32_t>(uniform(static_cast<int>(b.off)));
                    const int dst = uniform(static_cast<int>(at.stages_lds + (static_cast<unsigned>(u) % C::kStages) * C::STAGE_BYTES +
                                                             at.wave * (C::IPW * 1024)));
                    pipe_issue_band_fresh(reinterpret_cast<const uint8_t*>(a.k_new) + off,
                                          reinterpret_cast<const uint8_t*>(a.v_new) + off + static_cast<int64_t>(-1 - tag) * a.v_fresh_delta, dst);
                    return;
                }
            }
            at.issue_unit(u);
        };
        int issued = prefilled;  // ring fill: kStages - 1 units in flight
        for (; issued < C::kStages - 1 && issued < n_units; ++issued) issue_unit(issued);

        auto tile_of = [&](int r) { return smem + C::STAGES_OFF + (static_cast<unsigned>(r) % C::kStages) * C::STAGE_BYTES; };
        // Unit r must have landed: only younger units may still be outstanding.  Behind the barrier
        // every wave has finished the units before `done` (their K and their V tile), and unit x
        // may overwrite the stage of unit x - kStages while x - kStages < done: `can_issue` says
        // whether the wave has a unit to fetch now.
        auto admit = [&](int r, int done) {
            at.wait_younger(issued - r - 1);
            __builtin_amdgcn_s_barrier();
            return issued < n_units && issued < done + C::kStages;
        };
        // The two waves of a SIMD run half a step apart.  Everything that is not matrix work -- the
        // issue of the tile loads (which keeps a wave standing for hundreds of cycles while memory
        // is busy), the plan entries, the decision about the running maximum -- is done by the lower
        // half of the workgroup behind its matrix work, at the end of a step, and by the upper half
        // in front of it: while one wave of a SIMD does that, the other has the matrix unit.
        const bool compute_first = at.wave < NW / 2;
        // Under the block-causal mask: the fresh key position up to which every query row of the current
        // run's row tile sees everything (set where a run begins).  A fresh tile that ends at or below it
        // needs no mask; in a prefill those are all of a row tile's tiles but the last few.
        // Without a cache (where the staircases are: row tiles of eight diffusion blocks) that limit is the one of
        // this wave's rows (wave_clear_limit(): negative if its rows differ in what they see): one threshold for the
        // wave where they agree, and no mask block for a tile it sees nothing of.  The other variants keep the limit of
        // the row tile and the row-by-row threshold: the second way to the limit costs their tile loop scalar
        // registers, which the compiler then keeps in vector lanes (C3, which masks nothing, +0.7 %).
        int bc_clear = 0;
        // Mask of the score set that holds unit r, if that tile needs one; updates the lane maximum.
        auto mask = [&](int r, bool set_a, float& mx_lane) {
            const TileInfo t = at.tile_info_of(r);
            const int clear = PREFILL && bc_clear < 0 ? -bc_clear : bc_clear;
            const bool bc = !t.is_ctx && a.mask_mode == DFX_MASK_BLOCK_CAUSAL && t.base + C::TN > clear;
            if (!(t.base + C::TN > t.limit || t.holes != 0 || bc)) return;
            int lim = t.limit;
            if constexpr (PREFILL) {
                if (bc) lim = min(lim, bc_clear > 0 ? clear : at.visible_limit(at.units[r]));
                if (bc && bc_clear > 0 && lim <= t.base) {  // the wave's rows see nothing of this tile
                    if (set_a) pipe_hide_a(mx_lane);
                    else pipe_hide_b(mx_lane);
                    return;
                }
            } else {
                if (bc) lim = min(lim, at.visible_limit(at.units[r]));
            }
            const int thr = lim - t.base - (DISTINCT ? 8 : 4) * at.half;
            const uint32_t holes = static_cast<uint32_t>(t.holes);
            if (set_a) {
                if constexpr (kHoleRows == 8) PB::mask_a_8(thr, holes, mx_lane);
                else PB::mask_a_16(thr, holes, mx_lane);
            } else {
                if constexpr (kHoleRows == 8) PB::mask_b_8(thr, holes, mx_lane);
                else PB::mask_b_16(thr, holes, mx_lane);
            }
        };

        int rel = 0;
        while (rel < n_units) {
            // a run of units of one item: all of this workgroup's piece of it, or up to the end of the plan
            const UnitDesc d = at.units[rel];
            const int run_end = min(rel + uniform(d.run), n_units);
            // (an item that opens inside the chunk was adopted when the run before it ended)
            if (a.mask_mode == DFX_MASK_BLOCK_CAUSAL)
                bc_clear = uniform(PREFILL ? at.wave_clear_limit(uniform(d.rt), uniform(d.q_len)) : at.clear_limit(uniform(d.rt), uniform(d.q_len)));

            // S^T of the run's first tile (into score set A), with nothing to overlap it with
            if (admit(rel, rel)) issue_unit(issued++);
            // For the plain steps behind the run's first step (below), read now, with the first tile's
            // matrix work between the reads and their use: how many there are, and the band offset
            // of the unit the first of them fetches (in steady state, which is checked there, step
            // rel + 1 fetches unit rel + 1 + kStages - 1, whatever the first step had to fetch).
            const int plain_word = at.units[min(rel + 1, n_units - 1)].flags;
            auto band_offset = [&](int unit) { return static_cast<uint64_t>(at.bands[unit * NW + at.wave].off); };
            // (fresh rows: the index of the band's first row, from which the V offset follows where v_new has
            // another token stride than k_new; cached rows have one offset for both)
            auto band_row = [&](int unit) { return PREFILL ? -1 - at.bands[unit * NW + at.wave].is_ctx : 0; };
            const uint64_t off_first = band_offset(min(rel + C::kStages, n_units - 1));
            const int row_first = band_row(min(rel + C::kStages, n_units - 1));
            float mx_lane = 0.0f;  // the lane's maximum over the score set that is consumed next
            float neg_m = 0.0f;    // minus the running maximum the exponentials of the next step refer to
            // Raise the running maximum (and rescale O^T and the row sum) if the tile about to be
            // consumed exceeds it by more than the threshold.
            auto prepare = [&] {
                const float m_tile = wave_xor32_max(mx_lane) * a.c;
                float& m_run = at.m_run[0];
                if (__any(m_tile > m_run + kRescaleThreshold)) {
                    const float m_new = fmaxf(m_run, m_tile);
                    // (the first tile of a piece finds every row at -inf and O^T at zero: nothing to rescale)
                    if (__any(m_run != -INFINITY)) {
                        const float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_run - m_new);
                        at.l_run[0] *= alpha;
                        PB::rescale_outputs(alpha);
                    }
                    m_run = m_new;
                }
                neg_m = (m_run == -INFINITY) ? 0.0f : -m_run;
            };
            if (busy) {
                PB::first_scores(at.lds_address(tile_of(rel)) + at.k_lane, mx_lane);
                mask(rel, true, mx_lane);
                if (compute_first) prepare();
            }
            // step r: softmax and O^T of unit r, S^T of unit r + 1; the two score sets swap roles
            // The next item of this chunk, if there is one: its query rows are requested in the last
            // step of this run and waited for behind that step's matrix work, one step later than the
            // youngest tile load in flight was issued, instead of in front of an idle matrix unit.
            const bool next_opens = run_end < n_units;
            // (requested behind the S^T of the run's last tile, the last matrix work that reads the query rows
            // in place -- a step and a half before they are waited for; in the last step where there was no
            // such step, or a plain one)
            bool queries_asked = false;
            auto step = [&](int r, bool cur_is_a) {
                if constexpr (DISTINCT) {  // (unit r landed before the step that read its K tile; every wave comes here)
                    const TileInfo tr = at.tile_info_of(r);
                    if (!tr.is_ctx) at.transpose_fresh_v(r);
                    else if (tr.holes != 0) at.clear_v_tail(r, 0);  // (a page without a table entry: page 0 was read in its place)
                    else if (tr.base + C::TN > tr.limit) at.clear_v_tail(r, tr.limit - tr.base);
                }
                const bool has_next = r + 1 < run_end;
                const bool fetch = has_next && admit(r + 1, r);
                if (!has_next && next_opens && !queries_asked) at.request_queries(at.units[run_end]);
                const bool ask_queries = next_opens && r + 2 == run_end;
                queries_asked = queries_asked || ask_queries;
                if (!compute_first || !busy) {
                    if (fetch) issue_unit(issued);
                    if (busy) prepare();
                }
                if (!busy && ask_queries) at.request_queries(at.units[run_end]);
                if (busy) {
                    const uint32_t v_cur = at.lds_address(tile_of(r) + C::MAT_BYTES) + at.v_lane;
                    if (has_next) {
                        const uint32_t k_next = at.lds_address(tile_of(r + 1)) + at.k_lane;
                        if (cur_is_a) {
                            PB::step_ab_x(k_next, v_cur, a.c, neg_m, at.l_run[0]);
                            if (ask_queries) at.request_queries(at.units[run_end]);
                            PB::step_ab_y(a.c, neg_m, at.l_run[0], mx_lane);
                        } else {
                            PB::step_ba_x(k_next, v_cur, a.c, neg_m, at.l_run[0]);
                            if (ask_queries) at.request_queries(at.units[run_end]);
                            PB::step_ba_y(a.c, neg_m, at.l_run[0], mx_lane);
                        }
                        mask(r + 1, !cur_is_a, mx_lane);
                    } else {
                        if (cur_is_a) {
                            PB::last_a_x(v_cur, a.c, neg_m, at.l_run[0]);
                            PB::last_a_y(a.c, neg_m, at.l_run[0]);
                        } else {
                            PB::last_b_x(v_cur, a.c, neg_m, at.l_run[0]);
                            PB::last_b_y(a.c, neg_m, at.l_run[0]);
                        }
                    }
                    if (compute_first) {
                        if (fetch) issue_unit(issued);
                        if (has_next) prepare();
                    }
                }
                if (fetch) ++issued;
            };
            // A plain step (mark_plain_steps()): the same work with the decisions taken out; `off` is
            // the offset of this wave's band of the unit to fetch.
            auto plain_step = [&](int r, bool cur_is_a, int64_t off, int row) {
                auto issue_band = [&](int dst) {
                    if constexpr (PREFILL) {
                        pipe_issue_band_fresh(reinterpret_cast<const uint8_t*>(a.k_new) + off,
                                              reinterpret_cast<const uint8_t*>(a.v_new) + off + static_cast<int64_t>(row) * a.v_fresh_delta, dst);
                    } else if constexpr (DISTINCT) {
                        const int64_t kvh = static_cast<int64_t>(static_cast<uint64_t>(off) >> 52);
                        const int64_t page = (off >> 20) & 0xffffffffll, in_page = off & 0xfffff;
                        const uint8_t* kb = a.k_cache + (page * a.kd_sp + kvh * a.kd_sh + in_page * 8 + at.wave_s * 2 * a.kd_sc) * 2;
                        pipe_d_issue_band(kb, kb + a.kd_sc * 2, a.v_cache + (page * a.vd_sp + kvh * a.vd_sh + in_page) * 2, dst);
                    } else if constexpr (HD == 64) {
                        pipe64_issue_band(a.k_cache + off, a.v_cache + off, dst);
                    } else {
                        pipe_issue_band(a.k_cache + off, a.v_cache + off, dst);
                    }
                };
                wait_async_loads<C::LOADS_PER_UNIT>();  // unit r + 1 has landed; unit r + 2 may be on its way
                __builtin_amdgcn_s_barrier();
                const int dst = uniform(static_cast<int>(at.stages_lds + (static_cast<unsigned>(issued) % C::kStages) * C::STAGE_BYTES +
                                                         at.wave * (C::IPW * 1024)));
                if (!compute_first || !busy) {
                    issue_band(dst);
                    if (busy) prepare();
                }
                if (busy) {
                    const uint32_t v_cur = at.lds_address(tile_of(r) + C::MAT_BYTES) + at.v_lane;
                    const uint32_t k_next = at.lds_address(tile_of(r + 1)) + at.k_lane;
                    if (cur_is_a) {
                        PB::step_ab_x(k_next, v_cur, a.c, neg_m, at.l_run[0]);
                        PB::step_ab_y(a.c, neg_m, at.l_run[0], mx_lane);
                    } else {
                        PB::step_ba_x(k_next, v_cur, a.c, neg_m, at.l_run[0]);
                        PB::step_ba_y(a.c, neg_m, at.l_run[0], mx_lane);
                    }
                    if (compute_first) {
                        issue_band(dst);
                        prepare();
                    }
                }
                ++issued;
            };
            auto uniform_offset = [&](uint64_t off) {
                return (static_cast<int64_t>(uniform(static_cast<int>(off >> 32))) << 32) | static_cast<uint32_t>(uniform(static_cast<int>(off)));
            };
            // From its second step on a run is in steady state, three units ahead (its first step fetches
            // a unit or not, depending on how the run before it ended).  The plain steps that follow the
            // first step are taken in pairs (score sets B then A), each reading the band offset of the
            // step after it a step ahead; what is left of the run goes through the general step.
            bool first_step = true;
            while (rel < run_end) {
                step(rel++, true);
                if (first_step && rel < run_end && issued == rel + C::kStages - 1) {
                    uint64_t off = off_first;
                    int row = row_first;
                    for (int pairs = (uniform(plain_word) >> kUnitPlainShift) >> 1; pairs > 0; --pairs) {
                        const uint64_t off_next = band_offset(issued + 1);  // (in the table: the second step of the pair is plain)
                        const int row_next = band_row(issued + 1);
                        plain_step(rel++, false, uniform_offset(off), uniform(row));
                        off = band_offset(min(issued + 1, n_units - 1));  // used if another pair follows
                        row = band_row(min(issued + 1, n_units - 1));
                        plain_step(rel++, true, uniform_offset(off_next), uniform(row_next));
                    }
                }
                first_step = false;
                if (rel < run_end) step(rel++, false);
            }
            if (next_opens) wait_async_loads<0>();  // the next item's query rows (and the tiles requested before them)
            at.finish_run(rel - 1, split);
            if (next_opens) {
                if constexpr (!PREFILL && HD == 128) {
                    if (rope) at.rope_queries(at.units[run_end]);
                }
                at.adopt_item(at.units[run_end]);
            }
        }
    });
}

// The FP8 kernel with the pipelined tile step: the ring holds the codes as stored (4 stages of
// 16 KB), and the blocks of attn_pipe_gen.h read two widened K tiles and two widened V tiles.  In
// step r (softmax and O^T of unit r, S^T of unit r + 1) every wave widens its own rows of K of
// unit r + 2 and of V of unit r + 1 -- the tiles the step before has just released -- and then
// fetches unit r + 5 into the stage that frees.  Steps and units correspond one to one across the
// items of a chunk, so the widening runs on through the ends of runs.  A wave only reads codes it
// has loaded itself: the ring needs no barrier, and the step's one barrier orders the widened tiles.
// The scales: cached K rows count k_scale (folded into the softmax constant of that tile), cached V
// rows v_scale (O^T is kept in units of it: a fresh tile's exponentials are raised by 1 / v_scale
// through their exponent, and its row sums, gathered apart, are multiplied back).
template <int NW>
__global__ void __launch_bounds__(64 * NW, 1) __attribute__((amdgpu_num_vgpr(32)))
paged_attn_pipe_fp8_kernel(const KArgs a) {
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    constexpr int HD = 128;
    using C = StreamCfg<HD, 1, NW, false, 1>;
    using SA = StreamAttn<HD, 1, NW, false, 1, true>;
    static_assert(C::kStages == 4 && C::LOADS_PER_UNIT == 2, "ring depth and wait counts below");
    SA at(a, smem);
    pipe_reserve();
    {
        const uint32_t o = static_cast<uint32_t>(at.lane / C::CPR) * static_cast<uint32_t>(a.c_st) + (at.lane % C::CPR) * 16;
        pipe_set_load_offsets(o, o);
        const int row = at.wave * C::ROWS_PER_WAVE + at.lane / C::CPR, cc = at.lane % C::CPR;
        const uint32_t wide = at.lds_address(at.wide_k(0));
        pipe_set_widen_addresses(at.stages_lds + at.wave * (C::IPW * 1024) + at.lane * 16,
                                 wide + SA::L::chunk_offset(row, 2 * cc), wide + SA::L::chunk_offset(row, 2 * cc + 1));
    }
    static_assert(C::IPW == 1, "pipe_widen: one load of codes per wave and matrix");
    const bool rope = a.rope_table != nullptr;  // (with it the store travels with the rotation of the fresh K rows)
    if (!rope) store_fresh_rows<HD, true, 1>(a);
    const bool busy = at.wave < a.busy_waves;
    constexpr int kHoleRows = C::ROWS_PER_WAVE;
    static_assert(kHoleRows == 8, "mask blocks of attn_pipe_gen.h");
    bool requested_early = false;
    auto on_work = [&](const WgWork& w) {
        UnitDesc d;
        d.q0 = w.q0;
        d.q_len = w.q_len;
        d.kvh = w.kvh;
        d.rt = w.rt;
        at.request_queries(d);
        requested_early = true;
    };
    auto as_scalar = [](float x) { return __builtin_bit_cast(float, uniform(__builtin_bit_cast(int, x))); };
    // The current item's constants, in scalar registers from the moment the item is adopted (worked out
    // where they are used, the compiler keeps their inputs in vector registers, and those in scratch):
    // the log2-domain scale of a tile of cached rows, and what raises a fresh tile's exponentials by
    // 1 / v_scale.
    float c_ctx = 0.0f, fresh_shift = 0.0f;
    auto adopt = [&](const UnitDesc& d) {
        at.adopt_item(d);
        c_ctx = as_scalar(a.c * at.k_mul);
        fresh_shift = as_scalar(__builtin_amdgcn_logf(at.v_inv));
    };
    at.for_each_chunk([&](int n_units) {
        const WgSplit& split = at.split;
        const bool opens = (uniform(at.units[0].flags) & kUnitFirst) != 0;
        if (opens && !requested_early) at.request_queries(at.units[0]);
        requested_early = false;
        if (rope) {  // (as in the bf16 kernel)
            int64_t pos = 0;
            if (opens) pos = at.rope_query_position(at.units[0]);
            const bool any = at.template rope_fresh_rows_of_chunk<true>(n_units);
            if (opens) at.request_rope_angles(pos);
            if (any) {
                wait_async_loads<0>();
                __syncthreads();
            }
        }
        at.mark_plain_steps(n_units);  // (while the query rows are on their way; first read behind a barrier)
        if (opens) {
            wait_async_loads<0>();
            if (rope) pipe_rope_queries();
            adopt(at.units[0]);
        }
        // ring fill, and the tiles the first step reads
        int issued = 0;
        for (; issued < C::kStages && issued < n_units; ++issued) at.issue_unit(issued);
        at.wait_younger(max(issued - 2, 0));  // units 0 and 1 have landed
        at.template widen_matrix<false>(0);
        at.template widen_matrix<true>(0);
        if (n_units > 1) at.template widen_matrix<false>(1);
        if (issued < n_units) at.issue_unit(issued++);  // into the stage of unit 0

        auto mask = [&](int r, bool set_a, float& mx_lane) {
            const TileInfo t = at.tile_info_of(r);
            const bool bc = !t.is_ctx && a.mask_mode == DFX_MASK_BLOCK_CAUSAL;
            if (!(t.base + C::TN > t.limit || t.holes != 0 || bc)) return;
            int lim = t.limit;
            if (bc) lim = min(lim, at.visible_limit(at.units[r]));
            const int thr = lim - t.base - 4 * at.half;
            const uint32_t holes = static_cast<uint32_t>(t.holes);
            if (set_a) pipe_mask_a_8(thr, holes, mx_lane);
            else pipe_mask_b_8(thr, holes, mx_lane);
        };
        const bool compute_first = at.wave < NW / 2;

        int rel = 0;
        while (rel < n_units) {
            const UnitDesc d = at.units[rel];
            const int run_end = min(rel + uniform(d.run), n_units);
            auto scale_of = [&](int r) { return (uniform(at.units[r].flags) & kUnitCtx) ? c_ctx : a.c; };

            float mx_lane = 0.0f;
            float neg_m = 0.0f;
            auto prepare = [&](float c) {
                const float m_tile = wave_xor32_max(mx_lane) * c;
                float& m_run = at.m_run[0];
                if (__any(m_tile > m_run + kRescaleThreshold)) {
                    const float m_new = fmaxf(m_run, m_tile);
                    if (__any(m_run != -INFINITY)) {
                        const float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_run - m_new);
                        at.l_run[0] *= alpha;
                        pipe_rescale_outputs(alpha);
                    }
                    m_run = m_new;
                }
                neg_m = (m_run == -INFINITY) ? 0.0f : -m_run;
            };
            // every wave has widened K of the run's first unit (at the latest a step ago; the chunk's
            // first two units just now)
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_s_barrier();
            if (busy) {
                pipe_first_scores(at.lds_address(at.wide_k(rel)) + at.k_lane, mx_lane);
                mask(rel, true, mx_lane);
                if (compute_first) prepare(scale_of(rel));
            }
            const bool next_opens = run_end < n_units;
            // for the plain steps behind the run's first step: how many, and where the first of them fetches
            const int plain_word = at.units[min(rel + 1, n_units - 1)].flags;
            const uint64_t off_first = static_cast<uint64_t>(at.bands[min(rel + C::kStages + 2, n_units - 1) * NW + at.wave].off);
            auto step = [&](int r, bool cur_is_a) {
                const bool has_next = r + 1 < run_end;
                // every wave has widened K of unit r + 1 and V of unit r and is done with step r - 1
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_s_barrier();
                auto refill = [&] {
                    if (r + 2 < n_units) {
                        at.wait_younger(issued - r - 3);
                        at.template widen_matrix<false>(r + 2);
                    }
                    if (r + 1 < n_units) at.template widen_matrix<true>(r + 1);
                    if (issued < n_units && issued < r + 2 + C::kStages) at.issue_unit(issued++);
                };
                const int flags = uniform(at.units[r].flags);
                const bool cur_fresh = !(flags & kUnitCtx);
                const float c_cur = cur_fresh ? a.c : c_ctx;
                if (!compute_first || !busy) {
                    refill();
                    if (!has_next && next_opens) at.request_queries(at.units[run_end]);
                    if (busy) prepare(c_cur);
                } else if (!has_next && next_opens) {
                    at.request_queries(at.units[run_end]);
                }
                if (busy) {
                    const uint32_t v_cur = at.lds_address(at.wide_v(r)) + at.v_lane;
                    const float l_before = at.l_run[0];
                    float l_step = cur_fresh ? 0.0f : l_before;
                    const float nm = cur_fresh ? neg_m + fresh_shift : neg_m;
                    if (has_next) {
                        const uint32_t k_next = at.lds_address(at.wide_k(r + 1)) + at.k_lane;
                        if (cur_is_a) {
                            pipe_step_ab_x(k_next, v_cur, c_cur, nm, l_step);
                            pipe_step_ab_y(c_cur, nm, l_step, mx_lane);
                        } else {
                            pipe_step_ba_x(k_next, v_cur, c_cur, nm, l_step);
                            pipe_step_ba_y(c_cur, nm, l_step, mx_lane);
                        }
                        mask(r + 1, !cur_is_a, mx_lane);
                    } else {
                        if (cur_is_a) {
                            pipe_last_a_x(v_cur, c_cur, nm, l_step);
                            pipe_last_a_y(c_cur, nm, l_step);
                        } else {
                            pipe_last_b_x(v_cur, c_cur, nm, l_step);
                            pipe_last_b_y(c_cur, nm, l_step);
                        }
                    }
                    at.l_run[0] = cur_fresh ? fmaf(l_step, at.out_mul, l_before) : l_step;
                    if (compute_first) {
                        refill();
                        if (has_next) prepare(scale_of(r + 1));
                    }
                }
            };
            // A plain step (mark_plain_steps()): units r, r + 1 and r + 2 are tiles of cached rows, nothing to
            // mask, and the unit to fetch is a full band of cached rows at `off`.
            auto plain_step = [&](int r, bool cur_is_a, int64_t off) {
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_s_barrier();
                auto refill = [&] {
                    wait_async_loads<2 * C::LOADS_PER_UNIT>();  // unit r + 2 has landed
                    pipe_widen((static_cast<unsigned>(r + 2) % C::kStages) * C::STAGE_BYTES,
                               (static_cast<unsigned>(r + 1) % C::kStages) * C::STAGE_BYTES + C::MAT_BYTES,
                               (r & 1) * SA::L::MAT_BYTES, (2 + ((r + 1) & 1)) * SA::L::MAT_BYTES);
                    pipe_issue_band_fp8(a.k_cache + off, a.v_cache + off,
                                        uniform(static_cast<int>(at.stages_lds + (static_cast<unsigned>(issued) % C::kStages) * C::STAGE_BYTES +
                                                                 at.wave * (C::IPW * 1024))));
                };
                if (!compute_first || !busy) {
                    refill();
                    if (busy) prepare(c_ctx);
                }
                if (busy) {
                    const uint32_t v_cur = at.lds_address(at.wide_v(r)) + at.v_lane;
                    const uint32_t k_next = at.lds_address(at.wide_k(r + 1)) + at.k_lane;
                    if (cur_is_a) {
                        pipe_step_ab_x(k_next, v_cur, c_ctx, neg_m, at.l_run[0]);
                        pipe_step_ab_y(c_ctx, neg_m, at.l_run[0], mx_lane);
                    } else {
                        pipe_step_ba_x(k_next, v_cur, c_ctx, neg_m, at.l_run[0]);
                        pipe_step_ba_y(c_ctx, neg_m, at.l_run[0], mx_lane);
                    }
                    if (compute_first) {
                        refill();
                        prepare(c_ctx);
                    }
                }
                ++issued;
            };
            auto band_offset = [&](int unit) { return static_cast<uint64_t>(at.bands[unit * NW + at.wave].off); };
            auto uniform_offset = [&](uint64_t off) {
                return (static_cast<int64_t>(uniform(static_cast<int>(off >> 32))) << 32) | static_cast<uint32_t>(uniform(static_cast<int>(off)));
            };
            bool first_step = true;
            while (rel < run_end) {
                step(rel++, true);
                // in steady state the step about to run fetches unit rel + kStages + 1
                if (first_step && rel < run_end && issued == rel + C::kStages + 1) {
                    uint64_t off = off_first;
                    for (int pairs = (uniform(plain_word) >> kUnitPlainShift) >> 1; pairs > 0; --pairs) {
                        const uint64_t off_next = band_offset(issued + 1);
                        plain_step(rel++, false, uniform_offset(off));
                        off = band_offset(min(issued + 1, n_units - 1));
                        plain_step(rel++, true, uniform_offset(off_next));
                    }
                }
                first_step = false;
                if (rel < run_end) step(rel++, false);
            }
            if (next_opens) wait_async_loads<0>();
            at.finish_run(rel - 1, split);
            if (next_opens) {
                if (rope) at.rope_queries(at.units[run_end]);
                adopt(at.units[run_end]);
            }
        }
    }, on_work);
}

}  // namespace dfx
