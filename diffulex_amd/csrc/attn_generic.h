// Generic tile path of the paged-attention kernel: any page size, bf16 or FP8-E4M3 cache.
//
// A 64-token tile goes global --16-byte loads--> registers --> LDS, K and V in the swizzled
// row-major layout of attn_tile.h, so the matrix and softmax arithmetic is the one the streaming
// path uses.  FP8 codes are widened to bf16 on the way into LDS (the widening is exact), so the
// arithmetic is the same for both cache types; the per-head scales are folded into the softmax
// constants.  One tile is staged in registers while the previous one is computed.
#pragma once

#include "attn_tile.h"

namespace dfx {

template <int HD, int NB>
struct GenericCfg : Shape<HD, NB> {
    using S = Shape<HD, NB>;
    static constexpr int K_BYTES = TileLayout<HD>::MAT_BYTES;
    static constexpr int STAGE_BYTES = 2 * K_BYTES;  // K tile, V tile
    // the block-table entries of the piece of an item being processed, so that the tile loop
    // does not chase a table entry in global memory before every row it loads
    static constexpr int kTableEntries = 4096;
    static constexpr int STAGES_OFF = (S::PREFIX_BYTES + S::MISC_BYTES + 255) / 256 * 256;  // tiles start at a multiple of 256
    static constexpr int TABLE_OFF = STAGES_OFF + 2 * STAGE_BYTES;
    static constexpr int LDS_BYTES = TABLE_OFF + kTableEntries * 4;
    static constexpr int CH16 = S::TN * HD * 2 / 16 / kThreads;  // 16-byte chunks per lane, bf16 tile
    static constexpr int CH8 = S::TN * HD / 16 / kThreads;       // 16-byte chunks per lane, fp8 tile
};

// DISTINCT: the cache is in the "distinct" layout, K [pages, H, hd / 8, page, 8] and V [pages, H,
// hd, page] (bf16): a 16-byte load still brings one 8-element chunk of a K row, but 8 consecutive
// tokens of one d for V -- one chunk of a d-major V tile, which is what the V^T operand reads.
template <int HD, int NB, bool FP8, bool DISTINCT = false>
struct GenericAttn : TileMath<HD, NB, kWaves> {
    using Base = TileMath<HD, NB, kWaves>;
    using L = TileLayout<HD>;
    using C = GenericCfg<HD, NB>;
    using Base::a;
    using Base::col;
    using Base::half;
    using Base::kvh;
    using Base::n0;
    using Base::o;
    using Base::qf;
    using Base::s;
    using Base::sh;
    using Base::tid;

    uint8_t* lds;
    int* prefix;
    int* misc;
    int* table;        // block-table entries [table_p0, table_p0 + table_n) of sequence s, if table_n > 0
    int table_p0, table_n;
    u32x4 kst[C::CH16], vst[C::CH16];
    bool staged_fp8, staged_distinct;

    DFX_D GenericAttn(const KArgs& args, uint8_t* smem)
        : Base(args), lds(smem), prefix(reinterpret_cast<int*>(smem)),
          misc(reinterpret_cast<int*>(smem + C::PREFIX_BYTES)), table(reinterpret_cast<int*>(smem + C::TABLE_OFF)),
          table_p0(0), table_n(0) {}

    // Copy the block-table entries that tiles [tile0, tile1) of the current sequence need into LDS
    // (skipped, and looked up in global memory instead, if they do not fit).  The caller's
    // barrier makes them visible.
    DFX_D void cache_block_table(int tile0, int tile1) {
        table_n = 0;
        const int tok0 = tile0 * C::TN;
        const int tok1 = min(tile1 * C::TN, sh.ctx);
        if (tok1 <= tok0) return;
        const int p0 = tok0 / a.page_size, p1 = (tok1 - 1) / a.page_size;
        if (p1 - p0 + 1 > C::kTableEntries) return;
        table_p0 = p0;
        table_n = p1 - p0 + 1;
        for (int i = tid; i < table_n; i += kThreads) {
            const int p = p0 + i;
            table[i] = p < a.max_pages ? a.block_tables[static_cast<int64_t>(s) * a.bt_stride + p] : -1;
        }
    }

    DFX_D uint8_t* k_stage(int b) const { return lds + C::STAGES_OFF + b * C::STAGE_BYTES; }
    DFX_D uint8_t* v_stage(int b) const { return k_stage(b) + C::K_BYTES; }

    // physical page of context token `tok` and the token's place in it; ok is cleared if the
    // block table has no valid entry for it
    DFX_D int64_t page_of(int tok, bool& ok, int& off) const {
        const int p = a.page_shift >= 0 ? (tok >> a.page_shift) : (tok / a.page_size);
        off = tok - p * a.page_size;
        int64_t page = -1;
        if (table_n > 0) page = table[p - table_p0];
        else if (p < a.max_pages) page = a.block_tables[static_cast<int64_t>(s) * a.bt_stride + p];
        ok = ok && page >= 0 && page < a.n_pages;
        return page;
    }

    DFX_D int64_t cache_row_offset(int tok, bool& ok) const {
        int off;
        const int64_t page = page_of(tok, ok, off);
        return page * a.c_sp + off * a.c_st + kvh * a.c_sh;
    }

    // Distinct layout, global -> registers.  K: the 64 lanes of a wave take one chunk column of 64
    // consecutive tokens (1 KiB contiguous inside a page); V: eight consecutive lanes take the
    // eight 8-token groups of one d (128 contiguous bytes).
    DFX_D void issue_distinct(int base, int limit) {
        static_assert(kThreads % C::TN == 0 && kThreads % 8 == 0, "a thread's chunks share their token (K) and token group (V)");
        // K: chunk c = tid + kThreads * i is (token c % TN, chunk column c / TN): one token per thread
        {
            const int tok = base + tid % C::TN;
            bool ok = tok < limit;
            int off = 0;
            int64_t page = 0;
            if (ok) page = page_of(tok, ok, off);
            const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k_cache) + (ok ? page * a.kd_sp + kvh * a.kd_sh + off * 8 : 0) +
                                 (tid / C::TN) * a.kd_sc;
#pragma unroll
            for (int i = 0; i < C::CH16; ++i) {
                u32x4 kk = {0, 0, 0, 0};
                if (ok) kk = *reinterpret_cast<const u32x4*>(kp + i * (kThreads / C::TN) * a.kd_sc);
                kst[i] = kk;
            }
        }
        // V: chunk c is (token group c % 8, d = c / 8): one group of 8 tokens per thread
        {
            const int tok = base + (tid % 8) * 8;
            bool ok = tok < limit;
            int off = 0;  // a multiple of 8: pages hold a multiple of 8 tokens
            int64_t page = 0;
            if (ok) page = page_of(tok, ok, off);
            const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v_cache) + (ok ? page * a.vd_sp + kvh * a.vd_sh + off : 0) +
                                 (tid / 8) * a.vd_sd;
#pragma unroll
            for (int i = 0; i < C::CH16; ++i) {
                u32x4 vv = {0, 0, 0, 0};
                if (ok) vv = *reinterpret_cast<const u32x4*>(vp + i * (kThreads / 8) * a.vd_sd);
                vst[i] = vv;
            }
            // tokens past the end of the context read as zeros (the group that holds the end only):
            // a mask per 32-bit word of two tokens
            const int n_valid = limit - tok;
            if (ok && n_valid < 8) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t keep = (2 * k < n_valid ? 0x0000ffffu : 0u) | (2 * k + 1 < n_valid ? 0xffff0000u : 0u);
#pragma unroll
                    for (int i = 0; i < C::CH16; ++i) vst[i][k] &= keep;
                }
            }
        }
    }

    // The V tile stays d-major in LDS (TileMath::vt_chunk_offset, accumulate_dmajor).  This kernel feeds
    // the key rows to S^T in their own order, so inside a 16-token slab the matrix instruction's
    // contraction index runs over tokens 0-3, 8-11 (lower half of the wave) and 4-7, 12-15 (upper half),
    // as the score registers hold them; the two chunks of a slab are stored in that order, so that a
    // lane's operand is one 16-byte read: chunk 2 * slab + h = tokens 4h..4h+3 then 8+4h..8+4h+3 of the slab.
    using Base::vt_chunk_offset;
    // byte offset of token `tok` (0..63) of row d
    DFX_HD static int vt_token_offset(int d, int tok) {
        const int r16 = tok & 15;
        return vt_chunk_offset(d, (tok >> 4) * 2 + ((r16 >> 2) & 1)) + ((r16 >> 3) * 4 + (r16 & 3)) * 2;
    }

    DFX_D void commit_distinct(uint8_t* ks, uint8_t* vs) const {
        int t = tid;
        asm volatile("" : "+v"(t));  // (addresses worked out here, not kept as invariants of the tile loop: see commit())
#pragma unroll
        for (int i = 0; i < C::CH16; ++i) {
            const int c = t + kThreads * i;
            *reinterpret_cast<u32x4*>(ks + L::chunk_offset(c % C::TN, c / C::TN)) = kst[i];
            // a chunk of the cache is tokens 8 tg .. 8 tg + 7 of one d: its halves go to the slab's two chunks
            const int tg = c % 8, d = c / 8;
            const u32x2 lo = {vst[i][0], vst[i][1]}, hi = {vst[i][2], vst[i][3]};
            *reinterpret_cast<u32x2*>(vs + vt_token_offset(d, tg * 8)) = lo;
            *reinterpret_cast<u32x2*>(vs + vt_token_offset(d, tg * 8 + 4)) = hi;
        }
    }

    // global -> registers (rows past the end of the sequence become zeros)
    DFX_D void issue(int tile) {
        const bool is_ctx = tile < sh.n_ctx_tiles;
        const int base = (is_ctx ? tile : tile - sh.n_ctx_tiles) * C::TN;
        const int limit = is_ctx ? sh.ctx : sh.new_len;
        staged_distinct = DISTINCT && is_ctx;
        if (DISTINCT && is_ctx) {
            staged_fp8 = false;
            issue_distinct(base, limit);
        } else if (FP8 && is_ctx) {
            staged_fp8 = true;
            constexpr int CPR = HD / 16;
#pragma unroll
            for (int i = 0; i < C::CH8; ++i) {
                const int c = tid + kThreads * i;
                const int row = c / CPR, cc = c % CPR;
                const int tok = base + row;
                bool ok = tok < limit;
                u32x4 kk = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
                if (ok) {
                    const int64_t off = cache_row_offset(tok, ok) + cc * 16;
                    if (ok) {
                        kk = *reinterpret_cast<const u32x4*>(a.k_cache + off);
                        vv = *reinterpret_cast<const u32x4*>(a.v_cache + off);
                    }
                }
                kst[i] = kk;
                vst[i] = vv;
            }
        } else {
            staged_fp8 = false;
            constexpr int CPR = HD / 8;
#pragma unroll
            for (int i = 0; i < C::CH16; ++i) {
                const int c = tid + kThreads * i;
                const int row = c / CPR, cc = c % CPR;
                const int tok = base + row;
                bool ok = tok < limit;
                u32x4 kk = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
                if (ok) {
                    if (is_ctx) {
                        const int64_t off = cache_row_offset(tok, ok) + cc * 8;
                        if (ok) {
                            kk = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(a.k_cache) + off);
                            vv = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(a.v_cache) + off);
                        }
                    } else {
                        const int64_t t = n0 + tok;
                        kk = *reinterpret_cast<const u32x4*>(a.k_new + t * a.kn_st + kvh * a.kn_sh + cc * 8);
                        vv = *reinterpret_cast<const u32x4*>(a.v_new + t * a.vn_st + kvh * a.vn_sh + cc * 8);
                    }
                }
                kst[i] = kk;
                vst[i] = vv;
            }
        }
    }

    // registers -> LDS
    DFX_D void commit(int buf) const {
        uint8_t* ks = k_stage(buf);
        uint8_t* vs = v_stage(buf);
        if (DISTINCT && staged_distinct) {
            commit_distinct(ks, vs);
        } else if (FP8 && staged_fp8) {
            constexpr int CPR = HD / 16;  // 16-code chunks per row, each widening to two bf16 chunks
#pragma unroll
            for (int i = 0; i < C::CH8; ++i) {
                const int c = tid + kThreads * i;
                const int row = c / CPR, cc = c % CPR;
                u32x4 lo, hi;
                widen16(kst[i], lo, hi);
                *reinterpret_cast<u32x4*>(ks + L::chunk_offset(row, 2 * cc)) = lo;
                *reinterpret_cast<u32x4*>(ks + L::chunk_offset(row, 2 * cc + 1)) = hi;
                widen16(vst[i], lo, hi);
                *reinterpret_cast<u32x4*>(vs + L::chunk_offset(row, 2 * cc)) = lo;
                *reinterpret_cast<u32x4*>(vs + L::chunk_offset(row, 2 * cc + 1)) = hi;
            }
        } else {
            constexpr int CPR = HD / 8;
            int t = tid;
            // (fresh rows of the distinct kernel, one tile per item: their 8 * CH16 scatter addresses are
            // worked out here, from a thread number the compiler cannot follow -- as loop invariants of
            // the tile loop they would take more registers than there are, for both tile buffers)
            if constexpr (DISTINCT) asm volatile("" : "+v"(t));
#pragma unroll
            for (int i = 0; i < C::CH16; ++i) {
                const int c = t + kThreads * i;
                const int row = c / CPR, cc = c % CPR;
                *reinterpret_cast<u32x4*>(ks + L::chunk_offset(row, cc)) = kst[i];
                if constexpr (DISTINCT) {
                    // into the d-major V tile, two bytes at a time
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const uint32_t w = vst[i][j >> 1];
                        *reinterpret_cast<uint16_t*>(vs + vt_token_offset(cc * 8 + j, row)) =
                            static_cast<uint16_t>((j & 1) ? (w >> 16) : w);
                    }
                } else {
                    *reinterpret_cast<u32x4*>(vs + L::chunk_offset(row, cc)) = vst[i];
                }
            }
        }
    }

    // one tile of attention from LDS
    DFX_D void compute(int buf, int tile) {
        TileInfo t = this->tile_info(sh, kvh, tile, FP8);
        if (t.is_ctx) {  // tokens on pages without a valid block-table entry are skipped: one token per lane
            const int tok = t.base + this->lane;
            bool ok = true;
            int off;
            if (tok < t.limit) page_of(tok, ok, off);
            t.holes = __ballot(!ok);
        }
        f32x16 sc[2][NB];
        this->scores(k_stage(buf), sc);
        bf16x8 pb[NB][2][2];
        this->template softmax_tile<FP8, 1>(sc, t, pb, [&] { this->outputs_ready(); });
        if constexpr (DISTINCT) this->accumulate_dmajor(v_stage(buf), pb);  // (one form for every tile: two, chosen at run time, would
        else this->accumulate(v_stage(buf), pb);                      //  have the accumulators copied where the paths meet)
    }

    DFX_D void run_segment(int rt, int tile0, int tile1, int item_tiles, int64_t item_begin, const WgSplit& split) {
        const bool complete = tile0 == 0 && tile1 == item_tiles;
        this->load_queries(rt);
        __syncthreads();  // the previous segment's last tile and block-table entries may still be read from LDS
        cache_block_table(tile0, tile1);
        __syncthreads();
        int buf = 0;
        issue(tile0);
        for (int t = tile0; t < tile1; ++t) {
            commit(buf);
            __syncthreads();
            if (t + 1 < tile1) issue(t + 1);
            compute(buf, t);
            buf ^= 1;
        }
        this->outputs_ready();
        float l_tot[NB];
        this->row_sums(l_tot);
        if (complete) this->store_output(rt, l_tot);
        else finish_cut_item(*this, rt, item_begin, item_tiles, split, -1, l_tot, misc + kMaxWaves + 1);
    }
};

template <int HD, int NB, bool FP8, bool DISTINCT = false>
__global__ void __launch_bounds__(kThreads) paged_attn_generic_kernel(const KArgs a) {
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    GenericAttn<HD, NB, FP8, DISTINCT> at(a, smem);
    if constexpr (!DISTINCT) store_fresh_rows<HD, FP8>(a);
    const UnitSummary summary = build_unit_prefix<Shape<HD, NB>::RT>(a, at.prefix, at.misc);
    const int per_head = summary.per_head;
    const int64_t total = static_cast<int64_t>(per_head) * a.h_kv;
    if (total == 0) return;
    const int w = blockIdx.x;
    const int n_active = a.fixed_wg ? a.n_wg
                                    : effective_workgroups(total, static_cast<int64_t>(summary.items) * a.h_kv,
                                                           summary.max_tiles, a.n_wg);
    if (w >= n_active) return;
    const WgSplit split = make_wg_split(total, n_active);
    const int64_t begin = split.first(w);
    const int64_t end = split.first(w + 1);
    if (begin >= end) return;

    int kvh = static_cast<int>(begin / per_head);
    const int rem = static_cast<int>(begin - static_cast<int64_t>(kvh) * per_head);
    int s = locate_sequence(a, at.prefix, at.misc, rem);
    int u = rem - at.prefix[s];
    int64_t pos = begin;
    while (pos < end) {
        at.set_sequence(s, kvh);
        if constexpr (FP8) at.out_mul = a.v_scale[kvh];
        int rt, tile0, n_tiles;
        locate_unit(at.sh, u, rt, tile0, n_tiles);
        const int64_t seg_end = min(pos + (n_tiles - tile0), end);
        const int tile1 = tile0 + static_cast<int>(seg_end - pos);
        at.run_segment(rt, tile0, tile1, n_tiles, pos - tile0, split);
        u += tile1 - tile0;
        pos = seg_end;
        if (pos >= end) break;
        if (u == at.sh.units) {
            u = 0;
            do {
                if (++s == a.num_seqs) {
                    s = 0;
                    ++kvh;
                }
            } while (at.prefix[s + 1] == at.prefix[s]);
        }
    }
}

}  // namespace dfx
