// Tiles of fresh rows on their way into a cache in the distinct layout (K [pages, H, hd / 8, page, 8], V [pages, H,
// hd, page]), shared by the store kernel and by the rotary embedding that stores: 16 tokens of one head staged in
// LDS so that both sides move 16 bytes per lane -- rows read as they lie, K written as chunk columns of consecutive
// tokens, V written transposed, eight consecutive tokens of one d per store where those eight have consecutive
// slots starting at a multiple of 8 inside one page (two bytes at a time otherwise).
#pragma once

#include "dfx_common.h"

namespace dfx {

template <int HD>
struct DistinctTile {
    static constexpr int kTokens = 16;
    static constexpr int CPR = HD / 8;         // 16-byte chunks per row
    static constexpr int VPITCH = HD * 2 + 4;  // V rows padded by one word: column reads then spread over the banks
    static constexpr int K_BYTES = kTokens * HD * 2;
    static constexpr int V_BYTES = kTokens * VPITCH;

    // where chunk cc of token row r of the K tile lies (chunks swizzled by the row)
    DFX_D static int k_offset(int r, int cc) { return r * (HD * 2) + ((cc ^ (r % CPR)) * 16); }
    DFX_D static void put_v(uint8_t* v_tile, int r, int cc, u32x4 vv) {
        uint32_t* vrow = reinterpret_cast<uint32_t*>(v_tile + r * VPITCH + cc * 16);
        vrow[0] = vv.x; vrow[1] = vv.y; vrow[2] = vv.z; vrow[3] = vv.w;
    }

    // The staged tile (every thread of the workgroup, behind the barrier that completes it) into the caches:
    // slot_of[r] is the slot of token row r, negative for rows to skip; kst / vst: element strides of page,
    // head and chunk column (K) / d (V).
    DFX_D static void store(const uint8_t* k_tile, const uint8_t* v_tile, const int64_t* slot_of, uint16_t* k_cache,
                            uint16_t* v_cache, const int64_t* kst, const int64_t* vst, int h, int page_size, int tid,
                            int n_threads) {
        // K: consecutive lanes take consecutive tokens of one chunk column
        for (int c = tid; c < kTokens * CPR; c += n_threads) {
            const int r = c % kTokens, cc = c / kTokens;
            const int64_t slot = slot_of[r];
            if (slot < 0) continue;
            const int64_t blk = slot / page_size, off = slot - blk * page_size;
            const u32x4 kk = *reinterpret_cast<const u32x4*>(k_tile + k_offset(r, cc));
            *reinterpret_cast<u32x4*>(k_cache + blk * kst[0] + h * kst[1] + cc * kst[2] + off * 8) = kk;
        }
        // V: eight consecutive lanes take the eight 8-token groups of one d
        for (int c = tid; c < (kTokens / 8) * HD; c += n_threads) {
            const int tg = c % (kTokens / 8), d = c / (kTokens / 8);
            const int r0 = tg * 8;
            uint16_t e[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) e[j] = *reinterpret_cast<const uint16_t*>(v_tile + (r0 + j) * VPITCH + d * 2);
            const int64_t s0 = slot_of[r0];
            bool run = s0 >= 0 && (s0 % 8) == 0 && (s0 % page_size) + 8 <= page_size;
#pragma unroll
            for (int j = 1; j < 8; ++j) run = run && slot_of[r0 + j] == s0 + j;
            if (run) {
                const int64_t blk = s0 / page_size, off = s0 - blk * page_size;
                u32x4 w;
                w.x = e[0] | (static_cast<uint32_t>(e[1]) << 16);
                w.y = e[2] | (static_cast<uint32_t>(e[3]) << 16);
                w.z = e[4] | (static_cast<uint32_t>(e[5]) << 16);
                w.w = e[6] | (static_cast<uint32_t>(e[7]) << 16);
                *reinterpret_cast<u32x4*>(v_cache + blk * vst[0] + h * vst[1] + d * vst[2] + off) = w;
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int64_t slot = slot_of[r0 + j];
                    if (slot < 0) continue;
                    const int64_t blk = slot / page_size, off = slot - blk * page_size;
                    v_cache[blk * vst[0] + h * vst[1] + d * vst[2] + off] = e[j];
                }
            }
        }
    }
};

}  // namespace dfx
