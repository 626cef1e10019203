// Generic tile path of the paged-attention kernel: any page size, bf16 or FP8-E4M3 cache.
//
// A 64-token tile goes global --16-byte loads--> registers --> LDS, K as [token][d] rows with
// a 16-byte skew, V transposed to [d][token] (2-byte LDS stores) with the token order the PV
// product wants.  FP8 codes are widened to bf16 on the way into LDS (the widening is exact),
// so the MFMA loop is the same for both cache types; the per-head scales are folded into the
// softmax constants.  One tile is staged in registers while the previous one is computed.
#pragma once

#include "attn_common.h"

namespace dfx {

template <int HD, int NB>
struct GenericCfg : Shape<HD, NB> {
    using S = Shape<HD, NB>;
    static constexpr int KSTRIDE = HD * 2 + 16;     // bytes per K row in LDS
    static constexpr int VSTRIDE = S::TN * 2 + 16;  // bytes per V^T row in LDS
    static constexpr int K_BYTES = S::TN * KSTRIDE;
    static constexpr int V_BYTES = HD * VSTRIDE;
    static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
    static constexpr int LDS_BYTES = S::PREFIX_BYTES + S::MISC_BYTES + 2 * STAGE_BYTES;
    static constexpr int CH16 = S::TN * HD * 2 / 16 / kThreads;  // 16-byte chunks per lane, bf16 tile
    static constexpr int CH8 = S::TN * HD / 16 / kThreads;       // 16-byte chunks per lane, fp8 tile
};

// Two e4m3 codes (bytes 0,1 or 2,3 of w) -> two bf16 packed in a dword.  An e4m3 value has 3
// mantissa bits, so the upper half of its fp32 form is its bf16 form.
template <bool HI>
DFX_D uint32_t fp8x2_to_bf16x2(uint32_t w) {
    const f32x2 f = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w), HI);
    return (__float_as_uint(f.x) >> 16) | (__float_as_uint(f.y) & 0xffff0000u);
}

// Position of token row r inside a V^T row: within every 16 tokens the 4-token groups
// (0,1,2,3) are stored in the order (0,2,1,3), so that the eight contraction elements a
// lane of half h needs for one MFMA, tokens {4h..4h+3} and {8+4h..8+4h+3}, are contiguous.
DFX_D int vt_pos(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

template <int HD, int NB, bool FP8>
struct GenericAttn : AttnState<HD, NB> {
    using Base = AttnState<HD, NB>;
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
    u32x4 kst[C::CH16], vst[C::CH16];
    bool staged_fp8;

    DFX_D GenericAttn(const KArgs& args, uint8_t* smem)
        : Base(args), lds(smem), prefix(reinterpret_cast<int*>(smem)),
          misc(reinterpret_cast<int*>(smem + C::PREFIX_BYTES)) {}

    DFX_D uint8_t* k_stage(int b) const { return lds + C::PREFIX_BYTES + C::MISC_BYTES + b * C::STAGE_BYTES; }
    DFX_D uint8_t* v_stage(int b) const { return k_stage(b) + C::K_BYTES; }

    DFX_D int64_t cache_row_offset(int tok, bool& ok) const {
        const int p = a.page_shift >= 0 ? (tok >> a.page_shift) : (tok / a.page_size);
        const int off = tok - p * a.page_size;
        int64_t page = -1;
        if (p < a.max_pages) page = a.block_tables[static_cast<int64_t>(s) * a.bt_stride + p];
        ok = ok && page >= 0 && page < a.n_pages;
        return page * a.c_sp + off * a.c_st + kvh * a.c_sh;
    }

    // global -> registers (rows past the end of the sequence become zeros)
    DFX_D void issue(int tile) {
        const bool is_ctx = tile < sh.n_ctx_tiles;
        const int base = (is_ctx ? tile : tile - sh.n_ctx_tiles) * C::TN;
        const int limit = is_ctx ? sh.ctx : sh.new_len;
        if (FP8 && is_ctx) {
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

    DFX_D void put_v8(uint8_t* vs, int d0, int row, u32x4 v) const {
        uint16_t* base = reinterpret_cast<uint16_t*>(vs + d0 * C::VSTRIDE) + vt_pos(row);
        constexpr int RS = C::VSTRIDE / 2;
        base[0 * RS] = static_cast<uint16_t>(v.x);
        base[1 * RS] = static_cast<uint16_t>(v.x >> 16);
        base[2 * RS] = static_cast<uint16_t>(v.y);
        base[3 * RS] = static_cast<uint16_t>(v.y >> 16);
        base[4 * RS] = static_cast<uint16_t>(v.z);
        base[5 * RS] = static_cast<uint16_t>(v.z >> 16);
        base[6 * RS] = static_cast<uint16_t>(v.w);
        base[7 * RS] = static_cast<uint16_t>(v.w >> 16);
    }

    DFX_D static void widen16(u32x4 codes, u32x4& lo, u32x4& hi) {
        lo = u32x4{fp8x2_to_bf16x2<false>(codes.x), fp8x2_to_bf16x2<true>(codes.x),
                   fp8x2_to_bf16x2<false>(codes.y), fp8x2_to_bf16x2<true>(codes.y)};
        hi = u32x4{fp8x2_to_bf16x2<false>(codes.z), fp8x2_to_bf16x2<true>(codes.z),
                   fp8x2_to_bf16x2<false>(codes.w), fp8x2_to_bf16x2<true>(codes.w)};
    }

    // registers -> LDS
    DFX_D void commit(int buf) const {
        uint8_t* ks = k_stage(buf);
        uint8_t* vs = v_stage(buf);
        if (FP8 && staged_fp8) {
            constexpr int CPR = HD / 16;
#pragma unroll
            for (int i = 0; i < C::CH8; ++i) {
                const int c = tid + kThreads * i;
                const int row = c / CPR, cc = c % CPR;
                u32x4 lo, hi;
                widen16(kst[i], lo, hi);
                u32x4* kd = reinterpret_cast<u32x4*>(ks + row * C::KSTRIDE + cc * 32);
                kd[0] = lo;
                kd[1] = hi;
                widen16(vst[i], lo, hi);
                put_v8(vs, cc * 16, row, lo);
                put_v8(vs, cc * 16 + 8, row, hi);
            }
        } else {
            constexpr int CPR = HD / 8;
#pragma unroll
            for (int i = 0; i < C::CH16; ++i) {
                const int c = tid + kThreads * i;
                const int row = c / CPR, cc = c % CPR;
                *reinterpret_cast<u32x4*>(ks + row * C::KSTRIDE + cc * 16) = kst[i];
                put_v8(vs, cc * 8, row, vst[i]);
            }
        }
    }

    // one tile of attention from LDS
    DFX_D void compute(int buf, int tile) {
        const TileInfo t = this->tile_info(sh, kvh, tile, FP8);
        const uint8_t* ks = k_stage(buf);
        const uint8_t* vs = v_stage(buf);

        f32x16 sc[2][NB];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int qb = 0; qb < NB; ++qb)
#pragma unroll
                for (int e = 0; e < 16; ++e) sc[tb][qb][e] = 0.0f;

        const uint8_t* krow = ks + col * C::KSTRIDE + half * 16;
#pragma unroll
        for (int slab = 0; slab < C::NSLAB; ++slab) {
            bf16x8 ka[2];
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
                ka[tb] = *reinterpret_cast<const bf16x8*>(krow + tb * 32 * C::KSTRIDE + slab * 32);
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int qb = 0; qb < NB; ++qb)
                    sc[tb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[tb], qf[qb][slab], sc[tb][qb], 0, 0, 0);
        }

        bf16x8 pb[NB][2][2];
        this->template softmax_tile<FP8>(sc, t, pb, [] {});

        const uint8_t* vrow = vs + col * C::VSTRIDE + half * 16;
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int sl = 0; sl < 2; ++sl)
#pragma unroll
                for (int db = 0; db < C::NDB; ++db) {
                    const bf16x8 va =
                        *reinterpret_cast<const bf16x8*>(vrow + db * 32 * C::VSTRIDE + (tb * 32 + sl * 16) * 2);
#pragma unroll
                    for (int qb = 0; qb < NB; ++qb)
                        o[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[qb][tb][sl], o[db][qb], 0, 0, 0);
                }
    }

    DFX_D void run_segment(int rt, int tile0, int tile1, int64_t item_begin, const WgSplit& split, int slot) {
        const bool complete = tile0 == 0 && tile1 == this->sh.n_tiles;
        this->load_queries(rt);
        __syncthreads();  // the previous segment's last tile may still be read from LDS
        int buf = 0;
        issue(tile0);
        for (int t = tile0; t < tile1; ++t) {
            commit(buf);
            __syncthreads();
            if (t + 1 < tile1) issue(t + 1);
            compute(buf, t);
            buf ^= 1;
        }
        float l_tot[NB];
        this->row_sums(l_tot);
        if (complete) this->store_output(rt, l_tot);
        else finish_cut_item(*this, rt, item_begin, this->sh.n_tiles, split, slot, l_tot, misc + kMaxWaves + 1);
    }
};

template <int HD, int NB, bool FP8>
__global__ void __launch_bounds__(kThreads) paged_attn_generic_kernel(const KArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    GenericAttn<HD, NB, FP8> at(a, smem);
    const int per_head = build_unit_prefix<Shape<HD, NB>::RT>(a, at.prefix, at.misc);
    const int64_t total = static_cast<int64_t>(per_head) * a.h_kv;
    if (total == 0) return;
    const int w = blockIdx.x;
    const WgSplit split = make_wg_split(total, a.n_wg);
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
        const int n_tiles = at.sh.n_tiles;
        const int rt = u / n_tiles;
        const int tile0 = u - rt * n_tiles;
        const int64_t seg_end = min(pos + (n_tiles - tile0), end);
        const int tile1 = tile0 + static_cast<int>(seg_end - pos);
        at.run_segment(rt, tile0, tile1, pos - tile0, split, partial_slot(w, pos, begin));
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
