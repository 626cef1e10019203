// Streaming tile path of the paged-attention kernel (bf16 KV, page_size a multiple of 16).
//
// K/V tiles go HBM -> LDS directly (global_load_lds_dwordx4, 16 bytes per lane, never through
// registers) into a ring of kStages stages, so several tiles are in flight per compute unit
// while the matrix cores work on an older one.  The ring runs over the workgroup's whole unit
// range: tiles of the next (sequence, head) item are already on their way while the current
// item is finished.
//
// LDS tile layout: row-major [token][head_dim] as in the cache, with the 16-byte chunks of a
// row XOR-swizzled by the row index.  A direct-to-LDS load writes lane i's 16 bytes at
// wave_base + 16*i, so the swizzle is applied on the global side: lane i fetches the chunk
// that belongs at position i.
//   K operand (A of S^T = K Q^T): ds_read_b128 of chunk (2*slab + h) of row (lane % 32).
//   V operand (A of O^T += V^T P^T): needs 8 tokens of one d per lane, i.e. a column of the
//     tile.  ds_read_b64_tr_b16 transposes inside groups of 16 lanes: lane i of a group
//     receives element (i % 4) of what lanes {i/4, 4 + i/4, 8 + i/4, 12 + i/4} of the group
//     addressed.  Source lane s therefore points at token row (s / 4), elements 4*(s % 4)..+3
//     of a 16-wide d range, and lane i ends up with 4 consecutive tokens of d = i.
//
// The asynchronous loads are issued from inline assembly and waited for with explicit
// s_waitcnt vmcnt(n): the compiler does not model them, so it neither drains them at every
// barrier nor before every LDS read.  vmcnt retires in order, so waits the compiler adds for
// its own loads/stores can only be stricter than needed, never too weak.
#pragma once

#include "attn_common.h"

namespace dfx {

template <int HD, int NB>
struct StreamCfg : Shape<HD, NB> {
    using S = Shape<HD, NB>;
    static constexpr int ROWB = HD * 2;               // bytes per token row
    static constexpr int CPR = ROWB / 16;             // 16-byte chunks per row
    static constexpr int RPI = 1024 / ROWB;           // rows one wave-wide load covers
    static constexpr int MAT_BYTES = S::TN * ROWB;    // K (or V) tile
    static constexpr int STAGE_BYTES = 2 * MAT_BYTES;
    static constexpr int kStages = 4;
    static constexpr int IPW = MAT_BYTES / 1024 / kWaves;  // loads per wave per matrix per tile
    static constexpr int LOADS_PER_UNIT = 2 * IPW;
    static constexpr int ROWS_PER_WAVE = IPW * RPI;        // 16
    static constexpr int LDS_BYTES = S::PREFIX_BYTES + S::MISC_BYTES + kStages * STAGE_BYTES;
    static_assert(ROWS_PER_WAVE == 16, "a wave loads a 16-row band of each tile");

    // chunk position = chunk index ^ swizzle(row); 16 consecutive rows of one chunk column hit
    // 16 different 16-byte bank groups (the LDS has 64 banks)
    DFX_HD static int swizzle(int row) { return HD == 128 ? (row & 15) : ((row >> 1) & 7); }
};

DFX_D uint32_t lds_offset(const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); }

// One wave-wide 16-byte-per-lane direct-to-LDS load; lane i's data lands at lds_wave_base + 16*i.
DFX_D void async_load16(const void* gptr, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt"
                 :
                 : "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base))
                 : "memory", "m0");
}

template <int N>
DFX_D void wait_async_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Position in the workgroup's unit range, with the shape of the sequence it is in.
struct UnitCursor {
    int64_t pos;
    int kvh, s, u;
    SeqShape sh;
    int n0;
};

template <int HD, int NB>
struct StreamAttn : AttnState<HD, NB> {
    using Base = AttnState<HD, NB>;
    using C = StreamCfg<HD, NB>;
    using Base::a;
    using Base::col;
    using Base::half;
    using Base::lane;
    using Base::o;
    using Base::qf;
    using Base::wave;

    uint8_t* lds;
    int* prefix;
    int* misc;
    uint32_t stage0;  // LDS byte offset of stage 0

    DFX_D StreamAttn(const KArgs& args, uint8_t* smem)
        : Base(args), lds(smem), prefix(reinterpret_cast<int*>(smem)),
          misc(reinterpret_cast<int*>(smem + C::PREFIX_BYTES)),
          stage0(lds_offset(smem) + C::PREFIX_BYTES + C::MISC_BYTES) {}

    DFX_D void cursor_enter(UnitCursor& c) const {
        c.sh = load_seq_shape(a, c.s, C::RT);
        c.n0 = a.cu_new[c.s];
    }

    DFX_D void cursor_advance(UnitCursor& c, int64_t end) const {
        ++c.pos;
        ++c.u;
        if (c.pos >= end) return;
        if (c.u == c.sh.units) {
            c.u = 0;
            do {
                if (++c.s == a.num_seqs) {
                    c.s = 0;
                    ++c.kvh;
                }
            } while (prefix[c.s + 1] == prefix[c.s]);
            cursor_enter(c);
        }
    }

    // Start the loads of the unit at c into ring stage `stage` (this wave's 16-row band of K and V).
    DFX_D void issue_unit(const UnitCursor& c, int stage) const {
        const int tile = c.u % c.sh.n_tiles;
        const bool is_ctx = tile < c.sh.n_ctx_tiles;
        const int base = (is_ctx ? tile : tile - c.sh.n_ctx_tiles) * C::TN;
        const int limit = is_ctx ? c.sh.ctx : c.sh.new_len;
        // Rows past the end re-read the last valid rows (finite data; their scores are masked).
        int band = base + wave * C::ROWS_PER_WAVE;
        if (band >= limit) band = ((limit - 1) / C::ROWS_PER_WAVE) * C::ROWS_PER_WAVE;
        const uint8_t* kbase;
        const uint8_t* vbase;
        int64_t row_stride;  // bytes
        if (is_ctx) {
            const int p = a.page_shift >= 0 ? (band >> a.page_shift) : (band / a.page_size);
            int64_t page = a.block_tables[static_cast<int64_t>(c.s) * a.bt_stride + p];
            page = page < 0 ? 0 : (page >= a.n_pages ? a.n_pages - 1 : page);
            const int64_t off = (page * a.c_sp + static_cast<int64_t>(band - p * a.page_size) * a.c_st + c.kvh * a.c_sh) * 2;
            kbase = a.k_cache + off;
            vbase = a.v_cache + off;
            row_stride = a.c_st * 2;
        } else {
            const int64_t t = c.n0 + band;
            kbase = reinterpret_cast<const uint8_t*>(a.k_new + t * a.kn_st + c.kvh * a.kn_sh);
            vbase = reinterpret_cast<const uint8_t*>(a.v_new + t * a.vn_st + c.kvh * a.vn_sh);
            row_stride = a.kn_st * 2;
        }
        const int64_t v_row_stride = is_ctx ? row_stride : a.vn_st * 2;
        const int last = limit - 1 - band;  // last valid row of the band (>= 0)
        const uint32_t dst = stage0 + stage * C::STAGE_BYTES + wave * (C::IPW * 1024);
#pragma unroll
        for (int j = 0; j < C::IPW; ++j) {
            int r = j * C::RPI + lane / C::CPR;          // row inside the band
            const int lds_row = wave * C::ROWS_PER_WAVE + r;
            const int chunk = (lane % C::CPR) ^ C::swizzle(lds_row);
            r = min(r, last);
            async_load16(kbase + r * row_stride + chunk * 16, dst + j * 1024);
            async_load16(vbase + r * v_row_stride + chunk * 16, dst + C::MAT_BYTES + j * 1024);
        }
    }

    DFX_D bf16x8 read_k(uint32_t k_lds, int tb, int slab) const {
        const int row = tb * 32 + col;
        const int pos = (2 * slab + half) ^ C::swizzle(row);
        return *reinterpret_cast<const bf16x8*>(lds + (k_lds - lds_offset(lds)) + row * C::ROWB + pos * 16);
    }

    // V^T operand for token slab (tb, sl) and d block db.
    DFX_D bf16x8 read_vt(uint32_t v_lds, int tb, int sl, int db) const {
        typedef short short4v __attribute__((ext_vector_type(4)));
        typedef short short8v __attribute__((ext_vector_type(8)));
        const int g16 = lane >> 4, sl16 = lane & 15;
        short4v r[2];
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) {
            const int row = tb * 32 + sl * 16 + ii * 8 + (g16 >> 1) * 4 + (sl16 >> 2);
            const int chunk = db * 4 + (g16 & 1) * 2 + ((sl16 & 3) >> 1);
            const int pos = chunk ^ C::swizzle(row);
            const uint8_t* p = lds + (v_lds - lds_offset(lds)) + row * C::ROWB + pos * 16 + (sl16 & 1) * 8;
            r[ii] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                reinterpret_cast<short4v __attribute__((address_space(3)))*>(
                    reinterpret_cast<uintptr_t>(p)));
        }
        const short8v v = __builtin_shufflevector(r[0], r[1], 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, v);
    }

    DFX_D void compute(int stage, const TileInfo& t) {
        const uint32_t k_lds = stage0 + stage * C::STAGE_BYTES;
        const uint32_t v_lds = k_lds + C::MAT_BYTES;
        f32x16 sc[2][NB];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int qb = 0; qb < NB; ++qb)
#pragma unroll
                for (int e = 0; e < 16; ++e) sc[tb][qb][e] = 0.0f;
#pragma unroll
        for (int slab = 0; slab < C::NSLAB; ++slab) {
            bf16x8 ka[2];
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) ka[tb] = read_k(k_lds, tb, slab);
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int qb = 0; qb < NB; ++qb)
                    sc[tb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[tb], qf[qb][slab], sc[tb][qb], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        bf16x8 pb[NB][2][2];
        this->template softmax_tile<false>(sc, t, pb);
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int sl = 0; sl < 2; ++sl)
#pragma unroll
                for (int db = 0; db < C::NDB; ++db) {
                    const bf16x8 va = read_vt(v_lds, tb, sl, db);
#pragma unroll
                    for (int qb = 0; qb < NB; ++qb)
                        o[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[qb][tb][sl], o[db][qb], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
    }
};

template <int HD, int NB>
__global__ void __launch_bounds__(kThreads) paged_attn_stream_kernel(const KArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    using C = StreamCfg<HD, NB>;
    StreamAttn<HD, NB> at(a, smem);
    const int per_head = build_unit_prefix<C::RT>(a, at.prefix, at.misc);
    const int64_t total = static_cast<int64_t>(per_head) * a.h_kv;
    if (total == 0) return;
    const int w = blockIdx.x;
    const int64_t begin = wg_first_unit(w, total, a.n_wg);
    const int64_t end = wg_first_unit(w + 1, total, a.n_wg);
    if (begin >= end) return;

    UnitCursor ld;
    ld.pos = begin;
    ld.kvh = static_cast<int>(begin / per_head);
    const int rem = static_cast<int>(begin - static_cast<int64_t>(ld.kvh) * per_head);
    ld.s = locate_sequence(a, at.prefix, at.misc, rem);
    ld.u = rem - at.prefix[ld.s];
    at.cursor_enter(ld);
    UnitCursor cp = ld;

    // fill the ring: kStages - 1 units in flight
    int64_t issued = begin;
    for (int i = 0; i < C::kStages - 1 && ld.pos < end; ++i) {
        at.issue_unit(ld, static_cast<int>((issued - begin) % C::kStages));
        at.cursor_advance(ld, end);
        ++issued;
    }

    while (cp.pos < end) {
        // one segment: units of the same (sequence, head, row tile)
        at.s = cp.s;
        at.kvh = cp.kvh;
        at.sh = cp.sh;
        at.q0 = a.cu_q[cp.s];
        at.n0 = cp.n0;
        const int n_tiles = cp.sh.n_tiles;
        const int rt = cp.u / n_tiles;
        const int tile0 = cp.u - rt * n_tiles;
        const int64_t seg_begin = cp.pos;
        const int64_t seg_end = min(cp.pos + (n_tiles - tile0), end);
        const int tile1 = tile0 + static_cast<int>(seg_end - cp.pos);
        at.load_queries(rt);
        for (int tile = tile0; tile < tile1; ++tile) {
            // the unit at cp.pos must have landed: allow only the younger ones to be outstanding
            const int younger = static_cast<int>(issued - cp.pos) - 1;
            if (younger >= 2) wait_async_loads<2 * C::LOADS_PER_UNIT>();
            else if (younger == 1) wait_async_loads<C::LOADS_PER_UNIT>();
            else wait_async_loads<0>();
            __builtin_amdgcn_s_barrier();
            // every wave has finished the previous unit: its stage may be overwritten
            if (ld.pos < end) {
                at.issue_unit(ld, static_cast<int>((issued - begin) % C::kStages));
                at.cursor_advance(ld, end);
                ++issued;
            }
            const TileInfo t = at.tile_info(cp.sh, cp.kvh, tile, false);
            at.compute(static_cast<int>((cp.pos - begin) % C::kStages), t);
            at.cursor_advance(cp, end);
        }
        float l_tot[NB];
        at.row_sums(l_tot);
        const bool complete = tile0 == 0 && tile1 == n_tiles;
        if (complete) at.store_output(rt, l_tot);
        else at.store_partial(partial_slot(w, seg_begin, begin), l_tot);
    }
}

}  // namespace dfx
