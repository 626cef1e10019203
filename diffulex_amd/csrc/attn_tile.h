// Tile arithmetic shared by the paged-attention kernels: the LDS layout of a K or V tile, the
// matrix-instruction helpers, and S^T = K Q^T / O^T += V^T P^T on tiles in that layout.
//
// LDS tile layout: row-major [token][head_dim] as in the cache, with the 16-byte chunks of a
// row XOR-swizzled by the row index.
//   K operand (A of S^T = K Q^T): ds_read_b128 of chunk (2*slab + h) of row (lane % 32).
//   V operand (A of O^T += V^T P^T): needs 8 tokens of one d per lane, i.e. a column of the
//     tile.  ds_read_b64_tr_b16 transposes inside groups of 16 lanes: lane i of a group
//     receives element (i % 4) of what lanes {i/4, 4 + i/4, 8 + i/4, 12 + i/4} of the group
//     addressed.  Source lane s therefore points at token row (s / 4), elements 4*(s % 4)..+3
//     of a 16-wide d range, and lane i ends up with 4 consecutive tokens of d = i.
#pragma once

#include "attn_common.h"

namespace dfx {

DFX_D int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
// The thread's number in its workgroup, worked out where this is called (two instructions and a
// scalar) instead of being kept from the kernel's entry on: under register pressure the kept one,
// and every address derived from it ahead of a loop, is spilled to scratch, and a reload is a
// trip to memory.  `wave_number`: the wave's number as a wave-uniform value.
DFX_D int thread_number_here(int wave_number) {
    int zero = 0;
    asm volatile("" : "+v"(zero));  // (so that the count below is not computed early either)
    const int lane = static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, static_cast<uint32_t>(zero))));
    return wave_number * 64 + lane;
}

// Two e4m3 codes (bytes 0,1 or 2,3 of w) -> two bf16 packed in a dword, in one instruction
// (v_cvt_scalef32_pk_bf16_fp8 with scale 1).  An e4m3 value has 3 mantissa bits, so the widening is
// exact; checked against v_cvt_pk_f32_fp8 + truncation for all 65 536 pairs of codes.
template <bool HI>
DFX_D uint32_t fp8x2_to_bf16x2(uint32_t w) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, HI));
}

// 16 e4m3 codes -> 16 bf16 (two 16-byte chunks, in order).
DFX_D void widen16(u32x4 codes, u32x4& lo, u32x4& hi) {
    lo = u32x4{fp8x2_to_bf16x2<false>(codes.x), fp8x2_to_bf16x2<true>(codes.x),
               fp8x2_to_bf16x2<false>(codes.y), fp8x2_to_bf16x2<true>(codes.y)};
    hi = u32x4{fp8x2_to_bf16x2<false>(codes.z), fp8x2_to_bf16x2<true>(codes.z),
               fp8x2_to_bf16x2<false>(codes.w), fp8x2_to_bf16x2<true>(codes.w)};
}

template <int HD>
struct TileLayout {
    static constexpr int ROWB = HD * 2;                   // bytes per token row
    static constexpr int CPR = ROWB / 16;                 // 16-byte chunks per row
    static constexpr int MAT_BYTES = kTileTokens * ROWB;  // one K (or V) tile
    // chunk position = chunk index ^ swizzle(row).  The swizzle is a permutation of row bits chosen
    // for both operand reads:
    //   ds_read_b128 (K): 16 lanes = 16 consecutive rows of one chunk column per 256-byte LDS cycle
    //     -> the low four row bits (three plus the row's 128-byte half for head_dim 64) must give
    //     16 different positions: any bijection does;
    //   ds_read_b64_tr_b16 (V^T): 32 lanes = 4 consecutive rows x 4 consecutive chunks x 2 halves
    //     per cycle -> the rows' two low bits must move the chunk by multiples of 4, or the four
    //     rows land on the same 16 banks (a plain `row & 15` does that: 4-way conflicts, 8 cycles
    //     per instruction instead of 2).
    // Hence: row bits 0,1 -> position bits 2,3 and row bits 2,3 -> position bits 0,1 (head_dim
    // 128); for 128-byte rows the odd rows already sit 64 banks further, so row bit 1 -> position
    // bit 2 and row bits 2,3 -> position bits 0,1.
    DFX_HD static int swizzle(int row) {
        return HD == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
    }
    // byte offset of 16-byte chunk c of token row r inside a tile
    DFX_HD static int chunk_offset(int r, int c) { return r * ROWB + ((c ^ swizzle(r)) * 16); }
};

// The matrix instructions of the tile loop are issued from inline assembly so that the register
// file split is fixed by their operand constraints: the O^T accumulators live in the accumulation
// registers, which only matrix instructions touch in the loop, and the score accumulators in
// ordinary vector registers, where the softmax works on them in place.  Being volatile they keep
// their program order: an accumulator is reused every 4th (scores) or 8th (output) instruction,
// far beyond the result latency.  What the compiler can no longer do for them is insert the wait
// states the ISA requires around matrix instructions: each one is therefore preceded by two wait
// states (a vector-ALU result may feed it), and mfma_results_ready() / mfma_outputs_ready() put
// 18 wait states, the longest the ISA asks for, between a matrix result and a vector-ALU reader.
DFX_D void mfma_scores_first(f32x16& sc, bf16x8 k, bf16x8 q) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(sc) : "v"(k), "v"(q));
}
DFX_D void mfma_scores(f32x16& sc, bf16x8 k, bf16x8 q) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(sc) : "v"(k), "v"(q));
}
DFX_D void mfma_output(f32x16& acc, bf16x8 v, bf16x8 p) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(v), "v"(p));
}
DFX_D void mfma_results_ready(f32x16& x0, f32x16& x1, f32x16& x2, f32x16& x3) {
    asm volatile("s_nop 15\n\ts_nop 1" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));
}
DFX_D void mfma_results_ready(f32x16& x0, f32x16& x1) {
    asm volatile("s_nop 15\n\ts_nop 1" : "+v"(x0), "+v"(x1));
}
DFX_D void mfma_outputs_ready(f32x16& x0, f32x16& x1, f32x16& x2, f32x16& x3) {
    asm volatile("s_nop 15\n\ts_nop 1" : "+a"(x0), "+a"(x1), "+a"(x2), "+a"(x3));
}
DFX_D void mfma_outputs_ready(f32x16& x0, f32x16& x1) {
    asm volatile("s_nop 15\n\ts_nop 1" : "+a"(x0), "+a"(x1));
}

template <int HD, int NB, int NW, bool HIDDEN = false>
struct TileMath : AttnState<HD, NB, NW, HIDDEN> {
    using Base = AttnState<HD, NB, NW, HIDDEN>;
    using S = Shape<HD, NB, NW>;
    using L = TileLayout<HD>;
    using Base::col;
    using Base::half;
    using Base::lane;
    using Base::o;
    using Base::qf;

    // LDS addressing.  A tile starts at a multiple of its row pitch (256 or 128 bytes), so the
    // chunk swizzle, an XOR on bits 4..7 of the offset, can be applied to the finished address:
    //   K operand (tb, slab):       ((tile + k_lane) ^ (slab * 32)) + tb * 32 rows
    //   V operand (tb, sl, db, ii): ((tile + v_lane) ^ (z * 16)) + (tb * 32 + sl * 16 + ii * 8) rows,
    //                               z = (db * 4) ^ swizzle(ii * 8)
    // with one per-lane constant each.  Per tile that is one addition and a few XORs; the rest
    // folds into the instructions' immediate offsets.  (swizzle(r0 + x) == swizzle(r0) ^ swizzle(x)
    // holds for the row splits used here: 32-row blocks, and ii * 8 + (0..7) inside 16 rows.)
    uint32_t k_lane, v_lane;

    DFX_D explicit TileMath(const KArgs& args) : Base(args) {
        k_lane = col * L::ROWB + ((half ^ L::swizzle(col)) * 16);
        const int g16 = lane >> 4, sl16 = lane & 15;
        const int lrow = (g16 >> 1) * 4 + (sl16 >> 2);         // 0..7
        const int c = (g16 & 1) * 2 + ((sl16 & 3) >> 1);       // 0..3
        v_lane = lrow * L::ROWB + ((c ^ L::swizzle(lrow)) * 16) + (sl16 & 1) * 8;
    }

    DFX_D static uint32_t lds_address(const uint8_t* p) {
        return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p));
    }

    // ---- tile arithmetic -------------------------------------------------------------------
    // kx: the K tile's address plus k_lane, XORed with slab * 32
    DFX_D bf16x8 read_k(uint32_t kx, int tb) const {
        typedef __attribute__((address_space(3))) bf16x8 lds_bf16x8;
        return *(const lds_bf16x8*)static_cast<uintptr_t>(kx + tb * 32 * L::ROWB);
    }

    // V^T operand for token slab (tb, sl) and d block db; vx[db * 2 + ii]: the V tile's address
    // plus v_lane, XORed with ((db * 4) ^ swizzle(ii * 8)) * 16.
    static constexpr int kVx = S::NDB * 2;
    DFX_D bf16x8 read_vt(const uint32_t (&vx)[kVx], int tb, int sl, int db) const {
        typedef short short4v __attribute__((ext_vector_type(4)));
        typedef short short8v __attribute__((ext_vector_type(8)));
        typedef __attribute__((address_space(3))) short4v lds_short4v;
        short4v r[2];
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) {
            const uint32_t p = vx[db * 2 + ii] + (tb * 32 + sl * 16 + ii * 8) * L::ROWB;
            r[ii] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)static_cast<uintptr_t>(p));
        }
        const short8v v = __builtin_shufflevector(r[0], r[1], 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, v);
    }

    // The LDS operands of the next step are requested before the matrix instructions of the
    // current one: being volatile assembly those pin the order, so the LDS latency is hidden
    // only by what the source puts in between.
    DFX_D void scores(const uint8_t* k_tile, f32x16 (&sc)[2][NB]) const {
        const uint32_t k0 = lds_address(k_tile) + k_lane;
        bf16x8 ka[2][2];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) ka[0][tb] = read_k(k0, tb);
#pragma unroll
        for (int slab = 0; slab < S::NSLAB; ++slab) {
            if (slab + 1 < S::NSLAB) {
                const uint32_t kx = k0 ^ ((slab + 1) * 32);
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) ka[(slab + 1) & 1][tb] = read_k(kx, tb);
            }
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int qb = 0; qb < NB; ++qb) {
                    if (slab == 0) mfma_scores_first(sc[tb][qb], ka[slab & 1][tb], qf[qb][slab]);
                    else mfma_scores(sc[tb][qb], ka[slab & 1][tb], qf[qb][slab]);
                }
        }
        if constexpr (NB == 2) mfma_results_ready(sc[0][0], sc[0][1], sc[1][0], sc[1][1]);
        else mfma_results_ready(sc[0][0], sc[1][0]);
    }

    // Wait states before vector instructions read the O^T accumulators (rescale, epilogue).
    DFX_D void outputs_ready() {
        if constexpr (HIDDEN) {
            pipe_outputs_ready();
            return;
        }
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            if constexpr (S::NDB == 4) mfma_outputs_ready(o[0][qb], o[1][qb], o[2][qb], o[3][qb]);
            else mfma_outputs_ready(o[0][qb], o[1][qb]);  // (never one accumulator twice: the second would be a copy,
                                                          //  made before the wait states)
        }
    }

    // For the path of a branch that leaves the accumulators alone: names them as matrix-instruction
    // operands there too, so that where the paths meet both values already live in the
    // accumulation registers and none is carried through ordinary registers around the loop.
    DFX_D void outputs_untouched() {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            if constexpr (S::NDB == 4) asm volatile("" : "+a"(o[0][qb]), "+a"(o[1][qb]), "+a"(o[2][qb]), "+a"(o[3][qb]));
            else asm volatile("" : "+a"(o[0][qb]), "+a"(o[1][qb]));
        }
    }

    DFX_D void accumulate(const uint8_t* v_tile, const bf16x8 (&pb)[NB][2][2]) {
        constexpr int kSteps = 4 * S::NDB;  // (tb, sl, db)
        uint32_t vx[kVx];
        vx[0] = lds_address(v_tile) + v_lane;
#pragma unroll
        for (int z = 1; z < kVx; ++z) vx[z] = vx[0] ^ ((((z >> 1) * 4) ^ L::swizzle((z & 1) * 8)) * 16);
        bf16x8 va[3];
        va[0] = read_vt(vx, 0, 0, 0);
        va[1] = read_vt(vx, 0, 0, 1);
#pragma unroll
        for (int st = 0; st < kSteps; ++st) {
            const int tb = st / (2 * S::NDB), sl = (st / S::NDB) & 1, db = st % S::NDB;
            if (st + 2 < kSteps) {
                const int n = st + 2;
                va[n % 3] = read_vt(vx, n / (2 * S::NDB), (n / S::NDB) & 1, n % S::NDB);
            }
#pragma unroll
            for (int qb = 0; qb < NB; ++qb) mfma_output(o[db][qb], va[st % 3], pb[qb][tb][sl]);
        }
        // the compiler may move the accumulators to other registers right behind this stream
        outputs_ready();
    }

    // ---- tiles of a cache in the distinct layout ------------------------------------------------
    // K [pages, H, HD / 8, page, 8]: 64 consecutive tokens of one chunk column are 1 KiB contiguous, and that
    // is how the tile lies in LDS: chunk-major, [HD / 8 chunk columns][64 tokens][16 bytes].  The operand of
    // (token block tb, slab) is chunk column 2 * slab + half, 32 consecutive tokens: 16 lanes read 256
    // contiguous bytes, no swizzle needed.  The lane that feeds matrix row r reads token swap_quads(r): with
    // quads 1 and 2 of every 16 rows swapped the score registers of a lane hold 8 consecutive tokens
    // (softmax_tile<.., NATURAL>), which is the order a d-major V row holds them in.
    DFX_HD static int swap_quads(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }
    static constexpr int CHUNK_COL_BYTES = kTileTokens * 16;
    DFX_D void scores_chunk_major(const uint8_t* k_tile, f32x16 (&sc)[2][NB]) const {
        typedef __attribute__((address_space(3))) bf16x8 lds_bf16x8;
        const uint32_t k0 = lds_address(k_tile) + static_cast<uint32_t>(half * CHUNK_COL_BYTES + swap_quads(col) * 16);
        auto read = [&](int slab, int tb) {
            return *(const lds_bf16x8*)static_cast<uintptr_t>(k0 + slab * 2 * CHUNK_COL_BYTES + tb * 32 * 16);
        };
        bf16x8 ka[2][2];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) ka[0][tb] = read(0, tb);
#pragma unroll
        for (int slab = 0; slab < S::NSLAB; ++slab) {
            if (slab + 1 < S::NSLAB) {
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) ka[(slab + 1) & 1][tb] = read(slab + 1, tb);
            }
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int qb = 0; qb < NB; ++qb) {
                    if (slab == 0) mfma_scores_first(sc[tb][qb], ka[slab & 1][tb], qf[qb][slab]);
                    else mfma_scores(sc[tb][qb], ka[slab & 1][tb], qf[qb][slab]);
                }
        }
        if constexpr (NB == 2) mfma_results_ready(sc[0][0], sc[0][1], sc[1][0], sc[1][1]);
        else mfma_results_ready(sc[0][0], sc[1][0]);
    }

    // V [pages, H, HD, page] is d-major, and so is its tile in LDS: row d holds the tile's 64 tokens (128
    // bytes, eight 16-byte chunks of 8 tokens), which is the V^T operand's shape already.  Chunks are
    // swizzled by (d / 2) % 8: 16 consecutive d of one chunk column then cover all 64 banks once.
    DFX_HD static int vt_chunk_offset(int d, int chunk) { return d * (kTileTokens * 2) + ((chunk ^ ((d >> 1) & 7)) * 16); }

    // O^T += V^T P^T from a d-major V tile: the operand of (token slab tb, sl; d block db) is one 16-byte
    // read per lane, row db * 32 + col, chunk tb * 4 + sl * 2 + half -- the 8 tokens whose probabilities
    // the lane's half of the wave holds in pb[.][tb][sl], in the same order (the caller's business: the
    // chunk holds them as its layout says).
    DFX_D void accumulate_dmajor(const uint8_t* v_tile, const bf16x8 (&pb)[NB][2][2]) {
        typedef __attribute__((address_space(3))) bf16x8 lds_bf16x8;
        constexpr int kSteps = 4 * S::NDB;  // (tb, sl, db)
        // Row db * 32 + col, chunk (tb * 4 + sl * 2 + half) ^ swizzle: the swizzle depends on col only and
        // tb * 4 + sl * 2 is even, so the lane's part of the address is one constant, the slab an XOR
        // on bits 5..6 of the finished address (tiles start at multiples of 256) and the d block an
        // immediate offset -- four address registers instead of one per operand.
        const uint32_t v0 = lds_address(v_tile) + static_cast<uint32_t>(vt_chunk_offset(col, half));
        auto read = [&](int st) {
            const int tb = st / (2 * S::NDB), sl = (st / S::NDB) & 1, db = st % S::NDB;
            return *(const lds_bf16x8*)static_cast<uintptr_t>((v0 ^ ((tb * 4 + sl * 2) * 16)) + db * 32 * (kTileTokens * 2));
        };
        bf16x8 va[3];
        va[0] = read(0);
        va[1] = read(1);
#pragma unroll
        for (int st = 0; st < kSteps; ++st) {
            const int tb = st / (2 * S::NDB), sl = (st / S::NDB) & 1, db = st % S::NDB;
            if (st + 2 < kSteps) va[(st + 2) % 3] = read(st + 2);
#pragma unroll
            for (int qb = 0; qb < NB; ++qb) mfma_output(o[db][qb], va[st % 3], pb[qb][tb][sl]);
        }
        outputs_ready();
    }
};

}  // namespace dfx
