// State and arithmetic shared by the paged-attention kernels: kernel arguments, the per-lane
// attention state of one (sequence, KV head, row tile) item, the online softmax on S^T and
// the epilogues (normalised rows, partial results, merge of partial results).
//
// MFMA 32x32x16 bf16 register layouts relied upon (lane l, h = l / 32):
//   A: row l % 32, contraction elements 8h .. 8h+7        B: column l % 32, same elements
//   C/D: column l % 32, rows 8*i + 4*h + j for accumulator index 4*i + j
// S^T = K Q^T puts one query in one lane column, so the softmax row statistics are a
// register reduction plus one cross-half shuffle, and the S^T accumulators, rounded to bf16,
// are already the B operand of O^T += V^T P^T: elements 8*sl .. 8*sl+7 of block tb are
// tokens 32*tb + 16*sl + {4h..4h+3, 8+4h..8+4h+3}.
#pragma once

#include "attn_pipe_gen.h"
#include "dfx_common.h"
#include "fp8_e4m3.h"
#include "partition.h"

namespace dfx {

constexpr int kThreads = 256;  // workgroup size of the 4-wave kernels
constexpr int kWaves = 4;
constexpr int kMaxWaves = 8;
constexpr int kMaxSeqs = 4095;
constexpr float kLog2e = 1.4426950408889634f;
// The running row maximum is only raised (and the accumulators rescaled) when a tile exceeds it
// by more than this many powers of two; until then probabilities up to 2^8 are accumulated
// against the stale maximum, which fp32 accumulators and bf16 probabilities hold without loss.
constexpr float kRescaleThreshold = 8.0f;

struct KArgs {
    const uint16_t* q;
    const uint16_t* k_new;
    const uint16_t* v_new;
    const uint8_t* k_cache;
    const uint8_t* v_cache;
    uint16_t* out;
    const int32_t* block_tables;
    const int32_t* context_lens;
    const int32_t* cu_q;
    const int32_t* cu_new;
    const float* k_scale;
    const float* v_scale;
    float* workspace;  // partial-result slots
    int* arrivals;     // one arrival counter per workgroup, zero between launches
    const void* store_slots;  // fused KV-cache store: slot per fresh row, or null
    int store_slots_i64;
    int64_t n_new;            // rows of k_new / v_new (and of the slot mapping)
    int32_t n_q;              // rows of q / out: no row at or beyond it is read or written, whatever the offsets say
    // Rotary embedding inside the launch (pipelined kernels; null table: off).  q and k_src hold the
    // projections as they leave the linear layer; the query rows are rotated in the Q operand registers, the
    // fresh K rows of an item by the workgroup that owns the item's fresh tiles, from k_src into k_new (which
    // is then an output of the launch that its own tile loads read back), and into the cache with the store.
    const float* rope_table;  // [rope_max_pos, head_dim] fp32: cosines, then sines
    const void* rope_pos;     // position of token t: row t of q and row t of k_src / k_new / v_new (the same tokens)
    int rope_pos_i64;
    int64_t rope_max_pos;
    const uint16_t* k_src;
    int64_t ks_st, ks_sh;
    int64_t v_fresh_delta;    // streaming paths: (token stride of v_new - token stride of k_new) in bytes
    const uint8_t* plan;      // launch plan built by the plan kernels, or null
    uint32_t plan_signature;  // of this launch's configuration: a plan made for another one is ignored
    int32_t plan_capacity;    // unit descriptors the plan buffer has room for (fixes where its tables start)
    int64_t q_st, q_sh, kn_st, kn_sh, vn_st, vn_sh, o_st, o_sh;
    int64_t c_sp, c_st, c_sh;  // cache strides in elements: page, token, head
    // "distinct" cache layout (generic path only), strides in elements: K [page, head, d / 8, token, 8],
    // V [page, head, d, token]
    int64_t kd_sp, kd_sh, kd_sc, vd_sp, vd_sh, vd_sd;
    int64_t bt_stride, n_pages;
    int num_seqs, h_kv, group, page_size, page_shift, max_pages, dbs, mask_mode, n_wg;
    int fixed_wg;  // the caller fixed the number of workgroups: all of them take part
    int busy_waves;  // streaming kernels: waves from this one on have query rows in no item of the launch
    float c;  // scale * log2(e)
};

// Sizes that do not depend on how a kernel stages its tiles.
// HD: head_dim; NB: 32-row query blocks per wave; NW: waves per workgroup.
template <int HD, int NB, int NW = kWaves>
struct Shape {
    static constexpr int TN = kTileTokens;
    static constexpr int THREADS = 64 * NW;
    static constexpr int RT = 32 * NB * NW;      // query rows per row tile
    static constexpr int NSLAB = HD / 16;        // contraction slabs of Q K^T
    static constexpr int NDB = HD / 32;          // 32-row blocks of O^T
    static constexpr int PREFIX_BYTES = (kMaxSeqs + 1) * 4;
    static constexpr int MISC_BYTES = 128;
    // A partial result is stored per 32-row query block b = wave * NB + qb, whatever the shape of
    // the workgroup that wrote it, in an area of BLOCK_FLOATS floats: 2 * NDB chunks of 64 x 16
    // bytes of fp16 accumulators, then 64 x 16 bytes of row statistics (the format is described at
    // AttnState::store_partial).
    static constexpr int BLOCKS = NB * NW;
    static constexpr int BLOCK_FLOATS = 256 * (2 * NDB + 1);
    static constexpr int SLOT_FLOATS = BLOCKS * BLOCK_FLOATS;
};

// max(x of lane i, x of lane i ^ 32): v_permlane32_swap exchanges the halves of a wave inside the
// vector ALU (a __shfl_xor is an LDS instruction with a round trip of its own per tile).
DFX_D float wave_xor32_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
DFX_D float wave_xor32_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

DFX_D float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

DFX_D int block_inclusive_scan(int v, int* scratch, int& block_total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int x = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int y = __shfl_up(x, d);
        if (lane >= d) x += y;
    }
    if (lane == 63) scratch[wave] = x;
    __syncthreads();
    int off = 0, tot = 0;
    const int n_waves = blockDim.x >> 6;
#pragma unroll
    for (int w = 0; w < kMaxWaves; ++w) {
        if (w < n_waves) {
            const int t = scratch[w];
            if (w < wave) off += t;
            tot += t;
        }
    }
    __syncthreads();
    block_total = tot;
    return x + off;
}

DFX_D SeqShape load_seq_shape(const KArgs& a, int s, int rows_per_tile) {
    const int ctx = (a.context_lens != nullptr && a.k_cache != nullptr) ? a.context_lens[s] : 0;
    const int q_len = a.cu_q[s + 1] - a.cu_q[s];
    // fresh rows are clamped to the rows k_new / v_new have (padded batches carry offsets beyond them)
    const int64_t n0 = min(static_cast<int64_t>(a.cu_new[s]), a.n_new), n1 = min(static_cast<int64_t>(a.cu_new[s + 1]), a.n_new);
    const int new_len = static_cast<int>(n1 - n0);
    return make_seq_shape(ctx, q_len, new_len, a.group, rows_per_tile, a.mask_mode == DFX_MASK_BLOCK_CAUSAL, a.dbs);
}

// What the softmax needs to know about one KV tile.
struct TileInfo {
    int base;      // index of the tile's first token within its kind (context or fresh)
    int limit;     // number of valid tokens of that kind
    bool is_ctx;
    float c_tile;  // logit -> log2 domain factor (scale * log2 e, times k_scale for FP8 context)
    float v_mul;   // factor applied to P before the PV product: 1, except 1 / v_scale for the fresh (bf16)
                   // tiles of a launch on an FP8 cache, whose O^T is kept in units of v_scale
    uint64_t holes;  // bit b: tokens base + b * HOLE_ROWS .. + HOLE_ROWS - 1 (HOLE_ROWS: a parameter of
                     // softmax_tile) sit on a page whose block-table entry is negative or out of range
                     // and are skipped, as the reference skips such pages
                     // (diffulex_kernel/python/dllm_flash_attn.py:260-261)
};

// HIDDEN: the O^T accumulators live in the fixed registers of attn_pipe_gen.h instead of `o`
// (pipelined kernel); the epilogues reach them one 32-row d block at a time through get_o / set_o.
template <int HD, int NB, int NW = kWaves, bool HIDDEN = false>
struct AttnState {
    using S = Shape<HD, NB, NW>;
    static_assert(!HIDDEN || ((HD == 128 || HD == 64) && NB == 1), "register map of attn_pipe_gen.h");

    const KArgs& a;
    const int tid, lane, wave, col, half;

    SeqShape sh;
    int s, kvh, q0, n0;
    bf16x8 qf[NB][S::NSLAB];
    f32x16 o[S::NDB][NB];
    float m_run[NB], l_run[NB];
    int vis_limit[NB];
    float out_mul = 1.0f;  // O^T is accumulated in units of this (v_scale of the item's head on an FP8 cache)

    DFX_D explicit AttnState(const KArgs& args)
        : a(args), tid(threadIdx.x), lane(threadIdx.x & 63), wave(threadIdx.x >> 6), col(threadIdx.x & 31),
          half((threadIdx.x >> 5) & 1) {}

    DFX_D f32x16 get_o(int db, int qb) const {
        if constexpr (HIDDEN) return pipe_get_output(db);
        else return o[db][qb];
    }
    DFX_D void set_o(int db, int qb, const f32x16& v) {
        if constexpr (HIDDEN) pipe_set_output(db, v);
        else o[db][qb] = v;
    }

    DFX_D void set_sequence(int seq, int kv_head) {
        s = seq;
        kvh = kv_head;
        sh = load_seq_shape(a, s, S::RT);
        q0 = a.cu_q[s];
        n0 = a.cu_new[s];
    }

    DFX_D TileInfo tile_info(const SeqShape& shp, int kv_head, int tile, bool fp8) const {
        TileInfo t;
        t.is_ctx = tile < shp.n_ctx_tiles;
        t.base = (t.is_ctx ? tile : tile - shp.n_ctx_tiles) * S::TN;
        t.limit = t.is_ctx ? shp.ctx : shp.new_len;
        t.c_tile = a.c;
        t.v_mul = 1.0f;
        t.holes = 0;
        if (fp8) {
            if (t.is_ctx) t.c_tile = fmaxf(a.c * a.k_scale[kv_head], 1e-30f);
            else t.v_mul = 1.0f / a.v_scale[kv_head];
        }
        return t;
    }

    DFX_D int row_of(int rt, int qb) const { return rt * S::RT + (wave * NB + qb) * 32 + col; }

    DFX_D void reset_accumulators() {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            m_run[qb] = -INFINITY;
            l_run[qb] = 0.0f;
            if constexpr (!HIDDEN) {
#pragma unroll
                for (int db = 0; db < S::NDB; ++db)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[db][qb][e] = 0.0f;
            }
        }
        if constexpr (HIDDEN && HD == 128) pipe_zero_outputs();
        if constexpr (HIDDEN && HD == 64) pipe64_zero_outputs();
    }

    // Q rows of row tile rt into B-operand registers (zeros for rows past G * q_len).
    DFX_D void load_queries(int rt) {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            const int r = row_of(rt, qb);
            bool valid = r < a.group * sh.q_len;
            const int g = valid ? r / sh.q_len : 0;
            const int i = valid ? r - g * sh.q_len : 0;
            valid = valid && i < a.n_q - q0;
            vis_limit[qb] = (i / a.dbs + 1) * a.dbs;
            const uint16_t* qp = a.q + (q0 + i) * a.q_st + (kvh * a.group + g) * a.q_sh + half * 8;
#pragma unroll
            for (int slab = 0; slab < S::NSLAB; ++slab) {
                u32x4 v = {0, 0, 0, 0};
                if (valid) v = *reinterpret_cast<const u32x4*>(qp + slab * 16);
                qf[qb][slab] = __builtin_bit_cast(bf16x8, v);
            }
        }
        reset_accumulators();
    }

    // Mask, online softmax and bf16 rounding of one tile's S^T; updates m_run, l_run and
    // rescales o when a row maximum grows.  pb[qb][tb][sl] is the B operand of the PV product.
    // before_rescale() runs ahead of any vector-ALU access to o (kernels that issue their matrix
    // instructions behind the compiler's back insert the required wait states there).
    // NATURAL: the key rows went into S^T = K Q^T with quads 1 and 2 of every 16 swapped (scores_chunk_major),
    // so that a lane's registers hold the scores of tokens 8 * half .. 8 * half + 7 of a 16-token slab, in
    // order -- the order of a d-major V row; holes then come a tile at a time (any bit set: all of it).
    template <bool SCALE_P, int HOLE_ROWS, bool NATURAL = false, typename BeforeRescale>
    DFX_D void softmax_tile(f32x16 (&sc)[2][NB], const TileInfo& t, bf16x8 (&pb)[NB][2][2],
                            BeforeRescale&& before_rescale) {
        const bool mask_valid = t.base + S::TN > t.limit;
        const bool mask_bc = !t.is_ctx && a.mask_mode == DFX_MASK_BLOCK_CAUSAL;
        static_assert(HOLE_ROWS == 1 || HOLE_ROWS % 8 == 0, "a lane's 4 * half offset must stay inside a hole unit");
        if (mask_valid || mask_bc || t.holes != 0) {
            // token-granular holes: this lane's tokens sit 4 * half higher
            const uint64_t holes = (HOLE_ROWS == 1 && half) ? (t.holes >> 4) : t.holes;
#pragma unroll
            for (int qb = 0; qb < NB; ++qb) {
                int lim = t.limit;
                if (mask_bc) lim = min(lim, vis_limit[qb]);
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int in_tile = NATURAL ? tb * 32 + (e >> 3) * 16 + ((e >> 2) & 1) * 4 + (e & 3) : tb * 32 + (e >> 2) * 8 + (e & 3);
                        const int tok = t.base + in_tile + half * (NATURAL ? 8 : 4);
                        const bool hole = NATURAL ? holes != 0 : ((holes >> (in_tile / HOLE_ROWS)) & 1) != 0;
                        if (tok >= lim || hole) sc[tb][qb][e] = -INFINITY;
                    }
            }
        }
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            float mx = -INFINITY;
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[tb][qb][e]);
            mx = wave_xor32_max(mx);
            const float m_tile = mx * t.c_tile;
            if (__any(m_tile > m_run[qb] + kRescaleThreshold)) {
                const float m_new = fmaxf(m_run[qb], m_tile);
                // (the first tile of a piece finds every row at -inf and O^T at zero: nothing to rescale)
                if (__any(m_run[qb] != -INFINITY)) {
                    before_rescale();
                    const float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_run[qb] - m_new);
                    l_run[qb] *= alpha;
#pragma unroll
                    for (int db = 0; db < S::NDB; ++db)
#pragma unroll
                        for (int e = 0; e < 16; ++e) o[db][qb][e] *= alpha;
                }
                m_run[qb] = m_new;
            }
            const float m_safe = (m_run[qb] == -INFINITY) ? 0.0f : m_run[qb];
            float lsum = 0.0f;
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) {
                float p[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    p[e] = fast_exp2(__builtin_fmaf(sc[tb][qb][e], t.c_tile, -m_safe));
                    lsum += p[e];
                }
                if (SCALE_P && t.v_mul != 1.0f) {  // (wave-uniform; fresh tiles of an FP8 launch only)
#pragma unroll
                    for (int e = 0; e < 16; ++e) p[e] *= t.v_mul;
                }
#pragma unroll
                for (int sl = 0; sl < 2; ++sl) {
                    bf16x8 v;
#pragma unroll
                    for (int e = 0; e < 8; e += 2) {
                        const bf16x2 r = __builtin_convertvector(f32x2{p[sl * 8 + e], p[sl * 8 + e + 1]}, bf16x2);
                        v[e] = r.x;
                        v[e + 1] = r.y;
                    }
                    pb[qb][tb][sl] = v;
                }
            }
            l_run[qb] += lsum;
        }
    }

    DFX_D void row_sums(float (&l_tot)[NB]) const {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) l_tot[qb] = wave_xor32_sum(l_run[qb]);
    }

    // Whether the 32 rows of block qb of this wave exist in row tile rt of the current item.
    DFX_D bool block_has_rows(int rt, int qb) const {
        return rt * S::RT + (wave * NB + qb) * 32 < a.group * sh.q_len;
    }

    // Normalised rows: accumulator 4*i + j of block db is element d = 32*db + 8*i + 4*half + j.
    // The two lanes of a row (half 0 and 1) hold the two halves of every 16-byte chunk of the
    // row; they exchange them (v_permlane32_swap) so that each stores whole chunks: the lower
    // lane the even ones, the upper lane the odd ones.
    DFX_D void store_output(int rt, const float (&l_tot)[NB]) const {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            const int r = row_of(rt, qb);
            bool valid = r < a.group * sh.q_len;
            const int g = valid ? r / sh.q_len : 0;
            const int i = valid ? r - g * sh.q_len : 0;
            valid = valid && i < a.n_q - q0;  // (a plan made before the offsets were rewritten in place may say otherwise)
            // a row none of whose keys is visible (every page of its context a hole, no fresh rows)
            // has a zero sum: it gets zeros, not 0 * inf
            const float inv = l_tot[qb] > 0.0f ? out_mul / l_tot[qb] : 0.0f;
            uint16_t* op = a.out + (q0 + i) * a.o_st + (kvh * a.group + g) * a.o_sh + half * 8;
#pragma unroll
            for (int db = 0; db < S::NDB; ++db) {
                const f32x16 ov = get_o(db, qb);
#pragma unroll
                for (int pair = 0; pair < 2; ++pair) {
                    uint32_t w[2][2];  // [chunk of the pair][dword of this lane's half of it]
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        const int ii = pair * 2 + c;
                        w[c][0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(
                            f32x2{ov[ii * 4 + 0] * inv, ov[ii * 4 + 1] * inv}, bf16x2));
                        w[c][1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(
                            f32x2{ov[ii * 4 + 2] * inv, ov[ii * 4 + 3] * inv}, bf16x2));
                    }
                    // afterwards x[0] is the lower-half dword and x[1] the upper-half dword of
                    // chunk `half` of the pair
                    const auto x0 = __builtin_amdgcn_permlane32_swap(w[0][0], w[1][0], false, false);
                    const auto x1 = __builtin_amdgcn_permlane32_swap(w[0][1], w[1][1], false, false);
                    const u32x4 chunk = {x0[0], x1[0], x0[1], x1[1]};
                    if (valid) *reinterpret_cast<u32x4*>(op + db * 32 + pair * 16) = chunk;
                }
            }
        }
    }

    DFX_D float* slot_ptr(int slot) const { return a.workspace + static_cast<int64_t>(slot) * S::SLOT_FLOATS; }

    // Partial results travel between workgroups on different XCDs, whose L2 caches are not
    // coherent with each other for ordinary accesses.  They are therefore written and read with
    // device-scope accesses (the sc1 cache-policy bit of the buffer instructions), which go
    // through to memory, instead of bracketing ordinary accesses with device-scope fences: such a
    // fence writes back and invalidates the whole L2 of the XCD, which costs far more than these
    // few kilobytes.  16 bytes per lane: one such instruction keeps the address unit busy as
    // long as a 4-byte one.
    typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
    static constexpr int kDeviceScope = 16;  // cache policy: sc1

    DFX_D __amdgpu_buffer_rsrc_t block_resource(int slot, int qb) const {
        // (the wave's number made opaque here: its share of the address, worked out at the kernel's entry,
        // would wait in scratch until an item is cut, and the reload is a trip to memory)
        int w = wave;
        asm volatile("" : "+v"(w));
        float* bp = slot_ptr(slot) + (w * NB + qb) * S::BLOCK_FLOATS;
        return __builtin_amdgcn_make_buffer_rsrc(bp, 0, S::BLOCK_FLOATS * 4, 0x00020000);
    }

    // A stored piece of an item: per 32-row block the unnormalised accumulators as fp16 relative to
    // a power of two per query row (the exponent of the row's largest magnitude, so scaling is
    // exact and every value lands in (-2, 2)), then per lane 16 bytes {running maximum, row sum,
    // that power of two, 0} in fp32.  Chunk c (accumulators 8 * (c & 1) .. + 7 of d block c >> 1)
    // is 16 bytes at (c * 64 + lane) * 16, the statistics at kStatsOff + lane * 16.  Half the
    // bytes of an fp32 copy: moving a piece is limited by the memory path of one compute unit.
    // The rounding (2^-12 of the row's largest accumulator) is an eighth of what the bf16 output
    // rounding adds afterwards.
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    static constexpr int kChunks = S::NDB * 2;
    static constexpr int kStatsOff = kChunks * 64 * 16;
    static_assert(kStatsOff + 64 * 16 == S::BLOCK_FLOATS * 4, "a block fills its slot exactly");

    // 2^-(exponent of mx) and its inverse (1 for zero); mx >= 0.
    DFX_D static void row_scale(float mx, float& down, float& up) {
        uint32_t e = (__float_as_uint(mx) >> 23) & 0xffu;
        e = e > 253u ? 253u : e;  // infinities and NaNs stay what they are in fp16 whatever the scale
        const uint32_t d = e == 0 ? 127u : 254u - e;
        down = __uint_as_float(d << 23);
        up = __uint_as_float((254u - d) << 23);
    }

    // The largest magnitude among the accumulators of the lane's query row (both lanes of the row).
    DFX_D float row_magnitude(int qb) const {
        float mx = 0.0f;
#pragma unroll
        for (int db = 0; db < S::NDB; ++db) {
            const f32x16 ov = get_o(db, qb);
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, fabsf(ov[e]));
        }
        return wave_xor32_max(mx);
    }

    DFX_D static uint32_t to_f16x2(float x, float y) {
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{x, y}, f16x2));
    }
    DFX_D static f32x2 from_f16x2(uint32_t w) {
        return __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
    }

    // (the lane's number made opaque where a piece is moved: offsets derived from it at the kernel's entry
    // would wait in scratch until an item is cut)
    DFX_D int lane_here() const {
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    }

    DFX_D void store_partial(int slot, const float (&l_tot)[NB]) const {
        if (wave >= a.busy_waves) return;  // no rows in any item of the launch: merge_partial skips it too
        const int lane = lane_here();
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            const __amdgpu_buffer_rsrc_t rs = block_resource(slot, qb);
            float down, up;
            row_scale(row_magnitude(qb), down, up);
#pragma unroll
            for (int c = 0; c < kChunks; ++c) {
                const int db = c >> 1, e0 = (c & 1) * 8;
                const f32x16 ov = get_o(db, qb);
                u32x4v w;
                w.x = to_f16x2(ov[e0 + 0] * down, ov[e0 + 1] * down);
                w.y = to_f16x2(ov[e0 + 2] * down, ov[e0 + 3] * down);
                w.z = to_f16x2(ov[e0 + 4] * down, ov[e0 + 5] * down);
                w.w = to_f16x2(ov[e0 + 6] * down, ov[e0 + 7] * down);
                __builtin_amdgcn_raw_buffer_store_b128(w, rs, (c * 64 + lane) * 16, 0, kDeviceScope);
            }
            const f32x4 st = {m_run[qb], l_tot[qb], up, 0.0f};
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4v, st), rs, kStatsOff + lane * 16, 0,
                                                   kDeviceScope);
        }
    }

    // Round the accumulators to what store_partial() would have stored.  A workgroup that merges a
    // stored piece into its own piece does this first: had the two arrived in the other order,
    // the other side would have read this piece in its stored form, and the result must not
    // depend on who merges.
    DFX_D void round_to_stored_form() {
        if (wave >= a.busy_waves) return;
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            float down, up;
            row_scale(row_magnitude(qb), down, up);
#pragma unroll
            for (int db = 0; db < S::NDB; ++db) {
                f32x16 ov = get_o(db, qb);
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    const f32x2 v = from_f16x2(to_f16x2(ov[e] * down, ov[e + 1] * down));
                    ov[e] = v.x * up;
                    ov[e + 1] = v.y * up;
                }
                set_o(db, qb, ov);
            }
        }
    }

    // HIDDEN kernels: the wave's block of the stored piece `slot` on its way into the registers of the score
    // sets (free between two runs), all nine loads at once -- through the compiler's few registers they would go
    // three at a time, a trip to memory each.  Asked for before this workgroup rounds its own piece, which takes
    // as long as the trip.
    DFX_D void request_partial(int slot) const {
        static_assert(HIDDEN && NB == 1, "registers of attn_pipe_gen.h");
        if (wave >= a.busy_waves) return;
        int w = wave;
        asm volatile("" : "+v"(w));
        const uint8_t* p = reinterpret_cast<const uint8_t*>(slot_ptr(slot) + w * S::BLOCK_FLOATS) + lane_here() * 16;
        if constexpr (HD == 128) pipe_request_partial(p, p + 3 * 1024, p + 6 * 1024);
        else pipe64_request_partial(p, p + 4 * 1024);
    }

    // Merge one stored piece into the running state (l_run holds whole-row sums here): the piece in `slot`, or
    // (REQUESTED) the one request_partial() has asked for.
    DFX_D void merge_partial(int slot) { merge_partial_from<false>(slot); }
    DFX_D void merge_requested_partial() { merge_partial_from<true>(0); }
    template <bool REQUESTED>
    DFX_D void merge_partial_from(int slot) {
        // No fused multiply-add in here: a * wa + b * wb must round both products, or merging a
        // into b and b into a differ in the last bit (an fma keeps one product exact, and which
        // one depends on who merges).  __fmul_rn / __fadd_rn would not do: they are plain operators
        // in this toolchain and fuse like any other.
#pragma clang fp contract(off)
        if (wave >= a.busy_waves) return;
        const int lane = lane_here();
        if constexpr (REQUESTED) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            __amdgpu_buffer_rsrc_t rs;
            if constexpr (!REQUESTED) rs = block_resource(slot, qb);
            // piece c of the block: chunks 0 .. kChunks - 1, then the statistics
            auto piece = [&](int c) {
                if constexpr (REQUESTED) return __builtin_bit_cast(u32x4v, pipe_partial_chunk(c));
                else return __builtin_amdgcn_raw_buffer_load_b128(rs, (c * 64 + lane) * 16, 0, kDeviceScope);
            };
            const f32x4 st = __builtin_bit_cast(f32x4, piece(kChunks));
            const float mp = st[0], lp = st[1], up = st[2];
            const float mn = fmaxf(m_run[qb], mp);
            const float wa = (m_run[qb] == -INFINITY) ? 0.0f : fast_exp2(m_run[qb] - mn);
            const float wb = (mp == -INFINITY) ? 0.0f : fast_exp2(mp - mn);
            // products and sum are rounded separately: merging a into b then gives the same bits as
            // b into a, so it does not matter which of two pieces does the merging
            const float la = l_run[qb] * wa, lb = lp * wb;
            l_run[qb] = la + lb;
            m_run[qb] = mn;
#pragma unroll
            for (int db = 0; db < S::NDB; ++db) {
                f32x16 ov = get_o(db, qb);
#pragma unroll
                for (int hc = 0; hc < 2; ++hc) {
                    const int c = db * 2 + hc, e0 = hc * 8;
                    const u32x4v w = piece(c);
                    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const f32x2 h = from_f16x2(ws[j]);
                        const float b0 = h.x * up, b1 = h.y * up;  // exact: a power of two
                        const float oa0 = ov[e0 + 2 * j] * wa, ob0 = b0 * wb;
                        const float oa1 = ov[e0 + 2 * j + 1] * wa, ob1 = b1 * wb;
                        ov[e0 + 2 * j] = oa0 + ob0;
                        ov[e0 + 2 * j + 1] = oa1 + ob1;
                    }
                }
                set_o(db, qb, ov);
            }
        }
    }
};

// Epilogue of a piece of an item that the partition cut into pieces owned by consecutive
// workgroups.  The pieces are merged pairwise up a fixed binary tree; nobody waits for anybody.
//
// Pieces are numbered from the item's end: piece 0 is the one its owner works on at the very
// start of its range (the earliest to finish), piece p - 1 the one its owner reaches at the end of
// its range (the latest).  At the level with subtrees of `half` pieces, the node that starts at
// piece f (a multiple of 2 * half) joins subtree [f, f + half) with subtree [f + half, f + 2 *
// half) if the latter exists; a subtree without a sibling moves up unchanged.  Whoever carries a
// subtree's state arrives at the node through its arrival counter: the first of the two stores
// the state (in the partial-result slot of the subtree's first piece, whose earlier contents have
// been consumed by then) and leaves; the second merges the stored state into its own and carries
// the result up; at the root it writes the rows.  The carrier of the later half looks at the
// counter first and, if the other half is already there (the usual case), does not store at all.
// Every merge takes both operands in their stored (rounded) form and is commutative bit for bit
// (see merge_partial), and the tree is fixed, so the rows do not depend on the order of arrival.
// With the late pieces at the high end, the workgroup that reaches its piece last has the fewest
// merges left to do: the others have met lower in the tree, while they had time to spare.
//
// The counter of the node whose second subtree starts at piece r is the one indexed by the
// workgroup that owns piece r (r >= 1: those workgroups own the item's units but not its last
// ones, and no two items share such a workgroup).  Must be called by every thread of the
// workgroup; l_tot are whole-row sums; `flag` is one int of LDS.  Returns whether this workgroup
// wrote the rows.
template <int HD, int NB, int NW, bool HIDDEN>
DFX_D bool finish_cut_item(AttnState<HD, NB, NW, HIDDEN>& at, int rt, int64_t item_begin, int n_tiles, const WgSplit& split,
                           int partner, const float (&l_tot)[NB], int* flag, int64_t piece_begin = 0) {
    const KArgs& a = at.a;
    const int me = static_cast<int>(blockIdx.x);
    const int64_t item_last = item_begin + n_tiles - 1;
    // with fewer units than workgroups every workgroup owns one unit or none: each unit is a piece
    const bool sparse = split.q == 0;
    const int64_t total = split.q * split.n_wg + split.r;
    int wa, wb;
    owners_of_units(split, me, item_begin, item_last, wa, wb);
    // Pairing partition (partner >= 0): two pieces, the item's first tiles (piece 0, processed by the
    // partner of the item's owner at the very start of its work) and the rest (piece 1, the owner's);
    // both are the first thing their workgroup does, hence its first partial-result slot.
    const bool paired = partner >= 0;
    const bool my_piece_is_first = piece_begin == item_begin;
    const int p = paired ? 2 : (sparse ? n_tiles : wb - wa + 1);
    auto owner_of_piece = [&](int j) {
        if (paired) return (j == 0) == my_piece_is_first ? me : partner;
        return sparse ? wg_of_unit(item_last - j, total, split.n_wg) : wb - j;
    };
    auto slot_of_piece = [&](int j) {
        const int w = owner_of_piece(j);
        if (paired) return 2 * w;
        const int64_t ws = split.first(w);
        return partial_slot(w, ws > item_begin ? ws : item_begin, ws);
    };
    // the first piece of the subtree carried
    int j = paired ? (my_piece_is_first ? 0 : 1) : (sparse ? static_cast<int>(item_last - split.first(me)) : wb - me);
#pragma unroll
    for (int qb = 0; qb < NB; ++qb) at.l_run[qb] = l_tot[qb];

    for (int half = 1; half < p; half <<= 1) {
        const bool later_half = (j & half) != 0;
        const int second = (j & ~(2 * half - 1)) + half;  // first piece of the node's second subtree
        if (!later_half && second >= p) continue;         // no sibling at this level
        int* counter = a.arrivals + owner_of_piece(second);
        bool sibling_there = false;
        if (later_half) {
            if (threadIdx.x == 0) *flag = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            sibling_there = *flag == 1;
            __syncthreads();
        }
        if (!sibling_there) {
            at.store_partial(slot_of_piece(j), at.l_run);
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this thread's write-through stores have completed
            __syncthreads();
            if (threadIdx.x == 0) *flag = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            sibling_there = *flag == 1;
            __syncthreads();
            if (!sibling_there) return false;  // the sibling's carrier will find this state
        }
        const int other = slot_of_piece(later_half ? second - half : second);
        if constexpr (HIDDEN) {
            at.request_partial(other);
            at.round_to_stored_form();
            at.merge_requested_partial();
        } else {
            at.round_to_stored_form();
            at.merge_partial(other);
        }
        if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        j &= ~(2 * half - 1);
    }
    float l_all[NB];
#pragma unroll
    for (int qb = 0; qb < NB; ++qb) l_all[qb] = at.l_run[qb];
    at.store_output(rt, l_all);
    return true;
}

// Fused KV-cache store: fresh row t of k_new / v_new goes to cache slot store_slots[t] (what
// dfx_kv_store_unified does in a launch of its own).  The 16-byte chunks of all rows are dealt
// round-robin to the threads of the whole grid; every workgroup calls this once.  The slots
// written are outside every attended context (caller's contract), so nothing in this launch
// reads them.
// kBatch: chunks a thread has in flight (all loads of a batch are issued before its stores).  A kernel
// that leaves the compiler few registers takes 1: four chunks' addresses and data do not fit there,
// and data spilled to scratch makes two more trips to memory.
template <int HD, bool FP8, int kBatch = 4>
DFX_D void store_fresh_rows(const KArgs& a) {
    if (a.store_slots == nullptr) return;
    constexpr int kChunksPerHead = HD / 8;
    const int chunks_per_token = a.h_kv * kChunksPerHead;
    // (never beyond the rows k_new / v_new and the slot mapping have, whatever the offsets say)
    const int64_t n_rows = min(static_cast<int64_t>(a.cu_new[a.num_seqs]), a.n_new);
    const int64_t total = n_rows * chunks_per_token;
    const int64_t n_slots = a.n_pages * a.page_size;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    uint8_t* kc = const_cast<uint8_t*>(a.k_cache);
    uint8_t* vc = const_cast<uint8_t*>(a.v_cache);
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; base < total;
         base += stride * kBatch) {
        int64_t slot[kBatch], src_k[kBatch], src_v[kBatch], dst[kBatch];
        int head[kBatch];
        u32x4 k8[kBatch], v8[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int64_t idx = base + j * stride;
            slot[j] = -1;
            if (idx < total) {
                const int64_t t = idx / chunks_per_token;
                const int r = static_cast<int>(idx - t * chunks_per_token);
                const int h = r / kChunksPerHead, c = r - h * kChunksPerHead;
                head[j] = h;
                src_k[j] = t * a.kn_st + h * a.kn_sh + c * 8;
                src_v[j] = t * a.vn_st + h * a.vn_sh + c * 8;
                dst[j] = h * a.c_sh + c * 8;
                slot[j] = a.store_slots_i64 ? static_cast<const int64_t*>(a.store_slots)[t]
                                            : static_cast<int64_t>(static_cast<const int32_t*>(a.store_slots)[t]);
            }
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            if (slot[j] < 0 || slot[j] >= n_slots) {
                slot[j] = -1;
                continue;
            }
            k8[j] = *reinterpret_cast<const u32x4*>(a.k_new + src_k[j]);
            v8[j] = *reinterpret_cast<const u32x4*>(a.v_new + src_v[j]);
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            if (slot[j] < 0) continue;
            const int64_t page = a.page_shift >= 0 ? (slot[j] >> a.page_shift) : slot[j] / a.page_size;
            const int64_t d = page * a.c_sp + (slot[j] - page * a.page_size) * a.c_st + dst[j];  // elements
            if constexpr (FP8) {
                *reinterpret_cast<u32x2*>(kc + d) = quantise8(k8[j], a.k_scale[head[j]]);
                *reinterpret_cast<u32x2*>(vc + d) = quantise8(v8[j], a.v_scale[head[j]]);
            } else {
                *reinterpret_cast<u32x4*>(kc + d * 2) = k8[j];
                *reinterpret_cast<u32x4*>(vc + d * 2) = v8[j];
            }
        }
    }
}

// Exclusive prefix of units(s) into prefix[0..num_seqs]; also the per-head total, the number of
// items per KV head and the tile count of the longest item.
struct UnitSummary {
    int per_head;    // units per KV head
    int items;       // (sequence, row tile) items per KV head
    int max_tiles;   // KV tiles of the longest item
};

template <int RT>
DFX_D UnitSummary build_unit_prefix(const KArgs& a, int* prefix, int* scratch) {
    // scratch: [0, kMaxWaves) is used by the scan, [16, 16 + kMaxWaves) and [24, 24 + kMaxWaves) hold
    // per-wave item counts and tile maxima (register reductions; atomics on one LDS word from
    // every lane cost microseconds here)
    int carry = 0, items = 0, max_tiles = 0;
    const int n_threads = blockDim.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    for (int base = 0; base < a.num_seqs; base += n_threads) {
        const int sq = base + threadIdx.x;
        int u = 0, rows = 0, tiles = 0;
        if (sq < a.num_seqs) {
            const SeqShape shp = load_seq_shape(a, sq, RT);
            u = shp.units;
            if (u > 0) {
                rows = shp.n_row_tiles;
                tiles = shp.n_tiles;
            }
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            rows += __shfl_xor(rows, d);
            tiles = max(tiles, __shfl_xor(tiles, d));
        }
        if (lane == 0) {
            scratch[16 + wave] = rows;
            scratch[24 + wave] = tiles;
        }
        int tot;
        const int incl = block_inclusive_scan(u, scratch, tot);  // (its barriers also publish the two arrays)
        if (sq < a.num_seqs) prefix[sq + 1] = carry + incl;
        carry += tot;
        for (int w = 0; w < n_waves; ++w) {
            items += scratch[16 + w];
            max_tiles = max(max_tiles, scratch[24 + w]);
        }
        if (base + n_threads < a.num_seqs) __syncthreads();  // before the next round overwrites the arrays
    }
    if (threadIdx.x == 0) prefix[0] = 0;
    __syncthreads();
    UnitSummary r;
    r.per_head = carry;
    r.items = items;
    r.max_tiles = max_tiles;
    return r;
}

// The sequence whose unit range contains rem (0 <= rem < per-head total).
DFX_D int locate_sequence(const KArgs& a, const int* prefix, int* scratch, int rem) {
    for (int sq = threadIdx.x; sq < a.num_seqs; sq += blockDim.x)
        if (prefix[sq] <= rem && rem < prefix[sq + 1]) scratch[kMaxWaves] = sq;
    __syncthreads();
    const int r = scratch[kMaxWaves];
    __syncthreads();
    return r;
}

}  // namespace dfx
