// Block-diffusion paged attention for gfx950 (MI355X), bf16 and FP8-E4M3 KV.
//
// One persistent workgroup (4 wavefronts) per compute unit walks an equal share of the
// linear work list described in partition.h.  For one (sequence, KV head, row tile) item
// the workgroup holds every query row that shares the KV head -- all G = H_q / H_kv heads
// of every query token, up to 128*NB rows -- so each K/V tile is fetched from HBM once
// per KV head and reused by the whole GQA group.
//
// Data flow per 64-token tile:
//   global --16-byte loads--> registers --> LDS  (K as [token][d], V transposed [d][token];
//                                                 FP8 codes are widened to bf16 here)
//   S^T = K Q^T   v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q kept in registers
//   online softmax on S^T: a query is one lane column, so row max / row sum are a
//                          register reduction plus one cross-half shuffle
//   O^T += V^T P^T   the S^T accumulators, rounded to bf16, are already in the B-operand
//                    layout; V^T rows come from LDS in the matching token order
//
// MFMA 32x32x16 register layouts relied upon (lane l, h = l / 32):
//   A: row l % 32, contraction elements 8h .. 8h+7        B: column l % 32, same elements
//   C/D: column l % 32, rows 8*i + 4*h + j for accumulator index 4*i + j
#include "dfx_common.h"
#include "partition.h"

namespace dfx {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kMaxSeqs = 4095;
constexpr float kLog2e = 1.4426950408889634f;

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
    float* workspace;
    int64_t q_st, q_sh, kn_st, kn_sh, vn_st, vn_sh, o_st, o_sh;
    int64_t c_sp, c_st, c_sh;  // cache strides in elements: page, token, head
    int64_t bt_stride, n_pages;
    int num_seqs, h_kv, group, page_size, page_shift, max_pages, dbs, mask_mode, n_wg;
    float c;  // scale * log2(e)
};

template <int HD, int NB>
struct Cfg {
    static constexpr int TN = kTileTokens;
    static constexpr int RT = 32 * NB * kWaves;     // query rows per row tile
    static constexpr int NSLAB = HD / 16;           // contraction slabs of Q K^T
    static constexpr int NDB = HD / 32;             // 32-row blocks of O^T
    static constexpr int KSTRIDE = HD * 2 + 16;     // bytes per K row in LDS (16-byte skew)
    static constexpr int VSTRIDE = TN * 2 + 16;     // bytes per V^T row in LDS
    static constexpr int K_BYTES = TN * KSTRIDE;
    static constexpr int V_BYTES = HD * VSTRIDE;
    static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
    static constexpr int PREFIX_BYTES = (kMaxSeqs + 1) * 4;
    static constexpr int MISC_BYTES = 64;
    static constexpr int LDS_BYTES = PREFIX_BYTES + MISC_BYTES + 2 * STAGE_BYTES;
    static constexpr int CH16 = TN * HD * 2 / 16 / kThreads;   // 16-byte chunks per lane, bf16 tile
    static constexpr int CH8 = TN * HD / 16 / kThreads;        // 16-byte chunks per lane, fp8 tile
    static constexpr int O_VEC4 = NB * NDB * 4;                // float4 per lane in a partial
    static constexpr int SLOT_FLOATS = kThreads * (O_VEC4 * 4 + 2 * NB);
};

DFX_D float wave_xor32_max(float x) { return fmaxf(x, __shfl_xor(x, 32)); }

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
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        const int t = scratch[w];
        if (w < wave) off += t;
        tot += t;
    }
    __syncthreads();
    block_total = tot;
    return x + off;
}

DFX_D SeqShape load_seq_shape(const KArgs& a, int s, int rows_per_tile) {
    const int ctx = (a.context_lens != nullptr && a.k_cache != nullptr) ? a.context_lens[s] : 0;
    const int q_len = a.cu_q[s + 1] - a.cu_q[s];
    const int new_len = a.cu_new[s + 1] - a.cu_new[s];
    return make_seq_shape(ctx, q_len, new_len, a.group, rows_per_tile);
}

// Two e4m3 codes (bytes 0,1 or 2,3 of w) -> two bf16 packed in a dword.  The widening is
// exact: an e4m3 value has 3 mantissa bits, so the upper half of its fp32 form is its bf16 form.
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
struct Attn {
    using C = Cfg<HD, NB>;

    const KArgs& a;
    uint8_t* lds;
    int* prefix;   // exclusive prefix of units over sequences, [num_seqs + 1]
    int* misc;
    const int tid, lane, wave, col, half;

    // per-segment state
    SeqShape sh;
    int s, kvh, q0, n0;
    bf16x8 qf[NB][C::NSLAB];
    f32x16 o[C::NDB][NB];
    float m_run[NB], l_run[NB];
    int vis_limit[NB];
    // staged tile (registers)
    u32x4 kst[C::CH16], vst[C::CH16];
    bool staged_fp8;

    DFX_D Attn(const KArgs& args, uint8_t* smem)
        : a(args), lds(smem), prefix(reinterpret_cast<int*>(smem)),
          misc(reinterpret_cast<int*>(smem + C::PREFIX_BYTES)), tid(threadIdx.x), lane(threadIdx.x & 63),
          wave(threadIdx.x >> 6), col(threadIdx.x & 31), half((threadIdx.x >> 5) & 1) {}

    DFX_D uint8_t* k_stage(int b) const { return lds + C::PREFIX_BYTES + C::MISC_BYTES + b * C::STAGE_BYTES; }
    DFX_D uint8_t* v_stage(int b) const { return k_stage(b) + C::K_BYTES; }

    // ---- global -> registers -------------------------------------------------------------
    DFX_D int64_t cache_row_offset(int tok, bool& ok) const {
        const int p = a.page_shift >= 0 ? (tok >> a.page_shift) : (tok / a.page_size);
        const int off = tok - p * a.page_size;
        int64_t page = -1;
        if (p < a.max_pages) page = a.block_tables[static_cast<int64_t>(s) * a.bt_stride + p];
        ok = ok && page >= 0 && page < a.n_pages;
        return page * a.c_sp + off * a.c_st + kvh * a.c_sh;
    }

    DFX_D void issue(int tile) {
        const bool is_ctx = tile < sh.n_ctx_tiles;
        const int base = (is_ctx ? tile : tile - sh.n_ctx_tiles) * C::TN;
        const int limit = is_ctx ? sh.ctx : sh.new_len;
        if (FP8 && is_ctx) {
            staged_fp8 = true;
            constexpr int CPR = HD / 16;  // chunks per row
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

    // ---- registers -> LDS ----------------------------------------------------------------
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

    // ---- one tile of attention from LDS ---------------------------------------------------
    DFX_D void compute(int buf, int tile) {
        const bool is_ctx = tile < sh.n_ctx_tiles;
        const int base = (is_ctx ? tile : tile - sh.n_ctx_tiles) * C::TN;
        const int limit = is_ctx ? sh.ctx : sh.new_len;
        float c_tile = a.c, v_mul = 1.0f;
        if (FP8 && is_ctx) {
            c_tile = fmaxf(a.c * a.k_scale[kvh], 1e-30f);
            v_mul = a.v_scale[kvh];
        }
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

        const bool mask_valid = base + C::TN > limit;
        const bool mask_bc = !is_ctx && a.mask_mode == DFX_MASK_BLOCK_CAUSAL;
        if (mask_valid || mask_bc) {
#pragma unroll
            for (int qb = 0; qb < NB; ++qb) {
                int lim = limit;
                if (mask_bc) lim = min(lim, vis_limit[qb]);
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int tok = base + tb * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
                        if (tok >= lim) sc[tb][qb][e] = -INFINITY;
                    }
            }
        }

        bf16x8 pb[NB][2][2];
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            float mx = -INFINITY;
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[tb][qb][e]);
            mx = wave_xor32_max(mx);
            const float m_new = fmaxf(m_run[qb], mx * c_tile);
            if (__any(m_new > m_run[qb])) {
                const float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_run[qb] - m_new);
                l_run[qb] *= alpha;
#pragma unroll
                for (int db = 0; db < C::NDB; ++db)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[db][qb][e] *= alpha;
                m_run[qb] = m_new;
            }
            const float m_safe = (m_run[qb] == -INFINITY) ? 0.0f : m_run[qb];
            float lsum = 0.0f;
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) {
                float p[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    p[e] = fast_exp2(__builtin_fmaf(sc[tb][qb][e], c_tile, -m_safe));
                    lsum += p[e];
                    if (FP8) p[e] *= v_mul;
                }
#pragma unroll
                for (int sl = 0; sl < 2; ++sl) {
                    bf16x8 v;
#pragma unroll
                    for (int e = 0; e < 8; e += 2) {
                        const bf16x2 t = __builtin_convertvector(f32x2{p[sl * 8 + e], p[sl * 8 + e + 1]}, bf16x2);
                        v[e] = t.x;
                        v[e + 1] = t.y;
                    }
                    pb[qb][tb][sl] = v;
                }
            }
            l_run[qb] += lsum;
        }

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

    // ---- segment prologue / epilogue ------------------------------------------------------
    DFX_D int row_of(int rt, int qb) const { return rt * C::RT + wave * (32 * NB) + qb * 32 + col; }

    DFX_D void load_queries(int rt) {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            const int r = row_of(rt, qb);
            const bool valid = r < a.group * sh.q_len;
            const int g = valid ? r / sh.q_len : 0;
            const int i = valid ? r - g * sh.q_len : 0;
            vis_limit[qb] = (i / a.dbs + 1) * a.dbs;
            const uint16_t* qp = a.q + (q0 + i) * a.q_st + (kvh * a.group + g) * a.q_sh + half * 8;
#pragma unroll
            for (int slab = 0; slab < C::NSLAB; ++slab) {
                u32x4 v = {0, 0, 0, 0};
                if (valid) v = *reinterpret_cast<const u32x4*>(qp + slab * 16);
                qf[qb][slab] = __builtin_bit_cast(bf16x8, v);
            }
            m_run[qb] = -INFINITY;
            l_run[qb] = 0.0f;
#pragma unroll
            for (int db = 0; db < C::NDB; ++db)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[db][qb][e] = 0.0f;
        }
    }

    // Write normalised rows: accumulator 4*i + j of block db is element d = 32*db + 8*i + 4*half + j.
    DFX_D void store_output(int rt, const float (&l_tot)[NB]) const {
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            const int r = row_of(rt, qb);
            if (r >= a.group * sh.q_len) continue;
            const int g = r / sh.q_len;
            const int i = r - g * sh.q_len;
            const float inv = 1.0f / l_tot[qb];
            uint16_t* op = a.out + (q0 + i) * a.o_st + (kvh * a.group + g) * a.o_sh + half * 4;
#pragma unroll
            for (int db = 0; db < C::NDB; ++db)
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    const bf16x2 lo = __builtin_convertvector(
                        f32x2{o[db][qb][ii * 4 + 0] * inv, o[db][qb][ii * 4 + 1] * inv}, bf16x2);
                    const bf16x2 hi = __builtin_convertvector(
                        f32x2{o[db][qb][ii * 4 + 2] * inv, o[db][qb][ii * 4 + 3] * inv}, bf16x2);
                    u32x2 w;
                    w.x = __builtin_bit_cast(uint32_t, lo);
                    w.y = __builtin_bit_cast(uint32_t, hi);
                    *reinterpret_cast<u32x2*>(op + db * 32 + ii * 8) = w;
                }
        }
    }

    DFX_D float* slot_ptr(int slot) const { return a.workspace + static_cast<int64_t>(slot) * C::SLOT_FLOATS; }

    DFX_D void store_partial(int slot, const float (&l_tot)[NB]) const {
        float* sp = slot_ptr(slot);
        f32x4* ov = reinterpret_cast<f32x4*>(sp);
#pragma unroll
        for (int qb = 0; qb < NB; ++qb)
#pragma unroll
            for (int db = 0; db < C::NDB; ++db)
#pragma unroll
                for (int ii = 0; ii < 4; ++ii)
                    ov[((qb * C::NDB + db) * 4 + ii) * kThreads + tid] =
                        f32x4{o[db][qb][ii * 4 + 0], o[db][qb][ii * 4 + 1], o[db][qb][ii * 4 + 2],
                              o[db][qb][ii * 4 + 3]};
        float* ml = sp + C::O_VEC4 * 4 * kThreads;
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            ml[qb * kThreads + tid] = m_run[qb];
            ml[(NB + qb) * kThreads + tid] = l_tot[qb];
        }
    }

    // Merge one stored partial into the running state (m_run, l_run hold totals here).
    DFX_D void merge_partial(int slot) {
        const float* sp = slot_ptr(slot);
        const f32x4* ov = reinterpret_cast<const f32x4*>(sp);
        const float* ml = sp + C::O_VEC4 * 4 * kThreads;
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            const float mp = ml[qb * kThreads + tid];
            const float lp = ml[(NB + qb) * kThreads + tid];
            const float mn = fmaxf(m_run[qb], mp);
            const float wa = (m_run[qb] == -INFINITY) ? 0.0f : fast_exp2(m_run[qb] - mn);
            const float wb = (mp == -INFINITY) ? 0.0f : fast_exp2(mp - mn);
            l_run[qb] = l_run[qb] * wa + lp * wb;
            m_run[qb] = mn;
#pragma unroll
            for (int db = 0; db < C::NDB; ++db)
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    const f32x4 v = ov[((qb * C::NDB + db) * 4 + ii) * kThreads + tid];
#pragma unroll
                    for (int j = 0; j < 4; ++j) o[db][qb][ii * 4 + j] = o[db][qb][ii * 4 + j] * wa + v[j] * wb;
                }
        }
    }

    DFX_D void set_sequence(int seq, int kv_head) {
        s = seq;
        kvh = kv_head;
        sh = load_seq_shape(a, s, C::RT);
        q0 = a.cu_q[s];
        n0 = a.cu_new[s];
    }

    DFX_D void run_segment(int rt, int tile0, int tile1, bool complete, int slot) {
        load_queries(rt);
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
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) l_tot[qb] = l_run[qb] + __shfl_xor(l_run[qb], 32);
        if (complete) store_output(rt, l_tot);
        else store_partial(slot, l_tot);
    }

    // Fill prefix[] with the exclusive prefix of units(s); returns the per-head total.
    DFX_D int build_prefix() {
        int carry = 0;
        for (int base = 0; base < a.num_seqs; base += kThreads) {
            const int sq = base + tid;
            const int u = sq < a.num_seqs ? load_seq_shape(a, sq, C::RT).units : 0;
            int tot;
            const int incl = block_inclusive_scan(u, misc, tot);
            if (sq < a.num_seqs) prefix[sq + 1] = carry + incl;
            carry += tot;
        }
        if (tid == 0) prefix[0] = 0;
        __syncthreads();
        return carry;
    }

    // The sequence whose unit range contains rem (0 <= rem < per-head total).
    DFX_D int locate(int rem) {
        for (int sq = tid; sq < a.num_seqs; sq += kThreads)
            if (prefix[sq] <= rem && rem < prefix[sq + 1]) misc[8] = sq;
        __syncthreads();
        const int r = misc[8];
        __syncthreads();
        return r;
    }
};

template <int HD, int NB, bool FP8>
__global__ void __launch_bounds__(kThreads) paged_attn_kernel(const KArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    Attn<HD, NB, FP8> at(a, smem);
    const int per_head = at.build_prefix();
    const int64_t total = static_cast<int64_t>(per_head) * a.h_kv;
    if (total == 0) return;
    const int w = blockIdx.x;
    const int64_t begin = wg_first_unit(w, total, a.n_wg);
    const int64_t end = wg_first_unit(w + 1, total, a.n_wg);
    if (begin >= end) return;

    int kvh = static_cast<int>(begin / per_head);
    const int rem = static_cast<int>(begin - static_cast<int64_t>(kvh) * per_head);
    int s = at.locate(rem);
    int u = rem - at.prefix[s];
    int64_t pos = begin;
    while (pos < end) {
        at.set_sequence(s, kvh);
        const int n_tiles = at.sh.n_tiles;
        const int rt = u / n_tiles;
        const int tile0 = u - rt * n_tiles;
        const int64_t seg_end = min(pos + (n_tiles - tile0), end);
        const int tile1 = tile0 + static_cast<int>(seg_end - pos);
        const bool complete = tile0 == 0 && tile1 == n_tiles;
        at.run_segment(rt, tile0, tile1, complete, partial_slot(w, pos, begin));
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

// One workgroup per (row tile, sequence, KV head): if the item was cut by the partition,
// merge its pieces and write the rows; otherwise the main kernel has already written them.
template <int HD, int NB>
__global__ void __launch_bounds__(kThreads) paged_attn_combine_kernel(const KArgs a) {
    __shared__ int scan_scratch[kWaves];
    Attn<HD, NB, false> at(a, nullptr);  // no LDS stages here: only the register state and the epilogue
    using C = Cfg<HD, NB>;
    const int rt = blockIdx.x, s = blockIdx.y, kvh = blockIdx.z;
    // units before sequence s and per-head total, by a strided block reduction
    int before = 0, all = 0;
    for (int sq = threadIdx.x; sq < a.num_seqs; sq += kThreads) {
        const int u = load_seq_shape(a, sq, C::RT).units;
        all += u;
        if (sq < s) before += u;
    }
    int tot_all, tot_before;
    block_inclusive_scan(all, scan_scratch, tot_all);
    block_inclusive_scan(before, scan_scratch, tot_before);
    at.set_sequence(s, kvh);
    if (rt >= at.sh.n_row_tiles || at.sh.n_tiles == 0) return;
    const int64_t total = static_cast<int64_t>(tot_all) * a.h_kv;
    const int64_t item_begin = static_cast<int64_t>(kvh) * tot_all + tot_before + static_cast<int64_t>(rt) * at.sh.n_tiles;
    const int64_t item_end = item_begin + at.sh.n_tiles;
    const int wa = wg_of_unit(item_begin, total, a.n_wg);
    const int wb = wg_of_unit(item_end - 1, total, a.n_wg);
    if (wa == wb) return;
#pragma unroll
    for (int qb = 0; qb < NB; ++qb) {
        at.m_run[qb] = -INFINITY;
        at.l_run[qb] = 0.0f;
#pragma unroll
        for (int db = 0; db < C::NDB; ++db)
#pragma unroll
            for (int e = 0; e < 16; ++e) at.o[db][qb][e] = 0.0f;
    }
    for (int w = wa; w <= wb; ++w) {
        const int64_t ws = wg_first_unit(w, total, a.n_wg);
        const int64_t we = wg_first_unit(w + 1, total, a.n_wg);
        if (ws >= we) continue;
        const int64_t pb = ws > item_begin ? ws : item_begin;
        at.merge_partial(partial_slot(w, pb, ws));
    }
    float l_tot[NB];
#pragma unroll
    for (int qb = 0; qb < NB; ++qb) l_tot[qb] = at.l_run[qb];
    at.store_output(rt, l_tot);
}


struct Plan {
    int hd, nb, n_wg;
    bool fp8;
    int64_t slot_floats;
    int lds_bytes;
};

int device_cu_count() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return -1;
        cached[dev] = n;
    }
    return cached[dev];
}

int make_plan(const dfx_attn_params* p, Plan& plan) {
    if (p == nullptr) return DFX_ERR_INVALID_ARG;
    if (p->num_seqs < 0 || p->num_q_heads <= 0 || p->num_kv_heads <= 0 || p->head_dim <= 0 || p->max_seqlen_q < 0 ||
        p->max_workgroups < 0)
        return DFX_ERR_INVALID_ARG;
    if (p->num_q_heads % p->num_kv_heads != 0) return DFX_ERR_INVALID_ARG;
    if (p->head_dim != 64 && p->head_dim != 128) return DFX_ERR_UNSUPPORTED;
    if (p->num_seqs > kMaxSeqs) return DFX_ERR_UNSUPPORTED;
    if (p->kv_dtype != DFX_KV_BF16 && p->kv_dtype != DFX_KV_FP8_E4M3) return DFX_ERR_INVALID_ARG;
    const int64_t rows = static_cast<int64_t>(p->num_q_heads / p->num_kv_heads) * p->max_seqlen_q;
    plan.hd = p->head_dim;
    plan.nb = rows <= 32 * kWaves ? 1 : 2;
    plan.fp8 = p->kv_dtype == DFX_KV_FP8_E4M3 && p->k_cache != nullptr;
    if (p->max_workgroups > 0) {
        plan.n_wg = p->max_workgroups;
    } else {
        plan.n_wg = device_cu_count();
        if (plan.n_wg <= 0) return DFX_ERR_LAUNCH;
    }
    if (plan.n_wg > 65535) return DFX_ERR_INVALID_ARG;
    if (plan.hd == 64) {
        plan.slot_floats = plan.nb == 1 ? Cfg<64, 1>::SLOT_FLOATS : Cfg<64, 2>::SLOT_FLOATS;
        plan.lds_bytes = Cfg<64, 1>::LDS_BYTES;
    } else {
        plan.slot_floats = plan.nb == 1 ? Cfg<128, 1>::SLOT_FLOATS : Cfg<128, 2>::SLOT_FLOATS;
        plan.lds_bytes = Cfg<128, 1>::LDS_BYTES;
    }
    return DFX_OK;
}

int64_t plan_workspace_bytes(const Plan& plan) { return 2 * static_cast<int64_t>(plan.n_wg) * plan.slot_floats * 4; }

template <int HD, int NB, bool FP8>
int launch(const KArgs& ka, const Plan& plan, int rt_max, hipStream_t st) {
    auto main_k = paged_attn_kernel<HD, NB, FP8>;
    auto comb_k = paged_attn_combine_kernel<HD, NB>;
    constexpr int lds = Cfg<HD, NB>::LDS_BYTES;
    static bool configured = false;  // raising the dynamic LDS limit is idempotent
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(main_k), hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds) != hipSuccess)
            return DFX_ERR_LAUNCH;
        configured = true;
    }
    hipLaunchKernelGGL(main_k, dim3(plan.n_wg), dim3(kThreads), lds, st, ka);
    if (hipGetLastError() != hipSuccess) return DFX_ERR_LAUNCH;
    if (plan.n_wg > 1 && rt_max > 0) {
        hipLaunchKernelGGL(comb_k, dim3(rt_max, ka.num_seqs, ka.h_kv), dim3(kThreads), 0, st, ka);
        if (hipGetLastError() != hipSuccess) return DFX_ERR_LAUNCH;
    }
    return DFX_OK;
}

}  // namespace
}  // namespace dfx

using namespace dfx;

extern "C" int64_t dfx_paged_attn_workspace_bytes(const dfx_attn_params* p) {
    Plan plan;
    const int rc = make_plan(p, plan);
    if (rc != DFX_OK) return rc;
    return plan_workspace_bytes(plan);
}

extern "C" int dfx_paged_attn(const dfx_attn_params* p, dfx_stream_t stream) {
    Plan plan;
    const int rc = make_plan(p, plan);
    if (rc != DFX_OK) return rc;
    if (p->num_seqs == 0 || p->max_seqlen_q == 0) return DFX_OK;
    if (!p->q || !p->k_new || !p->v_new || !p->out || !p->cu_seqlens_q || !p->cu_seqlens_new)
        return DFX_ERR_INVALID_ARG;
    const bool has_cache = p->k_cache != nullptr;
    if (has_cache != (p->v_cache != nullptr)) return DFX_ERR_INVALID_ARG;
    if (has_cache && (!p->block_tables || p->page_size <= 0 || p->max_pages_per_seq < 0 || p->n_pages < 0))
        return DFX_ERR_INVALID_ARG;
    if (plan.fp8 && (!p->k_scale || !p->v_scale)) return DFX_ERR_INVALID_ARG;
    if (!(p->scale > 0.0f) || p->diffusion_block_size <= 0) return DFX_ERR_INVALID_ARG;
    if (p->mask_mode != DFX_MASK_FULL && p->mask_mode != DFX_MASK_BLOCK_CAUSAL) return DFX_ERR_INVALID_ARG;
    const int64_t strides8[] = {p->q_stride_token,  p->q_stride_head,   p->kn_stride_token, p->kn_stride_head,
                                p->vn_stride_token, p->vn_stride_head};
    for (int64_t v : strides8)
        if (v < 0 || v % 8 != 0) return DFX_ERR_INVALID_ARG;
    if (p->o_stride_token % 4 != 0 || p->o_stride_head % 4 != 0) return DFX_ERR_INVALID_ARG;
    if (!aligned16(p->q) || !aligned16(p->k_new) || !aligned16(p->v_new) || !aligned16(p->out))
        return DFX_ERR_INVALID_ARG;
    if (has_cache) {
        const int64_t gran = plan.fp8 ? 16 : 8;
        if (p->cache_stride_page % gran || p->cache_stride_token % gran || p->cache_stride_head % gran)
            return DFX_ERR_INVALID_ARG;
        if (!aligned16(p->k_cache) || !aligned16(p->v_cache)) return DFX_ERR_INVALID_ARG;
    }
    const int64_t need = plan_workspace_bytes(plan);
    if (plan.n_wg > 1 && (p->workspace == nullptr || p->workspace_bytes < need || !aligned16(p->workspace)))
        return DFX_ERR_WORKSPACE;

    KArgs ka;
    ka.q = static_cast<const uint16_t*>(p->q);
    ka.k_new = static_cast<const uint16_t*>(p->k_new);
    ka.v_new = static_cast<const uint16_t*>(p->v_new);
    ka.k_cache = static_cast<const uint8_t*>(p->k_cache);
    ka.v_cache = static_cast<const uint8_t*>(p->v_cache);
    ka.out = static_cast<uint16_t*>(p->out);
    ka.block_tables = p->block_tables;
    ka.context_lens = p->context_lens;
    ka.cu_q = p->cu_seqlens_q;
    ka.cu_new = p->cu_seqlens_new;
    ka.k_scale = p->k_scale;
    ka.v_scale = p->v_scale;
    ka.workspace = static_cast<float*>(p->workspace);
    ka.q_st = p->q_stride_token;
    ka.q_sh = p->q_stride_head;
    ka.kn_st = p->kn_stride_token;
    ka.kn_sh = p->kn_stride_head;
    ka.vn_st = p->vn_stride_token;
    ka.vn_sh = p->vn_stride_head;
    ka.o_st = p->o_stride_token;
    ka.o_sh = p->o_stride_head;
    ka.c_sp = p->cache_stride_page;
    ka.c_st = p->cache_stride_token;
    ka.c_sh = p->cache_stride_head;
    ka.bt_stride = p->block_table_stride;
    ka.n_pages = p->n_pages;
    ka.num_seqs = p->num_seqs;
    ka.h_kv = p->num_kv_heads;
    ka.group = p->num_q_heads / p->num_kv_heads;
    ka.page_size = has_cache ? p->page_size : 1;
    ka.page_shift = -1;
    if ((ka.page_size & (ka.page_size - 1)) == 0) {
        ka.page_shift = 0;
        while ((1 << ka.page_shift) < ka.page_size) ++ka.page_shift;
    }
    ka.max_pages = p->max_pages_per_seq;
    ka.dbs = p->diffusion_block_size;
    ka.mask_mode = p->mask_mode;
    ka.n_wg = plan.n_wg;
    ka.c = p->scale * kLog2e;

    const int rows_per_tile = 32 * plan.nb * kWaves;
    const int64_t rows = static_cast<int64_t>(ka.group) * p->max_seqlen_q;
    const int64_t rt_max = (rows + rows_per_tile - 1) / rows_per_tile;
    if (rt_max > 65535) return DFX_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int rtm = static_cast<int>(rt_max);
#define DFX_ATTN_CASE(HD_, NB_)                                                     \
    if (plan.hd == HD_ && plan.nb == NB_)                                           \
        return plan.fp8 ? launch<HD_, NB_, true>(ka, plan, rtm, st) : launch<HD_, NB_, false>(ka, plan, rtm, st);
    DFX_ATTN_CASE(64, 1)
    DFX_ATTN_CASE(64, 2)
    DFX_ATTN_CASE(128, 1)
    DFX_ATTN_CASE(128, 2)
#undef DFX_ATTN_CASE
    return DFX_ERR_UNSUPPORTED;
}
