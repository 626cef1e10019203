// Rotary position embedding of the fresh Q and K rows, optionally fused with the paged KV-cache
// store of the rotated K and of V (gfx950).
//
// Pure HBM-bandwidth work.  One lane owns the pair of 16-byte chunks (c, c + head_dim / 16) of
// one head row: the two halves a rotation mixes.  It reads both, the eight cosines and sines of
// its positions' angle table row, rotates in fp32 exactly as the reference does (two rounded
// products, one rounded sum, then round-to-nearest-even to bf16), writes both chunks back and,
// for K, also into the row's cache slot; V lanes only copy into the cache.  Consecutive lanes
// cover consecutive chunks, so a wavefront moves whole runs of a token row.  (A cache in the distinct layout is
// written by workgroups of their own, 16 tokens of a KV head each, through LDS: rope_store_distinct_kernel.)
#include "dfx_common.h"
#include "fp8_e4m3.h"
#include "distinct_tile.h"

namespace dfx {
namespace {

constexpr int kThreads = 256;

struct RopeArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* q_out;
    uint16_t* k_out;
    int64_t q_st, k_st, v_st, qo_st, ko_st;
    const float* table;  // [max_position, head_dim]: cosines, then sines
    int64_t max_position;
    int64_t n_tokens;
    int h_q, h_kv, hd;
    int v_heads;  // h_kv when V is stored, else 0
    void* k_cache;
    void* v_cache;
    int64_t n_slots;
    const float* k_scale;
    const float* v_scale;
    // distinct layout (bf16): K [pages, h_kv, hd / 8, page, 8], V [pages, h_kv, hd, page], strides in elements
    int distinct, page_size;
    int64_t kd[3], vd[3];
};

DFX_D u32x4 pack8(const float (&y)[8]) {
    u32x4 w;
    w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{y[0], y[1]}, bf16x2));
    w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{y[2], y[3]}, bf16x2));
    w.z = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{y[4], y[5]}, bf16x2));
    w.w = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{y[6], y[7]}, bf16x2));
    return w;
}

DFX_D void unpack8(u32x4 w, float (&x)[8]) {
    const uint32_t d[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[2 * i] = __builtin_bit_cast(float, d[i] << 16);
        x[2 * i + 1] = __builtin_bit_cast(float, d[i] & 0xffff0000u);
    }
}

// y1 = x1 * cos - x2 * sin, y2 = x2 * cos + x1 * sin, every product and sum rounded on its own
// (diffulex/layer/rotary_embedding.py:13-16 evaluates them as separate fp32 tensor operations).
DFX_D void rotate8(const float (&x1)[8], const float (&x2)[8], const float (&c)[8], const float (&s)[8],
                   float (&y1)[8], float (&y2)[8]) {
#pragma clang fp contract(off)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float a = x1[i] * c[i], b = x2[i] * s[i];
        const float d = x2[i] * c[i], e = x1[i] * s[i];
        y1[i] = a - b;
        y2[i] = d + e;
    }
}

// The chunk pair (lo, hi = lo + hd / 2) of the head row at `src` rotated by the angles of position `pos`.
template <typename PosT>
DFX_D void rotate_pair(const RopeArgs& a, const uint16_t* src, const PosT* __restrict__ positions, int64_t t, int lo, int hi,
                       u32x4& o1, u32x4& o2) {
    const u32x4 w1 = *reinterpret_cast<const u32x4*>(src + lo);
    const u32x4 w2 = *reinterpret_cast<const u32x4*>(src + hi);
    // a position outside the table is a caller error (the reference's gather would fail); it is
    // clamped here so that no lane reads outside the table
    int64_t pos = static_cast<int64_t>(positions[t]);
    pos = pos < 0 ? 0 : (pos >= a.max_position ? a.max_position - 1 : pos);
    const float* row = a.table + pos * a.hd;
    float cs[8], sn[8];
    *reinterpret_cast<f32x4*>(cs) = *reinterpret_cast<const f32x4*>(row + lo);
    *reinterpret_cast<f32x4*>(cs + 4) = *reinterpret_cast<const f32x4*>(row + lo + 4);
    *reinterpret_cast<f32x4*>(sn) = *reinterpret_cast<const f32x4*>(row + hi);
    *reinterpret_cast<f32x4*>(sn + 4) = *reinterpret_cast<const f32x4*>(row + hi + 4);
    float x1[8], x2[8], y1[8], y2[8];
    unpack8(w1, x1);
    unpack8(w2, x2);
    rotate8(x1, x2, cs, sn, y1, y2);
    o1 = pack8(y1);
    o2 = pack8(y2);
}

// One thread's work of the flat launch: work item idx of n_tokens * (h_q + h_kv + v_heads) * hd / 16.
template <bool FP8, typename PosT, typename SlotT>
DFX_D void rope_work_item(const RopeArgs& a, const PosT* __restrict__ positions, const SlotT* __restrict__ slots, int64_t idx) {
    const int cph = a.hd >> 4;  // chunk pairs per head row
    const int slots_per_token = (a.h_q + a.h_kv + a.v_heads) * cph;
    if (idx >= a.n_tokens * slots_per_token) return;
    const int64_t t = idx / slots_per_token;
    const int r = static_cast<int>(idx - t * slots_per_token);
    const int head = r / cph;  // q heads, then k heads, then v heads
    const int c = r - head * cph;
    const int lo = c * 8, hi = lo + (a.hd >> 1);

    int64_t slot = -1;
    if (slots != nullptr) {
        slot = static_cast<int64_t>(slots[t]);
        if (slot >= a.n_slots) slot = -1;
    }
    const int64_t cache_row = static_cast<int64_t>(a.h_kv) * a.hd;

    if (head >= a.h_q + a.h_kv) {  // V: cache copy only
        if (slot < 0) return;
        const int h = head - a.h_q - a.h_kv;
        const uint16_t* src = a.v + t * a.v_st + h * a.hd;
        const u32x4 w1 = *reinterpret_cast<const u32x4*>(src + lo);
        const u32x4 w2 = *reinterpret_cast<const u32x4*>(src + hi);
        const int64_t dst = slot * cache_row + h * a.hd;
        if constexpr (FP8) {
            uint8_t* vc = static_cast<uint8_t*>(a.v_cache) + dst;
            *reinterpret_cast<u32x2*>(vc + lo) = quantise8(w1, a.v_scale[h]);
            *reinterpret_cast<u32x2*>(vc + hi) = quantise8(w2, a.v_scale[h]);
        } else {
            uint16_t* vc = static_cast<uint16_t*>(a.v_cache) + dst;
            *reinterpret_cast<u32x4*>(vc + lo) = w1;
            *reinterpret_cast<u32x4*>(vc + hi) = w2;
        }
        return;
    }

    const bool is_k = head >= a.h_q;
    const int h = is_k ? head - a.h_q : head;
    const uint16_t* src = is_k ? a.k + t * a.k_st + h * a.hd : a.q + t * a.q_st + h * a.hd;
    uint16_t* dst = is_k ? a.k_out + t * a.ko_st + h * a.hd : a.q_out + t * a.qo_st + h * a.hd;
    u32x4 o1, o2;
    rotate_pair(a, src, positions, t, lo, hi, o1, o2);
    *reinterpret_cast<u32x4*>(dst + lo) = o1;
    *reinterpret_cast<u32x4*>(dst + hi) = o2;
    if (is_k && slot >= 0) {
        const int64_t off = slot * cache_row + h * a.hd;
        if constexpr (FP8) {
            uint8_t* kc = static_cast<uint8_t*>(a.k_cache) + off;
            *reinterpret_cast<u32x2*>(kc + lo) = quantise8(o1, a.k_scale[h]);
            *reinterpret_cast<u32x2*>(kc + hi) = quantise8(o2, a.k_scale[h]);
        } else {
            uint16_t* kc = static_cast<uint16_t*>(a.k_cache) + off;
            *reinterpret_cast<u32x4*>(kc + lo) = o1;
            *reinterpret_cast<u32x4*>(kc + hi) = o2;
        }
    }
}

template <bool FP8, typename PosT, typename SlotT>
__global__ void __launch_bounds__(kThreads)
rope_kv_store_kernel(const RopeArgs a, const PosT* __restrict__ positions, const SlotT* __restrict__ slots) {
    rope_work_item<FP8>(a, positions, slots, static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x);
}

// The same with the store going into a cache in the distinct layout (bf16).  The first q_blocks workgroups rotate
// the Q rows as above; each of the others takes 16 tokens of one KV head: rotates their K rows (k_out receives
// them as well), stages them and the V rows in LDS and writes both the way dfx_kv_store_distinct does
// (distinct_tile.h) -- one chunk at a time from the rotating threads, the V rows would leave two bytes at a time.
template <typename PosT, typename SlotT, int HD>
__global__ void __launch_bounds__(kThreads)
rope_store_distinct_kernel(const RopeArgs a, const PosT* __restrict__ positions, const SlotT* __restrict__ slots, int q_blocks) {
    using Tile = DistinctTile<HD>;
    __shared__ __attribute__((aligned(16))) uint8_t k_tile[Tile::K_BYTES];
    __shared__ __attribute__((aligned(16))) uint8_t v_tile[Tile::V_BYTES];
    __shared__ int64_t slot_of[Tile::kTokens];
    const int tid = threadIdx.x;
    if (static_cast<int>(blockIdx.x) < q_blocks) {
        RopeArgs q_only = a;
        q_only.h_kv = q_only.v_heads = 0;
        rope_work_item<false>(q_only, positions, static_cast<const SlotT*>(nullptr), static_cast<int64_t>(blockIdx.x) * kThreads + tid);
        return;
    }
    const int tile = static_cast<int>(blockIdx.x) - q_blocks;
    const int h = tile % a.h_kv;
    const int64_t t0 = static_cast<int64_t>(tile / a.h_kv) * Tile::kTokens;
    if (tid < Tile::kTokens) {
        const int64_t t = t0 + tid;
        int64_t slot = t < a.n_tokens ? static_cast<int64_t>(slots[t]) : -1;
        if (slot >= a.n_slots) slot = -1;
        slot_of[tid] = slot;
    }
    constexpr int cph = HD / 16;
    for (int w = tid; w < Tile::kTokens * cph; w += kThreads) {
        const int r = w / cph, c = w % cph;
        const int64_t t = t0 + r;
        u32x4 o1 = {0, 0, 0, 0}, o2 = {0, 0, 0, 0};
        if (t < a.n_tokens) {
            const int lo = c * 8, hi = lo + HD / 2;
            rotate_pair(a, a.k + t * a.k_st + h * HD, positions, t, lo, hi, o1, o2);
            uint16_t* dst = a.k_out + t * a.ko_st + h * HD;
            *reinterpret_cast<u32x4*>(dst + lo) = o1;
            *reinterpret_cast<u32x4*>(dst + hi) = o2;
        }
        *reinterpret_cast<u32x4*>(k_tile + Tile::k_offset(r, c)) = o1;
        *reinterpret_cast<u32x4*>(k_tile + Tile::k_offset(r, c + cph)) = o2;
    }
    for (int c = tid; c < Tile::kTokens * Tile::CPR; c += kThreads) {
        const int r = c / Tile::CPR, cc = c % Tile::CPR;
        const int64_t t = t0 + r;
        u32x4 vv = {0, 0, 0, 0};
        if (t < a.n_tokens) vv = *reinterpret_cast<const u32x4*>(a.v + t * a.v_st + h * HD + cc * 8);
        Tile::put_v(v_tile, r, cc, vv);
    }
    __syncthreads();
    Tile::store(k_tile, v_tile, slot_of, static_cast<uint16_t*>(a.k_cache), static_cast<uint16_t*>(a.v_cache), a.kd, a.vd, h,
                a.page_size, tid, kThreads);
}

template <typename PosT>
int launch_rope_distinct(const RopeArgs& a, const void* positions, const void* slots, int slot_type, hipStream_t st) {
    const int64_t q_work = a.n_tokens * a.h_q * (a.hd >> 4);
    const int64_t q_blocks = (q_work + kThreads - 1) / kThreads;
    const int64_t tiles = (a.n_tokens + DistinctTile<128>::kTokens - 1) / DistinctTile<128>::kTokens * a.h_kv;
    if (q_blocks + tiles > INT32_MAX) return DFX_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(q_blocks + tiles)), block(kThreads);
    const PosT* pos = static_cast<const PosT*>(positions);
#define DFX_ROPE_DISTINCT(SLOT_T, HD_)                                                                                   \
    hipLaunchKernelGGL((rope_store_distinct_kernel<PosT, SLOT_T, HD_>), grid, block, 0, st, a, pos,                      \
                       static_cast<const SLOT_T*>(slots), static_cast<int>(q_blocks))
    if (a.hd == 128) {
        if (slot_type == DFX_INDEX_I64) DFX_ROPE_DISTINCT(int64_t, 128);
        else DFX_ROPE_DISTINCT(int32_t, 128);
    } else {
        if (slot_type == DFX_INDEX_I64) DFX_ROPE_DISTINCT(int64_t, 64);
        else DFX_ROPE_DISTINCT(int32_t, 64);
    }
#undef DFX_ROPE_DISTINCT
    return launch_status();
}

template <bool FP8, typename PosT>
int launch_rope(const RopeArgs& a, const void* positions, const void* slots, int slot_type, hipStream_t st) {
    const int64_t work = a.n_tokens * (a.h_q + a.h_kv + a.v_heads) * (a.hd >> 4);
    const int64_t blocks = (work + kThreads - 1) / kThreads;
    if (blocks > INT32_MAX) return DFX_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
    const PosT* pos = static_cast<const PosT*>(positions);
    if (slot_type == DFX_INDEX_I64)
        hipLaunchKernelGGL((rope_kv_store_kernel<FP8, PosT, int64_t>), grid, block, 0, st, a, pos,
                           static_cast<const int64_t*>(slots));
    else
        hipLaunchKernelGGL((rope_kv_store_kernel<FP8, PosT, int32_t>), grid, block, 0, st, a, pos,
                           static_cast<const int32_t*>(slots));
    return launch_status();
}

}  // namespace
}  // namespace dfx

extern "C" int dfx_rope_kv_store(const dfx_rope_params* p, dfx_stream_t stream) {
    using namespace dfx;
    if (!p) return DFX_ERR_INVALID_ARG;
    if (p->n_tokens < 0 || p->num_q_heads < 0 || p->num_kv_heads < 0 || p->head_dim <= 0 || p->max_position <= 0)
        return DFX_ERR_INVALID_ARG;
    if (p->n_tokens == 0 || p->num_q_heads + p->num_kv_heads == 0) return DFX_OK;
    if (p->head_dim % 16 != 0) return DFX_ERR_UNSUPPORTED;
    if (!p->positions || !p->cos_sin_cache) return DFX_ERR_INVALID_ARG;
    if (p->position_index_type != DFX_INDEX_I32 && p->position_index_type != DFX_INDEX_I64) return DFX_ERR_INVALID_ARG;
    const bool store = p->slot_mapping != nullptr;
    const bool fp8 = p->kv_dtype == DFX_KV_FP8_E4M3;
    if (!fp8 && p->kv_dtype != DFX_KV_BF16) return DFX_ERR_INVALID_ARG;

    RopeArgs a{};
    a.q = static_cast<const uint16_t*>(p->q);
    a.k = static_cast<const uint16_t*>(p->k);
    a.v = static_cast<const uint16_t*>(p->v);
    a.q_out = static_cast<uint16_t*>(p->q_out);
    a.k_out = static_cast<uint16_t*>(p->k_out);
    a.q_st = p->q_stride_token;
    a.k_st = p->k_stride_token;
    a.v_st = p->v_stride_token;
    a.qo_st = p->q_out_stride_token;
    a.ko_st = p->k_out_stride_token;
    a.table = p->cos_sin_cache;
    a.max_position = p->max_position;
    a.n_tokens = p->n_tokens;
    a.h_q = p->num_q_heads;
    a.h_kv = p->num_kv_heads;
    a.hd = p->head_dim;
    const int64_t q_row = static_cast<int64_t>(a.h_q) * a.hd, kv_row = static_cast<int64_t>(a.h_kv) * a.hd;
    if (a.h_q > 0) {
        if (!a.q || !a.q_out || !aligned16(a.q) || !aligned16(a.q_out)) return DFX_ERR_INVALID_ARG;
        if (a.q_st < q_row || a.qo_st < q_row || a.q_st % 8 || a.qo_st % 8) return DFX_ERR_INVALID_ARG;
    }
    if (a.h_kv > 0) {
        if (!a.k || !a.k_out || !aligned16(a.k) || !aligned16(a.k_out)) return DFX_ERR_INVALID_ARG;
        if (a.k_st < kv_row || a.ko_st < kv_row || a.k_st % 8 || a.ko_st % 8) return DFX_ERR_INVALID_ARG;
    }
    if (!aligned16(a.table)) return DFX_ERR_INVALID_ARG;
    if (store) {
        if (a.h_kv == 0 || !a.v || !p->k_cache || !p->v_cache || p->n_slots < 0) return DFX_ERR_INVALID_ARG;
        if (!aligned16(a.v) || a.v_st < kv_row || a.v_st % 8) return DFX_ERR_INVALID_ARG;
        if (!aligned16(p->k_cache) || !aligned16(p->v_cache)) return DFX_ERR_INVALID_ARG;
        if (p->slot_index_type != DFX_INDEX_I32 && p->slot_index_type != DFX_INDEX_I64) return DFX_ERR_INVALID_ARG;
        if (fp8 != (p->k_scale != nullptr) || fp8 != (p->v_scale != nullptr)) return DFX_ERR_INVALID_ARG;
        if (p->cache_layout != DFX_CACHE_UNIFIED && p->cache_layout != DFX_CACHE_DISTINCT) return DFX_ERR_INVALID_ARG;
        if (p->cache_layout == DFX_CACHE_DISTINCT) {
            if (fp8 || (p->head_dim != 64 && p->head_dim != 128)) return DFX_ERR_UNSUPPORTED;
            if (p->page_size <= 0 || p->n_slots % p->page_size != 0) return DFX_ERR_INVALID_ARG;
            for (int i = 0; i < 3; ++i) {
                if (p->kc_stride[i] < 0 || p->kc_stride[i] % 8 || p->vc_stride[i] < 0) return DFX_ERR_INVALID_ARG;
                a.kd[i] = p->kc_stride[i];
                a.vd[i] = p->vc_stride[i];
            }
            a.distinct = 1;
            a.page_size = p->page_size;
        }
        a.v_heads = a.h_kv;
        a.k_cache = p->k_cache;
        a.v_cache = p->v_cache;
        a.n_slots = p->n_slots;
        a.k_scale = p->k_scale;
        a.v_scale = p->v_scale;
    } else if (p->k_cache || p->v_cache || p->k_scale || p->v_scale) {
        return DFX_ERR_INVALID_ARG;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a.distinct)
        return p->position_index_type == DFX_INDEX_I64
                   ? launch_rope_distinct<int64_t>(a, p->positions, p->slot_mapping, p->slot_index_type, st)
                   : launch_rope_distinct<int32_t>(a, p->positions, p->slot_mapping, p->slot_index_type, st);
    const bool q8 = store && fp8;
    if (p->position_index_type == DFX_INDEX_I64)
        return q8 ? launch_rope<true, int64_t>(a, p->positions, p->slot_mapping, p->slot_index_type, st)
                  : launch_rope<false, int64_t>(a, p->positions, p->slot_mapping, p->slot_index_type, st);
    return q8 ? launch_rope<true, int32_t>(a, p->positions, p->slot_mapping, p->slot_index_type, st)
              : launch_rope<false, int32_t>(a, p->positions, p->slot_mapping, p->slot_index_type, st);
}
