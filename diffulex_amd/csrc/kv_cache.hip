// Paged KV-cache store (slot_mapping scatter) and load (block_table gather) for gfx950.
//
// All three are pure HBM-bandwidth kernels: every lane moves one 16-byte chunk of K
// and one of V per step, consecutive lanes cover consecutive chunks of a token row, so
// a wavefront reads and writes whole 1 KiB runs.  The FP8 variants quantise in
// registers between the load and the (half-width) store.
#include "dfx_common.h"
#include "fp8_e4m3.h"
#include "distinct_tile.h"

namespace dfx {
namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------- store, unified layout
// One lane per 8-element chunk of a token row (K and V both).
template <bool FP8, typename SlotT>
__global__ void __launch_bounds__(kThreads)
kv_store_unified_vec8(const uint16_t* __restrict__ key, const uint16_t* __restrict__ value, int64_t key_stride,
                      int64_t value_stride, void* __restrict__ k_cache, void* __restrict__ v_cache,
                      const SlotT* __restrict__ slots, int64_t n_tokens, int64_t n_slots, int row_elems,
                      int head_dim, const float* __restrict__ k_scale, const float* __restrict__ v_scale) {
    const int chunks_per_row = row_elems >> 3;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (idx >= n_tokens * chunks_per_row) return;
    const int64_t t = idx / chunks_per_row;
    const int c = static_cast<int>(idx - t * chunks_per_row);
    const int64_t slot = static_cast<int64_t>(slots[t]);
    if (slot < 0 || slot >= n_slots) return;
    const u32x4 k8 = *reinterpret_cast<const u32x4*>(key + t * key_stride + c * 8);
    const u32x4 v8 = *reinterpret_cast<const u32x4*>(value + t * value_stride + c * 8);
    const int64_t dst = slot * row_elems + c * 8;
    if constexpr (FP8) {
        const int head = (c * 8) / head_dim;
        *reinterpret_cast<u32x2*>(static_cast<uint8_t*>(k_cache) + dst) = quantise8(k8, k_scale[head]);
        *reinterpret_cast<u32x2*>(static_cast<uint8_t*>(v_cache) + dst) = quantise8(v8, v_scale[head]);
    } else {
        *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(k_cache) + dst) = k8;
        *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(v_cache) + dst) = v8;
    }
}

// Element-wise fallback for rows that are not 16-byte friendly.
template <bool FP8, typename SlotT>
__global__ void __launch_bounds__(kThreads)
kv_store_unified_scalar(const uint16_t* __restrict__ key, const uint16_t* __restrict__ value, int64_t key_stride,
                        int64_t value_stride, void* __restrict__ k_cache, void* __restrict__ v_cache,
                        const SlotT* __restrict__ slots, int64_t n_tokens, int64_t n_slots, int row_elems,
                        int head_dim, const float* __restrict__ k_scale, const float* __restrict__ v_scale) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (idx >= n_tokens * row_elems) return;
    const int64_t t = idx / row_elems;
    const int e = static_cast<int>(idx - t * row_elems);
    const int64_t slot = static_cast<int64_t>(slots[t]);
    if (slot < 0 || slot >= n_slots) return;
    const uint16_t kb = key[t * key_stride + e];
    const uint16_t vb = value[t * value_stride + e];
    const int64_t dst = slot * row_elems + e;
    if constexpr (FP8) {
        const int head = e / head_dim;
        static_cast<uint8_t*>(k_cache)[dst] = quantise_e4m3(bf16_bits_to_f32(kb), k_scale[head]);
        static_cast<uint8_t*>(v_cache)[dst] = quantise_e4m3(bf16_bits_to_f32(vb), v_scale[head]);
    } else {
        static_cast<uint16_t*>(k_cache)[dst] = kb;
        static_cast<uint16_t*>(v_cache)[dst] = vb;
    }
}

// ---------------------------------------------------------------- store, distinct layout
struct DistinctStrides {
    int64_t k[5];
    int64_t v[4];
};

template <typename SlotT>
__global__ void __launch_bounds__(kThreads)
kv_store_distinct_kernel(const uint16_t* __restrict__ key, const uint16_t* __restrict__ value, int64_t key_stride,
                         int64_t value_stride, uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
                         DistinctStrides st, const SlotT* __restrict__ slots, int64_t n_tokens, int64_t n_pages,
                         int page_size, int x, int row_elems, int head_dim) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (idx >= n_tokens * row_elems) return;
    const int64_t t = idx / row_elems;
    const int e = static_cast<int>(idx - t * row_elems);
    const int64_t slot = static_cast<int64_t>(slots[t]);
    if (slot < 0) return;
    const int64_t blk = slot / page_size;
    const int64_t off = slot - blk * page_size;
    if (blk >= n_pages) return;
    const int h = e / head_dim;
    const int d = e - h * head_dim;
    k_cache[blk * st.k[0] + h * st.k[1] + (d / x) * st.k[2] + off * st.k[3] + (d % x) * st.k[4]] =
        key[t * key_stride + e];
    v_cache[blk * st.v[0] + h * st.v[1] + d * st.v[2] + off * st.v[3]] = value[t * value_stride + e];
}

// The same store for x == 8 two-byte elements and dense inner dimensions, 16 tokens of one head per
// workgroup, staged through LDS so that both sides move 16 bytes per lane: rows are read the way
// they lie in the operands (256 contiguous bytes per token and head), K leaves as one chunk
// column of consecutive tokens (their 16-byte pieces are adjacent in the cache when their slots
// are), and V leaves transposed, eight consecutive tokens of one d per store where those eight
// have consecutive slots starting at a multiple of 8 in one page (two bytes at a time otherwise).
constexpr int kDistinctTokens = DistinctTile<128>::kTokens;

template <typename SlotT, int HD>
__global__ void __launch_bounds__(kThreads)
kv_store_distinct_tiled(const uint16_t* __restrict__ key, const uint16_t* __restrict__ value, int64_t key_stride,
                        int64_t value_stride, uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
                        DistinctStrides st, const SlotT* __restrict__ slots, int64_t n_tokens, int64_t n_pages,
                        int page_size) {
    using Tile = DistinctTile<HD>;
    __shared__ __attribute__((aligned(16))) uint8_t k_tile[Tile::K_BYTES];
    __shared__ __attribute__((aligned(16))) uint8_t v_tile[Tile::V_BYTES];
    __shared__ int64_t slot_of[kDistinctTokens];
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kDistinctTokens;
    const int h = blockIdx.y;
    const int tid = threadIdx.x;
    if (tid < kDistinctTokens) {
        const int64_t t = t0 + tid;
        int64_t slot = t < n_tokens ? static_cast<int64_t>(slots[t]) : -1;
        if (slot >= 0 && slot / page_size >= n_pages) slot = -1;
        slot_of[tid] = slot;
    }
    for (int c = tid; c < kDistinctTokens * Tile::CPR; c += kThreads) {
        const int r = c / Tile::CPR, cc = c % Tile::CPR;
        const int64_t t = t0 + r;
        u32x4 kk = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
        if (t < n_tokens) {
            kk = *reinterpret_cast<const u32x4*>(key + t * key_stride + h * HD + cc * 8);
            vv = *reinterpret_cast<const u32x4*>(value + t * value_stride + h * HD + cc * 8);
        }
        *reinterpret_cast<u32x4*>(k_tile + Tile::k_offset(r, cc)) = kk;
        Tile::put_v(v_tile, r, cc, vv);
    }
    __syncthreads();
    Tile::store(k_tile, v_tile, slot_of, k_cache, v_cache, st.k, st.v, h, page_size, tid, kThreads);
}

// ---------------------------------------------------------------- load (gather)
// grid = (row blocks, sequences).  A block copies kRowsPerBlock consecutive output rows of
// one sequence; each lane moves 16 output bytes of K and of V per step.
constexpr int kRowsPerBlock = 32;

template <bool FP8>
__global__ void __launch_bounds__(kThreads)
kv_load_kernel(const uint8_t* __restrict__ k_cache, const uint8_t* __restrict__ v_cache,
               const uint16_t* __restrict__ k_new, const uint16_t* __restrict__ v_new, int64_t k_new_stride,
               int64_t v_new_stride, uint8_t* __restrict__ k_out, uint8_t* __restrict__ v_out,
               const int32_t* __restrict__ block_tables, int64_t bt_stride, const int32_t* __restrict__ context_lens,
               const int32_t* __restrict__ seq_lens_new, const int32_t* __restrict__ cu_q,
               const int32_t* __restrict__ cu_k, int max_pages, int64_t n_pages, int page_size, int row_bytes,
               int head_dim, const float* __restrict__ k_scale, const float* __restrict__ v_scale) {
    const int s = blockIdx.y;
    const int ctx = context_lens[s];
    const int n_new = seq_lens_new[s];
    const int total = ctx + n_new;
    const int row0 = blockIdx.x * kRowsPerBlock;
    if (row0 >= total) return;
    const int64_t out_row0 = cu_k[s];
    const int64_t new_row0 = cu_q[s];
    const int chunks_per_row = row_bytes >> 4;
    const int n_chunks = kRowsPerBlock * chunks_per_row;
    for (int i = threadIdx.x; i < n_chunks; i += kThreads) {
        const int r = row0 + i / chunks_per_row;
        const int c = i % chunks_per_row;
        if (r >= total) break;
        u32x4 kk, vv;
        if (r < ctx) {
            const int p = r / page_size;
            if (p >= max_pages) continue;
            const int64_t page = block_tables[s * bt_stride + p];
            if (page < 0 || page >= n_pages) continue;
            const int64_t src = (page * page_size + (r - p * page_size)) * row_bytes + c * 16;
            kk = *reinterpret_cast<const u32x4*>(k_cache + src);
            vv = *reinterpret_cast<const u32x4*>(v_cache + src);
        } else {
            const int64_t t = new_row0 + (r - ctx);
            if constexpr (FP8) {  // 16 output codes come from 16 bf16 = two 16-byte chunks
                const int head = (c * 16) / head_dim;
                const float ks = k_scale[head], vs = v_scale[head];
                const u32x4* kp = reinterpret_cast<const u32x4*>(k_new + t * k_new_stride + c * 16);
                const u32x4* vp = reinterpret_cast<const u32x4*>(v_new + t * v_new_stride + c * 16);
                const u32x2 k0 = quantise8(kp[0], ks), k1 = quantise8(kp[1], ks);
                const u32x2 v0 = quantise8(vp[0], vs), v1 = quantise8(vp[1], vs);
                kk = u32x4{k0.x, k0.y, k1.x, k1.y};
                vv = u32x4{v0.x, v0.y, v1.x, v1.y};
            } else {
                kk = *reinterpret_cast<const u32x4*>(k_new + t * k_new_stride + c * 8);
                vv = *reinterpret_cast<const u32x4*>(v_new + t * v_new_stride + c * 8);
            }
        }
        const int64_t dst = (out_row0 + r) * row_bytes + c * 16;
        *reinterpret_cast<u32x4*>(k_out + dst) = kk;
        *reinterpret_cast<u32x4*>(v_out + dst) = vv;
    }
}

template <typename F>
int with_slot_type(int slot_index_type, F&& f) {
    if (slot_index_type == DFX_INDEX_I32) return f(static_cast<const int32_t*>(nullptr));
    if (slot_index_type == DFX_INDEX_I64) return f(static_cast<const int64_t*>(nullptr));
    return DFX_ERR_INVALID_ARG;
}

}  // namespace
}  // namespace dfx

using namespace dfx;

extern "C" int dfx_kv_store_unified(const void* key, const void* value, int64_t key_stride, int64_t value_stride,
                                    void* k_cache, void* v_cache, const void* slot_mapping, int slot_index_type,
                                    int64_t n_tokens, int64_t n_slots, int n_kv_heads, int head_dim, int kv_dtype,
                                    const float* k_scale, const float* v_scale, dfx_stream_t stream) {
    if (n_tokens < 0 || n_slots < 0 || n_kv_heads <= 0 || head_dim <= 0) return DFX_ERR_INVALID_ARG;
    if (n_tokens == 0) return DFX_OK;
    if (!key || !value || !k_cache || !v_cache || !slot_mapping) return DFX_ERR_INVALID_ARG;
    const bool fp8 = kv_dtype == DFX_KV_FP8_E4M3;
    if (!fp8 && kv_dtype != DFX_KV_BF16) return DFX_ERR_INVALID_ARG;
    if (fp8 != (k_scale != nullptr) || fp8 != (v_scale != nullptr)) return DFX_ERR_INVALID_ARG;
    const int64_t row = static_cast<int64_t>(n_kv_heads) * head_dim;
    if (row > INT32_MAX || key_stride < row || value_stride < row) return DFX_ERR_INVALID_ARG;
    const bool vec = (head_dim % 8 == 0) && (key_stride % 8 == 0) && (value_stride % 8 == 0) && aligned16(key) &&
                     aligned16(value) && aligned16(k_cache) && aligned16(v_cache);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* kp = static_cast<const uint16_t*>(key);
    const uint16_t* vp = static_cast<const uint16_t*>(value);
    return with_slot_type(slot_index_type, [&](auto* tag) {
        using SlotT = std::remove_const_t<std::remove_pointer_t<decltype(tag)>>;
        const SlotT* slots = static_cast<const SlotT*>(slot_mapping);
        const int64_t work = n_tokens * (vec ? row / 8 : row);
        const int64_t blocks = (work + kThreads - 1) / kThreads;
        if (blocks > INT32_MAX) return static_cast<int>(DFX_ERR_UNSUPPORTED);
        dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
#define DFX_LAUNCH_STORE(KERNEL, FP8)                                                                        \
    hipLaunchKernelGGL((KERNEL<FP8, SlotT>), grid, block, 0, st, kp, vp, key_stride, value_stride, k_cache,  \
                       v_cache, slots, n_tokens, n_slots, static_cast<int>(row), head_dim, k_scale, v_scale)
        if (vec) {
            if (fp8) DFX_LAUNCH_STORE(kv_store_unified_vec8, true);
            else DFX_LAUNCH_STORE(kv_store_unified_vec8, false);
        } else {
            if (fp8) DFX_LAUNCH_STORE(kv_store_unified_scalar, true);
            else DFX_LAUNCH_STORE(kv_store_unified_scalar, false);
        }
#undef DFX_LAUNCH_STORE
        return launch_status();
    });
}

extern "C" int dfx_kv_store_distinct(const void* key, const void* value, int64_t key_stride, int64_t value_stride,
                                     void* k_cache, void* v_cache, const int64_t kc_stride[5],
                                     const int64_t vc_stride[4], const void* slot_mapping, int slot_index_type,
                                     int64_t n_tokens, int64_t n_pages, int page_size, int x, int n_kv_heads,
                                     int head_dim, dfx_stream_t stream) {
    if (n_tokens < 0 || n_pages < 0 || page_size <= 0 || x <= 0 || n_kv_heads <= 0 || head_dim <= 0)
        return DFX_ERR_INVALID_ARG;
    if (head_dim % x != 0) return DFX_ERR_INVALID_ARG;
    if (n_tokens == 0) return DFX_OK;
    if (!key || !value || !k_cache || !v_cache || !slot_mapping || !kc_stride || !vc_stride)
        return DFX_ERR_INVALID_ARG;
    const int64_t row = static_cast<int64_t>(n_kv_heads) * head_dim;
    if (row > INT32_MAX || key_stride < row || value_stride < row) return DFX_ERR_INVALID_ARG;
    DistinctStrides ds;
    for (int i = 0; i < 5; ++i) ds.k[i] = kc_stride[i];
    for (int i = 0; i < 4; ++i) ds.v[i] = vc_stride[i];
    hipStream_t st = static_cast<hipStream_t>(stream);
    // 16-byte moves on both sides where the shapes allow (x == 8, dense inner dimensions, aligned)
    const bool tiled = x == 8 && (head_dim == 64 || head_dim == 128) && ds.k[4] == 1 && ds.k[3] == 8 && ds.v[3] == 1 &&
                       ds.k[0] % 8 == 0 && ds.k[1] % 8 == 0 && ds.k[2] % 8 == 0 && ds.v[0] % 8 == 0 &&
                       ds.v[1] % 8 == 0 && ds.v[2] % 8 == 0 && key_stride % 8 == 0 && value_stride % 8 == 0 &&
                       aligned16(key) && aligned16(value) && aligned16(k_cache) && aligned16(v_cache) &&
                       n_kv_heads <= 65535;
    return with_slot_type(slot_index_type, [&](auto* tag) {
        using SlotT = std::remove_const_t<std::remove_pointer_t<decltype(tag)>>;
        if (tiled) {
            const int64_t tiles = (n_tokens + kDistinctTokens - 1) / kDistinctTokens;
            if (tiles > INT32_MAX) return static_cast<int>(DFX_ERR_UNSUPPORTED);
            const dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(n_kv_heads));
            auto kern = head_dim == 128 ? kv_store_distinct_tiled<SlotT, 128> : kv_store_distinct_tiled<SlotT, 64>;
            hipLaunchKernelGGL(kern, grid, dim3(kThreads), 0, st, static_cast<const uint16_t*>(key),
                               static_cast<const uint16_t*>(value), key_stride, value_stride,
                               static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), ds,
                               static_cast<const SlotT*>(slot_mapping), n_tokens, n_pages, page_size);
            return launch_status();
        }
        const int64_t blocks = (n_tokens * row + kThreads - 1) / kThreads;
        if (blocks > INT32_MAX) return static_cast<int>(DFX_ERR_UNSUPPORTED);
        hipLaunchKernelGGL((kv_store_distinct_kernel<SlotT>), dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0,
                           st, static_cast<const uint16_t*>(key), static_cast<const uint16_t*>(value), key_stride,
                           value_stride, static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), ds,
                           static_cast<const SlotT*>(slot_mapping), n_tokens, n_pages, page_size, x,
                           static_cast<int>(row), head_dim);
        return launch_status();
    });
}

extern "C" int dfx_kv_load(const void* k_cache, const void* v_cache, const void* k_new, const void* v_new,
                           int64_t k_new_stride, int64_t v_new_stride, void* k_out, void* v_out,
                           const int32_t* block_tables, int64_t block_table_stride, const int32_t* context_lens,
                           const int32_t* seq_lens_new, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                           int num_seqs, int max_pages_per_seq, int64_t n_pages, int page_size, int n_kv_heads,
                           int head_dim, int64_t max_total_len, int kv_dtype, const float* k_scale,
                           const float* v_scale, dfx_stream_t stream) {
    if (num_seqs < 0 || max_pages_per_seq < 0 || n_pages < 0 || page_size <= 0 || n_kv_heads <= 0 ||
        head_dim <= 0 || max_total_len < 0)
        return DFX_ERR_INVALID_ARG;
    if (num_seqs == 0 || max_total_len == 0) return DFX_OK;
    if (!k_cache || !v_cache || !k_new || !v_new || !k_out || !v_out || !block_tables || !context_lens ||
        !seq_lens_new || !cu_seqlens_q || !cu_seqlens_k)
        return DFX_ERR_INVALID_ARG;
    const bool fp8 = kv_dtype == DFX_KV_FP8_E4M3;
    if (!fp8 && kv_dtype != DFX_KV_BF16) return DFX_ERR_INVALID_ARG;
    if (fp8 != (k_scale != nullptr) || fp8 != (v_scale != nullptr)) return DFX_ERR_INVALID_ARG;
    const int64_t row_elems = static_cast<int64_t>(n_kv_heads) * head_dim;
    const int64_t row_bytes = row_elems * (fp8 ? 1 : 2);
    if (row_bytes > INT32_MAX || k_new_stride < row_elems || v_new_stride < row_elems) return DFX_ERR_INVALID_ARG;
    // 16-byte chunks that never straddle a head (the FP8 path picks one scale per chunk)
    if (row_bytes % 16 != 0 || head_dim % 16 != 0 || k_new_stride % 8 != 0 || v_new_stride % 8 != 0)
        return DFX_ERR_UNSUPPORTED;
    if (!aligned16(k_cache) || !aligned16(v_cache) || !aligned16(k_new) || !aligned16(v_new) || !aligned16(k_out) ||
        !aligned16(v_out))
        return DFX_ERR_INVALID_ARG;
    if (num_seqs > 65535) return DFX_ERR_UNSUPPORTED;
    const int64_t row_blocks = (max_total_len + kRowsPerBlock - 1) / kRowsPerBlock;
    if (row_blocks > INT32_MAX) return DFX_ERR_UNSUPPORTED;
    dim3 grid(static_cast<unsigned>(row_blocks), static_cast<unsigned>(num_seqs)), block(kThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define DFX_LAUNCH_LOAD(FP8)                                                                                      \
    hipLaunchKernelGGL((kv_load_kernel<FP8>), grid, block, 0, st, static_cast<const uint8_t*>(k_cache),           \
                       static_cast<const uint8_t*>(v_cache), static_cast<const uint16_t*>(k_new),                 \
                       static_cast<const uint16_t*>(v_new), k_new_stride, v_new_stride,                           \
                       static_cast<uint8_t*>(k_out), static_cast<uint8_t*>(v_out), block_tables,                  \
                       block_table_stride, context_lens, seq_lens_new, cu_seqlens_q, cu_seqlens_k,                \
                       max_pages_per_seq, n_pages, page_size, static_cast<int>(row_bytes), head_dim, k_scale,     \
                       v_scale)
    if (fp8) DFX_LAUNCH_LOAD(true);
    else DFX_LAUNCH_LOAD(false);
#undef DFX_LAUNCH_LOAD
    return launch_status();
}
