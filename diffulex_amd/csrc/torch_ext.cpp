// PyTorch operator library for the gfx950 kernels: torch.ops.diffulex_amd.*
//
// Every operator takes at::Tensors, checks what the C ABI cannot (devices, dtypes, shapes), fills
// the parameter block of include/diffulex_amd.h from sizes, strides and data pointers, and calls
// the exported C function of libdiffulex_amd.so on PyTorch's current HIP stream.  Nothing is
// computed here and nothing is allocated: outputs and scratch are arguments.  Host code only.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include "../../include/diffulex_amd.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

dfx_stream_t current_stream() { return static_cast<dfx_stream_t>(c10::hip::getCurrentHIPStream().stream()); }

void check(int rc, const char* what) {
    TORCH_CHECK(rc == DFX_OK, what, ": ", dfx_status_string(rc), " (", rc, ")");
}

bool has(const OptTensor& t) { return t.has_value() && t->defined() && t->numel() > 0; }

void* ptr(const Tensor& t) { return t.data_ptr(); }
void* ptr(const OptTensor& t) { return has(t) ? t->data_ptr() : nullptr; }

bool is_fp8_cache(const Tensor& c) { return c.scalar_type() == at::kFloat8_e4m3fn || c.scalar_type() == at::kByte; }

int index_type(const Tensor& t, const char* name) {
    if (t.scalar_type() == at::kInt) return DFX_INDEX_I32;
    TORCH_CHECK(t.scalar_type() == at::kLong, name, " must be int32 or int64");
    return DFX_INDEX_I64;
}

void check_i32(const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name,
                " must be a contiguous int32 device tensor");
}

const float* scale_ptr(const OptTensor& s, int n_heads, const char* name) {
    TORCH_CHECK(has(s), "an FP8 KV cache needs ", name);
    TORCH_CHECK(s->is_cuda() && s->scalar_type() == at::kFloat && s->is_contiguous() && s->numel() == n_heads, name,
                " must be a contiguous fp32 device tensor with one entry per KV head");
    return static_cast<const float*>(s->data_ptr());
}

// ---- paged attention ------------------------------------------------------------------------
// The operators of this family share one argument list.
#define DFX_ATTN_ARGS                                                                                              \
    const Tensor &q, const Tensor &k, const Tensor &v, const OptTensor &k_cache, const OptTensor &v_cache,         \
        const OptTensor &out, const OptTensor &block_tables, const OptTensor &context_lens, const Tensor &cu_q,    \
        const Tensor &cu_new, const OptTensor &k_scale, const OptTensor &v_scale, const OptTensor &store_slots,    \
        const OptTensor &plan, double scale, int64_t max_seqlen_q, int64_t mask_mode, int64_t dbs, int64_t max_wg, \
        int64_t flags, int64_t cache_layout, const OptTensor &rope_cos_sin, const OptTensor &rope_positions,       \
        const OptTensor &k_rotated
#define DFX_ATTN_PASS                                                                                              \
    q, k, v, k_cache, v_cache, out, block_tables, context_lens, cu_q, cu_new, k_scale, v_scale, store_slots, plan, \
        scale, max_seqlen_q, mask_mode, dbs, max_wg, flags, cache_layout, rope_cos_sin, rope_positions, k_rotated
#define DFX_ATTN_SCHEMA                                                                                            \
    "Tensor q, Tensor k, Tensor v, Tensor(a!)? k_cache, Tensor(b!)? v_cache, Tensor(c!)? out, Tensor? block_tables, "          \
    "Tensor? context_lens, Tensor cu_seqlens_q, Tensor cu_seqlens_new, Tensor? k_scale, Tensor? v_scale, "         \
    "Tensor? store_slot_mapping, Tensor? plan, float scale, int max_seqlen_q, int mask_mode, "                     \
    "int diffusion_block_size, int max_workgroups, int flags, int cache_layout, Tensor? rope_cos_sin, "            \
    "Tensor? rope_positions, Tensor(e!)? k_rotated"

dfx_attn_params attn_params(DFX_ATTN_ARGS) {
    TORCH_CHECK(q.is_cuda() && q.scalar_type() == at::kBFloat16 && k.scalar_type() == at::kBFloat16 &&
                    v.scalar_type() == at::kBFloat16,
                "q, k and v must be bf16 device tensors");
    TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.sizes() == k.sizes(), "q: [T, H_q, hd]; k, v: [T_new, H_kv, hd]");
    TORCH_CHECK(q.stride(2) == 1 && k.stride(2) == 1 && v.stride(2) == 1, "the head dimension must be dense");
    const int64_t h_q = q.size(1), hd = q.size(2), h_kv = k.size(1);
    TORCH_CHECK(k.size(2) == hd && h_kv > 0 && h_q % h_kv == 0, "head counts / head_dim of q and k do not fit");
    check_i32(cu_q, "cu_seqlens_q");
    check_i32(cu_new, "cu_seqlens_new");
    const int64_t num_seqs = cu_q.numel() - 1;
    TORCH_CHECK(cu_new.numel() == num_seqs + 1, "cu_seqlens_q and cu_seqlens_new differ in length");
    dfx_attn_params p = {};
    const bool cache = has(k_cache);
    TORCH_CHECK(cache == has(v_cache), "k_cache and v_cache come together");
    p.kv_dtype = DFX_KV_BF16;
    if (cache) {
        TORCH_CHECK(has(block_tables) && has(context_lens), "a cache needs block_tables and context_lens");
        TORCH_CHECK(block_tables->is_cuda() && block_tables->scalar_type() == at::kInt && block_tables->dim() == 2 &&
                        block_tables->stride(1) == 1 && block_tables->size(0) == num_seqs,
                    "block_tables must be int32 [num_seqs, max_pages] with dense rows");
        check_i32(*context_lens, "context_lens");
        TORCH_CHECK(context_lens->numel() == num_seqs, "context_lens must have one entry per sequence");
        p.k_cache = k_cache->data_ptr();
        p.v_cache = v_cache->data_ptr();
        p.block_tables = static_cast<const int32_t*>(block_tables->data_ptr());
        p.context_lens = static_cast<const int32_t*>(context_lens->data_ptr());
        p.block_table_stride = block_tables->stride(0);
        p.max_pages_per_seq = static_cast<int32_t>(block_tables->size(1));
        p.n_pages = k_cache->size(0);
        if (cache_layout == DFX_CACHE_DISTINCT) {
            TORCH_CHECK(k_cache->dim() == 5 && v_cache->dim() == 4 && k_cache->scalar_type() == at::kBFloat16 &&
                            v_cache->scalar_type() == at::kBFloat16,
                        "distinct layout: k_cache [pages, H, hd / 8, page, 8], v_cache [pages, H, hd, page], bf16");
            const int64_t page = k_cache->size(3);
            TORCH_CHECK(k_cache->size(1) == h_kv && k_cache->size(2) * k_cache->size(4) == hd && k_cache->size(4) == 8 &&
                            v_cache->size(0) == p.n_pages && v_cache->size(1) == h_kv && v_cache->size(2) == hd &&
                            v_cache->size(3) == page,
                        "distinct layout: cache shapes do not fit the heads");
            TORCH_CHECK(!has(store_slots), "the distinct layout has a store launch of its own");
            p.page_size = static_cast<int32_t>(page);
            p.cache_layout = DFX_CACHE_DISTINCT;
            for (int i = 0; i < 5; ++i) p.kc_stride[i] = k_cache->stride(i);
            for (int i = 0; i < 4; ++i) p.vc_stride[i] = v_cache->stride(i);
        } else {
            TORCH_CHECK(cache_layout == DFX_CACHE_UNIFIED, "unknown cache layout");
            TORCH_CHECK(k_cache->dim() == 4 && k_cache->sizes() == v_cache->sizes() && k_cache->size(2) == h_kv &&
                            k_cache->size(3) == hd && k_cache->strides() == v_cache->strides() && k_cache->stride(3) == 1,
                        "unified layout: caches [pages, page, H_kv, hd], laid out alike");
            p.page_size = static_cast<int32_t>(k_cache->size(1));
            p.cache_stride_page = k_cache->stride(0);
            p.cache_stride_token = k_cache->stride(1);
            p.cache_stride_head = k_cache->stride(2);
            if (is_fp8_cache(*k_cache)) {
                p.kv_dtype = DFX_KV_FP8_E4M3;
                p.k_scale = scale_ptr(k_scale, static_cast<int>(h_kv), "k_scale");
                p.v_scale = scale_ptr(v_scale, static_cast<int>(h_kv), "v_scale");
            } else {
                TORCH_CHECK(k_cache->element_size() == 2, "unsupported cache dtype");
            }
        }
    }
    p.q = q.data_ptr();
    p.k_new = k.data_ptr();
    p.v_new = v.data_ptr();
    p.cu_seqlens_q = static_cast<const int32_t*>(cu_q.data_ptr());
    p.cu_seqlens_new = static_cast<const int32_t*>(cu_new.data_ptr());
    p.q_stride_token = q.stride(0);
    p.q_stride_head = q.stride(1);
    p.kn_stride_token = k.stride(0);
    p.kn_stride_head = k.stride(1);
    p.vn_stride_token = v.stride(0);
    p.vn_stride_head = v.stride(1);
    if (has(out)) {
        TORCH_CHECK(out->is_cuda() && out->scalar_type() == at::kBFloat16 && out->sizes() == q.sizes() &&
                        out->stride(2) == 1,
                    "out must be a bf16 device tensor shaped like q");
        p.out = out->data_ptr();
        p.o_stride_token = out->stride(0);
        p.o_stride_head = out->stride(1);
    }
    p.num_seqs = static_cast<int32_t>(num_seqs);
    p.num_q_heads = static_cast<int32_t>(h_q);
    p.num_kv_heads = static_cast<int32_t>(h_kv);
    p.head_dim = static_cast<int32_t>(hd);
    p.num_new_tokens = k.size(0);
    p.num_q_tokens = static_cast<int32_t>(q.size(0));
    if (has(rope_cos_sin)) {
        TORCH_CHECK(rope_cos_sin->is_cuda() && rope_cos_sin->scalar_type() == at::kFloat && rope_cos_sin->is_contiguous() &&
                        rope_cos_sin->dim() == 2 && rope_cos_sin->size(1) == hd,
                    "rope_cos_sin: contiguous fp32 [max_position, head_dim]");
        TORCH_CHECK(has(rope_positions) && rope_positions->is_cuda() && rope_positions->is_contiguous() &&
                        rope_positions->numel() == q.size(0) && q.size(0) == k.size(0),
                    "rope_positions: one position per token, the same tokens in q and k");
        TORCH_CHECK(has(k_rotated) && k_rotated->is_cuda() && k_rotated->scalar_type() == at::kBFloat16 &&
                        k_rotated->sizes() == k.sizes() && k_rotated->stride(2) == 1,
                    "k_rotated: a bf16 device tensor shaped like k");
        p.rope_cos_sin = static_cast<const float*>(rope_cos_sin->data_ptr());
        p.rope_positions = rope_positions->data_ptr();
        p.rope_position_index_type = index_type(*rope_positions, "rope_positions");
        p.rope_max_position = rope_cos_sin->size(0);
        p.k_rotated = k_rotated->data_ptr();
        p.kr_stride_token = k_rotated->stride(0);
        p.kr_stride_head = k_rotated->stride(1);
    }
    p.max_seqlen_q = static_cast<int32_t>(max_seqlen_q);
    p.diffusion_block_size = static_cast<int32_t>(dbs);
    p.mask_mode = static_cast<int32_t>(mask_mode);
    p.max_workgroups = static_cast<int32_t>(max_wg);
    p.flags = static_cast<uint32_t>(flags);
    p.scale = static_cast<float>(scale);
    if (has(store_slots)) {
        TORCH_CHECK(cache && store_slots->is_cuda() && store_slots->is_contiguous() && store_slots->numel() == k.size(0),
                    "`N`: ", k.size(0), ", `slot_mapping.numel()`: ", store_slots->numel());
        p.store_slot_mapping = store_slots->data_ptr();
        p.store_slot_index_type = index_type(*store_slots, "store_slot_mapping");
    }
    if (has(plan)) {
        TORCH_CHECK(plan->is_cuda() && plan->is_contiguous() && plan->scalar_type() == at::kByte, "plan: uint8 device tensor");
        p.plan = plan->data_ptr();
        p.plan_bytes = plan->numel();
    }
    return p;
}

// workspace: uint8 scratch of at least paged_attention_workspace_bytes; static_scratch: use the
// library's static device array instead.
void paged_attention(DFX_ATTN_ARGS, const OptTensor& workspace, bool static_scratch) {
    dfx_attn_params p = attn_params(DFX_ATTN_PASS);
    TORCH_CHECK(p.out != nullptr, "paged_attention needs out");
    if (static_scratch) {
        check(dfx_paged_attn_static(&p, current_stream()), "dfx_paged_attn_static");
        return;
    }
    if (has(workspace)) {
        TORCH_CHECK(workspace->is_cuda() && workspace->is_contiguous(), "workspace: contiguous device tensor");
        p.workspace = workspace->data_ptr();
        p.workspace_bytes = workspace->numel() * workspace->element_size();
    }
    check(dfx_paged_attn(&p, current_stream()), "dfx_paged_attn");
}

int64_t paged_attention_workspace_bytes(DFX_ATTN_ARGS) {
    dfx_attn_params p = attn_params(DFX_ATTN_PASS);
    const int64_t n = dfx_paged_attn_workspace_bytes(&p);
    if (n < 0) check(static_cast<int>(n), "dfx_paged_attn_workspace_bytes");
    return n;
}

// Bytes of a plan with room for max_units units; -2 where no plan applies (generic tile path).
int64_t paged_attention_plan_bytes(DFX_ATTN_ARGS, int64_t max_units) {
    dfx_attn_params p = attn_params(DFX_ATTN_PASS);
    return dfx_paged_attn_plan_bytes(&p, max_units);
}

void paged_attention_plan(DFX_ATTN_ARGS, Tensor plan_out) {
    dfx_attn_params p = attn_params(DFX_ATTN_PASS);
    TORCH_CHECK(plan_out.is_cuda() && plan_out.is_contiguous() && plan_out.scalar_type() == at::kByte,
                "plan_out: uint8 device tensor");
    check(dfx_paged_attn_plan(&p, plan_out.data_ptr(), plan_out.numel(), current_stream()), "dfx_paged_attn_plan");
}

int64_t stream_capture_id() { return dfx_stream_capture_id(current_stream()); }

// ---- KV cache ---------------------------------------------------------------------------------
void kv_store_unified(const Tensor& key, const Tensor& value, Tensor k_cache, Tensor v_cache, const Tensor& slot_mapping,
                      const OptTensor& k_scale, const OptTensor& v_scale) {
    TORCH_CHECK(key.dim() == 3 && value.sizes() == key.sizes(), "key, value: [N, H_kv, hd]");
    const int64_t n = key.size(0), heads = key.size(1), hd = key.size(2), row = heads * hd;
    TORCH_CHECK(key.stride(2) == 1 && value.stride(2) == 1 && key.stride(1) == hd && value.stride(1) == hd,
                "key and value rows must be dense");
    TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && k_cache.stride(1) == row &&
                    v_cache.stride(1) == row,
                "caches: contiguous [pages, page, H_kv, hd]");
    TORCH_CHECK(n == slot_mapping.numel(), "`N`: ", n, ", `slot_mapping.numel()`: ", slot_mapping.numel());
    TORCH_CHECK(key.is_cuda() && k_cache.is_cuda() && slot_mapping.is_cuda() && slot_mapping.is_contiguous(),
                "device tensors, slot_mapping contiguous");
    TORCH_CHECK(key.element_size() == 2 && value.element_size() == 2, "key and value must have 2-byte elements");
    int kv_dtype = DFX_KV_BF16;
    const float *ks = nullptr, *vs = nullptr;
    if (is_fp8_cache(k_cache)) {
        kv_dtype = DFX_KV_FP8_E4M3;
        ks = scale_ptr(k_scale, static_cast<int>(heads), "k_scale");
        vs = scale_ptr(v_scale, static_cast<int>(heads), "v_scale");
    } else {
        TORCH_CHECK(k_cache.element_size() == 2, "unsupported cache dtype");
    }
    check(dfx_kv_store_unified(key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0), k_cache.data_ptr(),
                               v_cache.data_ptr(), slot_mapping.data_ptr(), index_type(slot_mapping, "slot_mapping"), n,
                               k_cache.size(0) * k_cache.size(1), static_cast<int>(heads), static_cast<int>(hd), kv_dtype,
                               ks, vs, current_stream()),
          "dfx_kv_store_unified");
}

void kv_store_distinct(const Tensor& key, const Tensor& value, Tensor k_cache, Tensor v_cache, const Tensor& slot_mapping) {
    TORCH_CHECK(key.dim() == 3 && value.sizes() == key.sizes() && k_cache.dim() == 5 && v_cache.dim() == 4,
                "key, value: [N, H, hd]; k_cache: [pages, H, hd / x, page, x]; v_cache: [pages, H, hd, page]");
    const int64_t n = key.size(0), heads = key.size(1), hd = key.size(2), x = k_cache.size(4);
    TORCH_CHECK(k_cache.size(2) * x == hd && k_cache.size(1) == heads, "k_cache does not fit key");
    TORCH_CHECK(n == slot_mapping.numel(), "`N`: ", n, ", `slot_mapping.numel()`: ", slot_mapping.numel());
    TORCH_CHECK(key.stride(2) == 1 && value.stride(2) == 1 && key.stride(1) == hd && value.stride(1) == hd,
                "key and value rows must be dense");
    TORCH_CHECK(key.element_size() == 2 && k_cache.element_size() == 2 && v_cache.element_size() == 2, "2-byte elements");
    TORCH_CHECK(key.is_cuda() && k_cache.is_cuda() && slot_mapping.is_cuda() && slot_mapping.is_contiguous(),
                "device tensors, slot_mapping contiguous");
    int64_t kcs[5], vcs[4];
    for (int i = 0; i < 5; ++i) kcs[i] = k_cache.stride(i);
    for (int i = 0; i < 4; ++i) vcs[i] = v_cache.stride(i);
    check(dfx_kv_store_distinct(key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0), k_cache.data_ptr(),
                                v_cache.data_ptr(), kcs, vcs, slot_mapping.data_ptr(),
                                index_type(slot_mapping, "slot_mapping"), n, k_cache.size(0),
                                static_cast<int>(k_cache.size(3)), static_cast<int>(x), static_cast<int>(heads),
                                static_cast<int>(hd), current_stream()),
          "dfx_kv_store_distinct");
}

void kv_load(const Tensor& k_cache, const Tensor& v_cache, const Tensor& k_new, const Tensor& v_new, Tensor k_out,
             Tensor v_out, const Tensor& block_tables, const Tensor& context_lens, const Tensor& seq_lens_new,
             const Tensor& cu_q, const Tensor& cu_k, int64_t max_total_len, const OptTensor& k_scale,
             const OptTensor& v_scale) {
    TORCH_CHECK(k_cache.sizes() == v_cache.sizes() && k_new.sizes() == v_new.sizes() && k_cache.dim() == 4,
                "caches [pages, page, H_kv, hd] alike; k_new, v_new alike");
    const int64_t heads = k_cache.size(2), hd = k_cache.size(3);
    const int64_t num_seqs = block_tables.size(0);
    TORCH_CHECK(cu_q.sizes() == cu_k.sizes() && cu_q.size(0) == num_seqs + 1, "cu_seqlens have num_seqs + 1 entries");
    TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous(), "caches must be contiguous");
    TORCH_CHECK(k_new.stride(2) == 1 && k_new.stride(1) == hd && v_new.stride(2) == 1 && v_new.stride(1) == hd,
                "fresh rows must be dense");
    check_i32(context_lens, "context_lens");
    check_i32(seq_lens_new, "seq_lens");
    check_i32(cu_q, "cu_seqlens_q");
    check_i32(cu_k, "cu_seqlens_k");
    TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.stride(1) == 1,
                "block_tables: int32 with dense rows");
    TORCH_CHECK(k_out.is_contiguous() && v_out.is_contiguous() && k_out.scalar_type() == k_cache.scalar_type() &&
                    v_out.sizes() == k_out.sizes(),
                "outputs: contiguous, of the cache's dtype");
    int kv_dtype = DFX_KV_BF16;
    const float *ks = nullptr, *vs = nullptr;
    if (is_fp8_cache(k_cache)) {
        kv_dtype = DFX_KV_FP8_E4M3;
        ks = scale_ptr(k_scale, static_cast<int>(heads), "k_scale");
        vs = scale_ptr(v_scale, static_cast<int>(heads), "v_scale");
    }
    // an empty tensor has no data pointer; no fresh row is read then, any valid pointer serves
    const void* kn = k_new.numel() ? k_new.data_ptr() : k_cache.data_ptr();
    const void* vn = v_new.numel() ? v_new.data_ptr() : v_cache.data_ptr();
    check(dfx_kv_load(k_cache.data_ptr(), v_cache.data_ptr(), kn, vn, k_new.stride(0), v_new.stride(0), k_out.data_ptr(),
                      v_out.data_ptr(), static_cast<const int32_t*>(block_tables.data_ptr()), block_tables.stride(0),
                      static_cast<const int32_t*>(context_lens.data_ptr()),
                      static_cast<const int32_t*>(seq_lens_new.data_ptr()), static_cast<const int32_t*>(cu_q.data_ptr()),
                      static_cast<const int32_t*>(cu_k.data_ptr()), static_cast<int>(num_seqs),
                      static_cast<int>(block_tables.size(1)), k_cache.size(0), static_cast<int>(k_cache.size(1)),
                      static_cast<int>(heads), static_cast<int>(hd), max_total_len, kv_dtype, ks, vs, current_stream()),
          "dfx_kv_load");
}

// ---- rotary embedding (+ KV-cache store) ------------------------------------------------------
int64_t rows_of(const Tensor& x, int64_t head_size, int64_t& heads, const char* name) {
    TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kBFloat16 && (x.dim() == 2 || x.dim() == 3) && x.stride(-1) == 1, name,
                ": bf16 device tensor [T, H * hd] or [T, H, hd]");
    if (x.dim() == 3) {
        TORCH_CHECK(x.size(2) == head_size && x.stride(1) == head_size, name, ": heads must be dense");
        heads = x.size(1);
    } else {
        TORCH_CHECK(x.size(1) % head_size == 0, name, ": row length is not a multiple of head_size");
        heads = x.size(1) / head_size;
    }
    return x.size(0);
}

void rope_kv_store(const Tensor& positions, const Tensor& query, const Tensor& key, Tensor q_out, Tensor k_out,
                   const Tensor& cos_sin_cache, int64_t head_size, const OptTensor& value, const OptTensor& k_cache,
                   const OptTensor& v_cache, const OptTensor& slot_mapping, const OptTensor& k_scale,
                   const OptTensor& v_scale) {
    TORCH_CHECK(cos_sin_cache.is_cuda() && cos_sin_cache.scalar_type() == at::kFloat && cos_sin_cache.is_contiguous(),
                "cos_sin_cache: contiguous fp32 device tensor");
    int64_t hq, hk;
    const int64_t tq = rows_of(query, head_size, hq, "query"), tk = rows_of(key, head_size, hk, "key");
    TORCH_CHECK(positions.is_contiguous() && tq == tk && tq == positions.numel(), "one position per token row of query and key");
    dfx_rope_params p = {};
    p.q = query.data_ptr();
    p.k = key.data_ptr();
    p.q_out = q_out.data_ptr();
    p.k_out = k_out.data_ptr();
    p.q_stride_token = query.stride(0);
    p.k_stride_token = key.stride(0);
    p.q_out_stride_token = q_out.stride(0);
    p.k_out_stride_token = k_out.stride(0);
    p.positions = positions.data_ptr();
    p.position_index_type = index_type(positions, "positions");
    p.cos_sin_cache = static_cast<const float*>(cos_sin_cache.data_ptr());
    p.max_position = cos_sin_cache.size(0);
    p.n_tokens = tq;
    p.num_q_heads = static_cast<int32_t>(hq);
    p.num_kv_heads = static_cast<int32_t>(hk);
    p.head_dim = static_cast<int32_t>(head_size);
    p.kv_dtype = DFX_KV_BF16;
    if (has(slot_mapping)) {
        TORCH_CHECK(has(value) && has(k_cache) && has(v_cache), "the store needs value and both caches");
        int64_t hv;
        const int64_t tv = rows_of(*value, head_size, hv, "value");
        const int64_t row = hk * head_size;
        TORCH_CHECK(tv == tk && hv == hk, "value does not fit key");
        const bool distinct = k_cache->dim() == 5;   // K [pages, H_kv, hd / 8, page, 8], V [pages, H_kv, hd, page]
        if (distinct) {
            TORCH_CHECK(v_cache->dim() == 4 && k_cache->size(1) == hk && v_cache->size(1) == hk && k_cache->size(4) == 8 &&
                            k_cache->size(2) * 8 == head_size && v_cache->size(2) == head_size &&
                            k_cache->size(3) == v_cache->size(3) && k_cache->size(0) == v_cache->size(0) &&
                            k_cache->stride(4) == 1 && k_cache->stride(3) == 8 && v_cache->stride(3) == 1 &&
                            k_cache->scalar_type() == at::kBFloat16 && v_cache->scalar_type() == at::kBFloat16,
                        "distinct layout: bf16 K [pages, H_kv, hd / 8, page, 8] and V [pages, H_kv, hd, page], tokens dense");
            p.cache_layout = DFX_CACHE_DISTINCT;
            p.page_size = static_cast<int32_t>(k_cache->size(3));
            for (int i = 0; i < 3; ++i) {
                p.kc_stride[i] = k_cache->stride(i);
                p.vc_stride[i] = v_cache->stride(i);
            }
        } else {
            TORCH_CHECK(k_cache->is_contiguous() && v_cache->is_contiguous() && k_cache->dim() == 4 &&
                            k_cache->stride(1) == row && v_cache->stride(1) == row,
                        "caches: contiguous [pages, page, H_kv, hd]");
        }
        TORCH_CHECK(slot_mapping->is_contiguous() && slot_mapping->numel() == tk, "`N`: ", tk,
                    ", `slot_mapping.numel()`: ", slot_mapping->numel());
        p.v = value->data_ptr();
        p.v_stride_token = value->stride(0);
        p.k_cache = k_cache->data_ptr();
        p.v_cache = v_cache->data_ptr();
        p.slot_mapping = slot_mapping->data_ptr();
        p.slot_index_type = index_type(*slot_mapping, "slot_mapping");
        p.n_slots = distinct ? k_cache->size(0) * k_cache->size(3) : k_cache->size(0) * k_cache->size(1);
        if (!distinct && is_fp8_cache(*k_cache)) {
            p.kv_dtype = DFX_KV_FP8_E4M3;
            p.k_scale = scale_ptr(k_scale, static_cast<int>(hk), "k_scale");
            p.v_scale = scale_ptr(v_scale, static_cast<int>(hk), "v_scale");
        }
    }
    check(dfx_rope_kv_store(&p, current_stream()), "dfx_rope_kv_store");
}

// ---- decode metadata ---------------------------------------------------------------------------
void build_decode_metadata(int64_t strategy, const Tensor& block_tables, const Tensor& block_state, int64_t page_size,
                           int64_t dbs, const OptTensor& num_tokens, const OptTensor& num_pages,
                           const OptTensor& prompt_len, const OptTensor& num_diffusion_blocks, Tensor positions,
                           Tensor slot_mapping, Tensor cu_q, Tensor cu_k, Tensor context_lens, Tensor seq_lens,
                           Tensor summary, int64_t token_capacity, int64_t padded_seqs, int64_t padded_tokens,
                           const OptTensor& token_ids, const OptTensor& input_ids) {
    const int64_t n = block_tables.size(0);
    const int64_t rows = std::max(n, padded_seqs);
    TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
                    block_tables.stride(1) == 1,
                "block_tables: int32 [num_seqs, max_pages] with dense rows");
    TORCH_CHECK(block_state.is_cuda() && block_state.scalar_type() == at::kByte && block_state.stride(-1) == 1,
                "block_state: uint8 device tensor");
    for (const OptTensor* t : {&num_tokens, &num_pages, &prompt_len, &num_diffusion_blocks}) {
        if (has(*t)) {
            check_i32(**t, "per-sequence input");
            TORCH_CHECK((*t)->numel() == n, "per-sequence inputs have one entry per sequence");
        }
    }
    check_i32(slot_mapping, "slot_mapping");
    check_i32(cu_q, "cu_seqlens_q");
    check_i32(cu_k, "cu_seqlens_k");
    check_i32(context_lens, "context_lens");
    check_i32(seq_lens, "seq_lens");
    check_i32(summary, "summary");
    TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == at::kLong && positions.is_contiguous(), "positions: int64");
    TORCH_CHECK(positions.numel() >= token_capacity && slot_mapping.numel() >= token_capacity && cu_q.numel() >= rows + 1 &&
                    cu_k.numel() >= rows + 1 && context_lens.numel() >= rows && seq_lens.numel() >= rows &&
                    summary.numel() >= 8,
                "an output tensor is too small");
    dfx_metadata_params p = {};
    p.strategy = static_cast<int32_t>(strategy);
    p.num_seqs = static_cast<int32_t>(n);
    p.page_size = static_cast<int32_t>(page_size);
    p.diffusion_block_size = static_cast<int32_t>(dbs);
    p.num_tokens = static_cast<const int32_t*>(ptr(num_tokens));
    p.prompt_len = static_cast<const int32_t*>(ptr(prompt_len));
    p.block_state = static_cast<const uint8_t*>(block_state.data_ptr());
    p.block_state_stride = block_state.dim() == 2 ? block_state.stride(0) : 1;
    p.num_diffusion_blocks = static_cast<const int32_t*>(ptr(num_diffusion_blocks));
    p.block_tables = static_cast<const int32_t*>(block_tables.data_ptr());
    p.block_table_stride = block_tables.stride(0);
    p.num_pages = static_cast<const int32_t*>(ptr(num_pages));
    p.positions = static_cast<int64_t*>(positions.data_ptr());
    p.slot_mapping = static_cast<int32_t*>(slot_mapping.data_ptr());
    p.token_capacity = token_capacity;
    p.cu_seqlens_q = static_cast<int32_t*>(cu_q.data_ptr());
    p.cu_seqlens_k = static_cast<int32_t*>(cu_k.data_ptr());
    p.context_lens = static_cast<int32_t*>(context_lens.data_ptr());
    p.seq_lens = static_cast<int32_t*>(seq_lens.data_ptr());
    p.padded_seqs = static_cast<int32_t>(padded_seqs);
    p.padded_tokens = padded_tokens;
    p.summary = static_cast<int32_t*>(summary.data_ptr());
    TORCH_CHECK(has(token_ids) == has(input_ids), "token_ids and input_ids go together");
    if (has(token_ids)) {
        TORCH_CHECK(token_ids->is_cuda() && token_ids->scalar_type() == at::kLong && token_ids->dim() == 2 &&
                        token_ids->size(0) == n && token_ids->stride(1) == 1,
                    "token_ids: int64 [num_seqs, max_len] with dense rows");
        TORCH_CHECK(input_ids->is_cuda() && input_ids->scalar_type() == at::kLong && input_ids->is_contiguous() &&
                        input_ids->numel() >= token_capacity,
                    "input_ids: int64 [token_capacity]");
        p.token_ids = static_cast<const int64_t*>(token_ids->data_ptr());
        p.token_ids_stride = token_ids->stride(0);
        p.input_ids = static_cast<int64_t*>(input_ids->data_ptr());
    }
    check(dfx_build_decode_metadata(&p, current_stream()), "dfx_build_decode_metadata");
}

}  // namespace

TORCH_LIBRARY(diffulex_amd, m) {
    m.def("paged_attention(" DFX_ATTN_SCHEMA ", Tensor? workspace, bool static_scratch) -> ()");
    m.def("paged_attention_workspace_bytes(" DFX_ATTN_SCHEMA ") -> int");
    m.def("paged_attention_plan_bytes(" DFX_ATTN_SCHEMA ", int max_units) -> int");
    m.def("paged_attention_plan(" DFX_ATTN_SCHEMA ", Tensor(d!) plan_out) -> ()");
    m.def("stream_capture_id() -> int", stream_capture_id);
    m.def("kv_store_unified(Tensor key, Tensor value, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor slot_mapping, "
          "Tensor? k_scale, Tensor? v_scale) -> ()");
    m.def("kv_store_distinct(Tensor key, Tensor value, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor slot_mapping) -> ()");
    m.def("kv_load(Tensor k_cache, Tensor v_cache, Tensor k_new, Tensor v_new, Tensor(a!) k_out, Tensor(b!) v_out, "
          "Tensor block_tables, Tensor context_lens, Tensor seq_lens_new, Tensor cu_seqlens_q, Tensor cu_seqlens_k, "
          "int max_total_len, Tensor? k_scale, Tensor? v_scale) -> ()");
    m.def("rope_kv_store(Tensor positions, Tensor query, Tensor key, Tensor(a!) q_out, Tensor(b!) k_out, Tensor cos_sin_cache, "
          "int head_size, Tensor? value, Tensor(c!)? k_cache, Tensor(d!)? v_cache, Tensor? slot_mapping, Tensor? k_scale, "
          "Tensor? v_scale) -> ()");
    m.def("build_decode_metadata(int strategy, Tensor block_tables, Tensor block_state, int page_size, "
          "int diffusion_block_size, Tensor? num_tokens, Tensor? num_pages, Tensor? prompt_len, "
          "Tensor? num_diffusion_blocks, Tensor(a!) positions, Tensor(b!) slot_mapping, Tensor(c!) cu_seqlens_q, "
          "Tensor(d!) cu_seqlens_k, Tensor(e!) context_lens, Tensor(f!) seq_lens, Tensor(g!) summary, int token_capacity, int padded_seqs, "
          "int padded_tokens, Tensor? token_ids, Tensor(h!)? input_ids) -> ()");
}

// The kernels exist for the GPU only: the operators are registered for device tensors and nothing else.
TORCH_LIBRARY_IMPL(diffulex_amd, CUDA, m) {
    m.impl("paged_attention", paged_attention);
    m.impl("paged_attention_workspace_bytes", paged_attention_workspace_bytes);
    m.impl("paged_attention_plan_bytes", paged_attention_plan_bytes);
    m.impl("paged_attention_plan", paged_attention_plan);
    m.impl("kv_store_unified", kv_store_unified);
    m.impl("kv_store_distinct", kv_store_distinct);
    m.impl("kv_load", kv_load);
    m.impl("rope_kv_store", rope_kv_store);
    m.impl("build_decode_metadata", build_decode_metadata);
}
