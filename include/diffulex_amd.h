/*
 * diffulex_amd: C ABI of the MI355X (gfx950) dLLM decoding hot path.
 *
 * One shared library, libdiffulex_amd.so, exports the functions below.  They
 * take plain device pointers, element strides, sizes and a HIP stream; they
 * never allocate, never synchronise with the host and never throw.  Every
 * function returns 0 (DFX_OK) or a negative dfx_status; on a non-zero return
 * nothing has been launched.
 *
 * "Replaces" names the reference (zhijie-group/Diffulex) interface whose device
 * work the entry point takes over; paths are relative to the reference tree.
 */
#ifndef DIFFULEX_AMD_H_
#define DIFFULEX_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DFX_ABI_VERSION 8

typedef void* dfx_stream_t; /* a hipStream_t; NULL is the default stream */

typedef enum dfx_status {
    DFX_OK = 0,
    DFX_ERR_INVALID_ARG = -1, /* null pointer, negative size, misaligned pointer or stride */
    DFX_ERR_UNSUPPORTED = -2, /* a shape this build has no kernel for (see each function) */
    DFX_ERR_WORKSPACE = -3,   /* workspace missing or smaller than dfx_paged_attn_workspace_bytes */
    DFX_ERR_LAUNCH = -4,      /* the HIP runtime refused the launch */
    DFX_ERR_SCRATCH_LIMIT = -5 /* dfx_paged_attn_static: the shape needs more than DFX_STATIC_SCRATCH_BYTES */
} dfx_status;

typedef enum dfx_kv_dtype {
    DFX_KV_BF16 = 0,    /* 2-byte elements, copied bit for bit (bf16; fp16 works for store/load) */
    DFX_KV_FP8_E4M3 = 1 /* OCP e4m3fn codes with one fp32 scale per KV head */
} dfx_kv_dtype;

typedef enum dfx_mask_mode {
    DFX_MASK_FULL = 0,        /* every fresh token of the sequence is visible to every query */
    DFX_MASK_BLOCK_CAUSAL = 1 /* fresh token j visible to query i iff j < (i / dbs + 1) * dbs */
} dfx_mask_mode;

typedef enum dfx_cache_layout { DFX_CACHE_UNIFIED = 0, DFX_CACHE_DISTINCT = 1 } dfx_cache_layout;

typedef enum dfx_index_type { DFX_INDEX_I32 = 0, DFX_INDEX_I64 = 1 } dfx_index_type;

/* dfx_attn_params.flags */
#define DFX_ATTN_GENERIC_PATH 1 /* use the generic tile path even where the streaming path applies */
#define DFX_ATTN_NO_PIPELINE 2  /* streaming path: the plain tile loop instead of the software-pipelined one */
#define DFX_ATTN_PAIRING 4      /* dfx_paged_attn_plan: the pairing partition where it applies (see there) */
#define DFX_ATTN_EQUAL_RANGES 8 /* dfx_paged_attn_plan: equal ranges of the unit space, as a launch without a plan cuts
                                   them (the plan's own cut points are placed by cost; see there) */
#define DFX_ATTN_BATCH_ORDER 16 /* dfx_paged_attn_plan: keep the sequences in the batch's order when the work is dealt
                                   to the workgroups (by default the plan may deal them in another order; see there) */

/* ABI version of the loaded library (== DFX_ABI_VERSION it was built with). */
int dfx_abi_version(void);

/* Static string for a dfx_status value. */
const char* dfx_status_string(int status);

/*
 * Paged KV-cache store, unified layout.
 * Replaces: store_kvcache_unified_layout + dllm_store_kvcache_kernel_unified
 *           (diffulex_kernel/python/kv_cache_kernels.py:110-124, :11-32).
 *
 * key/value: [n_tokens, n_kv_heads, head_dim] bf16, innermost two dims dense,
 * row stride key_stride / value_stride (elements).  Caches: [n_slots, n_kv_heads,
 * head_dim] dense, n_slots = pages * page_size.  For each token t with
 * slot = slot_mapping[t]: slot < 0 is skipped, otherwise cache[slot] = row t.
 * slot >= n_slots is skipped as well (the reference would write out of bounds).
 * Duplicate slots are a caller error (unordered writes), as in the reference.
 *
 * kv_dtype == DFX_KV_FP8_E4M3: caches hold 1-byte codes and each element is
 * stored as RNE_e4m3fn(clamp(float(x) / scale[head], -448, 448)); k_scale and
 * v_scale are fp32[n_kv_heads].  With DFX_KV_BF16 they must be NULL.
 */
int dfx_kv_store_unified(const void* key, const void* value, int64_t key_stride, int64_t value_stride,
                         void* k_cache, void* v_cache, const void* slot_mapping, int slot_index_type,
                         int64_t n_tokens, int64_t n_slots, int n_kv_heads, int head_dim, int kv_dtype,
                         const float* k_scale, const float* v_scale, dfx_stream_t stream);

/*
 * Paged KV-cache store, "distinct" (vLLM-style) layout.
 * Replaces: store_kvcache_distinct_layout + dllm_store_kvcache_kernel_distinct
 *           (diffulex_kernel/python/kv_cache_kernels.py:86-107, :35-83).
 *
 * k_cache: [pages, H, head_dim / x, page_size, x], v_cache: [pages, H, head_dim,
 * page_size], both 2-byte elements, addressed through the element strides given
 * (kc_stride: pages, H, head_dim/x, page_size, x; vc_stride: pages, H, head_dim,
 * page_size).  Element (h, d) of token t with slot s goes to
 * k_cache[s / page_size, h, d / x, s % page_size, d % x] and
 * v_cache[s / page_size, h, d, s % page_size].
 */
int dfx_kv_store_distinct(const void* key, const void* value, int64_t key_stride, int64_t value_stride,
                          void* k_cache, void* v_cache, const int64_t kc_stride[5], const int64_t vc_stride[4],
                          const void* slot_mapping, int slot_index_type, int64_t n_tokens, int64_t n_pages,
                          int page_size, int x, int n_kv_heads, int head_dim, dfx_stream_t stream);

/*
 * Paged KV-cache load: gather every sequence's cached context through its block
 * table and append its fresh K/V rows, into packed [total, n_kv_heads, head_dim]
 * buffers of the cache's element type.
 * Replaces: load_kvcache + load_kvcache_kernel
 *           (diffulex_kernel/python/kv_cache_kernels.py:230-279, :127-227).
 *
 * Sequence s writes rows [cu_seqlens_k[s], cu_seqlens_k[s] + context_lens[s])
 * from pages block_tables[s, 0..], page p contributing min(page_size,
 * context - p * page_size) rows (a full last page IS copied, unlike the reference
 * kernel), then seq_lens_new[s] rows from k_new/v_new starting at row
 * cu_seqlens_q[s].  max_total_len bounds the rows of any one sequence (it sizes
 * the launch; larger sequences would be truncated, smaller values waste nothing).
 * Outputs are caller-allocated.  With DFX_KV_FP8_E4M3 the fresh rows (bf16) are
 * quantised with k_scale/v_scale as in dfx_kv_store_unified.
 */
int dfx_kv_load(const void* k_cache, const void* v_cache, const void* k_new, const void* v_new,
                int64_t k_new_stride, int64_t v_new_stride, void* k_out, void* v_out,
                const int32_t* block_tables, int64_t block_table_stride, const int32_t* context_lens,
                const int32_t* seq_lens_new, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                int num_seqs, int max_pages_per_seq, int64_t n_pages, int page_size, int n_kv_heads,
                int head_dim, int64_t max_total_len, int kv_dtype, const float* k_scale,
                const float* v_scale, dfx_stream_t stream);

/*
 * Block-diffusion paged attention.
 * Replaces: dllm_flash_attn_decode (both decode modes) and its TileLang kernels
 *           (diffulex_kernel/python/dllm_flash_attn.py:599-637, :163-347, :350-536),
 *           including the load_kvcache + flash_attn_varlen_func pair of the
 *           "varlen" mode, and, with k_cache == NULL, dllm_flash_attn_prefill
 *           (dllm_flash_attn.py:539-596, :23-160).
 *
 * For every sequence s, query rows q[cu_seqlens_q[s] .. cu_seqlens_q[s+1]) attend
 * to (a) the context_lens[s] cached tokens reached through block_tables[s, :]
 * and (b) the fresh rows k_new/v_new[cu_seqlens_new[s] .. cu_seqlens_new[s+1]),
 * masked by mask_mode (query i and fresh token j are indices inside the
 * sequence's own rows).  O = softmax(scale * Q K^T) V with fp32 accumulation,
 * GQA by kv_head = q_head / (num_q_heads / num_kv_heads).
 *
 * Supported: head_dim 64 or 128; num_q_heads a multiple of num_kv_heads; any
 * page_size >= 1; num_seqs <= 4095; scale > 0.  Strides are in elements; the
 * innermost (head_dim) dimension of q, k_new, v_new, out and the caches is dense
 * and every row start is 16-byte aligned.
 */
typedef struct dfx_attn_params {
    const void* q;               /* [T_q, num_q_heads, head_dim] bf16 */
    const void* k_new;           /* [T_new, num_kv_heads, head_dim] bf16 */
    const void* v_new;
    const void* k_cache;         /* [n_pages, page_size, num_kv_heads, head_dim]; NULL: no cached context */
    const void* v_cache;
    void* out;                   /* [T_q, num_q_heads, head_dim] bf16.  Rows of a sequence that has no key at all
                                    (no context, no fresh rows) are left unwritten, as the reference leaves
                                    them (dllm_flash_attn.py:343-345); a row whose keys are all on skipped
                                    pages gets zeros. */
    const int32_t* block_tables; /* [num_seqs, block_table_stride]; a page whose entry is < 0 (or >= n_pages) is
                                    skipped: its tokens take no part, as in the reference (dllm_flash_attn.py:260-261) */
    const int32_t* context_lens; /* [num_seqs]; NULL means 0 everywhere */
    const int32_t* cu_seqlens_q;   /* [num_seqs + 1] */
    const int32_t* cu_seqlens_new; /* [num_seqs + 1] offsets of the fresh K/V rows */
    const float* k_scale;        /* fp32 [num_kv_heads], DFX_KV_FP8_E4M3 only */
    const float* v_scale;
    void* workspace;             /* >= dfx_paged_attn_workspace_bytes(), 256-byte aligned, zero-filled
                                    once before its first use (every call leaves it ready for the next) */
    int64_t workspace_bytes;
    int64_t q_stride_token, q_stride_head;
    int64_t kn_stride_token, kn_stride_head; /* k_new */
    int64_t vn_stride_token, vn_stride_head; /* v_new */
    int64_t o_stride_token, o_stride_head;
    int64_t cache_stride_page, cache_stride_token, cache_stride_head; /* same for k_cache and v_cache */
    int64_t block_table_stride;
    int64_t n_pages;
    int32_t num_seqs, num_q_heads, num_kv_heads, head_dim;
    int32_t page_size, max_pages_per_seq;
    int32_t max_seqlen_q;        /* upper bound of any sequence's query rows */
    int32_t diffusion_block_size;
    int32_t kv_dtype;            /* dfx_kv_dtype of the caches (k_new/v_new are always bf16) */
    int32_t mask_mode;           /* dfx_mask_mode */
    int32_t max_workgroups;      /* 0: up to one (two for small row counts) per compute unit, fewer when the
                                    batch is small (chosen on the device from the lengths); >0: exactly this
                                    many persistent workgroups */
    int32_t flags;               /* DFX_ATTN_* bits, 0 by default */
    float scale;
    /* Fused KV-cache store (the store + decode pair of diffulex/attention/attn_impl.py:54-69 in
     * one launch).  NULL: attend only.  Otherwise [T_new] slots of type store_slot_index_type:
     * the launch also writes fresh row t of k_new / v_new to cache slot store_slot_mapping[t],
     * exactly as dfx_kv_store_unified would (negative and out-of-range slots skipped, FP8 caches
     * quantised with k_scale / v_scale), through the cache strides given above.  The slots
     * written must lie outside the context_lens[s] tokens any sequence attends to in this call
     * (true for the reference's runners, which store the block that follows the context):
     * other workgroups read those pages while this one writes.  The caches are written
     * through k_cache / v_cache although the pointers are declared const. */
    const void* store_slot_mapping;
    int32_t store_slot_index_type; /* dfx_index_type */
    /* Launch plan built by dfx_paged_attn_plan for this configuration (NULL: the kernel plans for
     * itself, as it also does if the plan was made for another configuration or its buffer was too
     * small for the batch). */
    const void* plan;
    int64_t plan_bytes;
    /* Rows of k_new / v_new (and entries of store_slot_mapping).  Fresh rows the offsets in
     * cu_seqlens_new point beyond it are neither attended nor stored (padded batches, e.g. the
     * reference's graph-capture metadata, carry such offsets).  0: unknown, the offsets are trusted;
     * required (> 0) with store_slot_mapping. */
    int64_t num_new_tokens;
    /* Layout of k_cache / v_cache.  DFX_CACHE_UNIFIED (0): [pages, page_size, H_kv, head_dim] through
     * cache_stride_*.  DFX_CACHE_DISTINCT: the layout dfx_kv_store_distinct writes, K [pages, H_kv,
     * head_dim / 8, page_size, 8] and V [pages, H_kv, head_dim, page_size], bf16, through the element
     * strides below (kc_stride[3] == 8, kc_stride[4] == 1, vc_stride[3] == 1, the others multiples of
     * 8; page_size a multiple of 8).  The reference stores into this layout
     * (diffulex_kernel/python/kv_cache_kernels.py:35-83) but its decode refuses it
     * (diffulex/attention/attn_impl.py:66-69); here it is decoded.  head_dim 128 with pages of a multiple
     * of 64 tokens (fresh K and V with one head stride, vc_stride[2] below 2^22) streams -- the K tile
     * chunk-major and the V tile d-major in LDS, as the layout has them, through the same pipelined step as
     * the unified layout -- and takes a plan; other shapes,
     * and DFX_ATTN_GENERIC_PATH, run the generic tile path, which takes none.  No fused store, no FP8, no
     * rotary embedding inside the launch with it.  What a page holds behind a sequence's end is never
     * used, whatever it is. */
    int32_t cache_layout;
    /* Rows of q and out.  No row at or beyond it is read or written, whatever cu_seqlens_q (or a plan
     * built from an earlier state of it) says.  0: unknown, the offsets are trusted. */
    int32_t num_q_tokens;
    int64_t kc_stride[5];
    int64_t vc_stride[4];
    /* Rotary position embedding inside the launch (NULL table: off; q and k_new are then used as they are).
     * Replaces: RotaryEmbedding.forward on the Q and K projections right before the attention layer
     *           (diffulex/model/dream.py:94-99, diffulex/layer/rotary_embedding.py:39-66), the launch
     *           dfx_rope_kv_store otherwise does.
     * q and k_new hold the projections as they leave the linear layer.  Row t of q and row t of k_new / v_new
     * are the same token (cu_seqlens_new equals cu_seqlens_q), at position rope_positions[t]; rope_cos_sin is
     * the table of dfx_rope_kv_store ([rope_max_position, head_dim] fp32: cosines, then sines).  The query rows
     * are rotated on their way into the matrix instructions and never written; the rotated fresh K rows go to
     * k_rotated ([T_new, num_kv_heads, head_dim] bf16, its own strides, NOT k_new itself: rows may be rotated
     * by more than one workgroup), which the launch reads back, and, with store_slot_mapping, into the cache
     * (FP8 caches: quantised after the rounding to bf16) next to the V rows.  Same bits as dfx_rope_kv_store
     * followed by this call without rope.  Only where the software-pipelined kernels run (head_dim 128, page
     * size a multiple of 16, more than 64 query rows per KV head and sequence or few items per compute unit,
     * a cache present): DFX_ERR_UNSUPPORTED otherwise -- run dfx_rope_kv_store first then. */
    const float* rope_cos_sin;
    const void* rope_positions;
    int32_t rope_position_index_type; /* dfx_index_type */
    int32_t reserved2;
    int64_t rope_max_position;
    void* k_rotated;
    int64_t kr_stride_token, kr_stride_head;
} dfx_attn_params;

/* Bytes of scratch dfx_paged_attn needs for these shapes.  It depends on the sizes (num_seqs, heads,
 * head_dim, max_seqlen_q), on max_workgroups (0: the current device's compute-unit count, doubled
 * for the small shapes that run two workgroups per compute unit), on flags, on kv_dtype and on
 * whether k_new and v_new share their head stride (which selects the tile path) -- never on device
 * data.  Negative: dfx_status.
 * The workspace starts with DFX_WORKSPACE_COUNTER_BYTES of arrival counters, which
 * the kernel expects to be zero and resets before it ends: zero-fill that area of a
 * new workspace once (hipMemsetAsync, or a fill kernel under graph capture).  Calls
 * that share a workspace must not overlap in time. */
#define DFX_WORKSPACE_COUNTER_BYTES (1 << 18)
int64_t dfx_paged_attn_workspace_bytes(const dfx_attn_params* params);

int dfx_paged_attn(const dfx_attn_params* params, dfx_stream_t stream);

/*
 * The launch plan of dfx_paged_attn, built once per decoding step and shared by the attention
 * launches of all layers.
 * Replaces: nothing on the device.  The reference builds its per-step attention metadata on the
 *           host (diffulex/strategy/d2f/engine/model_runner.py:244-261, :283-289) and every one of
 *           its kernel launches re-derives its work from it; here the partition of the batch over
 *           the workgroups, every tile's page address and the pieces of items shared between
 *           workgroups are worked out once, on the device, and the launches read them.
 *
 * A plan depends on the lengths (context_lens, cu_seqlens_q, cu_seqlens_new), the block tables, the
 * shapes, max_workgroups, flags and the strides of the caches and of k_new -- not on the base
 * pointers of q, k_new, v_new, out and the caches, nor on scale: the per-layer views of one cache
 * allocation share a plan.  The kernels recognise a plan made for other shapes, strides, flags or
 * metadata ADDRESSES and ignore it; they cannot see that the CONTENTS of the metadata arrays were
 * rewritten in place since: after such an update the caller builds the plan again (a stale plan
 * gives wrong rows, never an access outside the tensors as sized by n_pages, num_new_tokens and
 * num_q_tokens).  It is built on `stream` with no host synchronisation (safe to record
 * into a graph).  With at least 8 units and at most two items per workgroup the plan places the cut
 * points between the workgroups' ranges of the unit space by cost rather than by unit count (whole
 * sequences where they fit, no pieces of a few tiles: a sweep with the smallest capacity per
 * workgroup that works, which makes the plan kernel take about 30 us -- a plan is worth building
 * for several launches, not for one; the sweep runs over the sequences in the batch's order and with
 * the k-th longest followed by the k-th shortest, and keeps whichever order needs the smaller capacity);
 * DFX_ATTN_EQUAL_RANGES in flags keeps the equal ranges a launch without a plan uses (the results of
 * the two differ in the last bits: other pieces are merged).  DFX_ATTN_PAIRING in flags asks for the pairing partition where there are at most
 * as many (sequence, KV head, row tile) items as workgroups: every item gets a home workgroup and
 * only the excess of long items moves, which needs a third of the partial results that equal ranges
 * of the unit space need, at about the same speed.
 *
 * dfx_paged_attn_plan_bytes: bytes of plan buffer for up to max_units units (one unit = one
 * 64-token KV tile of one KV head of one row tile of one sequence; an upper bound is
 * num_kv_heads * row_tiles * (num_seqs * ceil(max_context / 64) + T_new / 64 + num_seqs)).  A buffer
 * too small for the batch at hand is detected on the device and the plan ignored.  Streaming-path
 * shapes only (page_size a multiple of 16, k_new and v_new laid out alike; FP8 with head_dim 128):
 * DFX_ERR_UNSUPPORTED otherwise.  The buffer must be 256-byte aligned.
 */
int64_t dfx_paged_attn_plan_bytes(const dfx_attn_params* params, int64_t max_units);
/* 0 if `stream` is not being captured into a graph, otherwise a positive number that identifies
 * the capture (-1: the runtime could not tell).  For callers that cache plans: a plan built
 * outside a capture, or inside another one, is not part of the graph being recorded and must be
 * built again inside it.  No counterpart in the reference. */
int64_t dfx_stream_capture_id(dfx_stream_t stream);
int dfx_paged_attn_plan(const dfx_attn_params* params, void* plan, int64_t plan_bytes, dfx_stream_t stream);

/*
 * Attention metadata of one decode step, built on the device.
 * Replaces: the Python loops of prepare_decode and the six host-to-device copies that follow them
 *           (diffulex/strategy/block_diffusion/engine/model_runner.py:114-173 with
 *           BDSequence.diffusion_decoding_inputs, block_diffusion/engine/sequence.py:186-191;
 *           diffulex/strategy/d2f/engine/model_runner.py:137-262 with
 *           D2FSequence.diffusion_decoding_inputs, d2f/engine/sequence.py:357-370), and the
 *           zero-fill-then-copy of the graph buffers in run_model
 *           (block_diffusion/engine/model_runner.py:176-197).  The layout CHECK_SLOT_MAPPING
 *           demands (diffulex/utils/checker.py:1-27) holds by construction.
 *
 * A sequence is described by what those loops read from it (all arrays on the device, so a
 * scheduler that keeps its state there needs no copy at all):
 *   DFX_META_BLOCK_DIFFUSION: num_tokens[s] = len(seq) after next_diffusion_step, block_state[s *
 *     block_state_stride] = state of its last diffusion block, num_pages[s] = len(seq.block_table).
 *     The step feeds the last diffusion_block_size tokens: context_lens[s] = num_tokens[s] - dbs,
 *     cu_seqlens_q and cu_seqlens_k advance by dbs; an ACTIVE block contributes dbs entries -1 to the
 *     slot mapping, a TO_CACHE block the slots of the last dbs / page_size pages of its table row
 *     (page by page, page_size slots each), an IN_CACHE block nothing.
 *   DFX_META_D2F: prompt_len[s] = seq.input_num_tokens (the size of diffusion block 0),
 *     num_diffusion_blocks[s] and block_state[s * block_state_stride + b] for each of its blocks, in
 *     the only order the reference's state machine produces: IN_CACHE* TO_CACHE* ACTIVE*, block 0 in the
 *     cache.  Blocks after the first have dbs tokens; num_tokens (optional) gives len(seq) where the
 *     last block is shorter.  The step feeds every block after the cached ones: context_lens[s] =
 *     cached tokens, cu_seqlens_q advances by len(seq) - cached, cu_seqlens_k by len(seq), seq_lens[s] =
 *     fed tokens; a token to be cached at position g of the sequence gets slot
 *     block_tables[s][g / page_size] * page_size + g % page_size, every token from the first active
 *     block on gets -1.
 * positions[i] (int64) = position in its sequence of the i-th fed token; input_ids[i] (optional) = the
 * token the sequence holds there.
 *
 * padded_seqs / padded_tokens (0: none): the output arrays are the buffers of a captured graph of
 * that batch size; entries beyond the step's own are set to 0, as the reference's run_model leaves
 * them (cu_seqlens_*[num_seqs + 1 .. padded_seqs], context_lens / seq_lens[num_seqs .. padded_seqs),
 * positions / slot_mapping up to padded_tokens).  Block-table rows are the caller's.
 *
 * summary[8] (int32, device; read it only if the host needs the numbers): fed tokens, slot-mapping
 * entries, max_seqlen_q, max_seqlen_k, need_kv_cache_store, 1 if token_capacity was too small
 * (nothing is written beyond it), 1 + index of the first sequence in a state the reference's loop
 * would raise on (such a sequence contributes nothing; 0: none), sum of cu_seqlens_k steps.
 *
 * One launch of one workgroup, no host synchronisation, no allocation; safe to capture.
 * DFX_ERR_UNSUPPORTED: more than 8192 sequences.
 */
typedef enum dfx_block_state { DFX_BLOCK_IN_CACHE = 0, DFX_BLOCK_TO_CACHE = 1, DFX_BLOCK_ACTIVE = 2 } dfx_block_state;
typedef enum dfx_meta_strategy { DFX_META_BLOCK_DIFFUSION = 0, DFX_META_D2F = 1 } dfx_meta_strategy;

typedef struct dfx_metadata_params {
    int32_t strategy; /* dfx_meta_strategy */
    int32_t num_seqs;
    int32_t page_size;            /* tokens per page (the reference's kvcache_block_size) */
    int32_t diffusion_block_size;
    /* inputs */
    const int32_t* num_tokens;           /* [num_seqs]; optional for D2F */
    const int32_t* prompt_len;           /* [num_seqs]; D2F only */
    const uint8_t* block_state;          /* dfx_block_state codes, see above */
    int64_t block_state_stride;          /* elements between sequences */
    const int32_t* num_diffusion_blocks; /* [num_seqs]; D2F only */
    const int32_t* block_tables;         /* [num_seqs, block_table_stride] page ids */
    int64_t block_table_stride;
    const int32_t* num_pages;            /* [num_seqs]; block diffusion only */
    /* outputs */
    int64_t* positions;    /* [token_capacity] */
    int32_t* slot_mapping; /* [token_capacity] */
    int64_t token_capacity;
    int32_t* cu_seqlens_q; /* [max(num_seqs, padded_seqs) + 1] */
    int32_t* cu_seqlens_k;
    int32_t* context_lens; /* [max(num_seqs, padded_seqs)] */
    int32_t* seq_lens;     /* the same size, or NULL */
    int32_t padded_seqs;
    int32_t reserved;
    int64_t padded_tokens;
    int32_t* summary; /* [8] */
    /* The step's token ids (both NULL: not wanted).  token_ids: the sequences' tokens as the scheduler
     * keeps them on the device, int64 [num_seqs, token_ids_stride], row s holding at least
     * len(sequence s) entries; input_ids [token_capacity] receives, for every fed token, the token at
     * its position of its sequence (the concatenation of cur_input_ids in the reference's loops:
     * block_diffusion/engine/model_runner.py:126-130, d2f/engine/model_runner.py:153-158), padded
     * with zeros up to padded_tokens. */
    const int64_t* token_ids;
    int64_t token_ids_stride;
    int64_t* input_ids;
} dfx_metadata_params;

int dfx_build_decode_metadata(const dfx_metadata_params* params, dfx_stream_t stream);

/*
 * dfx_paged_attn without a caller-provided workspace, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.
 *
 * Same arguments, results and kernels as dfx_paged_attn; params->workspace and
 * params->workspace_bytes are ignored.  The arrival counters and partial-result slots live in a
 * static device array of DFX_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held
 * until the process ends.  The call allocates and frees nothing.  Shapes for which
 * dfx_paged_attn_workspace_bytes() exceeds DFX_STATIC_SCRATCH_BYTES are refused with
 * DFX_ERR_SCRATCH_LIMIT (lower max_workgroups, or use dfx_paged_attn).  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (two streams, two threads)
 * race, as calls of dfx_paged_attn that share a workspace do.
 */
#define DFX_STATIC_SCRATCH_BYTES (40u << 20)
int dfx_paged_attn_static(const dfx_attn_params* params, dfx_stream_t stream);

/*
 * Rotary position embedding of the fresh Q and K rows, optionally fused with the
 * unified-layout KV-cache store of the rotated K and of V.
 * Replaces: RotaryEmbedding.forward + apply_rotary_emb
 *           (diffulex/layer/rotary_embedding.py:39-66, :7-17), called on the
 *           projections right before the attention layer
 *           (diffulex/model/dream.py:94-99), and, with slot_mapping != NULL, the
 *           store_kvcache_unified_layout launch that follows it
 *           (diffulex/attention/attn_impl.py:54-57).
 *
 * For token t with p = positions[t], head h and i < head_dim / 2:
 *   c = cos_sin_cache[p, i], s = cos_sin_cache[p, head_dim / 2 + i]
 *   out[t, h, i]                = bf16(x[t, h, i] * c - x[t, h, head_dim / 2 + i] * s)
 *   out[t, h, head_dim / 2 + i] = bf16(x[t, h, head_dim / 2 + i] * c + x[t, h, i] * s)
 * in fp32 with every product and sum rounded separately (no fused multiply-add),
 * then rounded to nearest even: the bits of the reference's eager evaluation.
 * q_out / k_out may be q / k (in place) or separate buffers.  Positions outside
 * [0, max_position) are a caller error (clamped, so nothing is read out of bounds).
 *
 * slot_mapping != NULL: token t's rotated K row and its V row also go to cache
 * slot slot_mapping[t] exactly as dfx_kv_store_unified would put them (slots < 0
 * or >= n_slots skipped; FP8 caches quantise the bf16-rounded rotated K).
 * slot_mapping == NULL: v, k_cache, v_cache, k_scale, v_scale must be NULL.
 *
 * Supported: head_dim a multiple of 16; heads dense inside a token row; strides
 * (elements) multiples of 8; every pointer 16-byte aligned.
 */
typedef struct dfx_rope_params {
    const void* q;      /* [n_tokens, num_q_heads, head_dim] bf16 */
    const void* k;      /* [n_tokens, num_kv_heads, head_dim] bf16 */
    const void* v;      /* [n_tokens, num_kv_heads, head_dim] bf16, read only for the store */
    void* q_out;        /* rotated q */
    void* k_out;        /* rotated k */
    int64_t q_stride_token, k_stride_token, v_stride_token;
    int64_t q_out_stride_token, k_out_stride_token;
    const void* positions; /* [n_tokens] */
    int32_t position_index_type; /* dfx_index_type */
    const float* cos_sin_cache;  /* [max_position, head_dim] fp32: cosines, then sines */
    int64_t max_position;
    int64_t n_tokens;
    int32_t num_q_heads, num_kv_heads, head_dim;
    int32_t kv_dtype;            /* dfx_kv_dtype of the caches */
    void* k_cache;               /* [n_slots, num_kv_heads, head_dim] dense */
    void* v_cache;
    const void* slot_mapping;    /* [n_tokens] or NULL */
    int32_t slot_index_type;     /* dfx_index_type */
    int64_t n_slots;
    const float* k_scale;        /* fp32[num_kv_heads], FP8 caches only */
    const float* v_scale;
    /* Layout of the caches the store writes.  DFX_CACHE_UNIFIED (0): as above.  DFX_CACHE_DISTINCT: what
     * dfx_kv_store_distinct writes with x == 8 -- K [pages, num_kv_heads, head_dim / 8, page_size, 8] and
     * V [pages, num_kv_heads, head_dim, page_size], bf16 -- through the element strides of their first three
     * dimensions (multiples of 8; tokens of a page 8 elements apart in K, dense in V); slot s is token
     * s % page_size of page s / page_size, n_slots = pages * page_size. */
    int32_t cache_layout;
    int32_t page_size;
    int64_t kc_stride[3];
    int64_t vc_stride[3];
} dfx_rope_params;

int dfx_rope_kv_store(const dfx_rope_params* params, dfx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* DIFFULEX_AMD_H_ */
