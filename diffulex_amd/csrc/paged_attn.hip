// Block-diffusion paged attention for gfx950 (MI355X): kernel dispatch and C entry points.
//
// One persistent workgroup (4 wavefronts) per compute unit walks an equal share of the linear
// work list described in partition.h.  For one (sequence, KV head, row tile) item the
// workgroup holds every query row that shares the KV head -- all G = H_q / H_kv heads of
// every query token, up to 128*NB rows -- so each K/V tile is fetched from HBM once per KV
// head and reused by the whole GQA group.  Two tile paths feed the same MFMA / online-softmax
// core (attn_tile.h): the streaming path (attn_stream.h: direct-to-LDS loads in a 4-stage
// ring; page sizes that are multiples of 16; bf16 KV, or FP8-E4M3 KV with head_dim 128) and
// the generic path (attn_generic.h: any page size, any layout of the fresh K/V).
#include <atomic>
#include <mutex>

#include "attn_common.h"
#include "attn_generic.h"
#include "attn_stream.h"
#include "plan.h"

// Scratch of dfx_paged_attn_static: the arrival counters and partial-result slots that
// dfx_paged_attn takes from its caller, for callers that cannot allocate device memory.  Every
// GPU the library runs on holds its own copy until the process ends.  The name is a host-side
// stand-in for the symbol; its device address comes from hipGetSymbolAddress (static_scratch()).
static __device__ __align__(256) unsigned char scratch[DFX_STATIC_SCRATCH_BYTES];

namespace dfx {
namespace {

constexpr int kMaxWorkgroups = 65535;

struct Plan {
    int hd, nb, n_wg;
    bool fp8;
    bool stream;   // streaming tile path (else generic)
    bool distinct; // the cache is in the "distinct" layout (streaming path where its kernel serves the shape, else generic)
    bool compact;  // streaming path, two workgroups per compute unit
    bool pipelined;  // streaming path, 8 waves, 4-stage ring: software-pipelined tile step
    int64_t slot_floats;
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
    // The streaming path addresses a cached K row and its V row with one offset: page size a
    // multiple of 16; fresh K and V may differ in their token stride, not in their head stride.

    plan.distinct = p->cache_layout == DFX_CACHE_DISTINCT && p->k_cache != nullptr;
    if (p->cache_layout != DFX_CACHE_UNIFIED && p->cache_layout != DFX_CACHE_DISTINCT) return DFX_ERR_INVALID_ARG;
    if (plan.distinct && plan.fp8) return DFX_ERR_UNSUPPORTED;
    plan.stream = !(p->flags & DFX_ATTN_GENERIC_PATH) && !plan.distinct &&
                  (p->k_cache == nullptr || (p->page_size > 0 && p->page_size % 16 == 0)) &&
                  (p->rope_cos_sin != nullptr ? p->kr_stride_head : p->kn_stride_head) == p->vn_stride_head;
    // The distinct layout on the streaming path: head_dim 128, a tile inside one page, the 16-byte chunks the
    // loads move (x == 8, tokens dense in V), offsets inside a (page, head) in 32 bits; one kernel, 8 waves.
    const bool dstream = plan.distinct && !(p->flags & DFX_ATTN_GENERIC_PATH) && plan.hd == 128 && p->page_size > 0 &&
                         p->page_size % 64 == 0 && p->page_size < (1 << 20) && p->kn_stride_head == p->vn_stride_head &&
                         p->kc_stride[4] == 1 && p->kc_stride[3] == 8 && p->vc_stride[3] == 1 &&
                         p->vc_stride[2] >= 0 && p->vc_stride[2] < (1 << 22) && p->rope_cos_sin == nullptr &&
                         p->num_kv_heads < (1 << 12) && p->n_pages < (1ll << 32);  // (what a tile's descriptor packs)
    if (dstream) {
        plan.stream = true;
        plan.nb = 2;
    }
    // head_dim 128, 65..128 rows: the 8-wave pipelined kernels (their waves without rows only fetch) are
    // faster than 4 waves with a compiler-scheduled step, with or without a second workgroup on the
    // compute unit (C4 -7 %, 112 or 128 rows at the C3 shape -18 %).  Fewer rows: the same (64 or 48 rows
    // at the C3 shape -17 %, 32 rows -1 to -15 %) while a workgroup has few items to open and close; with
    // four short items each the two workgroups per compute unit are ahead (64 rows: by 22 %, 32 rows: by
    // 7 %), and a launch cannot see lengths.
    // (head_dim 64, whose tiles are half the bytes and the matrix work: 4 waves, two workgroups per compute unit, stay
    // ahead up to the 128 rows they can hold -- 96 rows of the C4 kind: 150 us against 169 -- and the 8-wave pipelined
    // kernel takes over from 129 rows on: 224 rows of the C3 kind 42.4 us against 47.3)
    if (plan.stream && plan.hd == 128 && !(p->flags & DFX_ATTN_NO_PIPELINE)) {
        const int64_t items = static_cast<int64_t>(p->num_seqs) * p->num_kv_heads;
        if (rows > 64 || items <= 2 * static_cast<int64_t>(device_cu_count())) plan.nb = 2;
    }
    plan.compact = plan.stream && !plan.fp8 && plan.nb == 1 && p->num_seqs <= kCompactMaxSeqs;

    // (8 waves only: with 4 waves a wave has twice the tile loads to address, and the 32 registers
    // the pipelined kernel leaves the compiler no longer hold that without spilling in the loop)
    plan.pipelined = plan.stream && !plan.compact && (plan.hd == 128 || !plan.fp8) && plan.nb == 2 &&
                     !(p->flags & DFX_ATTN_NO_PIPELINE);
    if (p->max_workgroups > 0) {
        plan.n_wg = p->max_workgroups;
    } else {
        plan.n_wg = device_cu_count();
        if (plan.n_wg <= 0) return DFX_ERR_LAUNCH;
        if (plan.compact) plan.n_wg *= 2;
    }
    if (plan.n_wg > kMaxWorkgroups) return DFX_ERR_INVALID_ARG;
    if (plan.hd == 64) plan.slot_floats = plan.nb == 1 ? Shape<64, 1>::SLOT_FLOATS : Shape<64, 2>::SLOT_FLOATS;
    else plan.slot_floats = plan.nb == 1 ? Shape<128, 1>::SLOT_FLOATS : Shape<128, 2>::SLOT_FLOATS;
    return DFX_OK;
}

// Workspace layout: arrival counters (one int per workgroup), then two partial-result slots per
// workgroup.  The counter area has the same size whatever the launch (room for the largest
// grid): calls with different workgroup counts may share a workspace, and the counters must
// never land where an earlier call left partial results.
static_assert((kMaxWorkgroups + 1) * 4 == DFX_WORKSPACE_COUNTER_BYTES, "one counter per workgroup of the largest grid");
int64_t counter_bytes(const Plan&) { return DFX_WORKSPACE_COUNTER_BYTES; }
int64_t plan_workspace_bytes(const Plan& plan) {
    return counter_bytes(plan) + 2 * static_cast<int64_t>(plan.n_wg) * plan.slot_floats * 4;
}

// Raising a kernel's dynamic LDS limit is idempotent but not free: done once per device and kernel.
bool ensure_lds_limit(const void* kernel, int slot, int lds) {
    static std::atomic<uint64_t> configured[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    const uint64_t bit = 1ull << slot;
    if (configured[dev].load(std::memory_order_acquire) & bit) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return false;
    configured[dev].fetch_or(bit, std::memory_order_release);
    return true;
}

// PATH: 0 generic bf16, 1 generic FP8, 2 streaming bf16, 3 streaming FP8, 4 generic bf16 on a distinct-layout cache,
// 5 streaming bf16 on a distinct-layout cache.
// pa == nullptr: the attention launch.  Otherwise the two plan kernels for that launch (streaming
// paths only).
template <int HD, int NB, int PATH>
int launch(const KArgs& ka, const Plan& plan, hipStream_t st, const PlanArgs* pa) {
    void (*main_k)(const KArgs);
    void (*plan_k)(const KArgs, const PlanArgs) = nullptr;
    void (*fill_k)(const KArgs, const PlanArgs) = nullptr;
    int lds, threads = kThreads, fill_lds = 0, slot;
    int plan_slot = 30;  // (the plan kernel exists for row tiles of 128 and of 256 rows)
    constexpr int NW = 4 * NB;  // streaming paths: one 32-row query block per wave
    constexpr int kSlotBase = (HD == 128 ? 0 : 8) + (NB == 1 ? 0 : 4);
    if constexpr (PATH == 3) {
        // head_dim 128: one query block per wave, 4 or 8 waves; head_dim 64: 4 waves of 1 or 2 blocks
        constexpr int FNB = HD == 128 ? 1 : NB, FNW = HD == 128 ? NW : 4;
        main_k = paged_attn_stream_fp8_kernel<HD, FNB, FNW>;
        using C = StreamCfg<HD, FNB, FNW, false, 1>;
        lds = C::LDS_BYTES;
        plan_k = paged_attn_plan_kernel<C::RT>;
            plan_slot = C::RT == 256 ? 31 : 30;
        fill_k = paged_attn_plan_fill_kernel<HD, FNB, FNW, false, 1>;
        fill_lds = C::STAGES_OFF;
        threads = 64 * FNW;
        slot = kSlotBase + 3;
        if constexpr (HD == 128 && FNW == 8) {
            if (plan.pipelined) {
                main_k = paged_attn_pipe_fp8_kernel<FNW>;
                slot = 28;
            }
        }
    } else if constexpr (PATH == 2) {
        // 4 waves for up to 128 rows (then two workgroups per compute unit where the batch allows),
        // 8 waves (two per SIMD) for up to 256
        if (NB == 1 && plan.compact) {
            using C = StreamCfg<HD, 1, 4, true>;
            main_k = paged_attn_stream_kernel<HD, 1, 4, true>;
            lds = C::LDS_BYTES;
            plan_k = paged_attn_plan_kernel<C::RT>;
            plan_slot = C::RT == 256 ? 31 : 30;
            fill_k = paged_attn_plan_fill_kernel<HD, 1, 4, true, 2>;
            fill_lds = C::STAGES_OFF;
            slot = kSlotBase + 1;
        } else {
            using C = StreamCfg<HD, 1, NW, false>;
            main_k = paged_attn_stream_kernel<HD, 1, NW, false>;
            slot = kSlotBase + 0;
            if constexpr (HD == 128 && NW == 8) {
                if (plan.pipelined) {
                    main_k = paged_attn_pipe_kernel<NW>;
                    slot = kSlotBase + 2;
                    // no cache: the variant whose plain steps fetch fresh rows
                    if (ka.k_cache == nullptr) {
                        main_k = paged_attn_pipe_kernel<NW, true>;
                        slot = 29;
                    }
                }
            }
            if constexpr (HD == 64 && NW == 8) {
                if (plan.pipelined) {
                    main_k = paged_attn_pipe_kernel<NW, false, false, 64>;
                    slot = 34;
                }
            }
            lds = C::LDS_BYTES;
            plan_k = paged_attn_plan_kernel<C::RT>;
            plan_slot = C::RT == 256 ? 31 : 30;
            fill_k = paged_attn_plan_fill_kernel<HD, 1, NW, false, 2>;
            fill_lds = C::STAGES_OFF;
        }
        threads = 64 * NW;
    } else if constexpr (PATH == 5) {
        static_assert(HD == 128 && NB == 2, "the distinct layout's streaming kernel");
        using C = StreamCfg<HD, 1, NW, false>;
        main_k = paged_attn_stream_kernel<HD, 1, NW, false, true>;
        slot = 32;
        if (plan.pipelined) {
            main_k = paged_attn_pipe_kernel<NW, false, true>;
            slot = 33;
        }
        lds = C::LDS_BYTES;
        plan_k = paged_attn_plan_kernel<C::RT>;
        plan_slot = C::RT == 256 ? 31 : 30;
        fill_k = paged_attn_plan_fill_kernel<HD, 1, NW, false, 2, true>;
        fill_lds = C::STAGES_OFF;
        threads = 64 * NW;
    } else if constexpr (PATH == 4) {
        main_k = paged_attn_generic_kernel<HD, NB, false, true>;
        lds = GenericCfg<HD, NB>::LDS_BYTES;
        slot = 24 + kSlotBase / 4;
    } else {
        main_k = paged_attn_generic_kernel<HD, NB, PATH == 1>;
        lds = GenericCfg<HD, NB>::LDS_BYTES;
        slot = 16 + kSlotBase / 4 * 2 + PATH;
    }
    if (pa != nullptr) {
        if (plan_k == nullptr) return DFX_ERR_UNSUPPORTED;
        if (!ensure_lds_limit(reinterpret_cast<const void*>(plan_k), plan_slot, kPlanKernelLdsBytes)) return DFX_ERR_LAUNCH;
        hipLaunchKernelGGL(plan_k, dim3(1), dim3(512), kPlanKernelLdsBytes, st, ka, *pa);
        hipLaunchKernelGGL(fill_k, dim3(plan.n_wg), dim3(threads), fill_lds, st, ka, *pa);
        return hipGetLastError() == hipSuccess ? DFX_OK : DFX_ERR_LAUNCH;
    }
    if (!ensure_lds_limit(reinterpret_cast<const void*>(main_k), slot, lds)) return DFX_ERR_LAUNCH;
    hipLaunchKernelGGL(main_k, dim3(plan.n_wg), dim3(threads), lds, st, ka);
    if (hipGetLastError() != hipSuccess) return DFX_ERR_LAUNCH;
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

namespace {

// Argument checks shared by the entry points (everything but the workspace).  `empty`: the call is
// valid and there is nothing to launch.
int check_args(const dfx_attn_params* p, Plan& plan, bool& empty) {
    empty = false;
    const int rc = make_plan(p, plan);
    if (rc != DFX_OK) return rc;
    // no query rows, no launch: a store asked for with such a call would be skipped silently
    if (p->store_slot_mapping != nullptr && p->num_seqs > 0 && p->max_seqlen_q == 0) return DFX_ERR_INVALID_ARG;
    if (p->num_seqs == 0 || p->max_seqlen_q == 0) {
        empty = true;
        return DFX_OK;
    }
    if (!p->q || !p->k_new || !p->v_new || !p->out || !p->cu_seqlens_q || !p->cu_seqlens_new)
        return DFX_ERR_INVALID_ARG;
    const bool has_cache = p->k_cache != nullptr;
    if (has_cache != (p->v_cache != nullptr)) return DFX_ERR_INVALID_ARG;
    if (has_cache && (!p->block_tables || p->page_size <= 0 || p->max_pages_per_seq < 0 || p->n_pages < 0))
        return DFX_ERR_INVALID_ARG;
    if (plan.fp8 && (!p->k_scale || !p->v_scale)) return DFX_ERR_INVALID_ARG;
    if (p->num_new_tokens < 0 || p->num_q_tokens < 0) return DFX_ERR_INVALID_ARG;
    if (p->store_slot_mapping != nullptr) {
        if (!has_cache || p->num_new_tokens <= 0) return DFX_ERR_INVALID_ARG;  // the store needs the row count
        if (p->store_slot_index_type != DFX_INDEX_I32 && p->store_slot_index_type != DFX_INDEX_I64)
            return DFX_ERR_INVALID_ARG;
    }
    if (!(p->scale > 0.0f) || p->diffusion_block_size <= 0) return DFX_ERR_INVALID_ARG;
    if (p->mask_mode != DFX_MASK_FULL && p->mask_mode != DFX_MASK_BLOCK_CAUSAL) return DFX_ERR_INVALID_ARG;
    if (p->rope_cos_sin != nullptr) {
        if (!plan.pipelined || !has_cache || plan.distinct || plan.hd != 128) return DFX_ERR_UNSUPPORTED;
        if (!p->rope_positions || !p->k_rotated || p->rope_max_position <= 0 || p->k_rotated == p->k_new) return DFX_ERR_INVALID_ARG;
        if (p->rope_position_index_type != DFX_INDEX_I32 && p->rope_position_index_type != DFX_INDEX_I64) return DFX_ERR_INVALID_ARG;
        if (p->kr_stride_token < 0 || p->kr_stride_token % 8 || p->kr_stride_head < 0 || p->kr_stride_head % 8) return DFX_ERR_INVALID_ARG;
        if (!aligned16(p->rope_cos_sin) || !aligned16(p->k_rotated)) return DFX_ERR_INVALID_ARG;
    }
    const int64_t strides8[] = {p->q_stride_token,  p->q_stride_head,   p->kn_stride_token, p->kn_stride_head,
                                p->vn_stride_token, p->vn_stride_head};
    for (int64_t v : strides8)
        if (v < 0 || v % 8 != 0) return DFX_ERR_INVALID_ARG;
    if (p->o_stride_token % 4 != 0 || p->o_stride_head % 4 != 0) return DFX_ERR_INVALID_ARG;
    if (!aligned16(p->q) || !aligned16(p->k_new) || !aligned16(p->v_new) || !aligned16(p->out))
        return DFX_ERR_INVALID_ARG;
    if (plan.distinct) {
        // 16-byte loads: x == 8 two-byte elements, tokens dense in V, everything else a multiple of 8
        if (p->kc_stride[4] != 1 || p->kc_stride[3] != 8 || p->vc_stride[3] != 1) return DFX_ERR_UNSUPPORTED;
        if (p->page_size % 8 != 0) return DFX_ERR_UNSUPPORTED;
        for (int i = 0; i < 3; ++i)
            if (p->kc_stride[i] < 0 || p->kc_stride[i] % 8 || p->vc_stride[i] < 0 || p->vc_stride[i] % 8) return DFX_ERR_INVALID_ARG;
        if (p->store_slot_mapping != nullptr) return DFX_ERR_UNSUPPORTED;  // dfx_kv_store_distinct stores into this layout
        if (!aligned16(p->k_cache) || !aligned16(p->v_cache)) return DFX_ERR_INVALID_ARG;
    } else if (has_cache) {
        const int64_t gran = plan.fp8 ? 16 : 8;
        if (p->cache_stride_page % gran || p->cache_stride_token % gran || p->cache_stride_head % gran)
            return DFX_ERR_INVALID_ARG;
        if (!aligned16(p->k_cache) || !aligned16(p->v_cache)) return DFX_ERR_INVALID_ARG;
    }
    return DFX_OK;
}

// Checks and launch; `workspace` replaces p->workspace.
// The launch configuration a plan depends on (everything but the tensors' base pointers, the
// scale and the store): a plan made for another configuration is ignored by the kernels.
uint32_t plan_signature(const dfx_attn_params* p, const Plan& plan) {
    uint64_t h = 1469598103934665603ull;
    auto mix = [&](uint64_t v) {
        for (int i = 0; i < 8; ++i) {
            h ^= (v >> (8 * i)) & 0xffu;
            h *= 1099511628211ull;
        }
    };
    mix(plan.hd); mix(plan.nb); mix(plan.n_wg); mix(plan.fp8); mix(plan.stream); mix(plan.compact);
    mix(p->num_seqs); mix(p->num_q_heads); mix(p->num_kv_heads); mix(p->page_size); mix(p->max_pages_per_seq);
    mix(p->max_seqlen_q); mix(p->num_new_tokens); mix(p->diffusion_block_size); mix(p->mask_mode); mix(p->max_workgroups);
    // (the fresh K rows the tiles are made of: with the rotary embedding inside the launch, the rotated copy)
    const bool rope = p->rope_cos_sin != nullptr;
    mix(rope ? p->kr_stride_token : p->kn_stride_token); mix(rope ? p->kr_stride_head : p->kn_stride_head); mix(p->vn_stride_token); mix(p->cache_stride_page); mix(p->cache_stride_token);
    mix(p->cache_stride_head); mix(p->block_table_stride); mix(p->n_pages); mix(p->k_cache != nullptr);
    mix(reinterpret_cast<uintptr_t>(p->block_tables)); mix(reinterpret_cast<uintptr_t>(p->context_lens));
    mix(reinterpret_cast<uintptr_t>(p->cu_seqlens_q)); mix(reinterpret_cast<uintptr_t>(p->cu_seqlens_new));
    mix(static_cast<uint32_t>(p->flags)); mix(plan.pipelined);
    if (plan.distinct) {
        mix(1);
        for (int i = 0; i < 3; ++i) { mix(p->kc_stride[i]); mix(p->vc_stride[i]); }
    }
    const uint32_t sig = static_cast<uint32_t>(h ^ (h >> 32));
    return sig == 0 ? 1u : sig;
}

int plan_waves(const Plan& plan) { return (plan.compact || (plan.fp8 && plan.hd == 64)) ? 4 : 4 * plan.nb; }

// Unit descriptors a plan buffer of `bytes` has room for behind its fixed part.
int64_t plan_capacity(int64_t bytes, const PlanLayout& fixed, int waves) {
    const int64_t per_unit = static_cast<int64_t>(sizeof(UnitDesc)) + waves * static_cast<int64_t>(sizeof(BandDesc));
    const int64_t n = (bytes - fixed.bytes) / per_unit;
    return n > 0x7fffffff ? 0x7fffffff : n;
}

// Checks and launch; `workspace` replaces p->workspace.  plan_out != nullptr: instead of the
// attention launch, build its plan into plan_out (plan_bytes of room).
int run_paged_attn(const dfx_attn_params* p, void* workspace, int64_t workspace_bytes, dfx_stream_t stream,
                   void* plan_out = nullptr, int64_t plan_bytes = 0) {
    Plan plan;
    bool empty;
    const int rc = check_args(p, plan, empty);
    if (rc != DFX_OK || empty) return rc;
    const bool has_cache = p->k_cache != nullptr;
    const int64_t need = plan_workspace_bytes(plan);
    if (plan_out == nullptr && plan.n_wg > 1 &&
        (workspace == nullptr || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0))
        return DFX_ERR_WORKSPACE;
    PlanArgs pa;
    if (plan_out != nullptr) {
        if (!plan.stream) return DFX_ERR_UNSUPPORTED;
        if ((reinterpret_cast<uintptr_t>(plan_out) & 255u) != 0) return DFX_ERR_INVALID_ARG;
        const PlanLayout fixed = plan_layout(p->num_seqs, plan.n_wg, 0, plan_waves(plan));
        if (plan_bytes < fixed.bytes) return DFX_ERR_WORKSPACE;
        pa.buf = static_cast<uint8_t*>(plan_out);
        pa.capacity = plan_capacity(plan_bytes, fixed, plan_waves(plan));
        pa.n_wg = plan.n_wg;
        pa.waves = plan_waves(plan);
        pa.signature = plan_signature(p, plan);
        pa.allow_pairing = (p->flags & DFX_ATTN_PAIRING) ? 1 : 0;
        pa.equal_ranges = (p->flags & DFX_ATTN_EQUAL_RANGES) ? 1 : 0;
        pa.batch_order = (p->flags & DFX_ATTN_BATCH_ORDER) ? 1 : 0;
    }

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
    ka.store_slots = has_cache ? p->store_slot_mapping : nullptr;
    ka.store_slots_i64 = p->store_slot_index_type == DFX_INDEX_I64;
    ka.arrivals = static_cast<int*>(workspace);
    ka.workspace = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + counter_bytes(plan));
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
    ka.kd_sp = p->kc_stride[0]; ka.kd_sh = p->kc_stride[1]; ka.kd_sc = p->kc_stride[2];
    ka.vd_sp = p->vc_stride[0]; ka.vd_sh = p->vc_stride[1]; ka.vd_sd = p->vc_stride[2];
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
    ka.fixed_wg = p->max_workgroups > 0;
    {
        const int64_t rows = static_cast<int64_t>(ka.group) * p->max_seqlen_q;
        ka.busy_waves = static_cast<int>(rows >= 32 * kMaxWaves ? kMaxWaves : (rows + 31) / 32);
    }
    ka.c = p->scale * kLog2e;
    ka.n_new = p->num_new_tokens > 0 ? p->num_new_tokens : INT64_MAX;
    ka.n_q = p->num_q_tokens > 0 ? p->num_q_tokens : INT32_MAX;
    ka.rope_table = p->rope_cos_sin;
    ka.rope_pos = p->rope_positions;
    ka.rope_pos_i64 = p->rope_position_index_type == DFX_INDEX_I64;
    ka.rope_max_pos = p->rope_max_position;
    ka.k_src = nullptr;
    ka.ks_st = ka.ks_sh = 0;
    if (p->rope_cos_sin != nullptr) {
        // the tiles of fresh K rows are read from where the launch puts the rotated rows
        ka.k_src = ka.k_new;
        ka.ks_st = ka.kn_st;
        ka.ks_sh = ka.kn_sh;
        ka.k_new = static_cast<const uint16_t*>(p->k_rotated);
        ka.kn_st = p->kr_stride_token;
        ka.kn_sh = p->kr_stride_head;
    }
    ka.v_fresh_delta = (p->vn_stride_token - ka.kn_st) * 2;
    ka.plan = nullptr;
    ka.plan_capacity = 0;
    ka.plan_signature = plan_signature(p, plan);
    if (plan_out == nullptr && plan.stream && p->plan != nullptr) {
        const PlanLayout fixed = plan_layout(p->num_seqs, plan.n_wg, 0, plan_waves(plan));
        if (p->plan_bytes < fixed.bytes || (reinterpret_cast<uintptr_t>(p->plan) & 255u) != 0) return DFX_ERR_INVALID_ARG;
        ka.plan = static_cast<const uint8_t*>(p->plan);
        // where the plan's tables start follows from the buffer's size: the same size as when it was built, or the
        // kernel finds another capacity in the header and plans for itself
        ka.plan_capacity = static_cast<int32_t>(plan_capacity(p->plan_bytes, fixed, plan_waves(plan)));
    }

    hipStream_t st = static_cast<hipStream_t>(stream);
    const PlanArgs* pap = plan_out != nullptr ? &pa : nullptr;
#define DFX_ATTN_CASE(HD_, NB_)                                               \
    if (plan.hd == HD_ && plan.nb == NB_) {                                   \
        if (plan.stream && plan.fp8) return launch<HD_, NB_, 3>(ka, plan, st, pap); \
        if (plan.stream && !plan.distinct) return launch<HD_, NB_, 2>(ka, plan, st, pap); \
        if (plan.distinct) return launch<HD_, NB_, 4>(ka, plan, st, pap);     \
        if (plan.fp8) return launch<HD_, NB_, 1>(ka, plan, st, pap);          \
        return launch<HD_, NB_, 0>(ka, plan, st, pap);                        \
    }
    if (plan.stream && plan.distinct) return launch<128, 2, 5>(ka, plan, st, pap);
    DFX_ATTN_CASE(64, 1)
    DFX_ATTN_CASE(64, 2)
    DFX_ATTN_CASE(128, 1)
    DFX_ATTN_CASE(128, 2)
#undef DFX_ATTN_CASE
    return DFX_ERR_UNSUPPORTED;
}

}  // namespace

namespace {

__global__ void zero_words_kernel(int* p, int n) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = 0;
}

struct StaticScratch {
    void* ptr = nullptr;   // device address of this device's copy of `scratch`
    bool zeroed = false;   // an executed (not merely captured) launch has cleared the counters
};

// Address of the current device's scratch array, looked up once per device.
int static_scratch(StaticScratch*& out) {
    constexpr int kMaxDevices = 64;
    static StaticScratch table[kMaxDevices];
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return DFX_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(mu);
    if (table[dev].ptr == nullptr) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return DFX_ERR_LAUNCH;
        table[dev].ptr = ptr;
    }
    out = &table[dev];
    return DFX_OK;
}

}  // namespace

extern "C" int dfx_paged_attn_static(const dfx_attn_params* p, dfx_stream_t stream) {
    Plan plan;
    bool empty;
    const int rc = check_args(p, plan, empty);
    if (rc != DFX_OK || empty) return rc;
    if (plan_workspace_bytes(plan) > static_cast<int64_t>(DFX_STATIC_SCRATCH_BYTES)) return DFX_ERR_SCRATCH_LIMIT;
    StaticScratch* sc = nullptr;
    const int rs = static_scratch(sc);
    if (rs != DFX_OK) return rs;
    // The arrival counters must be zero when a launch starts; every launch leaves them zero.  The
    // first launch on a device clears them with a fill kernel (never a memset: this call may be
    // recorded into a graph).  A launch that is only captured has not run, so captures keep
    // recording the fill until an eager launch has executed it.
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess) return DFX_ERR_LAUNCH;
    bool fill;
    {
        static std::mutex mu;
        std::lock_guard<std::mutex> lock(mu);
        fill = !sc->zeroed;
        if (fill && cap == hipStreamCaptureStatusNone) sc->zeroed = true;
    }
    if (fill) {
        const int n = static_cast<int>(counter_bytes(plan) / 4);
        hipLaunchKernelGGL(zero_words_kernel, dim3(64), dim3(256), 0, st, static_cast<int*>(sc->ptr), n);
        if (hipGetLastError() != hipSuccess) return DFX_ERR_LAUNCH;
    }
    return run_paged_attn(p, sc->ptr, static_cast<int64_t>(DFX_STATIC_SCRATCH_BYTES), stream);
}

extern "C" int64_t dfx_stream_capture_id(dfx_stream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    if (hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &status, &id) != hipSuccess) return -1;
    return status == hipStreamCaptureStatusActive ? static_cast<int64_t>(id) + 1 : 0;
}

extern "C" int64_t dfx_paged_attn_plan_bytes(const dfx_attn_params* p, int64_t max_units) {
    Plan plan;
    const int rc = make_plan(p, plan);
    if (rc != DFX_OK) return rc;
    if (!plan.stream) return DFX_ERR_UNSUPPORTED;
    if (max_units < 0) return DFX_ERR_INVALID_ARG;
    return plan_layout(p->num_seqs, plan.n_wg, max_units, plan_waves(plan)).bytes;
}

extern "C" int dfx_paged_attn_plan(const dfx_attn_params* p, void* plan_buf, int64_t plan_bytes, dfx_stream_t stream) {
    if (p == nullptr || plan_buf == nullptr) return DFX_ERR_INVALID_ARG;
    return run_paged_attn(p, nullptr, 0, stream, plan_buf, plan_bytes);
}

extern "C" int dfx_paged_attn(const dfx_attn_params* p, dfx_stream_t stream) {
    if (p == nullptr) return DFX_ERR_INVALID_ARG;
    return run_paged_attn(p, p->workspace, p->workspace_bytes, stream);
}
