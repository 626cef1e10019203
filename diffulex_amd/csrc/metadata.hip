// Attention metadata of one decode step, built on the device from per-sequence state.
//
// The reference fills these arrays in Python loops over its sequence objects and copies six
// small tensors to the device every step.  Here one workgroup does it: a thread per sequence
// derives the sequence's lengths from the states of its diffusion blocks, a block-wide prefix
// sum turns them into the cu_seqlens arrays, and a wave per sequence then writes the positions
// and the slot mapping of its tokens.  Nothing is read back: the maxima and the store flag go to
// a small summary array on the device.  Integer work only; results are bit-exact by construction.
#include "dfx_common.h"

namespace dfx {
namespace {

constexpr int kMetaThreads = 1024;
constexpr int kMetaMaxSeqs = 8192;  // per-sequence slot offsets are kept in shared memory

struct SeqMeta {
    int ctx;        // tokens already in the cache
    int q_len;      // tokens of this step (query rows)
    int k_len;      // what cu_seqlens_k advances by
    int seq_len;    // tokens fed to the model
    int n_store;    // leading slot-mapping entries that are real slots
    int n_slots;    // slot-mapping entries in all
    bool stores;    // sets need_kv_cache_store
    bool bad;       // a state the reference's loop cannot be in (it would raise)
};

// Block diffusion: one block of dbs tokens per sequence, the last dbs tokens of the sequence
// (block_diffusion/engine/sequence.py:186-191, model_runner.py:127-149).
DFX_D SeqMeta bd_sequence(const dfx_metadata_params& p, int s) {
    SeqMeta m;
    const int dbs = p.diffusion_block_size;
    const int n = p.num_tokens[s];
    const int state = p.block_state[static_cast<int64_t>(s) * p.block_state_stride];
    m.ctx = n - dbs;
    m.q_len = m.k_len = m.seq_len = dbs;
    m.n_store = state == DFX_BLOCK_TO_CACHE ? (dbs / p.page_size) * p.page_size : 0;
    m.n_slots = state == DFX_BLOCK_ACTIVE ? dbs : m.n_store;
    m.bad = n < dbs || state > DFX_BLOCK_ACTIVE || (m.n_store > 0 && p.num_pages[s] < dbs / p.page_size);
    m.stores = state == DFX_BLOCK_TO_CACHE;  // (also where a page is larger than a block and no slot results)
    if (m.bad) m.n_store = m.n_slots = 0;
    return m;
}

// D2F: every diffusion block after the cached ones is fed; blocks to be cached get slots, blocks
// from the first active one on get -1 (d2f/engine/sequence.py:357-370, model_runner.py:150-228).
// Reachable states are IN_CACHE* TO_CACHE* ACTIVE* with block 0 in the cache.
DFX_D SeqMeta d2f_sequence(const dfx_metadata_params& p, int s) {
    SeqMeta m;
    const int dbs = p.diffusion_block_size;
    const int n_blocks = p.num_diffusion_blocks[s];
    const uint8_t* st = p.block_state + static_cast<int64_t>(s) * p.block_state_stride;
    const int prompt = p.prompt_len[s];
    const int total = p.num_tokens != nullptr ? p.num_tokens[s] : prompt + (n_blocks - 1) * dbs;
    const int last_size = n_blocks > 1 ? total - prompt - (n_blocks - 2) * dbs : prompt;
    int n_in = 0, n_to = 0, n_act = 0;
    bool bad = n_blocks < 1 || last_size < 1 || last_size > dbs + (n_blocks > 1 ? 0 : prompt);
    for (int b = 0; b < n_blocks; ++b) {
        const int x = st[b];
        if (x == DFX_BLOCK_IN_CACHE) {
            bad |= n_to + n_act > 0;
            ++n_in;
        } else if (x == DFX_BLOCK_TO_CACHE) {
            bad |= n_act > 0;
            ++n_to;
        } else if (x == DFX_BLOCK_ACTIVE) {
            ++n_act;
        } else {
            bad = true;
        }
    }
    bad |= n_in == 0;  // the reference indexes its last cached block
    const bool short_last = n_blocks > 1 && last_size != dbs;
    bad |= short_last && n_act > 0;  // its padding of active blocks assumes whole blocks
    m.ctx = n_in > 0 ? prompt + (n_in - 1) * dbs - ((short_last && n_in == n_blocks) ? dbs - last_size : 0) : 0;
    m.q_len = total - m.ctx;
    m.k_len = total;
    m.seq_len = m.q_len;
    m.n_store = n_act > 0 ? n_to * dbs : m.q_len;
    m.n_slots = m.q_len;
    m.bad = bad || m.q_len < 0;
    m.stores = !m.bad && n_to > 0;
    if (m.bad) m.ctx = m.q_len = m.k_len = m.seq_len = m.n_store = m.n_slots = 0;
    return m;
}

DFX_D SeqMeta sequence_meta(const dfx_metadata_params& p, int s) {
    return p.strategy == DFX_META_D2F ? d2f_sequence(p, s) : bd_sequence(p, s);
}

struct Sums {
    int q, k, slots;
};

// Exclusive prefix sums over the workgroup's threads; `total` gets the grand totals.
DFX_D Sums block_exclusive_scan(Sums mine, int (*buf)[kMetaThreads], Sums& total) {
    const int t = threadIdx.x;
    buf[0][t] = mine.q;
    buf[1][t] = mine.k;
    buf[2][t] = mine.slots;
    __syncthreads();
    for (int d = 1; d < kMetaThreads; d <<= 1) {
        int add[3] = {0, 0, 0};
        if (t >= d) {
            for (int j = 0; j < 3; ++j) add[j] = buf[j][t - d];
        }
        __syncthreads();
        for (int j = 0; j < 3; ++j) buf[j][t] += add[j];
        __syncthreads();
    }
    total = {buf[0][kMetaThreads - 1], buf[1][kMetaThreads - 1], buf[2][kMetaThreads - 1]};
    return {buf[0][t] - mine.q, buf[1][t] - mine.k, buf[2][t] - mine.slots};
}

__global__ void __launch_bounds__(kMetaThreads) build_decode_metadata_kernel(const dfx_metadata_params p) {
    __shared__ int scan[3][kMetaThreads];
    __shared__ int slot_off[kMetaMaxSeqs];
    __shared__ int red[4];  // max q, max k, need store, first bad sequence + 1
    const int t = threadIdx.x;
    const int n = p.num_seqs;
    if (t < 4) red[t] = 0;
    const int chunk = (n + kMetaThreads - 1) / kMetaThreads;
    const int s0 = min(t * chunk, n), s1 = min(s0 + chunk, n);

    Sums mine = {0, 0, 0};
    int max_q = 0, max_k = 0, store = 0, bad = 0;
    for (int s = s0; s < s1; ++s) {
        const SeqMeta m = sequence_meta(p, s);
        mine.q += m.q_len;
        mine.k += m.k_len;
        mine.slots += m.n_slots;
        max_q = max(max_q, m.q_len);
        max_k = max(max_k, m.k_len);
        store |= m.stores;
        if (m.bad && bad == 0) bad = s + 1;
    }
    Sums total;
    Sums run = block_exclusive_scan(mine, scan, total);
    if (max_q > 0) atomicMax(&red[0], max_q);
    if (max_k > 0) atomicMax(&red[1], max_k);
    if (store) atomicOr(&red[2], 1);
    if (bad) atomicMax(&red[3], kMetaMaxSeqs + 1 - bad);  // the smallest offending index wins

    if (t == 0) p.cu_seqlens_q[0] = p.cu_seqlens_k[0] = 0;
    for (int s = s0; s < s1; ++s) {
        const SeqMeta m = sequence_meta(p, s);
        slot_off[s] = run.slots;
        run.q += m.q_len;
        run.k += m.k_len;
        run.slots += m.n_slots;
        p.cu_seqlens_q[s + 1] = run.q;
        p.cu_seqlens_k[s + 1] = run.k;
        p.context_lens[s] = m.ctx;
        if (p.seq_lens != nullptr) p.seq_lens[s] = m.seq_len;
    }
    __syncthreads();

    // positions and slots, a wave per sequence
    const int lane = t & 63, wave = t >> 6;
    const int page = p.page_size, dbs = p.diffusion_block_size;
    for (int s = wave; s < n; s += kMetaThreads / 64) {
        const SeqMeta m = sequence_meta(p, s);
        // (block diffusion feeds dbs tokens per sequence; for D2F every fed token has a slot entry)
        const int64_t q0 = p.strategy == DFX_META_D2F ? slot_off[s] : static_cast<int64_t>(s) * dbs;
        for (int i = lane; i < m.seq_len; i += 64) {
            if (q0 + i < p.token_capacity) {
                p.positions[q0 + i] = m.ctx + i;
                if (p.input_ids != nullptr) p.input_ids[q0 + i] = p.token_ids[static_cast<int64_t>(s) * p.token_ids_stride + m.ctx + i];
            }
        }
        const int32_t* table = p.block_tables + static_cast<int64_t>(s) * p.block_table_stride;
        const int64_t o0 = slot_off[s];
        for (int i = lane; i < m.n_slots; i += 64) {
            int slot = -1;
            if (i < m.n_store) {
                if (p.strategy == DFX_META_D2F) {
                    const int g = m.ctx + i;  // position in the sequence == position in its pages
                    slot = table[g / page] * page + g % page;
                } else {
                    const int first = p.num_pages[s] - dbs / page;  // the block's pages end the table
                    slot = table[first + i / page] * page + i % page;
                }
            }
            if (o0 + i < p.token_capacity) p.slot_mapping[o0 + i] = slot;
        }
    }

    // the tail of buffers sized for a larger (captured) batch reads as zeros
    for (int64_t i = total.q + t; i < p.padded_tokens && i < p.token_capacity; i += kMetaThreads) {
        p.positions[i] = 0;
        if (p.input_ids != nullptr) p.input_ids[i] = 0;
    }
    for (int64_t i = total.slots + t; i < p.padded_tokens && i < p.token_capacity; i += kMetaThreads)
        p.slot_mapping[i] = 0;
    for (int s = n + t; s < p.padded_seqs; s += kMetaThreads) {
        p.cu_seqlens_q[s + 1] = 0;
        p.cu_seqlens_k[s + 1] = 0;
        p.context_lens[s] = 0;
        if (p.seq_lens != nullptr) p.seq_lens[s] = 0;
    }
    __syncthreads();
    if (t == 0) {
        p.summary[0] = total.q;
        p.summary[1] = total.slots;
        p.summary[2] = red[0];
        p.summary[3] = red[1];
        p.summary[4] = red[2];
        p.summary[5] = (total.q > p.token_capacity || total.slots > p.token_capacity) ? 1 : 0;
        p.summary[6] = red[3] ? kMetaMaxSeqs + 1 - red[3] : 0;
        p.summary[7] = total.k;
    }
}

}  // namespace
}  // namespace dfx

extern "C" int dfx_build_decode_metadata(const dfx_metadata_params* p, dfx_stream_t stream) {
    using namespace dfx;
    if (p == nullptr) return DFX_ERR_INVALID_ARG;
    if (p->strategy != DFX_META_BLOCK_DIFFUSION && p->strategy != DFX_META_D2F) return DFX_ERR_INVALID_ARG;
    if (p->num_seqs < 0 || p->page_size <= 0 || p->diffusion_block_size <= 0 || p->token_capacity < 0 ||
        p->padded_seqs < 0 || p->padded_tokens < 0 || p->block_state_stride < 0 || p->block_table_stride < 0)
        return DFX_ERR_INVALID_ARG;
    if (p->num_seqs > kMetaMaxSeqs) return DFX_ERR_UNSUPPORTED;
    if (p->padded_tokens > p->token_capacity) return DFX_ERR_INVALID_ARG;
    if (p->cu_seqlens_q == nullptr || p->cu_seqlens_k == nullptr || p->summary == nullptr) return DFX_ERR_INVALID_ARG;
    if (p->num_seqs > 0 || p->padded_seqs > 0) {
        if (p->context_lens == nullptr) return DFX_ERR_INVALID_ARG;
    }
    if (p->token_capacity > 0 && (p->positions == nullptr || p->slot_mapping == nullptr)) return DFX_ERR_INVALID_ARG;
    if ((p->input_ids != nullptr) != (p->token_ids != nullptr) || p->token_ids_stride < 0) return DFX_ERR_INVALID_ARG;
    if (p->num_seqs > 0) {
        if (p->block_state == nullptr || p->block_tables == nullptr) return DFX_ERR_INVALID_ARG;
        if (p->strategy == DFX_META_BLOCK_DIFFUSION) {
            if (p->num_tokens == nullptr || p->num_pages == nullptr) return DFX_ERR_INVALID_ARG;
        } else {
            if (p->prompt_len == nullptr || p->num_diffusion_blocks == nullptr) return DFX_ERR_INVALID_ARG;
        }
    }
    hipLaunchKernelGGL(build_decode_metadata_kernel, dim3(1), dim3(kMetaThreads), 0, static_cast<hipStream_t>(stream),
                       *p);
    return launch_status();
}
