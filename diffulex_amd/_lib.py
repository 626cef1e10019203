"""ctypes binding of libdiffulex_amd.so (declarations follow include/diffulex_amd.h).

There is no fallback: if the library is missing the import of any operator
raises, so a GPU run can never silently take another path.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libdiffulex_amd.so"

DFX_ABI_VERSION = 8
DFX_OK = 0
DFX_KV_BF16, DFX_KV_FP8_E4M3 = 0, 1
DFX_MASK_FULL, DFX_MASK_BLOCK_CAUSAL = 0, 1
DFX_INDEX_I32, DFX_INDEX_I64 = 0, 1
DFX_ATTN_GENERIC_PATH = 1
DFX_ATTN_NO_PIPELINE = 2
DFX_ATTN_PAIRING = 4
DFX_ATTN_EQUAL_RANGES = 8
DFX_ATTN_BATCH_ORDER = 16
DFX_ERR_SCRATCH_LIMIT = -5
DFX_STATIC_SCRATCH_BYTES = 40 << 20
DFX_WORKSPACE_COUNTER_BYTES = 1 << 18

EXPORTS = (
    "dfx_abi_version", "dfx_status_string", "dfx_kv_store_unified", "dfx_kv_store_distinct",
    "dfx_kv_load", "dfx_paged_attn_workspace_bytes", "dfx_paged_attn", "dfx_paged_attn_static", "dfx_paged_attn_plan_bytes", "dfx_paged_attn_plan", "dfx_stream_capture_id",
    "dfx_rope_kv_store", "dfx_build_decode_metadata",
)


class AttnParams(C.Structure):
    """Mirror of ``dfx_attn_params``."""
    _fields_ = [
        ("q", C.c_void_p), ("k_new", C.c_void_p), ("v_new", C.c_void_p),
        ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("out", C.c_void_p),
        ("block_tables", C.c_void_p), ("context_lens", C.c_void_p),
        ("cu_seqlens_q", C.c_void_p), ("cu_seqlens_new", C.c_void_p),
        ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
        ("q_stride_token", C.c_int64), ("q_stride_head", C.c_int64),
        ("kn_stride_token", C.c_int64), ("kn_stride_head", C.c_int64),
        ("vn_stride_token", C.c_int64), ("vn_stride_head", C.c_int64),
        ("o_stride_token", C.c_int64), ("o_stride_head", C.c_int64),
        ("cache_stride_page", C.c_int64), ("cache_stride_token", C.c_int64), ("cache_stride_head", C.c_int64),
        ("block_table_stride", C.c_int64), ("n_pages", C.c_int64),
        ("num_seqs", C.c_int32), ("num_q_heads", C.c_int32), ("num_kv_heads", C.c_int32), ("head_dim", C.c_int32),
        ("page_size", C.c_int32), ("max_pages_per_seq", C.c_int32), ("max_seqlen_q", C.c_int32),
        ("diffusion_block_size", C.c_int32), ("kv_dtype", C.c_int32), ("mask_mode", C.c_int32),
        ("max_workgroups", C.c_int32), ("flags", C.c_int32), ("scale", C.c_float),
        ("store_slot_mapping", C.c_void_p), ("store_slot_index_type", C.c_int32),
        ("plan", C.c_void_p), ("plan_bytes", C.c_int64), ("num_new_tokens", C.c_int64),
        ("cache_layout", C.c_int32), ("num_q_tokens", C.c_int32), ("kc_stride", C.c_int64 * 5), ("vc_stride", C.c_int64 * 4),
        ("rope_cos_sin", C.c_void_p), ("rope_positions", C.c_void_p), ("rope_position_index_type", C.c_int32),
        ("reserved2", C.c_int32), ("rope_max_position", C.c_int64), ("k_rotated", C.c_void_p),
        ("kr_stride_token", C.c_int64), ("kr_stride_head", C.c_int64),
    ]


class RopeParams(C.Structure):
    """Mirror of ``dfx_rope_params``."""
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("q_out", C.c_void_p), ("k_out", C.c_void_p),
        ("q_stride_token", C.c_int64), ("k_stride_token", C.c_int64), ("v_stride_token", C.c_int64),
        ("q_out_stride_token", C.c_int64), ("k_out_stride_token", C.c_int64),
        ("positions", C.c_void_p), ("position_index_type", C.c_int32),
        ("cos_sin_cache", C.c_void_p), ("max_position", C.c_int64), ("n_tokens", C.c_int64),
        ("num_q_heads", C.c_int32), ("num_kv_heads", C.c_int32), ("head_dim", C.c_int32), ("kv_dtype", C.c_int32),
        ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("slot_mapping", C.c_void_p), ("slot_index_type", C.c_int32), ("n_slots", C.c_int64),
        ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
        ("cache_layout", C.c_int32), ("page_size", C.c_int32), ("kc_stride", C.c_int64 * 3), ("vc_stride", C.c_int64 * 3),
    ]


class MetadataParams(C.Structure):
    """Mirror of ``dfx_metadata_params``."""
    _fields_ = [
        ("strategy", C.c_int32), ("num_seqs", C.c_int32), ("page_size", C.c_int32), ("diffusion_block_size", C.c_int32),
        ("num_tokens", C.c_void_p), ("prompt_len", C.c_void_p), ("block_state", C.c_void_p),
        ("block_state_stride", C.c_int64), ("num_diffusion_blocks", C.c_void_p),
        ("block_tables", C.c_void_p), ("block_table_stride", C.c_int64), ("num_pages", C.c_void_p),
        ("positions", C.c_void_p), ("slot_mapping", C.c_void_p), ("token_capacity", C.c_int64),
        ("cu_seqlens_q", C.c_void_p), ("cu_seqlens_k", C.c_void_p), ("context_lens", C.c_void_p),
        ("seq_lens", C.c_void_p), ("padded_seqs", C.c_int32), ("reserved", C.c_int32),
        ("padded_tokens", C.c_int64), ("summary", C.c_void_p),
        ("token_ids", C.c_void_p), ("token_ids_stride", C.c_int64), ("input_ids", C.c_void_p),
    ]


DFX_BLOCK_IN_CACHE, DFX_BLOCK_TO_CACHE, DFX_BLOCK_ACTIVE = 0, 1, 2
DFX_META_BLOCK_DIFFUSION, DFX_META_D2F = 0, 1
DFX_CACHE_UNIFIED, DFX_CACHE_DISTINCT = 0, 1


class DfxError(RuntimeError):
    pass


_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build the gfx950 kernels first (python -m diffulex_amd.build). "
            "diffulex_amd has no fallback path.")
    lib = C.CDLL(str(LIB_PATH))
    i64, i32, vp = C.c_int64, C.c_int, C.c_void_p
    lib.dfx_abi_version.restype = i32
    lib.dfx_abi_version.argtypes = []
    lib.dfx_status_string.restype = C.c_char_p
    lib.dfx_status_string.argtypes = [i32]
    lib.dfx_kv_store_unified.restype = i32
    lib.dfx_kv_store_unified.argtypes = [vp, vp, i64, i64, vp, vp, vp, i32, i64, i64, i32, i32, i32, vp, vp, vp]
    lib.dfx_kv_store_distinct.restype = i32
    lib.dfx_kv_store_distinct.argtypes = [vp, vp, i64, i64, vp, vp, C.POINTER(i64), C.POINTER(i64), vp, i32,
                                          i64, i64, i32, i32, i32, i32, vp]
    lib.dfx_kv_load.restype = i32
    lib.dfx_kv_load.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp, i64, vp, vp, vp, vp, i32, i32, i64, i32,
                                i32, i32, i64, i32, vp, vp, vp]
    lib.dfx_paged_attn_workspace_bytes.restype = i64
    lib.dfx_paged_attn_workspace_bytes.argtypes = [C.POINTER(AttnParams)]
    lib.dfx_paged_attn.restype = i32
    lib.dfx_paged_attn.argtypes = [C.POINTER(AttnParams), vp]
    lib.dfx_paged_attn_plan_bytes.restype = i64
    lib.dfx_paged_attn_plan_bytes.argtypes = [C.POINTER(AttnParams), i64]
    lib.dfx_stream_capture_id.restype = i64
    lib.dfx_stream_capture_id.argtypes = [vp]
    lib.dfx_paged_attn_plan.restype = i32
    lib.dfx_paged_attn_plan.argtypes = [C.POINTER(AttnParams), vp, i64, vp]
    lib.dfx_paged_attn_static.restype = i32
    lib.dfx_paged_attn_static.argtypes = [C.POINTER(AttnParams), vp]
    lib.dfx_rope_kv_store.restype = i32
    lib.dfx_rope_kv_store.argtypes = [C.POINTER(RopeParams), vp]
    lib.dfx_build_decode_metadata.restype = i32
    lib.dfx_build_decode_metadata.argtypes = [C.POINTER(MetadataParams), vp]
    if lib.dfx_abi_version() != DFX_ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI {lib.dfx_abi_version()}, expected {DFX_ABI_VERSION}: rebuild it")
    _lib = lib
    return lib


OPS_PATH = LIB_PATH.parent / "_torch_ops.so"
_ops = None


def ops():
    """``torch.ops.diffulex_amd``: the operator library that binds the C ABI to PyTorch tensors
    and streams (csrc/torch_ext.cpp).  The Python operators go through it; ``load()`` above (ctypes)
    is the direct view of the same C functions."""
    global _ops
    if _ops is None:
        import torch
        if not OPS_PATH.exists():
            raise ImportError(f"{OPS_PATH} is missing: build it first (python -m diffulex_amd.build). "
                              "diffulex_amd has no fallback path.")
        load()  # checks the ABI version of the kernel library the operator library links to
        torch.ops.load_library(str(OPS_PATH))
        _ops = torch.ops.diffulex_amd
    return _ops


def check(status: int, what: str) -> None:
    if status != DFX_OK:
        msg = load().dfx_status_string(int(status)).decode()
        raise DfxError(f"{what}: {msg} ({status})")
