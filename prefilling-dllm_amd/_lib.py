"""ctypes binding of libpdllm_hip.so (the C ABI declared in include/pdllm.h).

The library is the product path: there is no fallback.  If it is missing the import of
this module raises, so every operator that needs it fails loudly.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# (PDLLM_LIB names another build of the same library, e.g. to compare two kernel versions in one session)
LIB_PATH = os.environ.get("PDLLM_LIB") or os.path.join(_HERE, "libpdllm_hip.so")

PDLLM_OK = 0
ERRORS = {
    -1: ("NULL", ValueError),
    -2: ("SHAPE", ValueError),
    -3: ("STRIDE", ValueError),
    -4: ("DTYPE", ValueError),
    -5: ("WORKSPACE", RuntimeError),
    -6: ("LAUNCH", RuntimeError),
    -7: ("UNSUPPORTED", NotImplementedError),
    -8: ("SCRATCH_LIMIT", RuntimeError),
}

KV_BF16, KV_FP8_E4M3 = 0, 1
MASK_FULL, MASK_CAUSAL, MASK_DENSE = 0, 1, 2

i32, i64, f32, vp = C.c_int32, C.c_int64, C.c_float, C.c_void_p


class AttnDesc(C.Structure):
    """Mirror of struct pdllm_attn_desc (include/pdllm.h)."""

    _fields_ = [
        ("q", vp), ("k_new", vp), ("v_new", vp), ("out", vp),
        ("k_cache", vp), ("v_cache", vp), ("k_scale", vp), ("v_scale", vp),
        ("block_table", vp), ("q_start_loc", vp),
        ("range_ptr", vp), ("range_start", vp), ("range_len", vp),
        ("mask", vp), ("workspace", vp), ("workspace_bytes", i64),
        ("q_stride", i64), ("kn_stride", i64), ("vn_stride", i64), ("o_stride", i64),
        ("cache_page_stride", i64), ("cache_token_stride", i64), ("cache_head_stride", i64),
        ("mask_stride", i64), ("n_tokens", i64), ("n_pages", i64),
        ("bt_stride", i32), ("scale_page_stride", i32), ("scale_head_stride", i32),
        ("n_req", i32), ("max_q_len", i32), ("max_ctx_len", i32), ("max_ranges", i32),
        ("num_q_heads", i32), ("num_kv_heads", i32), ("head_dim", i32),
        ("page_size", i32), ("kv_dtype", i32), ("mask_mode", i32),
        ("num_splits", i32), ("rows_per_group", i32), ("sm_scale", f32),
        ("slot_table", vp), ("slot_table_stride", i64), ("tiles_per_workgroup", i32),
        ("active_slot_mapping", vp),
    ]


# name -> (restype, argtypes); every symbol include/pdllm.h declares
SIGNATURES = {
    "pdllm_status_string": (C.c_char_p, [C.c_int]),
    "pdllm_abi_version": (C.c_int, []),
    "pdllm_kv_store": (C.c_int, [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp]),
    "pdllm_kv_store_fp8": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, i32, i64, i64, vp]),
    "pdllm_slot_mapping": (C.c_int, [vp, i64, i64, i64, i32, vp, vp]),
    "pdllm_kv_load": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, i64, vp, vp, vp, i32, i64, i64, i32, i64, i64, i64, vp]),
    "pdllm_attn_workspace_bytes": (i64, [C.POINTER(AttnDesc)]),
    "pdllm_sparse_decode_attn": (C.c_int, [C.POINTER(AttnDesc), vp]),
    "pdllm_chunk_prefill_attn": (C.c_int, [C.POINTER(AttnDesc), vp, vp]),
    "pdllm_attn_plan": (C.c_int, [C.POINTER(AttnDesc), i32, C.POINTER(i32), C.POINTER(i32)]),
    "pdllm_attn_plan_describe": (C.c_int, [C.POINTER(AttnDesc), i32, C.c_char_p, i32]),
    "pdllm_attn_slot_table_stride": (i64, [C.POINTER(AttnDesc)]),
    "pdllm_attn_build_slot_table": (C.c_int, [C.POINTER(AttnDesc), vp, i64, vp]),
    "pdllm_selfinfo_logprob": (C.c_int, [vp, i64, vp, i64, i64, vp, i64, vp, vp]),
    "pdllm_vocab_workspace_bytes": (i64, [i64, i64]),
    "pdllm_chunk_score_reduce": (C.c_int, [vp, i64, i64, i32, vp, vp]),
    "pdllm_topk_lowest_index": (C.c_int, [vp, i64, i64, i64, i64, i32, vp, vp]),
    "pdllm_evict_colsum": (C.c_int, [vp, i64, i64, i64, i64, i64, vp, i64, vp, vp]),
    "pdllm_evict_colsum_workspace_bytes": (i64, [i64, i64, i64]),
    "pdllm_evict_keep_from_probs": (C.c_int, [vp, i64, i64, i64, i64, i64, i64, i32, i32, vp, i64, vp, vp, vp]),
    "pdllm_kv_compact_per_head_workspace_bytes": (i64, [i64, i32, i32, i32]),
    "pdllm_kv_compact_per_head": (C.c_int, [vp, i64, i32, vp, i64, vp, i64, i64, i64, i32, i32, i32, i64, i32, vp, i64, vp]),
    "pdllm_evict_score_qk_workspace_bytes": (i64, [i64, i64, i64, i32, i32, i32]),
    "pdllm_evict_score_qk": (C.c_int, [vp, vp, i64, i64, i64, i32, i32, i32, f32, i32, i32, vp, i64, vp, vp]),
    "pdllm_token_score_pool_group": (C.c_int, [vp, i64, i64, i32, i32, i64, vp, vp]),
    "pdllm_topb_keep_bos": (C.c_int, [vp, i64, i64, i64, i64, i32, i32, vp, vp]),
    "pdllm_kv_gather": (C.c_int, [vp, vp, i64, vp, i64, i64, i64, i32, i32, i32, i64, i32, vp, vp]),
    "pdllm_kv_scatter": (C.c_int, [vp, vp, i64, i64, i64, i32, i32, i32, i64, i32, vp, vp]),
    "pdllm_conf_argmax": (C.c_int, [vp, i64, vp, i64, i64, i64, i64, i32, vp, i64, vp, vp, vp]),
    "pdllm_threshold_unmask": (C.c_int, [vp, vp, vp, i64, i64, i64, f32, vp, vp, vp]),
    "pdllm_kv_copy_pages": (C.c_int, [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp]),
    "pdllm_rope_qk_store": (C.c_int, [vp, i64, i32, vp, i64, vp, i64, i32, i32, vp, vp, i64, i64, vp, vp, vp, i64, vp]),
    "pdllm_vote_histogram": (C.c_int, [vp, i64, i64, vp, vp]),
    "pdllm_denoise_unmask": (C.c_int, [vp, i64, vp, i64, i64, i64, i64, i32, vp, i64, f32, vp, i64, vp, vp, vp, vp, vp]),
    "pdllm_denoise_unmask_static": (C.c_int, [vp, i64, vp, i64, i64, i64, i64, i32, vp, i64, f32, vp, vp, vp, vp, vp]),
    "pdllm_chunk_select": (C.c_int, [vp, i64, vp, i64, i64, i64, i32, i64, i32, vp, i64, vp, vp, vp, vp]),
    "pdllm_rope_inplace": (C.c_int, [vp, i64, vp, vp, i64, i64, i32, i32, vp]),
    "pdllm_anchor_delta_add": (C.c_int, [vp, i64, vp, i64, vp, i64, i64, vp, vp, i64, vp, i64, i64, i64, i64, i32, i32,
                                         i32, i32, i32, f32, f32, i32, vp]),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C prefilling-dllm_amd/csrc`).  There is no CPU fallback."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(status: int, what: str) -> None:
    """Turn a status code into the exception class the reference raises for that kind of error."""
    if status == PDLLM_OK:
        return
    name, exc = ERRORS.get(int(status), ("UNKNOWN", RuntimeError))
    msg = lib.pdllm_status_string(int(status)).decode()
    raise exc(f"{what}: PDLLM_ERR_{name} ({msg})")
