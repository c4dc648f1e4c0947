"""ctypes binding of libeagle_mi355x.so (declared in include/eagle_mi355x.h).

The library is never built or replaced at import time: a missing library is a
hard error (there is no CPU or eager fallback).  Build it with
`python -m mlx_eagle_spec_decoding_tree_amd.build`.
"""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_long, c_longlong, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libeagle_mi355x.so")

_lib = None

# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "eagle_status_string": (c_char_p, [c_int]),
    "eagle_abi_version": (c_int, []),
    "eagle_check_device": (c_int, []),
    "eagle_qmm_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "eagle_qmm_w4g64_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p, c_size_t, c_void_p]),
    "eagle_qmm_noalloc_scratch_bytes": (c_size_t, []),
    "eagle_qmm_w4g64_f16_noalloc": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p]),
    "eagle_qmm_small_supported": (c_int, [c_int] * 5),
    "eagle_qmm_small_w4g64_f16": (c_int, [c_void_p, c_void_p, c_float] + [c_void_p] * 6 + [c_int] * 6 + [c_void_p]),
    "eagle_qkv_rope_small_supported": (c_int, [c_int] * 5),
    "eagle_qkv_rope_small_w4g64_f16": (c_int, [c_void_p, c_void_p, c_float] + [c_void_p] * 9 + [c_int] * 5
                                       + [c_long, c_int, c_int, c_void_p]),
    "eagle_qmv_supported": (c_int, [c_int] * 2),
    "eagle_qmv_w4g64_f16": (c_int, [c_void_p] * 6 + [c_int] * 4 + [c_void_p]),
    "eagle_qmv_rows_supported": (c_int, [c_int] * 3),
    "eagle_qmv_rows_w4g64_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p]),
    "eagle_qmm_plan": (c_int, [c_int, c_int, c_int, c_void_p]),
    "eagle_qmm_swiglu_w4g64_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p, c_size_t, c_void_p]),
    "eagle_qmm_workspace_bytes_tuned": (c_size_t, [c_int] * 3),
    "eagle_qmm_w4g64_f16_tuned": (c_int, [c_void_p] * 6 + [c_int] * 8 + [c_void_p, c_size_t, c_void_p]),
    "eagle_qmm_gemm_w4g64_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p]),
    "eagle_qmm_gemm_swiglu_w4g64_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p]),
    "eagle_qmm_slab_count": (c_int, [c_int] * 2),
    "eagle_qmm_slab_steps": (c_int, [c_int] * 3),
    "eagle_qmm_slab_partial_bytes": (c_size_t, [c_int] * 3),
    "eagle_qmm_slab_partial_bytes_rows": (c_size_t, [c_int] * 4),
    "eagle_qmm_slab_partial_w4g64": (c_int, [c_void_p] * 5 + [c_size_t] + [c_int] * 6 + [c_void_p]),
    "eagle_qmm_tiled_supported": (c_int, [c_int] * 3),
    "eagle_qmm_tiled_sb_bytes": (c_size_t, [c_int] * 2),
    "eagle_qmm_tile_w4g64": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_void_p]),
    "eagle_qmm_slab_partial_tiled_w4g64": (c_int, [c_void_p] * 4 + [c_size_t] + [c_int] * 5 + [c_void_p]),
    "eagle_qmm_slab_swiglu_tiled_w4g64_f16": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_void_p]),
    "eagle_qmm_rows_tiled_supported": (c_int, [c_int] * 3),
    "eagle_qmm_rows_tiled_w4g64_f16": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_void_p]),
    "eagle_qmm_slab_swiglu_supported": (c_int, [c_int] * 3),
    "eagle_qmm_slab_swiglu_preferred": (c_int, [c_int] * 3),
    "eagle_qmm_slab_swiglu_w4g64_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p]),
    "eagle_slab_sum_f16": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "eagle_rmsnorm_slabs_f16": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                                        c_int, c_int, c_void_p]),
    "eagle_rope_kv_append_slabs_f16": (c_int, [c_void_p, c_int] + [c_void_p] * 6 + [c_int] * 4
                                       + [c_long, c_void_p]),
    "eagle_embed_w4g64_f16": (c_int, [c_void_p] * 5 + [c_int] * 3 + [c_void_p]),
    "eagle_rope_arrayed_f16": (c_int, [c_void_p] * 3 + [c_float, c_void_p] + [c_int] * 4 + [c_void_p]),
    "eagle_rope_kv_append_f16": (c_int, [c_void_p] * 5 + [c_float] + [c_void_p] * 4 + [c_int] * 4
                                 + [c_long, c_long, c_void_p]),
    "eagle_rope_kv_append_table_f16": (c_int, [c_void_p] * 8 + [c_int] * 4 + [c_long, c_long, c_void_p]),
    "eagle_tree_attention_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "eagle_tree_attention_f16": (c_int, [c_void_p] * 6 + [c_int] * 4 + [c_long, c_int, c_float,
                                                                       c_void_p, c_size_t, c_void_p]),
    "eagle_draft_attention_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_long, c_int, c_float,
                                                                        c_void_p, c_size_t, c_void_p]),
    "eagle_tree_attention_wide_workspace_bytes": (c_size_t, [c_int] * 4),
    "eagle_tree_attention_wide_f16": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_long, c_int, c_float,
                                                                            c_void_p, c_size_t, c_void_p]),
    "eagle_logsoftmax_topk_workspace_bytes": (c_size_t, [c_int, c_long]),
    "eagle_logsoftmax_topk_f16": (c_int, [c_void_p] * 2 + [c_int, c_long, c_int, c_int]
                                  + [c_void_p] * 3 + [c_size_t, c_void_p]),
    "eagle_draft_tree_init": (c_int, [c_void_p] * 2 + [c_int] + [c_void_p] * 7),
    "eagle_draft_tree_level": (c_int, [c_void_p] * 2 + [c_int] * 3 + [c_void_p] * 9),
    "eagle_spec_begin": (c_int, [c_void_p] * 5),
    "eagle_spec_update": (c_int, [c_void_p] * 3 + [c_int] + [c_void_p] * 5 + [c_int, c_void_p]),
    "eagle_causal_attention_workspace_bytes": (c_size_t, [c_int] * 4),
    "eagle_causal_attention_f16": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_long, c_int, c_float,
                                                                         c_void_p, c_size_t, c_void_p]),
    "eagle_rope_table_f32": (c_int, [c_void_p, c_void_p, c_float, c_int, c_int, c_void_p, c_void_p]),
    "eagle_rmsnorm_f16": (c_int, [c_void_p] * 3 + [c_float] + [c_void_p] * 2 + [c_int] * 2 + [c_void_p]),
    "eagle_silu_mul_f16": (c_int, [c_void_p] * 3 + [c_int] * 2 + [c_void_p]),
    "eagle_add_f16": (c_int, [c_void_p] * 3 + [c_long, c_void_p]),
    "eagle_argmax_workspace_bytes": (c_size_t, [c_int, c_long]),
    "eagle_argmax_rows_f16": (c_int, [c_void_p] * 2 + [c_int, c_long, c_void_p, c_size_t, c_void_p]),
    "eagle_process_draft_tree": (c_int, [c_void_p] * 4 + [c_int] * 3 + [c_void_p] * 5),
    "eagle_post_process_draft_tree": (c_int, [c_void_p] * 2 + [c_int] + [c_void_p] * 3),
    "eagle_greedy_accept": (c_int, [c_void_p] * 4 + [c_int] + [c_void_p] * 3),
    "eagle_kv_compact_f16": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p]),
    "eagle_fill_i32": (c_int, [c_void_p, c_int32, c_long, c_void_p]),
    "eagle_tree_positions": (c_int, [c_void_p] * 3 + [c_int, c_void_p]),
    "eagle_advance_len": (c_int, [c_void_p, c_int, c_void_p]),
}


class EagleLibraryMissing(RuntimeError):
    pass


def lib():
    """The loaded C-ABI library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise EagleLibraryMissing(
                f"{LIB_PATH} not found: build the HIP extension first "
                "(python -m mlx_eagle_spec_decoding_tree_amd.build); there is no fallback path")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def status_string(rc):
    return lib().eagle_status_string(rc).decode()


def check(rc, what):
    """Raise the Python error that corresponds to a non-zero status."""
    if rc == 0:
        return
    msg = f"{what}: {status_string(rc)} (status {rc})"
    if rc in (1, 2, 3, 4, 5):
        raise ValueError(msg)
    raise RuntimeError(msg)
