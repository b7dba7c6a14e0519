"""ctypes binding of libet_amd.so (the C ABI declared in include/et_amd.h).

The library is the product; there is no fallback.  If it is missing the import
of any et_amd operator fails loudly.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libet_amd.so")

_vp, _ip, _i, _f, _u64, _sz = C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_uint64, C.c_size_t

# name -> (restype, argtypes); mirrors include/et_amd.h one to one
PROTOTYPES = {
    "et_strerror": (C.c_char_p, [_i]),
    "et_last_error": (C.c_char_p, []),
    "et_abi_version": (_i, []),
    "et_skip_layernorm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "et_tile_spmm_add_bias": (_i, [_vp, _vp, _ip, _ip, _vp, _i, _i, _i, _vp, _vp]),
    "et_tile_spmm_add_bias_gelu": (_i, [_vp, _vp, _ip, _ip, _vp, _i, _i, _i, _vp, _vp]),
    "et_row_spmm_add_bias_gelu": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "et_row_spmm_add_bias": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "et_row_spmm_add_bias_multi": (_i, [C.POINTER(_vp), _vp, C.POINTER(_vp), C.POINTER(_vp), _ip, _i, _i, _i, _vp]),
    "et_row_spmm_prefers_gemm": (_i, [_i, _i, _i]),
    "et_OTF_attention": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _ip, _f, _vp]),
    "et_OTF_attention_summary": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _ip, _f, _vp]),
    "et_OTF_attention_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _ip, _f, _vp]),
    "et_attention_mask_summary_bytes": (C.c_size_t, [_i]),
    "et_attention_mask_summary": (_i, [_vp, _i, _vp, _vp]),
    "et_attention_mask_summary_attach": (_i, [_vp, _i, _vp]),
    "et_OTF_attention_varlen": (_i, [_vp, _vp, _vp, _vp, _vp, _ip, _i, _i, _i, _i, _f, _vp]),
    "et_OTF_attention_qk_width": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _ip, _f, _vp]),
    "et_Prune_attention": (_i, [_vp, _vp, _vp, _vp, _ip, _i, _ip, _ip, _i, _vp, _i, _i, _i, _i, _ip, _f, _vp]),
    "et_sharedQK_attention": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _ip, _f, _vp]),
    "et_qk_scores": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "et_tile_plan_create": (_i, [C.POINTER(_vp), _i, _i, _i, _vp, _ip, _ip, _vp]),
    "et_tile_plan_destroy": (None, [_vp]),
    "et_tile_plan_run": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "et_tile_plan_run_ln": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "et_tile_plan_ln_fusable": (_i, [_vp]),
    "et_tile_plan_run_ffn_ln": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "et_tile_plan_ffn_fusable": (_i, [_vp, _vp]),
    "et_tile_plan_run_tail": (_i, [_vp] * 12 + [_i, _vp]),
    "et_tile_plan_tail_fusable": (_i, [_vp, _vp, _vp]),
    "et_tile_plan_run_tail_ws": (_i, [_vp] * 12 + [_i, _vp, _sz, _vp]),
    "et_tile_plan_tail_prepare": (_i, [_vp, _vp, _vp]),
    "et_tile_plan_tail_ws_bytes": (_sz, [_vp, _vp, _vp, _i]),
    "et_tail_ws_bytes_for": (_sz, [_i, _i]),
    "et_wait_status_take": (_i, []),
    "et_wait_status_raise_for_test": (None, []),
    "et_tile_plan_run_multi": (_i, [C.POINTER(_vp), C.POINTER(_vp), _i, _vp, _i, _vp]),
    "et_tile_plan_query": (_i, [_vp, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)]),
    "et_prune_tile_mat": (_i, [_vp, _i, _i, _f, _ip, _ip]),
    "et_prune_row_mat": (_i, [_vp, _i, _i, _f, _ip]),
    "et_tile_mat_save": (_i, [C.c_char_p, _i, _i, _i, _ip, _ip, _vp, _vp]),
    "et_tile_mat_peek": (_i, [C.c_char_p, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)]),
    "et_tile_mat_load": (_i, [C.c_char_p, _i, _i, _i, _ip, _ip, _vp, _vp]),
    "et_row_mat_save": (_i, [C.c_char_p, _i, _i, _i, _ip, _vp, _vp]),
    "et_row_mat_peek": (_i, [C.c_char_p, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)]),
    "et_row_mat_load": (_i, [C.c_char_p, _i, _i, _i, _ip, _vp, _vp]),
    "et_gen_sparse_tile_mat": (_i, [_i, _i, _f, _u64, _ip, _ip]),
    "et_gen_sparse_row_mat": (_i, [_i, _f, _u64, _ip]),
    "et_gen_head_balanced_rows": (_i, [_i, _i, _i, _u64, _ip]),
    "et_tile_mat_validate": (_i, [_i, _i, _i, _ip, _ip]),
    "et_tile_pack": (_i, [_vp, _i, _i, _ip, _ip, _vp]),
    "et_head_ptr": (_i, [_ip, _i, _i, _i, _ip]),
    "et_pack_rows": (_i, [_vp, _vp, _ip, _i, _i, _i, _vp]),
    "et_unpack_rows": (_i, [_vp, _vp, _ip, _i, _i, _i, _vp]),
    "et_pack_rows_ordered": (_i, [_vp, _vp, _ip, _ip, _i, _i, _i, _vp]),
    "et_unpack_rows_ordered": (_i, [_vp, _vp, _ip, _ip, _i, _i, _i, _vp]),
    "et_scatter_cols": (_i, [_vp, _vp, _ip, _i, _i, _i, _i, _vp]),
    "et_scatter_skip_layernorm": (_i, [_vp, _vp, _ip, _i, _i, _vp, _vp, _vp, _i, _i, _vp]),
    # include/et_encoder.h
    "et_linear_tile_create": (_i, [C.POINTER(_vp), _i, _i, _i, _i, _vp, _ip, _ip, _vp, _i]),
    "et_linear_tile_destroy": (None, [_vp]),
    "et_linear_tile_run": (_i, [_vp, _vp, _vp, _vp]),
    "et_linear_tile_run_rows": (_i, [_vp, _vp, _vp, _i, _vp]),
    "et_linear_tile_run_rows_ln": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "et_linear_tile_run_rows_ffn_ln": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "et_linear_tile_ffn_fusable": (_i, [_vp, _vp]),
    "et_linear_tile_run_rows_tail": (_i, [_vp] * 12 + [_i, _vp]),
    "et_linear_tile_tail_fusable": (_i, [_vp, _vp, _vp]),
    "et_linear_tile_run_rows_tail_ws": (_i, [_vp] * 12 + [_i, _vp, _sz, _vp]),
    "et_linear_tile_tail_prepare": (_i, [_vp, _vp, _vp]),
    "et_linear_tile_tail_ws_bytes": (_sz, [_vp, _vp, _vp, _i]),
    "et_linear_tile_run_multi": (_i, [C.POINTER(_vp), C.POINTER(_vp), _i, _vp, _i, _vp]),
    "et_linear_row_create": (_i, [C.POINTER(_vp), _i, _i, _i, _vp, _ip, _i, _vp, _i]),
    "et_linear_row_set_gelu": (_i, [_vp, _i]),
    "et_linear_row_destroy": (None, [_vp]),
    "et_linear_row_run": (_i, [_vp, _vp, _vp, _vp]),
    "et_linear_row_query": (_i, [_vp, C.POINTER(_i), C.POINTER(_i), C.POINTER(_vp), C.POINTER(_vp)]),
    "et_encoder_create": (_i, [C.POINTER(_vp), _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                _vp, _vp, _vp, _vp, _vp]),
    "et_encoder_attnaware_create": (_i, [C.POINTER(_vp), _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                          _vp, _vp, _vp, _vp, _vp]),
    "et_encoder_destroy": (None, [_vp]),
    "et_encoder_buffer_size": (_sz, [_i, _i, _i, _i, _i]),
    "et_encoder_run": (_i, [_vp, _vp, _vp]),
    "et_encoder_set_stream": (_i, [_vp, _vp]),
    "et_encoder_set_log2_scale": (_i, [_vp, _f]),
    "et_encoder_set_seq_lens": (_i, [_vp, _ip]),
    "et_encoder_set_shared_qk": (_i, [_vp, _i]),
    "et_encoder_stack_create": (_i, [C.POINTER(_vp), C.POINTER(_vp), _i, _i, _i, _i]),
    "et_encoder_stack_destroy": (None, [_vp]),
    "et_encoder_stack_run": (_i, [_vp, _vp, _vp, _vp, _vp]),
    "et_malloc": (_i, [C.POINTER(_vp), _sz]),
    "et_free": (_i, [_vp]),
    "et_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "et_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "et_memcpy_d2d_async": (_i, [_vp, _vp, _sz, _vp]),
    "et_fill_zero": (_i, [_vp, _sz, _vp]),
    "et_copy": (_i, [_vp, _vp, _sz, _vp]),
    "et_stream_create": (_i, [C.POINTER(_vp)]),
    "et_stream_destroy": (_i, [_vp]),
    "et_stream_synchronize": (_i, [_vp]),
    "et_device_synchronize": (_i, []),
    "et_device_cu_count": (_i, []),
    "et_tuning_set": (_i, [C.c_char_p, _i]),
}

_lib = None


class EtError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"et_amd error {code}: {msg}")
        self.code = code


def lib():
    """Load libet_amd.so (built by et_amd/build.py); raise if it is absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m et_amd.build` "
                "(there is no CPU or PyTorch fallback for the HIP kernels)")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc):
    """Raise EtError for a negative return code; pass non-negative values through."""
    if rc < 0:
        l = lib()
        raise EtError(rc, f"{l.et_strerror(rc).decode()} — {l.et_last_error().decode()}")
    return rc
