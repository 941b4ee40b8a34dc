"""ctypes binding of libtgis_hip.so (include/tgis_hip.h) for torch tensors on an MI355X.

This is the drop-in boundary #5 of SURVEY.md §8(b): where the reference imports CUDA extension modules
(`flash_attn_2_cuda`, `dropout_layer_norm`, `rotary_emb`, `exllamav2_kernels`; utils/flash_attn.py:23,
utils/layers.py:361,403-404, utils/gptq/exllamav2.py:7) this module loads one C-ABI shared library and
passes raw device pointers, sizes and the current HIP stream.  There is no CPU or eager-torch fallback:
if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.getenv("TGIS_HIP_LIB") or os.path.join(os.path.dirname(_HERE), "lib", "libtgis_hip.so")

F16, BF16, F32 = 0, 1, 2
KV_PAGE_TOKENS = 32

OP_GPTQ_GEMM, OP_ATTN, OP_DENSE_GEMM, OP_NORM, OP_ROPE_KV, OP_ACT, OP_SAMPLE = range(7)
OP_SCAN, OP_MOE_GEMM = 8, 9

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_f = ctypes.c_float
_vp = ctypes.c_void_p



# name -> (restype, argtypes); must list every symbol declared in include/tgis_hip.h
SIGNATURES = {
    "tgis_version": (ctypes.c_char_p, []),
    "tgis_arch": (ctypes.c_char_p, []),
    "tgis_clear_error": (None, []),
    "tgis_last_error": (ctypes.c_char_p, []),
    "tgis_device_info": (_c_int, [_c_int, ctypes.POINTER(_c_int), ctypes.POINTER(_c_i64), ctypes.c_char_p, _c_int]),
    "tgis_timing_enable": (_c_int, [_c_int]),
    "tgis_timing_reset": (_c_int, []),
    "tgis_timing_read": (_c_int, [_c_int, ctypes.POINTER(_c_i64), ctypes.POINTER(ctypes.c_double)]),
    "tgis_gptq_prepared_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "tgis_gptq_prepare": (_c_int, [_vp, _vp, _vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_int, _vp, _vp]),
    "tgis_gptq_gemm_fused_rows": (_c_i64, [_c_i64, _c_i64, _c_int, _c_int]),
    "tgis_gptq_gemm_workspace_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "tgis_gptq_gemm_f16": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
                                    _c_int, _vp, _c_i64, _vp]),
    "tgis_gptq_gemm_partial_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "tgis_gptq_gemm_f16_partial": (_c_int, [_vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _vp, _c_i64,
                                            ctypes.POINTER(_c_int), ctypes.POINTER(_c_i64), _vp]),
    "tgis_gptq_dequant_f16": (_c_int, [_vp, _vp, _c_i64, _c_i64, _c_i64, _c_int, _vp]),
    "tgis_dense_gemm_rope": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64,
                                      _c_i64, _c_i64, _c_i64, _c_int, _vp]),
    "tgis_gptq_rope_ok": (_c_int, [_c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_i64]),
    "tgis_gptq_fragments_ok": (_c_int, [_c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_int]),
    "tgis_dense_rope_ok": (_c_int, [_c_i64, _c_i64, _c_i64, _c_i64]),
    "tgis_gptq_gemm_rope_f16": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _c_i64,
                                         _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _vp]),
    "tgis_dense_prepared_bytes": (_c_i64, [_c_i64, _c_i64]),
    "tgis_dense_prepare": (_c_int, [_vp, _c_i64, _c_i64, _c_int, _c_int, _vp, _vp]),
    "tgis_dense_gemm_workspace_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "tgis_dense_gemm": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_int,
                                 _c_int, _vp, _c_i64, _vp]),
    "tgis_dense_gemm_partial_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "tgis_dense_gemm_partial": (_c_int, [_vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _vp, _c_i64,
                                         ctypes.POINTER(_c_int), ctypes.POINTER(_c_i64), _vp]),
    "tgis_rmsnorm_residual": (_c_int, [_vp, _vp, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_f, _c_int, _vp]),
    "tgis_rmsnorm_residual_partial": (_c_int, [_vp, _c_int, _c_i64, _vp, _vp, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_f,
                                               _c_int, _vp]),
    "tgis_layernorm_residual": (_c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_i64, _c_f, _c_int, _vp]),
    "tgis_layernorm_residual_partial": (_c_int, [_vp, _c_int, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_i64,
                                                 _c_f, _c_int, _vp]),
    "tgis_rope_kv_write": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_int, _c_int, _c_int,
                                    _c_int, _c_int, _vp]),
    "tgis_rope_kv_write_partial": (_c_int, [_vp, _c_int, _c_i64, _vp, _vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64,
                                            _c_int, _c_int, _c_int, _c_int, _c_int, _vp]),
    "tgis_rope_kv_write_prefill": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64,
                                            _c_int, _c_int, _c_int, _c_int, _c_int, _vp]),
    "tgis_attn_num_splits": (_c_int, [_c_i64, _c_int, _c_int, _c_i64, _c_i64]),
    "tgis_attn_workspace_bytes": (_c_i64, [_c_i64, _c_int, _c_int, _c_int, _c_int]),
    "tgis_attn_paged": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _vp, _vp, _vp, _c_i64, _c_i64, _c_int, _c_int,
                                 _c_int, _c_i64, _c_i64, _c_f, _c_int, _c_int, _vp, _c_i64, _vp]),
    "tgis_act_mul": (_c_int, [_vp, _vp, _c_i64, _c_i64, _c_int, _c_int, _vp]),
    "tgis_gelu": (_c_int, [_vp, _vp, _c_i64, _c_int, _c_int, _vp]),
    "tgis_embedding": (_c_int, [_vp, _vp, _vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _vp]),
    "tgis_decode_slots": (_c_int, [_vp, _vp, _c_i64, _vp, _vp, _c_i64, _vp]),
    "tgis_decode_advance": (_c_int, [_vp, _vp, _vp, _vp, _c_i64, _vp, _vp, _vp, _vp, _c_i64, _vp]),
    "tgis_argmax_logprob": (_c_int, [_vp, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _vp, _vp, _vp, _c_i64, _vp]),
    "tgis_argmax_scratch_bytes": (_c_i64, [_c_i64]),
    "tgis_warp_sample": (_c_int, [_vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64,
                                  _c_i64, _c_i64, _vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "tgis_embedding_scaled_f32": (_c_int, [_vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_f, _c_int, _vp]),
    "tgis_sandwich_norm_f32": (_c_int, [_vp, _vp, _c_i64, _c_int, _vp, _c_f, _vp, _vp, _c_f, _vp, _c_int, _c_i64, _c_i64, _c_f,
                                        _vp]),
    "tgis_sandwich_norm_f32_partial": (_c_int, [_vp, _vp, _c_int, _c_i64, _vp, _c_f, _vp, _vp, _c_f, _vp, _c_int, _c_i64, _c_i64,
                                                _c_f, _vp]),
    "tgis_dense_gemm_clamped_glu": (_c_int, [_vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_f, _c_f, _vp, _c_i64,
                                             _vp]),
    "tgis_glu": (_c_int, [_vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_int, _c_f, _c_f, _c_int, _vp]),
    "tgis_qk_norm_kv_write": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _c_f, _c_f, _c_int, _vp, _c_i64, _vp, _vp, _vp, _c_i64,
                                       _c_int, _c_int, _c_int, _c_int, _c_int, _vp]),
    "tgis_attn_varlen": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_i64,
                                  _c_int, _c_int, _c_int, _c_int, _c_f, _c_int, _c_int, _vp]),
    "tgis_token_shift_mix": (_c_int, [_vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _c_int, _vp, _c_i64, _c_i64, _c_int, _vp]),
    "tgis_wkv_decay": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _c_int, _c_i64, _c_int, _vp]),
    "tgis_wkv_scan": (_c_int, [_vp, _vp, _vp, _vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _vp, _vp, _vp, _c_i64,
                               _c_i64, _c_int, _c_int, _c_f, _c_int, _vp]),
    "tgis_moe_row_capacity": (_c_i64, [_c_i64, _c_i64]),
    "tgis_moe_route": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_i64, _c_int, _c_int, _c_int, _vp]),
    "tgis_moe_align": (_c_int, [_vp, _c_i64, _c_int, _vp, _c_i64, _vp, _vp, _vp, _vp]),
    "tgis_moe_gemm": (_c_int, [_vp, _c_i64, _vp, _c_int, _vp, _vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_int, _vp, _c_i64, _c_i64,
                               _c_int, _vp]),
    "tgis_moe_combine": (_c_int, [_vp, _c_i64, _vp, _vp, _c_int, _vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_int, _vp]),
    "tgis_residual_update_f32": (_c_int, [_vp, _vp, _c_i64, _c_int, _vp, _c_f, _c_f, _vp, _vp, _c_f, _vp, _c_int, _c_i64, _c_i64,
                                          _c_f, _vp]),
    "tgis_residual_update_f32_partial": (_c_int, [_vp, _vp, _c_int, _c_i64, _vp, _c_f, _c_f, _vp, _vp, _c_f, _vp, _c_int, _c_i64,
                                                  _c_i64, _c_f, _vp]),
    "tgis_xielu": (_c_int, [_vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_f, _c_f, _c_int, _vp]),
    "tgis_dense_gemm_xielu": (_c_int, [_vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_f, _c_f, _vp, _c_i64, _vp]),
    "tgis_dense_gemm_gelu_lookup": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_i64,
                                             _c_int, _vp, _c_i64, _vp]),
    "tgis_sigmoid_gate_mul": (_c_int, [_vp, _c_i64, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_int, _vp]),
    "tgis_logit_softcap": (_c_int, [_vp, _c_i64, _c_i64, _c_i64, _c_f, _vp]),
    "tgis_gelu_gated_lookup": (_c_int, [_vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_int, _vp]),
    "tgis_rms_norm_rows": (_c_int, [_vp, _c_i64, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_f, _c_int, _vp]),
    "tgis_kv_norm_write": (_c_int, [_vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_f,
                                    _c_int, _vp]),
    "tgis_latent_kv_write": (_c_int, [_vp, _c_i64, _vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _c_int, _c_int,
                                      _c_int, _c_int, _c_int, _c_f, _c_int, _vp]),
    "tgis_attn_varlen_ext": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_i64,
                                      _c_int, _c_int, _c_int, _c_int, _c_f, _vp, _vp, _c_int, _vp, _c_i64, _vp, _c_i64, _c_int, _c_int,
                                      _vp]),
    "tgis_short_conv_silu": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_int, _c_int, _vp]),
    "tgis_delta_state_floats": (_c_i64, [_c_int, _c_int]),
    "tgis_delta_scan": (_c_int, [_vp, _c_i64, _vp, _c_i64, _vp, _c_i64, _vp, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _vp, _vp,
                                 _vp, _vp, _c_i64, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_f, _c_f, _c_f, _c_int, _vp]),
    "tgis_rope_rows_kv_write": (_c_int, [_vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_int, _c_int, _c_int,
                                         _c_int, _c_int, _c_int, _vp]),
    "tgis_attn_varlen_win": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_i64,
                                      _c_int, _c_int, _c_int, _c_int, _c_f, _c_int, _c_int, _vp, _vp, _c_i64, _c_int, _c_f, _vp, _c_i64,
                                      _c_int, _c_int, _vp]),
    "tgis_gated_linear_scan": (_c_int, [_vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_f,
                                        _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_int, _c_f, _c_int, _vp, _c_int, _vp]),
    "tgis_moe_route_ext": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_int, _vp, _vp, _vp, _c_i64, _c_i64, _c_int, _c_int, _c_int, _vp]),
    "tgis_parallel_residual_f32": (_c_int, [_vp, _vp, _c_i64, _c_int, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _c_int, _vp, _vp, _c_i64, _vp,
                                            _c_int, _vp, _c_int, _c_i64, _vp, _vp, _vp, _c_f, _vp, _c_int, _c_i64, _c_i64, _c_f, _vp]),
    "tgis_rope_rows_unit_kv_write": (_c_int, [_vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_int, _c_int, _c_int,
                                              _c_int, _c_int, _c_f, _c_int, _vp]),
    "tgis_attn_mixed_heads": (_c_int, [_vp, _c_i64, _vp, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64,
                                       _c_i64, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int, _vp, _c_i64, _c_int, _c_int, _vp]),
    "tgis_linear_scan": (_c_int, [_vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _c_int, _c_f, _c_int, _c_int, _c_int, _c_f,
                                  _vp, _c_int, _vp, _c_i64, _c_int, _vp, _vp, _vp, _vp, _vp, _c_i64, _c_f, _c_i64, _c_i64, _c_i64,
                                  _c_int, _c_int, _c_int, _c_f, _vp, _c_int, _vp]),
    "tgis_causal_conv": (_c_int, [_vp, _c_i64, _c_int, _vp, _vp, _c_int, _vp, _c_i64, _vp, _vp, _vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64,
                                  _c_i64, _c_int, _c_int, _c_int, _c_int, _vp]),
    "tgis_selective_scan": (_c_int, [_vp, _c_i64, _vp, _c_i64, _c_int, _vp, _vp, _c_i64, _c_i64, _c_i64, _vp, _c_i64, _vp, _vp, _vp, _vp,
                                     _vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _vp]),
    "tgis_scaled_residual_norm": (_c_int, [_vp, _vp, _vp, _c_i64, _c_int, _vp, _vp, _c_i64, _c_int, _vp, _vp, _vp, _vp, _c_int, _c_i64,
                                           _c_i64, _c_f, _c_int, _vp, _c_i64, _c_int, _vp, _vp, _c_f, _c_int, _vp]),
    "tgis_rms_pair_mean": (_c_int, [_vp, _c_i64, _c_int, _vp, _c_f, _vp, _c_i64, _c_int, _vp, _c_f, _vp, _c_i64, _c_i64, _c_f, _c_int, _vp]),
    "tgis_poly_norm": (_c_int, [_vp, _c_i64, _vp, _c_i64, _c_i64, _c_i64, _c_f, _c_f, _c_f, _c_f, _c_f, _c_int, _vp]),
    "tgis_moe_route_grouped": (_c_int, [_vp, _c_i64, _vp, _vp, _c_int, _c_int, _c_f, _vp, _vp, _c_i64, _c_i64, _c_int, _c_int, _c_int, _vp]),
}

_lib = None


class TgisHipError(RuntimeError):
    pass


def load_library(path: Optional[str] = None) -> ctypes.CDLL:
    """dlopen the C-ABI library and bind every declared symbol.  Needs no GPU (no compute is run)."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or os.getenv("TGIS_HIP_LIB") or LIB_PATH
    if not os.path.exists(p):
        raise TgisHipError(
            f"{p} not found: build the HIP extension first (python -c 'import __graft_entry__ as g; g.build()')"
        )
    lib = ctypes.CDLL(p)
    partial = os.path.basename(p) != "libtgis_hip.so"  # a one-family build (buildlib.FAMILY_UNITS)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        except AttributeError:
            if not partial:
                raise
            continue  # calling it raises AttributeError naming the symbol
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def _check(rc: int, what: str):
    if rc != 0:
        msg = load_library().tgis_last_error().decode()
        raise TgisHipError(f"{what} failed (code {rc}): {msg}")


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float16:
        return F16
    if dt == torch.bfloat16:
        return BF16
    raise TgisHipError(f"unsupported dtype {dt} (float16 / bfloat16 only)")


def _ptr(t: Optional[torch.Tensor]):
    if t is None:
        return None
    if not t.is_cuda:
        raise TgisHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    return t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """hipStream_t of torch's current stream.  The raw getter skips the Stream object that
    torch.cuda.current_stream() builds (a third of the host time of an eager decode step went there)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def version() -> str:
    return load_library().tgis_version().decode()


def timing_enable(on: bool):
    _check(load_library().tgis_timing_enable(int(on)), "tgis_timing_enable")


def timing_reset():
    _check(load_library().tgis_timing_reset(), "tgis_timing_reset")


def timing_read(op: int):
    c = _c_i64()
    ms = ctypes.c_double()
    _check(load_library().tgis_timing_read(op, ctypes.byref(c), ctypes.byref(ms)), "tgis_timing_read")
    return c.value, ms.value


# ---- workspaces ---------------------------------------------------------------------------------
class Workspace:
    """Zero-initialised scratch for split-K slabs / arrival counters and attention splits.

    One per stream of work.  The first 4096 bytes hold the arrival counters that the GEMM kernels leave
    at zero after every call, so the buffer is zeroed exactly once, at allocation."""

    def __init__(self, nbytes: int, device):
        self.buf = torch.zeros(max(int(nbytes), 4096), dtype=torch.uint8, device=device)
        # Buffers replaced by larger ones stay allocated: HIP graphs captured while they were current hold their raw
        # pointers (slabs, arrival counters, attention splits).  Each buffer's counters are only ever touched by the
        # launches that captured it, so old graphs and new launches never share state.
        self.retired = []

    def ensure(self, nbytes: int):
        if self.buf.numel() < nbytes:
            self.retired.append(self.buf)
            self.buf = torch.zeros(max(int(nbytes), 2 * self.buf.numel()), dtype=torch.uint8, device=self.buf.device)

    @property
    def ptr(self):
        return self.buf.data_ptr()

    @property
    def nbytes(self):
        return self.buf.numel()


# ---- activations in MFMA-fragment order (TGIS_LD_FRAGMENTS) ------------------------------------------------------------
LD_FRAGMENTS = -32


class FragAct:
    """A [M <= 64, K] f16 activation stored in fragment order (include/tgis_hip.h, TGIS_LD_FRAGMENTS): what the decode
    step's norm / attention / SiLU epilogue hand to the int4 GEMM behind them.  `buf` holds ceil(M / 32) * 32 * K elements."""

    def __init__(self, buf: torch.Tensor, M: int, K: int):
        assert 1 <= M <= 64 and K % 64 == 0 and buf.dtype == torch.float16 and buf.numel() == (M + 31) // 32 * 32 * K
        self.buf, self.M, self.K = buf, M, K
        self.dtype, self.device = buf.dtype, buf.device

    @property
    def shape(self):
        return (self.M, self.K)

    @staticmethod
    def empty(M: int, K: int, device) -> "FragAct":
        return FragAct(torch.empty((M + 31) // 32 * 32 * K, dtype=torch.float16, device=device), M, K)

    @staticmethod
    def from_rows(x: torch.Tensor) -> "FragAct":
        """Row-major [M, K] -> fragment order (torch ops; tests and cold paths only)."""
        M, K = x.shape
        rb = (M + 31) // 32
        full = torch.zeros((rb * 32, K), dtype=x.dtype, device=x.device)
        full[:M] = x
        # (row block, m, step, half, i, e) -> [row block][step][i][half][m][e]
        f = full.view(rb, 32, K // 64, 2, 4, 8).permute(0, 2, 4, 3, 1, 5).contiguous().view(-1)
        return FragAct(f, M, K)

    def to_rows(self) -> torch.Tensor:
        K, rb = self.K, (self.M + 31) // 32
        return self.buf.view(rb, K // 64, 4, 2, 32, 8).permute(0, 4, 1, 3, 2, 5).reshape(rb * 32, K)[:self.M].contiguous()


def gptq_fragments_ok(M: int, w: "GptqWeight", act: int = 0) -> bool:
    """Should an M-row activation reach this int4 GEMM in fragment order (tgis_gptq_fragments_ok)?  act 3 = the rope image."""
    key = ("frag_ok", M, act)
    cache = w.__dict__.setdefault("_frag_ok", {})
    got = cache.get(key)
    if got is None:
        got = cache[key] = bool(load_library().tgis_gptq_fragments_ok(M, w.K, w.N, w.groups, int(w.perm is not None), act))
    return got


# ---- GPTQ ------------------------------------------------------------------------------------------
class GptqWeight:
    """Prepared (repacked) GPTQ matrix; owner of the device image. Mirrors the q_handle of
    Ex4bitLinearV2.post_init (utils/gptq/exllamav2.py:124-137)."""

    def __init__(self, qweight, qzeros, scales, g_idx, bits: int, groupsize: int, gate_up: bool = False,
                 rope: Optional[tuple] = None):
        """rope = (D, rotated heads): the image of a fused qkv projection for gptq_gemm_rope (TGIS_GPTQ_ROPE_IMAGE)."""
        self.flags = 1 if gate_up else 0
        if rope is not None:
            assert not gate_up
            self.flags = 2 | (int(rope[0]) << 8) | (int(rope[1]) << 20)
        self.partial_plan = {}  # pass count -> (slab bytes, S, ld) of the deferred-reduce form, filled on first use
        if bits != 4:
            raise TgisHipError("only 4-bit GPTQ is supported (exllamav2.py:105)")
        lib = load_library()
        self.K = qweight.shape[0] * 8
        self.N = qweight.shape[1]
        self.groups = qzeros.shape[0]
        if self.K % 32 or self.N % 32:
            raise TgisHipError("GPTQ height and width must be multiples of 32 (exllamav2.py:118-119)")
        dev = qweight.device
        nbytes = lib.tgis_gptq_prepared_bytes(self.K, self.N, self.groups)
        self.image = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        qweight = qweight.contiguous()
        qzeros = qzeros.contiguous()
        scales = scales.to(torch.float16).contiguous()
        self.perm = None
        self.in_features = self.K  # columns of the activation (differs from K only for padded act-order row shards)
        gi = None
        perm_buf = None
        explicit = None
        if isinstance(g_idx, tuple):  # ("perm", gather index [K] with -1 = zero, activation columns): rows are in image order
            _, explicit, self.in_features = g_idx
            assert explicit.numel() == self.K
            g_idx = None
        if g_idx is not None:
            gi = g_idx.to("cpu", torch.int32).contiguous()
            perm_buf = torch.empty(self.K, dtype=torch.int32, device=dev)
        _check(
            lib.tgis_gptq_prepare(
                _ptr(qweight), _ptr(qzeros), _ptr(scales), gi.data_ptr() if gi is not None else None,
                _ptr(perm_buf), self.K, self.N, self.groups, self.flags, _ptr(self.image), _stream()),
            "tgis_gptq_prepare")
        if gi is not None:
            gs = self.K // self.groups
            trivial = bool((gi == (torch.arange(self.K, dtype=torch.int32) // gs)).all())
            if not trivial:
                self.perm = perm_buf
        if explicit is not None:
            self.perm = explicit.to(dev, torch.int32).contiguous()
        torch.cuda.current_stream().synchronize()  # qweight/qzeros/scales may be freed by the caller

    def workspace_bytes(self, M: int) -> int:
        return load_library().tgis_gptq_gemm_workspace_bytes(M, self.K, self.N)

    def fused_rows(self, act: int = 0) -> int:
        """Largest M the fused kernels of tgis_gptq_gemm_f16 should be given (beyond: dequantise + library GEMM)."""
        return load_library().tgis_gptq_gemm_fused_rows(self.K, self.groups, int(self.perm is not None), act)


def gptq_gemm(x, w: GptqWeight, ws: Workspace, bias=None, act: int = 0, out=None, out_frag: bool = False):
    """act 0: out[M,N] = x @ dequant(W) (+bias); act 1: x is [M,2K], silu(x[:, :K]) * x[:, K:] is the operand;
    act 2 (weight prepared with gate_up=True): out[M,N/2] = silu(gate) * up.
    x may be a FragAct (decode, M <= 64); with act 2 the result may then leave as a FragAct too (out_frag)."""
    assert act != 2 or w.flags & 1, "act=2 needs a weight prepared with gate_up=True"
    if isinstance(x, FragAct):
        assert x.K == w.K and act in (0, 2) and w.perm is None
        M = x.M
        if out_frag:
            assert act == 2 and out is None
            res = FragAct.empty(M, w.N // 2, x.device)
            optr, ldo = _ptr(res.buf), LD_FRAGMENTS
        else:
            res = out if out is not None else torch.empty((M, w.N // 2 if act == 2 else w.N), dtype=torch.float16,
                                                          device=x.device)
            optr, ldo = _ptr(res), res.stride(0)
        ws.ensure(w.workspace_bytes(M))
        _check(
            load_library().tgis_gptq_gemm_f16(_ptr(x.buf), LD_FRAGMENTS, _ptr(w.image), _ptr(bias), None, optr, ldo, M, w.K,
                                              w.N, w.groups, act, ws.ptr, ws.nbytes, _stream()), "tgis_gptq_gemm_f16")
        return res
    assert not out_frag, "a fragment-order output needs a fragment-order activation"
    assert x.dtype == torch.float16 and x.dim() == 2 and x.stride(1) == 1
    M = x.shape[0]
    assert x.shape[1] == (2 * w.in_features if act == 1 else w.in_features), (x.shape, w.in_features, act)
    assert act != 1 or w.in_features == w.K
    if out is None:
        out = torch.empty((M, w.N // 2 if act == 2 else w.N), dtype=torch.float16, device=x.device)
    ws.ensure(w.workspace_bytes(M))
    _check(
        load_library().tgis_gptq_gemm_f16(_ptr(x), x.stride(0), _ptr(w.image), _ptr(bias), _ptr(w.perm), _ptr(out),
                                          out.stride(0), M, w.K, w.N, w.groups, act, ws.ptr, ws.nbytes, _stream()),
        "tgis_gptq_gemm_f16")
    return out


class Partial:
    """fp32 split-K partial sums [ceil(M/32), S, 32, ld] of a GEMM whose reduce is deferred to the consumer kernel
    (rmsnorm_residual / rope_kv_write accept it in place of the f16 activation)."""

    def __init__(self, slabs: torch.Tensor, S: int, ld: int, M: int, N: int, bias):
        self.slabs, self.S, self.ld, self.M, self.N, self.bias = slabs, S, ld, M, N, bias
        self.dtype = torch.float16
        self.device = slabs.device

    @property
    def shape(self):
        return (self.M, self.N)


PARTIAL_MAX_M = 256  # rows up to which a GEMM may leave its split-K sum to the consumer kernel


def gptq_gemm_partial(x: torch.Tensor, w: GptqWeight, bias=None, act: int = 0) -> Partial:
    """Launch the GEMM but leave the split-K reduce (and bias) to the consumer.  Slabs are stored in 32-row units:
    [ceil(M/32)][S][32][ld]."""
    lib = load_library()
    if isinstance(x, FragAct):  # decode, <= 64 rows: the fragment-order kernel and ITS split plan
        assert x.K == w.K and act == 0 and w.perm is None
        # the split plan of the fragment-order kernel depends on the row class (plan_wide: <= 32 rows / 33 - 64 rows)
        M, key, xp, ldx = x.M, ("frag", x.M > 32), _ptr(x.buf), LD_FRAGMENTS
    else:
        assert x.dtype == torch.float16 and x.dim() == 2 and x.stride(1) == 1 and x.shape[0] <= PARTIAL_MAX_M
        M = x.shape[0]
        key, xp, ldx = ((M + 63) // 64 if M > 32 else 0), _ptr(x), x.stride(0)  # plan depends on M through its pass count
    plan = w.partial_plan.get(key)  # (slab bytes, S, ld): asked from the library once per weight and pass count
    if plan is None:
        nbytes = lib.tgis_gptq_gemm_partial_bytes(M, w.K, w.N)
        slabs = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
        S = _c_int()
        ld = _c_i64()
        _check(
            lib.tgis_gptq_gemm_f16_partial(xp, ldx, _ptr(w.image), _ptr(w.perm), M, w.K, w.N,
                                           w.groups, act, _ptr(slabs), nbytes, ctypes.byref(S), ctypes.byref(ld),
                                           _stream()), "tgis_gptq_gemm_f16_partial")
        w.partial_plan[key] = (nbytes, S.value, ld.value)
        return Partial(slabs, S.value, ld.value, M, w.N, bias)
    nbytes, S, ld = plan
    slabs = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    _check(
        lib.tgis_gptq_gemm_f16_partial(xp, ldx, _ptr(w.image), _ptr(w.perm), M, w.K, w.N,
                                       w.groups, act, _ptr(slabs), nbytes, None, None, _stream()),
        "tgis_gptq_gemm_f16_partial")
    return Partial(slabs, S, ld, M, w.N, bias)


def gptq_rope_ok(M: int, w: GptqWeight, D: int) -> bool:
    return bool(load_library().tgis_gptq_rope_ok(M, w.K, w.N, w.groups, int(w.perm is not None), D))


def rope_gemm_ok(M: int, w, D: int) -> bool:
    """Whether the fused qkv + rotary + cache-write launch should serve M rows of this weight (int4 or dense image)."""
    key = ("rope_ok", M)
    cache = w.__dict__.setdefault("_rope_ok", {})
    got = cache.get(key)
    if got is None:
        if isinstance(w, GptqWeight):
            got = gptq_rope_ok(M, w, D)
        else:
            got = bool(load_library().tgis_dense_rope_ok(M, w.K, w.N, D))
        cache[key] = got
    return got


def gptq_gemm_rope(x: torch.Tensor, w: GptqWeight, bias, cos, sin, positions, slots, k_pool, v_pool, H: int, Hkv: int,
                   D: int, out=None) -> torch.Tensor:
    """qkv projection + rotary embedding + cache write in one launch (decode, M <= 64; `w` is the rope image of the fused
    qkv weight).  Returns a [M, (H + 2 Hkv) D] tensor whose first H D columns hold the rotated q (the k / v columns are not
    written: they went straight into their cache pages)."""
    if isinstance(x, FragAct):
        assert x.K == w.K
        M, xp, ldx = x.M, _ptr(x.buf), LD_FRAGMENTS
    else:
        assert x.dtype == torch.float16 and x.dim() == 2 and x.stride(1) == 1 and x.shape[1] == w.K
        M, xp, ldx = x.shape[0], _ptr(x), x.stride(0)
    assert w.flags & 2 and w.N == (H + 2 * Hkv) * D
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32 and cos.dtype == torch.float16
    assert cos.shape[1] * 2 == D, "the fused epilogue covers the full rotary span only"
    if out is None:
        out = torch.empty((M, w.N), dtype=torch.float16, device=x.device)
    _check(
        load_library().tgis_gptq_gemm_rope_f16(xp, ldx, _ptr(w.image), _ptr(bias), _ptr(positions), _ptr(slots),
                                               _ptr(cos), _ptr(sin), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool),
                                               M, w.K, w.N, w.groups, H, Hkv, D, _stream()),
        "tgis_gptq_gemm_rope_f16")
    return out


def gptq_dequant(w: GptqWeight) -> torch.Tensor:
    """Dense f16 [K,N] (rows in the prepared order: permuted by w.perm for act-order matrices)."""
    out = torch.empty((w.K, w.N), dtype=torch.float16, device=w.image.device)
    _check(load_library().tgis_gptq_dequant_f16(_ptr(w.image), _ptr(out), w.K, w.N, w.groups, w.flags, _stream()),
           "tgis_gptq_dequant_f16")
    return out


# ---- dense ------------------------------------------------------------------------------------------
class DenseWeight:
    """torch-Linear weight [N,K] repacked into MFMA tile order.  gate_up=True: the weight is the Llama MLP's
    [gate | up] and the image interleaves the pairs for the SiLU*up epilogue (dense_gemm(act=2))."""

    def __init__(self, weight: torch.Tensor, gate_up: bool = False, rope: Optional[tuple] = None):
        lib = load_library()
        assert weight.dim() == 2
        self.N, self.K = weight.shape
        self.dtype = weight.dtype
        self.flags = 1 if gate_up else 0
        if rope is not None:  # (D, rotated heads): the image of a fused qkv projection for dense_gemm_rope
            assert not gate_up
            self.flags = 2 | (int(rope[0]) << 8) | (int(rope[1]) << 20)
        weight = weight.contiguous()
        self.image = torch.empty(lib.tgis_dense_prepared_bytes(self.N, self.K), dtype=torch.uint8,
                                 device=weight.device)
        _check(lib.tgis_dense_prepare(_ptr(weight), self.N, self.K, dtype_code(weight.dtype), self.flags,
                                      _ptr(self.image), _stream()), "tgis_dense_prepare")
        torch.cuda.current_stream().synchronize()

    def workspace_bytes(self, M: int) -> int:
        return load_library().tgis_dense_gemm_workspace_bytes(M, self.K, self.N)


def dense_gemm(x: torch.Tensor, w: DenseWeight, ws: Workspace, bias=None, out_f32: bool = False, act: int = 0,
               out=None) -> torch.Tensor:
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype == w.dtype
    M = x.shape[0]
    assert x.shape[1] == (2 * w.K if act == 1 else w.K)
    assert (act == 2) == bool(w.flags & 1), "act 2 runs on (and only on) a gate|up image"
    if out is None:
        out = torch.empty((M, w.N // 2 if act == 2 else w.N), dtype=torch.float32 if out_f32 else w.dtype,
                          device=x.device)
    ws.ensure(w.workspace_bytes(M))
    _check(
        load_library().tgis_dense_gemm(_ptr(x), x.stride(0), _ptr(w.image), _ptr(bias), _ptr(out), out.stride(0), M,
                                       w.K, w.N, dtype_code(w.dtype), int(out_f32), act, ws.ptr, ws.nbytes,
                                       _stream()), "tgis_dense_gemm")
    return out


def dense_gemm_partial(x: torch.Tensor, w: DenseWeight, bias=None, act: int = 0) -> Partial:
    """Launch the dense GEMM but leave the split-K reduce (and bias) to the consumer kernel."""
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype == w.dtype and x.shape[0] <= PARTIAL_MAX_M
    lib = load_library()
    nbytes = lib.tgis_dense_gemm_partial_bytes(x.shape[0], w.K, w.N)
    slabs = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    S = _c_int()
    ld = _c_i64()
    _check(
        lib.tgis_dense_gemm_partial(_ptr(x), x.stride(0), _ptr(w.image), x.shape[0], w.K, w.N, dtype_code(w.dtype), act,
                                    _ptr(slabs), nbytes, ctypes.byref(S), ctypes.byref(ld), _stream()),
        "tgis_dense_gemm_partial")
    p = Partial(slabs, S.value, ld.value, x.shape[0], w.N, bias)
    p.dtype = w.dtype
    return p


def dense_gemm_rope(x: torch.Tensor, w: DenseWeight, bias, cos, sin, positions, slots, k_pool, v_pool, H: int, Hkv: int,
                    D: int, out=None) -> torch.Tensor:
    """Dense qkv projection + rotary embedding + cache write in one launch (decode, M <= 64; `w` is the rope image of the
    fused qkv weight).  Returns [M, (H + 2 Hkv) D] whose first H D columns hold the rotated q."""
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype == w.dtype and x.shape[1] == w.K
    assert w.flags & 2 and w.N == (H + 2 * Hkv) * D and cos.dtype == w.dtype and cos.shape[1] * 2 == D
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32
    M = x.shape[0]
    if out is None:
        out = torch.empty((M, w.N), dtype=w.dtype, device=x.device)
    _check(
        load_library().tgis_dense_gemm_rope(_ptr(x), x.stride(0), _ptr(w.image), _ptr(bias), _ptr(positions), _ptr(slots),
                                            _ptr(cos), _ptr(sin), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), M,
                                            w.K, w.N, H, Hkv, D, dtype_code(w.dtype), _stream()),
        "tgis_dense_gemm_rope")
    return out


def clear_error() -> None:
    """Drop a stale HIP error (aborted graph capture) so that it is not blamed on the next launch."""
    load_library().tgis_clear_error()


# ---- norms --------------------------------------------------------------------------------------------
def rmsnorm_residual(x, residual, weight, eps: float, y=None, res_out=None, frag: bool = False):
    """(y, res) = fused add + RMSNorm; mirrors LlamaRMSNorm.forward (flash_llama_modeling.py:113-152).
    frag (rows <= 32, f16): y is returned as a FragAct, the layout the int4 GEMM behind the norm reads."""
    rows, hidden = x.shape
    yf = None
    if frag:
        assert y is None and rows <= 64 and hidden % 64 == 0 and x.dtype == torch.float16
        yf = FragAct.empty(rows, hidden, x.device)
        y, ldy = yf.buf, LD_FRAGMENTS
    else:
        ldy = hidden
    if isinstance(x, Partial):
        if y is None:
            y = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
        if res_out is None:
            res_out = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)  # the reduced (+ residual) stream
        _check(
            load_library().tgis_rmsnorm_residual_partial(_ptr(x.slabs), x.S, x.ld, _ptr(x.bias), _ptr(residual),
                                                         _ptr(weight), _ptr(y), ldy, _ptr(res_out), rows, hidden,
                                                         float(eps), dtype_code(x.dtype), _stream()),
            "tgis_rmsnorm_residual_partial")
        return (yf if frag else y), res_out
    assert x.dim() == 2 and x.is_contiguous()
    if y is None:
        y = torch.empty_like(x)
    if res_out is None:
        res_out = torch.empty_like(x) if residual is not None else x
    _check(
        load_library().tgis_rmsnorm_residual(_ptr(x), _ptr(residual), _ptr(weight), _ptr(y), ldy,
                                             _ptr(res_out) if residual is not None else None, rows, hidden,
                                             float(eps), dtype_code(x.dtype), _stream()), "tgis_rmsnorm_residual")
    return (yf if frag else y), res_out


def layernorm_residual(x, residual, weight, bias, eps: float, y=None, res_out=None):
    """(y, res) = fused add + LayerNorm; mirrors FastLayerNorm.forward (utils/layers.py:363-396)."""
    if isinstance(x, Partial):
        rows, hidden = x.shape
        if y is None:
            y = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
        if res_out is None:
            res_out = torch.empty_like(y)  # always materialised: it is the reduced (+residual) stream
        _check(
            load_library().tgis_layernorm_residual_partial(_ptr(x.slabs), x.S, x.ld, _ptr(x.bias), _ptr(residual),
                                                           _ptr(weight), _ptr(bias), _ptr(y), _ptr(res_out), rows,
                                                           hidden, float(eps), dtype_code(x.dtype), _stream()),
            "tgis_layernorm_residual_partial")
        return y, res_out
    assert x.dim() == 2 and x.is_contiguous()
    rows, hidden = x.shape
    if y is None:
        y = torch.empty_like(x)
    if res_out is None:
        res_out = torch.empty_like(x) if residual is not None else x
    _check(
        load_library().tgis_layernorm_residual(_ptr(x), _ptr(residual), _ptr(weight), _ptr(bias), _ptr(y),
                                               _ptr(res_out) if residual is not None else None, rows, hidden,
                                               float(eps), dtype_code(x.dtype), _stream()),
        "tgis_layernorm_residual")
    return y, res_out


# ---- rope + kv write, attention --------------------------------------------------------------------------
def rope_kv_write(qkv, cos, sin, positions, slots, k_pool, v_pool, H: int, Hkv: int, D: int, rot_dim: int):
    """Rotates q,k in place and writes k,v to the cache.  `qkv` may be a Partial: the reduced, rotated activation is
    then materialised into a fresh [T, (H+2Hkv)D] tensor, which is returned (the plain form returns qkv itself)."""
    if isinstance(qkv, Partial):
        T = qkv.M
        out = torch.empty((T, qkv.N), dtype=qkv.dtype, device=qkv.device)
        _check(
            load_library().tgis_rope_kv_write_partial(_ptr(qkv.slabs), qkv.S, qkv.ld, _ptr(qkv.bias), _ptr(out),
                                                      out.stride(0), _ptr(cos), _ptr(sin), _ptr(positions),
                                                      _ptr(slots), _ptr(k_pool), _ptr(v_pool), T, H, Hkv, D, rot_dim,
                                                      dtype_code(out.dtype), _stream()), "tgis_rope_kv_write_partial")
        return out
    assert qkv.dim() == 2 and qkv.stride(1) == 1
    T = qkv.shape[0]
    _check(
        load_library().tgis_rope_kv_write(_ptr(qkv), qkv.stride(0), _ptr(cos), _ptr(sin), _ptr(positions),
                                          _ptr(slots), _ptr(k_pool), _ptr(v_pool), T, H, Hkv, D, rot_dim,
                                          dtype_code(qkv.dtype), _stream()), "tgis_rope_kv_write")
    return qkv


def rope_kv_write_prefill(qkv, cos, sin, positions, cu_seqlens, block_tables, k_pool, v_pool, max_len: int, H: int,
                          Hkv: int, D: int, rot_dim: int):
    """rope_kv_write for a fresh prefill (token i of a sequence = cache position i): page-wise cache writes."""
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and block_tables.is_contiguous()
    B = block_tables.shape[0]
    _check(
        load_library().tgis_rope_kv_write_prefill(_ptr(qkv), qkv.stride(0), _ptr(cos), _ptr(sin), _ptr(positions),
                                                  _ptr(cu_seqlens), _ptr(block_tables), block_tables.shape[1],
                                                  _ptr(k_pool), _ptr(v_pool), B, qkv.shape[0], max_len, H, Hkv, D,
                                                  rot_dim, dtype_code(qkv.dtype), _stream()),
        "tgis_rope_kv_write_prefill")
    return qkv


def attn_num_splits(B: int, Hkv: int, H: int, max_q_len: int, max_ctx: int) -> int:
    return load_library().tgis_attn_num_splits(B, Hkv, H, max_q_len, max_ctx)


def attn_workspace_bytes(total_q: int, H: int, Hkv: int, D: int, num_splits: int) -> int:
    return load_library().tgis_attn_workspace_bytes(total_q, H, Hkv, D, num_splits)


def attn_paged(q, ld_q: int, k_pool, v_pool, block_tables, ctx_lens, cu_seqlens_q, out, B: int, H: int, Hkv: int,
               D: int, max_q_len: int, max_ctx: int, scale: float, num_splits: int, ws: Optional[Workspace]):
    """q is a (view into a) [T, *] activation whose row stride is ld_q elements; out [T, H*D], or (decode, B <= 32) a
    FragAct of that shape for the o_proj GEMM."""
    assert block_tables.dtype == torch.int32 and ctx_lens.dtype == torch.int32 and cu_seqlens_q.dtype == torch.int32
    assert block_tables.is_contiguous()
    if isinstance(out, FragAct):
        assert max_q_len == 1 and out.K == H * D and out.M == B
        optr, ldo = _ptr(out.buf), LD_FRAGMENTS
    else:
        assert out.is_contiguous()
        optr, ldo = _ptr(out), H * D
    wptr, wbytes = (ws.ptr, ws.nbytes) if ws is not None else (None, 0)
    _check(
        load_library().tgis_attn_paged(_ptr(q), ld_q, _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
                                       block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_seqlens_q), optr, ldo, B, H,
                                       Hkv, D, max_q_len, max_ctx, float(scale), dtype_code(q.dtype), num_splits,
                                       wptr, wbytes, _stream()), "tgis_attn_paged")
    return out


# ---- elementwise / sampling ---------------------------------------------------------------------------------
def act_mul(gate_up, I: int, out=None):
    T = gate_up.shape[0]
    assert gate_up.is_contiguous() and gate_up.shape[1] == 2 * I
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _check(load_library().tgis_act_mul(_ptr(gate_up), _ptr(out), T, I, 1, dtype_code(gate_up.dtype), _stream()),
           "tgis_act_mul")
    return out


def gelu(x, tanh_approx: bool, out=None):
    assert x.is_contiguous()
    if out is None:
        out = torch.empty_like(x)
    _check(load_library().tgis_gelu(_ptr(x), _ptr(out), x.numel(), int(tanh_approx), dtype_code(x.dtype), _stream()),
           "tgis_gelu")
    return out


def embedding(ids, table, positions=None, pos_table=None, id_offset: int = 0, out=None):
    assert ids.dtype == torch.int64 and ids.is_contiguous() and table.is_contiguous()
    T = ids.numel()
    E = table.shape[1]
    if out is None:
        out = torch.empty((T, E), dtype=table.dtype, device=table.device)
    _check(
        load_library().tgis_embedding(_ptr(ids), _ptr(table), _ptr(positions), _ptr(pos_table), _ptr(out), T, E,
                                      table.shape[0], id_offset, dtype_code(table.dtype), _stream()),
        "tgis_embedding")
    return out


def decode_slots(positions, block_tables, slots, ctx_lens):
    B = positions.numel()
    _check(
        load_library().tgis_decode_slots(_ptr(positions), _ptr(block_tables), block_tables.shape[1], _ptr(slots),
                                         _ptr(ctx_lens), B, _stream()), "tgis_decode_slots")


def decode_advance(ids, position_ids, all_input_ids=None, cu_seqlens=None, cu_seqlens_q=None, stage_ids=None,
                   stage_positions=None):
    """After a decode step (flash_causal_lm.py:457,499,533-535 in one launch): position_ids += 1 in place, the new ids
    scattered into all_input_ids at the new positions, cu_seqlens += cu_seqlens_q in place; returns a private copy of
    `ids`.  stage_ids / stage_positions (a decode graph's static inputs) receive the next step's inputs as well."""
    B = ids.numel()
    assert ids.dtype == torch.int64 and position_ids.dtype == torch.int64 and position_ids.numel() == B
    assert ids.is_contiguous() and position_ids.is_contiguous()
    out = torch.empty_like(ids)
    ld = 0
    if all_input_ids is not None:
        assert all_input_ids.dtype == torch.int64 and all_input_ids.stride(1) == 1 and all_input_ids.shape[0] >= B
        ld = all_input_ids.stride(0)
    if cu_seqlens is not None:
        assert cu_seqlens.dtype == torch.int32 and cu_seqlens_q.dtype == torch.int32
        assert cu_seqlens.numel() == B + 1 and cu_seqlens_q.numel() == B + 1
    if stage_ids is not None:
        assert stage_ids.dtype == torch.int64 and stage_ids.numel() == B
    if stage_positions is not None:
        assert stage_positions.dtype == torch.int32 and stage_positions.numel() == B
    _check(
        load_library().tgis_decode_advance(_ptr(ids), _ptr(out), _ptr(position_ids), _ptr(all_input_ids), ld,
                                           _ptr(cu_seqlens), _ptr(cu_seqlens_q), _ptr(stage_ids), _ptr(stage_positions),
                                           B, _stream()), "tgis_decode_advance")
    return out


def argmax_scratch(B: int, device) -> torch.Tensor:
    """Scratch that lets argmax_logprob split the rows of a small batch over several workgroups each."""
    return torch.empty(max(16, load_library().tgis_argmax_scratch_bytes(B)), dtype=torch.uint8, device=device)


def argmax_logprob(logits, ids_out=None, logprob_out=None, scratch=None):
    assert logits.dim() == 2 and logits.stride(1) == 1
    B, V = logits.shape
    if ids_out is None:
        ids_out = torch.empty(B, dtype=torch.int64, device=logits.device)
    if logprob_out is None:
        logprob_out = torch.empty(B, dtype=torch.float32, device=logits.device)
    f32 = logits.dtype == torch.float32
    _check(
        load_library().tgis_argmax_logprob(_ptr(logits), logits.stride(0), B, V, int(f32),
                                           0 if f32 else dtype_code(logits.dtype), _ptr(ids_out),
                                           _ptr(logprob_out), _ptr(scratch), scratch.numel() if scratch is not None else 0,
                                           _stream()), "tgis_argmax_logprob")
    return ids_out, logprob_out


def warp_sample(logits, temperature=None, top_k=None, top_p_cut=None, typical_p=None, rep_penalty=None,
                input_ids=None, exclude_id: int = -1, eos_adjust=None, eos_id: int = -1, do_sample=None, rng=None):
    """The whole next-token chooser for a batch in one launch (tgis_warp_sample).  Returns (next_ids int64 [B],
    logprob f32 [B] of the chosen ids under the warped scores, lse f32 [B], warped scores f32 [B,V])."""
    assert logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1
    B, V = logits.shape
    dev = logits.device
    for t, dt in ((temperature, torch.float32), (top_k, torch.int32), (top_p_cut, torch.float32),
                  (typical_p, torch.float32), (rep_penalty, torch.float32), (do_sample, torch.int32)):
        assert t is None or (t.dtype == dt and t.numel() == B and t.is_contiguous() and t.device == dev)
    assert rng is None or (rng.dtype == torch.int64 and rng.shape == (B, 2) and rng.is_contiguous())
    assert eos_adjust is None or (eos_adjust.dtype == torch.float32 and eos_adjust.shape == (B, 2)
                                  and eos_adjust.is_contiguous())
    L = ld_ids = 0
    if input_ids is not None:
        assert input_ids.dtype == torch.int64 and input_ids.dim() == 2 and input_ids.shape[0] == B
        assert input_ids.stride(1) == 1
        L, ld_ids = input_ids.shape[1], input_ids.stride(0)
    scores = torch.empty((B, V), dtype=torch.float32, device=dev)
    ids = torch.empty(B, dtype=torch.int64, device=dev)
    lps = torch.empty(B, dtype=torch.float32, device=dev)
    lse = torch.empty(B, dtype=torch.float32, device=dev)
    _check(
        load_library().tgis_warp_sample(
            _ptr(logits), logits.stride(0), _ptr(scores), V, B, V, _ptr(temperature), _ptr(top_k), _ptr(top_p_cut),
            _ptr(typical_p), _ptr(rep_penalty), _ptr(input_ids), ld_ids, L, exclude_id, _ptr(eos_adjust), eos_id,
            _ptr(do_sample), _ptr(rng), _ptr(ids), _ptr(lps), _ptr(lse), _stream()), "tgis_warp_sample")
    return ids, lps, lse, scores


# ---- fp32-residual / ragged-step family ---------------------------------------------------------------------------------
def dtype_code3(dt: torch.dtype) -> int:
    """float16 / bfloat16 / float32: the entry points of the fp32-residual family take all three."""
    if dt == torch.float32:
        return F32
    return dtype_code(dt)


def _f32(t: Optional[torch.Tensor], what: str):
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
        raise TgisHipError(f"{what} must be a contiguous float32 tensor")
    return _ptr(t)


def _i32(t: Optional[torch.Tensor], what: str):
    if t is not None and (t.dtype != torch.int32 or not t.is_contiguous()):
        raise TgisHipError(f"{what} must be a contiguous int32 tensor")
    return _ptr(t)


def embedding_scaled_f32(ids: torch.Tensor, table: torch.Tensor, scale: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    assert ids.dtype == torch.int64 and ids.dim() == 1 and table.dim() == 2 and table.is_contiguous()
    if out is None:
        out = torch.empty((ids.shape[0], table.shape[1]), dtype=torch.float32, device=table.device)
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape == (ids.shape[0], table.shape[1])
    _check(load_library().tgis_embedding_scaled_f32(_ptr(ids), _ptr(table), _ptr(out), ids.shape[0], table.shape[1],
                                                    table.shape[0], float(scale), dtype_code3(table.dtype), _stream()),
           "tgis_embedding_scaled_f32")
    return out


def sandwich_norm_f32(x: torch.Tensor, delta: Optional[torch.Tensor], post_w: Optional[torch.Tensor],
                      pre_w: Optional[torch.Tensor], eps: float, y_dtype: Optional[torch.dtype] = None, post_add: float = 1.0,
                      pre_add: float = 1.0):
    """x [rows, E] fp32 is updated in place with the normed `delta` (if any); returns the pre-normed y (or None)."""
    rows, E = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    y = torch.empty((rows, E), dtype=y_dtype, device=x.device) if pre_w is not None else None
    if isinstance(delta, Partial):  # the split-K slabs of the GEMM before: summed inside the launch
        assert delta.shape == (rows, E) and delta.bias is None
        _check(load_library().tgis_sandwich_norm_f32_partial(
            _ptr(x), _ptr(delta.slabs), delta.S, delta.ld, _f32(post_w, "post_w"), float(post_add), _ptr(x),
            _f32(pre_w, "pre_w"), float(pre_add), _ptr(y), dtype_code3(y_dtype) if y is not None else F32, rows, E, float(eps),
            _stream()), "tgis_sandwich_norm_f32_partial")
        return y
    if delta is not None:
        assert delta.shape == x.shape and delta.stride(1) == 1
    _check(load_library().tgis_sandwich_norm_f32(
        _ptr(x), _ptr(delta), delta.stride(0) if delta is not None else 0, dtype_code3(delta.dtype) if delta is not None else F32,
        _f32(post_w, "post_w"), float(post_add), _ptr(x), _f32(pre_w, "pre_w"), float(pre_add), _ptr(y),
        dtype_code3(y_dtype) if y is not None else F32, rows, E, float(eps), _stream()), "tgis_sandwich_norm_f32")
    return y


def dense_gemm_clamped_glu(x: torch.Tensor, w: DenseWeight, ws: Workspace, alpha: float, limit: float) -> torch.Tensor:
    """x @ [gate | up] with g = min(gate, limit), u = clamp(up, +-limit), g * sigmoid(alpha g) * (u + 1) in the epilogue
    (decode-sized M; `w` is a gate | up image)."""
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype == w.dtype and x.shape[1] == w.K and w.flags & 1
    M = x.shape[0]
    out = torch.empty((M, w.N // 2), dtype=w.dtype, device=x.device)
    ws.ensure(w.workspace_bytes(M))
    _check(load_library().tgis_dense_gemm_clamped_glu(_ptr(x), x.stride(0), _ptr(w.image), _ptr(out), out.stride(0), M, w.K, w.N,
                                                      dtype_code(w.dtype), float(alpha), float(limit), ws.ptr, ws.nbytes,
                                                      _stream()), "tgis_dense_gemm_clamped_glu")
    return out


def glu(gate_up: torch.Tensor, I: int, mode: int = 0, alpha: float = 1.0, limit: float = 0.0) -> torch.Tensor:
    assert gate_up.dim() == 2 and gate_up.stride(1) == 1 and gate_up.shape[1] == 2 * I
    out = torch.empty((gate_up.shape[0], I), dtype=gate_up.dtype, device=gate_up.device)
    _check(load_library().tgis_glu(_ptr(gate_up), gate_up.stride(0), _ptr(out), I, gate_up.shape[0], I, mode, float(alpha),
                                   float(limit), dtype_code3(gate_up.dtype), _stream()), "tgis_glu")
    return out


def qk_norm_kv_write(qkv, positions, slots, q_gain, k_gain, eps: float, gain_coef: float, gain_every: int, v_first, v_lambda,
                     k_pool, v_pool, H: int, G: int, dk: int, dv: int):
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and k_pool.dtype == qkv.dtype and v_pool.dtype == qkv.dtype
    assert positions.shape[0] == qkv.shape[0] and slots.shape[0] == qkv.shape[0]
    assert v_first is None or (v_first.dtype == qkv.dtype and v_first.stride(1) == 1 and v_first.shape == (qkv.shape[0], G * dv))
    _check(load_library().tgis_qk_norm_kv_write(
        _ptr(qkv), qkv.stride(0), _i32(positions, "positions"), _i32(slots, "slots"), _f32(q_gain, "q_gain"),
        _f32(k_gain, "k_gain"), float(eps), float(gain_coef), int(gain_every), _ptr(v_first),
        v_first.stride(0) if v_first is not None else 0, _f32(v_lambda, "v_lambda") if v_first is not None else None,
        _ptr(k_pool), _ptr(v_pool), qkv.shape[0], H, G, dk, dv, dtype_code3(qkv.dtype), _stream()), "tgis_qk_norm_kv_write")


def attn_varlen(q, k_pool, v_pool, block_tables, ctx_lens, cu_seqlens_q, H: int, G: int, dk: int, dv: int, scale: float,
                max_q_len: int = 1, max_ctx: int = 1, impl: int = 0):
    """q [T, >= H dk] (row stride free); returns [T, H dv].  max_q_len: the longest run of one sequence in the step;
    max_ctx: the longest context; impl 0 auto / 1 general kernel / 2 matrix-core kernel."""
    assert q.dim() == 2 and q.stride(1) == 1 and block_tables.dim() == 2
    T = q.shape[0]
    out = torch.empty((T, H * dv), dtype=q.dtype, device=q.device)
    _check(load_library().tgis_attn_varlen(
        _ptr(q), q.stride(0), _ptr(k_pool), _ptr(v_pool), _i32(block_tables, "block_tables"), block_tables.shape[1],
        _i32(ctx_lens, "ctx_lens"), _i32(cu_seqlens_q, "cu_seqlens_q"), ctx_lens.shape[0], _ptr(out), out.stride(0), T,
        max(int(max_q_len), 1), max(int(max_ctx), 1), H, G, dk, dv, float(scale), impl, dtype_code3(q.dtype), _stream()),
        "tgis_attn_varlen")
    return out


def token_shift_mix(h, shift_state, state_slots, cu_seqlens_q, positions, mu, out_dtype):
    """h [T, W] fp32, mu [S, W] fp32 -> [S, T, W] in out_dtype."""
    T, W = h.shape
    out = torch.empty((mu.shape[0], T, W), dtype=out_dtype, device=h.device)
    _check(load_library().tgis_token_shift_mix(
        _f32(h, "h"), _f32(shift_state, "shift_state"), _i32(state_slots, "state_slots"), _i32(cu_seqlens_q, "cu_seqlens_q"),
        _i32(positions, "positions"), state_slots.shape[0], _f32(mu, "mu"), mu.shape[0], _ptr(out), T, W, dtype_code3(out_dtype),
        _stream()), "tgis_token_shift_mix")
    return out


def wkv_decay(a, w2t, w0):
    """a [T, rank] -> log decay [T, C] fp32."""
    assert a.dim() == 2 and a.stride(1) == 1 and w2t.shape[0] == a.shape[1]
    out = torch.empty((a.shape[0], w2t.shape[1]), dtype=torch.float32, device=a.device)
    _check(load_library().tgis_wkv_decay(_ptr(a), a.stride(0), _f32(w2t, "w2t"), _f32(w0, "w0"), _ptr(out), a.shape[0], a.shape[1],
                                         w2t.shape[1], dtype_code3(a.dtype), _stream()), "tgis_wkv_decay")
    return out


def wkv_scan(r, k, v, gate, logw, u, gain, state, shift_state, h, state_slots, cu_seqlens_q, positions, H: int, d: int, eps: float):
    """r / k / v / gate [T, H d] views with one common row stride; returns [T, H d]."""
    T = r.shape[0]
    ld = r.stride(0)
    assert all(t.stride(0) == ld and t.stride(1) == 1 and t.dtype == r.dtype for t in (k, v, gate))
    out = torch.empty((T, H * d), dtype=r.dtype, device=r.device)
    _check(load_library().tgis_wkv_scan(
        _ptr(r), _ptr(k), _ptr(v), _ptr(gate), ld, _f32(logw, "logw"), _f32(u, "u"), _f32(gain, "gain"), _f32(state, "state"),
        _f32(shift_state, "shift_state"), _f32(h, "h"), h.shape[1], _i32(state_slots, "state_slots"),
        _i32(cu_seqlens_q, "cu_seqlens_q"), _i32(positions, "positions"), _ptr(out), out.stride(0), state_slots.shape[0], H, d,
        float(eps), dtype_code3(r.dtype), _stream()), "tgis_wkv_scan")
    return out


def moe_row_capacity(n_pairs: int, E: int) -> int:
    return load_library().tgis_moe_row_capacity(n_pairs, E)


def moe_route(h, router_w, shared_gate_w, k: int, router_b=None, softmax_top: bool = False):
    """(idx int32 [T, k], weight fp32 [T, k], shared gate fp32 [T] or None).  weight: the sigmoid of each chosen logit, or
    (softmax_top) the softmax over the chosen logits only; router_b [E] fp32 is added to the logits."""
    T, W = h.shape
    E = router_w.shape[0]
    idx = torch.empty((T, k), dtype=torch.int32, device=h.device)
    weight = torch.empty((T, k), dtype=torch.float32, device=h.device)
    sg = torch.empty((T,), dtype=torch.float32, device=h.device) if shared_gate_w is not None else None
    if router_b is None and not softmax_top:
        _check(load_library().tgis_moe_route(_ptr(h), h.stride(0), _f32(router_w, "router_w"), _f32(shared_gate_w, "shared_gate_w"),
                                             _ptr(idx), _ptr(weight), _ptr(sg), T, W, E, k, dtype_code3(h.dtype), _stream()),
               "tgis_moe_route")
    else:
        _check(load_library().tgis_moe_route_ext(_ptr(h), h.stride(0), _f32(router_w, "router_w"), _f32(router_b, "router_b"),
                                                 _f32(shared_gate_w, "shared_gate_w"), int(softmax_top), _ptr(idx), _ptr(weight), _ptr(sg),
                                                 T, W, E, k, dtype_code3(h.dtype), _stream()), "tgis_moe_route_ext")
    return idx, weight, sg


def moe_align(idx: torch.Tensor, E: int):
    """(sorted [cap], tile_expert [cap / 32], pos_of_pair [pairs], n_tiles [1]) for idx [T, k]."""
    n = idx.numel()
    cap = moe_row_capacity(n, E)
    dev = idx.device
    sorted_ = torch.empty((cap,), dtype=torch.int32, device=dev)
    tile_expert = torch.empty((cap // 32,), dtype=torch.int32, device=dev)
    pos = torch.empty((n,), dtype=torch.int32, device=dev)
    n_tiles = torch.empty((1,), dtype=torch.int32, device=dev)
    _check(load_library().tgis_moe_align(_i32(idx, "idx"), n, E, _ptr(sorted_), cap, _ptr(tile_expert), _ptr(pos), _ptr(n_tiles),
                                         _stream()), "tgis_moe_align")
    return sorted_, tile_expert, pos, n_tiles


def moe_gemm(A, weights, N: int, tile_expert, n_tiles, capacity: int, sorted_=None, pair_div: int = 1, pair_scale=None,
             glu_act: bool = False):
    """weights [E, N (glu: 2 N), K]; returns [capacity, N]."""
    assert A.dim() == 2 and A.stride(1) == 1 and weights.dim() == 3 and weights.is_contiguous() and weights.dtype == A.dtype
    K = weights.shape[2]
    assert weights.shape[1] == (2 * N if glu_act else N) and A.shape[1] == K
    out = torch.empty((capacity, N), dtype=A.dtype, device=A.device)
    _check(load_library().tgis_moe_gemm(
        _ptr(A), A.stride(0), _i32(sorted_, "sorted"), pair_div, _f32(pair_scale, "pair_scale"), _ptr(tile_expert), _ptr(n_tiles),
        _ptr(weights), weights.stride(0), N, K, int(glu_act), _ptr(out), out.stride(0), capacity, dtype_code3(A.dtype), _stream()),
        "tgis_moe_gemm")
    return out


def moe_combine(rows, pos_of_pair, k: int, T: int, pair_weight=None, shared=None, shared_gate=None):
    W = rows.shape[1]
    out = torch.empty((T, W), dtype=rows.dtype, device=rows.device)
    _check(load_library().tgis_moe_combine(
        _ptr(rows), rows.stride(0), _i32(pos_of_pair, "pos_of_pair"), _f32(pair_weight, "pair_weight"), k, _ptr(shared),
        shared.stride(0) if shared is not None else 0, _f32(shared_gate, "shared_gate"), _ptr(out), out.stride(0), T, W,
        dtype_code3(rows.dtype), _stream()), "tgis_moe_combine")
    return out


# ---- pre-norm hybrids with a residual multiplier: residual update, activations, cache writes, delta rule ---------------------
def residual_update_f32(x: torch.Tensor, delta, post_w: Optional[torch.Tensor], pre_w: Optional[torch.Tensor], eps: float,
                        y_dtype: Optional[torch.dtype] = None, post_add: float = 0.0, pre_add: float = 0.0,
                        post_scale: float = 1.0, cast: bool = False):
    """x [rows, E] fp32 is updated in place: x += post_scale * delta (normed with post_w if given).  Returns y = norm(x) *
    (pre_w + pre_add) in y_dtype, or x rounded to y_dtype (`cast`, no pre_w), or None.  delta: a tensor or the split-K slabs
    of the projection before (`Partial`)."""
    rows, E = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    want_y = pre_w is not None or cast
    y = torch.empty((rows, E), dtype=y_dtype, device=x.device) if want_y else None
    yd = dtype_code3(y_dtype) if want_y else F32
    lib = load_library()
    if isinstance(delta, Partial):
        assert delta.shape == (rows, E) and delta.bias is None
        _check(lib.tgis_residual_update_f32_partial(
            _ptr(x), _ptr(delta.slabs), delta.S, delta.ld, _f32(post_w, "post_w"), float(post_add), float(post_scale), _ptr(x),
            _f32(pre_w, "pre_w"), float(pre_add), _ptr(y), yd, rows, E, float(eps), _stream()), "tgis_residual_update_f32_partial")
        return y
    if delta is not None:
        assert delta.shape == x.shape and delta.stride(1) == 1
    _check(lib.tgis_residual_update_f32(
        _ptr(x), _ptr(delta), delta.stride(0) if delta is not None else 0, dtype_code3(delta.dtype) if delta is not None else F32,
        _f32(post_w, "post_w"), float(post_add), float(post_scale), _ptr(x), _f32(pre_w, "pre_w"), float(pre_add), _ptr(y), yd,
        rows, E, float(eps), _stream()), "tgis_residual_update_f32")
    return y


def xielu(x: torch.Tensor, ap: float, an: float) -> torch.Tensor:
    assert x.dim() == 2 and x.stride(1) == 1
    out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    _check(load_library().tgis_xielu(_ptr(x), x.stride(0), _ptr(out), out.stride(0), x.shape[0], x.shape[1], float(ap), float(an),
                                     dtype_code3(x.dtype), _stream()), "tgis_xielu")
    return out


def dense_gemm_xielu(x: torch.Tensor, w: DenseWeight, ws: Workspace, ap: float, an: float) -> torch.Tensor:
    """xielu(x @ W^T) in one launch (decode-sized M, plain image)."""
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype == w.dtype and x.shape[1] == w.K and not w.flags
    M = x.shape[0]
    out = torch.empty((M, w.N), dtype=w.dtype, device=x.device)
    ws.ensure(w.workspace_bytes(M))
    _check(load_library().tgis_dense_gemm_xielu(_ptr(x), x.stride(0), _ptr(w.image), _ptr(out), out.stride(0), M, w.K, w.N,
                                                dtype_code(w.dtype), float(ap), float(an), ws.ptr, ws.nbytes, _stream()),
           "tgis_dense_gemm_xielu")
    return out


def dense_gemm_gelu_lookup(x: torch.Tensor, w: DenseWeight, ws: Workspace, ids: torch.Tensor, table: torch.Tensor, col0: int) -> torch.Tensor:
    """gelu_tanh(x @ W^T) * table[ids][:, col0:col0 + N] in one launch (decode-sized M, plain image)."""
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype == w.dtype and x.shape[1] == w.K and not w.flags
    assert table.dim() == 2 and table.stride(1) == 1 and table.dtype == w.dtype and ids.dtype == torch.int64 and ids.shape[0] == x.shape[0]
    M = x.shape[0]
    out = torch.empty((M, w.N), dtype=w.dtype, device=x.device)
    ws.ensure(w.workspace_bytes(M))
    _check(load_library().tgis_dense_gemm_gelu_lookup(_ptr(x), x.stride(0), _ptr(w.image), _ptr(ids), _ptr(table), table.stride(0),
                                                      int(col0), table.shape[0], _ptr(out), out.stride(0), M, w.K, w.N,
                                                      dtype_code(w.dtype), ws.ptr, ws.nbytes, _stream()), "tgis_dense_gemm_gelu_lookup")
    return out


def sigmoid_gate_mul(x: torch.Tensor, gate: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x * sigmoid(gate); x and gate [T, C] views with unit column stride; in place when out is x."""
    assert x.dim() == 2 and x.stride(1) == 1 and gate.stride(1) == 1 and gate.shape == x.shape and gate.dtype == x.dtype
    if out is None:
        out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    _check(load_library().tgis_sigmoid_gate_mul(_ptr(x), x.stride(0), _ptr(gate), gate.stride(0), _ptr(out), out.stride(0), x.shape[0],
                                                x.shape[1], dtype_code3(x.dtype), _stream()), "tgis_sigmoid_gate_mul")
    return out


def logit_softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    assert logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1
    _check(load_library().tgis_logit_softcap(_ptr(logits), logits.stride(0), logits.shape[0], logits.shape[1], float(cap), _stream()),
           "tgis_logit_softcap")
    return logits


def gelu_gated_lookup(gate: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int) -> torch.Tensor:
    """gelu_tanh(gate [T, C]) * table[ids][:, col0:col0 + C]."""
    assert gate.dim() == 2 and gate.stride(1) == 1 and table.dim() == 2 and table.stride(1) == 1 and table.dtype == gate.dtype
    assert ids.dtype == torch.int64 and ids.shape[0] == gate.shape[0]
    T, C = gate.shape
    out = torch.empty((T, C), dtype=gate.dtype, device=gate.device)
    _check(load_library().tgis_gelu_gated_lookup(_ptr(gate), gate.stride(0), _ptr(ids), _ptr(table), table.stride(0), int(col0),
                                                 table.shape[0], _ptr(out), out.stride(0), T, C, dtype_code3(gate.dtype), _stream()),
           "tgis_gelu_gated_lookup")
    return out


def rms_norm_rows(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x [T, C] (row stride free) -> contiguous x / rms(x) * w."""
    assert x.dim() == 2 and x.stride(1) == 1 and w.shape[0] == x.shape[1]
    out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    _check(load_library().tgis_rms_norm_rows(_ptr(x), x.stride(0), _f32(w, "w"), _ptr(out), out.stride(0), x.shape[0], x.shape[1],
                                             float(eps), dtype_code3(x.dtype), _stream()), "tgis_rms_norm_rows")
    return out


def kv_norm_write(qkv: torch.Tensor, k_col0: int, v_col0: int, slots, k_pool, v_pool, G: int, dk: int, dv: int, v_norm: bool,
                  eps: float):
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and k_pool.dtype == qkv.dtype and v_pool.dtype == qkv.dtype
    assert slots.shape[0] == qkv.shape[0]
    _check(load_library().tgis_kv_norm_write(_ptr(qkv), qkv.stride(0), int(k_col0), int(v_col0), _i32(slots, "slots"), _ptr(k_pool),
                                             _ptr(v_pool), qkv.shape[0], G, dk, dv, int(bool(v_norm)), float(eps),
                                             dtype_code3(qkv.dtype), _stream()), "tgis_kv_norm_write")


def latent_kv_write(q, ckv, c_gain, inv_freq, positions, slots, q_abs, k_pool, v_pool, H: int, dn: int, dr: int, kv_rank: int,
                    rot_dims: int, eps: float):
    assert q.dim() == 2 and q.stride(1) == 1 and ckv.stride(1) == 1 and q_abs.stride(1) == 1
    assert ckv.dtype == q.dtype and q_abs.dtype == q.dtype and k_pool.dtype == q.dtype and v_pool.dtype == q.dtype
    assert positions.shape[0] == q.shape[0] and slots.shape[0] == q.shape[0] and inv_freq.shape[0] * 2 >= rot_dims
    _check(load_library().tgis_latent_kv_write(
        _ptr(q), q.stride(0), _ptr(ckv), ckv.stride(0), _f32(c_gain, "c_gain"), _f32(inv_freq, "inv_freq"),
        _i32(positions, "positions"), _i32(slots, "slots"), _ptr(q_abs), q_abs.stride(0), _ptr(k_pool), _ptr(v_pool), q.shape[0],
        H, dn, dr, kv_rank, rot_dims, float(eps), dtype_code3(q.dtype), _stream()), "tgis_latent_kv_write")


def attn_varlen_ext(q, k_pool, v_pool, block_tables, ctx_lens, cu_seqlens_q, H: int, G: int, dk: int, dv: int, scale: float,
                    r1=None, r2=None, chunk: int = 0, gate=None, max_q_len: int = 1, max_ctx: int = 1, impl: int = 0,
                    ws: Optional[Workspace] = None):
    """attn_varlen with a block mask (`chunk`), a distance bias per query head (r1, r2 [H] fp32) and / or a sigmoid output
    gate (gate [T, H dv], a view with unit column stride).  ws: scratch that lets a decode step with few sequences x cached
    heads deal its pages to several workgroups."""
    assert gate is None or (gate.dtype == q.dtype and gate.stride(1) == 1 and gate.shape == (q.shape[0], H * dv))
    assert q.dim() == 2 and q.stride(1) == 1 and block_tables.dim() == 2
    assert (r1 is None) == (r2 is None) and (r1 is None or (r1.shape[0] == H and r2.shape[0] == H))
    T = q.shape[0]
    out = torch.empty((T, H * dv), dtype=q.dtype, device=q.device)
    _check(load_library().tgis_attn_varlen_ext(
        _ptr(q), q.stride(0), _ptr(k_pool), _ptr(v_pool), _i32(block_tables, "block_tables"), block_tables.shape[1],
        _i32(ctx_lens, "ctx_lens"), _i32(cu_seqlens_q, "cu_seqlens_q"), ctx_lens.shape[0], _ptr(out), out.stride(0), T,
        max(int(max_q_len), 1), max(int(max_ctx), 1), H, G, dk, dv, float(scale), _f32(r1, "r1"), _f32(r2, "r2"), int(chunk), _ptr(gate),
        gate.stride(0) if gate is not None else 0, (ws.ptr + 4096) if ws is not None else None,  # past the GEMMs' arrival counters
        (ws.nbytes - 4096) if ws is not None else 0, impl,
        dtype_code3(q.dtype), _stream()), "tgis_attn_varlen_ext")
    return out


def delta_state_floats(dk: int, dv: int) -> int:
    n = load_library().tgis_delta_state_floats(dk, dv)
    if n < 0:
        raise TgisHipError(f"the delta-rule scan serves key and value widths up to 256 (got {dk}, {dv})")
    return n


def short_conv_silu(x, w, tail, state_slots, cu_seqlens_q, positions, C: int) -> torch.Tensor:
    """x [T, >= C]: the first C columns pass a causal per-channel convolution (w [C, taps] fp32) and SiLU -> [T, C] fp32."""
    assert x.dim() == 2 and x.stride(1) == 1 and w.shape[0] == C
    out = torch.empty((x.shape[0], C), dtype=torch.float32, device=x.device)
    _check(load_library().tgis_short_conv_silu(
        _ptr(x), x.stride(0), _f32(w, "w"), _f32(tail, "tail"), _i32(state_slots, "state_slots"), _i32(cu_seqlens_q, "cu_seqlens_q"),
        _i32(positions, "positions"), state_slots.shape[0], _ptr(out), x.shape[0], C, w.shape[1], dtype_code3(x.dtype), _stream()),
        "tgis_short_conv_silu")
    return out


def delta_scan(conv, a, b, gate, A_log, dt_bias, gain, state, tail, proj, state_slots, cu_seqlens_q, positions, H: int, G: int,
               dk: int, dv: int, taps: int, eps: float, unit_eps: float, q_scale: float) -> torch.Tensor:
    """conv [T, 2 G dk + H dv] fp32; a [T, H dk], b [T, H], gate [T, H dv], proj [T, >= C] views in the activation dtype."""
    T = conv.shape[0]
    assert conv.dtype == torch.float32 and conv.is_contiguous()
    assert all(t.stride(1) == 1 and t.dtype == a.dtype for t in (a, b, gate, proj))
    out = torch.empty((T, H * dv), dtype=a.dtype, device=a.device)
    _check(load_library().tgis_delta_scan(
        _ptr(conv), conv.shape[1], _ptr(a), a.stride(0), _ptr(b), b.stride(0), _ptr(gate), gate.stride(0), _f32(A_log, "A_log"),
        _f32(dt_bias, "dt_bias"), _f32(gain, "gain"), _f32(state, "state"), _f32(tail, "tail"), _ptr(proj), proj.stride(0),
        _i32(state_slots, "state_slots"), _i32(cu_seqlens_q, "cu_seqlens_q"), _i32(positions, "positions"), _ptr(out), out.stride(0),
        state_slots.shape[0], H, G, dk, dv, taps, float(eps), float(unit_eps), float(q_scale), dtype_code3(a.dtype), _stream()),
        "tgis_delta_scan")
    return out


# ---- parallel layers with gated residuals: rotation in the "rows" layout, windowed attention, gated linear scan, update ------
def rope_rows_kv_write(proj, q_col0: int, k_col0: int, v_col0: int, inv_freq, positions, slots, k_pool, v_pool, H: int, G: int,
                       dk: int, dv: int, rot_dims: int):
    """q (in place) and k (into the K pages) of proj [T, ld] rotated in interleaved pairs over their first rot_dims channels; v into
    the V pages."""
    assert proj.dim() == 2 and proj.stride(1) == 1 and k_pool.dtype == proj.dtype and v_pool.dtype == proj.dtype
    assert positions.shape[0] == proj.shape[0] and slots.shape[0] == proj.shape[0]
    assert rot_dims == 0 or inv_freq.shape[0] >= rot_dims // 2
    _check(load_library().tgis_rope_rows_kv_write(
        _ptr(proj), proj.stride(0), q_col0, k_col0, v_col0, _f32(inv_freq, "inv_freq") if rot_dims else None, _i32(positions, "positions"),
        _i32(slots, "slots"), _ptr(k_pool), _ptr(v_pool), proj.shape[0], H, G, dk, dv, rot_dims, dtype_code3(proj.dtype), _stream()),
        "tgis_rope_rows_kv_write")


def attn_varlen_win(q, k_pool, v_pool, block_tables, ctx_lens, cu_seqlens_q, H: int, G: int, dk: int, dv: int, scale: float,
                    window: int = 0, keep_first: int = 0, sink=None, gate=None, gate_per_head: bool = False, out_scale: float = 1.0,
                    out=None, max_q_len: int = 1, max_ctx: int = 1, impl: int = 0, ws: Optional[Workspace] = None):
    """attn_varlen with a sliding window that keeps the first positions, a sink logit per head (sink [H] fp32), a sigmoid output
    gate (per head: gate [T, H]; per channel: gate [T, H dv]) and a factor on the output.  out: a [T, H dv] view (unit column
    stride) of the caller's buffer, or None."""
    assert q.dim() == 2 and q.stride(1) == 1 and block_tables.dim() == 2
    T = q.shape[0]
    assert gate is None or (gate.dtype == q.dtype and gate.stride(1) == 1 and gate.shape == (T, H if gate_per_head else H * dv))
    assert sink is None or sink.shape[0] == H
    if out is None:
        out = torch.empty((T, H * dv), dtype=q.dtype, device=q.device)
    assert out.shape == (T, H * dv) and out.stride(1) == 1 and out.dtype == q.dtype
    _check(load_library().tgis_attn_varlen_win(
        _ptr(q), q.stride(0), _ptr(k_pool), _ptr(v_pool), _i32(block_tables, "block_tables"), block_tables.shape[1],
        _i32(ctx_lens, "ctx_lens"), _i32(cu_seqlens_q, "cu_seqlens_q"), ctx_lens.shape[0], _ptr(out), out.stride(0), T,
        max(int(max_q_len), 1), max(int(max_ctx), 1), H, G, dk, dv, float(scale), int(window), int(keep_first), _f32(sink, "sink"),
        _ptr(gate), gate.stride(0) if gate is not None else 0, int(gate_per_head), float(out_scale),
        (ws.ptr + 4096) if ws is not None else None, (ws.nbytes - 4096) if ws is not None else 0, impl, dtype_code3(q.dtype), _stream()),
        "tgis_attn_varlen_win")
    return out


def gated_linear_scan(proj, q_col0: int, f_col0: int, v_col0: int, f_bias, lower, gain, state, state_slots, cu_seqlens_q, positions,
                      H: int, dk: int, dv: int, eps: float, q_act: bool = True, out_scale: float = 1.0, out=None, max_q_len: int = 0):
    """S <- diag(f) S + (1 - f) v^T, o = S^T q per (sequence, head) on columns of proj [T, ld]; f = lower + (1 - lower) *
    sigmoid(proj_f + f_bias); q = silu(proj_q) if q_act; out = rms_norm(o) * gain * out_scale -> [T, H dv] (or the view `out`)."""
    assert proj.dim() == 2 and proj.stride(1) == 1
    T = proj.shape[0]
    if out is None:
        out = torch.empty((T, H * dv), dtype=proj.dtype, device=proj.device)
    assert out.shape == (T, H * dv) and out.stride(1) == 1 and out.dtype == proj.dtype
    assert state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, dk, dv)
    mq = int(max_q_len) if max_q_len > 0 else max(T, 1)
    # long steps: room for the unnormed read-outs, so that the kernel may deal a head's columns to several workgroups
    scratch = torch.empty((T, H * dv), dtype=torch.float32, device=proj.device) if mq > 2 else None
    _check(load_library().tgis_gated_linear_scan(
        _ptr(proj), proj.stride(0), q_col0, f_col0, v_col0, _f32(f_bias, "f_bias"), _f32(lower, "lower"), _f32(gain, "gain"),
        _ptr(state), _i32(state_slots, "state_slots"), _i32(cu_seqlens_q, "cu_seqlens_q"), _i32(positions, "positions"), _ptr(out),
        out.stride(0), float(out_scale), state_slots.shape[0], T, mq, H, dk, dv, float(eps), int(q_act), _ptr(scratch),
        dtype_code3(proj.dtype), _stream()),
        "tgis_gated_linear_scan")
    return out


def _delta_args(d, bias, rows: int, E: int, dtype):
    """(pointer, row stride, slabs, bias pointer) of a sublayer result: a tensor, or the split-K slabs of its projection."""
    if d is None:
        return None, 0, 0, None
    if isinstance(d, Partial):
        assert d.shape == (rows, E) and d.dtype == dtype
        b = d.bias if d.bias is not None else bias
        assert b is None or (b.dtype == dtype and b.shape[0] == E)
        return _ptr(d.slabs), d.ld, d.S, _ptr(b)
    assert d.shape == (rows, E) and d.stride(1) == 1 and d.dtype == dtype
    assert bias is None or (bias.dtype == dtype and bias.shape[0] == E)
    return _ptr(d), d.stride(0), 0, _ptr(bias)


def parallel_residual_f32(x, a, gate_a, gate_bias_a, b, gate_b, gate_bias_b, act_dtype, hist, n_prev: int, mix, x_out, pre_w,
                          eps: float, y_dtype, pre_add: float = 0.0, bias_a=None, bias_b=None):
    """v = x + sigmoid(gate_a + gate_bias_a) a + sigmoid(gate_b + gate_bias_b) b;  hist[n_prev] = v;  x_out = sum_j mix[j] hist[j];
    returns y = rms_norm(x_out) * (pre_w + pre_add) in y_dtype (None without pre_w).  a / b: tensors of act_dtype or `Partial`
    split-K slabs (whose bias, if any, is added here); gates are [rows, E] views of logits; hist [>= n_prev + 1, rows, E] fp32
    or None (then x_out = v)."""
    rows, E = x.shape
    assert x.dtype == torch.float32 and x.stride(1) == 1 and x.stride(0) == E and x_out.dtype == torch.float32 and x_out.is_contiguous()
    for g, gb in ((gate_a, gate_bias_a), (gate_b, gate_bias_b)):
        assert g is None or (g.dtype == act_dtype and g.stride(1) == 1 and g.shape == (rows, E))
        assert gb is None or (gb.dtype == act_dtype and gb.shape[0] == E)
    pa, lda, sa, ba = _delta_args(a, bias_a, rows, E, act_dtype)
    pb, ldb, sb, bb = _delta_args(b, bias_b, rows, E, act_dtype)
    if hist is not None:
        assert hist.dtype == torch.float32 and hist.is_contiguous() and hist.shape[0] > n_prev and tuple(hist.shape[1:]) == (rows, E)
        assert mix.dtype == torch.float32 and mix.shape[0] == n_prev + 1
    y = torch.empty((rows, E), dtype=y_dtype, device=x.device) if pre_w is not None else None
    _check(load_library().tgis_parallel_residual_f32(
        _ptr(x), pa, lda, sa, ba, _ptr(gate_a), gate_a.stride(0) if gate_a is not None else 0, _ptr(gate_bias_a),
        pb, ldb, sb, bb, _ptr(gate_b), gate_b.stride(0) if gate_b is not None else 0, _ptr(gate_bias_b), dtype_code3(act_dtype),
        _ptr(hist), int(n_prev), hist.stride(0) if hist is not None else 0, _f32(mix, "mix") if hist is not None else None, _ptr(x_out),
        _f32(pre_w, "pre_w"), float(pre_add), _ptr(y), dtype_code3(y_dtype) if y is not None else F32, rows, E, float(eps), _stream()),
        "tgis_parallel_residual_f32")
    return y


# ---- scaled parallel layers: input convolutions, selective scan, head-mixed attention, general linear scan --------------------
def _is_f32(t: torch.Tensor) -> int:
    return int(t.dtype == torch.float32)


def rope_rows_unit_kv_write(proj, q_col0: int, k_col0: int, v_col0: int, inv_freq, positions, slots, k_pool, v_pool, H: int, G: int,
                            dk: int, dv: int, rot_dims: int, unit_eps: float):
    """rope_rows_kv_write, then every q and k head divided by sqrt(mean(x^2) + unit_eps) (q in place, k in its page)."""
    assert proj.dim() == 2 and proj.stride(1) == 1 and k_pool.dtype == proj.dtype and v_pool.dtype == proj.dtype
    assert positions.shape[0] == proj.shape[0] and slots.shape[0] == proj.shape[0]
    assert rot_dims == 0 or inv_freq.shape[0] >= rot_dims // 2
    _check(load_library().tgis_rope_rows_unit_kv_write(
        _ptr(proj), proj.stride(0), q_col0, k_col0, v_col0, _f32(inv_freq, "inv_freq") if rot_dims else None, _i32(positions, "positions"),
        _i32(slots, "slots"), _ptr(k_pool), _ptr(v_pool), proj.shape[0], H, G, dk, dv, rot_dims, float(unit_eps),
        dtype_code3(proj.dtype), _stream()), "tgis_rope_rows_unit_kv_write")


def attn_mixed_heads(q, k_pool, v_pool, block_tables, ctx_lens, cu_seqlens_q, mix, H: int, G: int, dk: int, dv: int, scale: float,
                     window: int = 0, gate=None, out=None, max_q_len: int = 1, max_ctx: int = 1, ws: Optional[Workspace] = None,
                     impl: int = 0):
    """Softmax attention over the paged cache with the heads' scores mixed by mix [H, H] (fp32) before the softmax; q [T, H dk]
    (a view with unit column stride), gate [T, H dv] or None -> [T, H dv].  ws: scratch for the key-split form of decode steps."""
    assert q.dim() == 2 and q.stride(1) == 1 and block_tables.dim() == 2 and mix.shape == (H, H) and mix.is_contiguous()
    T = q.shape[0]
    assert gate is None or (gate.dtype == q.dtype and gate.stride(1) == 1 and gate.shape == (T, H * dv))
    if out is None:
        out = torch.empty((T, H * dv), dtype=q.dtype, device=q.device)
    assert out.shape == (T, H * dv) and out.stride(1) == 1 and out.dtype == q.dtype
    _check(load_library().tgis_attn_mixed_heads(
        _ptr(q), q.stride(0), _ptr(k_pool), _ptr(v_pool), _i32(block_tables, "block_tables"), block_tables.shape[1],
        _i32(ctx_lens, "ctx_lens"), _i32(cu_seqlens_q, "cu_seqlens_q"), ctx_lens.shape[0], _f32(mix, "mix"), _ptr(gate),
        gate.stride(0) if gate is not None else 0, _ptr(out), out.stride(0), T, max(int(max_q_len), 1), max(int(max_ctx), 1), H, G, dk, dv,
        float(scale), int(window), (ws.ptr + 4096) if ws is not None else None, (ws.nbytes - 4096) if ws is not None else 0,
        int(impl), dtype_code3(q.dtype), _stream()), "tgis_attn_mixed_heads")
    return out


def linear_scan(proj, q_col0: int, k_col0: int, f_col0: int, v_col0: int, state, state_slots, cu_seqlens_q, positions, H: int, dk: int,
                dv: int, eps: float, gain, decay_mode: int = 0, f_bias=None, lower=None, head_decay=None, inv_tau: float = 1.0,
                q_act: bool = False, k_act: bool = False, v_act: bool = False, q_scale: float = 1.0, norm_rows: bool = False, gate=None,
                gate_act: int = 0, out_scale: float = 1.0, out=None, max_q_len: int = 0):
    """S <- diag(a) S + k v^T, o = S^T q on columns of proj [T, ld]; see tgis_linear_scan for the forms.  -> [T, H dv]."""
    assert proj.dim() == 2 and proj.stride(1) == 1
    T = proj.shape[0]
    if out is None:
        out = torch.empty((T, H * dv), dtype=proj.dtype, device=proj.device)
    assert out.shape == (T, H * dv) and out.stride(1) == 1 and out.dtype == proj.dtype
    assert state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, dk, dv)
    assert gain.shape[0] == (H * dv if norm_rows else dv)
    assert gate is None or (gate.dtype == proj.dtype and gate.stride(1) == 1 and gate.shape == (T, H * dv))
    mq = int(max_q_len) if max_q_len > 0 else max(T, 1)
    scratch = torch.empty((T, H * dv), dtype=torch.float32, device=proj.device) if (mq > 2 or norm_rows) else None
    _check(load_library().tgis_linear_scan(
        _ptr(proj), proj.stride(0), q_col0, k_col0, f_col0, v_col0, _f32(f_bias, "f_bias"), _f32(lower, "lower"),
        _f32(head_decay, "head_decay"), int(decay_mode), float(inv_tau), int(q_act), int(k_act), int(v_act), float(q_scale),
        _f32(gain, "gain"), int(norm_rows), _ptr(gate), gate.stride(0) if gate is not None else 0, int(gate_act) if gate is not None else 0,
        _ptr(state), _i32(state_slots, "state_slots"), _i32(cu_seqlens_q, "cu_seqlens_q"), _i32(positions, "positions"), _ptr(out),
        out.stride(0), float(out_scale), state_slots.shape[0], T, mq, H, dk, dv, float(eps), _ptr(scratch), dtype_code3(proj.dtype),
        _stream()), "tgis_linear_scan")
    return out


def causal_conv(x, w, bias, tail, state_slots, cu_seqlens_q, positions, out_dtype, act: bool = False, residual: bool = False,
                max_q_len: int = 0) -> torch.Tensor:
    """x [T, >= C] (fp32 or out_dtype), w [sets, C, taps] fp32, bias [sets, C] or None, tail [slots, >= (taps - 1) * C] fp32 (a view
    whose rows are the slots) -> out [sets, T, C]; the tail is moved on to the step's end."""
    sets, C, taps = w.shape
    assert x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= C and w.is_contiguous() and (x.dtype == out_dtype or x.dtype == torch.float32)
    assert tail is None or (tail.dtype == torch.float32 and tail.dim() == 2 and tail.stride(1) == 1)
    T = x.shape[0]
    out = torch.empty((sets, T, C), dtype=out_dtype, device=x.device)
    _check(load_library().tgis_causal_conv(
        _ptr(x), x.stride(0), int(x.dtype == torch.float32 and out_dtype != torch.float32), _f32(w, "w"), _f32(bias, "bias"), sets,
        _ptr(tail), tail.stride(0) if tail is not None else 0, _i32(state_slots, "state_slots"), _i32(cu_seqlens_q, "cu_seqlens_q"),
        _i32(positions, "positions"), state_slots.shape[0], _ptr(out), C, T * C, int(max_q_len) if max_q_len > 0 else max(T, 1), C, taps,
        int(act), int(residual), dtype_code3(out_dtype), _stream()), "tgis_causal_conv")
    return out


def selective_scan(x, dt, dt_bias, bc, b_col0: int, c_col0: int, z, A_log, D, state, state_slots, cu_seqlens_q, positions, N: int,
                   max_q_len: int = 0):
    """x, z [T, inner] views, dt [T, inner] (fp32 or the activation dtype), bc [T, ld] with B | C at their columns -> [T, inner]."""
    T, inner = x.shape
    assert all(t.stride(1) == 1 for t in (x, dt, bc, z)) and z.shape == x.shape and dt.shape == x.shape
    assert state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (inner, N)
    out = torch.empty((T, inner), dtype=x.dtype, device=x.device)
    _check(load_library().tgis_selective_scan(
        _ptr(x), x.stride(0), _ptr(dt), dt.stride(0), int(dt.dtype == torch.float32 and x.dtype != torch.float32), _f32(dt_bias, "dt_bias"),
        _ptr(bc), bc.stride(0), b_col0, c_col0, _ptr(z), z.stride(0), _f32(A_log, "A_log"), _f32(D, "D"), _ptr(state),
        _i32(state_slots, "state_slots"), _i32(cu_seqlens_q, "cu_seqlens_q"), _i32(positions, "positions"), _ptr(out), out.stride(0),
        state_slots.shape[0], int(max_q_len) if max_q_len > 0 else max(T, 1), inner, N, dtype_code3(x.dtype), _stream()),
        "tgis_selective_scan")
    return out


def scaled_residual_norm(x_in, a, s1, b, s2, v, w, eps: float, act_dtype, x_out=None, h_f32: bool = True, mean_free: bool = True,
                         keep_x: bool = True, pair=None):
    """x_out = x_in + s1 * a + s2 * b + v (every term optional), h = norm(x_out) * w (w None: no norm).  -> (x_out, h); x_out may be
    x_in; keep_x False: only h is wanted.  pair = (a2, wa, wa2, coef): the first term is coef * (a / rms(a) * wa + a2 / rms(a2) * wa2)."""
    a2, wa, wa2, coef = pair if pair is not None else (None, None, None, 0.0)
    assert a2 is None or (a is not None and a2.shape == a.shape and a2.stride(1) == 1 and a2.dtype in (torch.float32, act_dtype))
    ref = x_in if x_in is not None else (a if a is not None else b)
    T, W = ref.shape
    if x_out is None and keep_x:
        x_out = torch.empty((T, W), dtype=torch.float32, device=ref.device)
    assert x_in is None or (x_in.dtype == torch.float32 and x_in.is_contiguous())
    assert x_out is None or (x_out.dtype == torch.float32 and x_out.is_contiguous())
    for t in (a, b):
        assert t is None or (t.stride(1) == 1 and t.dtype in (torch.float32, act_dtype))
    h = None
    if w is not None:
        h = torch.empty((T, W), dtype=torch.float32 if h_f32 else act_dtype, device=ref.device)
    _check(load_library().tgis_scaled_residual_norm(
        _ptr(x_in), _ptr(x_out), _ptr(a), a.stride(0) if a is not None else 0, _is_f32(a) if a is not None else 0, _f32(s1, "s1"),
        _ptr(b), b.stride(0) if b is not None else 0, _is_f32(b) if b is not None else 0, _f32(s2, "s2"), _f32(v, "v"), _f32(w, "w"),
        _ptr(h), int(h_f32 or act_dtype == torch.float32), T, W, float(eps), int(mean_free), _ptr(a2), a2.stride(0) if a2 is not None else 0,
        _is_f32(a2) if a2 is not None else 0, _f32(wa, "wa"), _f32(wa2, "wa2"), float(coef), dtype_code3(act_dtype), _stream()),
        "tgis_scaled_residual_norm")
    return x_out, h


def rms_pair_mean(a, wa, ca: float, b, wb, cb: float, eps: float, act_dtype) -> torch.Tensor:
    """ca * a / rms(a) * wa + cb * b / rms(b) * wb -> fp32 [T, W]."""
    T, W = a.shape
    assert a.stride(1) == 1 and b.stride(1) == 1 and b.shape == a.shape
    y = torch.empty((T, W), dtype=torch.float32, device=a.device)
    _check(load_library().tgis_rms_pair_mean(_ptr(a), a.stride(0), _is_f32(a), _f32(wa, "wa"), float(ca), _ptr(b), b.stride(0), _is_f32(b),
                                             _f32(wb, "wb"), float(cb), _ptr(y), T, W, float(eps), dtype_code3(act_dtype), _stream()),
           "tgis_rms_pair_mean")
    return y


def poly_norm(z: torch.Tensor, c1: float, c2: float, c3: float, c0: float, eps: float) -> torch.Tensor:
    """c1 z / rms(z) + c2 z^2 / rms(z^2) + c3 z^3 / rms(z^3) + c0 over the rows of z."""
    assert z.dim() == 2 and z.stride(1) == 1
    y = torch.empty(z.shape, dtype=z.dtype, device=z.device)
    _check(load_library().tgis_poly_norm(_ptr(z), z.stride(0), _ptr(y), y.stride(0), z.shape[0], z.shape[1], float(c1), float(c2),
                                         float(c3), float(c0), float(eps), dtype_code3(z.dtype), _stream()), "tgis_poly_norm")
    return y


def moe_route_grouped(h, router_w, correction, k: int, n_groups: int = 1, keep_groups: int = 1, renorm_eps: float = 0.0):
    """(idx [T, k] int32, weight [T, k] fp32): softmax scores over all experts, choice by score + correction among the best
    groups, weights = chosen scores / (their sum + renorm_eps)."""
    T, W = h.shape
    E = router_w.shape[0]
    idx = torch.empty((T, k), dtype=torch.int32, device=h.device)
    weight = torch.empty((T, k), dtype=torch.float32, device=h.device)
    _check(load_library().tgis_moe_route_grouped(_ptr(h), h.stride(0), _f32(router_w, "router_w"), _f32(correction, "correction"),
                                                 int(n_groups), int(keep_groups), float(renorm_eps), _ptr(idx), _ptr(weight), T, W, E, k,
                                                 dtype_code3(h.dtype), _stream()), "tgis_moe_route_grouped")
    return idx, weight
