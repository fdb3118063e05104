"""ctypes binding of libsae_hip.so (the C ABI declared in include/sae_hip.h).

The library is built in-tree by `make -C language-model-saes_amd/csrc` (or
`__graft_entry__.build()`).  There is no CPU fallback: if the shared object is missing or
a call returns a non-zero status, a RuntimeError is raised.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsae_hip.so")

SAE_F32, SAE_BF16 = 0, 1

# name -> (restype, argtypes); mirrors include/sae_hip.h declaration by declaration
_P, _I, _L, _F = c_void_p, c_int, c_int64, c_double
SIGNATURES = {
    "sae_abi_version": (_I, []),
    "sae_last_error": (c_char_p, []),
    "sae_cast_f32_to_bf16": (_I, [_P, _P, _L, _P]),
    "sae_row_norm": (_I, [_P, _P, _L, _L, _P]),
    "sae_transpose_f32": (_I, [_P, _P, _L, _L, _P]),
    "sae_col_sum_workspace_bytes": (_L, [_L, _L]),
    "sae_col_sum": (_I, [_P, _P, _L, _L, _I, _P, _L, _P]),
    "sae_col_sum_static": (_I, [_P, _P, _L, _L, _I, _P]),
    "sae_encoder_gemm": (_I, [_P, _P, _P, _L, _L, _L, _I, _I, _P]),
    "sae_select_topk_row": (_I, [_P, _I, _P, _P, _L, _L, _I, _P, _P, _P, _P, _P]),
    "sae_encoder_gemm_bias": (_I, [_P, _P, _P, _L, _L, _L, _P, _P, _P]),
    "sae_encoder_gemm_granule_max": (_I, [_P, _P, _P, _L, _L, _L, _L, _P, _P, _P, _P]),
    "sae_encoder_gemm_granule_max_lowp": (_I, [_P, _P, _P, _L, _L, _L, _L, _P, _P, _P, _P]),
    "sae_select_topk_row_granule": (_I, [_P, _P, _P, _P, _L, _L, _I, _L, _L, _P, _P, _P, _P, _P]),
    "sae_select_topk_row_granule_lowp": (_I, [_P, _P, _P, _P, _L, _L, _I, _L, _L, _P, _P, _P, _P, _P]),
    "sae_granule_max": (_I, [_P, _P, _P, _L, _L, _L, _L, _P, _P]),
    "sae_merge_layer_codes": (_I, [_P, _P, _P, _L, _L, _L, _L, _P, _P, _P, _P, _P, _P]),
    "sae_union_group_codes": (_I, [_P, _P, _P, _L, _L, _L, _P, _P, _P, _P, _P]),
    "sae_select_topk_row_lowp": (_I, [_P, _P, _P, _P, _L, _L, _I, _P, _P, _P, _P, _P]),
    "sae_select_topk_row_ex": (_I, [_P, _I, _P, _P, _P, _L, _L, _I, _P, _P, _P, _P, _I, _P]),
    "sae_select_topk_batch_workspace_bytes": (_L, [_L, _L]),
    "sae_select_topk_batch": (_I, [_P, _I, _P, _P, _P, _L, _L, _L, _P, _P, _P, _L, _P, _P, _P, _P, _L, _P]),
    "sae_select_topk_batch_lowp": (_I, [_P, _P, _P, _P, _P, _L, _L, _L, _P, _P, _P, _L, _P, _P, _P, _P, _L, _P]),
    "sae_select_topk_batch_granule": (_I, [_P, _P, _P, _P, _L, _L, _L, _P, _P, _P, _L, _P, _P, _P, _P, _L, _P]),
    "sae_sparse_decode_fwd": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _L, _L, _L, _P]),
    "sae_sparse_decode_bwd_dval": (_I, [_P, _P, _P, _P, _P, _I, _P, _L, _L, _L, _L, _P]),
    "sae_sparse_decode_mse_fused": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _P]),
    "sae_sparse_decode_mse_fused_acc": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _P]),
    "sae_feature_index_workspace_bytes": (_L, [_L, _L, _L]),
    "sae_build_feature_index": (_I, [_P, _P, _P, _L, _L, _L, _P, _P, _P, _P, _L, _P]),
    "sae_sparse_grad_rows": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _L, _L, _P]),
    "sae_adam_step": (_I, [_P, _P, _I, _P, _P, _L, _F, _F, _F, _F, _L, _P, _P, _L, _P, _P]),
    "sae_sparse_adam_step": (_I, [_P, _P, _P, _P, _L, _F, _F, _F, _F, _P, _P, _P, _P]),
    "sae_grad_sq_nnz": (_I, [_P, _L, _P, _P]),
    "sae_adam_step_sparse_rows": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _P, _L, _L, _F, _F, _F, _F, _L, _P, _P, _P, _P, _P, _P, _L, _P, _P, _P, _P, _P]),
    "sae_adam_step_lowp": (_I, [_P, _P, _I, _P, _P, _L, _F, _F, _F, _F, _L, _P, _L, _P, _P]),
    "sae_adam_step_sparse_rows_lowp": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _P, _L, _L, _F, _F, _F, _F, _L, _P, _P, _P, _P, _P, _L, _P, _P, _P, _P]),
    "sae_gather_rows": (_I, [_P, _I, _P, _L, _L, _L, _P, _I, _F, _P]),
    "sae_transpose_to_bf16": (_I, [_P, _I, _P, _L, _L, _P, _P, _P]),
    "sae_code_to_dense": (_I, [_P, _P, _P, _P, _L, _L, _P, _P, _P]),
    "sae_code_to_dense_t": (_I, [_P, _P, _P, _P, _L, _L, _P, _P]),
    "sae_encoder_gemm_split_k": (_I, [_P, _P, _P, _L, _L, _L, _L, _P]),
    "sae_gemm_bf16": (_I, [_P, _I, _P, _I, _P, _I, _L, _L, _L, _L, _P]),
    "sae_mse_auxk_fused": (_I, [_P, _P, _P, _P, _F, _L, _L, _P, _P, _P, _P, _P, _P]),
    "sae_code_stats": (_I, [_P, _P, _P, _P, _P, _L, _L, _P, _P, _P, _P]),
    "sae_recon_stats": (_I, [_P, _P, _P, _P, _L, _L, _P, _P, _P, _P]),
    "sae_sparse_rows_grad_sq_nnz_workspace_bytes": (_L, [_L]),
    "sae_sparse_rows_grad_sq_nnz": (_I, [_P, _P, _P, _P, _P, _I, _L, _L, _P, _P, _P, _L, _P, _P, _P, _P]),
    "sae_jumprelu_fwd": (_I, [_P, _I, _P, _P, _P, _P, _L, _L, _F, _P, _P, _P, _P, _P]),
    "sae_jumprelu_bwd_workspace_bytes": (_L, [_L, _L]),
    "sae_attention_fwd": (_I, [_P, _P, _P, _L, _L, _L, _L, _L, _F, _P, _P, _P]),
    "sae_attention_bwd": (_I, [_P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _F, _P, _P, _P, _P, _P]),
    "sae_rotary_fwd": (_I, [_P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _I, _P, _P]),
    "sae_rotary_bwd_t": (_I, [_P, _P, _P, _L, _L, _L, _L, _L, _L, _I, _P]),
    "sae_row_sum": (_I, [_P, _I, _L, _L, _P, _P]),
    "sae_dense_row_nnz": (_I, [_P, _I, _L, _L, _P, _P]),
    "sae_dense_to_code": (_I, [_P, _I, _L, _L, _P, _P, _P, _L, _P, _P]),
    "sae_jumprelu_select_count": (_I, [_P, _I, _P, _P, _P, _P, _F, _L, _L, _P, _P]),
    "sae_jumprelu_select_emit": (_I, [_P, _I, _P, _P, _P, _P, _P, _F, _F, _L, _L, _P, _P, _P, _P, _L, _P, _P, _P]),
    "sae_encoder_gemm_jumprelu_margin": (_I, [_P, _P, _P, _L, _L, _L, _P, _P, _P, _P, _P]),
    "sae_feature_segment_sums": (_I, [_P, _P, _P, _P, _L, _P, _P, _P]),
    "sae_mfma_probe": (_I, [_P, _L, _L, _P, _P]),
    "sae_jumprelu_bwd": (_I, [_P, _I, _P, _P, _P, _P, _P, _P, _F, _P, _F, _L, _L, _P, _P, _P, _P, _P, _L, _P]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared object once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(needs hipcc; cross-compiles for gfx950 without a GPU). There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str = "") -> None:
    """Turn a non-zero status into a RuntimeError carrying the library's message."""
    if rc != 0:
        msg = load().sae_last_error()
        raise RuntimeError(f"libsae_hip {what} failed (status {rc}): {msg.decode() if msg else ''}")
