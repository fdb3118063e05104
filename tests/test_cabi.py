"""The C ABI: every function include/sae_hip.h declares is exported by libsae_hip.so and bound by
the ctypes layer with the same arity.  No kernel is launched here (runs without a GPU)."""

import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "sae_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    body = text[text.index('extern "C" {'):]
    out = {}
    for m in re.finditer(r"\b(?:int|int64_t|const char \*)\s*(sae_\w+)\s*\(([^;{]*)\)\s*;", body):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("void", "") else args.count(",") + 1
    return out


def test_header_declares_the_expected_families():
    names = set(declared_functions())
    for must in ("sae_encoder_gemm", "sae_select_topk_row", "sae_sparse_decode_fwd", "sae_sparse_decode_bwd_dval",
                 "sae_sparse_decode_mse_fused", "sae_build_feature_index", "sae_sparse_grad_rows", "sae_adam_step",
                 "sae_row_norm", "sae_last_error", "sae_abi_version"):
        assert must in names


def test_library_exports_every_declared_symbol(pkg):
    lib = ctypes.CDLL(pkg._lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in sae_hip.h but not exported"


def test_ctypes_bindings_match_header_arity(pkg):
    decl = declared_functions()
    sig = pkg._lib.SIGNATURES
    assert set(sig) == set(decl), (set(sig) ^ set(decl))
    for name, n in decl.items():
        assert len(sig[name][1]) == n, f"{name}: header has {n} parameters, binding has {len(sig[name][1])}"


def test_version_and_error_text(pkg):
    lib = pkg._lib.load()
    assert lib.sae_abi_version() == 1
    # argument validation happens before any device work: a null pointer is rejected on any machine
    rc = lib.sae_encoder_gemm(None, None, None, 1, 32, 1, 1, 1, None)
    assert rc == -1 and b"null pointer" in lib.sae_last_error()
    rc = lib.sae_select_topk_row(None, 0, None, None, 1, 1, 1, None, None, None, None, None)
    assert rc == -1
    assert lib.sae_feature_index_workspace_bytes(16, 100, 64) >= 4 * (2 * 100 + 64)
