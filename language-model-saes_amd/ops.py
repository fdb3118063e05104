"""Tensor-level wrappers over the C ABI: validate, allocate outputs, pass raw pointers.

Every function launches on torch's current stream of the tensors' device and returns without
synchronising.  torch is used for device memory and streams only.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import SAE_BF16, SAE_F32, check


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


class KernelTimer:
    """Collects HIP-event pairs around every library call made while it is installed, or, with `only`, around the calls
    of those names (two event records per call cost host time and a few per cent of a step made of many short launches).

    Events are recorded on the stream the kernels are launched on (torch's current stream), so
    `elapsed_time` is the device-side duration of that call's kernels.  Read after a synchronize.
    """

    def __init__(self, only=None):
        self.records: dict[str, list[tuple[torch.cuda.Event, torch.cuda.Event]]] = {}
        self.only = None if only is None else frozenset(only)

    def summary(self) -> dict[str, dict[str, float]]:
        out = {}
        for name, evs in self.records.items():
            ms = [a.elapsed_time(b) for a, b in evs]
            out[name] = {"calls": len(ms), "avg_ms": sum(ms) / len(ms), "total_ms": sum(ms)}
        return out


_timer: Optional[KernelTimer] = None


def set_kernel_timer(timer: Optional[KernelTimer]) -> None:
    global _timer
    _timer = timer


class _timed:
    def __init__(self, name: str):
        self.name = name

    def __enter__(self):
        t = _timer
        self.timer = t if t is not None and (t.only is None or self.name in t.only) else None
        if self.timer is not None:
            self.a = torch.cuda.Event(enable_timing=True)
            self.a.record()
        return self

    def __exit__(self, *exc):
        if self.timer is not None:
            b = torch.cuda.Event(enable_timing=True)
            b.record()
            self.timer.records.setdefault(self.name, []).append((self.a, b))
        return False


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return SAE_F32
    if t.dtype == torch.bfloat16:
        return SAE_BF16
    raise TypeError(f"unsupported dtype {t.dtype} (float32 or bfloat16 expected)")


def _req(t: torch.Tensor, name: str, dtype=None, ndim=None):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); the HIP path has no CPU fallback")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if ndim is not None and t.ndim != ndim:
        raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")


@dataclass
class SparseCode:
    """Feature activations in sparse form (see include/sae_hip.h, "Sparse code")."""

    idx: torch.Tensor       # int32 [n_slots]
    val: torch.Tensor       # fp32  [n_slots]
    row_off: torch.Tensor   # int64 [B]
    row_nnz: torch.Tensor   # int32 [B]
    n_tokens: int
    d_sae: int

    @property
    def n_slots(self) -> int:
        return self.idx.numel()

    def to_dense(self) -> torch.Tensor:
        """[B, F] fp32 tensor with the code scattered in (unused slots carry 0 at index 0)."""
        B, F = self.n_tokens, self.d_sae
        out = torch.zeros(B, F, dtype=torch.float32, device=self.val.device)
        slots = torch.arange(self.n_slots, device=self.val.device)
        tok = torch.searchsorted(self.row_off, slots, right=True) - 1
        valid = (slots - self.row_off[tok]) < self.row_nnz[tok]
        out.index_put_((tok[valid], self.idx[valid].long()), self.val[valid], accumulate=True)
        return out


def stack_codes(a: SparseCode, b: SparseCode) -> SparseCode:
    """The code of 2B virtual tokens: a's tokens first, then b's (same feature space).  Used to hand
    two sparse codes with different dense operands to the gradient-row kernels in one piece."""
    if a.d_sae != b.d_sae:
        raise ValueError("codes address different dictionaries")
    return SparseCode(torch.cat([a.idx, b.idx]), torch.cat([a.val, b.val]),
                      torch.cat([a.row_off, b.row_off + a.n_slots]), torch.cat([a.row_nnz, b.row_nnz]),
                      a.n_tokens + b.n_tokens, a.d_sae)


@dataclass
class FeatureIndex:
    feat_ptr: torch.Tensor   # int32 [F + 1]
    feat_slot: torch.Tensor  # int32 [n_slots]
    slot_tok: torch.Tensor   # int32 [n_slots]


# ---- element-wise ---------------------------------------------------------------------------

def cast_bf16(src: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _req(src, "src", torch.float32)
    if out is None:
        out = torch.empty(src.shape, dtype=torch.bfloat16, device=src.device)
    with _timed("cast_f32_to_bf16"):
        check(_lib.load().sae_cast_f32_to_bf16(src.data_ptr(), out.data_ptr(), src.numel(), _stream(src)), "cast_f32_to_bf16")
    return out


def row_norm(w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _req(w, "w", torch.float32, 2)
    F, d = w.shape
    if out is None:
        out = torch.empty(F, dtype=torch.float32, device=w.device)
    with _timed("row_norm"):
        check(_lib.load().sae_row_norm(w.data_ptr(), out.data_ptr(), F, d, _stream(w)), "row_norm")
    return out


def transpose(src: torch.Tensor) -> torch.Tensor:
    _req(src, "src", torch.float32, 2)
    r, c = src.shape
    out = torch.empty(c, r, dtype=torch.float32, device=src.device)
    with _timed("transpose_f32"):
        check(_lib.load().sae_transpose_f32(src.data_ptr(), out.data_ptr(), r, c, _stream(src)), "transpose_f32")
    return out


def col_sum(src: torch.Tensor, out: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    _req(src, "src", torch.float32, 2)
    B, n = src.shape
    lib = _lib.load()
    if out is None:
        out = torch.empty(n, dtype=torch.float32, device=src.device)
        accumulate = False
    ws_bytes = lib.sae_col_sum_workspace_bytes(B, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=src.device)
    with _timed("col_sum"):
        check(lib.sae_col_sum(src.data_ptr(), out.data_ptr(), B, n, int(accumulate), ws.data_ptr(), ws_bytes, _stream(src)), "col_sum")
    return out


def transpose_to_bf16(src: torch.Tensor, mask: Optional[torch.Tensor] = None, col_sums: bool = False):
    """bf16 [cols, rows] = src[rows, cols]^T (fp32 or bf16 source), entries whose `mask` (fp32, same shape) is not
    positive written as 0.  With `col_sums` also returns the fp32 column sums of the masked source (summed tile by
    tile in a fixed order); otherwise the second value is None."""
    _req(src, "src", ndim=2)
    if src.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"src must be fp32 or bf16, not {src.dtype}")
    r, c = src.shape
    if mask is not None:
        _req(mask, "mask", torch.float32, 2)
        if tuple(mask.shape) != (r, c):
            raise ValueError("mask must have the source's shape")
    out = torch.empty(c, r, dtype=torch.bfloat16, device=src.device)
    part = torch.empty((r + 63) // 64, c, dtype=torch.float32, device=src.device) if col_sums else None
    with _timed("transpose_to_bf16"):
        check(_lib.load().sae_transpose_to_bf16(src.data_ptr(), _dt(src), _ptr(mask), r, c, out.data_ptr(), _ptr(part),
                                                _stream(src)), "transpose_to_bf16")
    return out, (col_sum(part) if col_sums else None)


def code_to_dense(code: "SparseCode", n_cols: int, want_f32: bool = True, want_bf16: bool = False):
    """Dense [n_tokens, n_cols] rows of a sparse code, in fp32 and / or bf16 -> (f32 or None, bf16 or None)."""
    if not (want_f32 or want_bf16):
        raise ValueError("no output requested")
    B, dev = code.n_tokens, code.val.device
    f32 = torch.empty(B, n_cols, dtype=torch.float32, device=dev) if want_f32 else None
    b16 = torch.empty(B, n_cols, dtype=torch.bfloat16, device=dev) if want_bf16 else None
    with _timed("code_to_dense"):
        check(_lib.load().sae_code_to_dense(code.idx.data_ptr(), code.val.data_ptr(), code.row_off.data_ptr(),
                                            code.row_nnz.data_ptr(), B, int(n_cols), _ptr(f32), _ptr(b16), _stream(code.val)),
              "code_to_dense")
    return f32, b16


def code_to_dense_t(code: "SparseCode", n_cols: int) -> torch.Tensor:
    """bf16 [n_cols, n_tokens]: the dense matrix of a sparse code, transposed (the left operand of a product over tokens)."""
    B = code.n_tokens
    out = torch.empty(int(n_cols), B, dtype=torch.bfloat16, device=code.val.device)
    with _timed("code_to_dense_t"):
        check(_lib.load().sae_code_to_dense_t(code.idx.data_ptr(), code.val.data_ptr(), code.row_off.data_ptr(),
                                              code.row_nnz.data_ptr(), B, int(n_cols), out.data_ptr(), _stream(code.val)),
              "code_to_dense_t")
    return out


def dense_row_nnz(dense: torch.Tensor) -> torch.Tensor:
    """int32 [B]: the number of non-zero entries of every row of a dense [B, F] matrix (fp32 or bf16)."""
    _req(dense, "dense", ndim=2)
    B, F = dense.shape
    row_nnz = torch.empty(B, dtype=torch.int32, device=dense.device)
    with _timed("dense_row_nnz"):
        check(_lib.load().sae_dense_row_nnz(dense.data_ptr(), _dt(dense), B, F, row_nnz.data_ptr(), _stream(dense)), "dense_row_nnz")
    return row_nnz


def dense_to_code(dense: torch.Tensor, capacity: Optional[int] = None, max_entries: Optional[int] = None) -> Optional["SparseCode"]:
    """Sparse code of a dense [B, F] activation matrix (fp32 or bf16): every token's non-zero entries in ascending
    feature order, rows packed one after the other.  Without `capacity` the number of non-zeros is read back from the
    device to size the code (one synchronisation, as the reference's `nnz_max.item()`); `max_entries` then makes the
    call return None, before anything is written, when the matrix holds more non-zeros than that (the caller's sparsity
    gate).  With `capacity` (an upper bound the caller knows, e.g. k * B after a TopK activation) nothing is read back;
    entries past it are dropped and `row_nnz` is cut to what was written, so the code is truncated, never out of bounds."""
    _req(dense, "dense", ndim=2)
    B, F = dense.shape
    lib = _lib.load()
    row_nnz = torch.empty(B, dtype=torch.int32, device=dense.device)
    with _timed("dense_to_code"):
        check(lib.sae_dense_row_nnz(dense.data_ptr(), _dt(dense), B, F, row_nnz.data_ptr(), _stream(dense)), "dense_row_nnz")
        incl = torch.cumsum(row_nnz, 0, dtype=torch.int64)
        row_off = incl - row_nnz
        if capacity is None:
            cap = int(incl[-1].item())
            if max_entries is not None and cap > max_entries:
                return None
        else:
            cap = int(capacity)
        idx = torch.zeros(max(cap, 1), dtype=torch.int32, device=dense.device)
        val = torch.zeros(max(cap, 1), dtype=torch.float32, device=dense.device)
        check(lib.sae_dense_to_code(dense.data_ptr(), _dt(dense), B, F, row_off.data_ptr(), idx.data_ptr(), val.data_ptr(), cap,
                                    row_nnz.data_ptr() if capacity is not None else None, _stream(dense)), "dense_to_code")
    return SparseCode(idx, val, row_off, row_nnz, B, F)


def mse_auxk_fused(recon: torch.Tensor, label: torch.Tensor, aux_recon: Optional[torch.Tensor],
                   tok_w: Optional[torch.Tensor], alpha: float, want_bf16: bool = False):
    """-> (rec_tok [B], aux_tok [B] or None, g_aux [B, d] or None, grad_recon [B, d], grad_recon in bf16 or None):
    the per-token weighted squared error, the per-token weighted squared aux-k residual (l_aux = alpha * its sum),
    d loss / d aux_recon and d loss / d recon."""
    _req(recon, "recon", torch.float32, 2)
    _req(label, "label", torch.float32, 2)
    B, d = recon.shape
    if tuple(label.shape) != (B, d):
        raise ValueError("label must have recon's shape")
    if aux_recon is not None:
        _req(aux_recon, "aux_recon", torch.float32, 2)
        if tuple(aux_recon.shape) != (B, d):
            raise ValueError("aux_recon must have recon's shape")
    if tok_w is not None:
        _req(tok_w, "tok_w", torch.float32, 1)
    dev = recon.device
    rec_tok = torch.empty(B, dtype=torch.float32, device=dev)
    aux_tok = torch.empty(B, dtype=torch.float32, device=dev) if aux_recon is not None else None
    g_aux = torch.empty(B, d, dtype=torch.float32, device=dev) if aux_recon is not None else None
    grad = torch.empty(B, d, dtype=torch.float32, device=dev)
    grad16 = torch.empty(B, d, dtype=torch.bfloat16, device=dev) if want_bf16 else None
    with _timed("mse_auxk_fused"):
        check(_lib.load().sae_mse_auxk_fused(recon.data_ptr(), label.data_ptr(), _ptr(aux_recon), _ptr(tok_w), float(alpha), B, d,
                                             rec_tok.data_ptr(), _ptr(aux_tok), _ptr(g_aux), grad.data_ptr(), _ptr(grad16),
                                             _stream(recon)), "mse_auxk_fused")
    return rec_tok, aux_tok, g_aux, grad, grad16


# ---- encoder --------------------------------------------------------------------------------

def encoder_gemm(x: torch.Tensor, w_enc_t: torch.Tensor, out_dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """pre[B, F] = x[B, d] @ w_enc_t[F, d]^T (`out`: a contiguous [B, F] tensor of `out_dtype` to write into)."""
    _req(x, "x", ndim=2)
    _req(w_enc_t, "w_enc_t", ndim=2)
    if x.dtype != w_enc_t.dtype:
        raise TypeError(f"x ({x.dtype}) and w_enc_t ({w_enc_t.dtype}) must share a dtype")
    B, d = x.shape
    F, d2 = w_enc_t.shape
    if d != d2:
        raise ValueError(f"shape mismatch: x {tuple(x.shape)} vs w_enc_t {tuple(w_enc_t.shape)}")
    if out is not None:
        _req(out, "out", out_dtype, 2)
        if tuple(out.shape) != (B, F):
            raise ValueError(f"out must be {(B, F)}, got {tuple(out.shape)}")
    splits = gemm_split_k(B, d, F) if (x.dtype == torch.bfloat16 and out_dtype == torch.float32) else 1
    if splits > 1:
        partials = torch.empty(splits, B, F, dtype=torch.float32, device=x.device)
        with _timed("encoder_gemm"):
            check(_lib.load().sae_encoder_gemm_split_k(x.data_ptr(), w_enc_t.data_ptr(), partials.data_ptr(), splits, B, d, F,
                                                       _stream(x)), "encoder_gemm_split_k")
        return partials.sum(0) if out is None else torch.sum(partials, 0, out=out)
    pre = out if out is not None else torch.empty(B, F, dtype=out_dtype, device=x.device)
    with _timed("encoder_gemm"):
        check(
            _lib.load().sae_encoder_gemm(x.data_ptr(), w_enc_t.data_ptr(), pre.data_ptr(), B, d, F, _dt(x), _dt(pre), _stream(x)),
            "encoder_gemm",
        )
    return pre


def _k_major_read_pays(rows: int, other_rows: int, K: int, a_side: bool) -> bool:
    """Whether an operand stored [K, rows] is better read as it lies than copied into [rows, K] first.  Reading across
    the K-rows of the LDS tile takes two 8-byte reads per fragment instead of one 16-byte read: measured +16 % of the
    product's time for the operand whose rows are the output's rows (eight fragments per wave and k-step), +9 % for the
    other (four); a transposed copy moves 4 bytes per element at about 4.7 TB/s behind a launch of its own.  Both routes
    give the same bits."""
    t_gemm = 2.0 * rows * other_rows * K / 1.4e15
    extra = (0.16 if a_side else 0.09) * t_gemm
    copy = rows * K * 4.0 / 4.7e12 + 8e-6
    return extra <= copy


def gemm(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype, a_k_major: bool = False, b_k_major: bool = False,
         out: Optional[torch.Tensor] = None, copy_when_faster: bool = True) -> torch.Tensor:
    """out[M, N] = sum_k A[m, k] B[n, k] for bf16 operands in either layout: an operand is [rows, K] (its K values side by
    side, what `encoder_gemm` takes) or, with its `*_k_major` flag, [K, rows].  `gemm(g, x, dt, True, True)` is g^T @ x for
    g [tokens, m], x [tokens, n] (a weight gradient over the token axis); `gemm(acts, W, dt, False, True)` is acts @ W for
    W [K, n] (a dense decode).  A [K, rows] operand is read as it lies, with no transposed copy, unless
    `copy_when_faster` and a copy is the cheaper way for the shape (`_k_major_read_pays`); the result is the same bit
    for bit."""
    _req(a, "a", torch.bfloat16, 2)
    _req(b, "b", torch.bfloat16, 2)
    K, M = a.shape if a_k_major else (a.shape[1], a.shape[0])
    Kb, N = b.shape if b_k_major else (b.shape[1], b.shape[0])
    if K != Kb:
        raise ValueError(f"contraction lengths differ: a {tuple(a.shape)} (k-major {a_k_major}) vs b {tuple(b.shape)} (k-major {b_k_major})")
    if out is not None:
        _req(out, "out", out_dtype, 2)
        if tuple(out.shape) != (M, N):
            raise ValueError(f"out must be {(M, N)}, got {tuple(out.shape)}")
    if copy_when_faster:
        if a_k_major and not _k_major_read_pays(M, N, K, True):
            a, a_k_major = transpose_to_bf16(a)[0], False
        if b_k_major and not _k_major_read_pays(N, M, K, False):
            b, b_k_major = transpose_to_bf16(b)[0], False
    splits = gemm_split_k(M, K, N) if out_dtype == torch.float32 and (M * N) % 4 == 0 else 1
    lib = _lib.load()
    if splits > 1:
        partials = torch.empty(splits, M, N, dtype=torch.float32, device=a.device)
        with _timed("encoder_gemm"):
            check(lib.sae_gemm_bf16(a.data_ptr(), int(a_k_major), b.data_ptr(), int(b_k_major), partials.data_ptr(), SAE_F32, M, N, K,
                                    splits, _stream(a)), "gemm_bf16")
        return partials.sum(0) if out is None else torch.sum(partials, 0, out=out)
    res = out if out is not None else torch.empty(M, N, dtype=out_dtype, device=a.device)
    with _timed("encoder_gemm"):
        check(lib.sae_gemm_bf16(a.data_ptr(), int(a_k_major), b.data_ptr(), int(b_k_major), res.data_ptr(), _dt(res), M, N, K, 1,
                                _stream(a)), "gemm_bf16")
    return res


def gemm_split_k(B: int, d: int, F: int) -> int:
    """How many slices of the contraction axis a bf16 -> fp32 product [B, d] x [F, d]^T is cut into: products with few
    256 x 256 output tiles and a long contraction (weight gradients over the token axis) would occupy a fraction of the
    256 CUs; slices run as one launch and their fp32 results are summed in slice order (deterministic, and the same for
    every caller of a shape).  1: no split."""
    tiles = ((B + 255) // 256) * ((F + 255) // 256)
    if tiles > 128 or d < 4096:
        return 1
    for g in (4, 3, 2):
        if tiles * g <= 256 and d % (64 * g) == 0 and d // g >= 2048:
            return g
    return 1


def encoder_gemm_bias(x: torch.Tensor, w_t: torch.Tensor, col_bias: Optional[torch.Tensor] = None,
                      row_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 out[B, F] = bf16(float(bf16(x @ w_t^T)) + col_bias[F] + row_bias[B]): a projection with its bias as a bf16
    autocast product plus an fp32 bias gives it."""
    _req(x, "x", torch.bfloat16, 2)
    _req(w_t, "w_t", torch.bfloat16, 2)
    B, d = x.shape
    F, d2 = w_t.shape
    if d != d2:
        raise ValueError(f"shape mismatch: x {tuple(x.shape)} vs w_t {tuple(w_t.shape)}")
    for name, t, n in (("col_bias", col_bias, F), ("row_bias", row_bias, B)):
        if t is not None:
            _req(t, name, torch.float32)
            if t.numel() != n:
                raise ValueError(f"{name} must have {n} elements")
    out = torch.empty(B, F, dtype=torch.bfloat16, device=x.device)
    with _timed("encoder_gemm"):
        check(_lib.load().sae_encoder_gemm_bias(x.data_ptr(), w_t.data_ptr(), out.data_ptr(), B, d, F, _ptr(col_bias),
                                                _ptr(row_bias), _stream(x)), "encoder_gemm_bias")
    return out


GRANULE = 64                 # features per granule of the granule-maximum route
GRANULE_MAX_F = 64 * 4096
GRANULE_MAX_K = 512


def granule_route_supported(d: int, F: int, k: int) -> bool:
    """Shapes `encoder_gemm_granule_max` + `select_topk_row(..., granule_max=...)` take."""
    return d % 64 == 0 and F % GRANULE == 0 and F <= GRANULE_MAX_F and 1 <= k <= GRANULE_MAX_K


def encoder_gemm_granule_max(x: torch.Tensor, w_enc_t: torch.Tensor, b_enc: Optional[torch.Tensor],
                             scale: Optional[torch.Tensor], lowp: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 pre[B, F] = x @ w_enc_t^T plus granule_max [B, F / 64] (int32 holding uint32 keys): per token and aligned
    granule of 64 features the largest select key, i.e. the bits of (pre + b_enc) * scale where that is positive.
    With a leading group dimension on every argument (x [G, B, d], w_enc_t [G, F, d], b_enc / scale [G, F]) the G
    products run in one launch and the outputs are [G, B, F] and [G, B, F / 64]."""
    grouped = x.dim() == 3
    _req(x, "x", torch.bfloat16, 3 if grouped else 2)
    _req(w_enc_t, "w_enc_t", torch.bfloat16, 3 if grouped else 2)
    G = x.shape[0] if grouped else 1
    B, d = x.shape[-2:]
    F, d2 = w_enc_t.shape[-2:]
    if d != d2 or (grouped and w_enc_t.shape[0] != G):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)} vs w_enc_t {tuple(w_enc_t.shape)}")
    for name, t in (("b_enc", b_enc), ("scale", scale)):
        if t is not None:
            _req(t, name, torch.float32, 2 if grouped else 1)
            if t.numel() != G * F:
                raise ValueError(f"{name} must have {G * F} elements")
    lead = (G,) if grouped else ()
    pre = torch.empty(*lead, B, F, dtype=torch.bfloat16, device=x.device)
    gmax = torch.empty(*lead, B, max(F // GRANULE, 1), dtype=torch.int32, device=x.device)
    lib = _lib.load()
    fn = lib.sae_encoder_gemm_granule_max_lowp if lowp else lib.sae_encoder_gemm_granule_max   # keys in bf16 arithmetic
    with _timed("encoder_gemm"):
        check(fn(x.data_ptr(), w_enc_t.data_ptr(), pre.data_ptr(), G, B, d, F, _ptr(b_enc), _ptr(scale), gmax.data_ptr(),
                 _stream(x)), "encoder_gemm_granule_max")
    return pre, gmax


def granule_max(pre: torch.Tensor, b_enc: Optional[torch.Tensor], scale: Optional[torch.Tensor], rows_per_group: int = 0,
                n_rows: Optional[int] = None) -> torch.Tensor:
    """The granule maxima `encoder_gemm_granule_max` leaves, for a bf16 pre [B, F] from elsewhere.  `n_rows` (a multiple of
    B) > B: the maxima of n_rows virtual rows that share pre's B rows (row r reads pre row r % B) under the bias / scale
    vector of their group r / rows_per_group."""
    _req(pre, "pre", torch.bfloat16, 2)
    B, F = pre.shape
    rows = B if n_rows is None else int(n_rows)
    if rows % B:
        raise ValueError(f"n_rows = {rows} is not a multiple of pre's {B} rows")
    n_vec = F * (rows // rows_per_group if rows_per_group else 1)
    for name, t in (("b_enc", b_enc), ("scale", scale)):
        if t is not None:
            _req(t, name, torch.float32)
            if t.numel() != n_vec:
                raise ValueError(f"{name} must have {n_vec} elements")
    gmax = torch.empty(rows, max(F // GRANULE, 1), dtype=torch.int32, device=pre.device)
    with _timed("granule_max"):
        check(_lib.load().sae_granule_max(pre.data_ptr(), _ptr(b_enc), _ptr(scale), rows, F, int(rows_per_group), B, gmax.data_ptr(),
                                          _stream(pre)), "granule_max")
    return gmax


def encoder_gemm_jumprelu_margin(x: torch.Tensor, w_enc_t: torch.Tensor, b_enc: Optional[torch.Tensor], scale: Optional[torch.Tensor],
                                 theta: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 pre[B, F] = x @ w_enc_t^T plus granule_margin [B, F / 64] fp32: per token and aligned granule of 64 features the
    largest (pre + b_enc) * scale - theta (what `jumprelu_select(..., granule_margin=...)` prunes the row with)."""
    _req(x, "x", torch.bfloat16, 2)
    _req(w_enc_t, "w_enc_t", torch.bfloat16, 2)
    B, d = x.shape
    F, d2 = w_enc_t.shape
    if d != d2:
        raise ValueError(f"shape mismatch: x {tuple(x.shape)} vs w_enc_t {tuple(w_enc_t.shape)}")
    for name, t in (("b_enc", b_enc), ("scale", scale), ("theta", theta)):
        if t is not None:
            _req(t, name, torch.float32, 1)
            if t.numel() != F:
                raise ValueError(f"{name} must have {F} elements")
    pre = torch.empty(B, F, dtype=torch.bfloat16, device=x.device)
    margin = torch.empty(B, max(F // GRANULE, 1), dtype=torch.float32, device=x.device)
    with _timed("encoder_gemm"):
        check(_lib.load().sae_encoder_gemm_jumprelu_margin(x.data_ptr(), w_enc_t.data_ptr(), pre.data_ptr(), B, d, F, _ptr(b_enc),
                                                           _ptr(scale), theta.data_ptr(), margin.data_ptr(), _stream(x)),
              "encoder_gemm_jumprelu_margin")
    return pre, margin


def merge_layer_codes(code: SparseCode, L: int) -> Tuple[SparseCode, torch.Tensor]:
    """`code`: one select over L * B stacked rows (row l * B + b, at most k entries each, F features) -> the code over
    L * F features with L * k slots per token (feature l * F + f, ascending) and the entry counts [B, L]."""
    rows, F = code.n_tokens, code.d_sae
    if rows % L:
        raise ValueError(f"{rows} rows are not {L} layers of equally many tokens")
    B, k = rows // L, code.idx.numel() // rows
    dev = code.idx.device
    idx = torch.empty(B * L * k, dtype=torch.int32, device=dev)
    val = torch.empty(B * L * k, dtype=torch.float32, device=dev)
    row_off = torch.empty(B, dtype=torch.int64, device=dev)
    row_nnz = torch.empty(B, dtype=torch.int32, device=dev)
    layer_cnt = torch.empty(B, L, dtype=torch.int32, device=dev)
    with _timed("merge_layer_codes"):
        check(_lib.load().sae_merge_layer_codes(code.idx.data_ptr(), code.val.data_ptr(), code.row_nnz.data_ptr(), L, B, k, F,
                                                idx.data_ptr(), val.data_ptr(), row_off.data_ptr(), row_nnz.data_ptr(),
                                                layer_cnt.data_ptr(), _stream(code.idx)), "merge_layer_codes")
    return SparseCode(idx, val, row_off, row_nnz, B, L * F), layer_cnt


def union_group_codes(code: SparseCode, groups: int) -> SparseCode:
    """`code`: one select over groups * B stacked rows (row g * B + b, at most k entries each) -> the code over the B tokens
    that holds every (token, feature) once, with the sum of the values it carries in the token's rows; groups * k slots per
    token, distinct features in order of first appearance."""
    rows = code.n_tokens
    if rows % groups:
        raise ValueError(f"{rows} rows are not {groups} groups of equally many tokens")
    B, k = rows // groups, code.idx.numel() // rows
    if code.idx.numel() != rows * k or groups * k > 1024:
        raise ValueError("union_group_codes takes rows of equally many slots, at most 1024 per token in all")
    dev = code.idx.device
    idx = torch.empty(B * groups * k, dtype=torch.int32, device=dev)
    val = torch.empty(B * groups * k, dtype=torch.float32, device=dev)
    row_off = torch.empty(B, dtype=torch.int64, device=dev)
    row_nnz = torch.empty(B, dtype=torch.int32, device=dev)
    with _timed("union_group_codes"):
        check(_lib.load().sae_union_group_codes(code.idx.data_ptr(), code.val.data_ptr(), code.row_nnz.data_ptr(), groups, B, k,
                                                idx.data_ptr(), val.data_ptr(), row_off.data_ptr(), row_nnz.data_ptr(),
                                                _stream(code.idx)), "union_group_codes")
    return SparseCode(idx, val, row_off, row_nnz, B, code.d_sae)


# ---- select ---------------------------------------------------------------------------------

def select_topk_row(
    pre: torch.Tensor,
    b_enc: Optional[torch.Tensor],
    scale: Optional[torch.Tensor],
    k: int,
    cand_cap: Optional[int] = None,
    feat_mask: Optional[torch.Tensor] = None,
    lowp: bool = False,
    granule_max: Optional[torch.Tensor] = None,
    rows_per_group: int = 0,
    n_rows: Optional[int] = None,
) -> SparseCode:
    """Per-token TopK of (pre + b_enc) * scale.  `lowp`: bf16 `pre`, every intermediate rounded to bf16 (the
    arithmetic of a dictionary whose parameters are bf16 tensors).  `feat_mask` (0/1 per feature): the aux-k selection
    among the masked-in features, with the reference's key arithmetic for it.  `granule_max`: the second output of
    `encoder_gemm_granule_max` for the same pre, b_enc and scale; the row is then read only where a kept element
    can be (same result).  On that route `rows_per_group` > 0 says that the rows come in groups of that many and that
    b_enc / scale hold one vector of F per group; `n_rows` (a multiple of pre's row count) > that count says that the
    groups share pre's rows (row r of the code reads pre row r % pre.shape[0]: a crosscoder's heads over one summed
    encoding), granule_max then being `granule_max(pre, ..., n_rows=n_rows)`."""
    _req(pre, "pre", ndim=2)
    pre_rows, F = pre.shape
    B = pre_rows if n_rows is None else int(n_rows)
    if B % pre_rows or (B != pre_rows and granule_max is None):
        raise ValueError("n_rows needs the granule route and must be a multiple of pre's row count")
    n_vec = F * (B // rows_per_group if rows_per_group else 1)
    if rows_per_group and (granule_max is None or B % rows_per_group):
        raise ValueError("rows_per_group needs the granule route and must divide the number of rows")
    if lowp and (pre.dtype != torch.bfloat16 or cand_cap is not None):
        raise ValueError("lowp select takes a bf16 pre and no cand_cap")
    if granule_max is not None:
        if cand_cap is not None or feat_mask is not None or pre.dtype != torch.bfloat16:
            raise ValueError("the granule route takes a bf16 pre and neither cand_cap nor feat_mask")
        _req(granule_max, "granule_max", torch.int32, 2)
        if tuple(granule_max.shape) != (B, F // GRANULE) or F % GRANULE:
            raise ValueError(f"granule_max must be [{B}, {F}/{GRANULE}]")
    for name, t in (("b_enc", b_enc), ("scale", scale), ("feat_mask", feat_mask)):
        if t is not None:
            _req(t, name, torch.float32)
            if t.numel() != (F if name == "feat_mask" else n_vec):
                raise ValueError(f"{name} must have {n_vec} elements")
    k = int(k)
    dev = pre.device
    # zero-filled: slots a row does not use (fewer than k positive entries) then hold feature 0 with value 0
    idx = torch.empty(B * k, dtype=torch.int32, device=dev)     # the kernel writes every slot (zeros in unused ones)
    val = torch.empty(B * k, dtype=torch.float32, device=dev)
    row_off = torch.empty(B, dtype=torch.int64, device=dev)
    row_nnz = torch.empty(B, dtype=torch.int32, device=dev)
    lib = _lib.load()
    _t = _timed("select_topk_row[granule]" if granule_max is not None else "select_topk_row")
    _t.__enter__()
    if granule_max is not None:
        fn = lib.sae_select_topk_row_granule_lowp if lowp else lib.sae_select_topk_row_granule
        rc = fn(pre.data_ptr(), granule_max.data_ptr(), _ptr(b_enc), _ptr(scale), B, F, k, int(rows_per_group), pre_rows,
                idx.data_ptr(), val.data_ptr(), row_off.data_ptr(), row_nnz.data_ptr(), _stream(pre))
    elif lowp:
        rc = lib.sae_select_topk_row_lowp(pre.data_ptr(), _ptr(b_enc), _ptr(scale), _ptr(feat_mask), B, F, k, idx.data_ptr(),
                                          val.data_ptr(), row_off.data_ptr(), row_nnz.data_ptr(), _stream(pre))
    elif cand_cap is None and feat_mask is None:
        rc = lib.sae_select_topk_row(pre.data_ptr(), _dt(pre), _ptr(b_enc), _ptr(scale), B, F, k, idx.data_ptr(),
                                     val.data_ptr(), row_off.data_ptr(), row_nnz.data_ptr(), _stream(pre))
    else:
        rc = lib.sae_select_topk_row_ex(pre.data_ptr(), _dt(pre), _ptr(b_enc), _ptr(scale), _ptr(feat_mask), B, F, k,
                                        idx.data_ptr(), val.data_ptr(), row_off.data_ptr(), row_nnz.data_ptr(),
                                        4096 if cand_cap is None else int(cand_cap), _stream(pre))
    _t.__exit__()
    check(rc, "select_topk_row")
    return SparseCode(idx, val, row_off, row_nnz, B, F)


def select_topk_batch(
    pre: torch.Tensor,
    b_enc: Optional[torch.Tensor],
    scale: Optional[torch.Tensor],
    k_total,
    feat_mask: Optional[torch.Tensor] = None,
    capacity: Optional[int] = None,
    granule_max: Optional[torch.Tensor] = None,
    lowp: bool = False,
) -> SparseCode:
    """Batch-global TopK.  `k_total` is an int, or a device int64 tensor (then `capacity` is required).
    `lowp`: bf16 `pre`, every intermediate rounded to bf16 (the arithmetic of a dictionary held in bf16).
    `granule_max`: the second output of `encoder_gemm_granule_max` for the same bf16 pre, b_enc and scale (F a multiple
    of 256, no feat_mask); the select's one full pass over the matrix then shrinks to a histogram of those maxima."""
    _req(pre, "pre", ndim=2)
    B, F = pre.shape
    if lowp and pre.dtype != torch.bfloat16:
        raise ValueError("lowp select takes a bf16 pre")
    if granule_max is not None:
        if feat_mask is not None or pre.dtype != torch.bfloat16 or F % 256:
            raise ValueError("granule_max needs a bf16 pre with F a multiple of 256 and no feat_mask")
        _req(granule_max, "granule_max", torch.int32, 2)
        if tuple(granule_max.shape) != (B, F // GRANULE):
            raise ValueError(f"granule_max must be [{B}, {F // GRANULE}]")
    for name, t in (("b_enc", b_enc), ("scale", scale), ("feat_mask", feat_mask)):
        if t is not None:
            _req(t, name, torch.float32, 1)
            if t.numel() != F:
                raise ValueError(f"{name} must have {F} elements")
    dev = pre.device
    k_dev = None
    if isinstance(k_total, torch.Tensor):
        _req(k_total, "k_total", torch.int64)
        if capacity is None:
            raise ValueError("capacity is required when k_total lives on the device")
        k_dev, k_host = k_total, 0
    else:
        k_host = int(k_total)
        if capacity is None:
            capacity = max(min(k_host, B * F), 1)
    idx = torch.zeros(capacity, dtype=torch.int32, device=dev)
    val = torch.zeros(capacity, dtype=torch.float32, device=dev)
    row_off = torch.empty(B, dtype=torch.int64, device=dev)
    row_nnz = torch.empty(B, dtype=torch.int32, device=dev)
    lib = _lib.load()
    ws_bytes = lib.sae_select_topk_batch_workspace_bytes(B, F)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with _timed("select_topk_batch"):
        if granule_max is not None and lowp:
            rc = lib.sae_select_topk_batch_lowp(pre.data_ptr(), granule_max.data_ptr(), _ptr(b_enc), _ptr(scale), None, B, F, k_host,
                                                _ptr(k_dev), idx.data_ptr(), val.data_ptr(), capacity, row_off.data_ptr(),
                                                row_nnz.data_ptr(), None, ws.data_ptr(), ws_bytes, _stream(pre))
        elif granule_max is not None:
            rc = lib.sae_select_topk_batch_granule(pre.data_ptr(), granule_max.data_ptr(), _ptr(b_enc), _ptr(scale), B, F, k_host,
                                                   _ptr(k_dev), idx.data_ptr(), val.data_ptr(), capacity, row_off.data_ptr(),
                                                   row_nnz.data_ptr(), None, ws.data_ptr(), ws_bytes, _stream(pre))
        elif lowp:
            rc = lib.sae_select_topk_batch_lowp(pre.data_ptr(), None, _ptr(b_enc), _ptr(scale), _ptr(feat_mask), B, F, k_host,
                                                _ptr(k_dev), idx.data_ptr(), val.data_ptr(), capacity, row_off.data_ptr(),
                                                row_nnz.data_ptr(), None, ws.data_ptr(), ws_bytes, _stream(pre))
        else:
            rc = lib.sae_select_topk_batch(pre.data_ptr(), _dt(pre), _ptr(b_enc), _ptr(scale), _ptr(feat_mask), B, F, k_host,
                                           _ptr(k_dev), idx.data_ptr(), val.data_ptr(), capacity, row_off.data_ptr(),
                                           row_nnz.data_ptr(), None, ws.data_ptr(), ws_bytes, _stream(pre))
        check(rc, "select_topk_batch")
    return SparseCode(idx, val, row_off, row_nnz, B, F)


# ---- sparse decoder -------------------------------------------------------------------------

def _check_code(code: SparseCode, w_dec: torch.Tensor):
    _req(code.idx, "idx", torch.int32, 1)
    _req(code.val, "val", torch.float32, 1)
    _req(code.row_off, "row_off", torch.int64, 1)
    _req(code.row_nnz, "row_nnz", torch.int32, 1)
    _req(w_dec, "w_dec", ndim=2)
    if w_dec.shape[0] != code.d_sae:
        raise ValueError(f"w_dec has {w_dec.shape[0]} rows, the code addresses {code.d_sae} features")


def sparse_decode_fwd(code: SparseCode, w_dec: torch.Tensor, b_dec: Optional[torch.Tensor]) -> torch.Tensor:
    _check_code(code, w_dec)
    F, d = w_dec.shape
    B = code.n_tokens
    if b_dec is not None:
        _req(b_dec, "b_dec", torch.float32, 1)
    recon = torch.empty(B, d, dtype=torch.float32, device=w_dec.device)
    with _timed("sparse_decode_fwd"):
        check(
            _lib.load().sae_sparse_decode_fwd(code.idx.data_ptr(), code.val.data_ptr(), code.row_off.data_ptr(),
                                              code.row_nnz.data_ptr(), w_dec.data_ptr(), _dt(w_dec), _ptr(b_dec),
                                              recon.data_ptr(), B, d, F, _stream(w_dec)),
            "sparse_decode_fwd",
        )
    return recon


def sparse_decode_bwd_dval(code: SparseCode, grad_recon: torch.Tensor, w_dec: torch.Tensor) -> torch.Tensor:
    _check_code(code, w_dec)
    _req(grad_recon, "grad_recon", torch.float32, 2)
    F, d = w_dec.shape
    B = code.n_tokens
    dval = torch.empty(code.n_slots, dtype=torch.float32, device=w_dec.device)
    with _timed("sparse_decode_bwd_dval"):
        check(
            _lib.load().sae_sparse_decode_bwd_dval(code.idx.data_ptr(), code.row_off.data_ptr(), code.row_nnz.data_ptr(),
                                                   grad_recon.data_ptr(), w_dec.data_ptr(), _dt(w_dec), dval.data_ptr(),
                                                   B, d, F, code.n_slots, _stream(w_dec)),
            "sparse_decode_bwd_dval",
        )
    return dval


def sparse_decode_mse_fused(code: SparseCode, w_dec: torch.Tensor, b_dec: Optional[torch.Tensor], label: torch.Tensor,
                            tok_w: Optional[torch.Tensor], want_recon: bool = True, recon_out: Optional[torch.Tensor] = None,
                            loss_out: Optional[torch.Tensor] = None, dval_acc: Optional[torch.Tensor] = None,
                            grad_out: Optional[torch.Tensor] = None):
    """Returns (recon or None, loss_tok [B], grad_recon [B, d], dval [n_slots]).  `recon_out` [B, d] / `loss_out` [B] /
    `grad_out` [B, d] (fp32, contiguous) receive those outputs in place of fresh tensors; `dval_acc` [n_slots] has the
    value gradients added to it (and is returned as dval) instead of being overwritten: for a code several decoders share."""
    _check_code(code, w_dec)
    _req(label, "label", torch.float32, 2)
    F, d = w_dec.shape
    B = code.n_tokens
    if tuple(label.shape) != (B, d):
        raise ValueError(f"label must be {(B, d)}, got {tuple(label.shape)}")
    if tok_w is not None:
        _req(tok_w, "tok_w", torch.float32, 1)
    dev = w_dec.device
    if recon_out is not None:
        _req(recon_out, "recon_out", torch.float32, 2)
        if tuple(recon_out.shape) != (B, d):
            raise ValueError(f"recon_out must be {(B, d)}")
    if loss_out is not None:
        _req(loss_out, "loss_out", torch.float32, 1)
        if loss_out.numel() != B:
            raise ValueError(f"loss_out must hold {B} values")
    if dval_acc is not None:
        _req(dval_acc, "dval_acc", torch.float32, 1)
        if dval_acc.numel() != code.n_slots:
            raise ValueError(f"dval_acc must hold {code.n_slots} values")
    recon = recon_out if recon_out is not None else (torch.empty(B, d, dtype=torch.float32, device=dev) if want_recon else None)
    loss_tok = loss_out if loss_out is not None else torch.empty(B, dtype=torch.float32, device=dev)
    if grad_out is not None:
        _req(grad_out, "grad_out", torch.float32, 2)
        if tuple(grad_out.shape) != (B, d):
            raise ValueError(f"grad_out must be {(B, d)}")
    grad_recon = grad_out if grad_out is not None else torch.empty(B, d, dtype=torch.float32, device=dev)
    dval = dval_acc if dval_acc is not None else torch.empty(code.n_slots, dtype=torch.float32, device=dev)
    lib = _lib.load()
    fn = lib.sae_sparse_decode_mse_fused_acc if dval_acc is not None else lib.sae_sparse_decode_mse_fused
    with _timed("sparse_decode_mse_fused"):
        check(
            fn(code.idx.data_ptr(), code.val.data_ptr(), code.row_off.data_ptr(), code.row_nnz.data_ptr(), w_dec.data_ptr(),
               _dt(w_dec), _ptr(b_dec), label.data_ptr(), _ptr(tok_w), _ptr(recon), loss_tok.data_ptr(), grad_recon.data_ptr(),
               dval.data_ptr(), B, d, F, code.n_slots, _stream(w_dec)),
            "sparse_decode_mse_fused",
        )
    return recon, loss_tok, grad_recon, dval


# ---- sparse backward ------------------------------------------------------------------------

def build_feature_index(code: SparseCode) -> FeatureIndex:
    dev = code.idx.device
    B, F, n = code.n_tokens, code.d_sae, code.n_slots
    lib = _lib.load()
    ws_bytes = lib.sae_feature_index_workspace_bytes(B, F, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    feat_ptr = torch.empty(F + 1, dtype=torch.int32, device=dev)
    feat_slot = torch.empty(n, dtype=torch.int32, device=dev)
    slot_tok = torch.zeros(n, dtype=torch.int32, device=dev)
    with _timed("build_feature_index"):
        check(
            lib.sae_build_feature_index(code.idx.data_ptr(), code.row_off.data_ptr(), code.row_nnz.data_ptr(), B, F, n,
                                        feat_ptr.data_ptr(), feat_slot.data_ptr(), slot_tok.data_ptr(), ws.data_ptr(),
                                        ws_bytes, _stream(code.idx)),
            "build_feature_index",
        )
    return FeatureIndex(feat_ptr, feat_slot, slot_tok)


def sparse_grad_rows(fi: FeatureIndex, coef: torch.Tensor, dense: torch.Tensor, F: int, want_bias: bool = False,
                     out: Optional[torch.Tensor] = None):
    """out[f, :] = sum over feature f's slots of coef[slot] * dense[token(slot), :]; optional bias_out[f] = sum coef."""
    _req(coef, "coef", torch.float32, 1)
    _req(dense, "dense", ndim=2)
    d = dense.shape[1]
    dev = dense.device
    if out is None:
        out = torch.empty(F, d, dtype=torch.float32, device=dev)
    bias = torch.empty(F, dtype=torch.float32, device=dev) if want_bias else None
    with _timed("sparse_grad_rows[bf16 dense]" if dense.dtype == torch.bfloat16 else "sparse_grad_rows[f32 dense]"):
        check(
            _lib.load().sae_sparse_grad_rows(fi.feat_ptr.data_ptr(), fi.feat_slot.data_ptr(), fi.slot_tok.data_ptr(),
                                             coef.data_ptr(), dense.data_ptr(), _dt(dense), out.data_ptr(), _ptr(bias), F, d,
                                             _stream(dense)),
            "sparse_grad_rows",
        )
    return out, bias


# ---- optimiser ------------------------------------------------------------------------------

def adam_step(p: torch.Tensor, g: torch.Tensor, m: torch.Tensor, v: torch.Tensor, *, lr: float, beta1: float,
              beta2: float, eps: float, step: int, shadow_bf16: Optional[torch.Tensor] = None,
              row_norm_out: Optional[torch.Tensor] = None, row_len: int = 0,
              row_grad_coef: Optional[torch.Tensor] = None) -> None:
    """One Adam update; `g` may be bf16 (widened as it is read); with `row_grad_coef` (fp32, one value per row of
    `row_len` elements) the gradient of row r is g + row_grad_coef[r] * p.  A bf16 `p` (with bf16 `m`, `v`) takes the
    low-precision update that rounds after every element-wise operation, as torch's Adam does on bf16 tensors."""
    lowp = p.dtype == torch.bfloat16
    for name, t in (("p", p), ("g", g), ("m", m), ("v", v)):
        if name == "g" and t.dtype == torch.bfloat16:
            _req(t, name, torch.bfloat16)
        else:
            _req(t, name, torch.bfloat16 if lowp and name != "g" else torch.float32)
        if t.numel() != p.numel():
            raise ValueError(f"{name} must have {p.numel()} elements")
    if shadow_bf16 is not None:
        if lowp:
            raise ValueError("a bf16 parameter has no shadow copy")
        _req(shadow_bf16, "shadow_bf16", torch.bfloat16)
    if row_grad_coef is not None:
        _req(row_grad_coef, "row_grad_coef", torch.float32, 1)
        if row_len <= 0 or row_grad_coef.numel() * row_len != p.numel():
            raise ValueError("row_grad_coef needs row_len > 0 and one value per row")
    with _timed("adam_step[matrix]" if p.ndim == 2 else "adam_step[vector]"):
        if lowp:
            check(
                _lib.load().sae_adam_step_lowp(p.data_ptr(), g.data_ptr(), _dt(g), m.data_ptr(), v.data_ptr(), p.numel(), lr,
                                               beta1, beta2, eps, int(step), _ptr(row_norm_out), int(row_len),
                                               _ptr(row_grad_coef), _stream(p)),
                "adam_step_lowp",
            )
            return
        check(
            _lib.load().sae_adam_step(p.data_ptr(), g.data_ptr(), _dt(g), m.data_ptr(), v.data_ptr(), p.numel(), lr, beta1, beta2,
                                      eps, int(step), _ptr(shadow_bf16), _ptr(row_norm_out), int(row_len), _ptr(row_grad_coef),
                                      _stream(p)),
            "adam_step",
        )


def adam_step_sparse_rows(fi: FeatureIndex, coef: torch.Tensor, dense: torch.Tensor, p: torch.Tensor, m: torch.Tensor,
                          v: torch.Tensor, *, lr: float, beta1: float, beta2: float, eps: float, step: int,
                          shadow_bf16: Optional[torch.Tensor] = None, row_norm_out: Optional[torch.Tensor] = None,
                          bias_grad_out: Optional[torch.Tensor] = None, grad_scale: Optional[torch.Tensor] = None,
                          grad_sq_nnz_acc: Optional[torch.Tensor] = None, extra: Optional["DenseRowBlock"] = None,
                          row_grad_coef: Optional[torch.Tensor] = None) -> None:
    """Adam on a feature-major [F, d] matrix whose gradient rows are rebuilt from (fi, coef, dense);
    `row_grad_coef` (fp32 [F]) adds row_grad_coef[f] * p[f, :] to row f's gradient (the gradient through the row norm);
    `grad_scale` (device float scalar) multiplies the gradient first (gradient clipping);
    `grad_sq_nnz_acc` (device double[2]) += (sum g^2, #non-zero g) of the gradient consumed;
    `extra` adds a densely held block of gradient rows.  A bf16 `p` (with bf16 `m`, `v`) takes the low-precision
    update (no shadow copy, no row coefficient)."""
    lowp = p.dtype == torch.bfloat16
    for name, t in (("p", p), ("m", m), ("v", v)):
        _req(t, name, torch.bfloat16 if lowp else torch.float32, 2)
    if lowp and (shadow_bf16 is not None or row_grad_coef is not None):
        raise ValueError("the low-precision update takes neither a shadow copy nor a row coefficient")
    if row_grad_coef is not None:
        _req(row_grad_coef, "row_grad_coef", torch.float32, 1)
        if row_grad_coef.numel() != p.shape[0]:
            raise ValueError("row_grad_coef must have one entry per row")
    _req(coef, "coef", torch.float32, 1)
    _req(dense, "dense", ndim=2)
    F, d = p.shape
    if dense.shape[1] != d or m.shape != p.shape or v.shape != p.shape:
        raise ValueError("shape mismatch between p, m, v and the dense operand")
    if fi.feat_ptr.numel() != F + 1:
        raise ValueError("feature index was built for a different number of features")
    if shadow_bf16 is not None:
        _req(shadow_bf16, "shadow_bf16", torch.bfloat16)
    if grad_scale is not None:
        _req(grad_scale, "grad_scale", torch.float32)
    ws, ws_bytes = None, 0
    if grad_sq_nnz_acc is not None:
        _req(grad_sq_nnz_acc, "grad_sq_nnz_acc", torch.float64, 1)
        ws_bytes = 16 * F
        ws = torch.empty(2 * F, dtype=torch.float64, device=p.device)
    with _timed("adam_step_sparse_rows[bf16 dense]" if dense.dtype == torch.bfloat16 else "adam_step_sparse_rows[f32 dense]"):
        if lowp:
            check(
                _lib.load().sae_adam_step_sparse_rows_lowp(fi.feat_ptr.data_ptr(), fi.feat_slot.data_ptr(), fi.slot_tok.data_ptr(),
                                                           coef.data_ptr(), dense.data_ptr(), _dt(dense), p.data_ptr(),
                                                           m.data_ptr(), v.data_ptr(), F, d, lr, beta1, beta2, eps, int(step),
                                                           _ptr(row_norm_out), _ptr(bias_grad_out), _ptr(grad_scale),
                                                           _ptr(grad_sq_nnz_acc), _ptr(ws), ws_bytes, *_extra_ptrs(extra, F, d),
                                                           _stream(p)),
                "adam_step_sparse_rows_lowp",
            )
            return
        check(
            _lib.load().sae_adam_step_sparse_rows(fi.feat_ptr.data_ptr(), fi.feat_slot.data_ptr(), fi.slot_tok.data_ptr(),
                                                  coef.data_ptr(), dense.data_ptr(), _dt(dense), p.data_ptr(), m.data_ptr(),
                                                  v.data_ptr(), F, d, lr, beta1, beta2, eps, int(step), _ptr(shadow_bf16),
                                                  _ptr(row_norm_out), _ptr(bias_grad_out), _ptr(grad_scale),
                                                  _ptr(grad_sq_nnz_acc), _ptr(ws), ws_bytes, *_extra_ptrs(extra, F, d),
                                                  _ptr(row_grad_coef), _stream(p)),
            "adam_step_sparse_rows",
        )


@dataclass
class DenseRowBlock:
    """Gradient rows held densely for a subset of features: `row_map` int32 [F] (-1 or the row of `rows`),
    `rows` fp32 [n, d], `bias` fp32 [n] or None (added to the per-feature bias gradient)."""

    row_map: torch.Tensor
    rows: torch.Tensor
    bias: Optional[torch.Tensor] = None


def _extra_ptrs(extra: Optional[DenseRowBlock], F: int, d: int):
    if extra is None:
        return None, None, None
    _req(extra.row_map, "extra.row_map", torch.int32, 1)
    _req(extra.rows, "extra.rows", torch.float32, 2)
    if extra.row_map.numel() != F or extra.rows.shape[1] != d:
        raise ValueError("dense row block does not fit the matrix")
    if extra.bias is not None:
        _req(extra.bias, "extra.bias", torch.float32, 1)
    return extra.row_map.data_ptr(), extra.rows.data_ptr(), _ptr(extra.bias)


def sparse_rows_grad_sq_nnz(fi: FeatureIndex, coef: torch.Tensor, dense: torch.Tensor, acc: torch.Tensor,
                            bias_grad_out: Optional[torch.Tensor] = None, extra: Optional[DenseRowBlock] = None) -> None:
    """acc (device double[2]) += (sum of squares, number of non-zero entries) of the [F, d] gradient that
    (fi, coef, dense) stand for; optionally writes the per-feature bias gradient as well."""
    _req(coef, "coef", torch.float32, 1)
    _req(dense, "dense", ndim=2)
    _req(acc, "acc", torch.float64, 1)
    F, d = fi.feat_ptr.numel() - 1, dense.shape[1]
    lib = _lib.load()
    nbytes = lib.sae_sparse_rows_grad_sq_nnz_workspace_bytes(F)
    ws = torch.empty(nbytes // 8, dtype=torch.float64, device=dense.device)
    with _timed("sparse_rows_grad_sq_nnz"):
        check(
            lib.sae_sparse_rows_grad_sq_nnz(fi.feat_ptr.data_ptr(), fi.feat_slot.data_ptr(), fi.slot_tok.data_ptr(),
                                            coef.data_ptr(), dense.data_ptr(), _dt(dense), F, d, acc.data_ptr(),
                                            _ptr(bias_grad_out), ws.data_ptr(), nbytes, *_extra_ptrs(extra, F, d), _stream(dense)),
            "sparse_rows_grad_sq_nnz",
        )


def sparse_adam_step(p: torch.Tensor, g: torch.Tensor, m: torch.Tensor, v: torch.Tensor, step_state: torch.Tensor, *,
                     lr: float, beta1: float, beta2: float, eps: float, shadow_bf16: Optional[torch.Tensor] = None) -> None:
    """SparseAdam on contiguous fp32 storage; `step_state` is a device float tensor [1] (steps taken so far)."""
    for name, t in (("p", p), ("g", g), ("m", m), ("v", v)):
        _req(t, name, torch.float32)
        if t.numel() != p.numel():
            raise ValueError(f"{name} must have {p.numel()} elements")
    _req(step_state, "step_state", torch.float32)
    flag = torch.empty(1, dtype=torch.int32, device=p.device)
    with _timed("sparse_adam_step"):
        check(
            _lib.load().sae_sparse_adam_step(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), p.numel(), lr, beta1,
                                             beta2, eps, step_state.data_ptr(), flag.data_ptr(), _ptr(shadow_bf16), _stream(p)),
            "sparse_adam_step",
        )


def grad_sq_nnz(grads) -> torch.Tensor:
    """device double[2]: (sum of squares, number of non-zero entries) over a list of fp32 tensors (bf16 ones
    are widened first: the small parameters of a dictionary held in bf16)."""
    grads = [g for g in grads if g is not None]
    assert len(grads) > 0, "No gradients found"
    acc = torch.zeros(2, dtype=torch.float64, device=grads[0].device)
    lib = _lib.load()
    for g in grads:
        if not g.is_contiguous():
            g = g.t() if g.ndim == 2 and g.t().is_contiguous() else g.contiguous()
        if g.dtype == torch.bfloat16:
            g = g.float()
        _req(g, "grad", torch.float32)
        with _timed("grad_sq_nnz"):
            check(lib.sae_grad_sq_nnz(g.data_ptr(), g.numel(), acc.data_ptr(), _stream(g)), "grad_sq_nnz")
    return acc


# ---- JumpReLU ---------------------------------------------------------------------------------

def jumprelu_fwd(pre: torch.Tensor, b_enc: Optional[torch.Tensor], scale: Optional[torch.Tensor], theta: torch.Tensor,
                 tanh_c: float = 0.0, pen_norm: Optional[torch.Tensor] = None, want_tanh: bool = False, want_lp: bool = False, want_l0: bool = False):
    """acts [B, F] (dtype of pre) and the requested per-token sums (tanh penalty, Lp penalty, L0), each [B] or None."""
    _req(pre, "pre", ndim=2)
    B, F = pre.shape
    for name, v in (("b_enc", b_enc), ("scale", scale), ("theta", theta), ("pen_norm", pen_norm)):
        if v is not None:
            _req(v, name, torch.float32, 1)
            if v.numel() != F:
                raise ValueError(f"{name} must have {F} elements")
    dev = pre.device
    acts = torch.empty_like(pre)
    mk = lambda want: torch.empty(B, dtype=torch.float32, device=dev) if want else None  # noqa: E731
    tanh_tok, lp_tok, l0_tok = mk(want_tanh), mk(want_lp), mk(want_l0)
    with _timed("jumprelu_fwd"):
        check(_lib.load().sae_jumprelu_fwd(pre.data_ptr(), _dt(pre), _ptr(b_enc), _ptr(scale), _ptr(pen_norm), theta.data_ptr(), B, F,
                                           float(tanh_c), acts.data_ptr(), _ptr(tanh_tok), _ptr(lp_tok), _ptr(l0_tok),
                                           _stream(pre)), "jumprelu_fwd")
    return acts, tanh_tok, lp_tok, l0_tok


def jumprelu_bwd(pre: torch.Tensor, b_enc: Optional[torch.Tensor], scale: Optional[torch.Tensor], theta: torch.Tensor,
                 d_acts: torch.Tensor, g_tanh: Optional[torch.Tensor], tanh_c: float, g_lp: Optional[torch.Tensor],
                 window: float, pen_norm: Optional[torch.Tensor] = None, want_norm_grad: bool = False):
    """(d_pre [B, F], d_bias [F], d_theta [F], d_pen_norm [F] or None)"""
    _req(pre, "pre", ndim=2)
    _req(d_acts, "d_acts", pre.dtype, 2)
    if d_acts.shape != pre.shape:
        raise ValueError("d_acts must have the shape of pre")
    B, F = pre.shape
    for name, v in (("g_tanh", g_tanh), ("g_lp", g_lp)):
        if v is not None:
            _req(v, name, torch.float32, 1)
            if v.numel() != B:
                raise ValueError(f"{name} must have {B} elements")
    dev = pre.device
    lib = _lib.load()
    d_pre = torch.empty_like(pre)
    d_bias = torch.empty(F, dtype=torch.float32, device=dev)
    d_theta = torch.empty(F, dtype=torch.float32, device=dev)
    d_scale = torch.empty(F, dtype=torch.float32, device=dev) if want_norm_grad else None
    ws_bytes = lib.sae_jumprelu_bwd_workspace_bytes(B, F)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with _timed("jumprelu_bwd"):
        check(lib.sae_jumprelu_bwd(pre.data_ptr(), _dt(pre), _ptr(b_enc), _ptr(scale), _ptr(pen_norm), theta.data_ptr(),
                                   d_acts.data_ptr(),
                                   _ptr(g_tanh), float(tanh_c), _ptr(g_lp), float(window), B, F, d_pre.data_ptr(),
                                   d_bias.data_ptr(), d_theta.data_ptr(), _ptr(d_scale), ws.data_ptr(), ws_bytes,
                                   _stream(pre)), "jumprelu_bwd")
    return d_pre, d_bias, d_theta, d_scale


def jumprelu_select(pre: torch.Tensor, b_enc: Optional[torch.Tensor], scale: Optional[torch.Tensor], theta: torch.Tensor,
                    window: float, tanh_c: float = 0.0, pen_norm: Optional[torch.Tensor] = None, want_tanh: bool = False,
                    max_entries: Optional[int] = None, granule_margin: Optional[torch.Tensor] = None):
    """Sparse form of the JumpReLU activation: the code of every token's kept features (value u / s) and of the features
    inside the straight-through window that are not kept (value 0) -> (code, in_window fp32 [n_slots], tanh_tok [B] or
    None, l0_tok [B]), or None when the batch holds no such entry or more than `max_entries` of them (the caller then
    takes the dense route).  The entry count is read back from the device to size the code: one synchronisation per call, as the
    reference's sparsity gate (models/sae.py:355-358).  `granule_margin`: the second output of `encoder_gemm_jumprelu_margin`
    for the same arguments; the kernels then read only the granules of `pre` that can hold an entry."""
    _req(pre, "pre", ndim=2)
    B, F = pre.shape
    if granule_margin is not None:
        _req(granule_margin, "granule_margin", torch.float32, 2)
        if tuple(granule_margin.shape) != (B, F // GRANULE) or F % GRANULE or F > GRANULE_MAX_F:
            raise ValueError(f"granule_margin must be [{B}, {F}/{GRANULE}] with F a multiple of {GRANULE}, at most {GRANULE_MAX_F}")
    lib = _lib.load()
    row_nnz = torch.empty(B, dtype=torch.int32, device=pre.device)
    with _timed("jumprelu_select"):
        check(lib.sae_jumprelu_select_count(pre.data_ptr(), _dt(pre), _ptr(b_enc), _ptr(scale), theta.data_ptr(), _ptr(granule_margin),
                                            float(window), B, F, row_nnz.data_ptr(), _stream(pre)), "jumprelu_select_count")
        incl = torch.cumsum(row_nnz, 0, dtype=torch.int64)
        total = int(incl[-1].item())
        if total == 0 or (max_entries is not None and total > max_entries):
            return None
        row_off = incl - row_nnz
        cap = max(total, 1)
        idx = torch.zeros(cap, dtype=torch.int32, device=pre.device)
        val = torch.zeros(cap, dtype=torch.float32, device=pre.device)
        win = torch.zeros(cap, dtype=torch.float32, device=pre.device)
        tanh_tok = torch.empty(B, dtype=torch.float32, device=pre.device) if want_tanh else None
        l0_tok = torch.empty(B, dtype=torch.float32, device=pre.device)
        check(lib.sae_jumprelu_select_emit(pre.data_ptr(), _dt(pre), _ptr(b_enc), _ptr(scale), _ptr(pen_norm), theta.data_ptr(),
                                           _ptr(granule_margin), float(window), float(tanh_c), B, F, row_off.data_ptr(),
                                           idx.data_ptr(), val.data_ptr(),
                                           win.data_ptr(), total, _ptr(tanh_tok), l0_tok.data_ptr(), _stream(pre)),
              "jumprelu_select_emit")
    return SparseCode(idx, val, row_off, row_nnz, B, F), win, tanh_tok, l0_tok


def feature_segment_sums(fi: FeatureIndex, a: torch.Tensor, b: Optional[torch.Tensor] = None):
    """Per-feature sums of one or two per-slot fp32 arrays over the feature index -> (fp32 [F], fp32 [F] or None)."""
    _req(a, "a", torch.float32, 1)
    F = fi.feat_ptr.numel() - 1
    out_a = torch.empty(F, dtype=torch.float32, device=a.device)
    out_b = None
    if b is not None:
        _req(b, "b", torch.float32, 1)
        out_b = torch.empty(F, dtype=torch.float32, device=a.device)
    with _timed("feature_segment_sums"):
        check(_lib.load().sae_feature_segment_sums(fi.feat_ptr.data_ptr(), fi.feat_slot.data_ptr(), a.data_ptr(), _ptr(b), F,
                                                   out_a.data_ptr(), _ptr(out_b), _stream(a)), "feature_segment_sums")
    return out_a, out_b


def code_stats(code: SparseCode, tok_w: Optional[torch.Tensor] = None, freq_acc: Optional[torch.Tensor] = None,
               totals: Optional[torch.Tensor] = None, want_l0: bool = False) -> Optional[torch.Tensor]:
    """Activation statistics of a sparse code without densifying it: `freq_acc` (float [F]) += per-feature
    count of (masked) tokens with a positive activation; `totals` (double [3]) += (sum of values, number of
    positive values, masked number of positive values); returns the per-token L0 when asked for."""
    _req(code.idx, "code.idx", torch.int32)
    _req(code.val, "code.val", torch.float32)
    if tok_w is not None:
        _req(tok_w, "tok_w", torch.float32, 1)
        if tok_w.numel() != code.n_tokens:
            raise ValueError("tok_w must hold one weight per token")
    if freq_acc is not None:
        _req(freq_acc, "freq_acc", torch.float32, 1)
        if freq_acc.numel() != code.d_sae:
            raise ValueError("freq_acc must hold one entry per feature")
    if totals is not None:
        _req(totals, "totals", torch.float64, 1)
    l0 = torch.empty(code.n_tokens, dtype=torch.float32, device=code.val.device) if want_l0 else None
    with _timed("code_stats"):
        check(
            _lib.load().sae_code_stats(code.idx.data_ptr(), code.val.data_ptr(), code.row_off.data_ptr(), code.row_nnz.data_ptr(),
                                       _ptr(tok_w), code.n_tokens, code.d_sae, _ptr(freq_acc), _ptr(l0), _ptr(totals),
                                       _stream(code.val)),
            "code_stats",
        )
    return l0


def recon_stats(label: torch.Tensor, recon: torch.Tensor, label_mean: torch.Tensor, acc: torch.Tensor,
                tok_w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """acc (double [4]) += this step's (explained variance, legacy explained variance, L2 error, L2 error
    ratio); returns the step's four values (float [4])."""
    _req(label, "label", torch.float32, 2)
    _req(recon, "recon", torch.float32, 2)
    _req(label_mean, "label_mean", torch.float32, 1)
    _req(acc, "acc", torch.float64, 1)
    B, d = label.shape
    if recon.shape != label.shape or label_mean.numel() != d or acc.numel() < 4:
        raise ValueError("shape mismatch")
    if tok_w is not None:
        _req(tok_w, "tok_w", torch.float32, 1)
    ws = torch.empty(3 * B, dtype=torch.float32, device=label.device)
    out = torch.empty(4, dtype=torch.float32, device=label.device)
    with _timed("recon_stats"):
        check(
            _lib.load().sae_recon_stats(label.data_ptr(), recon.data_ptr(), label_mean.data_ptr(), _ptr(tok_w), B, d,
                                        ws.data_ptr(), acc.data_ptr(), out.data_ptr(), _stream(label)),
            "recon_stats",
        )
    return out


# ---- causal attention with grouped value heads ------------------------------------------------------------

ATTENTION_D_QK = (32, 64)
ATTENTION_D_V = (32, 64, 128)


def attention_shapes_supported(seq: int, d_qk: int, d_v: int) -> bool:
    """Whether the attention kernels are built for these head widths and sequence length."""
    return d_qk in ATTENTION_D_QK and d_v in ATTENTION_D_V and seq % 8 == 0


def _att_check(name: str, t: torch.Tensor, shape: tuple) -> None:
    _req(t, name, torch.bfloat16, 2)
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def attention_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, n_batch: int, seq: int, n_heads: int,
                  scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Causal softmax attention: q, k [T, n_heads * d_qk], v [T, n_heads * d_v] (bf16, T = n_batch * seq, a token's heads
    side by side) -> (out [T, n_heads * d_v] bf16, lse fp32 [n_batch, n_heads, seq]).  Projection biases belong in the
    products that form q, k and v (`encoder_gemm_bias`)."""
    T = n_batch * seq
    d_qk, d_v = q.shape[1] // n_heads, v.shape[1] // n_heads
    _att_check("q", q, (T, n_heads * d_qk)); _att_check("k", k, (T, n_heads * d_qk)); _att_check("v", v, (T, n_heads * d_v))
    out = torch.empty(T, n_heads * d_v, dtype=torch.bfloat16, device=q.device)
    lse = torch.empty(n_batch, n_heads, seq, dtype=torch.float32, device=q.device)
    with _timed("attention_fwd"):
        check(_lib.load().sae_attention_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), n_batch, seq, n_heads, d_qk, d_v,
                                            float(scale), out.data_ptr(), lse.data_ptr(), _stream(q)), "attention_fwd")
    return out, lse


def attention_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, dout: torch.Tensor, lse: torch.Tensor,
                  n_batch: int, seq: int, n_heads: int, scale: float, return_stacked: bool = False):
    """Backward of attention_fwd (operands as there, dout like out) -> (dqt, dkt [n_heads * d_qk, T], dvt [n_heads * d_v, T])
    in bf16, TRANSPOSED: the three are row blocks of one buffer [n_heads * (2 d_qk + d_v), T], the left operand of a
    weight-gradient product over the token axis, returned as a fourth value with `return_stacked`."""
    T = n_batch * seq
    d_qk, d_v = q.shape[1] // n_heads, v.shape[1] // n_heads
    for name, t, shape in (("q", q, (T, n_heads * d_qk)), ("k", k, (T, n_heads * d_qk)), ("v", v, (T, n_heads * d_v)),
                           ("out", out, (T, n_heads * d_v)), ("dout", dout, (T, n_heads * d_v))):
        _att_check(name, t, shape)
    _req(lse, "lse", torch.float32, 3)
    if tuple(lse.shape) != (n_batch, n_heads, seq):
        raise ValueError("lse must be [n_batch, n_heads, seq]")
    dev = q.device
    grads = torch.empty(n_heads * (2 * d_qk + d_v), T, dtype=torch.bfloat16, device=dev)
    dqt, dkt, dvt = grads[: n_heads * d_qk], grads[n_heads * d_qk: 2 * n_heads * d_qk], grads[2 * n_heads * d_qk:]
    workspace = torch.empty(2 * n_batch * n_heads * seq, dtype=torch.float32, device=dev)
    with _timed("attention_bwd"):
        check(_lib.load().sae_attention_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr(),
                                            lse.data_ptr(), n_batch, seq, n_heads, d_qk, d_v, float(scale), workspace.data_ptr(),
                                            dqt.data_ptr(), dkt.data_ptr(), dvt.data_ptr(), _stream(q)), "attention_bwd")
    return (dqt, dkt, dvt, grads) if return_stacked else (dqt, dkt, dvt)


def rotary_supported(seq: int, d_head: int, rotary_dim: int, rotary_scale: int = 1) -> bool:
    """Shapes `rotary_fwd` / `rotary_bwd_t` take."""
    return rotary_scale == 1 and seq % 8 == 0 and d_head % 8 == 0 and 0 < rotary_dim <= d_head and rotary_dim % 16 == 0


def rotary_fwd(acc: torch.Tensor, bias: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor, seq: int, n_heads: int,
               rotary_dim: int, adjacent_pairs: bool) -> torch.Tensor:
    """bf16 [T, n_heads d_head] = rotate(float(bf16(acc)) + bias): the projection's fp32 accumulators `acc`, the bias
    and the rotary embedding with tables cos / sin fp32 [n_ctx, rotary_dim]; a token's position is its index in its
    sequence of `seq` tokens."""
    _req(acc, "acc", torch.float32, 2)
    T, width = acc.shape
    for name, t in (("cos", cos), ("sin", sin)):
        _req(t, name, torch.float32, 2)
        if t.shape[1] != rotary_dim or t.shape != cos.shape:
            raise ValueError(f"{name} must be [n_ctx, {rotary_dim}]")
    if bias is not None:
        _req(bias, "bias", torch.float32, 1)
        if bias.numel() != width:
            raise ValueError(f"bias must have {width} elements")
    if width % n_heads:
        raise ValueError("acc's width must be a multiple of n_heads")
    out = torch.empty(T, width, dtype=torch.bfloat16, device=acc.device)
    with _timed("rotary_fwd"):
        check(_lib.load().sae_rotary_fwd(acc.data_ptr(), _ptr(bias), cos.data_ptr(), sin.data_ptr(), cos.shape[0], T, int(seq),
                                         int(n_heads), width // n_heads, int(rotary_dim), int(bool(adjacent_pairs)),
                                         out.data_ptr(), _stream(acc)), "rotary_fwd")
    return out


def rotary_bwd_t(grad_t: torch.Tensor, cos_t: torch.Tensor, sin_t: torch.Tensor, seq: int, n_heads: int, rotary_dim: int,
                 adjacent_pairs: bool) -> None:
    """In place on grad_t bf16 [n_heads d_head, T] (a gradient with respect to rotated queries / keys, transposed): the
    gradient with respect to what was rotated.  cos_t / sin_t: the tables transposed, fp32 [rotary_dim, n_ctx]."""
    _req(grad_t, "grad_t", torch.bfloat16, 2)
    rows, T = grad_t.shape
    for name, t in (("cos_t", cos_t), ("sin_t", sin_t)):
        _req(t, name, torch.float32, 2)
        if t.shape[0] != rotary_dim or t.shape != cos_t.shape:
            raise ValueError(f"{name} must be [{rotary_dim}, n_ctx]")
    if rows % n_heads:
        raise ValueError("grad_t's rows must be a multiple of n_heads")
    with _timed("rotary_bwd_t"):
        check(_lib.load().sae_rotary_bwd_t(grad_t.data_ptr(), cos_t.data_ptr(), sin_t.data_ptr(), cos_t.shape[1], T, int(seq),
                                           int(n_heads), rows // n_heads, int(rotary_dim), int(bool(adjacent_pairs)),
                                           _stream(grad_t)), "rotary_bwd_t")


def row_sum(src: torch.Tensor) -> torch.Tensor:
    """fp32 [rows] = sum over the columns of a bf16 / fp32 matrix [rows, cols]."""
    _req(src, "src", ndim=2)
    r, c = src.shape
    out = torch.empty(r, dtype=torch.float32, device=src.device)
    with _timed("row_sum"):
        check(_lib.load().sae_row_sum(src.data_ptr(), _dt(src), r, c, out.data_ptr(), _stream(src)), "row_sum")
    return out


def mfma_probe(device: torch.device, n_workgroups: int = 4096, iters: int = 4096) -> Tuple[float, float]:
    """Run the register-only MFMA loop (`sae_mfma_probe`) once and return (flop of the launch, milliseconds)."""
    import ctypes

    out = torch.empty(n_workgroups * 256, dtype=torch.float32, device=device)
    flop = ctypes.c_double(0.0)
    lib = _lib.load()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    check(lib.sae_mfma_probe(out.data_ptr(), n_workgroups, iters, ctypes.addressof(flop), _stream(out)), "mfma_probe")
    end.record()
    end.synchronize()
    return flop.value, start.elapsed_time(end)


def gather_rows(src: torch.Tensor, row_idx: torch.Tensor, out_dtype: Optional[torch.dtype] = None, scale: float = 1.0,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[i] = cast(scale * src[row_idx[i]]) for a [N, d] fp32 / bf16 buffer and int64 row indices."""
    _req(src, "src", ndim=2)
    _req(row_idx, "row_idx", torch.int64, 1)
    out_dtype = out_dtype or src.dtype
    n, d = row_idx.numel(), src.shape[1]
    if out is None:
        out = torch.empty(n, d, dtype=out_dtype, device=src.device)
    else:
        _req(out, "out", out_dtype, 2)
        if tuple(out.shape) != (n, d):
            raise ValueError("out has the wrong shape")
    if n == 0:
        return out
    with _timed("gather_rows"):
        check(
            _lib.load().sae_gather_rows(src.data_ptr(), _dt(src), row_idx.data_ptr(), src.shape[0], n, d, out.data_ptr(), _dt(out),
                                        float(scale), _stream(src)),
            "gather_rows",
        )
    return out
