"""The kernel operators of the reference's `kernels` package (src/llamascopium/kernels/__init__.py:1-6,
kernels/entrypoints.py:16-90) on the HIP path: the sparse decoder product a model switches to with
`cfg.use_triton_kernel` once its activations are sparse enough, and the encoder product whose backward goes sparse
when the incoming gradient is.  Same call signatures; the Triton-named entry points are aliases, so code written
against the reference keeps working.

    decode_with_hip_spmm_kernel(feature_acts [.., d_sae], decoder_weight)  -> [.., d_model]
    encode_with_hip_spmm_kernel(x [B, L, d], W_E [L, d, F], b_E [L, F], sparsity_threshold) -> [B, L, F]
    get_sparse_representation(x [B, d_sae]) -> (indices [B, nnz_max] int64, values [B, nnz_max])
"""

from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from . import ops


def _autocast_bf16() -> bool:
    return torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.bfloat16


def get_sparse_representation(x: torch.Tensor, pad_val: int = 0):
    """kernels/kernels.py:14-58: the padded [B, nnz_max] index / value pair of a dense [B, d_sae] tensor (non-zeros of
    each row in ascending column order, `pad_val` / 0 behind them; a batch without non-zeros gives [B, 1] of zeros).
    The kernels here work on the packed sparse code (`ops.dense_to_code`); this form is kept for callers of the
    reference's helper."""
    code = ops.dense_to_code(x.contiguous() if x.dtype in (torch.float32, torch.bfloat16) else x.float().contiguous())
    B = code.n_tokens
    nnz_max = max(int(code.row_nnz.max().item()), 1)
    pos = torch.arange(nnz_max, device=x.device)[None, :]
    valid = pos < code.row_nnz[:, None]
    src = (code.row_off[:, None] + pos).clamp_max(code.n_slots - 1)
    indices = torch.where(valid, code.idx.long()[src], torch.full((B, nnz_max), pad_val, dtype=torch.long, device=x.device))
    values = torch.where(valid, code.val[src], torch.zeros(B, nnz_max, device=x.device)).to(x.dtype)
    return indices, values


class _SparseDecode(torch.autograd.Function):
    """out = feature_acts @ W for a dense feature_acts whose rows are mostly zero: the sparse code of the matrix ->
    gather of the active decoder rows (TritonDecoderAutogradTopK's role, kernels/kernels.py:542-566).  Backward: the
    gradient of the activations at their non-zero positions (zero elsewhere, as the reference masks it), and the decoder
    gradient rows from the feature index of the code.

    `code` addresses the rows of `w_op` (and of `weight`, the tensor the gradient goes to).  When the rows of
    `feature_acts` are decoded by different blocks of `weight` (row r by block r % n_blocks: the heads of a crosscoder),
    `code.idx` carries the block offset and `local_idx` the column inside feature_acts."""

    @staticmethod
    def forward(ctx, feature_acts, weight, w_op, code, local_idx=None):
        ctx.code, ctx.w_op, ctx.local_idx = code, w_op, local_idx
        ctx.n_cols = feature_acts.shape[-1]
        ctx.in_dtype, ctx.w_dtype = feature_acts.dtype, weight.dtype
        return ops.sparse_decode_fwd(code, w_op, None)

    @staticmethod
    def backward(ctx, g):
        code, w_op = ctx.code, ctx.w_op
        g = g.float().contiguous()
        d_acts = d_w = None
        if ctx.needs_input_grad[0]:
            dval = ops.sparse_decode_bwd_dval(code, g, w_op)
            local = code if ctx.local_idx is None else dataclasses.replace(code, idx=ctx.local_idx, d_sae=ctx.n_cols)
            d_acts = ops.code_to_dense(dataclasses.replace(local, val=dval), ctx.n_cols)[0].to(ctx.in_dtype)
        if ctx.needs_input_grad[1]:
            fi = ops.build_feature_index(code)
            d_w = ops.sparse_grad_rows(fi, code.val, g, code.d_sae)[0].to(ctx.w_dtype)
        return d_acts, d_w, None, None, None


def _as_code_source(feature_acts: torch.Tensor) -> torch.Tensor:
    fa = feature_acts if feature_acts.dtype in (torch.float32, torch.bfloat16) else feature_acts.float()
    return fa.contiguous()


def sparse_decode_blocks(feature_acts: torch.Tensor, weight: torch.Tensor, w_operand: torch.Tensor, n_blocks: int = 1,
                         max_density: Optional[float] = None) -> Optional[torch.Tensor]:
    """feature_acts [rows, F] dense, weight / w_operand [n_blocks * F, d] (row r of feature_acts is decoded by block
    r % n_blocks: with n_blocks = 1 a plain `feature_acts @ weight`) -> fp32 [rows, d] through the sparse decoder kernels,
    differentiable in feature_acts and weight.  Returns None when more than `max_density` of the matrix is non-zero (the
    count is read on the host, as the reference's own gate reads `max_l0`, models/sae.py:355-361)."""
    fa = _as_code_source(feature_acts)
    rows, F = fa.shape
    limit = None if max_density is None else int(max_density * rows * F)
    code = ops.dense_to_code(fa, max_entries=limit)
    if code is None:
        return None
    local_idx = None
    if n_blocks > 1:
        slots = torch.arange(code.n_slots, device=fa.device)
        row = (torch.searchsorted(code.row_off, slots, right=True) - 1).clamp_(min=0)
        local_idx = code.idx
        code = dataclasses.replace(code, idx=(code.idx + (row % n_blocks).to(torch.int32) * F), d_sae=n_blocks * F)
    return _SparseDecode.apply(feature_acts, weight, w_operand, code, local_idx)


def decode_with_hip_spmm_kernel(feature_acts: torch.Tensor, decoder_weight: torch.Tensor, *,
                                w_operand: Optional[torch.Tensor] = None, capacity: Optional[int] = None,
                                transposed: Optional[bool] = None) -> torch.Tensor:
    """kernels/entrypoints.py:16-40.  feature_acts [.., d_sae] dense (or a torch sparse COO tensor), decoder_weight
    [d_sae, d_model]; the [d_model, d_sae] tensor the reference's own call site passes (`W_D.T.contiguous()`,
    models/sae.py:363) is read as its transpose: `transposed=True` says so, `transposed=None` tells the two layouts apart
    by shape and raises for a square weight, where the shape cannot tell.  Returns feature_acts @ decoder_weight in fp32.
    `w_operand`: a prepared copy of the weight for the gather (e.g. the bf16 copy under autocast).  `capacity`: an upper
    bound on the number of non-zeros (no read-back; entries past it are dropped)."""
    if feature_acts.is_sparse:
        feature_acts = feature_acts.to_dense()
    F = feature_acts.shape[-1]
    if transposed is None:
        if decoder_weight.ndim == 2 and decoder_weight.shape[0] == decoder_weight.shape[1] == F and w_operand is None:
            raise ValueError(f"decoder_weight is square ({F} x {F}): pass transposed=False for a [d_sae, d_model] weight or "
                             "transposed=True for the [d_model, d_sae] form of the reference's call site")
        transposed = decoder_weight.shape[0] != F and decoder_weight.shape[-1] == F
    if transposed:
        decoder_weight = decoder_weight.t()
    if decoder_weight.shape[0] != F:
        raise ValueError(f"decoder_weight {tuple(decoder_weight.shape)} does not match d_sae = {F}")
    if w_operand is None:
        w = decoder_weight.detach()
        w_operand = w if w.is_contiguous() else w.contiguous()
        if w_operand.dtype not in (torch.float32, torch.bfloat16):
            w_operand = w_operand.float()
    lead = feature_acts.shape[:-1]
    fa2 = feature_acts.reshape(-1, F)
    code = ops.dense_to_code(_as_code_source(fa2), capacity)
    out = _SparseDecode.apply(fa2, decoder_weight, w_operand, code, None)
    return out.view(*lead, out.shape[-1])


class _EncodeLayer(torch.autograd.Function):
    """x @ W_E + b_E on the GEMM kernel; in the backward pass, a gradient that is sparse enough (a TopK-family
    activation passes on only its kept entries) goes through the sparse kernels: d x gathers the active encoder rows,
    d W_E / d b_E come from the feature index of the gradient's code (TritonEncoderAutogradDynamicK,
    kernels/kernels.py:439-539)."""

    @staticmethod
    def forward(ctx, x, W_E, b_E, sparsity_threshold):
        amp = _autocast_bf16()
        wt = W_E.detach().t()
        wt = wt if wt.is_contiguous() else wt.contiguous()                      # [F, d]
        if amp and wt.dtype == torch.float32:
            x_op, w_op, out_dtype = ops.cast_bf16(x.float().contiguous()), ops.cast_bf16(wt), torch.bfloat16
        else:
            x_op, w_op, out_dtype = x.to(wt.dtype).contiguous(), wt, wt.dtype
        pre = ops.encoder_gemm(x_op, w_op, out_dtype)
        ctx.save_for_backward(x_op, w_op)
        ctx.thr, ctx.x_dtype, ctx.w_dtype, ctx.b_dtype = float(sparsity_threshold), x.dtype, W_E.dtype, b_E.dtype
        return pre + b_E

    @staticmethod
    def backward(ctx, g):
        x_op, w_op = ctx.saved_tensors
        g = g.contiguous()
        sparse = (g == 0).float().mean().item() > ctx.thr       # the reference decides on the host as well
        if sparse:
            code = ops.dense_to_code(g if g.dtype in (torch.float32, torch.bfloat16) else g.float())
            fi = ops.build_feature_index(code)
            dx = ops.sparse_decode_fwd(code, w_op, None).to(ctx.x_dtype) if ctx.needs_input_grad[0] else None
            rows, bias = ops.sparse_grad_rows(fi, code.val, x_op, code.d_sae, want_bias=True)
            dW = rows.t().to(ctx.w_dtype) if ctx.needs_input_grad[1] else None
            db = bias.to(ctx.b_dtype) if ctx.needs_input_grad[2] else None
            return dx, dW, db, None
        gg = g.to(w_op.dtype)
        dx = (gg @ w_op).to(ctx.x_dtype) if ctx.needs_input_grad[0] else None
        dW = (gg.t() @ x_op).t().to(ctx.w_dtype) if ctx.needs_input_grad[1] else None
        db = g.float().sum(0).to(ctx.b_dtype) if ctx.needs_input_grad[2] else None
        return dx, dW, db, None


def encode_with_hip_spmm_kernel(x: torch.Tensor, W_E: torch.Tensor, b_E: torch.Tensor,
                                sparsity_threshold: float = 0.996) -> torch.Tensor:
    """kernels/entrypoints.py:43-90: "bld,lds->bls" layer by layer, + b_E."""
    B, L, _ = x.shape
    return torch.stack([_EncodeLayer.apply(x[:, l, :], W_E[l], b_E[l], sparsity_threshold) for l in range(L)], dim=1)


# the reference's names
decode_with_triton_spmm_kernel = decode_with_hip_spmm_kernel
encode_with_triton_spmm_kernel = encode_with_hip_spmm_kernel
