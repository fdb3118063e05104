"""SparseAutoEncoder on the HIP path.

API of the reference's vanilla SAE / transcoder (src/llamascopium/models/sae.py:52-448):
parameters `W_E [d, F]`, `b_E [F]`, `W_D [F, d]`, `b_D [d]` (plus the optional GLU pair), methods
`encode`, `decode`, `forward`, `compute_loss`, the norm helpers and `init_parameters`.

Memory layout: `W_E` has the reference's shape [d_model, d_sae] but is stored feature-major
(strides (1, d_model), i.e. a transposed view of a contiguous [d_sae, d_model] buffer).  One
feature's encoder vector is then contiguous, like its decoder vector, which is what the GEMM
(K-contiguous operands), the sparse gradient rows and the fused optimiser want.

`compute_loss` takes the fused kernel path when the configuration allows it (TopK activation,
reconstruction loss only, no user hooks, 2-D activations on the GPU); every other configuration
runs the reference's op sequence over dense tensors with the select kernel behind the activation.
"""

from __future__ import annotations

import math
from typing import Any, Optional

import torch
from torch import nn

from . import ops
from .config import SAEConfig, register_sae_model
from .hooks import HookPoint
from .sparse_dictionary import LazyDict, SparseDictionary


def _autocast_dtype(device_type: str) -> Optional[torch.dtype]:
    if torch.is_autocast_enabled(device_type):
        return torch.get_autocast_dtype(device_type)
    return None


class _Holder:
    """Side outputs of the fused step that are not autograd tensors."""

    code: ops.SparseCode = None
    pre: torch.Tensor = None
    scale: Optional[torch.Tensor] = None
    defer_to: Optional["SparseAutoEncoder"] = None  # module whose optimiser consumes factored weight gradients
    model: Optional["SparseAutoEncoder"] = None
    aux: Optional[dict] = None      # aux-k request: {"is_dead": callable(code) -> bool [F], "k_aux": int, "coefficient": float}
    aux_code: ops.SparseCode = None
    l_aux: Optional[torch.Tensor] = None


class SparseRowGrad:
    """Gradient of a feature-major [F, d] weight in factored form:
    g[f, :] = sum over feature f's slots of coef[slot] * dense[token(slot), :].
    Produced by the fused backward when the optimiser can consume it directly (HipAdam), so the
    dense gradient never has to be written to HBM.  `dense()` materialises it on demand."""

    def __init__(self, fi: ops.FeatureIndex, coef: torch.Tensor, dense_operand: torch.Tensor, n_features: int,
                 bias_param: Optional[torch.Tensor] = None, extra: Optional[ops.DenseRowBlock] = None):
        self.fi, self.coef, self.dense_operand, self.n_features, self.bias_param = fi, coef, dense_operand, n_features, bias_param
        self.extra = extra    # gradient rows held densely for some features (added to the factored part)
        self.scale: Optional[torch.Tensor] = None    # device float[1] from gradient clipping, applied where rows are formed
        self.sq_nnz: Optional[torch.Tensor] = None   # cached (sum g^2, #non-zero) of the unscaled rows

    def dense(self, want_bias: Optional[bool] = None):
        """(rows [F, d] fp32, bias gradient [F] or None)"""
        rows, bias = ops.sparse_grad_rows(self.fi, self.coef, self.dense_operand, self.n_features,
                                          want_bias=self.bias_param is not None if want_bias is None else want_bias)
        if self.extra is not None:
            hit = self.extra.row_map >= 0
            src = self.extra.row_map.clamp_min(0).long()
            rows += torch.where(hit[:, None], self.extra.rows.index_select(0, src), torch.zeros_like(rows))
            if bias is not None and self.extra.bias is not None:
                bias += torch.where(hit, self.extra.bias.index_select(0, src), torch.zeros_like(bias))
        if self.scale is not None:
            rows.mul_(self.scale)
            if bias is not None:
                bias.mul_(self.scale)
        return rows, bias


class SparseRowGradPieces:
    """Factored gradient of a weight whose contiguous [rows, d] view splits into row blocks with separate
    feature indices or dense operands (the L encoder layers of a cross-layer transcoder): `pieces` is a list
    of (first_row, SparseRowGrad).  Rows outside every piece have zero gradient.  `bias_param` (optional) is
    the per-row bias whose gradient the pieces carry (flat index = row)."""

    def __init__(self, pieces, n_rows: int, bias_param: Optional[torch.Tensor] = None):
        self.pieces, self.n_rows, self.bias_param = list(pieces), int(n_rows), bias_param

    def dense(self):
        """(rows [n_rows, d] fp32, bias gradient [n_rows] or None)"""
        first = self.pieces[0][1]
        d = first.dense_operand.shape[1]
        rows = torch.zeros(self.n_rows, d, dtype=torch.float32, device=first.coef.device)
        bias = torch.zeros(self.n_rows, dtype=torch.float32, device=first.coef.device) if self.bias_param is not None else None
        for r0, sg in self.pieces:
            want = bias is not None
            part, b = ops.sparse_grad_rows(sg.fi, sg.coef, sg.dense_operand, sg.n_features, want_bias=want)
            if sg.scale is not None:
                part.mul_(sg.scale)
                if b is not None:
                    b.mul_(sg.scale)
            rows[r0:r0 + sg.n_features] = part
            if b is not None:
                bias[r0:r0 + sg.n_features] = b
        return rows, bias


class _DeadCount:
    """#dead on its way to the host: the count and its copy into pinned memory are enqueued when this is made, and
    `value()` waits for the copy only.  Kernels enqueued in between keep the GPU busy while the host waits and then
    prepares the launches that depend on the count."""

    def __init__(self, dead: torch.Tensor):
        self.host = torch.empty(1, dtype=torch.int64, pin_memory=True)
        self.host.copy_(dead.sum().reshape(1), non_blocking=True)
        self.event = torch.cuda.Event()
        self.event.record()

    def value(self) -> int:
        self.event.synchronize()
        return int(self.host[0])


def _aux_block_fits(B: int, d: int, amp: bool) -> bool:
    gran = 64 if amp else 32
    return B % gran == 0 and d % gran == 0


def _aux_dense_block(x_op, pre_dtype, w_enc_op, w_dec_op, b_E, scale, dead, k_aux: int, batch_wide: bool, amp: bool,
                     n_dead: Optional[int] = None, lowp: bool = False):
    """Forward half of the aux-k term on a compacted dead block.  Gathers the dead features' encoder / decoder
    rows into [n, d] matrices (n = #dead padded to the GEMM's K granule), recomputes their pre-activations with
    the encoder GEMM (same kernel, same accumulation order as the full product: identical values), selects among
    them, scatters the kept values into a dense [B, n] matrix and decodes it with one more GEMM.
    Returns None when the shapes do not fit the GEMM kernel or the block is too wide to pay; sizing the block
    needs #dead on the host (one synchronisation per step, as the reference's `int(is_dead.sum().item())`; `n_dead`
    hands in a count the caller already fetched)."""
    B, d = x_op.shape
    F = dead.numel()
    gran = 64 if amp else 32
    if not _aux_block_fits(B, d, amp):
        return None
    if n_dead is None:
        dead_idx = torch.nonzero(dead).squeeze(1)
        nd = int(dead_idx.numel())
    else:
        nd = int(n_dead)
        # ascending indices of the dead features without another wait: each takes the place its rank gives it
        rank = torch.cumsum(dead, 0) - 1
        dead_idx = torch.empty(nd + 1, dtype=torch.int64, device=dead.device)
        dead_idx.scatter_(0, torch.where(dead, rank, torch.full_like(rank, nd)), torch.arange(F, device=dead.device))
        dead_idx = dead_idx[:nd]
    if nd == 0:
        return {"n_dead": 0, "code": None}
    if nd > 64 * max(k_aux, 1) or B * (nd + gran) >= 2 ** 31:
        return None
    ndp = (nd + gran - 1) // gran * gran
    dev = x_op.device

    def rows_of(w):   # [nd, d] gathered, zero rows up to ndp
        out = torch.zeros(ndp, d, dtype=w.dtype, device=dev)
        out[:nd] = w.index_select(0, dead_idx)
        return out

    W_Et, W_D = rows_of(w_enc_op), rows_of(w_dec_op)
    b_d = torch.zeros(ndp, dtype=torch.float32, device=dev)
    b_d[:nd] = b_E.detach().float().index_select(0, dead_idx)
    s_d = None
    if scale is not None:
        s_d = torch.ones(ndp, dtype=torch.float32, device=dev)
        s_d[:nd] = scale.index_select(0, dead_idx)
    pre_d = ops.encoder_gemm(x_op, W_Et, pre_dtype)                                   # [B, ndp]
    kk = min(k_aux, nd)
    # with a norm scale the keys are `hidden_pre * is_dead * decoder_norm` op for op, hidden_pre being the quotient the
    # encoder returned (models/sparse_dictionary.py:958-966): the select's masked arithmetic with every block column in
    # (`lowp`: a dictionary held in bf16, whose tensors around the select are bf16)
    keep = torch.ones(ndp, dtype=torch.float32, device=dev) if s_d is not None else None
    code_d = (ops.select_topk_batch(pre_d, b_d, s_d, kk * B, feat_mask=keep, lowp=lowp) if batch_wide
              else ops.select_topk_row(pre_d, b_d, s_d, kk, feat_mask=keep, lowp=lowp))
    # dense [B, ndp] activations of the block: fp32 (the mask of the backward pass) and, under autocast, bf16
    A, A_b16 = ops.code_to_dense(code_d, ndp, want_f32=True, want_bf16=amp)
    A_op = A_b16 if amp else A
    # [B, d] = A @ W_D[dead]: bf16 operands read the gathered decoder rows as they lie
    aux_recon = (ops.gemm(A_op, W_D, torch.float32, b_k_major=True) if amp
                 else ops.encoder_gemm(A_op, W_D.t().contiguous(), torch.float32))
    # the same code with the dictionary's own feature ids (for callers that look at it); slots past the last
    # token's end are unused and keep index 0
    n_used = code_d.row_off[-1] + code_d.row_nnz[-1]
    valid = torch.arange(code_d.n_slots, device=dev) < n_used
    idx_full = torch.where(valid, dead_idx.index_select(0, code_d.idx.long().clamp_max(nd - 1)).to(torch.int32),
                           torch.zeros_like(code_d.idx))
    import dataclasses
    code_full = dataclasses.replace(code_d, idx=idx_full, d_sae=F)
    row_map = torch.full((F,), -1, dtype=torch.int32, device=dev)
    row_map[dead_idx] = torch.arange(nd, dtype=torch.int32, device=dev)
    return {"n_dead": nd, "ndp": ndp, "W_Et": W_Et, "W_D": W_D, "A": A, "A_op": A_op, "aux_recon": aux_recon,
            "code": code_full, "row_map": row_map}


def _code_slot_tokens(code: ops.SparseCode):
    """(token of every slot, whether the slot is in use) for a sparse code."""
    slots = torch.arange(code.n_slots, device=code.val.device)
    tok = torch.searchsorted(code.row_off, slots, right=True) - 1
    valid = (slots - code.row_off[tok]) < code.row_nnz[tok]
    return tok, valid


def _aux_dense_grads(blk, g_aux, x_op, amp: bool):
    """Backward half: with G = d loss / d aux_recon [B, d] and A the block's activations [B, n],
    d A = G W_D[dead]^T masked to the kept entries (the decoder-norm scale cancels as in the main path),
    dW_D[dead] = A^T G, dW_E^T[dead] = dA^T x, db_E[dead] = column sums of dA: three GEMMs with K = d, B, B."""
    nd = blk["n_dead"]
    A, A_op = blk["A"], blk["A_op"]
    g_aux = g_aux.contiguous()
    if amp:
        # bf16 operands
        G_op = ops.cast_bf16(g_aux)
        dA = ops.encoder_gemm(G_op, blk["W_D"], torch.float32)                         # [B, ndp]
        dpre_T, db_E = ops.transpose_to_bf16(dA, mask=A, col_sums=True)                 # d pre = dA where A > 0
        # the two products over the token axis read A, G and x as they lie (stored [tokens, .]); d pre arrives transposed
        # from the pass that masks it and sums its columns
        dW_D = ops.gemm(A_op, G_op, torch.float32, a_k_major=True, b_k_major=True)                                # [ndp, d]
        dW_Et = ops.gemm(dpre_T, x_op, torch.float32, b_k_major=True)                                              # [ndp, d]
        dpre = None   # formed on demand (only the gradient with respect to x wants it in this layout)
    else:
        dA = ops.encoder_gemm(g_aux, blk["W_D"], torch.float32)
        dpre = torch.where(A > 0, dA, torch.zeros_like(dA))
        dW_D = ops.encoder_gemm(A_op.t().contiguous(), g_aux.t().contiguous(), torch.float32)
        dW_Et = ops.encoder_gemm(dpre.t().contiguous(), x_op.t().contiguous(), torch.float32)
        db_E = ops.col_sum(dpre)
    return {"row_map": blk["row_map"], "dW_D": dW_D[:nd].contiguous(), "dW_Et": dW_Et[:nd].contiguous(),
            "db_E": db_E[:nd].contiguous(), "dpre": dpre, "dA": dA, "A": A, "W_Et": blk["W_Et"]}


class _FusedSparseStep(torch.autograd.Function):
    """encode -> TopK / BatchTopK -> decode -> masked-mean squared error (+ aux-k), forward and backward,
    in kernels.

    forward : GEMM, select (bias + norm scale fused), decode + loss + grad_recon + d val
    backward: feature index, dW_D / dW_E^T rows (or their factored form), db_E, db_D; no dense [B, F]
              tensor is formed.
    The decoder-norm scale enters as act(h * n) / n; its two derivative terms with respect to n cancel
    analytically, so no gradient flows to W_D through n.

    aux-k (models/sparse_dictionary.py:940-991): a second select restricted to dead features, decoded
    without bias; l_aux = alpha * mean_b |(label - recon) - aux_recon|^2 with the residual carrying
    gradient.  The two codes are stacked into one code over 2B virtual tokens so that a single feature
    index serves both gradients.
    """

    @staticmethod
    def forward(ctx, x, label, tok_w, W_E, b_E, W_D, b_D, k, amp, holder):
        sae = holder.model
        # a dictionary held in bf16 (cfg.dtype = bfloat16): the weights are their own bf16 operands, and the bias
        # sum, norm product and quotient around the select are bf16 tensors in the reference
        lowp = W_E.dtype == torch.bfloat16
        amp = amp or lowp
        w_enc_op = sae._w_enc_operand(amp)
        if lowp:
            b_E = b_E.float()
            b_D = b_D.float() if b_D is not None else None
        B = x.shape[0]
        batch_wide = sae.cfg.act_fn.lower() == "batchtopk"
        # TopK / BatchTopK on bf16 operands: the GEMM's epilogue leaves the largest select key of every 64-feature granule;
        # the per-token select then reads a row only in the granules that can hold a kept element, and the batch-wide
        # select is spared its one pass over the whole matrix.  The keys need the decoder
        # norms, so this route fetches them before the GEMM (and waits there for an overlapped decoder update).
        granule = (amp and getattr(sae, "granule_select", True) and not sae._update_pending()
                   and (ops.granule_route_supported(x.shape[1], w_enc_op.shape[0], int(k)) if not batch_wide
                        else x.shape[1] % 64 == 0 and w_enc_op.shape[0] % 256 == 0))
        gmax = None
        if granule:
            x_op = x if x.dtype == torch.bfloat16 else ops.cast_bf16(x.contiguous())
            scale = sae._decoder_norm_nograd() if sae.cfg.sparsity_include_decoder_norm else None
            if lowp and scale is not None:
                scale = scale.bfloat16().float()   # decoder_norm() of bf16 weights is a bf16 tensor
            pre, gmax = ops.encoder_gemm_granule_max(x_op, w_enc_op, b_E, scale, lowp=lowp)
        elif amp:
            x_op = x if x.dtype == torch.bfloat16 else ops.cast_bf16(x.contiguous())
            pre = ops.encoder_gemm(x_op, w_enc_op, torch.bfloat16)
        else:
            x_op = x.contiguous()
            pre = ops.encoder_gemm(x_op, w_enc_op, torch.float32)
        if not granule:
            # decoder-side operands are fetched after the GEMM is enqueued: an overlapped decoder update of the
            # previous step (see HipAdam) is waited for here, not before the GEMM
            scale = sae._decoder_norm_nograd() if sae.cfg.sparsity_include_decoder_norm else None
            if lowp and scale is not None:
                scale = scale.bfloat16().float()   # decoder_norm() of bf16 weights is a bf16 tensor
        w_dec_op = sae._w_dec_operand(amp)
        if batch_wide:
            code = ops.select_topk_batch(pre, b_E, scale, k * B, granule_max=gmax, lowp=lowp)
        else:
            code = ops.select_topk_row(pre, b_E, scale, k, lowp=lowp, granule_max=gmax)
        aux = holder.aux
        grad_recon_b16 = None   # set by the route that already has grad_recon in bf16
        if aux is None:
            recon, loss_tok, grad_recon, dval = ops.sparse_decode_mse_fused(code, w_dec_op, b_D, label, tok_w)
            loss = loss_tok.sum()
            l_aux = None
            grad_code, grad_dense_D, grad_coef_E, x_rows = code, grad_recon, dval, x_op
            ctx.aux_dense = None
        else:
            dead = aux["is_dead"](code)                       # bool [F], from the caller's dead statistics
            k_aux = int(aux["k_aux"])
            ctx.aux_dense = None
            dense_block = None
            recon = None
            if aux.get("dense", True) and _aux_block_fits(x_op.shape[0], x_op.shape[1], amp):
                # the block is sized by #dead: the count is fetched while the main decode, which does not depend on
                # it, runs
                count = _DeadCount(dead)
                recon = ops.sparse_decode_fwd(code, w_dec_op, b_D)
                dense_block = _aux_dense_block(x_op, pre.dtype, w_enc_op, w_dec_op, b_E, scale, dead, k_aux, batch_wide, amp,
                                               n_dead=count.value(), lowp=lowp)
            sae._last_aux_route = "dense" if dense_block is not None else "sparse"
            if dense_block is not None:
                # The dead block is small and hit by a large share of the tokens: its part of the step is three small
                # GEMMs on a compacted [n_dead, d] copy of the two weight blocks instead of gathers per (token, feature).
                blk = dense_block
                alpha = float(aux["coefficient"])
                # squared error, aux-k residual (the residual is not detached), d loss / d aux_recon and d loss / d recon
                rec_tok, aux_tok, g_aux, grad_recon, grad_recon_b16 = ops.mse_auxk_fused(
                    recon, label, blk["aux_recon"] if blk["n_dead"] else None, tok_w, alpha, want_bf16=amp)
                l_rec = rec_tok.sum()
                l_aux = alpha * aux_tok.sum() if aux_tok is not None else torch.zeros_like(l_rec)
                loss = l_rec + l_aux
                dval = ops.sparse_decode_bwd_dval(code, grad_recon, w_dec_op)
                if g_aux is not None:
                    ctx.aux_dense = _aux_dense_grads(blk, g_aux, x_op, amp)
                grad_code, grad_dense_D, grad_coef_E, x_rows = code, grad_recon, dval, x_op
                holder.aux_code = blk["code"]
            else:
                dead_f = dead.to(torch.float32)
                n_dead = dead.sum()
                if batch_wide:
                    k_dev = (torch.clamp(n_dead, max=k_aux) * B).to(torch.int64)
                    aux_code = ops.select_topk_batch(pre, b_E, scale, k_dev, feat_mask=dead_f, capacity=k_aux * B, lowp=lowp)
                else:
                    # min(k_aux, #dead) needs no host value: at most #dead entries can be positive
                    aux_code = ops.select_topk_row(pre, b_E, scale, min(k_aux, pre.shape[1]), feat_mask=dead_f, lowp=lowp)
                if recon is None:
                    recon = ops.sparse_decode_fwd(code, w_dec_op, b_D)
                aux_recon = ops.sparse_decode_fwd(aux_code, w_dec_op, None)
                has_dead = (n_dead > 0).to(torch.float32)
                w = tok_w[:, None]
                diff = recon - label
                r = (label - recon) - aux_recon
                alpha = float(aux["coefficient"]) * has_dead
                l_rec = (w * diff * diff).sum()
                l_aux = alpha * (w * r * r).sum()
                loss = l_rec + l_aux
                g_aux = (-2.0 * alpha) * w * r                     # d loss / d aux_recon
                grad_recon = 2.0 * w * diff + g_aux                # d loss / d recon (the residual is not detached)
                dval = ops.sparse_decode_bwd_dval(code, grad_recon, w_dec_op)
                dval_aux = ops.sparse_decode_bwd_dval(aux_code, g_aux, w_dec_op)
                grad_code = ops.stack_codes(code, aux_code)
                grad_dense_D = torch.cat([grad_recon, g_aux])
                grad_coef_E = torch.cat([dval, dval_aux])
                x_rows = torch.cat([x_op, x_op])
                holder.aux_code = aux_code
        if amp:
            # the decoder's weight gradient pairs the activations with the bf16-rounded output gradient, as the
            # backward of an autocast matmul does; the gather of those rows then moves half the bytes
            grad_dense_D = grad_recon_b16 if grad_recon_b16 is not None else ops.cast_bf16(grad_dense_D.contiguous())
        holder.code, holder.pre, holder.scale, holder.l_aux = code, pre, scale, l_aux
        ctx.grad_code, ctx.x_rows, ctx.grad_dense_D, ctx.grad_coef_E = grad_code, x_rows, grad_dense_D, grad_coef_E
        ctx.grad_recon = grad_recon
        ctx.n_tokens = B
        ctx.w_enc_op = w_enc_op
        ctx.has_b_D = b_D is not None
        ctx.param_dtype = W_E.dtype
        ctx.defer_to = holder.defer_to
        ctx.mark_non_differentiable(recon)
        ctx.set_materialize_grads(False)   # no [B, d] tensor of zeros for the output that carries no gradient
        return loss, recon

    @staticmethod
    def backward(ctx, g_loss, _g_recon):
        if g_loss is None:
            return (None,) * 10
        code = ctx.grad_code
        F = code.d_sae
        fi = ops.build_feature_index(code)
        g = g_loss.to(torch.float32)
        coef_dec = code.val * g          # dW_D[f] = sum val * grad_recon[token]
        coef_enc = ctx.grad_coef_E * g   # dW_E^T[f] = sum d(pre) * x[token]; kept entries are positive, so d(pre) = d val
        db_D = None
        if ctx.has_b_D:
            # a bf16 dictionary's reconstruction is a bf16 tensor, so the gradient summed for b_D is the bf16-rounded one
            # (of the tokens themselves: a stacked aux-k code appends the aux reconstruction's gradient, which has no bias)
            gr = ctx.grad_recon if ctx.param_dtype == torch.float32 else ctx.grad_dense_D[: ctx.n_tokens].float()
            db_D = ops.col_sum(gr) * g
        extra_D = extra_E = None
        ad = ctx.aux_dense
        if ad is not None:   # the dead block's rows, held densely
            extra_D = ops.DenseRowBlock(ad["row_map"], ad["dW_D"] * g, None)
            extra_E = ops.DenseRowBlock(ad["row_map"], ad["dW_Et"] * g, ad["db_E"] * g)
        sae = ctx.defer_to
        if sae is not None and getattr(sae.W_D, "_sparse_grad", None) is None and sae.W_D.grad is None \
                and getattr(sae.W_E, "_sparse_grad", None) is None and sae.W_E.grad is None:
            # hand the factored gradients to the optimiser; b_E's gradient is a by-product of its W_E pass
            sae.W_D._sparse_grad = SparseRowGrad(fi, coef_dec, ctx.grad_dense_D, F, extra=extra_D)
            sae.W_E._sparse_grad = SparseRowGrad(fi, coef_enc, ctx.x_rows, F, bias_param=sae.b_E, extra=extra_E)
            dW_D = dW_Et = db_E = None
        else:
            if sae is not None:  # a second backward before the optimiser ran: fall back to dense accumulation
                for prm in (sae.W_D, sae.W_E):
                    sg = getattr(prm, "_sparse_grad", None)
                    if sg is not None:
                        rows, bias = sg.dense()
                        rows = rows.to(prm.dtype)
                        prm.grad = rows if prm is sae.W_D else rows.t()
                        if bias is not None:
                            bias = bias.to(sg.bias_param.dtype)
                            sg.bias_param.grad = bias if sg.bias_param.grad is None else sg.bias_param.grad + bias
                        prm._sparse_grad = None
            dW_D, _ = SparseRowGrad(fi, coef_dec, ctx.grad_dense_D, F, extra=extra_D).dense()
            dW_Et, db_E = SparseRowGrad(fi, coef_enc, ctx.x_rows, F, extra=extra_E).dense(want_bias=True)
        dx = None
        if ctx.needs_input_grad[0]:
            import dataclasses
            dx = ops.sparse_decode_fwd(dataclasses.replace(code, val=coef_enc), ctx.w_enc_op, None)
            if dx.shape[0] != ctx.n_tokens:  # stacked code: fold the aux half back onto its tokens
                dx = dx[: ctx.n_tokens] + dx[ctx.n_tokens:]
            if ad is not None:
                dpre = ad["dpre"] if ad["dpre"] is not None else torch.where(ad["A"] > 0, ad["dA"], torch.zeros_like(ad["dA"]))
                dx = dx + (dpre.to(ad["W_Et"].dtype) @ ad["W_Et"]).to(torch.float32) * g
        dlabel = None
        if ctx.needs_input_grad[1]:
            dlabel = -ctx.grad_recon * g
        pd = ctx.param_dtype
        if pd != torch.float32:   # gradients of bf16 parameters are bf16 tensors
            dW_Et, db_E, dW_D, db_D = (None if t is None else t.to(pd) for t in (dW_Et, db_E, dW_D, db_D))
        return dx, dlabel, None, None if dW_Et is None else dW_Et.t(), db_E, dW_D, db_D, None, None, None


class _GluSparseStep(torch.autograd.Function):
    """The TopK / BatchTopK step of a dictionary with a gated encoder (models/sae.py:326-331:
    hidden_pre = (x W_E + b_E) * sigmoid(x W_E_glu + b_E_glu)): both encoder products on the GEMM kernel, the gate as
    element-wise ops, then select, fused decode + loss and gradient rows as in the plain step.  Only kept entries carry a
    gradient, so both encoders' weight gradients are gathered rows of x with one coefficient per kept entry:
    d pre = d val * gate for W_E and d val * (x W_E + b_E) * gate * (1 - gate) for W_E_glu; no dense [B, F] gradient and
    no dense backward product is formed."""

    @staticmethod
    def forward(ctx, x, label, tok_w, W_E, b_E, W_G, b_G, W_D, b_D, k, amp, holder):
        sae = holder.model
        w_enc_op, w_glu_op = sae._w_enc_operand(amp), sae._w_glu_operand(amp)
        x_op = (x if x.dtype == torch.bfloat16 else ops.cast_bf16(x.contiguous())) if amp else x.contiguous()
        out_dtype = torch.bfloat16 if amp else torch.float32
        pre, pre_g = ops.encoder_gemm(x_op, w_enc_op, out_dtype), ops.encoder_gemm(x_op, w_glu_op, out_dtype)
        lin = pre.float() + b_E
        gate = torch.sigmoid(pre_g.float() + b_G)
        hidden = lin * gate                                                        # [B, F] fp32, as the reference holds it
        scale = sae._decoder_norm_nograd() if sae.cfg.sparsity_include_decoder_norm else None
        B = x.shape[0]
        if sae.cfg.act_fn.lower() == "batchtopk":
            code = ops.select_topk_batch(hidden, None, scale, k * B)
        else:
            code = ops.select_topk_row(hidden, None, scale, k)
        recon, loss_tok, grad_recon, dval = ops.sparse_decode_mse_fused(code, sae._w_dec_operand(amp), b_D, label, tok_w)
        tok, valid = _code_slot_tokens(code)
        cell = torch.where(valid, tok * hidden.shape[1] + code.idx.long(), torch.zeros_like(tok))
        zero = torch.zeros((), dtype=torch.float32, device=x.device)
        ctx.lin = torch.where(valid, lin.flatten()[cell], zero)                    # per kept entry
        ctx.gate = torch.where(valid, gate.flatten()[cell], zero)
        ctx.code, ctx.x_op, ctx.grad_recon, ctx.dval, ctx.w_enc_op, ctx.w_glu_op = code, x_op, grad_recon, dval, w_enc_op, w_glu_op
        ctx.amp, ctx.has_b_D = bool(amp), b_D is not None
        holder.code, holder.hidden, holder.scale = code, hidden, scale
        ctx.mark_non_differentiable(recon)
        ctx.set_materialize_grads(False)
        return loss_tok.sum(), recon

    @staticmethod
    def backward(ctx, g_loss, _g_recon):
        if g_loss is None:
            return (None,) * 12
        code = ctx.code
        F = code.d_sae
        g = g_loss.to(torch.float32)
        fi = ops.build_feature_index(code)
        # under autocast the decoder's weight gradient pairs the activations with the bf16-rounded output gradient
        gd = ops.cast_bf16(ctx.grad_recon.contiguous()) if ctx.amp else ctx.grad_recon
        dW_D, _ = ops.sparse_grad_rows(fi, code.val * g, gd, F)
        d_hidden = ctx.dval * g                     # kept entries are positive and the norm's two terms cancel
        c_enc, c_glu = d_hidden * ctx.gate, d_hidden * ctx.lin * ctx.gate * (1.0 - ctx.gate)
        dW_Et, db_E = ops.sparse_grad_rows(fi, c_enc, ctx.x_op, F, want_bias=True)
        dW_Gt, db_G = ops.sparse_grad_rows(fi, c_glu, ctx.x_op, F, want_bias=True)
        db_D = ops.col_sum(ctx.grad_recon) * g if ctx.has_b_D else None
        dx = None
        if ctx.needs_input_grad[0]:
            import dataclasses
            dx = (ops.sparse_decode_fwd(dataclasses.replace(code, val=c_enc), ctx.w_enc_op, None)
                  + ops.sparse_decode_fwd(dataclasses.replace(code, val=c_glu), ctx.w_glu_op, None))
        dlabel = -ctx.grad_recon * g if ctx.needs_input_grad[1] else None
        return dx, dlabel, None, dW_Et.t(), db_E, dW_Gt.t(), db_G, dW_D, db_D, None, None, None


def _transposed(t: torch.Tensor) -> torch.Tensor:
    """[r, c] -> contiguous [c, r] in the same dtype (bf16 or fp32) through the transpose kernels."""
    t = t.contiguous()
    return ops.transpose_to_bf16(t)[0] if t.dtype == torch.bfloat16 else ops.transpose(t)


def _gemm_k_ok(k: int, dtype: torch.dtype) -> bool:
    """Whether the GEMM kernel takes a contraction of length k for this operand dtype."""
    return k % (64 if dtype == torch.bfloat16 else 32) == 0


def _rows_over_tokens(left: torch.Tensor, right: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """left^T @ right for left [B, m], right [B, n] -> [m, n]: a product over the token axis (a weight gradient).  bf16
    operands are read as they lie (both are stored [K, rows] for this product); fp32 operands are transposed first, for
    the fp32 kernel contracts over the contiguous axis of both."""
    if (left.dtype == torch.bfloat16 and right.dtype == torch.bfloat16 and left.shape[0] % 64 == 0 and left.shape[1] % 8 == 0
            and right.shape[1] % 8 == 0):
        return ops.gemm(left.contiguous(), right.contiguous(), out_dtype, a_k_major=True, b_k_major=True)
    if _gemm_k_ok(left.shape[0], left.dtype):
        return ops.encoder_gemm(_transposed(left), _transposed(right), out_dtype)
    return (left.t() @ right).to(out_dtype)       # a token count the kernel's K granule does not divide


class _EncoderGemm(torch.autograd.Function):
    """pre = x @ W_E through the GEMM kernel, for activations whose output is dense (JumpReLU): the incoming
    gradient is then dense as well, and the weight gradient d(pre)^T x is a product over the token axis on the same
    kernel."""

    @staticmethod
    def forward(ctx, x, W_E, w_op, amp, defer=False, given=None, grad_view=None):
        # grad_view: maps the gradient rows [F, K] (K = x's width) to the parameter's shape, for encoder weights that
        # are not a [d, F] view of a [F, d] buffer (a crosscoder's [H, d, F] over [F, H, d])
        if given is not None:             # (x operand, product) computed by the caller already
            x_op, pre = given
        elif amp:
            x_op = x if x.dtype == torch.bfloat16 else ops.cast_bf16(x.float().contiguous())
            pre = ops.encoder_gemm(x_op, w_op, torch.bfloat16)
        else:
            x_op = x.float().contiguous()
            pre = ops.encoder_gemm(x_op, w_op, torch.float32)
        ctx.save_for_backward(x_op, w_op)
        ctx.x_dtype, ctx.w_dtype = x.dtype, W_E.dtype
        # a bf16 weight gradient can stay bf16 until the optimiser reads it, when the parameter is stored feature-major
        ctx.param = W_E if (defer and amp and W_E.ndim == 2 and W_E.stride() == (1, W_E.shape[0])) else None
        ctx.grad_view = grad_view
        return pre

    @staticmethod
    def backward(ctx, g):
        x_op, w_op = ctx.saved_tensors
        gg = g.to(w_op.dtype)
        # the input's gradient is rarely wanted (activations carry none in training): a library product
        dx = (gg @ w_op).to(ctx.x_dtype) if ctx.needs_input_grad[0] else None
        dW = None
        if ctx.needs_input_grad[1]:
            rows = _rows_over_tokens(gg, x_op, w_op.dtype)                         # [F, d]
            if ctx.param is not None:
                _leave_lowp_grad(ctx.param, rows)
            elif ctx.grad_view is not None:
                dW = ctx.grad_view(rows).to(ctx.w_dtype)
            else:
                dW = rows.t().to(ctx.w_dtype)                                      # [d, F] with feature-major strides
        return dx, dW, None, None, None, None, None


def _leave_lowp_grad(param, rows: torch.Tensor) -> None:
    """Leave a bf16 weight gradient ([rows, d] over the parameter's storage) on the parameter for HipAdam, which
    widens it as its kernel reads it, instead of returning an fp32 copy to autograd."""
    prev = getattr(param, "_lowp_grad", None)
    param._lowp_grad = rows if prev is None else prev + rows


class _RowNormDeferred(torch.autograd.Function):
    """n[f] = ||W[f, :]||_2 with the value taken from the cache the optimiser keeps.  Its gradient,
    d W[f, :] = (d n_f / n_f) W[f, :] (what `torch.norm(W, dim=1)` sends back), is a per-row multiple of W: when
    `owner` is given it is left on the parameter as `_row_grad_coef` for HipAdam, which applies it inside its
    update kernel, instead of being formed as a dense [F, d] tensor and added to the other gradient."""

    @staticmethod
    def forward(ctx, W, n_value, owner):
        ctx.save_for_backward(n_value)
        ctx.param, ctx.owner = W, owner
        return n_value.clone()

    @staticmethod
    def backward(ctx, g_n):
        (n,) = ctx.saved_tensors
        W = ctx.param
        coef = torch.where(n > 0, g_n.to(torch.float32) / n, torch.zeros_like(n))
        if ctx.owner is not None:
            prev = getattr(W, "_row_grad_coef", None)
            W._row_grad_coef = coef if prev is None else prev + coef
            return None, None, None
        return (coef[:, None] * W.detach()).to(W.dtype), None, None


class _DenseDecode(torch.autograd.Function):
    """acts @ W_D for dense activations on the GEMM kernel (models/sae.py:367).  `w_op` is W_D [F, d] as the kernels
    read it (under autocast the bf16 copy the optimiser maintains, so that the per-step cast of the fp32 master and
    its backward are not run).  The forward product contracts over features: bf16 operands read W_D as it lies ([K, d]
    with K = features), fp32 operands a transposed copy `w_t` [d, F].
    Backward: d acts = g W_D^T contracts over d_model (W_D as it is), dW_D = acts^T g over the tokens."""

    @staticmethod
    def forward(ctx, acts, W_D, w_op, w_t=None, defer=False):
        acts = acts.contiguous()
        ctx.save_for_backward(acts, w_op)
        ctx.param = W_D if (defer and W_D.is_contiguous() and w_op.dtype == torch.bfloat16) else None
        ctx.w_dtype = W_D.dtype
        if w_t is None:
            return ops.gemm(acts, w_op, acts.dtype, b_k_major=True)
        return ops.encoder_gemm(acts, w_t, acts.dtype)

    @staticmethod
    def backward(ctx, g):
        acts, w_op = ctx.saved_tensors
        gg = g.to(w_op.dtype).contiguous()
        d_acts = ops.encoder_gemm(gg, w_op, w_op.dtype) if ctx.needs_input_grad[0] else None
        dW = None
        if ctx.needs_input_grad[1]:
            rows = _rows_over_tokens(acts, gg, w_op.dtype)                         # [F, d]
            if ctx.param is not None:
                _leave_lowp_grad(ctx.param, rows)
            else:
                dW = rows.to(ctx.w_dtype)
        return d_acts, dW, None, None, None


def dense_decode(model, acts: torch.Tensor, W_D: torch.Tensor, w_op: torch.Tensor, w_t_name: str, defer: bool = False):
    """acts [B, F] @ W_D [F, d] through `_DenseDecode` when the GEMM kernel takes the shapes, else None.  `w_op`: W_D as the
    kernels read it; the activations are cast to its dtype (under autocast the bf16 copy: what the reference's autocast
    matmul does to its operands).  A transposed fp32 copy is derived (and cached on `model` under `w_t_name`) only where
    the fp32 kernel needs one."""
    F, d = w_op.shape
    if acts.ndim != 2 or acts.shape[-1] != F or not acts.is_cuda or w_op.dtype not in (torch.float32, torch.bfloat16):
        return None
    acts = acts.to(w_op.dtype)
    # the forward contracts over F, the backward's d acts = g W_D^T over d: both must be whole slabs of the kernel
    if w_op.dtype == torch.bfloat16:
        if F % 64 == 0 and d % 64 == 0:
            return _DenseDecode.apply(acts, W_D, w_op, None, defer)
        return None
    if w_op.dtype == torch.float32 and F % 32 == 0 and d % 32 == 0:
        w_t = model._derive(w_t_name, W_D, lambda old: _transposed(w_op))
        return _DenseDecode.apply(acts, W_D, w_op, w_t, defer)
    return None


class _JumpReLUStep(torch.autograd.Function):
    """bias + decoder-norm scale + JumpReLU + the tanh / Lp penalty sums in one pass over [B, F]; the backward
    is one more pass that also yields the bias, threshold and decoder-norm gradients.  `norm` is the decoder
    norm; `scaled` says whether the activation is applied to h * norm (the penalties weigh by it either way)."""

    @staticmethod
    def forward(ctx, pre, b_E, norm, theta, scaled, tanh_c, window, want_tanh, want_lp):
        b = b_E.detach().float().contiguous()
        n = None if norm is None else norm.detach().float().contiguous()
        th = theta.detach().float().contiguous()
        acts, tanh_tok, lp_tok, _ = ops.jumprelu_fwd(pre.contiguous(), b, n if scaled else None, th, tanh_c, pen_norm=n,
                                                     want_tanh=want_tanh, want_lp=want_lp)
        ctx.save_for_backward(pre, b, th, *(() if n is None else (n,)))
        ctx.has_norm, ctx.scaled, ctx.tanh_c, ctx.window = n is not None, scaled, tanh_c, window
        ctx.b_dtype, ctx.th_dtype = b_E.dtype, theta.dtype
        return acts, tanh_tok, lp_tok

    @staticmethod
    def backward(ctx, g_acts, g_tanh, g_lp):
        pre, b, th, *rest = ctx.saved_tensors
        n = rest[0] if ctx.has_norm else None
        if g_acts is None:
            g_acts = torch.zeros_like(pre)
        fix = lambda g: None if g is None else g.float().contiguous()   # noqa: E731
        d_pre, d_bias, d_theta, d_norm = ops.jumprelu_bwd(
            pre.contiguous(), b, n if ctx.scaled else None, th, g_acts.to(pre.dtype).contiguous(), fix(g_tanh), ctx.tanh_c,
            fix(g_lp), ctx.window, pen_norm=n, want_norm_grad=ctx.has_norm and ctx.needs_input_grad[2])
        return d_pre, d_bias.to(ctx.b_dtype), d_norm, d_theta.to(ctx.th_dtype), None, None, None, None, None


def _code_penalty(code: ops.SparseCode, norm: torch.Tensor, kind: str, c: float, p: float, freq_scale: float, n_tokens: int):
    """The sparsity penalty of a sparse code before its coefficient (models/sparse_dictionary.py:888-925 on a = f n at
    the code's entries; entries that are zero add nothing to any of the three): per-token values [B] for "tanh" and
    "power", one scalar for "tanh-quad"; plus what the backward needs (per-token power sums / per-feature frequencies)."""
    tok, valid = _code_slot_tokens(code)
    a = torch.where(valid, code.val * norm[code.idx.long()], torch.zeros_like(code.val))
    B = code.n_tokens
    if kind == "tanh":
        pen = torch.zeros(B, dtype=torch.float32, device=a.device).index_add_(0, tok, torch.tanh(c * a))
        return pen, None
    if kind == "power":
        S = torch.zeros(B, dtype=torch.float32, device=a.device).index_add_(0, tok, a.pow(p))
        return S.pow(1.0 / p), S
    if kind == "tanh-quad":
        q = torch.zeros(code.d_sae, dtype=torch.float32, device=a.device).index_add_(0, code.idx.long(), torch.tanh(c * a)) / n_tokens
        return (q * (1 + q / freq_scale)).sum(), q
    raise ValueError(f"sparsity_loss_type f{kind} not supported.")


class _JumpReLUSparseStep(torch.autograd.Function):
    """The step of a dictionary whose activations are a sparse code, with a sparsity penalty: sparse decode + squared error
    (+ tanh / power / tanh-quad penalty) forward, and backward through the feature index of the code, like the plain TopK
    step.  For a JumpReLU the code holds every token's kept features and, with value 0, the features inside the
    straight-through window that are not kept (`win` flags them); for a TopK-family or ReLU dictionary it holds the
    kept entries, `win` is zero and the threshold a vector of zeros.  `dval` (the decoder's gradient at every entry) is
    what both the pre-activation gradient of kept entries and the threshold gradient of window entries start from.  With
    a = f n the penalised quantity, P' = d penalty / d a at the entry, and ga = dval + P' n:
        d pre   = ga at kept entries                              -> dW_E^T rows, db_E (factored)
        d theta = sum over window entries of (ga / s) (-theta / window)
        d n     = sum over kept entries of P' f
    exactly the sums the dense backward forms over [B, F] (the two derivative terms of act(h s) / s with respect to s
    cancel)."""

    @staticmethod
    def forward(ctx, theta, norm, W_E, b_E, W_D, b_D, label, tok_w, holder):
        sae, code = holder["model"], holder["code"]
        amp = holder["amp"]
        w_dec_op = sae._w_dec_operand(amp)
        recon, loss_tok, grad_recon, dval = ops.sparse_decode_mse_fused(code, w_dec_op, None if b_D is None else b_D.detach(),
                                                                        label, tok_w)
        loss = loss_tok.sum()
        l_s = None
        kind = holder.get("pen")
        if kind is not None:
            pen, aux = holder.get("pen_tok"), None
            if pen is None:
                pen, aux = _code_penalty(code, norm.detach().float(), kind, holder["tanh_c"], holder.get("p", 1),
                                         holder.get("frequency_scale", 0.01), code.n_tokens)
            l_s = holder["l1"] * pen
            loss = loss + ((tok_w * l_s).sum() if l_s.ndim else l_s)
            holder["pen_aux"] = aux
        holder["l_s"], holder["l_rec"] = l_s, loss_tok.sum()
        ctx.save_for_backward(theta.detach().float(), tok_w, grad_recon, dval, *(() if norm is None else (norm.detach().float(),)))
        ctx.holder, ctx.has_norm, ctx.has_b_D = holder, norm is not None, b_D is not None
        ctx.th_dtype = theta.dtype
        ctx.mark_non_differentiable(recon)
        ctx.set_materialize_grads(False)
        return loss, recon

    @staticmethod
    def backward(ctx, g_loss, _g_recon):
        if g_loss is None:
            return (None,) * 9
        theta, tok_w, grad_recon, dval, *rest = ctx.saved_tensors
        norm = rest[0] if ctx.has_norm else None
        h = ctx.holder
        sae, code, win = h["model"], h["code"], h["win"]
        F = code.d_sae
        g = g_loss.to(torch.float32)
        fi = ops.build_feature_index(code)
        idx = code.idx.long()
        val = code.val
        s_f = norm[idx] if (norm is not None and h["scaled"]) else None
        ga, dn_slot = dval, None
        kind = h.get("pen")
        if kind is not None:
            n_f = norm[idx]
            a = val * n_f
            if kind == "tanh":
                c = h["tanh_c"]
                t = torch.tanh(c * a)
                dpen = (h["l1"] * c) * tok_w[fi.slot_tok.long()] * (1.0 - t * t)
            elif kind == "power":
                p, S = float(h.get("p", 1)), h["pen_aux"][fi.slot_tok.long()]
                # d (sum a^p)^(1/p) / d a = S^(1/p - 1) a^(p - 1); torch's norm sends nothing to entries that are zero
                dpen = torch.where(a > 0, h["l1"] * tok_w[fi.slot_tok.long()] * S.clamp_min(1e-30).pow(1.0 / p - 1.0) * a.pow(p - 1.0),
                                   torch.zeros_like(a))
            else:   # tanh-quad: q_f = mean over tokens of tanh(c a); l_s = l1 sum_f q_f (1 + q_f / scale)
                c = h["tanh_c"]
                t = torch.tanh(c * a)
                q = h["pen_aux"][idx]
                dpen = (h["l1"] * c / code.n_tokens) * (1.0 + 2.0 * q / h.get("frequency_scale", 0.01)) * (1.0 - t * t)
            ga = dval + dpen * n_f
            dn_slot = (dpen * val).contiguous()
        d_pre = torch.where(val > 0, ga, torch.zeros_like(ga))
        d_theta = None
        if h.get("has_theta", True):
            th_f = theta[idx]
            dth_slot = win * (ga if s_f is None else ga / s_f) * (-th_f / h["window"])
            d_theta, d_norm = ops.feature_segment_sums(fi, dth_slot.contiguous(), dn_slot)
            d_theta = (d_theta * g).to(ctx.th_dtype)
        else:
            d_norm = ops.feature_segment_sums(fi, dn_slot)[0] if dn_slot is not None else None
        coef_dec, coef_enc = val * g, d_pre * g
        x_op = h["x_op"]
        grad_dense_D = ops.cast_bf16(grad_recon) if h["amp"] else grad_recon
        db_D = ops.col_sum(grad_recon) * g if ctx.has_b_D else None
        defer = h["defer"]
        if defer and all(getattr(p, "_sparse_grad", None) is None and p.grad is None for p in (sae.W_D, sae.W_E)):
            sae.W_D._sparse_grad = SparseRowGrad(fi, coef_dec, grad_dense_D, F)
            sae.W_E._sparse_grad = SparseRowGrad(fi, coef_enc, x_op, F, bias_param=sae.b_E)
            dW_D = dW_E = db_E = None
        else:
            dW_D, _ = ops.sparse_grad_rows(fi, coef_dec, grad_dense_D, F)
            dW_Et, db_E = ops.sparse_grad_rows(fi, coef_enc, x_op, F, want_bias=True)
            dW_E = dW_Et.t()
        return (d_theta, None if d_norm is None or not ctx.needs_input_grad[1] else d_norm * g,
                dW_E, db_E, dW_D, db_D, None, None, None)


@register_sae_model("sae")
class SparseAutoEncoder(SparseDictionary):
    def __init__(self, cfg: SAEConfig, device_mesh=None):
        super().__init__(cfg, device_mesh=device_mesh)
        self.cfg = cfg
        d, F = cfg.d_model, cfg.d_sae
        kw = dict(device=cfg.device, dtype=cfg.dtype)
        self.W_E = nn.Parameter(torch.empty(F, d, **kw).t())       # shape [d, F], feature-major storage
        self.b_E = nn.Parameter(torch.empty(F, **kw))
        self.W_D = nn.Parameter(torch.empty(F, d, **kw))
        if cfg.use_decoder_bias:
            self.b_D = nn.Parameter(torch.empty(d, **kw))
        if cfg.use_glu_encoder:
            self.W_E_glu = nn.Parameter(torch.empty(F, d, **kw).t())
            self.b_E_glu = nn.Parameter(torch.empty(F, **kw))
        self.hook_hidden_pre = HookPoint()
        self.hook_feature_acts = HookPoint()
        self.hook_reconstructed = HookPoint()
        # set by an optimiser that consumes SparseRowGrad (HipAdam): the fused backward then leaves W_E.grad /
        # W_D.grad unset and attaches the factored gradient as `param._sparse_grad` instead
        self.defer_weight_grads = False
        # aux-k: treat the dead features as a compact dense block (three small GEMMs) when shapes allow; False keeps
        # the sparse route (dead-feature entries stacked onto the main code) for every shape
        self.aux_dense_block = True
        # JumpReLU: take the sparse form of the step when the batch's activations are sparse enough (at most a fraction
        # 1 - cfg.sparsity_threshold_for_triton_spmm_kernel of [B, F] kept or inside the threshold window).  Looking
        # costs one pass over the pre-activation and one read-back; while the dictionary is dense it is done every
        # `jumprelu_sparse_probe_every` steps only.
        self.jumprelu_sparse_route = True
        self.jumprelu_sparse_probe_every = 16
        self._jr_dense_steps = 0

    # ---- an optimiser may still be updating W_D on another stream (see HipAdam.overlap_decoder_update) ----
    def set_pending_update(self, event) -> None:
        self._pending_update = event

    def _update_pending(self) -> bool:
        return getattr(self, "_pending_update", None) is not None

    def wait_pending_update(self) -> None:
        ev = getattr(self, "_pending_update", None)
        if ev is not None:
            torch.cuda.current_stream(self.W_D.device).wait_event(ev)
            self._pending_update = None

    def w_enc_t(self) -> torch.Tensor:
        """Contiguous [F, d] view of the encoder weight."""
        w = self.W_E.t()
        return w if w.is_contiguous() else w.contiguous()

    def _w_enc_operand(self, amp: bool) -> torch.Tensor:
        wt = self.w_enc_t().detach()
        if not amp or wt.dtype == torch.bfloat16:
            return wt
        return self._derive("W_E.bf16", self.W_E, lambda old: ops.cast_bf16(wt, old))

    def _w_glu_operand(self, amp: bool) -> torch.Tensor:
        """[F, d] operand of the gate's product: the parameter's own buffer, or its bf16 copy under autocast."""
        wt = self.W_E_glu.detach().t()
        wt = wt if wt.is_contiguous() else wt.contiguous()
        if not amp or wt.dtype == torch.bfloat16:
            return wt
        return self._derive("W_E_glu.bf16", self.W_E_glu, lambda old: ops.cast_bf16(wt, old))

    def _w_dec_operand(self, amp: bool) -> torch.Tensor:
        self.wait_pending_update()
        w = self.W_D.detach()
        if not amp or w.dtype == torch.bfloat16:
            return w
        return self._derive("W_D.bf16", self.W_D, lambda old: ops.cast_bf16(w, old))

    def _decoder_norm_nograd(self) -> torch.Tensor:
        self.wait_pending_update()
        return self._derive("W_D.norm", self.W_D, lambda old: ops.row_norm(self.W_D.detach().float(), old))

    # ---- norms (models/sae.py:136-188, 209-212) ----
    def encoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_E, p=2, dim=0, keepdim=keepdim)

    def decoder_norm(self, keepdim: bool = False) -> torch.Tensor:
        self.wait_pending_update()
        return torch.norm(self.W_D, p=2, dim=1, keepdim=keepdim)

    def decoder_bias_norm(self) -> torch.Tensor:
        if not self.cfg.use_decoder_bias:
            raise ValueError("Decoder bias is not used")
        return torch.norm(self.b_D, p=2, dim=0, keepdim=True)

    @torch.no_grad()
    def set_decoder_to_fixed_norm(self, value: float, force_exact: bool):
        if force_exact:
            self.W_D.mul_(value / self.decoder_norm(keepdim=True))
        else:
            self.W_D.mul_(value / torch.clamp(self.decoder_norm(keepdim=True), min=value))

    @torch.no_grad()
    def set_encoder_to_fixed_norm(self, value: float):
        self.W_E.mul_(value / self.encoder_norm(keepdim=True))

    @torch.no_grad()
    def transform_to_unit_decoder_norm(self):
        self.W_D.mul_(1 / self.decoder_norm(keepdim=True))

    @torch.no_grad()
    def standardize_parameters_of_dataset_norm(self):
        """models/sae.py:214-255: fold the dataset-wise norms into the weights, switch to "inference"."""
        assert self.cfg.norm_activation == "dataset-wise"
        assert self.dataset_average_activation_norm is not None
        fin = math.sqrt(self.cfg.d_model) / self.dataset_average_activation_norm[self.cfg.hook_point_in]
        fout = math.sqrt(self.cfg.d_model) / self.dataset_average_activation_norm[self.cfg.hook_point_out]
        self.b_E.div_(fin)
        if self.cfg.use_decoder_bias:
            self.b_D.div_(fout)
        self.W_D.mul_(fin / fout)
        self.cfg.norm_activation = "inference"

    @torch.no_grad()
    def init_encoder_with_decoder_transpose(self, factor: float = 1.0):
        self.W_E.copy_(self.W_D.t() * factor)

    @torch.no_grad()
    def init_encoder_bias_with_mean_hidden_pre(self, batch: dict[str, torch.Tensor]):
        """models/sae.py:511-515."""
        x = self.prepare_input(batch)[0]
        _, hidden_pre = self.encode(x, return_hidden_pre=True)
        self.b_E.sub_(hidden_pre.mean(dim=0).to(self.b_E.dtype))

    @torch.no_grad()
    def init_parameters(self, **kwargs):
        """models/sae.py:400-436: uniform encoder/decoder, zero biases."""
        super().init_parameters(**kwargs)
        eb, db = kwargs["encoder_uniform_bound"], kwargs["decoder_uniform_bound"]
        self.W_E.uniform_(-eb, eb)
        self.W_D.uniform_(-db, db)
        self.b_E.zero_()
        if self.cfg.use_decoder_bias:
            self.b_D.zero_()
        if self.cfg.use_glu_encoder:
            self.W_E_glu.uniform_(-eb, eb)
            self.b_E_glu.zero_()

    # ---- API path over dense tensors (models/sae.py:288-377) ----
    def _matmul_enc(self, x: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
        """x @ W for an encoder weight (W_E or the GLU gate): the GEMM kernel on GPU tensors whose shapes it takes,
        with its weight gradient as a product over the token axis on the same kernel; a library product otherwise."""
        amp = _autocast_dtype("cuda") == torch.bfloat16
        d = W.shape[0]
        if (x.is_cuda and W.is_cuda and W.ndim == 2 and x.shape[-1] == d and W.dtype in (torch.float32, torch.bfloat16)
                and _gemm_k_ok(d, torch.bfloat16 if (amp or W.dtype == torch.bfloat16) else torch.float32)):
            wt = W.detach().t()
            wt = wt if wt.is_contiguous() else wt.contiguous()          # [F, d]; a view for feature-major weights
            low = amp or wt.dtype == torch.bfloat16
            if low and wt.dtype != torch.bfloat16:
                name = "W_E.bf16" if W is self.W_E else ("W_E_glu.bf16" if W is getattr(self, "W_E_glu", None) else None)
                wt = self._derive(name, W, lambda old: ops.cast_bf16(wt, old)) if name is not None else ops.cast_bf16(wt)
            lead = x.shape[:-1]
            pre = _EncoderGemm.apply(x.reshape(-1, d), W, wt, low)
            return pre.view(*lead, pre.shape[-1])
        return x @ W

    def encode(self, x: torch.Tensor, return_hidden_pre: bool = False, **kwargs):
        x = x.to(self.W_E.dtype)
        hidden_pre = self._matmul_enc(x, self.W_E) + self.b_E
        if self.cfg.use_glu_encoder:
            hidden_pre = hidden_pre * torch.sigmoid(self._matmul_enc(x, self.W_E_glu) + self.b_E_glu)
        hidden_pre = self.hook_hidden_pre(hidden_pre)
        if self.cfg.sparsity_include_decoder_norm:
            hidden_pre = hidden_pre * self.decoder_norm()
        feature_acts = self.activation_function(hidden_pre)
        if self.cfg.sparsity_include_decoder_norm:
            feature_acts = feature_acts / self.decoder_norm()
            hidden_pre = hidden_pre / self.decoder_norm()
        if return_hidden_pre:
            return self.hook_feature_acts(feature_acts), hidden_pre
        return self.hook_feature_acts(feature_acts)

    def decode(self, feature_acts, **kwargs):
        if isinstance(feature_acts, ops.SparseCode):
            amp = _autocast_dtype("cuda") == torch.bfloat16
            reconstructed = ops.sparse_decode_fwd(feature_acts, self._w_dec_operand(amp),
                                                  self.b_D.detach() if self.cfg.use_decoder_bias else None)
            return self.hook_reconstructed(reconstructed)
        reconstructed = None
        if self.cfg.use_triton_kernel and feature_acts.is_cuda and self.cfg.d_model % 8 == 0 and self.W_D.dtype == torch.float32:
            # models/sae.py:355-367: the sparse decoder kernel once every token's activations are sparse enough
            # (and not all empty); the count is read on the host, as in the reference
            from .kernels import decode_with_hip_spmm_kernel

            fa2 = feature_acts.reshape(-1, feature_acts.shape[-1])
            nnz = ops.dense_row_nnz((fa2 if fa2.dtype in (torch.float32, torch.bfloat16) else fa2.float()).contiguous())
            max_l0 = int(nnz.max().item())
            if 0 < max_l0 < self.cfg.d_sae * (1 - self.cfg.sparsity_threshold_for_triton_spmm_kernel):
                amp = _autocast_dtype("cuda") == torch.bfloat16
                reconstructed = decode_with_hip_spmm_kernel(feature_acts, self.W_D, w_operand=self._w_dec_operand(amp), transposed=False)
        if reconstructed is None and feature_acts.is_cuda:
            # models/sae.py:367 on the GEMM kernel: bf16 operands read W_D as it lies, with the weight gradient as a product
            # over the token axis on the same kernel
            amp = _autocast_dtype("cuda") == torch.bfloat16
            out = dense_decode(self, feature_acts.reshape(-1, feature_acts.shape[-1]), self.W_D, self._w_dec_operand(amp), "W_D.t.f32")
            if out is not None:
                reconstructed = out.view(*feature_acts.shape[:-1], out.shape[-1])
        if reconstructed is None:
            reconstructed = feature_acts @ self.W_D
        if self.cfg.use_decoder_bias:
            reconstructed = reconstructed + self.b_D
        return self.hook_reconstructed(reconstructed)

    @torch.no_grad()
    def encode_sparse(self, x: torch.Tensor) -> ops.SparseCode:
        """Inference-time encode that stays sparse: GEMM + select, no dense [B, F] output."""
        assert self.cfg.act_fn.lower() == "topk", "encode_sparse covers the TopK activation"
        assert not self.cfg.use_glu_encoder, "encode_sparse does not cover the GLU encoder"
        amp = _autocast_dtype("cuda") == torch.bfloat16
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        w = self._w_enc_operand(amp)
        xo = ops.cast_bf16(x2.float()) if w.dtype == torch.bfloat16 and x2.dtype != torch.bfloat16 else x2.to(w.dtype)
        pre = ops.encoder_gemm(xo, w, torch.bfloat16 if amp else torch.float32)
        scale = self._decoder_norm_nograd() if self.cfg.sparsity_include_decoder_norm else None
        return ops.select_topk_row(pre, self.b_E.detach().float(), scale, self.current_k)

    def prepare_input(self, batch: dict[str, torch.Tensor], **kwargs):
        return batch[self.cfg.hook_point_in], {}, {}

    def prepare_label(self, batch: dict[str, torch.Tensor], **kwargs):
        return batch[self.cfg.hook_point_out]

    # ---- fused train-step loss ----
    def _no_hooks(self) -> bool:
        return not (self.hook_hidden_pre.has_hooks or self.hook_feature_acts.has_hooks or self.hook_reconstructed.has_hooks)

    def _fused_eligible(self, x, label, sparsity_loss_type, lp_coefficient, auxk_coefficient) -> bool:
        """TopK / BatchTopK: the plain step (reconstruction loss, optionally aux-k) or, with a sparsity penalty, the step
        with the penalty formed on the sparse code.  (An Lp coefficient is ignored for these activations, as the
        reference's loss does: models/sparse_dictionary.py:927.)"""
        amp = _autocast_dtype("cuda") == torch.bfloat16 or self.W_E.dtype == torch.bfloat16
        # what the kernels are built for: the GEMM's K granule, 16-byte decoder rows, and the feature index's token
        # limit (the sparse aux-k route stacks a second code onto the token axis); other shapes take the dense route
        shapes_fit = (self.cfg.d_model % (64 if amp else 32) == 0
                      and x.shape[0] * (2 if auxk_coefficient > 0.0 else 1) <= 131072)
        if sparsity_loss_type is not None and (auxk_coefficient > 0.0 or self.W_E.dtype != torch.float32
                                               or sparsity_loss_type not in ("tanh", "power", "tanh-quad")):
            return False
        return (
            self.cfg.act_fn.lower() in ("topk", "batchtopk")
            and x.is_cuda and x.ndim == 2 and label.ndim == 2 and shapes_fit
            and not self.cfg.use_glu_encoder and self._no_hooks()
            and (self.W_E.dtype == torch.float32
                 or (self.W_E.dtype == torch.bfloat16 and self.cfg.d_model % 64 == 0))
        )

    def _glu_eligible(self, x, label, sparsity_loss_type, lp_coefficient, auxk_coefficient) -> bool:
        amp = _autocast_dtype("cuda") == torch.bfloat16
        return (self.cfg.use_glu_encoder and self.cfg.act_fn.lower() in ("topk", "batchtopk") and x.is_cuda and x.ndim == 2
                and label.ndim == 2 and sparsity_loss_type is None and not (auxk_coefficient > 0.0) and self._no_hooks()
                and self.W_E.dtype == torch.float32 and self.cfg.d_model % (64 if amp else 32) == 0
                and self.cfg.d_model % 8 == 0 and x.shape[0] <= 131072)

    def _glu_loss(self, batch, x, label, l1_coefficient, lp_coefficient, auxk_coefficient, return_aux_data):
        mask = batch.get("mask")
        B = x.shape[0]
        amp = _autocast_dtype("cuda") == torch.bfloat16
        if mask is None:
            tok_w = torch.full((B,), 1.0 / B, dtype=torch.float32, device=x.device)
        else:
            m = mask.to(torch.float32)
            tok_w = m / m.sum()
        holder = _Holder()
        holder.model = self
        loss, recon = _GluSparseStep.apply(
            x.to(torch.float32) if x.dtype not in (torch.float32, torch.bfloat16) else x, label.to(torch.float32).contiguous(),
            tok_w, self.W_E, self.b_E, self.W_E_glu, self.b_E_glu, self.W_D, self.b_D if self.cfg.use_decoder_bias else None,
            int(self.current_k), amp, holder)
        if not return_aux_data:
            return loss
        code, hidden, scale = holder.code, holder.hidden, holder.scale
        eager = {"loss": loss, "l_rec": loss, "l_s": None, "l_p": None, "l_aux": None, "label": label, "mask": mask,
                 "reconstructed": recon, "l1_coefficient": l1_coefficient, "lp_coefficient": lp_coefficient,
                 "auxk_coefficient": auxk_coefficient, "sparse_code": code}
        lazy = {"n_tokens": (lambda: batch["tokens"].numel()) if mask is None else (lambda: int(mask.sum().item())),
                "feature_acts": code.to_dense,
                "hidden_pre": (lambda: (hidden * scale) / scale) if scale is not None else (lambda: hidden)}
        return LazyDict(eager, lazy)

    # ---- JumpReLU / ReLU train-step loss: dense activations, so the GEMM kernel for all five dense products + one fused
    # element-wise pass each way (a ReLU is the same kernels with a threshold of zero, which has no gradient) ----
    def _jumprelu_eligible(self, x, label, sparsity_loss_type, auxk_coefficient) -> bool:
        amp = _autocast_dtype("cuda") == torch.bfloat16
        return (
            self.cfg.act_fn.lower() in ("jumprelu", "relu") and x.is_cuda and x.ndim == 2 and label.ndim == 2
            and not self.cfg.use_glu_encoder and sparsity_loss_type in (None, "tanh", "power", "tanh-quad")
            and not (auxk_coefficient > 0.0) and self._no_hooks()
            and self.W_E.dtype == torch.float32 and self.cfg.d_sae % 8 == 0 and self.cfg.d_model % (64 if amp else 32) == 0
        )

    def _threshold_and_window(self):
        """(theta [F], window) of the activation: the JumpReLU's own, or zeros and any window for a ReLU (x > 0 is x > theta
        with theta = 0, and d theta = g (-theta / window) vanishes)."""
        jr = self.activation_function
        if self.cfg.act_fn.lower() == "jumprelu":
            return jr.get_jumprelu_threshold(), float(jr.jumprelu_threshold_window)
        zero = self.__dict__.get("_zero_theta")
        if zero is None or zero.device != self.b_E.device:
            zero = torch.zeros(self.cfg.d_sae, dtype=torch.float32, device=self.b_E.device)
            self.__dict__["_zero_theta"] = zero
        return zero, 1.0

    def _jumprelu_loss(self, batch, x, label, sparsity_loss_type, tanh_stretch_coefficient, l1_coefficient, lp_coefficient,
                       auxk_coefficient, return_aux_data, frequency_scale: float = 0.01, p: int = 1):
        from .sparse_dictionary import apply_token_mask

        mask = batch.get("mask")
        amp = _autocast_dtype("cuda") == torch.bfloat16
        is_jr = self.cfg.act_fn.lower() == "jumprelu"
        theta, window = self._threshold_and_window()
        defer = bool(self.defer_weight_grads and torch.is_grad_enabled())
        want_tanh, want_lp = sparsity_loss_type == "tanh", lp_coefficient > 0.0 and is_jr
        scaled = bool(self.cfg.sparsity_include_decoder_norm)
        w_enc_op = self._w_enc_operand(amp)
        given = None
        B = x.shape[0]
        if (self.jumprelu_sparse_route and not want_lp and B <= 131072
                and self.cfg.d_model % 8 == 0 and self._jr_dense_steps % max(1, self.jumprelu_sparse_probe_every) == 0):
            with torch.no_grad():
                x_op = (x if x.dtype == torch.bfloat16 else ops.cast_bf16(x.float().contiguous())) if amp else x.float().contiguous()
                n_raw = self._decoder_norm_nograd() if (scaled or sparsity_loss_type is not None) else None
                th_raw = theta.detach().float().contiguous()
                b_raw = self.b_E.detach().float()
                margin = None
                # once the route has been sparse, the product's epilogue also leaves every granule's largest margin over
                # its thresholds, and the select reads the pre-activations only where an entry can be
                if (amp and self._jr_dense_steps == 0 and getattr(self, "granule_select", True) and w_enc_op.dtype == torch.bfloat16
                        and self.cfg.d_model % 64 == 0 and self.cfg.d_sae % ops.GRANULE == 0 and self.cfg.d_sae <= ops.GRANULE_MAX_F):
                    pre_raw, margin = ops.encoder_gemm_jumprelu_margin(x_op, w_enc_op, b_raw, n_raw if scaled else None, th_raw)
                else:
                    pre_raw = ops.encoder_gemm(x_op, w_enc_op, torch.bfloat16 if amp else torch.float32)
                given = (x_op, pre_raw)
                budget = int(B * self.cfg.d_sae * (1.0 - self.cfg.sparsity_threshold_for_triton_spmm_kernel))
                picked = ops.jumprelu_select(pre_raw, b_raw, n_raw if scaled else None, th_raw, window,
                                             float(tanh_stretch_coefficient), pen_norm=n_raw,
                                             want_tanh=want_tanh, max_entries=budget, granule_margin=margin)
            if picked is not None:
                self._jr_dense_steps = 0
                code, win, tanh_tok, _l0 = picked
                return self._sparse_code_loss(batch, label, mask, code, win, x_op, pre_raw, amp, defer, theta, window,
                                              sparsity_loss_type, tanh_tok, float(tanh_stretch_coefficient), float(l1_coefficient),
                                              float(frequency_scale), p, lp_coefficient, auxk_coefficient, return_aux_data)
        self._jr_dense_steps += 1
        pre = _EncoderGemm.apply(x, self.W_E, w_enc_op, amp, defer, given)
        n = None
        want_dense_pen = sparsity_loss_type in ("power", "tanh-quad")
        if scaled or want_tanh or want_lp or want_dense_pen:
            n = _RowNormDeferred.apply(self.W_D, self._decoder_norm_nograd(), self if defer else None)
        acts, tanh_tok, lp_tok = _JumpReLUStep.apply(pre, self.b_E, n, theta, scaled, float(tanh_stretch_coefficient), window,
                                                     want_tanh, want_lp)
        reconstructed = dense_decode(self, acts, self.W_D, self._w_dec_operand(amp), "W_D.t.f32", defer)
        if reconstructed is None:
            reconstructed = acts @ self.W_D
        if self.cfg.use_decoder_bias:
            reconstructed = reconstructed + self.b_D
        l_rec = apply_token_mask((reconstructed - label).pow(2).sum(dim=-1), 1, mask, "mean")
        loss = l_rec
        l_s = l_p = None
        if want_tanh:
            l_s = l1_coefficient * tanh_tok
            loss = loss + apply_token_mask(l_s, 1, mask, "mean")
        elif want_dense_pen:
            # models/sparse_dictionary.py:888-925.  The products of the step stay on the GEMM kernel; these two penalties
            # are element-wise framework operations on the activations (their gradient joins the decoder's on the
            # way into the activation kernel's backward, and reaches W_D through the norm as a per-row coefficient)
            weighted = acts.float() * n
            if sparsity_loss_type == "power":
                l_s = torch.norm(weighted, p=p, dim=-1)
            else:
                freq = torch.tanh(tanh_stretch_coefficient * weighted).mean(dim=0)
                l_s = (freq * (1 + freq / frequency_scale)).sum(dim=-1)
            l_s = l1_coefficient * l_s
            loss = loss + apply_token_mask(l_s, min(1, l_s.ndim), mask if l_s.ndim else None, "mean")
        if want_lp:
            l_p = apply_token_mask(lp_coefficient * lp_tok, 1, mask, "mean")
            loss = loss + l_p
        if not return_aux_data:
            return loss
        b_E = self.b_E.detach()
        eager = {"loss": loss, "l_rec": l_rec, "l_s": l_s, "l_p": l_p, "l_aux": None, "label": label, "mask": mask,
                 "feature_acts": acts, "reconstructed": reconstructed, "l1_coefficient": l1_coefficient,
                 "lp_coefficient": lp_coefficient, "auxk_coefficient": auxk_coefficient}
        lazy = {"n_tokens": (lambda: batch["tokens"].numel()) if mask is None else (lambda: int(mask.sum().item())),
                "hidden_pre": lambda: pre.detach().float() + b_E}
        return LazyDict(eager, lazy)

    def _sparse_code_loss(self, batch, label, mask, code, win, x_op, pre_raw, amp, defer, theta, window, sparsity_loss_type,
                          pen_tok, tanh_c, l1_coefficient, frequency_scale, p, lp_coefficient, auxk_coefficient, return_aux_data):
        """Loss of a step whose activations are the sparse code `code` (JumpReLU / ReLU above the sparsity gate, or a TopK
        family selection) with an optional sparsity penalty, through `_JumpReLUSparseStep`."""
        B = code.n_tokens
        scaled = bool(self.cfg.sparsity_include_decoder_norm)
        if mask is None:
            tok_w = torch.full((B,), 1.0 / B, dtype=torch.float32, device=label.device)
        else:
            m = mask.to(torch.float32)
            tok_w = m / m.sum()
        n = None
        if scaled or sparsity_loss_type is not None:
            n = _RowNormDeferred.apply(self.W_D, self._decoder_norm_nograd(), self if defer else None)
        has_theta = self.cfg.act_fn.lower() == "jumprelu"
        if win is None:
            win = torch.zeros_like(code.val)
        holder = {"model": self, "code": code, "win": win, "pen": sparsity_loss_type, "pen_tok": pen_tok, "x_op": x_op, "amp": amp,
                  "defer": defer, "scaled": scaled, "tanh_c": tanh_c, "l1": l1_coefficient, "window": window, "p": p,
                  "frequency_scale": frequency_scale, "has_theta": has_theta}
        loss, recon = _JumpReLUSparseStep.apply(theta, n, self.W_E, self.b_E, self.W_D,
                                                self.b_D if self.cfg.use_decoder_bias else None,
                                                label.to(torch.float32).contiguous(), tok_w, holder)
        if not return_aux_data:
            return loss
        b_E = self.b_E.detach()
        scale = self._decoder_norm_nograd() if scaled else None

        def dense_hidden_pre():
            h0 = pre_raw.float() + b_E
            return (h0 * scale) / scale if scale is not None else h0

        eager = {"loss": loss, "l_rec": holder["l_rec"], "l_s": holder["l_s"], "l_p": None, "l_aux": None, "label": label,
                 "mask": mask, "reconstructed": recon, "l1_coefficient": l1_coefficient, "lp_coefficient": lp_coefficient,
                 "auxk_coefficient": auxk_coefficient, "sparse_code": code}
        lazy = {"n_tokens": (lambda: batch["tokens"].numel()) if mask is None else (lambda: int(mask.sum().item())),
                "feature_acts": code.to_dense,
                "hidden_pre": dense_hidden_pre}
        return LazyDict(eager, lazy)

    @torch.no_grad()
    def _select_code(self, x: torch.Tensor, amp: bool):
        """GEMM + TopK / BatchTopK select of an fp32 dictionary -> (x operand, pre, code): what the forward of the fused
        step does, for the routes that continue from the code with other losses."""
        w_enc_op = self._w_enc_operand(amp)
        B, k = x.shape[0], int(self.current_k)
        batch_wide = self.cfg.act_fn.lower() == "batchtopk"
        b_E = self.b_E.detach().float()
        scale = self._decoder_norm_nograd() if self.cfg.sparsity_include_decoder_norm else None
        gmax = None
        if amp:
            x_op = x if x.dtype == torch.bfloat16 else ops.cast_bf16(x.float().contiguous())
            granule = (getattr(self, "granule_select", True)
                       and (ops.granule_route_supported(x.shape[1], w_enc_op.shape[0], k) if not batch_wide
                            else x.shape[1] % 64 == 0 and w_enc_op.shape[0] % 256 == 0))
            if granule:
                pre, gmax = ops.encoder_gemm_granule_max(x_op, w_enc_op, b_E, scale)
            else:
                pre = ops.encoder_gemm(x_op, w_enc_op, torch.bfloat16)
        else:
            x_op = x.float().contiguous()
            pre = ops.encoder_gemm(x_op, w_enc_op, torch.float32)
        if batch_wide:
            code = ops.select_topk_batch(pre, b_E, scale, k * B, granule_max=gmax)
        else:
            code = ops.select_topk_row(pre, b_E, scale, k, granule_max=gmax)
        return x_op, pre, code

    def _flattened_loss(self, batch, x, label, kw):
        """[batch, seq_len, d_model] activations (models/sae.py:288-345 takes both forms): every loss term is a (masked) mean
        over all tokens, and BatchTopK flattens the two token axes itself, so the step runs on the [batch * seq_len, .]
        views and the per-token outputs are given their two axes back."""
        b, s, d = x.shape
        mask = batch.get("mask")
        flat = dict(batch)
        flat[self.cfg.hook_point_in] = x.reshape(b * s, d)
        flat[self.cfg.hook_point_out] = label.reshape(b * s, label.shape[-1])
        if mask is not None:
            flat["mask"] = mask.reshape(b * s)
        if self.cfg.hook_point_in == self.cfg.hook_point_out:
            flat[self.cfg.hook_point_out] = flat[self.cfg.hook_point_in]
        out = self.compute_loss(flat, **kw)
        if not kw.get("return_aux_data", True):
            return out

        def fix(v):
            if torch.is_tensor(v) and v.ndim >= 1 and v.shape[0] == b * s:
                return v.reshape(b, s, *v.shape[1:])
            return v

        if isinstance(out, LazyDict):
            eager = {k_: fix(v) for k_, v in dict.items(out) if v is not LazyDict._PENDING}
            lazy = {k_: (lambda f=f: fix(f())) for k_, f in out._lazy.items()}
            res = LazyDict(eager, lazy)
        else:
            res = {k_: fix(v) for k_, v in out.items()}
        res["label"], res["mask"] = label, mask
        return res

    def compute_loss(self, batch, label=None, *, sparsity_loss_type=None, tanh_stretch_coefficient: float = 4.0,
                     frequency_scale: float = 0.01, p: int = 1, l1_coefficient: float = 1.0,
                     lp_coefficient: float = 0.0, auxk_coefficient: float = 0.0, k_aux: int = 512,
                     update_dead_statistics=None, return_aux_data: bool = True, **kwargs):
        x, _, _ = self.prepare_input(batch)
        label = self.prepare_label(batch, **kwargs)
        if x.ndim == 3 and label.ndim == 3 and x.is_cuda and self._no_hooks():
            x2, l2 = x.reshape(-1, x.shape[-1]), label.reshape(-1, label.shape[-1])
            if (self._jumprelu_eligible(x2, l2, sparsity_loss_type, auxk_coefficient)
                    or self._fused_eligible(x2, l2, sparsity_loss_type, lp_coefficient, auxk_coefficient)):
                return self._flattened_loss(batch, x, label, dict(
                    sparsity_loss_type=sparsity_loss_type, tanh_stretch_coefficient=tanh_stretch_coefficient,
                    frequency_scale=frequency_scale, p=p, l1_coefficient=l1_coefficient, lp_coefficient=lp_coefficient,
                    auxk_coefficient=auxk_coefficient, k_aux=k_aux, update_dead_statistics=update_dead_statistics,
                    return_aux_data=return_aux_data, **kwargs))
        if self._glu_eligible(x, label, sparsity_loss_type, lp_coefficient, auxk_coefficient):
            return self._glu_loss(batch, x, label, l1_coefficient, lp_coefficient, auxk_coefficient, return_aux_data)
        if self._jumprelu_eligible(x, label, sparsity_loss_type, auxk_coefficient):
            return self._jumprelu_loss(batch, x, label, sparsity_loss_type, tanh_stretch_coefficient, l1_coefficient,
                                       lp_coefficient, auxk_coefficient, return_aux_data, frequency_scale, p)
        if not self._fused_eligible(x, label, sparsity_loss_type, lp_coefficient, auxk_coefficient):
            return super().compute_loss(
                batch, sparsity_loss_type=sparsity_loss_type, tanh_stretch_coefficient=tanh_stretch_coefficient,
                frequency_scale=frequency_scale, p=p, l1_coefficient=l1_coefficient, lp_coefficient=lp_coefficient,
                auxk_coefficient=auxk_coefficient, k_aux=k_aux, update_dead_statistics=update_dead_statistics,
                return_aux_data=return_aux_data, **kwargs)

        mask = batch.get("mask")
        B = x.shape[0]
        amp = _autocast_dtype("cuda") == torch.bfloat16
        if sparsity_loss_type is not None:
            # TopK / BatchTopK with a sparsity penalty: select as the plain step does, then decode, loss, penalty and the
            # backward on the code (the penalty's gradient joins the decoder's at every kept entry and reaches W_D
            # through the decoder norm)
            x_op, pre, code = self._select_code(x, amp)
            defer = bool(self.defer_weight_grads and torch.is_grad_enabled())
            theta, window = self._threshold_and_window() if self.cfg.act_fn.lower() == "jumprelu" else (
                torch.zeros(1, dtype=torch.float32, device=x.device), 1.0)
            return self._sparse_code_loss(batch, label, mask, code, None, x_op, pre, amp, defer, theta, window, sparsity_loss_type,
                                          None, float(tanh_stretch_coefficient), float(l1_coefficient), float(frequency_scale), p,
                                          lp_coefficient, auxk_coefficient, return_aux_data)
        if mask is None:
            tok_w = torch.full((B,), 1.0 / B, dtype=torch.float32, device=x.device)
        else:
            m = mask.to(torch.float32)
            tok_w = m / m.sum()
        holder = _Holder()
        holder.model = self
        if auxk_coefficient > 0.0:
            assert update_dead_statistics is not None, "update_dead_statistics must be set when auxk_coefficient > 0.0"

            def is_dead(code, _upd=update_dead_statistics, _mask=mask):
                sparse_upd = getattr(getattr(_upd, "__self__", None), "update_dead_statistics_sparse", None)
                if sparse_upd is not None:
                    return sparse_upd(code, _mask)
                return _upd(code.to_dense(), _mask, ("batch", "sae"))  # a callable that only knows dense activations

            holder.aux = {"is_dead": is_dead, "k_aux": k_aux, "coefficient": auxk_coefficient, "dense": self.aux_dense_block}
        holder.defer_to = self if self.defer_weight_grads and torch.is_grad_enabled() else None
        loss, recon = _FusedSparseStep.apply(
            x.to(torch.float32) if x.dtype not in (torch.float32, torch.bfloat16) else x,
            label.to(torch.float32).contiguous(), tok_w, self.W_E, self.b_E, self.W_D,
            self.b_D if self.cfg.use_decoder_bias else None, int(self.current_k), amp, holder)
        if not return_aux_data:
            return loss

        code, pre, b_E, scale = holder.code, holder.pre, self.b_E.detach(), holder.scale

        def dense_hidden_pre():
            h0 = pre.float() + b_E
            return (h0 * scale) / scale if scale is not None else h0

        l_aux = holder.l_aux
        eager = {
            "loss": loss, "l_rec": loss if l_aux is None else (loss - l_aux).detach(), "l_s": None, "l_p": None,
            "l_aux": l_aux, "label": label, "mask": mask,
            "reconstructed": recon, "l1_coefficient": l1_coefficient, "lp_coefficient": lp_coefficient,
            "auxk_coefficient": auxk_coefficient, "sparse_code": code,
        }
        if holder.aux_code is not None:
            eager["aux_sparse_code"] = holder.aux_code    # the aux-k term's selection among the dead features
        lazy = {
            "n_tokens": (lambda: batch["tokens"].numel()) if mask is None else (lambda: int(mask.sum().item())),
            "feature_acts": code.to_dense,
            "hidden_pre": dense_hidden_pre,
        }
        return LazyDict(eager, lazy)
