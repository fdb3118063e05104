"""Cross-layer transcoder on the HIP path.

API of the reference's CLT (src/llamascopium/models/clt.py:124-1125): L encoders `W_E [L, d, F]`,
`b_E [L, F]`; decoder groups `W_D[j] [j+1, F, d]` (sources 0..j writing to layer j) with biases
`b_D[j] [d]`; output layer j is  y_j = sum_{i<=j} f_i @ W_D[j][i] + b_D[j].

Memory layout: `W_E` has the reference's shape but each layer is stored feature-major (a permuted
view of a contiguous [L, F, d] buffer), so every layer's encoder is one call of the encoder GEMM.
A decoder group is contiguous, so `W_D[j]` read as a [(j+1)*F, d] matrix is the decoder of the
concatenated feature space of layers 0..j.

Fused path (TopK family): the activations of all layers are held as ONE sparse code over the
concatenated L*F feature space with every token's entries in ascending (layer, feature) order.
Output layer j then decodes the per-token PREFIX of that code (the entries of layers <= j) against
`W_D[j]`, i.e. the 78 dense [B, F] x [F, d] products of a 12-layer CLT become 12 sparse decodes, and
one feature index of the whole code serves every weight gradient (a feature range of it is the
index of a layer, a feature prefix the index of a decoder group).
"""

from __future__ import annotations

import dataclasses
import math
from typing import Any, Optional

import torch
from torch import nn

from . import ops
from .activation_functions import JumpReLU, _topk_mask_lowest_index, batch_topk_dense, topk_dense
from .config import CLTConfig, register_sae_model
from .sae import SparseRowGrad, SparseRowGradPieces, _autocast_dtype, _gemm_k_ok, _rows_over_tokens, dense_decode
from .sparse_dictionary import LazyDict, SparseDictionary

_TOPK_FAMILY = ("topk", "layertopk", "batchtopk", "batchlayertopk")


def _slot_tokens(code: ops.SparseCode):
    """(token of every slot [n_slots] int64, slot-is-inside-its-row [n_slots] bool)."""
    slots = torch.arange(code.n_slots, device=code.idx.device)
    tok = torch.searchsorted(code.row_off, slots, right=True) - 1
    tok = tok.clamp_(min=0)
    valid = (slots - code.row_off[tok]) < code.row_nnz[tok]
    return tok, valid


def merge_layer_codes(codes: list[ops.SparseCode]) -> tuple[ops.SparseCode, torch.Tensor]:
    """Per-layer codes over F features each -> one code over L*F features (feature l*F + f), every
    token's entries sorted by (layer, feature); also the per-token per-layer entry counts [B, L]."""
    L, B, F = len(codes), codes[0].n_tokens, codes[0].d_sae
    keys, vals = [], []
    sentinel = torch.iinfo(torch.int64).max
    for l, c in enumerate(codes):
        tok, valid = _slot_tokens(c)
        key = tok * (L * F) + (l * F) + c.idx.long()
        keys.append(torch.where(valid, key, torch.full_like(key, sentinel)))
        vals.append(c.val)
    key, perm = torch.sort(torch.cat(keys))
    val = torch.cat(vals)[perm]
    layer_cnt = torch.stack([c.row_nnz for c in codes], dim=1)                     # [B, L]
    row_nnz = layer_cnt.sum(dim=1).to(torch.int32)
    row_off = torch.cumsum(row_nnz, 0, dtype=torch.int64) - row_nnz
    idx = torch.where(key == sentinel, torch.zeros_like(key), key % (L * F)).to(torch.int32)
    return ops.SparseCode(idx, val.contiguous(), row_off, row_nnz, B, L * F), layer_cnt


def relabel_feature_major_code(code: ops.SparseCode, L: int, F: int) -> ops.SparseCode:
    """A code whose feature ids are f * L + l (the columns of a [B, F, L] matrix) -> the same entries under
    ids l * F + f, every token's entries re-sorted to ascend in (layer, feature).  Rows keep their extents."""
    tok, valid = _slot_tokens(code)
    raw = code.idx.long()
    new = (raw % L) * F + torch.div(raw, L, rounding_mode="floor")
    sentinel = torch.iinfo(torch.int64).max
    key, perm = torch.sort(torch.where(valid, tok * (L * F) + new, torch.full_like(new, sentinel)))
    idx = torch.where(key == sentinel, torch.zeros_like(key), key % (L * F)).to(torch.int32)
    # valid slots are packed row after row from slot 0 on (the batch select's layout), so sorted position = slot
    return dataclasses.replace(code, idx=idx, val=code.val[perm].contiguous())


def layer_counts(code: ops.SparseCode, L: int, F: int) -> torch.Tensor:
    """Entries per (token, layer) [B, L] of a code over L*F features."""
    tok, valid = _slot_tokens(code)
    cell = tok * L + torch.div(code.idx.long(), F, rounding_mode="floor")
    cell = torch.where(valid, cell, torch.zeros_like(cell))     # slots outside their row add 0 to cell 0
    cnt = torch.zeros(code.n_tokens * L, dtype=torch.int32, device=code.idx.device)
    cnt.scatter_add_(0, cell, valid.to(torch.int32))
    return cnt.view(code.n_tokens, L)


class _FusedCLTStep(torch.autograd.Function):
    """L encoder GEMMs -> TopK-family select -> L prefix decodes + squared error, forward and backward
    in kernels.  Arguments after `holder` are the parameters: W_E, b_E, W_D[0..L-1], b_D[0..L-1]."""

    @staticmethod
    def forward(ctx, x, label, amp, holder, W_E, b_E, *dec):
        m: "CrossLayerTranscoder" = holder["model"]
        B, L, d = x.shape
        F = m.cfg.d_sae
        k = int(m.current_k)
        act = m.cfg.act_fn.lower()
        w_enc_op = m._w_enc_operand(amp)                                   # [L, F, d]
        x_l = x.permute(1, 0, 2).contiguous()                              # [L, B, d]
        if amp:
            x_op = ops.cast_bf16(x_l.view(L * B, d)).view(L, B, d) if x_l.dtype != torch.bfloat16 else x_l
        else:
            x_op = x_l
        out_dtype = torch.bfloat16 if amp else torch.float32
        norms = m._norm_per_feature_nograd() if m.cfg.sparsity_include_decoder_norm else None     # [L, F]
        b_enc = b_E.detach().float().contiguous()
        if (act == "topk" and amp and getattr(m, "granule_select", True) and w_enc_op.dtype == torch.bfloat16
                and ops.granule_route_supported(d, F, min(k, F))):
            # per-layer TopK on bf16 operands: the L encoder products in one launch whose epilogue leaves the per-granule
            # key maxima, one select over the L * B stacked rows that reads a row only where those maxima allow a kept
            # entry, and one kernel that strings every token's layers together
            pre_all, gmax = ops.encoder_gemm_granule_max(x_op.contiguous(), w_enc_op, b_enc,
                                                         None if norms is None else norms.contiguous())
            stacked = ops.select_topk_row(pre_all.view(L * B, F), b_enc, None if norms is None else norms.contiguous(),
                                          min(k, F), granule_max=gmax.view(L * B, -1), rows_per_group=B)
            cat, layer_cnt = ops.merge_layer_codes(stacked, L)
            pres = list(pre_all.unbind(0))
        elif act in ("topk", "batchtopk"):
            pres = [ops.encoder_gemm(x_op[l], w_enc_op[l], out_dtype) for l in range(L)]
            sel = (lambda p, b, s: ops.select_topk_row(p, b, s, min(k, F))) if act == "topk" else \
                  (lambda p, b, s: ops.select_topk_batch(p, b, s, k * B))
            codes = [sel(pres[l], b_enc[l], None if norms is None else norms[l]) for l in range(L)]
            cat, layer_cnt = merge_layer_codes(codes)
        else:
            pres = [ops.encoder_gemm(x_op[l], w_enc_op[l], out_dtype) for l in range(L)]
            pre_cat = torch.stack(pres, dim=1).view(B, L * F) if act == "layertopk" else None
            flat = lambda t: None if t is None else t.reshape(L * F)      # noqa: E731
            if act == "layertopk":
                cat = ops.select_topk_row(pre_cat, flat(b_enc), flat(norms), min(k, L * F))
            else:
                # the reference flattens this scope as (batch, feature, layer) (clt.py:312: dim=(0, -1, -2)), which is
                # the order that decides ties at the threshold: select over the [B, F, L] arrangement, then relabel
                tr = lambda t: None if t is None else t.t().reshape(F * L).contiguous()   # noqa: E731
                cat = ops.select_topk_batch(torch.stack(pres, dim=2).view(B, F * L), tr(b_enc), tr(norms), k * B)
                cat = relabel_feature_major_code(cat, L, F)
            layer_cnt = layer_counts(cat, L, F)
        prefix = torch.cumsum(layer_cnt, dim=1).to(torch.int32)           # entries of layers <= j, per token
        tok_w = torch.full((B,), 1.0 / (L * B), dtype=torch.float32, device=x.device)
        w_dec_ops = m._w_dec_operands(amp)
        b_D = dec[L:]
        # the L decodes write their reconstructions, output gradients and per-token losses into one buffer each and add
        # their value gradients to one array: no stacking copy, no sum pass per layer, and the backward casts / sums the
        # output gradients of all layers in one launch each
        grads = torch.empty(L, B, d, dtype=torch.float32, device=x.device)
        recon = torch.empty(L, B, d, dtype=torch.float32, device=x.device)
        loss_toks = torch.empty(L, B, dtype=torch.float32, device=x.device)
        dval = torch.zeros(cat.n_slots, dtype=torch.float32, device=x.device)
        prefix_t = prefix.t().contiguous()                                # [L, B]
        for j in range(L):
            # the merged code is sorted by layer inside a token, so a token's first prefix[b, j] slots are its entries of
            # layers <= j; the kernel visits exactly those
            code_j = dataclasses.replace(cat, row_nnz=prefix_t[j], d_sae=(j + 1) * F)
            ops.sparse_decode_mse_fused(
                code_j, w_dec_ops[j].view((j + 1) * F, d), b_D[j].detach(), label[j].contiguous(), tok_w,
                recon_out=recon[j], loss_out=loss_toks[j], dval_acc=dval, grad_out=grads[j])
        loss = loss_toks.sum()
        holder.update(code=cat, pres=pres, norms=norms, layer_cnt=layer_cnt)
        ctx.cat, ctx.grads, ctx.dval, ctx.x_op, ctx.w_enc_op = cat, grads, dval, x_op, w_enc_op
        ctx.shape = (B, L, d, F)
        ctx.amp = bool(amp)
        ctx.defer_to = m if holder.get("defer") else None
        ctx.mark_non_differentiable(recon)
        return loss, recon

    @staticmethod
    def backward(ctx, g_loss, _g_recon):
        B, L, d, F = ctx.shape
        g = g_loss.to(torch.float32)
        cat = ctx.cat
        fi = ops.build_feature_index(cat)
        coef_dec = cat.val * g
        coef_enc = ctx.dval * g
        m = ctx.defer_to
        dec_params = None if m is None else list(m.W_D)
        defer = (m is not None and m.W_E.grad is None and getattr(m.W_E, "_sparse_grad", None) is None
                 and all(w.grad is None and getattr(w, "_sparse_grad", None) is None for w in dec_params))
        dW_D, dW_E, db_E = [], [], []
        enc_pieces = []
        db_D = list((ctx.grads.sum(dim=1) * g).unbind(0))            # [L, d]: every layer's bias gradient in one reduction
        gd_all = ops.cast_bf16(ctx.grads.view(L * B, d)).view(L, B, d) if (defer and ctx.amp) else ctx.grads
        for j in range(L):
            fi_j = ops.FeatureIndex(fi.feat_ptr[: (j + 1) * F + 1], fi.feat_slot, fi.slot_tok)      # features of layers <= j
            fi_l = ops.FeatureIndex(fi.feat_ptr[j * F: (j + 1) * F + 1], fi.feat_slot, fi.slot_tok)  # features of layer j
            if defer:
                # the optimiser rebuilds the rows where it consumes them; nothing dense is written here
                dec_params[j]._sparse_grad = SparseRowGrad(fi_j, coef_dec, gd_all[j], (j + 1) * F)
                enc_pieces.append((j * F, SparseRowGrad(fi_l, coef_enc, ctx.x_op[j], F)))
                dW_D.append(None)
                continue
            rows, _ = ops.sparse_grad_rows(fi_j, coef_dec, ctx.grads[j], (j + 1) * F)
            dW_D.append(rows.view(j + 1, F, d))
            rows_e, bias_e = ops.sparse_grad_rows(fi_l, coef_enc, ctx.x_op[j], F, want_bias=True)
            dW_E.append(rows_e); db_E.append(bias_e)
        if defer:
            m.W_E._sparse_grad = SparseRowGradPieces(enc_pieces, L * F, bias_param=m.b_E)
            dW_E = db_E = None
        else:
            dW_E = torch.stack(dW_E).permute(0, 2, 1)                   # [L, F, d] buffer seen as [L, d, F]
            db_E = torch.stack(db_E)
        dx = dlabel = None
        if ctx.needs_input_grad[0]:
            # d x[:, l] = sum over layer l's kept entries of d(pre) * W_E[l][:, f]
            w_all = ctx.w_enc_op.reshape(L * F, d)
            parts = []
            slot_layer = torch.div(cat.idx, F, rounding_mode="floor")
            for l in range(L):
                c = dataclasses.replace(cat, val=torch.where(slot_layer == l, coef_enc, torch.zeros_like(coef_enc)))
                parts.append(ops.sparse_decode_fwd(c, w_all, None))
            dx = torch.stack(parts, dim=1)
        if ctx.needs_input_grad[1]:
            dlabel = -ctx.grads * g
        return (dx, dlabel, None, None, dW_E, db_E, *dW_D, *db_D)


class _LayerEncoderGemm(torch.autograd.Function):
    """pre[b, l, :] = x[b, l, :] @ W_E[l] for every layer on the GEMM kernel (clt.py:559, "...ld,lds->...ls"): one launch
    per layer into one [L, B, F] buffer, returned as its [B, L, F] view.  Backward: per layer the weight gradient
    d(pre)^T x as a product over the token axis on the same kernel."""

    @staticmethod
    def forward(ctx, x, W_E, w_op, amp):
        B, L, d = x.shape
        F = w_op.shape[1]
        x_l = x.permute(1, 0, 2).contiguous()                                    # [L, B, d]
        if amp:
            x_op = x_l if x_l.dtype == torch.bfloat16 else ops.cast_bf16(x_l.float().view(L * B, d)).view(L, B, d)
        else:
            x_op = x_l.float()
        out_dtype = torch.bfloat16 if amp else torch.float32
        pre = torch.empty(L, B, F, dtype=out_dtype, device=x.device)
        for l in range(L):
            ops.encoder_gemm(x_op[l], w_op[l], out_dtype, out=pre[l])
        ctx.save_for_backward(x_op, w_op)
        ctx.x_dtype, ctx.w_dtype = x.dtype, W_E.dtype
        return pre.permute(1, 0, 2)

    @staticmethod
    def backward(ctx, g):
        x_op, w_op = ctx.saved_tensors
        L = x_op.shape[0]
        gl = g.permute(1, 0, 2).to(w_op.dtype).contiguous()                     # [L, B, F]
        dx = dW = None
        if ctx.needs_input_grad[0]:   # rare (activations carry no gradient in training): library products
            dx = torch.stack([gl[l] @ w_op[l] for l in range(L)], dim=1).to(ctx.x_dtype)
        if ctx.needs_input_grad[1]:
            rows = torch.stack([_rows_over_tokens(gl[l], x_op[l], w_op.dtype) for l in range(L)])      # [L, F, d]
            dW = rows.permute(0, 2, 1).to(ctx.w_dtype)
        return dx, dW, None, None


class _PrefixDecode(torch.autograd.Function):
    """out[j] = sum_{i <= j} feature_acts[:, i, :] @ W_D[j][i] for every output layer j (clt.py:630-709), for activations
    given as one sparse code over the L F concatenated features (ascending (layer, feature) inside a token): output layer j
    gathers the rows of W_D[j], read as [(j + 1) F, d], that the token's entries of layers <= j name.  Backward: the value
    gradients of the L decodes summed and scattered back to the dense activations, and per decoder group the gradient rows
    from the feature index (a feature prefix of the one index built for the whole code)."""

    @staticmethod
    def forward(ctx, acts2, code, prefix_t, dims, w_ops, *W_D):
        L, F, d = dims
        B = code.n_tokens
        out = torch.empty(L, B, d, dtype=torch.float32, device=acts2.device)
        for j in range(L):
            code_j = dataclasses.replace(code, row_nnz=prefix_t[j], d_sae=(j + 1) * F)
            out[j] = ops.sparse_decode_fwd(code_j, w_ops[j].view((j + 1) * F, d), None)
        ctx.code, ctx.prefix_t, ctx.dims, ctx.w_ops = code, prefix_t, dims, w_ops
        ctx.in_dtype, ctx.w_dtype = acts2.dtype, W_D[0].dtype
        return out

    @staticmethod
    def backward(ctx, g):
        L, F, d = ctx.dims
        code, prefix_t, w_ops = ctx.code, ctx.prefix_t, ctx.w_ops
        g = g.float().contiguous()
        d_acts = None
        if ctx.needs_input_grad[0]:
            dval = None
            for j in range(L):
                code_j = dataclasses.replace(code, row_nnz=prefix_t[j], d_sae=(j + 1) * F)
                dv = ops.sparse_decode_bwd_dval(code_j, g[j], w_ops[j].view((j + 1) * F, d))    # zero past the prefix
                dval = dv if dval is None else dval.add_(dv)
            d_acts = ops.code_to_dense(dataclasses.replace(code, val=dval), L * F)[0].to(ctx.in_dtype)
        dW = [None] * L
        if any(ctx.needs_input_grad[5:]):
            fi = ops.build_feature_index(code)
            for j in range(L):
                if ctx.needs_input_grad[5 + j]:
                    fi_j = ops.FeatureIndex(fi.feat_ptr[: (j + 1) * F + 1], fi.feat_slot, fi.slot_tok)
                    dW[j] = ops.sparse_grad_rows(fi_j, code.val, g[j], (j + 1) * F)[0].view(j + 1, F, d).to(ctx.w_dtype)
        return (d_acts, None, None, None, None, *dW)


@register_sae_model("clt")
class CrossLayerTranscoder(SparseDictionary):
    def __init__(self, cfg: CLTConfig, device_mesh=None):
        super().__init__(cfg, device_mesh=device_mesh)
        self.cfg = cfg
        L, d, F = cfg.n_layers, cfg.d_model, cfg.d_sae
        kw = dict(device=cfg.device, dtype=cfg.dtype)
        self.W_E = nn.Parameter(torch.empty(L, F, d, **kw).permute(0, 2, 1))   # shape [L, d, F], per-layer feature-major
        self.b_E = nn.Parameter(torch.empty(L, F, **kw))
        self.W_D = nn.ParameterList([nn.Parameter(torch.empty(i + 1, F, d, **kw)) for i in range(L)])
        self.b_D = nn.ParameterList([nn.Parameter(torch.empty(d, **kw)) for _ in range(L)])
        self._norm_cache: Optional[tuple[tuple[int, ...], torch.Tensor]] = None
        # set by an optimiser that consumes factored gradients (HipAdam): the fused backward then attaches them to
        # W_E / W_D[j] as `_sparse_grad` instead of writing dense gradient rows
        self.defer_weight_grads = False
        # `decode` of dense activations takes the sparse decoder kernels when they are sparse enough; False keeps the
        # dense products whatever the input
        self.sparse_api_decode = True

    # ---- activations (clt.py:232-387): the selection scope depends on the name ----
    def activation_function_factory(self, device_mesh=None):
        act = self.cfg.act_fn.lower()
        assert act in ["relu", "topk", "jumprelu", "batchtopk", "layertopk", "batchlayertopk"], (
            f"Not implemented activation function {self.cfg.act_fn}")
        if act == "relu":
            return lambda x: x * x.gt(0).to(x.dtype)
        if act == "jumprelu":
            return JumpReLU(self.cfg.jumprelu_threshold_window, shape=(self.cfg.n_layers, self.cfg.d_sae),
                            dims_to_keep_in_bwd=(-2, -1), device=self.cfg.device, dtype=self.cfg.dtype)
        if act == "topk":
            def topk_activation(x: torch.Tensor):
                if x.is_cuda:
                    return topk_dense(x, self.current_k)
                raise RuntimeError("the TopK activation runs on the GPU only (no CPU fallback in this build)")
            return topk_activation

        def scoped(x: torch.Tensor):
            # dense form of the wider scopes: positive part, then keep the k (or k * batch) largest of every
            # group; a group's members are flattened in the order the reference permutes them (selected dims last,
            # in the order named), so ties fall to the same element
            if x.is_cuda and x.ndim == 3 and x.shape[0] <= 131072:
                # the select kernels behind their dense-in / dense-out forms (lowest flattened index wins a tie, which is
                # the order of the arrangement each scope is handed over in)
                B, L, F = x.shape
                if act == "layertopk":
                    return topk_dense(x.reshape(B, L * F), self.current_k).view(B, L, F)
                if act == "batchtopk":
                    return torch.stack([batch_topk_dense(x[:, l, :].contiguous(), self.current_k * B) for l in range(L)], dim=1)
                flat = batch_topk_dense(x.permute(0, 2, 1).reshape(B, F * L), self.current_k * B)
                return flat.view(B, F, L).permute(0, 2, 1)
            r = x * x.gt(0).to(x.dtype)
            B, L, F = r.shape
            if act == "layertopk":
                groups, kk = r.reshape(B, L * F), self.current_k
            elif act == "batchtopk":
                groups, kk = r.permute(1, 0, 2).reshape(L, B * F), self.current_k * B
            else:  # batchlayertopk: dims (0, -1, -2) -> batch, feature, layer
                groups, kk = r.permute(0, 2, 1).reshape(1, B * F * L), self.current_k * B
            with torch.no_grad():
                mask = _topk_mask_lowest_index(groups, kk)
                if act == "layertopk":
                    mask = mask.view(B, L, F)
                elif act == "batchtopk":
                    mask = mask.view(L, B, F).permute(1, 0, 2)
                else:
                    mask = mask.view(B, F, L).permute(0, 2, 1)
            return r * mask.to(r.dtype)
        return scoped

    # ---- kernel operands ----
    def _w_enc_operand(self, amp: bool) -> torch.Tensor:
        wt = self.W_E.detach().permute(0, 2, 1)
        wt = wt if wt.is_contiguous() else wt.contiguous()
        if not amp or wt.dtype == torch.bfloat16:
            return wt
        L, d, F = self.cfg.n_layers, self.cfg.d_model, self.cfg.d_sae
        return self._derive("W_E.bf16", self.W_E, lambda old: ops.cast_bf16(
            wt.view(L * F, d), None if old is None else old.view(L * F, d))).view(L, F, d)

    def _w_dec_operands(self, amp: bool) -> list[torch.Tensor]:
        out = []
        for j, w in enumerate(self.W_D):
            wd = w.detach()
            if amp and wd.dtype != torch.bfloat16:
                F, d = self.cfg.d_sae, self.cfg.d_model
                wd = self._derive(f"W_D.{j}.bf16", w, lambda old, wd=wd, j=j: ops.cast_bf16(
                    wd.view((j + 1) * F, d), None if old is None else old.view((j + 1) * F, d))).view(j + 1, F, d)
            out.append(wd)
        return out

    def _norm_per_feature_nograd(self) -> torch.Tensor:
        """decoder_norm_per_feature() through the row-norm kernel, cached until a decoder group changes."""
        vers = tuple(w._version for w in self.W_D)
        if self._norm_cache is not None and self._norm_cache[0] == vers and self._norm_cache[1].device == self.W_D[0].device:
            return self._norm_cache[1]
        L, d, F = self.cfg.n_layers, self.cfg.d_model, self.cfg.d_sae
        with torch.no_grad():
            sq = torch.zeros(L, F, dtype=torch.float32, device=self.W_D[0].device)
            for j, w in enumerate(self.W_D):
                # the optimiser's row pass leaves a group's row norms behind; otherwise one pass of the row-norm kernel
                n = self._derive(f"W_D.{j}.norm", w, lambda old, w=w, j=j: ops.row_norm(
                    w.detach().float().view((j + 1) * F, d), old)).view(j + 1, F)
                sq[: j + 1] += n * n
            norms = sq.sqrt_()
        self._norm_cache = (vers, norms)
        return norms

    # ---- norms (clt.py:801-907) ----
    def decoder_norm(self, keepdim: bool = False):
        return torch.ones(self.cfg.n_decoders, device=self.W_E.device, dtype=self.cfg.dtype)

    def encoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_E, p=2, dim=1, keepdim=keepdim)

    def decoder_bias_norm(self):
        return torch.ones(self.cfg.n_layers, device=self.W_E.device, dtype=self.cfg.dtype)

    @torch.no_grad()
    def decoder_norm_per_feature(self, layer: Optional[int] = None) -> torch.Tensor:
        L, F = self.cfg.n_layers, self.cfg.d_sae
        norms = torch.zeros(L, F, dtype=self.cfg.dtype, device=self.W_E.device)
        if layer is not None:
            for layer_to in range(layer, L):
                norms[layer_to] = self.W_D[layer_to][layer].pow(2).sum(dim=-1).sqrt()
            return norms
        for layer_to, w in enumerate(self.W_D):
            norms[: layer_to + 1] = norms[: layer_to + 1] + w.pow(2).sum(dim=-1)
        return norms.sqrt()

    @torch.no_grad()
    def decoder_norm_per_decoder(self) -> torch.Tensor:
        return torch.cat([torch.norm(w, p=2, dim=(1, 2)) for w in self.W_D])

    def get_decoder_weights(self, layer_to: int) -> torch.Tensor:
        return self.W_D[layer_to]

    @torch.no_grad()
    def init_parameters(self, **kwargs):
        """clt.py:390-467: encoders U(+-1/sqrt(F)), every decoder U(+-1/sqrt(L d)), zero biases."""
        super().init_parameters(**kwargs)
        eb = 1.0 / math.sqrt(self.cfg.d_sae)
        db = 1.0 / math.sqrt(self.cfg.n_layers * self.cfg.d_model)
        self.W_E.uniform_(-eb, eb)
        self.b_E.zero_()
        for w in self.W_D:
            w.uniform_(-db, db)
            if self.cfg.init_cross_layer_decoder_all_zero:
                w[:-1] = 0
        for b in self.b_D:
            b.zero_()

    @torch.no_grad()
    def standardize_parameters_of_dataset_norm(self):
        """clt.py:908-937: fold the per-layer dataset norms into the parameters so that raw activations can be fed.
        With fin(l) = sqrt(d) / norm_in(l) and fout(l) = sqrt(d) / norm_out(l): the encoder weights stay, the encoder
        bias (and a JumpReLU threshold) of layer l is divided by fin(l) (features come out in raw-input units),
        W_D[layer_to][layer_from] is multiplied by fin(layer_from) / fout(layer_to) and b_D[layer_to] is divided by
        fout(layer_to).  In-place operations on the parameters themselves (not on `.data`), so the version counters
        move and cached bf16 copies / norms are rebuilt on their next use."""
        assert self.cfg.norm_activation == "dataset-wise"
        assert self.dataset_average_activation_norm is not None
        norms = self.dataset_average_activation_norm
        fin = lambda l: math.sqrt(self.cfg.d_model) / norms[self.cfg.hook_points_in[l]]    # noqa: E731
        fout = lambda l: math.sqrt(self.cfg.d_model) / norms[self.cfg.hook_points_out[l]]  # noqa: E731
        for layer_from in range(self.cfg.n_layers):
            self.b_E[layer_from].div_(fin(layer_from))
            if self.cfg.act_fn.lower() == "jumprelu":
                log_thr = self.activation_function.log_jumprelu_threshold
                log_thr[layer_from] = torch.log(log_thr[layer_from].exp() / fin(layer_from))
        for layer_to in range(self.cfg.n_layers):
            self.b_D[layer_to].div_(fout(layer_to))
            for layer_from in range(layer_to + 1):
                self.W_D[layer_to][layer_from].mul_(fin(layer_from) / fout(layer_to))
        self.cfg.norm_activation = "inference"

    # ---- API path over dense tensors (clt.py:527-709) ----
    def _layer_products(self, x: torch.Tensor) -> torch.Tensor:
        """einsum("...ld,lds->...ls", x, W_E) (clt.py:559): the GEMM kernel layer by layer on GPU tensors whose shapes it
        takes, the library routine otherwise."""
        L, d, F = self.cfg.n_layers, self.cfg.d_model, self.cfg.d_sae
        amp = _autocast_dtype("cuda") == torch.bfloat16
        low = amp or self.W_E.dtype == torch.bfloat16
        if (x.is_cuda and self.W_E.is_cuda and tuple(x.shape[-2:]) == (L, d) and self.W_E.dtype in (torch.float32, torch.bfloat16)
                and _gemm_k_ok(d, torch.bfloat16 if low else torch.float32)):
            lead = x.shape[:-2]
            pre = _LayerEncoderGemm.apply(x.reshape(-1, L, d).to(self.W_E.dtype), self.W_E, self._w_enc_operand(amp), low)
            return pre.reshape(*lead, L, F)
        return torch.einsum("...ld,lds->...ls", x, self.W_E)

    def encode(self, x: torch.Tensor, return_hidden_pre: bool = False, **kwargs):
        hidden_pre = self._layer_products(x) + self.b_E
        if self.cfg.sparsity_include_decoder_norm:
            hidden_pre = hidden_pre * self.decoder_norm_per_feature()
        feature_acts = self.activation_function(hidden_pre)
        if self.cfg.sparsity_include_decoder_norm:
            feature_acts = feature_acts / self.decoder_norm_per_feature()
        return (feature_acts, hidden_pre) if return_hidden_pre else feature_acts

    def decode(self, feature_acts: torch.Tensor, batch_first: bool = False, **kwargs):
        """feature_acts [.., L, F] -> [L, .., d] (clt.py:630-709).  Activations that are sparse enough (at most
        cfg.sparsity_threshold_for_csr of the entries non-zero: the reference's own bound for its sparse decode, counted on
        the device and read once) become one sparse code over the L F concatenated features and every output layer is a
        sparse decode of its per-token prefix, with a sparse backward.  Denser activations take one 2-D product per
        output layer, [.., (j + 1) F] x [(j + 1) F, d] (the reference's batched product over a permuted view, followed by a
        sum over the source layers, is the same sum; a library batched bf16 product over such a view returned wrong
        weight gradients for source layer 0 at 12 layers x 12288 features)."""
        L, d, F = self.cfg.n_layers, self.cfg.d_model, self.cfg.d_sae
        lead = feature_acts.shape[:-2]
        acts2 = feature_acts.reshape(-1, L * F)
        out = None
        if (self._sparse_decode_allowed(feature_acts) and tuple(feature_acts.shape[-2:]) == (L, F) and d % 8 == 0
                and self.W_D[0].dtype in (torch.float32, torch.bfloat16) and acts2.shape[0] <= 131072):
            src = (acts2 if acts2.dtype in (torch.float32, torch.bfloat16) else acts2.float()).contiguous()
            code = ops.dense_to_code(src, max_entries=int(self.cfg.sparsity_threshold_for_csr * src.numel()))
            if code is not None:
                amp = _autocast_dtype("cuda") == torch.bfloat16
                prefix_t = torch.cumsum(layer_counts(code, L, F), dim=1).to(torch.int32).t().contiguous()    # [L, B]
                out = _PrefixDecode.apply(acts2, code, prefix_t, (L, F, d), self._w_dec_operands(amp), *self.W_D)
                out = out + torch.stack(list(self.b_D)).unsqueeze(1)
        if out is None:
            amp = _autocast_dtype("cuda") == torch.bfloat16
            w_ops = self._w_dec_operands(amp) if feature_acts.is_cuda else None
            outs = []
            for j in range(L):
                part = None
                if w_ops is not None:   # the GEMM kernel on the layers' prefix (bf16 operands read W_D[j] as it lies)
                    part = dense_decode(self, acts2[:, : (j + 1) * F], self.W_D[j].view((j + 1) * F, d),
                                        w_ops[j].view((j + 1) * F, d), f"W_D.{j}.t.f32")
                if part is None:
                    part = acts2[:, : (j + 1) * F] @ self.W_D[j].view((j + 1) * F, d)
                outs.append(part + self.b_D[j])
            out = torch.stack(outs)
        out = out.view(L, *lead, d)
        return out.movedim(0, -2) if batch_first else out

    def prepare_input(self, batch: dict[str, torch.Tensor], **kwargs) -> tuple[torch.Tensor, dict[str, Any], dict[str, Any]]:
        xs = []
        for hp in self.cfg.hook_points_in:
            if hp not in batch:
                raise ValueError(f"Missing hook point {hp} in batch")
            xs.append(batch[hp])
        return torch.stack(xs, dim=xs[0].ndim - 1), {}, {}

    def prepare_label(self, batch: dict[str, torch.Tensor], **kwargs) -> torch.Tensor:
        ys = []
        for hp in self.cfg.hook_points_out:
            if hp not in batch:
                raise ValueError(f"Missing hook point {hp} in batch")
            ys.append(batch[hp])
        return torch.stack(ys, dim=0)

    # ---- loss (clt.py:1024-1104) ----
    def _fused_eligible(self, x, sparsity_loss_type) -> bool:
        amp = _autocast_dtype("cuda") == torch.bfloat16
        return (self.cfg.act_fn.lower() in _TOPK_FAMILY and x.is_cuda and x.ndim == 3 and sparsity_loss_type is None
                and self.W_E.dtype == torch.float32 and self.cfg.d_model % (64 if amp else 32) == 0)

    # ---- JumpReLU / ReLU: the activation on the threshold kernels, layer by layer ([L, F] thresholds, clt.py:247-257) ----
    def _threshold_kernels_eligible(self, x, sparsity_loss_type) -> bool:
        amp = _autocast_dtype("cuda") == torch.bfloat16
        return (self.cfg.act_fn.lower() in ("jumprelu", "relu") and x.is_cuda and x.ndim == 3 and self.W_E.dtype == torch.float32
                and self.cfg.d_sae % 8 == 0 and self.cfg.d_model % (64 if amp else 32) == 0
                and sparsity_loss_type in (None, "tanh", "power", "tanh-quad"))

    def _threshold_activations(self, x: torch.Tensor, want_tanh: bool, tanh_c: float):
        """encode() for a JumpReLU or ReLU transcoder with the element-wise part on `sae_jumprelu_fwd / bwd`: the L encoder
        products land in one [L, B, F] buffer, and each layer's slice takes one pass that adds the bias, scales by the
        per-feature decoder norms (constants: the reference computes them without gradient, clt.py:836), applies the
        layer's thresholds, divides again and, if asked, sums the tanh penalty per token; the backward pass is one kernel
        per layer as well (pre-activation, bias and threshold gradients).  -> (feature_acts [B, L, F], tanh sums [B, L] or
        None)."""
        from .sae import _JumpReLUStep

        L, d, F = self.cfg.n_layers, self.cfg.d_model, self.cfg.d_sae
        amp = _autocast_dtype("cuda") == torch.bfloat16
        pre = _LayerEncoderGemm.apply(x.to(self.W_E.dtype), self.W_E, self._w_enc_operand(amp), amp).permute(1, 0, 2)   # [L, B, F]
        scaled = bool(self.cfg.sparsity_include_decoder_norm)
        norms = self._norm_per_feature_nograd() if (scaled or want_tanh) else None
        if self.cfg.act_fn.lower() == "jumprelu":
            theta, window = self.activation_function.get_jumprelu_threshold(), float(self.activation_function.jumprelu_threshold_window)
        else:
            theta, window = torch.zeros(L, F, dtype=torch.float32, device=x.device), 1.0
        acts, pens = [], []
        for l in range(L):
            a, t, _ = _JumpReLUStep.apply(pre[l], self.b_E[l], None if norms is None else norms[l], theta[l], scaled, tanh_c, window,
                                          want_tanh, False)
            acts.append(a)
            pens.append(t)
        feature_acts = torch.stack(acts, dim=1)
        return feature_acts, (torch.stack(pens, dim=1) if want_tanh else None)

    def compute_loss(self, batch, label=None, *, sparsity_loss_type=None, tanh_stretch_coefficient: float = 4.0,
                     frequency_scale: float = 0.01, p: int = 1, l1_coefficient: float = 1.0, return_aux_data: bool = True,
                     **kwargs):
        x, enc_kw, dec_kw = self.prepare_input(batch)
        label = self.prepare_label(batch, **kwargs)
        mask = batch.get("mask")
        n_tokens = (lambda: batch["tokens"].numel()) if mask is None else (lambda: int(mask.sum().item()))
        if self._fused_eligible(x, sparsity_loss_type):
            amp = _autocast_dtype("cuda") == torch.bfloat16
            holder: dict[str, Any] = {"model": self, "defer": self.defer_weight_grads and torch.is_grad_enabled()}
            xin = x.to(torch.float32) if x.dtype not in (torch.float32, torch.bfloat16) else x
            loss, recon = _FusedCLTStep.apply(xin, label.to(torch.float32), amp, holder, self.W_E, self.b_E,
                                              *self.W_D, *self.b_D)
            if not return_aux_data:
                return loss
            B, L, F = x.shape[0], self.cfg.n_layers, self.cfg.d_sae
            eager = {"loss": loss, "l_rec": loss, "l_s": None, "label": label, "mask": mask, "reconstructed": recon,
                     "sparse_code": holder["code"]}
            lazy = {"n_tokens": n_tokens, "feature_acts": lambda: holder["code"].to_dense().view(B, L, F)}
            return LazyDict(eager, lazy)

        feature_acts = tanh_pen = None
        if self._threshold_kernels_eligible(x, sparsity_loss_type):
            feature_acts, tanh_pen = self._threshold_activations(x, sparsity_loss_type == "tanh", float(tanh_stretch_coefficient))
        else:
            feature_acts = self.encode(x, **enc_kw)
        reconstructed = self.decode(feature_acts, **dec_kw)
        l_rec = (reconstructed - label).pow(2).sum(dim=-1).mean()
        loss_dict: dict[str, Optional[torch.Tensor]] = {"l_rec": l_rec}
        loss = l_rec
        if sparsity_loss_type is not None:
            n = self.decoder_norm_per_feature()
            if sparsity_loss_type == "power":
                l_s = torch.norm(feature_acts * n, p=p, dim=-1)
            elif sparsity_loss_type == "tanh":
                l_s = tanh_pen if tanh_pen is not None else torch.tanh(tanh_stretch_coefficient * feature_acts * n).sum(dim=-1)
            elif sparsity_loss_type == "tanh-quad":
                t = torch.tanh(tanh_stretch_coefficient * feature_acts * n)
                freq = t.mean(dim=tuple(range(t.ndim - 1)))
                l_s = (freq * (1 + freq / frequency_scale)).sum(dim=-1)
            else:
                raise ValueError(f"sparsity_loss_type f{sparsity_loss_type} not supported.")
            l_s = l1_coefficient * l_s
            loss_dict["l_s"] = l_s
            loss = loss + l_s.mean()
        else:
            loss_dict["l_s"] = None
        if not return_aux_data:
            return loss
        return {"loss": loss, **loss_dict, "label": label, "mask": mask, "n_tokens": n_tokens(),
                "feature_acts": feature_acts, "reconstructed": reconstructed}
