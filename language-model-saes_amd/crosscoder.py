"""Crosscoder on the HIP path.

API of the reference's crosscoder (src/llamascopium/models/crosscoder.py:84-716): one encoder /
decoder pair per head (hook point), parameters `W_E [H, d, F]`, `b_E [H, F]`, `W_D [H, F, d]`,
`b_D [H, d]`.  The per-head encodings are summed into one shared pre-activation, every head then
applies the activation to that sum scaled by ITS OWN decoder norms, and decodes with its own
decoder.

Memory layout: `W_E` has the reference's shape but is stored feature-major (a permuted view of a
contiguous [F, H, d] buffer), so the head-summed encoding is ONE GEMM over the concatenated model
axis, x [B, H*d] @ [F, H*d]^T, on the same kernel as the plain SAE.  The per-head TopK then runs the
select kernel H times over that one pre-activation with H different scale vectors, and each head's
decode / loss / gradient rows use the sparse kernels with `W_D[h]`.
"""

from __future__ import annotations

import dataclasses
import math
from functools import reduce
from typing import Any, Optional

import torch
from torch import nn

from . import ops
from .config import CrosscoderConfig, register_sae_model
from .sae import SparseRowGrad, _autocast_dtype
from .sparse_dictionary import LazyDict, SparseDictionary


class _FusedCrosscoderStep(torch.autograd.Function):
    """GEMM over the concatenated heads -> per-head TopK select -> per-head sparse decode + squared error,
    forward and backward in kernels; no dense [B, H, F] tensor is formed.

    d loss / d pre[b, f] is the sum over heads of the kept entries' value gradients (act(h n)/n has unit
    slope on kept entries, and the two derivative terms with respect to n cancel), so `W_E`'s gradient is
    one pass of the gradient-row kernel over the H codes stacked on a virtual token axis whose tokens map
    back to the same B rows of x.
    """

    @staticmethod
    def forward(ctx, x, label, tok_w, W_E, b_E, W_D, b_D, k, amp, holder):
        m: "Crosscoder" = holder["model"]
        B, H, d = x.shape
        F = m.cfg.d_sae
        w_enc_op = m._w_enc_operand(amp)                              # [F, H*d]
        x_cat = x.reshape(B, H * d)
        if amp:
            x_op = x_cat if x_cat.dtype == torch.bfloat16 else ops.cast_bf16(x_cat.contiguous())
            pre = ops.encoder_gemm(x_op, w_enc_op, torch.bfloat16)
        else:
            x_op = x_cat.contiguous()
            pre = ops.encoder_gemm(x_op, w_enc_op, torch.float32)
        norms = m._decoder_norm_nograd()                              # [H, F]
        w_dec_op = m._w_dec_operand(amp)                              # [H, F, d]
        b_sum = b_E.detach().sum(dim=0)
        codes = []
        stacked = None
        # head-major copies of the per-token operands (one launch each instead of one per head), and one buffer per output
        # of the H decodes: reconstructions, output gradients, value gradients, per-token losses
        label_h = label.transpose(0, 1).contiguous()                     # [H, B, d]
        tokw_h = tok_w.t().contiguous()                                  # [H, B]
        b_D_h = b_D.detach().contiguous()
        recons = torch.empty(H, B, d, dtype=torch.float32, device=x.device)
        grads = torch.empty(H, B, d, dtype=torch.float32, device=x.device)
        loss_toks = torch.empty(H, B, dtype=torch.float32, device=x.device)
        dvals = []
        if (amp and pre.dtype == torch.bfloat16 and getattr(m, "granule_select", True) and ops.granule_route_supported(64, F, int(k))):
            # every head selects from the same summed encoding under its own decoder norms: ONE pass for the per-granule key
            # maxima of the H * B (head, token) rows and ONE select over them, each row reading only the granules that can
            # hold a kept entry, instead of H walks over whole rows; the rows come out head after head, which is the stacked
            # code the backward wants
            b_rep = b_sum.float().expand(H, F).contiguous()
            n_rep = norms.contiguous()
            gmax = ops.granule_max(pre, b_rep, n_rep, rows_per_group=B, n_rows=H * B)
            stacked = ops.select_topk_row(pre, b_rep, n_rep, k, granule_max=gmax, rows_per_group=B, n_rows=H * B)
        for h in range(H):
            if stacked is not None:
                sl, rows = slice(h * B * k, (h + 1) * B * k), slice(h * B, (h + 1) * B)
                code = ops.SparseCode(stacked.idx[sl], stacked.val[sl], stacked.row_off[rows] - h * B * k, stacked.row_nnz[rows], B, F)
            else:
                code = ops.select_topk_row(pre, b_sum, norms[h], k)
            _, _, _, dval = ops.sparse_decode_mse_fused(code, w_dec_op[h], b_D_h[h], label_h[h], tokw_h[h], recon_out=recons[h],
                                                        loss_out=loss_toks[h], grad_out=grads[h])
            codes.append(code); dvals.append(dval)
        loss = loss_toks.sum()
        recon = recons.transpose(0, 1)                                   # [B, H, d]
        holder["codes"], holder["pre"], holder["norms"], holder["b_sum"] = codes, pre, norms, b_sum
        ctx.codes, ctx.grads, ctx.dvals, ctx.x_op, ctx.w_enc_op = codes, grads, dvals, x_op, w_enc_op
        ctx.stacked = stacked
        ctx.amp = bool(amp)
        ctx.shape = (B, H, d, F)
        ctx.defer_to = m if holder.get("defer") else None
        ctx.mark_non_differentiable(recon)
        return loss, recon

    @staticmethod
    def backward(ctx, g_loss, _g_recon):
        B, H, d, F = ctx.shape
        g = g_loss.to(torch.float32)
        m = ctx.defer_to
        defer = (m is not None and all(w.grad is None and getattr(w, "_sparse_grad", None) is None for w in (m.W_E, m.W_D)))
        db_D = ctx.grads.sum(dim=1) * g                                  # [H, d]
        # the H codes on a virtual token axis: token h * B + b
        stacked = ctx.stacked if ctx.stacked is not None else reduce(ops.stack_codes, ctx.codes)
        coef = torch.cat(ctx.dvals) * g
        k = stacked.idx.numel() // (H * B)
        if stacked.idx.numel() == H * B * k and H * k <= 1024:
            # the heads keep nearly the same features of a token (one encoding, H sets of norms): every (token, feature) once,
            # with the heads' value gradients summed, so that the encoder's gradient rows gather a row of x once per pair
            # instead of once per head
            merged = ops.union_group_codes(dataclasses.replace(stacked, val=coef), H)
            fi, coef = ops.build_feature_index(merged), merged.val
        else:
            fi = ops.build_feature_index(stacked)
            fi = dataclasses.replace(fi, slot_tok=torch.remainder(fi.slot_tok, B).to(torch.int32))  # virtual token h*B + b -> row b of x
        if ctx.amp:
            # the decoder's weight gradient pairs the activations with the bf16-rounded output gradient, as the backward of
            # an autocast product does; the gathered rows then move half the bytes
            gd = ops.cast_bf16(ctx.grads.view(H * B, d))
        else:
            gd = ctx.grads.view(H * B, d)
        if defer:
            # The optimiser rebuilds the rows where it consumes them; nothing dense is written here.  The decoder
            # [H, F, d] is one matrix of H F rows: head h's code addresses rows h F .. (h + 1) F of it, and its dense
            # operand is head h's block of the stacked output gradients.
            idx_cat = torch.cat([c.idx + h * F for h, c in enumerate(ctx.codes)])
            cat_code = dataclasses.replace(stacked, idx=idx_cat, d_sae=H * F)
            m.W_D._sparse_grad = SparseRowGrad(ops.build_feature_index(cat_code), stacked.val * g, gd, H * F)
            m.W_E._sparse_grad = SparseRowGrad(fi, coef, ctx.x_op, F)
            db_sum, _ = ops.feature_segment_sums(fi, coef)
            dW_E = dW_D = None
        else:
            dW_D = []
            for h in range(H):
                fi_h = ops.build_feature_index(ctx.codes[h])
                rows, _ = ops.sparse_grad_rows(fi_h, ctx.codes[h].val * g, gd[h * B:(h + 1) * B], F)
                dW_D.append(rows)
            dW_D = torch.stack(dW_D)
            dW_Et, db_sum = ops.sparse_grad_rows(fi, coef, ctx.x_op, F, want_bias=True)                # [F, H*d], [F]
            dW_E = dW_Et.view(F, H, d).permute(1, 2, 0)
        db_E = db_sum.unsqueeze(0).expand(H, F)
        dx = dlabel = None
        if ctx.needs_input_grad[0]:
            parts = [ops.sparse_decode_fwd(dataclasses.replace(c, val=dv * g), ctx.w_enc_op, None)
                     for c, dv in zip(ctx.codes, ctx.dvals)]
            dx = reduce(torch.add, parts).view(B, H, d)
        if ctx.needs_input_grad[1]:
            dlabel = -ctx.grads.transpose(0, 1) * g
        return dx, dlabel, None, dW_E, db_E, dW_D, db_D, None, None, None


@register_sae_model("crosscoder")
class Crosscoder(SparseDictionary):
    def __init__(self, cfg: CrosscoderConfig, device_mesh=None):
        super().__init__(cfg, device_mesh=device_mesh)
        self.cfg = cfg
        assert cfg.sparsity_include_decoder_norm, "Sparsity should include decoder norm in Crosscoder"
        assert cfg.use_decoder_bias, "Decoder bias should be used in Crosscoder"
        H, d, F = cfg.n_heads, cfg.d_model, cfg.d_sae
        kw = dict(device=cfg.device, dtype=cfg.dtype)
        self.W_E = nn.Parameter(torch.empty(F, H, d, **kw).permute(1, 2, 0))   # shape [H, d, F], feature-major storage
        self.b_E = nn.Parameter(torch.empty(H, F, **kw))
        self.W_D = nn.Parameter(torch.empty(H, F, d, **kw))
        self.b_D = nn.Parameter(torch.empty(H, d, **kw))
        # set by an optimiser that consumes factored gradients (HipAdam): the weight gradients are then attached to the
        # parameters as `_sparse_grad` instead of being written as dense rows
        self.defer_weight_grads = False
        # `decode` of dense activations takes the sparse decoder kernels when they are sparse enough; False keeps the
        # reference's dense product whatever the input
        self.sparse_api_decode = True

    # ---- kernel operands ----
    def _w_enc_operand(self, amp: bool) -> torch.Tensor:
        H, d, F = self.cfg.n_heads, self.cfg.d_model, self.cfg.d_sae
        wt = self.W_E.detach().permute(2, 0, 1)
        wt = (wt if wt.is_contiguous() else wt.contiguous()).view(F, H * d)
        if not amp or wt.dtype == torch.bfloat16:
            return wt
        return self._derive("W_E.bf16", self.W_E, lambda old: ops.cast_bf16(wt, old))

    def _w_dec_operand(self, amp: bool) -> torch.Tensor:
        w = self.W_D.detach()
        if not amp or w.dtype == torch.bfloat16:
            return w
        H, d, F = self.cfg.n_heads, self.cfg.d_model, self.cfg.d_sae
        return self._derive("W_D.bf16", self.W_D, lambda old: ops.cast_bf16(
            w.view(H * F, d), None if old is None else old.view(H * F, d))).view(H, F, d)

    def _decoder_norm_nograd(self) -> torch.Tensor:
        H, d, F = self.cfg.n_heads, self.cfg.d_model, self.cfg.d_sae
        return self._derive("W_D.norm", self.W_D, lambda old: ops.row_norm(
            self.W_D.detach().float().view(H * F, d), None if old is None else old.view(H * F))).view(H, F)

    # ---- norms (crosscoder.py:471-520) ----
    def decoder_norm(self, keepdim: bool = False) -> torch.Tensor:
        return torch.norm(self.W_D, dim=-1, keepdim=keepdim)

    def encoder_norm(self, keepdim: bool = False) -> torch.Tensor:
        return torch.norm(self.W_E, dim=-2, keepdim=keepdim)

    def decoder_bias_norm(self) -> torch.Tensor:
        return torch.norm(self.b_D, dim=-1, keepdim=True)

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
        raise NotImplementedError("Transform to unit decoder norm is not supported for Crosscoder")

    @torch.no_grad()
    def standardize_parameters_of_dataset_norm(self):
        """crosscoder.py:521-538: only the biases are rescaled (input and output share a hook point)."""
        assert self.cfg.norm_activation == "dataset-wise"
        assert self.dataset_average_activation_norm is not None
        f = torch.tensor([math.sqrt(self.cfg.d_model) / self.dataset_average_activation_norm[hp] for hp in self.cfg.hook_points],
                         dtype=self.cfg.dtype, device=self.b_E.device)
        self.b_E.div_(f.view(self.cfg.n_heads, 1))
        self.b_D.div_(f.view(self.cfg.n_heads, 1))
        self.cfg.norm_activation = "inference"

    @torch.no_grad()
    def init_encoder_with_decoder_transpose(self, factor: float = 1.0):
        self.W_E.copy_(self.W_D.transpose(1, 2) * factor)

    @torch.no_grad()
    def init_parameters(self, **kwargs) -> None:
        """crosscoder.py:160-219: one head's uniform weights repeated for every head, zero biases."""
        super().init_parameters(**kwargs)
        eb, db = kwargs["encoder_uniform_bound"], kwargs["decoder_uniform_bound"]
        d, F = self.cfg.d_model, self.cfg.d_sae
        kw = dict(device=self.W_E.device, dtype=self.cfg.dtype)
        self.W_E.copy_(torch.empty(d, F, **kw).uniform_(-eb, eb).expand(self.cfg.n_heads, d, F))
        self.W_D.copy_(torch.empty(F, d, **kw).uniform_(-db, db).expand(self.cfg.n_heads, F, d))
        self.b_E.zero_()
        self.b_D.zero_()

    @torch.no_grad()
    def decoder_inner_product_matrices(self) -> torch.Tensor:
        return torch.einsum("isd,jsd->sij", self.W_D, self.W_D)

    @torch.no_grad()
    def decoder_similarity_matrices(self) -> torch.Tensor:
        n = self.decoder_norm()
        return self.decoder_inner_product_matrices() / torch.einsum("is,js->sij", n, n)

    # ---- API path over dense tensors (crosscoder.py:221-469) ----
    def _summed_encoding(self, x: torch.Tensor) -> torch.Tensor:
        """sum_h (x_h @ W_E[h] + b_E[h]) [.., F] (crosscoder.py:222-275, 353-375): on GPU tensors ONE product of the GEMM
        kernel over the concatenated model axis (K = H d, fp32 accumulation over all heads, one rounding under autocast
        where the reference rounds every head's product), whose weight gradient is a product over the token axis on
        the same kernel; the reference's op sequence otherwise."""
        H, d, F = self.cfg.n_heads, self.cfg.d_model, self.cfg.d_sae
        amp = _autocast_dtype("cuda") == torch.bfloat16
        low = amp or self.W_E.dtype == torch.bfloat16
        if (x.is_cuda and self.W_E.is_cuda and tuple(x.shape[-2:]) == (H, d) and self.W_E.dtype in (torch.float32, torch.bfloat16)
                and (H * d) % (64 if low else 32) == 0):
            from .sae import _EncoderGemm

            lead = x.shape[:-2]
            pre = _EncoderGemm.apply(x.reshape(-1, H * d).to(self.W_E.dtype), self.W_E, self._w_enc_operand(amp), low, False, None,
                                     lambda rows: rows.view(F, H, d).permute(1, 2, 0))
            return pre.view(*lead, F) + self.b_E.sum(dim=0)
        return (torch.einsum("...hd,hdf->...hf", x, self.W_E) + self.b_E).sum(dim=-2)

    def encode(self, x: torch.Tensor, return_hidden_pre: bool = False, **kwargs):
        H, F = self.cfg.n_heads, self.cfg.d_sae
        acc = self._summed_encoding(x)
        acc = acc.unsqueeze(-2).expand(*acc.shape[:-1], H, F)
        n = self.decoder_norm()
        feature_acts = self.activation_function(acc * n) / n
        return (feature_acts, acc) if return_hidden_pre else feature_acts

    def decode(self, feature_acts: torch.Tensor, **kwargs):
        """feature_acts [.., H, F] -> [.., H, d] (crosscoder.py:384-469).  Activations that are sparse enough (at most
        1 - cfg.sparsity_threshold_for_triton_spmm_kernel of the entries non-zero, counted on the device and read once, as
        the SAE's gate reads `max_l0`) go through the sparse decoder kernels, every head at once: row (token, head) of the
        activations gathers its rows from head h's block of W_D [H F, d]; its backward is the sparse one as well."""
        H, d, F = self.cfg.n_heads, self.cfg.d_model, self.cfg.d_sae
        if (self._sparse_decode_allowed(feature_acts) and tuple(feature_acts.shape[-2:]) == (H, F) and d % 8 == 0
                and self.W_D.dtype in (torch.float32, torch.bfloat16) and feature_acts.numel() < 2 ** 40):
            from .kernels import sparse_decode_blocks

            amp = _autocast_dtype("cuda") == torch.bfloat16
            lead = feature_acts.shape[:-2]
            out = sparse_decode_blocks(feature_acts.reshape(-1, F), self.W_D.view(H * F, d), self._w_dec_operand(amp).view(H * F, d),
                                       n_blocks=H, max_density=1.0 - self.cfg.sparsity_threshold_for_triton_spmm_kernel)
            if out is not None:
                return out.view(*lead, H, d) + self.b_D
        if feature_acts.is_cuda and tuple(feature_acts.shape[-2:]) == (H, F):
            # denser activations: one product of the GEMM kernel per head (bf16 operands read W_D[h] as it lies)
            from .sae import dense_decode

            amp = _autocast_dtype("cuda") == torch.bfloat16
            w_op = self._w_dec_operand(amp)
            fa = feature_acts.reshape(-1, H, F)
            outs = [dense_decode(self, fa[:, h], self.W_D[h], w_op[h], f"W_D.{h}.t.f32") for h in range(H)]
            if all(o is not None for o in outs):
                return torch.stack(outs, dim=1).view(*feature_acts.shape[:-2], H, d) + self.b_D
        return torch.einsum("...hf,hfd->...hd", feature_acts, self.W_D) + self.b_D

    def prepare_input(self, batch: dict[str, torch.Tensor], **kwargs) -> tuple[torch.Tensor, dict[str, Any], dict[str, Any]]:
        def pad_to_d_model(x: torch.Tensor) -> torch.Tensor:
            if x.shape[-1] > self.cfg.d_model:
                raise ValueError(f"Input tensor has {x.shape[-1]} dimensions, but expected {self.cfg.d_model}.")
            if x.shape[-1] < self.cfg.d_model:
                return torch.nn.functional.pad(x, (0, self.cfg.d_model - x.shape[-1]))
            return x
        return torch.stack([pad_to_d_model(batch[hp]) for hp in self.cfg.hook_points], dim=-2), {}, {}

    def prepare_label(self, batch: dict[str, torch.Tensor], **kwargs) -> torch.Tensor:
        return self.prepare_input(batch)[0]

    # ---- fused train-step loss ----
    def _fused_eligible(self, x, sparsity_loss_type, lp_coefficient, auxk_coefficient) -> bool:
        K = self.cfg.n_heads * self.cfg.d_model
        amp = _autocast_dtype("cuda") == torch.bfloat16
        return (
            self.cfg.act_fn.lower() == "topk" and x.is_cuda and x.ndim == 3
            and sparsity_loss_type is None and not (lp_coefficient > 0.0) and not (auxk_coefficient > 0.0)
            and self.W_E.dtype == torch.float32 and K % (64 if amp else 32) == 0 and self.cfg.d_model % 4 == 0
        )

    def compute_loss(self, batch, label=None, *, sparsity_loss_type=None, lp_coefficient: float = 0.0,
                     auxk_coefficient: float = 0.0, l1_coefficient: float = 1.0, return_aux_data: bool = True, **kwargs):
        x, _, _ = self.prepare_input(batch)
        if not self._fused_eligible(x, sparsity_loss_type, lp_coefficient, auxk_coefficient):
            return super().compute_loss(batch, sparsity_loss_type=sparsity_loss_type, lp_coefficient=lp_coefficient,
                                        auxk_coefficient=auxk_coefficient, l1_coefficient=l1_coefficient,
                                        return_aux_data=return_aux_data, **kwargs)
        label = x
        mask = batch.get("mask")
        B, H, _ = x.shape
        if mask is None:
            tok_w = torch.full((B, H), 1.0 / (B * H), dtype=torch.float32, device=x.device)
        else:
            assert tuple(mask.shape) == (B, H), f"Mask has shape {tuple(mask.shape)}, but input tensor has token part of shape {(B, H)}"
            mf = mask.to(torch.float32)
            tok_w = mf / mf.sum()
        amp = _autocast_dtype("cuda") == torch.bfloat16
        holder: dict[str, Any] = {"model": self, "defer": self.defer_weight_grads and torch.is_grad_enabled()}
        xin = x.to(torch.float32) if x.dtype not in (torch.float32, torch.bfloat16) else x
        loss, recon = _FusedCrosscoderStep.apply(xin.contiguous(), label.to(torch.float32).contiguous(), tok_w, self.W_E,
                                                 self.b_E, self.W_D, self.b_D, int(self.current_k), amp, holder)
        if not return_aux_data:
            return loss

        def dense_acts():
            return torch.stack([c.to_dense() for c in holder["codes"]], dim=1)

        def dense_hidden_pre():
            h0 = holder["pre"].float() + holder["b_sum"]
            return h0.unsqueeze(1).expand(B, H, h0.shape[-1])

        eager = {"loss": loss, "l_rec": loss, "l_s": None, "l_p": None, "l_aux": None, "label": label, "mask": mask,
                 "reconstructed": recon, "l1_coefficient": l1_coefficient, "lp_coefficient": lp_coefficient,
                 "auxk_coefficient": auxk_coefficient, "sparse_codes": holder["codes"]}
        lazy = {"n_tokens": (lambda: batch["tokens"].numel()) if mask is None else (lambda: int(mask.sum().item())),
                "feature_acts": dense_acts, "hidden_pre": dense_hidden_pre}
        return LazyDict(eager, lazy)
