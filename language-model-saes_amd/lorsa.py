"""Low-rank sparse attention (Lorsa) on the HIP path.

API of the reference's Lorsa (src/llamascopium/models/lorsa.py:109-1015): `n_qk_heads` query/key
heads `W_Q, W_K [h, d, q]`, and `d_sae` rank-1 value/output heads `W_V, W_O [F, d]`, each of which is
one dictionary feature; feature f mixes its values over key positions with the causal softmax
pattern of query/key head f // (F / h).

What runs where under bf16 autocast (the reference's default precision): the three projections are the
encoder GEMM kernel (`W_V` is feature-major already; the query / key weights are used through a
[heads * width, d_model] bf16 copy), the causal attention mixing and its backward are the matrix-core
attention kernels (no [s, s] matrix, no padding of the narrower query / key heads to the value width),
the weight gradients of the projections are GEMM-kernel products over the token axis, and the TopK
select, the sparse decode through `W_O`, the squared error, the `W_O` gradient rows and the scatter of
the value gradients back to the dense pre-activation are the sparse kernels of the SAE path.  With query / key
norms, rotary shapes the rotary kernels do not take, or user hooks on q and k, those are formed by torch operations and
the mixing alone runs on the attention kernels; in fp32, or with hooks on the scores or the pattern, the projections and
the mixing are torch library routines.
"""

from __future__ import annotations

import math
from typing import Any, Optional

import torch
import torch.nn.functional as Fnn
from torch import nn

from . import ops
from .config import LorsaConfig, register_sae_model
from .hooks import HookPoint
from .sae import SparseRowGrad, _autocast_dtype
from .sparse_dictionary import LazyDict, SparseDictionary


class RMSNormPerHead(nn.Module):
    """lorsa.py:1017-1052: x / sqrt(mean(x^2) + eps) * w with one weight vector per head."""

    def __init__(self, cfg: LorsaConfig, n_heads: Optional[int] = None, device_mesh=None):
        super().__init__()
        self.cfg = cfg
        self.eps = cfg.eps
        self.n_heads = n_heads if n_heads is not None else cfg.n_qk_heads
        self.w = nn.Parameter(torch.ones((self.n_heads, cfg.d_qk_head), dtype=cfg.dtype, device=cfg.device))
        self.hook_scale = HookPoint()
        self.hook_normalized = HookPoint()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.cfg.dtype not in [torch.float32, torch.float64]:
            x = x.to(torch.float32)
        scale = self.hook_scale((x.pow(2).mean(-1, keepdim=True) + self.eps).sqrt())
        return self.hook_normalized((x / scale * self.w).to(self.cfg.dtype))


class _ValueProjection(torch.autograd.Function):
    """v = x @ W_V^T through the encoder GEMM kernel.  The incoming gradient is dense (attention mixes
    every position), so both backward products are plain library GEMMs."""

    @staticmethod
    def forward(ctx, x2, W_V, w_op, amp):
        if amp:
            x_op = x2 if x2.dtype == torch.bfloat16 else ops.cast_bf16(x2.float().contiguous())
            v = ops.encoder_gemm(x_op, w_op, torch.bfloat16)
        else:
            x_op = x2.float().contiguous()
            v = ops.encoder_gemm(x_op, w_op, torch.float32)
        ctx.save_for_backward(x_op, w_op)
        return v

    @staticmethod
    def backward(ctx, g):
        x_op, w_op = ctx.saved_tensors
        gx = gw = None
        gg = g.to(w_op.dtype)
        if ctx.needs_input_grad[0]:
            gx = (gg @ w_op).float()
        if ctx.needs_input_grad[1]:
            gw = (gg.t() @ x_op).float()
        return gx, gw, None, None


class _ProjectAndMix(torch.autograd.Function):
    """x -> q, k, v projections -> causal attention mixing -> hidden_pre [T, F] (bf16), all on the GEMM and attention
    kernels, for configurations without query / key norms.

    forward : q = x W_Q, k = x W_K as [T, h dq], v = x W_V as [T, F]; the biases are added in the products' epilogues.
              With rotary embeddings q and k leave their products as fp32 accumulators, and one element-wise kernel
              rounds them, adds the bias and rotates (`ops.rotary_fwd`); the backward un-rotates d q^T, d k^T in place.
    backward: the attention backward takes the same operands (products over positions read their tiles across the
              rows) and returns dq^T, dk^T, dv^T [., T] in one buffer, which is exactly the operand of the
              weight-gradient product dW = d(.)^T x over the token axis (one GEMM for the three); bias gradients are its
              row sums."""

    @staticmethod
    def forward(ctx, x2, W_Q, W_K, W_V, b_Q, b_K, b_V, model, seq):
        cfg = model.cfg
        T = x2.shape[0]
        n_batch, h = T // seq, cfg.n_qk_heads
        x_op = x2 if x2.dtype == torch.bfloat16 else ops.cast_bf16(x2.float().contiguous())
        wq, wk, wv = model._w_qk_operand("W_Q"), model._w_qk_operand("W_K"), model._w_val_operand(True)
        # the biases join in the products' epilogues (bf16 product + fp32 bias, rounded to bf16 again: what the attention
        # gets under autocast); added per tile inside the attention kernels they would be re-added for every
        # (query block, key block) pair and cost those kernels as many vector instructions as their softmax
        flat = lambda b: b.detach().float().reshape(-1).contiguous()        # noqa: E731
        rot = model._rotary_tables() if cfg.positional_embedding_type == "rotary" else None
        if rot is None:
            q = ops.encoder_gemm_bias(x_op, wq, col_bias=flat(b_Q))         # [T, h dq]
            k = ops.encoder_gemm_bias(x_op, wk, col_bias=flat(b_K))
        else:
            cos, sin = rot[0], rot[1]
            q = ops.rotary_fwd(ops.encoder_gemm(x_op, wq, torch.float32), flat(b_Q), cos, sin, seq, h, cfg.rotary_dim,
                               cfg.rotary_adjacent_pairs)
            k = ops.rotary_fwd(ops.encoder_gemm(x_op, wk, torch.float32), flat(b_K), cos, sin, seq, h, cfg.rotary_dim,
                               cfg.rotary_adjacent_pairs)
        v = ops.encoder_gemm_bias(x_op, wv, col_bias=flat(b_V))             # [T, F]
        scale = 1.0 / model.attn_scale
        out, lse = ops.attention_fwd(q, k, v, n_batch, seq, h, scale)
        ctx.save_for_backward(x_op, wq, wk, wv, q, k, v, out, lse, b_Q.detach(), b_K.detach(), b_V.detach())
        ctx.dims = (n_batch, seq, h, scale)
        ctx.rotary = None if rot is None else (rot[2], rot[3], cfg.rotary_dim, cfg.rotary_adjacent_pairs)
        ctx.shapes = (tuple(W_Q.shape), tuple(W_K.shape))
        ctx.x_dtype = x2.dtype
        return out

    @staticmethod
    def backward(ctx, dz):
        x_op, wq, wk, wv, q, k, v, out, lse, b_Q, b_K, b_V = ctx.saved_tensors
        n_batch, seq, h, scale = ctx.dims
        dz = dz.contiguous() if dz.dtype == torch.bfloat16 else ops.cast_bf16(dz.float().contiguous())
        dqt, dkt, dvt, stacked = ops.attention_bwd(q, k, v, out, dz, lse, n_batch, seq, h, scale, return_stacked=True)
        d = x_op.shape[1]
        n_qk = q.shape[1]
        dq_w = n_qk // h
        if ctx.rotary is not None:   # the gradients arrive with respect to the rotated q, k
            cos_t, sin_t, rdim, adjacent = ctx.rotary
            ops.rotary_bwd_t(stacked[:n_qk], cos_t, sin_t, seq, h, rdim, adjacent)
            ops.rotary_bwd_t(stacked[n_qk: 2 * n_qk], cos_t, sin_t, seq, h, rdim, adjacent)
        # the three weight gradients d(.)^T x in one product over the token axis: the gradients share one buffer
        # [2 h dq + F, T], and a single launch fills the chip where three would each leave most of it idle
        rows = ops.gemm(stacked, x_op, torch.float32, b_k_major=True)       # [2 h dq + F, d]; x [T, d] read as it lies
        sums = ops.row_sum(stacked)

        def qk_weight_grad(part, shape):
            return part.view(h, dq_w, d).permute(0, 2, 1).contiguous().view(shape)

        dW_Q = qk_weight_grad(rows[:n_qk], ctx.shapes[0]) if ctx.needs_input_grad[1] else None
        dW_K = qk_weight_grad(rows[n_qk: 2 * n_qk], ctx.shapes[1]) if ctx.needs_input_grad[2] else None
        dW_V = rows[2 * n_qk:] if ctx.needs_input_grad[3] else None
        db_Q = sums[:n_qk].view(b_Q.shape) if ctx.needs_input_grad[4] else None
        db_K = sums[n_qk: 2 * n_qk].view(b_K.shape) if ctx.needs_input_grad[5] else None
        db_V = sums[2 * n_qk:].view(b_V.shape) if ctx.needs_input_grad[6] else None
        dx = None
        if ctx.needs_input_grad[0]:
            # rare (activations do not carry gradients in training): library products on the transposed gradients
            dx = (dqt.t().float() @ wq.float() + dkt.t().float() @ wk.float() + dvt.t().float() @ wv.float()).to(ctx.x_dtype)
        return dx, dW_Q, dW_K, dW_V, db_Q, db_K, db_V, None, None


class _AttentionMix(torch.autograd.Function):
    """Causal attention mixing of given bf16 q, k [T, h dq] and v [T, F] on the attention kernels.  For configurations
    whose queries and keys are formed by other operations than `_ProjectAndMix` knows (query / key norms, rotary widths
    its kernels do not take, user hooks on q or k): the library attention with its padded heads is still replaced; the
    gradients go back in the operands' layout for autograd to carry on with."""

    @staticmethod
    def forward(ctx, q, k, v, n_batch, seq, n_heads, scale):
        out, lse = ops.attention_fwd(q, k, v, n_batch, seq, n_heads, scale)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.dims = (n_batch, seq, n_heads, scale)
        return out

    @staticmethod
    def backward(ctx, dz):
        q, k, v, out, lse = ctx.saved_tensors
        n_batch, seq, n_heads, scale = ctx.dims
        dz = dz.contiguous() if dz.dtype == torch.bfloat16 else ops.cast_bf16(dz.float().contiguous())
        dqt, dkt, dvt = ops.attention_bwd(q, k, v, out, dz, lse, n_batch, seq, n_heads, scale)
        back = lambda t: ops.transpose_to_bf16(t)[0]                        # noqa: E731   [w, T] -> [T, w]
        return back(dqt), back(dkt), back(dvt), None, None, None, None


class _SparseTail(torch.autograd.Function):
    """hidden_pre [T, F] -> TopK select (decoder-norm scale fused) -> sparse decode through W_O + b_D ->
    masked-mean squared error.  Backward: W_O gradient rows from the feature index, b_D from a column
    sum, and the kept entries' value gradients scattered into a dense [T, F] gradient for the attention
    backward."""

    @staticmethod
    def forward(ctx, hidden_pre, label, tok_w, W_O, b_D, k, amp, holder):
        m: "LowRankSparseAttention" = holder["model"]
        scale = m._decoder_norm_nograd() if m.cfg.sparsity_include_decoder_norm else None
        hp = hidden_pre if hidden_pre.dtype in (torch.float32, torch.bfloat16) else hidden_pre.float()
        hp = hp.contiguous()
        if m.cfg.act_fn.lower() == "batchtopk":
            # the k * tokens largest over every token of the batch (the reference flattens batch and context first,
            # models/sparse_dictionary.py:769-792)
            code = ops.select_topk_batch(hp, None, scale, int(k) * hp.shape[0])
        elif hp.dtype == torch.bfloat16 and getattr(m, "granule_select", True) and ops.granule_route_supported(64, hp.shape[1], int(k)):
            # short rows: one streaming pass for the per-granule key maxima, then a select that reads a row only where a
            # kept entry can be, instead of one 1024-thread workgroup walking every row twice
            code = ops.select_topk_row(hp, None, scale, k, granule_max=ops.granule_max(hp, None, scale))
        else:
            code = ops.select_topk_row(hp, None, scale, k)
        w_op = m._w_dec_operand(amp)
        recon, loss_tok, grad_recon, dval = ops.sparse_decode_mse_fused(
            code, w_op, None if b_D is None else b_D.detach(), label, tok_w)
        holder["code"] = code
        ctx.code, ctx.grad_recon, ctx.dval = code, grad_recon, dval
        ctx.amp = bool(amp)
        ctx.dense_decoder_grad = bool(getattr(m, "dense_decoder_grad", True))
        ctx.defer_to = m if holder.get("defer") else None
        ctx.has_b_D = b_D is not None
        ctx.in_dtype = hidden_pre.dtype
        ctx.mark_non_differentiable(recon)
        return loss_tok.sum(), recon

    @staticmethod
    def backward(ctx, g_loss, _g_recon):
        code = ctx.code
        T, F = code.n_tokens, code.d_sae
        g = g_loss.to(torch.float32)
        m = ctx.defer_to
        d_model = ctx.grad_recon.shape[1]
        # A dictionary that is small against the batch (d_sae / k of a few hundred at most) gets its decoder gradient as
        # the dense product acts^T grad_recon on the matrix cores, what autograd forms for `feature_acts @ W_O` under
        # autocast: gathered gradient rows cost T k d_model bytes of gathers plus a feature index, the product T F d_model
        # flop (16 x 1024 tokens, 8192 features, k = 64: 0.84 ms of index + row pass against ~0.45 ms)
        if ctx.amp and ctx.dense_decoder_grad and T % 64 == 0 and d_model % 8 == 0 and F * T <= 400 * code.n_slots:
            import dataclasses
            acts_t = ops.code_to_dense_t(dataclasses.replace(code, val=code.val * g), F)           # [F, T] bf16
            gd = ops.cast_bf16(ctx.grad_recon.contiguous())                                       # [T, d] bf16, read as it lies
            dW_O = ops.gemm(acts_t, gd, torch.float32, b_k_major=True)  # [F, d]; few output tiles: the product splits its K
            fi = None
        else:
            fi = ops.build_feature_index(code)
        if fi is None:
            pass
        elif m is not None and m.W_O.grad is None and getattr(m.W_O, "_sparse_grad", None) is None:
            # the optimiser rebuilds the rows where it consumes them (under autocast from the bf16-rounded output
            # gradient, as the backward of an autocast matmul pairs them)
            gd = ops.cast_bf16(ctx.grad_recon.contiguous()) if ctx.amp else ctx.grad_recon
            m.W_O._sparse_grad = SparseRowGrad(fi, code.val * g, gd, F)
            dW_O = None
        else:
            dW_O, _ = ops.sparse_grad_rows(fi, code.val * g, ctx.grad_recon, F)
        db_D = ops.col_sum(ctx.grad_recon) * g if ctx.has_b_D else None
        d_hp = None
        if ctx.needs_input_grad[0] and ctx.in_dtype == torch.bfloat16:
            import dataclasses
            d_hp = ops.code_to_dense(dataclasses.replace(code, val=ctx.dval * g), F, want_f32=False, want_bf16=True)[1]
        elif ctx.needs_input_grad[0]:
            slots = torch.arange(code.n_slots, device=code.idx.device)
            tok = (torch.searchsorted(code.row_off, slots, right=True) - 1).clamp_(min=0)
            valid = (slots - code.row_off[tok]) < code.row_nnz[tok]
            cell = torch.where(valid, tok * F + code.idx.long(), torch.zeros_like(tok))
            d_hp = torch.zeros(T * F, dtype=torch.float32, device=code.idx.device)
            d_hp.scatter_add_(0, cell, torch.where(valid, ctx.dval * g, torch.zeros_like(ctx.dval)))
            d_hp = d_hp.view(T, F).to(ctx.in_dtype)
        dlabel = -ctx.grad_recon * g if ctx.needs_input_grad[1] else None
        return d_hp, dlabel, None, dW_O, db_D, None, None, None


@register_sae_model("lorsa")
class LowRankSparseAttention(SparseDictionary):
    def __init__(self, cfg: LorsaConfig, device_mesh=None):
        super().__init__(cfg, device_mesh=device_mesh)
        self.cfg = cfg
        kw = dict(device=cfg.device, dtype=cfg.dtype)
        P = lambda *shape: nn.Parameter(torch.empty(*shape, **kw))  # noqa: E731
        self.W_Q, self.W_K = P(cfg.n_qk_heads, cfg.d_model, cfg.d_qk_head), P(cfg.n_qk_heads, cfg.d_model, cfg.d_qk_head)
        self.W_V, self.W_O = P(cfg.n_ov_heads, cfg.d_model), P(cfg.n_ov_heads, cfg.d_model)
        self.b_Q, self.b_K = P(cfg.n_qk_heads, cfg.d_qk_head), P(cfg.n_qk_heads, cfg.d_qk_head)
        self.b_V = P(cfg.n_ov_heads)
        if cfg.use_decoder_bias:
            self.b_D = P(cfg.d_model)
        # set by an optimiser that consumes factored gradients (HipAdam): W_O's gradient is then attached to it as
        # `_sparse_grad` instead of being written as dense rows
        self.defer_weight_grads = False
        # False sends projections and attention mixing to the torch library routines in every configuration
        self.use_mix_kernels = True
        # False keeps W_O's gradient in factored form (feature index + gathered rows) whatever the shape
        self.dense_decoder_grad = True
        # `decode` of dense activations takes the sparse decoder kernels when they are sparse enough; False keeps the
        # reference's dense product whatever the input
        self.sparse_api_decode = True
        self.register_buffer("mask", torch.tril(torch.ones((cfg.n_ctx, cfg.n_ctx), device=cfg.device).bool()))
        self.register_buffer("IGNORE", torch.tensor(-torch.inf, device=cfg.device))
        if cfg.use_post_qk_ln:
            if cfg.normalization_type != "RMS":
                raise ValueError(f"Invalid normalization type for QK-norm: {cfg.normalization_type}")
            self.ln_q = RMSNormPerHead(cfg, n_heads=cfg.n_qk_heads)
            self.ln_k = RMSNormPerHead(cfg, n_heads=cfg.n_qk_heads)
        if cfg.positional_embedding_type == "rotary":
            sin, cos = self._calculate_sin_cos_rotary(cfg.rotary_dim, cfg.n_ctx, base=cfg.rotary_base, dtype=cfg.dtype,
                                                      device=cfg.device)
            self.register_buffer("rotary_sin", sin)
            self.register_buffer("rotary_cos", cos)
        for name in ("hidden_pre", "feature_acts", "reconstructed", "attn_pattern", "attn_score", "q", "k", "q_post_rot",
                     "k_post_rot"):
            setattr(self, f"hook_{name}", HookPoint())

    # ---- aliases (lorsa.py:242-257) ----
    @property
    def W_D(self) -> torch.Tensor:
        return self.W_O

    @property
    def W_E(self) -> torch.Tensor:
        return self.W_V.T

    @property
    def b_O(self):
        return self.b_D

    @property
    def attn_scale(self) -> float:
        assert self.cfg.attn_scale is not None, "attn_scale must be initialized during config post initialization"
        return self.cfg.attn_scale

    @torch.no_grad()
    def init_parameters(self, **kwargs):
        """lorsa.py:259-278."""
        super().init_parameters(**kwargs)
        nn.init.xavier_uniform_(self.W_Q)
        nn.init.xavier_uniform_(self.W_K)
        nn.init.normal_(self.W_V, mean=0, std=1 / math.sqrt(self.cfg.d_sae))
        nn.init.normal_(self.W_O, mean=0, std=1 / math.sqrt(self.cfg.d_model))
        for b in (self.b_Q, self.b_K, self.b_V):
            nn.init.zeros_(b)
        if self.cfg.use_decoder_bias:
            nn.init.zeros_(self.b_D)

    @torch.no_grad()
    def _calculate_sin_cos_rotary(self, rotary_dim: int, n_ctx: int, base: int = 10000, dtype=torch.float32, device="cpu"):
        """lorsa.py:524-575: angle[p, j] = p / freq[j]; adjacent pairs (GPT-J) or half-split pairs (NeoX) share a
        frequency; optional NTK-by-parts rescaling of the frequencies."""
        hp = torch.float32 if dtype != torch.float64 else torch.float64
        pos = torch.arange(n_ctx, dtype=hp, device=device)
        dim = torch.arange(rotary_dim // 2, dtype=hp, device=device)
        c = self.cfg
        if c.use_NTK_by_parts_rope:
            inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.int64, device=device).float() / rotary_dim))
            low_wl, high_wl = c.old_context_len / c.NTK_by_parts_low_freq_factor, c.old_context_len / c.NTK_by_parts_high_freq_factor
            wavelen = 2 * math.pi / inv_freq
            inv_llama = torch.where(wavelen > low_wl, inv_freq / c.NTK_by_parts_factor, inv_freq)
            smooth = (c.old_context_len / wavelen - c.NTK_by_parts_low_freq_factor) / (
                c.NTK_by_parts_high_freq_factor - c.NTK_by_parts_low_freq_factor)
            smoothed = (1 - smooth) * inv_llama / c.NTK_by_parts_factor + smooth * inv_llama
            medium = ~(wavelen < high_wl) * ~(wavelen > low_wl)
            freq = 1 / torch.where(medium, smoothed, inv_llama)
        else:
            freq = base ** (dim / (rotary_dim / 2))
        freq = freq.repeat_interleave(2) if c.rotary_adjacent_pairs else freq.repeat(2)
        angles = pos[:, None] / freq[None, :]
        return torch.sin(angles).to(dtype), torch.cos(angles).to(dtype)

    # ---- kernel operands ----
    def _w_val_operand(self, amp: bool) -> torch.Tensor:
        w = self.W_V.detach()
        if not amp or w.dtype == torch.bfloat16:
            return w
        return self._derive("W_V.bf16", self.W_V, lambda old: ops.cast_bf16(w, old))

    def _w_qk_operand(self, name: str) -> torch.Tensor:
        """bf16 [n_qk_heads * d_qk_head, d_model] copy of W_Q / W_K [h, d, q] (one head's output column = one row)."""
        p = getattr(self, name)
        h, d, dq = p.shape
        return self._derive(f"{name}.rows.bf16", p, lambda old: ops.cast_bf16(
            p.detach().float().permute(0, 2, 1).reshape(h * dq, d).contiguous(), old))

    def _rotary_tables(self):
        """(cos, sin [n_ctx, rotary_dim], cos^T, sin^T [rotary_dim, n_ctx]) fp32 on the buffers' device, as the rotary
        kernels read them; the transposed copies are made once per buffer."""
        cos, sin = self.rotary_cos, self.rotary_sin
        key = (cos.data_ptr(), sin.data_ptr(), cos._version, sin._version)
        cached = getattr(self, "_rotary_t", None)
        if cached is None or cached[0] != key:
            c32, s32 = cos.detach().float().contiguous(), sin.detach().float().contiguous()
            cached = (key, (c32, s32, c32.t().contiguous(), s32.t().contiguous()))
            self._rotary_t = cached
        return cached[1]

    def _mix_kernel_eligible(self, x: torch.Tensor) -> bool:
        """The projections + mixing run on the GEMM and attention kernels: bf16 autocast over fp32 parameters, no
        query / key norm between projection and scores, no user hook on the attention internals, and shapes the kernels
        (attention, and the rotary embedding when there is one) are built for."""
        cfg = self.cfg
        if not (self.use_mix_kernels and x.is_cuda and x.ndim == 3 and _autocast_dtype("cuda") == torch.bfloat16
                and self.W_V.dtype == torch.float32):
            return False
        if cfg.use_post_qk_ln:
            return False
        if cfg.positional_embedding_type == "rotary" and not (
                ops.rotary_supported(x.shape[1], cfg.d_qk_head, cfg.rotary_dim, cfg.rotary_scale)
                and x.shape[1] <= self.rotary_cos.shape[0] and self.rotary_cos.is_cuda):
            return False
        if any(getattr(self, f"hook_{n}").has_hooks for n in ("q", "k", "q_post_rot", "k_post_rot", "attn_pattern", "attn_score")):
            return False
        b, s, d = x.shape
        return (ops.attention_shapes_supported(s, cfg.d_qk_head, cfg.ov_group_size) and d % 64 == 0 and (b * s) % 64 == 0
                and cfg.d_sae == cfg.n_qk_heads * cfg.ov_group_size)

    def _attention_kernel_eligible(self, x: torch.Tensor) -> bool:
        """The mixing alone runs on the attention kernels, q, k and v being formed by the general op sequence: what is
        left when `_mix_kernel_eligible` declines for the way queries and keys are formed (query / key norms, other
        rotary shapes, hooks on q or k).  Hooks on the scores or the pattern need the [s, s] matrices and keep the
        library route."""
        cfg = self.cfg
        if not (self.use_mix_kernels and x.is_cuda and x.ndim == 3 and _autocast_dtype("cuda") == torch.bfloat16
                and self.W_V.dtype == torch.float32):
            return False
        if self.hook_attn_pattern.has_hooks or self.hook_attn_score.has_hooks:
            return False
        return (ops.attention_shapes_supported(x.shape[1], cfg.d_qk_head, cfg.ov_group_size)
                and cfg.d_sae == cfg.n_qk_heads * cfg.ov_group_size)

    def _w_dec_operand(self, amp: bool) -> torch.Tensor:
        w = self.W_O.detach()
        if not amp or w.dtype == torch.bfloat16:
            return w
        return self._derive("W_D.bf16", self.W_O, lambda old: ops.cast_bf16(w, old))

    def _decoder_norm_nograd(self) -> torch.Tensor:
        return self._derive("W_D.norm", self.W_O, lambda old: ops.row_norm(self.W_O.detach().float(), old))

    # ---- norms (lorsa.py:577-640, 946-958) ----
    def encoder_norm(self, keepdim: bool = False) -> torch.Tensor:
        return torch.norm(self.W_V, p=2, dim=1, keepdim=keepdim)

    def decoder_norm(self, keepdim: bool = False) -> torch.Tensor:
        return torch.norm(self.W_O, p=2, dim=1, keepdim=keepdim)

    def decoder_bias_norm(self) -> torch.Tensor:
        if not self.cfg.use_decoder_bias:
            raise ValueError("Decoder bias not used")
        return torch.norm(self.b_D, p=2, dim=0, keepdim=True)

    @torch.no_grad()
    def transform_to_unit_decoder_norm(self):
        norm = self.decoder_norm(keepdim=True)
        self.W_O /= norm
        self.W_V *= norm
        self.b_V *= norm.squeeze()

    @torch.no_grad()
    def set_decoder_to_fixed_norm(self, value: float, force_exact: bool):
        if force_exact:
            self.W_O.mul_(value / self.decoder_norm(keepdim=True).mean())
        else:
            self.W_O.mul_(value / torch.clamp(self.decoder_norm(keepdim=True).mean(), min=value))

    @torch.no_grad()
    def set_encoder_to_fixed_norm(self, value: float):
        raise NotImplementedError("set_encoder_to_fixed_norm does not make sense for lorsa")

    @torch.no_grad()
    def standardize_parameters_of_dataset_norm(self):
        assert self.cfg.norm_activation == "dataset-wise"
        assert self.dataset_average_activation_norm is not None
        fin = math.sqrt(self.cfg.d_model) / self.dataset_average_activation_norm[self.cfg.hook_point_in]
        fout = math.sqrt(self.cfg.d_model) / self.dataset_average_activation_norm[self.cfg.hook_point_out]
        self.W_Q.mul_(fin)
        self.W_K.mul_(fin)
        self.W_V.mul_(fin)
        self.W_O.div_(fout)
        self.b_D.div_(fout)
        self.cfg.norm_activation = "inference"

    @torch.no_grad()
    def init_encoder_bias_with_mean_hidden_pre(self, batch: dict[str, torch.Tensor]):
        x = self.prepare_input(batch)[0]
        _, hidden_pre = self.encode(x, return_hidden_pre=True)
        self.b_V.sub_(hidden_pre.mean(dim=[0, 1]))

    def load_full_state_dict(self, state_dict: dict[str, torch.Tensor], strict: bool = True) -> None:
        """lorsa.py:960-980: a checkpoint with fewer query/key heads is widened by repeating them."""
        state_dict = dict(state_dict)
        if "W_Q" in state_dict and self.cfg.n_qk_heads != state_dict["W_Q"].size(0):
            n_ckpt = state_dict["W_Q"].size(0)
            assert self.cfg.n_qk_heads % n_ckpt == 0
            rep = self.cfg.n_qk_heads // n_ckpt
            keys = ["W_Q", "W_K", "b_Q", "b_K"] + (["ln_q.w", "ln_k.w"] if self.cfg.use_post_qk_ln else [])
            for k in keys:
                state_dict[k] = torch.repeat_interleave(state_dict[k], rep, dim=0)
        super().load_full_state_dict(state_dict, strict=strict)

    # ---- projections and positional embedding (lorsa.py:784-904) ----
    def _rotate_every_two(self, x: torch.Tensor) -> torch.Tensor:
        rot = x.clone()
        if self.cfg.rotary_adjacent_pairs:
            rot[..., ::2] = -x[..., 1::2]
            rot[..., 1::2] = x[..., ::2]
        else:
            n = x.size(-1) // 2
            rot[..., :n] = -x[..., n:]
            rot[..., n:] = x[..., :n]
        return rot

    def _apply_rotary(self, x: torch.Tensor) -> torch.Tensor:
        x = x.repeat_interleave(self.cfg.rotary_scale, dim=-1)
        n_pos = x.size(1)
        x_rot = x[..., : self.cfg.rotary_dim] if self.cfg.rotary_dim < x.size(-1) else x
        x_pass = x[..., self.cfg.rotary_dim:]
        cos = self.rotary_cos[None, :n_pos, None, :]
        sin = self.rotary_sin[None, :n_pos, None, :]
        return torch.cat([x_rot * cos + self._rotate_every_two(x_rot) * sin, x_pass], dim=-1)

    def _project_values(self, x: torch.Tensor) -> torch.Tensor:
        """v = x @ W_V^T + b_V: the encoder GEMM kernel on the GPU, a library matmul elsewhere."""
        d, F = self.cfg.d_model, self.cfg.d_sae
        amp = _autocast_dtype("cuda") == torch.bfloat16
        if x.is_cuda and self.W_V.dtype == torch.float32 and d % (64 if amp else 32) == 0:
            v = _ValueProjection.apply(x.reshape(-1, d), self.W_V, self._w_val_operand(amp), amp)
            return v.view(*x.shape[:-1], F) + self.b_V
        return torch.einsum("bsd,Vd->bsV", x, self.W_V) + self.b_V

    def _compute_qkv(self, x: torch.Tensor):
        x = x.to(self.W_Q.dtype)
        q = self.hook_q(torch.einsum("bsd,Qdq->bsQq", x, self.W_Q) + self.b_Q)
        k = self.hook_k(torch.einsum("bsd,Kdk->bsKk", x, self.W_K) + self.b_K)
        v = self._project_values(x)
        if self.cfg.use_post_qk_ln:
            q, k = self.ln_q(q), self.ln_k(k)
        if self.cfg.positional_embedding_type == "rotary":
            q, k = self._apply_rotary(q), self._apply_rotary(k)
        return self.hook_q_post_rot(q), self.hook_k_post_rot(k), v

    def _apply_causal_mask(self, scores: torch.Tensor) -> torch.Tensor:
        s = scores.size(-2)
        return torch.where(self.mask[None, None, -s:, -s:], scores, self.IGNORE.to(scores.device))

    def _compute_attention_pattern(self, q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
        scores = torch.einsum("bqhd,bkhd->hbqk", q, k) / self.attn_scale
        return Fnn.softmax(self._apply_causal_mask(scores), dim=-1)

    def _compute_head_outputs(self, pattern: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """pattern [h, b, q, k], v [b, k, F] -> [b, q, F] (feature f uses head f // group)."""
        b, s, F = v.shape
        vg = v.view(b, s, self.cfg.n_qk_heads, self.cfg.ov_group_size)
        return torch.einsum("hbqk,bkhr->bqhr", pattern, vg).reshape(b, -1, F)

    def compute_hidden_pre(self, x: torch.Tensor) -> torch.Tensor:
        """lorsa.py:642-662: causal attention of every feature's value over key positions."""
        if self._mix_kernel_eligible(x):
            b, s, d = x.shape
            z = _ProjectAndMix.apply(x.reshape(b * s, d), self.W_Q, self.W_K, self.W_V, self.b_Q, self.b_K, self.b_V, self, s)
            return z.view(b, s, self.cfg.d_sae)
        q, k, v = self._compute_qkv(x)
        if self._attention_kernel_eligible(x):
            b, s, _ = x.shape
            flat = lambda t: t.reshape(b * s, -1).to(torch.bfloat16).contiguous()    # noqa: E731   (what the library casts to)
            z = _AttentionMix.apply(flat(q), flat(k), flat(v), b, s, self.cfg.n_qk_heads, 1.0 / self.attn_scale)
            return z.view(b, s, self.cfg.d_sae)
        query, key = q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3)
        value = v.reshape(*k.shape[:3], -1).permute(0, 2, 1, 3)
        amp_dtype = _autocast_dtype(x.device.type)      # under autocast the library casts the three operands itself
        to = amp_dtype if amp_dtype is not None else q.dtype
        query, key, value = query.to(to), key.to(to), value.to(to)
        dq, dv = query.shape[-1], value.shape[-1]
        if dq != dv and query.dtype in (torch.bfloat16, torch.float16) and dq % 8 == 0 and dv % 8 == 0:
            # the library's fused attention kernels want one head width: zero-pad the narrower side (zeros add
            # nothing to q.k; padded value columns are cut off again).  Unequal widths would fall back to the
            # unfused path, which materialises the [b, h, s, s] scores (measured 24 ms against 3.7 ms at
            # 16 x 64 x 1024 with widths 64 / 128).
            if dq < dv:
                query, key = Fnn.pad(query, (0, dv - dq)), Fnn.pad(key, (0, dv - dq))
            else:
                value = Fnn.pad(value, (0, dq - dv))
        z = Fnn.scaled_dot_product_attention(query, key, value, scale=1 / self.attn_scale, is_causal=True)[..., :dv]
        return z.permute(0, 2, 1, 3).reshape(*v.shape)

    # ---- API path over dense tensors (lorsa.py:683-782) ----
    def encode(self, x: torch.Tensor, return_hidden_pre: bool = False, return_attention_pattern: bool = False,
               return_attention_score: bool = False, hook_attn_scores: bool = False, **kwargs):
        pattern = scores = None
        if not (return_attention_pattern or return_attention_score or hook_attn_scores):
            hidden_pre = self.compute_hidden_pre(x)
        else:
            q, k, v = self._compute_qkv(x)
            scores = torch.einsum("bqhd,bkhd->bhqk", q, k) / self.attn_scale
            scores = self.hook_attn_score(self._apply_causal_mask(scores))             # [b, h, q, k]
            pattern = self.hook_attn_pattern(Fnn.softmax(scores, dim=-1))
            hidden_pre = self._compute_head_outputs(pattern.permute(1, 0, 2, 3), v)
        hidden_pre = self.hook_hidden_pre(hidden_pre)
        if self.cfg.sparsity_include_decoder_norm:
            hidden_pre = hidden_pre * self.decoder_norm()
        feature_acts = self.activation_function(hidden_pre)
        if self.cfg.sparsity_include_decoder_norm:
            feature_acts = feature_acts / self.decoder_norm()
            hidden_pre = hidden_pre / self.decoder_norm()
        out = [self.hook_feature_acts(feature_acts)]
        if return_hidden_pre:
            out.append(hidden_pre)
        if return_attention_pattern and pattern is not None:
            out.append(pattern)
        if return_attention_score and scores is not None:
            out.append(scores)
        return tuple(out) if len(out) > 1 else out[0]

    def decode(self, feature_acts, **kwargs):
        if isinstance(feature_acts, ops.SparseCode):
            amp = _autocast_dtype("cuda") == torch.bfloat16
            out = ops.sparse_decode_fwd(feature_acts, self._w_dec_operand(amp),
                                        self.b_D.detach() if self.cfg.use_decoder_bias else None)
            return self.hook_reconstructed(out)
        out = None
        F, d = self.cfg.d_sae, self.cfg.d_model
        if (self._sparse_decode_allowed(feature_acts) and feature_acts.shape[-1] == F and d % 8 == 0
                and self.W_O.dtype in (torch.float32, torch.bfloat16)):
            # lorsa.py:765-782 for activations that are sparse enough (at most 1 - cfg.sparsity_threshold_for_triton_spmm_kernel
            # of the entries non-zero, counted on the device and read once): the sparse decoder kernels, forward and backward
            from .kernels import sparse_decode_blocks

            amp = _autocast_dtype("cuda") == torch.bfloat16
            out = sparse_decode_blocks(feature_acts.reshape(-1, F), self.W_O, self._w_dec_operand(amp),
                                       max_density=1.0 - self.cfg.sparsity_threshold_for_triton_spmm_kernel)
            if out is not None:
                out = out.view(*feature_acts.shape[:-1], d)
        if out is None and feature_acts.is_cuda and feature_acts.shape[-1] == F:
            # denser activations: the GEMM kernel (bf16 operands read W_O as it lies)
            from .sae import dense_decode

            amp = _autocast_dtype("cuda") == torch.bfloat16
            out = dense_decode(self, feature_acts.reshape(-1, F), self.W_O, self._w_dec_operand(amp), "W_O.t.f32")
            if out is not None:
                out = out.view(*feature_acts.shape[:-1], d)
        if out is None:
            out = torch.einsum("bps,sd->bpd", feature_acts, self.W_O)
        if self.cfg.use_decoder_bias:
            out = out + self.b_D
        return self.hook_reconstructed(out)

    @torch.no_grad()
    def encode_z_patterns(self, x: torch.Tensor) -> torch.Tensor:
        """lorsa.py:850-862: per-feature attribution over key positions, pattern * value, for one sequence."""
        assert x.size(0) == 1, f"x must be of shape (1, seq_len, d_model), but got {x.shape}"
        q, k, v = self._compute_qkv(x)
        qk_idx = torch.arange(self.cfg.d_sae, device=x.device) // self.cfg.ov_group_size
        pattern = self._compute_attention_pattern(q, k)[qk_idx, 0]
        return pattern * v[0].t()[:, None, :]

    def prepare_input(self, batch: dict[str, torch.Tensor], **kwargs) -> tuple[torch.Tensor, dict[str, Any], dict[str, Any]]:
        return batch[self.cfg.hook_point_in], {}, {}

    def prepare_label(self, batch: dict[str, torch.Tensor], **kwargs):
        return batch[self.cfg.hook_point_out]

    # ---- fused train-step loss ----
    def _has_hooks(self) -> bool:
        return any(h.has_hooks for h in (self.hook_hidden_pre, self.hook_feature_acts, self.hook_reconstructed))

    def _fused_eligible(self, x, sparsity_loss_type, lp_coefficient, auxk_coefficient) -> bool:
        return (self.cfg.act_fn.lower() in ("topk", "batchtopk") and x.is_cuda and x.ndim == 3 and sparsity_loss_type is None
                and not (lp_coefficient > 0.0) and not (auxk_coefficient > 0.0) and not self._has_hooks()
                and self.W_O.dtype == torch.float32 and self.cfg.d_model % 8 == 0)

    def compute_loss(self, batch, label=None, *, sparsity_loss_type=None, lp_coefficient: float = 0.0,
                     auxk_coefficient: float = 0.0, l1_coefficient: float = 1.0, return_aux_data: bool = True, **kwargs):
        x, _, _ = self.prepare_input(batch)
        if not self._fused_eligible(x, sparsity_loss_type, lp_coefficient, auxk_coefficient):
            return super().compute_loss(batch, sparsity_loss_type=sparsity_loss_type, lp_coefficient=lp_coefficient,
                                        auxk_coefficient=auxk_coefficient, l1_coefficient=l1_coefficient,
                                        return_aux_data=return_aux_data, **kwargs)
        label = self.prepare_label(batch, **kwargs)
        mask = batch.get("mask")
        b, s, d = x.shape
        T, F = b * s, self.cfg.d_sae
        if mask is None:
            tok_w = torch.full((T,), 1.0 / T, dtype=torch.float32, device=x.device)
        else:
            mf = mask.to(torch.float32).reshape(T)
            tok_w = mf / mf.sum()
        amp = _autocast_dtype("cuda") == torch.bfloat16
        hidden_pre = self.compute_hidden_pre(x)                                    # [b, s, F], autograd-tracked
        holder: dict[str, Any] = {"model": self, "defer": self.defer_weight_grads and torch.is_grad_enabled()}
        loss, recon = _SparseTail.apply(hidden_pre.reshape(T, F), label.to(torch.float32).reshape(T, d).contiguous(), tok_w,
                                        self.W_O, self.b_D if self.cfg.use_decoder_bias else None, int(self.current_k), amp,
                                        holder)
        if not return_aux_data:
            return loss
        eager = {"loss": loss, "l_rec": loss, "l_s": None, "l_p": None, "l_aux": None, "label": label, "mask": mask,
                 "reconstructed": recon.view(b, s, d), "l1_coefficient": l1_coefficient, "lp_coefficient": lp_coefficient,
                 "auxk_coefficient": auxk_coefficient, "sparse_code": holder["code"]}
        lazy = {"n_tokens": (lambda: batch["tokens"].numel()) if mask is None else (lambda: int(mask.sum().item())),
                "feature_acts": lambda: holder["code"].to_dense().view(b, s, F),
                "hidden_pre": lambda: hidden_pre.detach().float()}
        return LazyDict(eager, lazy)
