"""CPU oracle for the crosscoder, cross-layer transcoder and Lorsa forward / loss paths.
TEST INFRASTRUCTURE ONLY: nothing in the product package may import this module.

Each class restates, op for op with torch CPU routines, what the reference's model computes in
`encode` / `decode` / `compute_loss`; backward comes from autograd over the restated forward, as it
does in the reference.  TopK ties go to the lowest index (see `sae_oracle.topk`).

Pinning status (tests/test_oracle_variants.py):
  * CrosscoderOracle ... the reference's own known answers (tests/unit/test_crosscoder.py:120-274:
                         summed hidden_pre, per-head decode, encoder / decoder / bias norms) plus a
                         scalar-loop brute force of the per-head activation and the loss
  * CLTOracle .......... scalar triple loop y_j = sum_{i<=j} f_i W_D[j][i] + b_D[j] on L=3, d=4, F=8;
                         equals SAEOracle when L=1; decoder_norm_per_feature by an explicit loop;
                         the four TopK scopes by brute-force sorts (no reference test of this model is
                         importable)
  * LorsaOracle ........ explicit [s, s] causal softmax attention in fp64 written as scalar loops on
                         s <= 8; equals standard multi-head attention when ov_group_size == head width;
                         rotary checked against the closed-form 2-D rotation (no reference test of this
                         model is importable)
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as Fnn

from .sae_oracle import JumpReLU, topk


def _base_activation(act_fn: str, owner, jumprelu_shape=None, window: float = 2.0, dtype=torch.float32):
    """models/sparse_dictionary.py:713-796 (the activations of the base class; `owner.current_k` is read at
    call time, like the reference's closure over `self`)."""
    act_fn = act_fn.lower()
    if act_fn == "relu":
        return lambda x: x * x.gt(0).to(x.dtype)
    if act_fn == "jumprelu":
        return JumpReLU(window, jumprelu_shape, dtype=dtype)
    if act_fn == "topk":
        def topk_activation(x):
            x = x * x.gt(0).to(x.dtype)
            return topk(x, k=owner.current_k, dim=-1)
        return topk_activation
    if act_fn == "batchtopk":
        def batch_topk(x):
            x = x * x.gt(0).to(x.dtype)
            shape = None
            if x.ndim == 3:
                shape = (x.size(0), x.size(1))
                x = x.flatten(end_dim=1)
            out = topk(x, k=owner.current_k * x.size(0), dim=(-2, -1), abs=True)
            return out.unflatten(0, shape) if shape is not None else out
        return batch_topk
    raise ValueError(f"Not implemented activation function {act_fn}")


# --------------------------------------------------------------------------------------
# crosscoder
# --------------------------------------------------------------------------------------


class CrosscoderOracle(torch.nn.Module):
    """models/crosscoder.py:84-716.  W_E [H, d, F], b_E [H, F], W_D [H, F, d], b_D [H, d]."""

    def __init__(self, n_heads: int, d_model: int, d_sae: int, *, act_fn: str = "relu", top_k: int = 50,
                 jumprelu_threshold_window: float = 2.0, dtype=torch.float32):
        super().__init__()
        self.n_heads, self.d_model, self.d_sae = n_heads, d_model, d_sae
        self.current_k = top_k
        z = lambda *s: torch.nn.Parameter(torch.zeros(*s, dtype=dtype))  # noqa: E731
        self.W_E, self.b_E = z(n_heads, d_model, d_sae), z(n_heads, d_sae)
        self.W_D, self.b_D = z(n_heads, d_sae, d_model), z(n_heads, d_model)
        self.activation_function = _base_activation(act_fn, self, (d_sae,), jumprelu_threshold_window, dtype)

    # crosscoder.py:472-505
    def decoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_D, dim=-1, keepdim=keepdim)

    def encoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_E, dim=-2, keepdim=keepdim)

    def decoder_bias_norm(self):
        return torch.norm(self.b_D, dim=-1, keepdim=True)

    # crosscoder.py:222-275 (vmap of matmul over the head axis) and :314-382
    def encode(self, x, return_hidden_pre: bool = False, **kwargs):
        per_head = torch.stack([x[..., h, :] @ self.W_E[h] for h in range(self.n_heads)], dim=-2) + self.b_E
        acc = per_head.sum(dim=-2)
        acc = acc.unsqueeze(-2).expand(*acc.shape[:-1], self.n_heads, self.d_sae)
        feature_acts = self.activation_function(acc * self.decoder_norm()) / self.decoder_norm()
        return (feature_acts, acc) if return_hidden_pre else feature_acts

    # crosscoder.py:384-469
    def decode(self, feature_acts, **kwargs):
        return torch.stack([feature_acts[..., h, :] @ self.W_D[h] for h in range(self.n_heads)], dim=-2) + self.b_D

    def forward(self, x):
        return self.decode(self.encode(x))

    # crosscoder.py:551-636: stack the hook points on a new axis before the model axis; label = input
    def prepare_input(self, batch: dict, hook_points):
        return torch.stack([batch[h] for h in hook_points], dim=-2)

    # models/sparse_dictionary.py:875-886: squared error summed over the model axis; the [batch, heads]
    # result is reduced by the 2-D loss specs (both axes averaged; a mask must cover both axes)
    def compute_loss(self, batch: dict, hook_points, mask: Optional[torch.Tensor] = None):
        x = self.prepare_input(batch, hook_points)
        label = x
        feature_acts, hidden_pre = self.encode(x, return_hidden_pre=True)
        reconstructed = self.decode(feature_acts)
        l_rec = (reconstructed - label).pow(2).sum(dim=-1)
        if mask is None:
            l_rec = l_rec.mean()
        else:
            assert tuple(mask.shape) == tuple(l_rec.shape)
            l_rec = (l_rec * mask.to(l_rec)).sum() / mask.sum()
        return {"loss": l_rec, "l_rec": l_rec, "feature_acts": feature_acts, "hidden_pre": hidden_pre,
                "reconstructed": reconstructed, "label": label}


# --------------------------------------------------------------------------------------
# cross-layer transcoder
# --------------------------------------------------------------------------------------


class CLTOracle(torch.nn.Module):
    """models/clt.py:124-1125.  W_E [L, d, F], b_E [L, F], W_D[l] [l+1, F, d], b_D[l] [d]."""

    def __init__(self, n_layers: int, d_model: int, d_sae: int, *, act_fn: str = "relu", top_k: int = 50,
                 sparsity_include_decoder_norm: bool = True, jumprelu_threshold_window: float = 2.0, dtype=torch.float32):
        super().__init__()
        self.n_layers, self.d_model, self.d_sae = n_layers, d_model, d_sae
        self.current_k = top_k
        self.sparsity_include_decoder_norm = sparsity_include_decoder_norm
        self.act_fn = act_fn.lower()
        P = torch.nn.Parameter
        self.W_E = P(torch.zeros(n_layers, d_model, d_sae, dtype=dtype))
        self.b_E = P(torch.zeros(n_layers, d_sae, dtype=dtype))
        self.W_D = torch.nn.ParameterList([P(torch.zeros(i + 1, d_sae, d_model, dtype=dtype)) for i in range(n_layers)])
        self.b_D = torch.nn.ParameterList([P(torch.zeros(d_model, dtype=dtype)) for _ in range(n_layers)])
        self.activation_function = self._make_activation(jumprelu_threshold_window, dtype)

    # clt.py:232-387: the selection scope differs per activation name
    def _make_activation(self, window, dtype):
        a = self.act_fn
        if a == "relu":
            return lambda x: x * x.gt(0).to(x.dtype)
        if a == "jumprelu":
            return JumpReLU(window, (self.n_layers, self.d_sae), dims_to_keep_in_bwd=(-2, -1), dtype=dtype)
        scopes = {"topk": (-1,), "layertopk": (-2, -1), "batchtopk": (0, -1), "batchlayertopk": (0, -1, -2)}
        if a not in scopes:
            raise ValueError(f"Not implemented activation function {a}")
        per_batch = a.startswith("batch")

        def act(x):
            x = x * x.gt(0).to(x.dtype)
            return topk(x, k=self.current_k * (x.size(0) if per_batch else 1), dim=scopes[a])
        return act

    # clt.py:837-876 (layer=None branch): feature (l, f) is read by decoders l..L-1; norm over all of them
    @torch.no_grad()
    def decoder_norm_per_feature(self):
        norms = torch.zeros(self.n_layers, self.d_sae, dtype=self.W_E.dtype)
        for layer_to, w in enumerate(self.W_D):
            norms[: layer_to + 1] = norms[: layer_to + 1] + w.pow(2).sum(dim=-1)
        return norms.sqrt()

    # clt.py:801-825: constant ones
    def decoder_norm(self, keepdim: bool = False):
        return torch.ones(self.n_layers * (self.n_layers + 1) // 2, dtype=self.W_E.dtype)

    def encoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_E, p=2, dim=1, keepdim=keepdim)

    def decoder_bias_norm(self):
        return torch.ones(self.n_layers, dtype=self.W_E.dtype)

    # clt.py:527-573: the scaled hidden_pre is what is returned; only feature_acts are unscaled again
    def encode(self, x, return_hidden_pre: bool = False, **kwargs):
        hidden_pre = torch.einsum("...ld,lds->...ls", x, self.W_E) + self.b_E
        if self.sparsity_include_decoder_norm:
            hidden_pre = hidden_pre * self.decoder_norm_per_feature()
        feature_acts = self.activation_function(hidden_pre)
        if self.sparsity_include_decoder_norm:
            feature_acts = feature_acts / self.decoder_norm_per_feature()
        return (feature_acts, hidden_pre) if return_hidden_pre else feature_acts

    # clt.py:630-709 (dense branch)
    def decode(self, feature_acts, batch_first: bool = False, **kwargs):
        out = []
        for layer_to in range(self.n_layers):
            contribution = (feature_acts[..., : layer_to + 1, :].permute(1, 0, 2) @ self.W_D[layer_to]).sum(0)
            out.append(contribution + self.b_D[layer_to])
        return torch.stack(out, dim=1 if batch_first else 0)

    def forward(self, x):
        return self.decode(self.encode(x))

    # clt.py:940-976
    def prepare_input(self, batch: dict, hook_points_in):
        xs = [batch[h] for h in hook_points_in]
        return torch.stack(xs, dim=xs[0].ndim - 1)

    def prepare_label(self, batch: dict, hook_points_out):
        return torch.stack([batch[h] for h in hook_points_out], dim=0)

    # clt.py:1024-1104
    def compute_loss(self, batch: dict, hook_points_in, hook_points_out, *, sparsity_loss_type=None,
                     tanh_stretch_coefficient: float = 4.0, frequency_scale: float = 0.01, p: int = 1,
                     l1_coefficient: float = 1.0):
        x = self.prepare_input(batch, hook_points_in)
        label = self.prepare_label(batch, hook_points_out)
        feature_acts = self.encode(x)
        reconstructed = self.decode(feature_acts)
        l_rec = (reconstructed - label).pow(2).sum(dim=-1).mean()
        loss, l_s = l_rec, None
        if sparsity_loss_type is not None:
            n = self.decoder_norm_per_feature()
            if sparsity_loss_type == "power":
                l_s = torch.norm(feature_acts * n, p=p, dim=-1)
            elif sparsity_loss_type == "tanh":
                l_s = torch.tanh(tanh_stretch_coefficient * feature_acts * n).sum(dim=-1)
            elif sparsity_loss_type == "tanh-quad":
                t = torch.tanh(tanh_stretch_coefficient * feature_acts * n)
                freq = t.mean(dim=tuple(range(t.ndim - 1)))
                l_s = (freq * (1 + freq / frequency_scale)).sum(dim=-1)
            else:
                raise ValueError(f"sparsity_loss_type f{sparsity_loss_type} not supported.")
            l_s = l1_coefficient * l_s
            loss = loss + l_s.mean()
        return {"loss": loss, "l_rec": l_rec, "l_s": l_s, "feature_acts": feature_acts, "reconstructed": reconstructed,
                "label": label}


# --------------------------------------------------------------------------------------
# low-rank sparse attention
# --------------------------------------------------------------------------------------


def rotary_sin_cos(rotary_dim: int, n_ctx: int, base: int = 10000, adjacent_pairs: bool = True, dtype=torch.float32):
    """models/lorsa.py:525-575 without the NTK-by-parts branch: angle[p, j] = p / base^(pair(j) / (rotary_dim/2))."""
    hp = torch.float64 if dtype == torch.float64 else torch.float32
    pos = torch.arange(n_ctx, dtype=hp)
    dim = torch.arange(rotary_dim // 2, dtype=hp)
    freq = base ** (dim / (rotary_dim / 2))
    freq = freq.repeat_interleave(2) if adjacent_pairs else freq.repeat(2)
    angles = pos[:, None] / freq[None, :]
    return torch.sin(angles).to(dtype), torch.cos(angles).to(dtype)


class LorsaOracle(torch.nn.Module):
    """models/lorsa.py:109-1015.  W_Q, W_K [h, d, q]; W_V, W_O [F, d]; b_Q, b_K [h, q]; b_V [F]; b_D [d].
    Each of the F value/output heads is one dictionary feature; feature f attends with the pattern of
    query/key head f // (F / h)."""

    def __init__(self, d_model: int, d_sae: int, n_qk_heads: int, d_qk_head: int, n_ctx: int, *, act_fn: str = "topk",
                 top_k: int = 50, positional_embedding_type: str = "none", rotary_dim: Optional[int] = None,
                 rotary_base: int = 10000, rotary_adjacent_pairs: bool = True, rotary_scale: int = 1,
                 attn_scale: Optional[float] = None, use_post_qk_ln: bool = False, eps: float = 1e-6,
                 use_decoder_bias: bool = True, sparsity_include_decoder_norm: bool = True,
                 jumprelu_threshold_window: float = 2.0, dtype=torch.float32):
        super().__init__()
        assert d_sae % n_qk_heads == 0, "n_ov_heads must be divisible by n_qk_heads"
        self.d_model, self.d_sae, self.n_qk_heads, self.d_qk_head, self.n_ctx = d_model, d_sae, n_qk_heads, d_qk_head, n_ctx
        self.ov_group_size = d_sae // n_qk_heads
        self.attn_scale = attn_scale if attn_scale is not None else d_qk_head ** 0.5
        self.positional_embedding_type = positional_embedding_type
        self.rotary_dim, self.rotary_adjacent_pairs, self.rotary_scale = rotary_dim, rotary_adjacent_pairs, rotary_scale
        self.use_post_qk_ln, self.eps = use_post_qk_ln, eps
        self.use_decoder_bias = use_decoder_bias
        self.sparsity_include_decoder_norm = sparsity_include_decoder_norm
        self.current_k = top_k
        z = lambda *s: torch.nn.Parameter(torch.zeros(*s, dtype=dtype))  # noqa: E731
        self.W_Q, self.W_K = z(n_qk_heads, d_model, d_qk_head), z(n_qk_heads, d_model, d_qk_head)
        self.W_V, self.W_O = z(d_sae, d_model), z(d_sae, d_model)
        self.b_Q, self.b_K, self.b_V = z(n_qk_heads, d_qk_head), z(n_qk_heads, d_qk_head), z(d_sae)
        if use_decoder_bias:
            self.b_D = z(d_model)
        if use_post_qk_ln:  # RMS norm per head (lorsa.py:1017-1052), weights start at one
            self.ln_q_w = torch.nn.Parameter(torch.ones(n_qk_heads, d_qk_head, dtype=dtype))
            self.ln_k_w = torch.nn.Parameter(torch.ones(n_qk_heads, d_qk_head, dtype=dtype))
        if positional_embedding_type == "rotary":
            sin, cos = rotary_sin_cos(rotary_dim, n_ctx, rotary_base, rotary_adjacent_pairs, dtype)
            self.register_buffer("rotary_sin", sin)
            self.register_buffer("rotary_cos", cos)
        self.activation_function = _base_activation(act_fn, self, (d_sae,), jumprelu_threshold_window, dtype)

    def decoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_O, p=2, dim=1, keepdim=keepdim)

    def encoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_V, p=2, dim=1, keepdim=keepdim)

    def _rms(self, x, w):
        scale = (x.pow(2).mean(-1, keepdim=True) + self.eps).sqrt()
        return x / scale * w

    # lorsa.py:864-904
    def _apply_rotary(self, x):
        x = x.repeat_interleave(self.rotary_scale, dim=-1)
        n_pos = x.size(1)
        x_rot, x_pass = x[..., : self.rotary_dim], x[..., self.rotary_dim:]
        flip = x_rot.clone()
        if self.rotary_adjacent_pairs:
            flip[..., ::2] = -x_rot[..., 1::2]
            flip[..., 1::2] = x_rot[..., ::2]
        else:
            n = x_rot.size(-1) // 2
            flip[..., :n] = -x_rot[..., n:]
            flip[..., n:] = x_rot[..., :n]
        cos = self.rotary_cos[None, :n_pos, None, :]
        sin = self.rotary_sin[None, :n_pos, None, :]
        return torch.cat([x_rot * cos + flip * sin, x_pass], dim=-1)

    # lorsa.py:784-829
    def _compute_qkv(self, x):
        x = x.to(self.W_Q.dtype)
        q = torch.einsum("bsd,Qdq->bsQq", x, self.W_Q) + self.b_Q
        k = torch.einsum("bsd,Kdk->bsKk", x, self.W_K) + self.b_K
        v = torch.einsum("bsd,Vd->bsV", x, self.W_V) + self.b_V
        if self.use_post_qk_ln:
            q, k = self._rms(q, self.ln_q_w), self._rms(k, self.ln_k_w)
        if self.positional_embedding_type == "rotary":
            q, k = self._apply_rotary(q), self._apply_rotary(k)
        return q, k, v

    # lorsa.py:683-763, the explicit-pattern branch (scores -> causal mask -> softmax -> per-head mixing)
    def encode(self, x, return_hidden_pre: bool = False, return_attention_pattern: bool = False, **kwargs):
        q, k, v = self._compute_qkv(x)
        s = x.shape[1]
        scores = torch.einsum("bqhd,bkhd->bhqk", q, k) / self.attn_scale
        causal = torch.tril(torch.ones(s, s, dtype=torch.bool))
        scores = torch.where(causal, scores, torch.tensor(-torch.inf, dtype=scores.dtype))
        pattern = Fnn.softmax(scores, dim=-1)                      # [b, h, q, k]
        vg = v.reshape(v.shape[0], s, self.n_qk_heads, self.ov_group_size)
        hidden_pre = torch.einsum("bhqk,bkhr->bqhr", pattern, vg).reshape(v.shape)
        if self.sparsity_include_decoder_norm:
            hidden_pre = hidden_pre * self.decoder_norm()
        feature_acts = self.activation_function(hidden_pre)
        if self.sparsity_include_decoder_norm:
            feature_acts = feature_acts / self.decoder_norm()
            hidden_pre = hidden_pre / self.decoder_norm()
        out = [feature_acts]
        if return_hidden_pre:
            out.append(hidden_pre)
        if return_attention_pattern:
            out.append(pattern)
        return tuple(out) if len(out) > 1 else out[0]

    # lorsa.py:765-782
    def decode(self, feature_acts, **kwargs):
        out = torch.einsum("bps,sd->bpd", feature_acts, self.W_O)
        if self.use_decoder_bias:
            out = out + self.b_D
        return out

    def forward(self, x):
        return self.decode(self.encode(x))

    # models/sparse_dictionary.py:875-886 with 3-D activations: mean over batch and context
    def compute_loss(self, batch: dict, hook_point_in: str = "in", hook_point_out: str = "out",
                     mask: Optional[torch.Tensor] = None):
        x, label = batch[hook_point_in], batch[hook_point_out]
        feature_acts, hidden_pre = self.encode(x, return_hidden_pre=True)
        reconstructed = self.decode(feature_acts)
        l_rec = (reconstructed - label).pow(2).sum(dim=-1)
        l_rec = l_rec.mean() if mask is None else (l_rec * mask.to(l_rec)).sum() / mask.sum()
        return {"loss": l_rec, "l_rec": l_rec, "feature_acts": feature_acts, "hidden_pre": hidden_pre,
                "reconstructed": reconstructed, "label": label}


def init_uniform_(module: torch.nn.Module, seed: int, bound: float = 0.5):
    """Seeded test weights: every parameter uniform in (-bound, bound), decoder-like matrices included."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for p in module.parameters():
            p.copy_((torch.rand(p.shape, generator=g, dtype=torch.float64) * 2 - 1).to(p.dtype) * bound)
    return module


__all__ = ["CrosscoderOracle", "CLTOracle", "LorsaOracle", "rotary_sin_cos", "init_uniform_"]
