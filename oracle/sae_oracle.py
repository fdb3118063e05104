"""CPU oracle for the sparse-autoencoder train step.  TEST INFRASTRUCTURE ONLY.

This module restates, op for op, the eager PyTorch sequence that the reference
(`llamascopium`) runs for one SAE optimisation step.  It exists to check the HIP
path; nothing in the product package may import it.  Only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` use it.

The reference's arithmetic lives in PyTorch, so the restatement is written with
torch CPU ops (the same library routines the reference calls), including the
wasteful dense `[B, F]` temporaries: the CPU timing of this module is meant to
be representative of the reference's eager path.

One deliberate difference: `torch.topk` breaks k-th-place ties in an
implementation-defined way.  The oracle picks the LOWEST INDEX among tied
values (stable descending sort), which is the rule the HIP select kernels
implement.  On tie-free inputs it selects exactly what `torch.topk` selects.

Each function cites the reference lines it follows (paths are relative to the
reference checkout, `src/llamascopium/...`).

Pinning status (see tests/test_oracle_*.py):
  * topk activation ........ pinned by the reference KAT (tests/unit/test_sae.py:92-113)
                             + brute force + torch.topk on tie-free rows
  * decoder/encoder norm ... pinned by closed forms on the reference fixture
                             (tests/unit/test_sae.py:31-55,58-89,116-123)
  * compute_norm_factor .... pinned by closed forms (tests/unit/test_sae.py:126-175)
  * encode/decode/MSE ...... pinned by fp64 numpy brute force + hand-computed fixture
  * batchtopk .............. pinned by brute-force global sort (no reference test)
  * jumprelu STE ........... pinned by fp64 numpy restatement of the 6-line formula
                             + special cases (no reference test)
  * aux-k, tanh/tanh-quad/power/Lp losses ... pinned by fp64 numpy brute force and
                             special cases (#dead=0, #dead<k_aux) (no reference test)
  * SparseAdam, grad norm .. pinned by hand cases (g=[0,3,4] -> 5/sqrt(2)) and a
                             scalar-loop restatement (no reference test)
  * Adam ................... torch.optim.Adam itself is the routine the reference calls
"""

from __future__ import annotations

import math
from typing import Callable, Optional

import torch

# --------------------------------------------------------------------------------------
# selection
# --------------------------------------------------------------------------------------


def topk_indices_lowest_index(x_flat: torch.Tensor, k: int) -> torch.Tensor:
    """Indices of the k largest entries along the last dim; ties -> lowest index.

    Stands in for `torch.topk(x, k, dim=-1, sorted=False)` at utils/math.py:147.
    A stable descending sort keeps equal keys in ascending-index order, so the first k
    entries are "largest value, then lowest index".
    """
    k = min(k, x_flat.shape[-1])
    order = torch.sort(x_flat, dim=-1, descending=True, stable=True).indices
    return order[..., :k]


def topk(
    x: torch.Tensor,
    k: int,
    dim=-1,
    *,
    return_threshold: bool = False,
    abs: bool = False,
):
    """Keep the k largest entries over `dim` (an int or a tuple of dims), zero the rest.

    Follows utils/math.py:81-171: permute the selected dims to the end, flatten them,
    build a boolean mask with scatter_, multiply (so the gradient of kept entries is the
    identity and of dropped entries zero), undo the permutation.
    """
    if isinstance(dim, int):
        dim = (dim,)
    dim = tuple(d if d >= 0 else d + x.ndim for d in dim)
    constant_dims = tuple(d for d in range(x.ndim) if d not in dim)
    perm = constant_dims + tuple(dim)
    xp = x.permute(perm)
    constant_shape = xp.shape[: len(constant_dims)]
    topk_shape = xp.shape[len(constant_dims):]
    x_flat = xp.flatten(start_dim=len(constant_dims))
    with torch.no_grad():
        keys = x_flat.abs() if abs else x_flat
        idx = topk_indices_lowest_index(keys, k)
        mask = torch.zeros_like(x_flat, dtype=torch.bool)
        mask.scatter_(dim=-1, index=idx, value=True)
        threshold = torch.gather(keys, -1, idx).min(dim=-1).values
    out_flat = x_flat * mask.to(x_flat.dtype)
    out_p = out_flat.reshape(*constant_shape, *topk_shape)
    inv = [0] * len(perm)
    for i, p in enumerate(perm):
        inv[p] = i
    out = out_p.permute(inv)
    if return_threshold:
        return out, threshold
    return out


class STEFunction(torch.autograd.Function):
    """JumpReLU with the rectangle-window straight-through threshold gradient.

    Follows activation_functions.py:15-64.
      forward : x * 1[x > theta]                       (strict >, :28,:36)
      backward: dx     = g * 1[x > theta]              (:53)
                dtheta = sum_over_dropped_dims g * (-theta/eps) * 1[|x-theta| < eps/2 and x > 0]   (:45-61)
    """

    @staticmethod
    def forward(ctx, x, theta, window: float, dims_to_keep_in_bwd):
        mask = x.gt(theta)
        ctx.save_for_backward(x, theta, torch.tensor(window, dtype=x.dtype), mask)
        ctx.dims_to_keep_in_bwd = dims_to_keep_in_bwd
        return x * mask

    @staticmethod
    def backward(ctx, g):
        x, theta, window, mask = ctx.saved_tensors
        in_window = ((x - theta).abs() < window * 0.5) * (x > 0.0)
        g_theta = torch.where(in_window, -theta / window, 0.0) * g
        g_x = g * mask
        drop = tuple(
            i for i in range(g_theta.ndim)
            if i not in ctx.dims_to_keep_in_bwd and i - g_theta.ndim not in ctx.dims_to_keep_in_bwd
        )
        g_theta = g_theta.sum(dim=drop)
        return g_x, g_theta, None, None


class JumpReLU(torch.nn.Module):
    """activation_functions.py:67-140: learnable log-threshold of shape `shape`."""

    def __init__(self, window: float, shape, dims_to_keep_in_bwd=(-1,), dtype=torch.float32):
        super().__init__()
        self.jumprelu_threshold_window = window
        self.shape = tuple(shape)
        self.dims_to_keep_in_bwd = tuple(dims_to_keep_in_bwd)
        self.dtype = dtype
        self.log_jumprelu_threshold = torch.nn.Parameter(torch.zeros(shape, dtype=dtype))

    def forward(self, x):
        # input cast to the module dtype and the result cast back (:113-122)
        y = STEFunction.apply(
            x.to(self.dtype), self.log_jumprelu_threshold.exp(), self.jumprelu_threshold_window, self.dims_to_keep_in_bwd
        )
        return y.to(x.dtype)

    def get_jumprelu_threshold(self):
        return self.log_jumprelu_threshold.exp()


# --------------------------------------------------------------------------------------
# masked reductions
# --------------------------------------------------------------------------------------


def apply_token_mask(t: torch.Tensor, n_token_dims: int, mask: Optional[torch.Tensor], reduction: str = "sum"):
    """Reduce the leading `n_token_dims` (batch[, context]) dims of `t`.

    Follows utils/tensor_specs.py:64-84.  Without a mask: plain sum/mean over the token
    dims.  With a 0/1 mask: sum_b t[b]*mask[b], divided by mask.sum() for "mean".
    """
    token_dims = tuple(range(n_token_dims))
    if mask is None:
        if n_token_dims == 0:
            return t
        return t.sum(dim=token_dims) if reduction == "sum" else t.mean(dim=token_dims)
    assert tuple(mask.shape) == tuple(t.shape[:n_token_dims]), "mask must cover exactly the token dims"
    m = mask.to(t)
    m = m.reshape(*m.shape, *([1] * (t.ndim - n_token_dims)))
    out = (t * m).sum(dim=token_dims)
    if reduction == "mean":
        out = out / mask.sum()
    return out


# --------------------------------------------------------------------------------------
# the SAE
# --------------------------------------------------------------------------------------


class SAEOracle(torch.nn.Module):
    """Vanilla SAE / transcoder of models/sae.py:53-448 restated for CPU.

    Parameters use the reference layout: W_E [d, F], b_E [F], W_D [F, d], b_D [d].
    """

    def __init__(
        self,
        d_model: int,
        d_sae: int,
        *,
        act_fn: str = "relu",
        top_k: int = 50,
        use_decoder_bias: bool = True,
        sparsity_include_decoder_norm: bool = True,
        jumprelu_threshold_window: float = 2.0,
        norm_activation: str = "inference",
        use_glu_encoder: bool = False,
        dtype=torch.float32,
    ):
        super().__init__()
        self.d_model, self.d_sae = d_model, d_sae
        self.act_fn = act_fn.lower()
        assert self.act_fn in ("relu", "topk", "jumprelu", "batchtopk"), f"Not implemented activation function {act_fn}"
        self.top_k = top_k
        self.current_k = top_k
        self.use_decoder_bias = use_decoder_bias
        self.sparsity_include_decoder_norm = sparsity_include_decoder_norm
        self.norm_activation = norm_activation
        self.use_glu_encoder = use_glu_encoder
        self.dataset_average_activation_norm = None
        self.dtype = dtype
        self.W_E = torch.nn.Parameter(torch.zeros(d_model, d_sae, dtype=dtype))
        self.b_E = torch.nn.Parameter(torch.zeros(d_sae, dtype=dtype))
        self.W_D = torch.nn.Parameter(torch.zeros(d_sae, d_model, dtype=dtype))
        if use_decoder_bias:
            self.b_D = torch.nn.Parameter(torch.zeros(d_model, dtype=dtype))
        if use_glu_encoder:
            self.W_E_glu = torch.nn.Parameter(torch.zeros(d_model, d_sae, dtype=dtype))
            self.b_E_glu = torch.nn.Parameter(torch.zeros(d_sae, dtype=dtype))
        if self.act_fn == "jumprelu":
            self.activation_function = JumpReLU(jumprelu_threshold_window, (d_sae,), dtype=dtype)
        else:
            self.activation_function = self._make_activation()

    # models/sparse_dictionary.py:713-796
    def _make_activation(self) -> Callable[[torch.Tensor], torch.Tensor]:
        if self.act_fn == "relu":
            return lambda x: x * x.gt(0).to(x.dtype)
        if self.act_fn == "topk":
            def topk_activation(x):
                x = x * x.gt(0).to(x.dtype)
                return topk(x, k=self.current_k, dim=-1)
            return topk_activation
        if self.act_fn == "batchtopk":
            def batch_topk(x):
                x = x * x.gt(0).to(x.dtype)
                shape = None
                if x.ndim == 3:
                    shape = (x.size(0), x.size(1))
                    x = x.flatten(end_dim=1)
                out = topk(x, k=self.current_k * x.size(0), dim=(-2, -1), abs=True)
                if shape is not None:
                    out = out.unflatten(0, shape)
                return out
            return batch_topk
        raise ValueError(self.act_fn)

    # models/sae.py:136-160
    def encoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_E, p=2, dim=0, keepdim=keepdim)

    def decoder_norm(self, keepdim: bool = False):
        return torch.norm(self.W_D, p=2, dim=1, keepdim=keepdim)

    def decoder_bias_norm(self):
        return torch.norm(self.b_D, p=2, dim=0, keepdim=True)

    # models/sae.py:176-188, 209-212
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

    # models/sparse_dictionary.py:427-457
    def compute_norm_factor(self, x: torch.Tensor, hook_point: str) -> torch.Tensor:
        if self.norm_activation == "token-wise":
            return math.sqrt(self.d_model) / torch.norm(x, 2, dim=-1, keepdim=True)
        if self.norm_activation == "batch-wise":
            return math.sqrt(self.d_model) / torch.norm(x, 2, dim=-1, keepdim=True).mean(dim=-2, keepdim=True)
        if self.norm_activation == "dataset-wise":
            assert self.dataset_average_activation_norm is not None
            return torch.tensor(
                math.sqrt(self.d_model) / self.dataset_average_activation_norm[hook_point], dtype=x.dtype
            )
        if self.norm_activation == "inference":
            return torch.tensor(1.0, dtype=x.dtype)
        raise ValueError(f"Not implemented norm_activation {self.norm_activation}")

    # models/sparse_dictionary.py:472-491
    def normalize_activations(self, batch: dict, hook_points=("in", "out")):
        scale = {k: self.compute_norm_factor(v, k) for k, v in batch.items() if k in hook_points}
        return {k: (v * scale[k] if k in scale else v) for k, v in batch.items()}

    # models/sae.py:288-345
    def encode(self, x: torch.Tensor, return_hidden_pre: bool = False, **kwargs):
        x = x.to(self.W_E.dtype)
        hidden_pre = x @ self.W_E + self.b_E
        if self.use_glu_encoder:
            hidden_pre = hidden_pre * torch.sigmoid(x @ self.W_E_glu + self.b_E_glu)
        if self.sparsity_include_decoder_norm:
            hidden_pre = hidden_pre * self.decoder_norm()
        feature_acts = self.activation_function(hidden_pre)
        if self.sparsity_include_decoder_norm:
            feature_acts = feature_acts / self.decoder_norm()
            hidden_pre = hidden_pre / self.decoder_norm()
        if return_hidden_pre:
            return feature_acts, hidden_pre
        return feature_acts

    # models/sae.py:347-377 (dense branch: the numerical reference)
    def decode(self, feature_acts: torch.Tensor, **kwargs):
        _max_l0 = feature_acts.gt(0).to(feature_acts).sum(dim=-1).max()  # the reference always pays these passes (:358)
        reconstructed = feature_acts @ self.W_D
        if self.use_decoder_bias:
            reconstructed = reconstructed + self.b_D
        return reconstructed

    def forward(self, x, encoder_kwargs={}, decoder_kwargs={}):
        return self.decode(self.encode(x, **encoder_kwargs), **decoder_kwargs)

    # models/sparse_dictionary.py:840-1007
    def compute_loss(
        self,
        batch: dict,
        *,
        hook_point_in: str = "in",
        hook_point_out: str = "out",
        sparsity_loss_type: Optional[str] = None,
        tanh_stretch_coefficient: float = 4.0,
        frequency_scale: float = 0.01,
        p: int = 1,
        l1_coefficient: float = 1.0,
        lp_coefficient: float = 0.0,
        auxk_coefficient: float = 0.0,
        k_aux: int = 512,
        update_dead_statistics=None,
        return_aux_data: bool = True,
    ):
        x = batch[hook_point_in]
        label = batch[hook_point_out]
        mask = batch.get("mask")
        feature_acts, hidden_pre = self.encode(x, return_hidden_pre=True)
        reconstructed = self.decode(feature_acts)
        ntd = label.ndim - 1  # token dims: batch[, context]

        l_rec = (reconstructed - label).pow(2).sum(dim=-1)
        l_rec = apply_token_mask(l_rec, ntd, mask, "mean")
        loss_dict = {"l_rec": l_rec}
        loss = l_rec

        if sparsity_loss_type is not None:
            if sparsity_loss_type == "power":
                l_s = torch.norm(feature_acts * self.decoder_norm(), p=p, dim=-1)
            elif sparsity_loss_type == "tanh":
                l_s = torch.tanh(tanh_stretch_coefficient * feature_acts * self.decoder_norm()).sum(dim=-1)
            elif sparsity_loss_type == "tanh-quad":
                score = torch.tanh(tanh_stretch_coefficient * feature_acts * self.decoder_norm())
                approx_frequency = score.mean(dim=tuple(range(score.ndim - 1)))
                l_s = (approx_frequency * (1 + approx_frequency / frequency_scale)).sum(dim=-1)
            else:
                raise ValueError(f"sparsity_loss_type f{sparsity_loss_type} not supported.")
            l_s = l1_coefficient * l_s
            loss_dict["l_s"] = l_s
            # tanh-quad is already a scalar: specs.loss() of a 0-dim tensor raises in the
            # reference (tensor_specs.py:36-43); the restatement reduces what there is to reduce.
            l_s = apply_token_mask(l_s, min(ntd, l_s.ndim), mask if l_s.ndim else None, "mean")
            loss = loss + l_s
        else:
            loss_dict["l_s"] = None

        if lp_coefficient > 0.0 and isinstance(self.activation_function, JumpReLU):
            theta = self.activation_function.get_jumprelu_threshold()
            l_p = torch.nn.functional.relu(theta - hidden_pre) * self.decoder_norm()
            l_p = lp_coefficient * l_p.sum(dim=-1)
            l_p = apply_token_mask(l_p, ntd, mask, "mean")
            loss_dict["l_p"] = l_p
            loss = loss + l_p
        else:
            loss_dict["l_p"] = None

        if auxk_coefficient > 0.0:
            assert update_dead_statistics is not None, "update_dead_statistics must be set when auxk_coefficient > 0.0"
            is_dead = update_dead_statistics(feature_acts, mask, ntd)
            e = label - reconstructed  # not detached (:949)
            current_k = self.current_k
            self.current_k = min(k_aux, int(is_dead.sum().item()))
            if self.current_k > 0:
                if self.sparsity_include_decoder_norm:
                    dead_hidden_pre = hidden_pre * is_dead * self.decoder_norm()
                else:
                    dead_hidden_pre = hidden_pre * is_dead
                dead_feature_acts = self.activation_function(dead_hidden_pre)
                if self.sparsity_include_decoder_norm:
                    dead_feature_acts = dead_feature_acts / self.decoder_norm()
                aux_reconstructed = dead_feature_acts @ self.W_D
                l_aux = (e - aux_reconstructed).pow(2).sum(dim=-1)
                l_aux = auxk_coefficient * l_aux
                l_aux = apply_token_mask(l_aux, ntd, mask, "mean")
                loss_dict["l_aux"] = l_aux
                loss = loss + l_aux
            else:
                loss_dict["l_aux"] = torch.zeros_like(l_rec)
            self.current_k = current_k
        else:
            loss_dict["l_aux"] = None

        if not return_aux_data:
            return loss
        return {
            "loss": loss,
            **loss_dict,
            "label": label,
            "mask": mask,
            "n_tokens": batch["tokens"].numel() if mask is None else int(mask.sum().item()),
            "feature_acts": feature_acts,
            "reconstructed": reconstructed,
            "hidden_pre": hidden_pre,
            "l1_coefficient": l1_coefficient,
            "lp_coefficient": lp_coefficient,
            "auxk_coefficient": auxk_coefficient,
        }

    # models/sparse_dictionary.py:501-510
    def get_parameters(self):
        jr = list(self.activation_function.parameters()) if isinstance(self.activation_function, JumpReLU) else []
        others = [p for p in self.parameters() if not any(p is q for q in jr)]
        return [{"params": others, "name": "others"}, {"params": jr, "name": "jumprelu"}]


# --------------------------------------------------------------------------------------
# trainer-side state on the path
# --------------------------------------------------------------------------------------


class DeadStatistics:
    """trainer.py:403-454: tokens since each feature last fired; dead = count >= threshold."""

    def __init__(self, d_sae: int, dead_threshold: float):
        self.tokens_since_last_activation = torch.zeros(d_sae, dtype=torch.long)
        self.is_dead = torch.zeros(d_sae, dtype=torch.bool)
        self.dead_threshold = dead_threshold

    @torch.no_grad()
    def update(self, feature_acts: torch.Tensor, mask: Optional[torch.Tensor], n_token_dims: int) -> torch.Tensor:
        valid_tokens = mask.sum() if mask is not None else feature_acts[..., 0].numel()
        acts_sum = apply_token_mask(feature_acts, n_token_dims, mask, "sum")
        activated = acts_sum.gt(0)
        self.tokens_since_last_activation = torch.where(
            activated,
            torch.zeros_like(self.tokens_since_last_activation),
            self.tokens_since_last_activation + valid_tokens,
        )
        self.is_dead = self.tokens_since_last_activation >= self.dead_threshold
        return self.is_dead


def k_schedule(
    cur_step: int,
    *,
    top_k: int,
    initial_k: float,
    k_cold_booting_steps: int,
    k_warmup_steps: int,
    k_schedule_type: str = "linear",
    k_exponential_factor: float = 3.0,
) -> int:
    """trainer.py:462-485: the k used at `cur_step` while k is annealed from initial_k to top_k."""
    if cur_step < k_cold_booting_steps:
        return int(initial_k)
    progress = min(1.0, (cur_step - k_cold_booting_steps) / k_warmup_steps)
    if k_schedule_type == "exponential":
        decay = (1.0 - math.exp(-k_exponential_factor * progress)) / (1.0 - math.exp(-k_exponential_factor))
        k = initial_k - (initial_k - top_k) * decay
    else:
        k = initial_k + (top_k - initial_k) * progress
    return max(top_k, math.ceil(k))


def l1_warmup(cur_step: int, warmup_steps: int, l1_coefficient: Optional[float]) -> float:
    """trainer.py:487-491."""
    if l1_coefficient is None:
        return 1.0
    return min(1.0, cur_step / warmup_steps) * l1_coefficient


# --------------------------------------------------------------------------------------
# optimiser-side functions on the path
# --------------------------------------------------------------------------------------


def compute_grad_norm(grads) -> torch.Tensor:
    """optim.py:257-277: ||(||g_i||_2)_i||_2 / sqrt(number of non-zero gradient entries)."""
    grads = [g for g in grads if g is not None]
    assert len(grads) > 0, "No gradients found"
    total = torch.stack([g.norm(2) for g in grads]).norm(2)
    nnz = sum((g != 0).sum() for g in grads)
    return total / nnz.sqrt()


def clip_grad_norm(grads, max_norm: float) -> torch.Tensor:
    """optim.py:280-292: scales the gradients in place when the norm above exceeds max_norm."""
    gn = compute_grad_norm(grads)
    if gn.item() > max_norm:
        for g in grads:
            if g is not None:
                g.mul_(max_norm / (gn.item() + 1e-6))
    return gn


class SparseAdamState:
    def __init__(self, p):
        self.step = 0
        self.exp_avg = torch.zeros_like(p)
        self.exp_avg_sq = torch.zeros_like(p)


@torch.no_grad()
def sparse_adam_step(p, g, st: SparseAdamState, *, lr, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0):
    """optim.py:183-254 for one parameter: moments decay everywhere, but gradient
    contributions and the parameter update apply only where g != 0; a parameter whose
    gradient is entirely zero is skipped (its step counter does not advance)."""
    if not g.any():
        return
    b1, b2 = betas
    st.step += 1
    bc1 = 1 - b1 ** st.step
    bc2 = 1 - b2 ** st.step
    if weight_decay != 0:
        g = g.add(p, alpha=weight_decay)
    mask = g != 0
    m = st.exp_avg * b1
    m = torch.where(mask, m + (1 - b1) * g, m)
    v = st.exp_avg_sq * b2
    v = torch.where(mask, v + (1 - b2) * g * g, v)
    st.exp_avg, st.exp_avg_sq = m, v
    step_size = lr * math.sqrt(bc2) / bc1
    denom = v.sqrt().add_(eps)
    p.sub_(torch.where(mask, step_size * m / denom, torch.zeros_like(p)))


def make_adam(model: SAEOracle, lr: float, betas=(0.9, 0.999), jumprelu_lr_factor: float = 1.0, foreach: bool = True):
    """trainer.py:349-390: torch.optim.Adam over the two parameter groups."""
    groups = []
    for g in model.get_parameters():
        if g["name"] == "jumprelu":
            g = {**g, "lr": jumprelu_lr_factor * lr}
        groups.append(g)
    groups = [g for g in groups if len(g["params"]) > 0]
    return torch.optim.Adam(groups, lr=lr, betas=betas, foreach=foreach)


def train_step(model: SAEOracle, opt, batch: dict, *, amp_dtype=None, **loss_kwargs) -> dict:
    """One iteration of the hot loop (trainer.py:605-647) without logging:
    compute_loss under autocast, backward, optimizer.step, zero_grad."""
    if amp_dtype is not None and amp_dtype != torch.float32:
        with torch.autocast("cpu", dtype=amp_dtype):
            ctx = model.compute_loss(batch, **loss_kwargs)
    else:
        ctx = model.compute_loss(batch, **loss_kwargs)
    ctx["loss"].backward()
    opt.step()
    opt.zero_grad()
    return ctx
