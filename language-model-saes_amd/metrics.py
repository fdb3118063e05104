"""Training metrics of the trainer's `_log` (src/llamascopium/metrics.py:22-329), computed from what the
fused step already holds: the sparse code `(idx, val)` and the `[B, d]` label / reconstruction.

The reference reads a dense `[B, F]` `feature_acts` in `FrequencyMetric`, `MeanFeatureActMetric` and
`L0Metric`; here one kernel pass over the `B k` kept slots feeds all three, and one pass over the two
`[B, d]` tensors feeds `ExplainedVarianceMetric` and `L2NormErrorMetric`.  Running sums stay on the
device; `compute()` (every `log_frequency` steps) is the only place that synchronises.  A context
without `sparse_code` (a model on the generic dense route) takes the reference's dense formulas.
Metric names, reductions and reset behaviour are the reference's.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from . import ops
from .optim import compute_grad_norm
from .sparse_dictionary import apply_token_mask


def item(x) -> float | int:
    return x.item() if isinstance(x, torch.Tensor) else x


class Record:
    """metrics.py:25-54: running value with a mean / sum / max / min reduction; `compute()` resets."""

    def __init__(self, reduction: str = "mean"):
        if reduction not in ("mean", "sum", "max", "min"):
            raise ValueError(f"Invalid reduction: {reduction}")
        self.value = None
        self.count = 0
        self.reduction = reduction

    def update(self, value, count=1):
        if isinstance(value, torch.Tensor) and value.dtype in (torch.bfloat16, torch.float16):
            value = value.to(torch.float32)
        self.count += count
        if self.value is None:
            self.value = value
        elif self.reduction in ("mean", "sum"):
            self.value = self.value + value
        elif isinstance(value, torch.Tensor) or isinstance(self.value, torch.Tensor):
            pick = torch.maximum if self.reduction == "max" else torch.minimum
            self.value = pick(torch.as_tensor(self.value, device=value.device), value)
        else:
            self.value = max(self.value, value) if self.reduction == "max" else min(self.value, value)

    def compute(self):
        assert self.value is not None, "Record must be updated before computing"
        result = self.value / self.count if self.reduction == "mean" else self.value
        self.value = None
        self.count = 0
        return result


class Metric:
    def update(self, ctx: dict) -> dict:
        return {}

    def compute(self) -> dict[str, Any]:
        raise NotImplementedError("Subclasses must implement this method")


def _n_token_dims(sae, feature_acts: torch.Tensor, mask: Optional[torch.Tensor]) -> int:
    """Leading dims of feature_acts that index tokens: (batch[, context]); a layers axis (CLT) is not one."""
    if mask is not None:
        return mask.ndim
    has_layers = getattr(getattr(sae, "cfg", None), "n_layers", None) is not None and feature_acts.ndim >= 3
    return feature_acts.ndim - 1 - (1 if has_layers else 0)


def _token_weights(ctx) -> Optional[torch.Tensor]:
    mask = ctx.get("mask")
    return None if mask is None else mask.reshape(-1).to(torch.float32).contiguous()


def _code_totals(ctx, freq_acc: Optional[torch.Tensor] = None) -> torch.Tensor:
    """double[3] = (sum of activations, #positive, masked #positive) of this step's code; computed once per
    step and shared between the metrics through the context."""
    totals = ctx.get("_code_totals")
    if totals is None or freq_acc is not None:
        code = ctx["sparse_code"]
        fresh = torch.zeros(3, dtype=torch.float64, device=code.val.device)
        ops.code_stats(code, tok_w=_token_weights(ctx), freq_acc=freq_acc, totals=fresh if totals is None else None)
        if totals is None:
            totals = fresh
            ctx["_code_totals"] = totals
    return totals


class GradientNormMetric(Metric):
    """metrics.py:78-99.  Both norms stay device scalars until `compute()`.  A norm marked as deferred in the
    context is a tensor that the coming optimizer step fills in; it is folded into the running maxima at the
    next call, when it holds its value (the trainer never defers on a step that reports)."""

    def __init__(self, sae):
        self.sae = sae
        self.gradient_norm = Record("max")
        self.gradient_norm_before_clipping = Record("max")
        self._pending: Optional[torch.Tensor] = None

    def _fold(self) -> None:
        if self._pending is not None:
            self.gradient_norm_before_clipping.update(self._pending)
            self.gradient_norm.update(self._pending)
            self._pending = None

    def update(self, ctx):
        self._fold()
        before = ctx.get("grad_norm_before_clipping")
        assert before is not None, "Gradient norm before clipping must be provided"
        if ctx.get("grad_norm_is_deferred"):
            self._pending = before      # one value for both: nothing was clipped and no parameter was left out
            return {"gradient_norm_per_param": before, "gradient_norm_before_clipping": before}
        self.gradient_norm_before_clipping.update(before)
        norm = compute_grad_norm(self.sae.parameters())
        self.gradient_norm.update(norm)
        return {"gradient_norm_per_param": norm, "gradient_norm_before_clipping": before}

    def compute(self):
        assert self._pending is None, "a deferred gradient norm cannot be reported in the step that defers it"
        return {
            "metrics/gradient_norm_per_param": item(self.gradient_norm.compute()),
            "metrics/gradient_norm_before_clipping": item(self.gradient_norm_before_clipping.compute()),
        }


class FrequencyMetric(Metric):
    """metrics.py:102-149: per-feature firing frequency over the logging window and its threshold counts."""

    def __init__(self, sae):
        self.sae = sae
        self.act_freq_scores = Record()
        self._acc: Optional[torch.Tensor] = None   # sparse route: the kernel adds straight into this
        self._count = 0

    def update(self, ctx):
        if "sparse_code" in ctx:
            code = ctx["sparse_code"]
            if self._acc is None:
                self._acc = torch.zeros(code.d_sae, dtype=torch.float32, device=code.val.device)
            _code_totals(ctx, freq_acc=self._acc)
            self._count = self._count + ctx["n_tokens"]
            return {}
        feature_acts, mask = ctx["feature_acts"], ctx.get("mask")
        scores = apply_token_mask((feature_acts > 0).float(), _n_token_dims(self.sae, feature_acts, mask), mask, "sum")
        self.act_freq_scores.update(scores, ctx["n_tokens"])
        return {"act_freq_scores": scores}

    def compute(self):
        if self._acc is not None:
            feature_sparsity = self._acc / self._count
            self._acc, self._count = None, 0
        else:
            feature_sparsity = self.act_freq_scores.compute()
        return {
            "sparsity/above_1e-1": item((feature_sparsity > 1e-1).sum()),
            "sparsity/above_1e-2": item((feature_sparsity > 1e-2).sum()),
            "sparsity/below_1e-5": item((feature_sparsity < 1e-5).sum()),
            "sparsity/below_1e-6": item((feature_sparsity < 1e-6).sum()),
            "sparsity/below_1e-7": item((feature_sparsity < 1e-7).sum()),
        }


class LossMetric(Metric):
    """metrics.py:152-186."""

    def __init__(self, sae):
        self.sae = sae
        self.loss, self.l_rec, self.l_s, self.l_p, self.l_aux = Record(), Record(), Record(), Record(), Record()

    def update(self, ctx):
        self.loss.update(ctx["loss"].detach())
        self.l_rec.update(ctx["l_rec"].detach().mean())
        for name, rec in (("l_s", self.l_s), ("l_p", self.l_p), ("l_aux", self.l_aux)):
            v = ctx.get(name)
            if v is not None:
                rec.update(v.detach().mean())
        return {}

    def compute(self):
        out = {"losses/overall_loss": item(self.loss.compute()), "losses/mse_loss": item(self.l_rec.compute())}
        for key, rec in (("losses/sparsity_loss", self.l_s), ("losses/lp_loss", self.l_p), ("losses/aux_loss", self.l_aux)):
            if rec.value is not None:
                out[key] = item(rec.compute())
        return out


class MeanFeatureActMetric(Metric):
    """metrics.py:189-204: sum of activations / number of positive activations (unmasked), averaged over steps."""

    def __init__(self, sae):
        self.sae = sae
        self.mean_feature_act = Record()

    def update(self, ctx):
        if "sparse_code" in ctx:
            t = _code_totals(ctx)
            self.mean_feature_act.update((t[0] / t[1]).to(torch.float32))
        else:
            acts = ctx["feature_acts"]
            self.mean_feature_act.update(acts.sum() / acts.gt(0).float().sum())
        return {}

    def compute(self):
        return {"metrics/mean_feature_act": item(self.mean_feature_act.compute())}


def _layer_major(sae, ctx) -> bool:
    """Whether label / reconstruction carry a leading layer axis that is no token axis: a cross-layer transcoder's
    [layers, batch, d_model] (models/clt.py:54-69), whose metrics the reference forms per layer (the token mask spans
    the batch axis only) and averages over layers when it reports."""
    label, mask = ctx["label"], ctx.get("mask")
    if label.ndim < 3 or not hasattr(getattr(sae, "cfg", None), "n_layers"):
        return False
    return label.shape[0] == sae.cfg.n_layers and (mask is None or tuple(mask.shape) == tuple(label.shape[1:-1]))


def _recon_step_stats(ctx, layer_major: bool = False) -> torch.Tensor:
    """float[4] of this step: explained variance, legacy explained variance, L2 error, L2 error ratio
    (one kernel pass over label and reconstruction; shared by the two metrics that read them).  `layer_major`: one such
    row per layer, float[layers, 4] transposed to [4, layers], so that index i is statistic i either way."""
    st = ctx.get("_recon_step_stats")
    if st is None:
        label, recon = ctx["label"].detach(), ctx["reconstructed"].detach()
        w = _token_weights(ctx)

        def one(lab, rec):
            lab = lab.reshape(-1, lab.shape[-1]).to(torch.float32).contiguous()
            rec = rec.reshape(-1, rec.shape[-1]).to(torch.float32).contiguous()
            if w is None:
                mean = ops.col_sum(lab) / lab.shape[0]
            else:
                mean = ops.col_sum(lab * w[:, None]) / w.sum()
            acc = torch.zeros(4, dtype=torch.float64, device=lab.device)
            return ops.recon_stats(lab, rec, mean.contiguous(), acc, tok_w=w)

        if layer_major:
            st = torch.stack([one(label[l], recon[l]) for l in range(label.shape[0])]).t().contiguous()
        else:
            st = one(label, recon)
        ctx["_recon_step_stats"] = st
    return st


def _dense_recon_stats(ctx, layer_major: bool = False):
    label, recon, mask = ctx["label"], ctx["reconstructed"], ctx.get("mask")
    if layer_major:     # per layer, as the reference's specs reduce (layers, batch, model) over the batch axis only
        rows = [_dense_recon_stats({"label": label[l], "reconstructed": recon[l], "mask": mask}) for l in range(label.shape[0])]
        return tuple(torch.stack([r[i] for r in rows]) for i in range(4))
    ntd = label.ndim - 1
    label_mean = apply_token_mask(label, ntd, mask, "mean")
    se = (recon - label).pow(2).sum(dim=-1)
    var = (label - label_mean).pow(2).sum(dim=-1)
    legacy = apply_token_mask(1 - se / var, ntd, mask, "mean")
    ev = 1 - apply_token_mask(se, ntd, mask, "mean") / apply_token_mask(var, ntd, mask, "mean")
    err = apply_token_mask(se.sqrt(), ntd, mask, "mean")
    ratio = err / apply_token_mask(label.norm(p=2, dim=-1), ntd, mask, "mean")
    return ev, legacy, err, ratio


def _mean_if_vector(x):
    return x.mean() if isinstance(x, torch.Tensor) and x.numel() > 1 else x


def _on_gpu_2d(ctx) -> bool:
    label = ctx["label"]
    return label.is_cuda and label.dtype in (torch.float32, torch.bfloat16)


class ExplainedVarianceMetric(Metric):
    """metrics.py:207-255."""

    def __init__(self, sae):
        self.sae = sae
        self.explained_variance = Record()
        self.explained_variance_legacy = Record()

    def update(self, ctx):
        lm = _layer_major(self.sae, ctx)
        if _on_gpu_2d(ctx):
            st = _recon_step_stats(ctx, lm)
            ev, legacy = st[0], st[1]
        else:
            ev, legacy, _, _ = _dense_recon_stats(ctx, lm)
        self.explained_variance.update(ev)
        self.explained_variance_legacy.update(legacy)
        return {"explained_variance": ev, "explained_variance_legacy": legacy}

    def compute(self):
        return {
            "metrics/explained_variance": item(self.explained_variance.compute().mean()),
            "metrics/explained_variance_legacy": item(self.explained_variance_legacy.compute().mean()),
        }


class L0Metric(Metric):
    """metrics.py:258-288: (masked) number of positive activations per token, averaged over the window."""

    def __init__(self, sae):
        self.sae = sae
        self.l0 = Record()

    def update(self, ctx):
        if "sparse_code" in ctx:
            l0 = _code_totals(ctx)[2].to(torch.float32)
        else:
            acts, mask = ctx["feature_acts"], ctx.get("mask")
            l0 = apply_token_mask((acts > 0).float().sum(dim=-1), _n_token_dims(self.sae, acts, mask), mask, "sum")
        self.l0.update(l0, ctx["n_tokens"])
        return {"l0": l0}

    def compute(self):
        return {"metrics/l0": item(self.l0.compute().mean())}


class L2NormErrorMetric(Metric):
    """metrics.py:291-314."""

    def __init__(self, sae):
        self.sae = sae
        self.l2_norm_error = Record()
        self.l2_norm_error_ratio = Record()

    def update(self, ctx):
        lm = _layer_major(self.sae, ctx)
        if _on_gpu_2d(ctx):
            st = _recon_step_stats(ctx, lm)
            err, ratio = st[2], st[3]
        else:
            _, _, err, ratio = _dense_recon_stats(ctx, lm)
        self.l2_norm_error.update(err)
        self.l2_norm_error_ratio.update(ratio)
        return {}

    def compute(self):
        return {
            # a cross-layer transcoder has one value per layer here (the reference's `.item()` would refuse them):
            # reported as their mean, as the explained variance is
            "metrics/l2_norm_error": item(_mean_if_vector(self.l2_norm_error.compute())),
            "metrics/l2_norm_error_ratio": item(_mean_if_vector(self.l2_norm_error_ratio.compute())),
        }


class ModelSpecificMetric(Metric):
    """metrics.py:317-329: whatever the model's `compute_training_metrics(**ctx)` reports, averaged."""

    def __init__(self, sae):
        self.sae = sae
        self.metrics: dict[str, Record] = {}

    def update(self, ctx):
        fn = getattr(type(self.sae), "compute_training_metrics", None)
        from .sparse_dictionary import SparseDictionary
        if fn is None or fn is SparseDictionary.compute_training_metrics:
            return {}  # the base hook reports nothing: do not resolve the context's lazy dense views for it
        for k, v in self.sae.compute_training_metrics(**ctx).items():
            self.metrics.setdefault(k, Record()).update(v)
        return {}

    def compute(self):
        return {k: item(v.compute()) for k, v in self.metrics.items()}


def default_metrics(sae) -> list[Metric]:
    """The list `Trainer._log` builds on its first call (trainer.py:522-532), in the reference's order."""
    return [FrequencyMetric(sae), LossMetric(sae), MeanFeatureActMetric(sae), ExplainedVarianceMetric(sae),
            L0Metric(sae), L2NormErrorMetric(sae), ModelSpecificMetric(sae), GradientNormMetric(sae)]
