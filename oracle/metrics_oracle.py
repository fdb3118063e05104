"""CPU oracle for the trainer's per-step metrics.  TEST INFRASTRUCTURE ONLY.

Restates, with dense torch CPU ops, what the reference's `Trainer._log` accumulates every step and
reports every `log_frequency` steps (`src/llamascopium/metrics.py`, `src/llamascopium/trainer.py:512-562`)
for a model whose `feature_acts` is `[batch, d_sae]` (the SAE): the per-feature firing frequency and its
threshold counts, mean feature activation, L0, explained variance (current and legacy), L2-norm error and
ratio, the loss means, and the gradient-norm maxima.  Nothing in the product package may import it.

Pinning status (tests/test_oracle_metrics.py):
  * frequency / L0 / mean act ... pinned by hand cases and a scalar-loop count
  * explained variance .......... pinned by closed forms: perfect reconstruction -> 1, reconstruction =
                                  the (masked) label mean -> 0 for the pooled form, label scaled by c about
                                  its mean -> 1 - (1 - c)^2, and an fp64 scalar-loop restatement
  * L2 error and ratio .......... pinned by a 3-4-5 hand case and recon = 0 -> ratio 1
  * Record ...................... pinned by hand sequences (mean / sum / max / min, reset on compute)
"""

from __future__ import annotations

from typing import Optional

import torch

from .sae_oracle import apply_token_mask


class Record:
    """metrics.py:22-54."""

    def __init__(self, reduction: str = "mean"):
        self.value = None
        self.count = 0
        self.reduction = reduction

    def update(self, value, count=1):
        if isinstance(value, torch.Tensor) and value.dtype in (torch.bfloat16, torch.float16):
            value = value.to(torch.float32)
        self.count += count
        if self.reduction in ("mean", "sum"):
            self.value = self.value + value if self.value is not None else value
        elif self.reduction == "max":
            self.value = max(self.value, value) if self.value is not None else value
        elif self.reduction == "min":
            self.value = min(self.value, value) if self.value is not None else value
        else:
            raise ValueError(f"Invalid reduction: {self.reduction}")

    def compute(self):
        assert self.value is not None, "Record must be updated before computing"
        result = self.value / self.count if self.reduction == "mean" else self.value
        self.value, self.count = None, 0
        return result


def act_freq_scores(feature_acts: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """metrics.py:113-118: number of (unmasked) tokens on which each feature is positive, [d_sae]."""
    return apply_token_mask((feature_acts > 0).float(), 1, mask, "sum")


def sparsity_thresholds(feature_sparsity: torch.Tensor) -> dict:
    """metrics.py:123-130."""
    return {
        "sparsity/above_1e-1": int((feature_sparsity > 1e-1).sum()),
        "sparsity/above_1e-2": int((feature_sparsity > 1e-2).sum()),
        "sparsity/below_1e-5": int((feature_sparsity < 1e-5).sum()),
        "sparsity/below_1e-6": int((feature_sparsity < 1e-6).sum()),
        "sparsity/below_1e-7": int((feature_sparsity < 1e-7).sum()),
    }


def mean_feature_act(feature_acts: torch.Tensor) -> torch.Tensor:
    """metrics.py:194-198 (the mask is not applied here in the reference)."""
    return feature_acts.sum() / feature_acts.gt(0).float().sum()


def l0_sum(feature_acts: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """metrics.py:268-276: masked token sum of the positive-activation indicator, then summed over d_sae."""
    return act_freq_scores(feature_acts, mask).sum()


def explained_variance(label: torch.Tensor, reconstructed: torch.Tensor, mask: Optional[torch.Tensor]):
    """metrics.py:214-243 -> (explained_variance, explained_variance_legacy)."""
    label_mean = apply_token_mask(label, 1, mask, "mean")
    per_token_l2_loss = (reconstructed - label).pow(2).sum(dim=-1)
    total_variance = (label - label_mean).pow(2).sum(dim=-1)
    legacy = apply_token_mask(1 - per_token_l2_loss / total_variance, 1, mask, "mean")
    l2_mean = apply_token_mask(per_token_l2_loss, 1, mask, "mean")
    var_mean = apply_token_mask(total_variance, 1, mask, "mean")
    return 1 - l2_mean / var_mean, legacy


def l2_norm_error(label: torch.Tensor, reconstructed: torch.Tensor, mask: Optional[torch.Tensor]):
    """metrics.py:297-303 -> (l2_norm_error, l2_norm_error_ratio)."""
    err = apply_token_mask((reconstructed - label).pow(2).sum(dim=-1).sqrt(), 1, mask, "mean")
    return err, err / apply_token_mask(label.norm(p=2, dim=-1), 1, mask, "mean")


class StepMetrics:
    """The SAE part of `Trainer._log`'s metric list (trainer.py:522-562), fed one step's context at a time."""

    def __init__(self):
        self.freq, self.l0 = Record(), Record()
        self.mean_act = Record()
        self.ev, self.ev_legacy = Record(), Record()
        self.err, self.err_ratio = Record(), Record()
        self.loss, self.l_rec, self.l_aux = Record(), Record(), Record()
        self.gn, self.gn_before = Record("max"), Record("max")

    def update(self, *, feature_acts, label, reconstructed, mask, n_tokens, loss, l_rec, l_aux=None,
               grad_norm_before_clipping=None, grad_norm=None):
        self.freq.update(act_freq_scores(feature_acts, mask), n_tokens)
        self.loss.update(loss)
        self.l_rec.update(l_rec.mean())
        if l_aux is not None:
            self.l_aux.update(l_aux.mean())
        self.mean_act.update(mean_feature_act(feature_acts))
        ev, legacy = explained_variance(label, reconstructed, mask)
        self.ev.update(ev)
        self.ev_legacy.update(legacy)
        self.l0.update(l0_sum(feature_acts, mask), n_tokens)
        err, ratio = l2_norm_error(label, reconstructed, mask)
        self.err.update(err)
        self.err_ratio.update(ratio)
        if grad_norm_before_clipping is not None:
            self.gn_before.update(float(grad_norm_before_clipping))
            self.gn.update(float(grad_norm))

    def compute(self) -> dict:
        out = sparsity_thresholds(self.freq.compute())
        out["losses/overall_loss"] = float(self.loss.compute())
        out["losses/mse_loss"] = float(self.l_rec.compute())
        if self.l_aux.value is not None:
            out["losses/aux_loss"] = float(self.l_aux.compute())
        out["metrics/mean_feature_act"] = float(self.mean_act.compute())
        out["metrics/explained_variance"] = float(self.ev.compute().mean())
        out["metrics/explained_variance_legacy"] = float(self.ev_legacy.compute().mean())
        out["metrics/l0"] = float(self.l0.compute().mean())
        out["metrics/l2_norm_error"] = float(self.err.compute())
        out["metrics/l2_norm_error_ratio"] = float(self.err_ratio.compute())
        if self.gn.value is not None:
            out["metrics/gradient_norm_per_param"] = float(self.gn.compute())
            out["metrics/gradient_norm_before_clipping"] = float(self.gn_before.compute())
        return out
