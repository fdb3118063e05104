"""Trainer step shell around the fused train step.

The parts of the reference's `Trainer` (src/llamascopium/trainer.py) that sit on the hot loop:
the k-annealing schedule and l1 warm-up of `_training_step` (:457-510), the dead-latent statistics
behind the aux-k loss (:403-454), optimizer / LR-schedule construction (:349-401, optim.py:23-139)
the loop body of `fit` (:605-665) and complete checkpoints with resuming (:155-307).  Logging sinks, wandb and the
progress bar are not part of this path; `fit` reports through an optional callback instead, and never forces a
device synchronisation on its own (the reference syncs every step for its progress bar).
"""

from __future__ import annotations

import json
import math
import os
from pathlib import Path
from typing import Callable, Iterable, Literal, Optional, Tuple

import torch
from pydantic import BaseModel, ConfigDict, Field
from torch.optim import lr_scheduler

from . import ops
from .config import TorchDtype
from .metrics import default_metrics
from .optim import HipAdam, HipSparseAdam, clip_grad_norm
from .sparse_dictionary import SparseDictionary, apply_token_mask


class TrainerConfig(BaseModel):
    model_config = ConfigDict(arbitrary_types_allowed=True)

    l1_coefficient: Optional[float] = 0.00008
    l1_coefficient_warmup_steps: int | float = 0.1
    lp_coefficient: Optional[float] = None
    auxk_coefficient: Optional[float] = None
    amp_dtype: Optional[TorchDtype] = Field(default=torch.bfloat16, exclude=True, validate_default=False)
    sparsity_loss_type: Literal["power", "tanh", "tanh-quad", None] = None
    tanh_stretch_coefficient: float = 4.0
    frequency_scale: float = 0.01
    p: int = 1
    initial_k: int | float | None = None
    k_warmup_steps: int | float = 0.1
    k_cold_booting_steps: int | float = 0
    k_schedule_type: Literal["linear", "exponential"] = "linear"
    k_exponential_factor: float = 3.0
    k_aux: int = 512
    dead_threshold: float = 10_000_000
    skip_metrics_calculation: bool = False
    lr: float = 0.0004
    betas: Tuple[float, float] = (0.9, 0.999)
    # "adam" / "sparseadam" as in the reference; both map to the HIP kernels
    optimizer_class: Literal["adam", "sparseadam"] = "adam"
    optimizer_foreach: bool = True
    lr_scheduler_name: Literal["constant", "constantwithwarmup", "constantwithwarmupsmooth", "linearwarmupdecay",
                               "cosineannealing", "cosineannealingwarmup", "cosineannealingwarmrestarts",
                               "exponentialwarmup"] = "constantwithwarmup"
    lr_end_ratio: float = 1 / 32
    lr_warm_up_steps: int | float = 5000
    lr_cool_down_steps: int | float = 0.2
    jumprelu_lr_factor: float = 1.0
    clip_grad_norm: float = 0.0
    total_training_tokens: int = 300_000_000
    log_frequency: int = 1000
    # checkpoints (trainer.py:107-124): model weights at `n_checkpoints` thresholds under exp_result_path/checkpoints;
    # a directory written by `Trainer.save_checkpoint` is resumed from with `from_pretrained_path`
    n_checkpoints: int = 0
    check_point_save_mode: Literal["log", "linear"] = "log"
    from_pretrained_path: Optional[str] = None
    exp_result_path: str = "results"

    def model_post_init(self, __context):
        assert self.lr_end_ratio <= 1, "lr_end_ratio must be in 0 to 1 (inclusive)."
        if self.from_pretrained_path is not None:
            assert os.path.exists(self.from_pretrained_path), f"from_pretrained_path {self.from_pretrained_path} does not exist"


def get_scheduler(scheduler_name: Optional[str], optimizer, **kwargs):
    """LambdaLR factories with the reference's formulas (src/llamascopium/optim.py:23-139)."""
    name = (scheduler_name or "constant").lower()
    warm = kwargs.get("warm_up_steps", 0)
    total = kwargs.get("training_steps")
    if name == "constant":
        return lr_scheduler.LambdaLR(optimizer, lr_lambda=lambda steps: 1.0)
    assert total is not None, "training_steps must be provided"
    if name == "constantwithwarmup":
        cool = kwargs.get("cool_down_steps", 0)
        end = kwargs.get("lr_end_ratio", 0.0)
        return lr_scheduler.LambdaLR(
            optimizer,
            lr_lambda=lambda steps: min(1.0, (steps + 1) / warm, end + (1 - end) / cool * max(total - steps, 1)),
        )
    if name == "constantwithwarmupsmooth":
        # two-piece warm-up (a line up to gamma * warm, then a parabola that lands flat on 1 at warm), a plateau,
        # and a cosine decay to 0 over the last 1.5 * warm steps; gamma = 0.5
        gamma = 0.5
        cool_from = total - int(1.5 * warm)

        def smooth(steps):
            if steps < gamma * warm:
                return 2 * (steps + 1) / (warm * (1 + gamma))
            if steps < warm:
                return 1 - ((steps / warm - 1) ** 2) / (1 - gamma ** 2)
            if steps < cool_from:
                return 1.0
            return 0.5 * (1 + math.cos(math.pi * (steps - cool_from) / (total - cool_from)))
        return lr_scheduler.LambdaLR(optimizer, smooth)
    if name == "cosineannealingwarmrestarts":
        return lr_scheduler.CosineAnnealingWarmRestarts(optimizer, T_0=total // kwargs.get("num_cycles", 1),
                                                        eta_min=kwargs.get("lr_end", 0))
    if name == "linearwarmupdecay":
        return lr_scheduler.LambdaLR(
            optimizer, lambda steps: (steps + 1) / warm if steps < warm else (total - steps) / (total - warm))
    if name == "cosineannealing":
        return lr_scheduler.CosineAnnealingLR(optimizer, T_max=total, eta_min=kwargs.get("lr_end", 0))
    if name == "cosineannealingwarmup":
        end = kwargs.get("lr_end", 0)

        def lam(steps):
            if steps < warm:
                return (steps + 1) / warm
            return end + 0.5 * (1 - end) * (1 + math.cos(math.pi * (steps - warm) / (total - warm)))
        return lr_scheduler.LambdaLR(optimizer, lam)
    if name == "exponentialwarmup":
        end = kwargs.get("lr_end", 1 / 32)
        return lr_scheduler.LambdaLR(
            optimizer, lambda steps: (steps + 1) / warm if steps < warm else math.pow(end, (steps - warm) / (total - warm)))
    raise ValueError(f"Unsupported scheduler: {scheduler_name}")


class Trainer:
    def __init__(self, cfg: TrainerConfig):
        self.cfg = cfg
        self.checkpoint_thresholds: list[int] = []
        self.cur_step = 0
        self.cur_tokens = 0
        self.total_training_steps = 0
        self.lr_warm_up_steps = self.lr_cool_down_steps = 0
        self.k_warmup_steps = self.k_cold_booting_steps = 0
        self.l1_coefficient_warmup_steps = 0
        self.optimizer = None
        self.scheduler = None
        self.tokens_since_last_activation: Optional[torch.Tensor] = None
        self.is_dead: Optional[torch.Tensor] = None
        self.metrics: list = []
        self.log_sink: Optional[Callable[[int, dict], None]] = None   # receives (step, metrics) every log_frequency steps
        self.last_logged: Optional[dict] = None

    # ---- trainer.py:310-346 ----
    def _initialize_trainer(self, sae: SparseDictionary, first_batch: dict):
        bs = first_batch["tokens"].numel()
        self.total_training_steps = self.cfg.total_training_tokens // bs

        def steps(v):
            if isinstance(v, float):
                assert 0 <= v <= 1.0
                return int(v * self.total_training_steps)
            return v

        self.lr_warm_up_steps = steps(self.cfg.lr_warm_up_steps)
        self.lr_cool_down_steps = steps(self.cfg.lr_cool_down_steps)
        self.k_warmup_steps = steps(self.cfg.k_warmup_steps)
        self.k_cold_booting_steps = steps(self.cfg.k_cold_booting_steps)
        self.l1_coefficient_warmup_steps = steps(self.cfg.l1_coefficient_warmup_steps)
        if self.cfg.n_checkpoints > 0:
            n, total = self.cfg.n_checkpoints, self.total_training_steps
            if self.cfg.check_point_save_mode == "linear":
                self.checkpoint_thresholds = list(range(0, total, total // n))[1:]
            else:   # "log": the reference multiplies these step counts by the batch size (trainer.py:339-343) and
                # compares them with the step counter; kept as it is
                self.checkpoint_thresholds = [math.ceil(2 ** (i / n * math.log2(total))) * bs for i in range(1, n)]

    # ---- trainer.py:155-307: a complete checkpoint (model, optimizer, scheduler, trainer state) and resuming ----
    _STATE_KEYS = ("cur_step", "cur_tokens", "total_training_steps", "lr_warm_up_steps", "lr_cool_down_steps",
                   "k_warmup_steps", "k_cold_booting_steps", "l1_coefficient_warmup_steps", "checkpoint_thresholds")

    def save_checkpoint(self, sae: SparseDictionary, checkpoint_path) -> Path:
        """Writes <checkpoint_path>/checkpoints/step_<cur_step>/ with the reference's file set: the model's
        hyper-parameters and `sae_weights.safetensors`, `trainer.pt`, `optimizer.pt`, `scheduler.pt`.  `trainer.pt`
        holds the trainer's counters and its config as a plain dict (the reference pickles the config object, which
        only its own package can read back); the optimizer file is a torch.optim.Adam state dict.  Returns the
        directory."""
        ckpt = Path(checkpoint_path) / "checkpoints" / f"step_{self.cur_step}"
        os.makedirs(ckpt, exist_ok=True)
        if self.optimizer is not None and hasattr(self.optimizer, "join"):
            self.optimizer.join()
        sae.cfg.save_hyperparameters(ckpt)
        sae.save_checkpoint(ckpt / "sae_weights.safetensors")
        state = {k: getattr(self, k) for k in self._STATE_KEYS}
        state["cfg"] = self.cfg.model_dump()
        state["amp_dtype"] = None if self.cfg.amp_dtype is None else str(self.cfg.amp_dtype)
        torch.save(state, ckpt / "trainer.pt")
        if self.optimizer is not None:
            torch.save(self.optimizer.state_dict(), ckpt / "optimizer.pt")
        if self.scheduler is not None:
            torch.save(self.scheduler.state_dict(), ckpt / "scheduler.pt")
        return ckpt

    @classmethod
    def from_checkpoint(cls, sae: SparseDictionary, checkpoint_path) -> "Trainer":
        """A trainer that continues where `save_checkpoint` stopped: counters and config from `trainer.pt`, a fresh
        optimizer and scheduler for `sae` (whose weights the caller loads from the same directory) with their saved
        states loaded.  `fit` then skips its own initialisation (cfg.from_pretrained_path is set)."""
        ckpt = Path(checkpoint_path)
        if not os.path.exists(ckpt / "trainer.pt"):
            raise ValueError(f"Trainer checkpoint not found at {ckpt / 'trainer.pt'}")
        state = torch.load(ckpt / "trainer.pt", map_location="cpu", weights_only=True)
        cfg = state.get("cfg")
        if cfg is None:
            raise ValueError("Checkpoint does not contain trainer config")
        cfg = dict(cfg)
        amp = state.get("amp_dtype")
        cfg["amp_dtype"] = None if amp is None else getattr(torch, str(amp).replace("torch.", ""))
        cfg["from_pretrained_path"] = str(checkpoint_path)
        trainer = cls(TrainerConfig(**cfg))
        for k in cls._STATE_KEYS:
            setattr(trainer, k, state[k])
        trainer._initialize_optimizer(sae)
        trainer.optimizer.load_state_dict(torch.load(ckpt / "optimizer.pt", map_location="cpu", weights_only=True))
        trainer.scheduler.load_state_dict(torch.load(ckpt / "scheduler.pt", map_location="cpu", weights_only=True))
        return trainer

    def _maybe_save_sae_checkpoint(self, sae: SparseDictionary) -> None:
        """trainer.py:563-574: the model's weights each time the step counter passes the next threshold."""
        if self.checkpoint_thresholds and self.cur_step >= self.checkpoint_thresholds[0]:
            path = os.path.join(self.cfg.exp_result_path, "checkpoints", f"{self.cur_step}.safetensors")
            os.makedirs(os.path.dirname(path), exist_ok=True)
            sae.save_checkpoint(path)
            self.checkpoint_thresholds.pop(0)

    # ---- trainer.py:349-401 ----
    def _initialize_optimizer(self, sae: SparseDictionary):
        groups = []
        for g in sae.get_parameters():
            if g["name"] == "jumprelu":
                g = {**g, "lr": self.cfg.jumprelu_lr_factor * self.cfg.lr}
            if len(g["params"]) > 0:
                groups.append(g)
        cls = {"adam": HipAdam, "sparseadam": HipSparseAdam}[self.cfg.optimizer_class]
        self.optimizer = cls(groups, lr=self.cfg.lr, betas=self.cfg.betas, model=sae)
        self.scheduler = get_scheduler(
            self.cfg.lr_scheduler_name, self.optimizer, warm_up_steps=self.lr_warm_up_steps,
            cool_down_steps=self.lr_cool_down_steps, training_steps=self.total_training_steps,
            lr_end_ratio=self.cfg.lr_end_ratio)

    # ---- trainer.py:403-454 ----
    def _initialize_dead_statistics(self, sae: SparseDictionary) -> None:
        dev = next(sae.parameters()).device
        self.tokens_since_last_activation = torch.zeros(sae.cfg.d_sae, device=dev, dtype=torch.long)
        self.is_dead = torch.zeros(sae.cfg.d_sae, device=dev, dtype=torch.bool)

    def _advance_dead_statistics(self, activated: torch.Tensor, valid_tokens) -> torch.Tensor:
        self.tokens_since_last_activation = torch.where(
            activated, torch.zeros_like(self.tokens_since_last_activation), self.tokens_since_last_activation + valid_tokens)
        self.is_dead = self.tokens_since_last_activation >= self.cfg.dead_threshold
        return self.is_dead

    @torch.no_grad()
    def update_dead_statistics(self, feature_acts: torch.Tensor, mask: Optional[torch.Tensor], specs) -> torch.Tensor:
        """Dense form, signature of the reference."""
        assert self.tokens_since_last_activation is not None, (
            "tokens_since_last_activation must be initialized before calling update_dead_statistics")
        valid = mask.sum() if mask is not None else feature_acts[..., 0].numel()
        acts_sum = apply_token_mask(feature_acts, feature_acts.ndim - 1, mask, "sum")
        return self._advance_dead_statistics(acts_sum.gt(0), valid)

    @torch.no_grad()
    def update_dead_statistics_sparse(self, code: ops.SparseCode, mask: Optional[torch.Tensor]) -> torch.Tensor:
        """Same statistics from the sparse code: a feature fired when its (masked) activations sum above 0."""
        assert self.tokens_since_last_activation is not None, (
            "tokens_since_last_activation must be initialized before calling update_dead_statistics")
        B = code.n_tokens
        slots = torch.arange(code.n_slots, device=code.val.device)
        tok = torch.searchsorted(code.row_off, slots, right=True) - 1
        valid_slot = (slots - code.row_off[tok]) < code.row_nnz[tok]
        vals = torch.where(valid_slot, code.val, torch.zeros_like(code.val))
        if mask is not None:
            vals = vals * mask.reshape(-1).to(vals)[tok]
        acts_sum = torch.zeros(code.d_sae, dtype=torch.float32, device=vals.device).index_add_(
            0, torch.where(valid_slot, code.idx.long(), torch.zeros_like(tok)), vals)
        valid = mask.sum() if mask is not None else B
        return self._advance_dead_statistics(acts_sum.gt(0), valid)

    # ---- trainer.py:457-510 ----
    def _training_step(self, sae: SparseDictionary, batch: dict) -> dict:
        if "topk" in sae.cfg.act_fn and self.k_warmup_steps > 0:
            assert self.cfg.initial_k is not None, "initial_k must be provided"
            assert self.cfg.initial_k >= sae.cfg.top_k, "initial_k must be greater than or equal to top_k"
            if self.cur_step < self.k_cold_booting_steps:
                sae.set_current_k(int(self.cfg.initial_k))
            else:
                progress = min(1.0, (self.cur_step - self.k_cold_booting_steps) / self.k_warmup_steps)
                if self.cfg.k_schedule_type == "exponential":
                    f = self.cfg.k_exponential_factor
                    decay = (1.0 - math.exp(-f * progress)) / (1.0 - math.exp(-f))
                    cur = self.cfg.initial_k - (self.cfg.initial_k - sae.cfg.top_k) * decay
                else:
                    cur = self.cfg.initial_k + (sae.cfg.top_k - self.cfg.initial_k) * progress
                sae.set_current_k(max(sae.cfg.top_k, math.ceil(cur)))
        l1 = (min(1.0, self.cur_step / self.l1_coefficient_warmup_steps) * self.cfg.l1_coefficient
              if self.cfg.l1_coefficient is not None else 1.0)
        lp = self.cfg.lp_coefficient if self.cfg.lp_coefficient is not None else 0.0
        auxk = self.cfg.auxk_coefficient if self.cfg.auxk_coefficient is not None else 0.0
        return sae.compute_loss(
            batch, sparsity_loss_type=self.cfg.sparsity_loss_type, tanh_stretch_coefficient=self.cfg.tanh_stretch_coefficient,
            p=self.cfg.p, return_aux_data=True, l1_coefficient=l1, lp_coefficient=lp, auxk_coefficient=auxk,
            frequency_scale=self.cfg.frequency_scale, k_aux=self.cfg.k_aux,
            update_dead_statistics=self.update_dead_statistics if auxk > 0.0 else None)

    # ---- trainer.py:512-562 ----
    @torch.no_grad()
    def _log(self, sae: SparseDictionary, ctx: dict) -> None:
        """Update every metric with this step's context; every `log_frequency` steps reduce them to
        numbers (the only host synchronisation of the logging path) and hand them to `log_sink`."""
        if not self.metrics:
            self.metrics = default_metrics(sae)
        for metric in self.metrics:
            ctx.update(metric.update(ctx))
        if (self.cur_step + 1) % self.cfg.log_frequency == 0:
            out: dict = {}
            for metric in self.metrics:
                out.update(metric.compute())
            out.update({
                "details/current_learning_rate": self.optimizer.param_groups[0]["lr"],
                "details/n_training_tokens": self.cur_tokens,
                "details/l1_coefficient": ctx.get("l1_coefficient"),
                "details/lp_coefficient": ctx.get("lp_coefficient"),
                "details/auxk_coefficient": ctx.get("auxk_coefficient"),
            })
            if hasattr(sae, "log_statistics"):
                out.update(sae.log_statistics())
            self.last_logged = out
            if self.log_sink is not None:
                self.log_sink(self.cur_step + 1, out)

    # ---- trainer.py:576-671 (loop body; no progress bar, files or wandb) ----
    def fit(self, sae: SparseDictionary, activation_stream: Iterable[dict],
            on_step: Optional[Callable[[int, dict], None]] = None) -> Optional[bool]:
        stream = iter(activation_stream)
        try:
            batch = next(stream)
        except StopIteration:
            return True
        self.prepare(sae, batch)
        try:
            while True:
                self.train_one_step(sae, batch, on_step)
                self._maybe_save_sae_checkpoint(sae)
                if self.cur_step >= self.total_training_steps:
                    break
                batch = next(stream)
        except StopIteration:
            return True
        return None

    def prepare(self, sae: SparseDictionary, first_batch: dict) -> None:
        """What `fit` sets up before its first step: step counts, optimizer, scheduler, dead statistics."""
        if self.optimizer is None:
            self._initialize_trainer(sae, first_batch)
            self._initialize_optimizer(sae)
        if self.cfg.auxk_coefficient is not None and self.cfg.auxk_coefficient > 0.0 and self.is_dead is None:
            self._initialize_dead_statistics(sae)

    def train_one_step(self, sae: SparseDictionary, batch: dict,
                       on_step: Optional[Callable[[int, dict], None]] = None) -> dict:
        """The body of the reference's loop (trainer.py:605-660) for one batch."""
        batch = sae.normalize_activations(batch)
        sae.train()
        if self.cfg.amp_dtype is not None and self.cfg.amp_dtype != torch.float32:
            with torch.autocast(device_type=next(sae.parameters()).device.type, dtype=self.cfg.amp_dtype):
                ctx = self._training_step(sae, batch)
        else:
            ctx = self._training_step(sae, batch)
        ctx["loss"].backward()
        # every step, as the reference does (trainer.py:629-639); factored weight gradients are reduced where they
        # are, nothing dense is materialised; the jumprelu threshold is excluded.  Without clipping the value is only
        # logged, so it is taken as a by-product of the optimizer step (valid once `optimizer.step()` has run).
        named = list(sae.named_parameters())
        clipped = [p for n, p in named if "log_jumprelu_threshold" not in n]
        reports = not self.cfg.skip_metrics_calculation and (self.cur_step + 1) % self.cfg.log_frequency == 0
        can_defer = (self.cfg.clip_grad_norm <= 0 and hasattr(self.optimizer, "deferred_grad_norm") and not reports
                     and on_step is None and len(clipped) == len(named))
        if can_defer:
            ctx["grad_norm_before_clipping"] = self.optimizer.deferred_grad_norm(clipped)
            ctx["grad_norm_is_deferred"] = True
        else:
            ctx["grad_norm_before_clipping"] = clip_grad_norm(
                clipped, max_norm=self.cfg.clip_grad_norm if self.cfg.clip_grad_norm > 0 else math.inf)
        if not self.cfg.skip_metrics_calculation:
            self._log(sae, ctx)
        if on_step is not None:
            on_step(self.cur_step, ctx)
        self.optimizer.step()
        self.optimizer.zero_grad()
        self.scheduler.step()
        self.cur_step += 1
        self.cur_tokens += batch["tokens"].numel() if batch.get("mask") is None else int(batch["mask"].sum().item())
        return ctx
