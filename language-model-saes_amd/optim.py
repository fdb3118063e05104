"""Optimisers of the train step on the HIP path.

`HipAdam` is `torch.optim.Adam` as the reference configures it (src/llamascopium/trainer.py:375-390:
lr, betas, eps 1e-8, no weight decay, no amsgrad) with the whole update of a parameter done by one
streaming kernel.  Its state uses torch.optim.Adam's key names (`step`, `exp_avg`, `exp_avg_sq`),
so optimizer checkpoints are interchangeable.

When a model is attached, the kernel that updates `W_E` / `W_D` also writes the bf16 copy the next
step's GEMM and row gathers read, and for `W_D` the per-feature L2 norm the next step's select
kernel scales by: both are by-products of data already in registers.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch.optim import Optimizer

from . import ops


def _flat_view(p: torch.Tensor) -> torch.Tensor:
    """A contiguous view over p's memory (p itself, or its transpose for feature-major 2-D weights)."""
    if p.is_contiguous():
        return p
    if p.ndim == 2 and p.t().is_contiguous():
        return p.t()
    raise ValueError(f"parameter with strides {p.stride()} is neither contiguous nor a transposed contiguous matrix")


class HipAdam(Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8, model=None):
        if lr < 0.0 or eps < 0.0 or not (0.0 <= betas[0] < 1.0) or not (0.0 <= betas[1] < 1.0):
            raise ValueError("invalid Adam hyper-parameters")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps))
        self._model = model
        self._roles: dict[int, str] = {}
        if model is not None:
            for name in ("W_E", "W_D"):
                p = getattr(model, name, None)
                if p is not None:
                    self._roles[id(p)] = name

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            b1, b2 = group["betas"]
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.dtype != torch.float32:
                    raise TypeError("HipAdam updates fp32 master parameters")
                st = self.state[p]
                if len(st) == 0:
                    st["step"] = torch.zeros((), dtype=torch.float32)
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                st["step"] += 1
                pv = _flat_view(p)
                same_layout = lambda t: _flat_view(t) if t.stride() == p.stride() else None  # noqa: E731
                gv, mv, vv = same_layout(p.grad), same_layout(st["exp_avg"]), same_layout(st["exp_avg_sq"])
                if gv is None:
                    gv = _flat_view(p.grad.contiguous()) if p.is_contiguous() else p.grad.t().contiguous()
                assert mv is not None and vv is not None, "optimizer state must share the parameter's layout"
                role = self._roles.get(id(p))
                shadow = norm_out = None
                row_len = 0
                if role is not None and pv.ndim == 2:
                    model = self._model
                    shadow = model.get_derived_buffer(f"{role}.bf16")
                    if role == "W_D":
                        norm_out = model.get_derived_buffer("W_D.norm")
                        if norm_out is None:
                            norm_out = torch.empty(pv.shape[0], dtype=torch.float32, device=p.device)
                        row_len = pv.shape[1] if pv.shape[1] % 4 == 0 else 0
                        if row_len == 0:
                            norm_out = None
                ops.adam_step(pv, gv, mv, vv, lr=group["lr"], beta1=b1, beta2=b2, eps=group["eps"],
                              step=int(st["step"].item()), shadow_bf16=shadow, row_norm_out=norm_out, row_len=row_len)
                # the kernel wrote through raw pointers: move the version counter like an in-place op would
                torch.autograd.graph.increment_version(p)
                if role is not None:
                    if shadow is not None:
                        self._model.set_derived(f"{role}.bf16", p, shadow)
                    if norm_out is not None:
                        self._model.set_derived("W_D.norm", p, norm_out)
        return loss
