"""A minimal HookPoint: an identity module that user hooks can observe or replace.

Stands in for transformer_lens.hook_points.HookPoint, which the reference's models use for
`hook_hidden_pre`, `hook_feature_acts` and `hook_reconstructed` (models/sae.py:131-134).
While no hook is registered the fused kernels may skip the tensor entirely.
"""

from __future__ import annotations

from typing import Callable

import torch
from torch import nn


class HookPoint(nn.Module):
    def __init__(self):
        super().__init__()
        self.fwd_hooks: list[Callable] = []
        self.name: str | None = None

    def add_hook(self, hook: Callable[[torch.Tensor, "HookPoint"], torch.Tensor | None]) -> None:
        self.fwd_hooks.append(hook)

    def remove_hooks(self) -> None:
        self.fwd_hooks.clear()

    @property
    def has_hooks(self) -> bool:
        return len(self.fwd_hooks) > 0

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        for h in self.fwd_hooks:
            out = h(x, self)
            if out is not None:
                x = out
        return x
