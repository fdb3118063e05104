"""Seeded synthetic activations and weight initialisation for benchmarks, smoke runs and tests.

Activation generator G(d, r, seed): x = 0.05 * N(0, 1)^{B x d} + z U^T with U in R^{d x r} the
Q factor of a seeded Gaussian (orthonormal columns) and z ~ N(0, 4); rows rescaled to norm sqrt(d).
Weights: W_E ~ U(-1/sqrt(d), 1/sqrt(d)) (the nn.Linear default bound), W_D = W_E^T with rows
normalised to unit L2, b_E = 0, b_D = mean of x.  Everything is drawn on the CPU generator so that
a CPU checker and the GPU path see identical inputs.
"""

from __future__ import annotations

import math

import torch


def activations(B: int, d: int, r: int, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    U, _ = torch.linalg.qr(torch.randn(d, r, generator=g))
    z = 2.0 * torch.randn(B, r, generator=g)
    x = 0.05 * torch.randn(B, d, generator=g) + z @ U.t()
    return x * (math.sqrt(d) / x.norm(dim=-1, keepdim=True))


def sae_weights(d: int, F: int, x: torch.Tensor, seed: int):
    """Returns (W_E^T [F, d], b_E [F], W_D [F, d], b_D [d]) as fp32 CPU tensors."""
    g = torch.Generator().manual_seed(seed + 7919)
    bound = 1.0 / math.sqrt(d)
    w_enc_t = (torch.rand(F, d, generator=g) * 2 - 1) * bound
    w_dec = w_enc_t / w_enc_t.norm(dim=1, keepdim=True)
    return w_enc_t, torch.zeros(F), w_dec.contiguous(), x.mean(0)


@torch.no_grad()
def load_weights(model, w_enc_t, b_E, W_D, b_D) -> None:
    """Copy (feature-major) weights into a SparseAutoEncoder-like module, whatever its layout."""
    model.W_E.copy_(w_enc_t.t())
    model.b_E.copy_(b_E)
    model.W_D.copy_(W_D)
    if getattr(model, "b_D", None) is not None:
        model.b_D.copy_(b_D)
