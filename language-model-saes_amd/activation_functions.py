"""Activation callables of the sparse dictionaries.

`JumpReLU` keeps the reference's module interface (activation_functions.py:67-140): a learnable
`log_jumprelu_threshold` and the rectangle-window straight-through gradient of `STEFunction`
(activation_functions.py:15-64).  `topk_dense` / `batch_topk_dense` are the dense-in/dense-out
forms of the TopK closures (models/sparse_dictionary.py:733-794), backed by the HIP select
kernel; the fused train step does not go through them (it never materialises the dense output).
"""

from __future__ import annotations

import torch

from . import ops


class STEFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, theta, window: float, dims_to_keep_in_bwd):
        mask = x.gt(theta)
        ctx.save_for_backward(x, theta, mask)
        ctx.window = window
        ctx.dims_to_keep_in_bwd = dims_to_keep_in_bwd
        return x * mask

    @staticmethod
    def backward(ctx, g):
        x, theta, mask = ctx.saved_tensors
        w = ctx.window
        in_window = ((x - theta).abs() < w * 0.5) & (x > 0.0)
        g_theta = torch.where(in_window, -theta / w, torch.zeros((), dtype=x.dtype, device=x.device)) * g
        keep = ctx.dims_to_keep_in_bwd
        drop = tuple(i for i in range(g_theta.ndim) if i not in keep and i - g_theta.ndim not in keep)
        return g * mask, g_theta.sum(dim=drop), None, None


class JumpReLU(torch.nn.Module):
    def __init__(self, jumprelu_threshold_window: float, *, shape, dims_to_keep_in_bwd=(-1,), device=None,
                 dtype=torch.float32, device_mesh=None):
        super().__init__()
        if device_mesh is not None:
            raise NotImplementedError("single-GPU build: device meshes are not supported")
        self.jumprelu_threshold_window = jumprelu_threshold_window
        self.shape = tuple(shape)
        self.dims_to_keep_in_bwd = tuple(dims_to_keep_in_bwd)
        self.dtype = dtype
        assert len(self.dims_to_keep_in_bwd) == len(self.shape), (
            f"dims_to_keep_in_bwd must have the same length as shape, got {self.dims_to_keep_in_bwd} and {self.shape}"
        )
        self.log_jumprelu_threshold = torch.nn.Parameter(torch.empty(self.shape, device=device, dtype=dtype))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = STEFunction.apply(x.to(self.dtype), self.log_jumprelu_threshold.exp(), self.jumprelu_threshold_window,
                              self.dims_to_keep_in_bwd)
        return y.to(x.dtype)

    def get_jumprelu_threshold(self) -> torch.Tensor:
        return self.log_jumprelu_threshold.exp()


class _TopKDense(torch.autograd.Function):
    """Dense [.., F] -> dense [.., F] per-token TopK through the select kernel.

    Matches `x * 1[x>0]` followed by utils/math.py:81-171 with dim=-1: kept entries pass their
    gradient through unchanged, everything else gets zero.
    """

    @staticmethod
    def forward(ctx, x: torch.Tensor, k: int):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        if x2.dtype not in (torch.float32, torch.bfloat16):
            x2 = x2.float()
        x2 = x2.contiguous()
        code = ops.select_topk_row(x2, None, None, min(int(k), shape[-1]))
        ctx.code = code
        ctx.in_dtype = x.dtype
        return code.to_dense().to(x.dtype).reshape(shape)

    @staticmethod
    def backward(ctx, g):
        code = ctx.code
        mask = code.to_dense() > 0
        return (g.reshape(mask.shape) * mask).reshape(g.shape).to(ctx.in_dtype), None


def topk_dense(x: torch.Tensor, k: int) -> torch.Tensor:
    return _TopKDense.apply(x, k)


def _topk_mask_lowest_index(x_flat: torch.Tensor, k: int) -> torch.Tensor:
    k = min(int(k), x_flat.shape[-1])
    order = torch.sort(x_flat, dim=-1, descending=True, stable=True).indices[..., :k]
    mask = torch.zeros_like(x_flat, dtype=torch.bool)
    mask.scatter_(-1, order, True)
    return mask


class _BatchTopKDense(torch.autograd.Function):
    """Dense [B, F] -> dense [B, F] batch-wide TopK through the batch select kernel: the k_total largest positive
    entries of the whole batch (ties -> lowest flattened index) keep their values and their gradient."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, k_total: int):
        x2 = (x if x.dtype in (torch.float32, torch.bfloat16) else x.float()).contiguous()
        code = ops.select_topk_batch(x2, None, None, min(int(k_total), x2.numel()))
        ctx.code, ctx.in_dtype = code, x.dtype
        return code.to_dense().to(x.dtype)

    @staticmethod
    def backward(ctx, g):
        mask = ctx.code.to_dense() > 0
        return (g * mask).to(ctx.in_dtype), None


def batch_topk_dense(x: torch.Tensor, k_total: int) -> torch.Tensor:
    """Keep the k_total largest positive entries of the whole [B, F] batch (ties -> lowest flattened index): the batch
    select kernel on GPU tensors it takes (F <= 2^30), a stable sort elsewhere."""
    if x.is_cuda and x.ndim == 2 and x.shape[1] <= 2 ** 30 and x.shape[0] <= 131072:
        return _BatchTopKDense.apply(x, k_total)
    r = x * x.gt(0).to(x.dtype)
    with torch.no_grad():
        mask = _topk_mask_lowest_index(r.reshape(1, -1), k_total).reshape(r.shape)
    return r * mask.to(r.dtype)
