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

import weakref
from typing import Optional

import torch
from torch.optim import Optimizer

from . import ops


class _null_ctx:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


def _flat_order(p: torch.Tensor):
    """Permutation of p's dims under which its memory is contiguous (None if there is none)."""
    if p.is_contiguous():
        return tuple(range(p.ndim))
    order = tuple(sorted(range(p.ndim), key=lambda i: -p.stride(i)))
    return order if p.permute(order).is_contiguous() else None


def _flat_view(p: torch.Tensor) -> torch.Tensor:
    """A contiguous view over p's memory (p itself, or the permutation that undoes a feature-major layout)."""
    order = _flat_order(p)
    if order is None:
        raise ValueError(f"parameter with strides {p.stride()} is not a permuted contiguous tensor")
    return p if order == tuple(range(p.ndim)) else p.permute(order)


def _grad_like(p: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """A [rows, d] gradient of p's contiguous storage, viewed with p's shape and strides."""
    order = _flat_order(p)
    g = rows.view([p.shape[i] for i in order])
    inv = [0] * len(order)
    for pos, dim in enumerate(order):
        inv[dim] = pos
    return g.permute(inv)


def _pieces(sg):
    """(first_row, SparseRowGrad) pairs of a factored gradient, single or in row blocks."""
    return sg.pieces if hasattr(sg, "pieces") else [(0, sg)]


def _contiguous_moments(sd: dict) -> dict:
    """A state dict whose moments are contiguous in the parameter's logical shape.  The per-parameter dicts that
    Optimizer.state_dict() returns are the optimiser's live ones, so they are copied, not edited."""
    sd["state"] = {i: {k: (v.contiguous() if k in ("exp_avg", "exp_avg_sq") and torch.is_tensor(v)
                           else (v.clone() if torch.is_tensor(v) else v))
                       for k, v in st.items()} for i, st in sd["state"].items()}
    return sd


def _relayout_loaded_state(opt: Optimizer, step_on_device: bool) -> None:
    """After Optimizer.load_state_dict: give `exp_avg` / `exp_avg_sq` the strides, dtype and device of their
    parameter (a checkpoint holds them contiguous in the logical shape; a feature-major W_E is not), and put the
    step counter where the optimiser keeps it (a host scalar for HipAdam, a device float[1] for HipSparseAdam)."""
    for group in opt.param_groups:
        for prm in group["params"]:
            st = opt.state.get(prm)
            if not st:
                continue
            for k in ("exp_avg", "exp_avg_sq"):
                t = st[k]
                if tuple(t.shape) != tuple(prm.shape):
                    raise ValueError(f"optimizer state {k} has shape {tuple(t.shape)}, parameter {tuple(prm.shape)}")
                if t.stride() != prm.stride() or t.dtype != prm.dtype or t.device != prm.device:
                    laid = torch.empty_like(prm, memory_format=torch.preserve_format)
                    laid.copy_(t)
                    st[k] = laid
            step = st.get("step", 0)
            # a copy of its own: Optimizer.load_state_dict passes a `step` tensor through as it is, so two optimisers
            # loaded from one in-memory state dict would otherwise count on the same tensor
            step = step.detach().float().clone() if torch.is_tensor(step) else torch.tensor(float(step), dtype=torch.float32)
            st["step"] = step.reshape(1).to(prm.device) if step_on_device else step.reshape(()).cpu()


class HipAdam(Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8, model=None,
                 defer_weight_grads: bool = True, overlap_decoder_update: bool = False):
        if lr < 0.0 or eps < 0.0 or not (0.0 <= betas[0] < 1.0) or not (0.0 <= betas[1] < 1.0):
            raise ValueError("invalid Adam hyper-parameters")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps))
        self._model = model
        self._roles: dict[int, str] = {}
        if model is not None:
            for name in ("W_E", "W_D"):
                p = getattr(model, name, None)
                if isinstance(p, torch.nn.ParameterList):
                    for j, q in enumerate(p):
                        self._roles[id(q)] = f"{name}.{j}"
                elif p is not None:
                    self._roles[id(p)] = name
            if defer_weight_grads and hasattr(model, "defer_weight_grads"):
                model.defer_weight_grads = True
        # Optional pipelining: the decoder's update (HBM-bound) runs on a second stream and overlaps the
        # next step's encoder GEMM (matrix-core / L2-bound), which reads only W_E.  The model waits for it
        # before anything of its own reads W_D, its bf16 copy or its row norms; code that touches W_D
        # outside the model must call `join()` first.
        self._overlap = bool(overlap_decoder_update) and model is not None and hasattr(model, "set_pending_update")
        self._side_stream = None
        self._norm_request = None   # (params, out): a gradient norm to be produced as a by-product of the next step()

    def deferred_grad_norm(self, params) -> torch.Tensor:
        """`compute_grad_norm(params)` as a device scalar that the next `step()` fills in: the sums of a factored
        weight gradient then come out of the Adam kernel that consumes it, at no extra pass.  For callers that do
        not need the value before the step (a logged diagnostic; clipping does).  Reading the tensor before
        `step()` has run gives garbage."""
        params = list(params)
        dev = next((p.device for p in params), torch.device("cuda"))
        if self._overlap or self._norm_request is not None:
            return compute_grad_norm(params)     # a second stream would race on the sums: take the direct route
        out = torch.empty((), dtype=torch.float32, device=dev)
        self._norm_request = (params, out)
        return out

    def join(self) -> None:
        """Make the current stream wait for an overlapped decoder update still in flight."""
        if self._model is not None and hasattr(self._model, "wait_pending_update"):
            self._model.wait_pending_update()

    def zero_grad(self, set_to_none: bool = True):
        super().zero_grad(set_to_none=set_to_none)
        for group in self.param_groups:
            for p in group["params"]:
                if getattr(p, "_sparse_grad", None) is not None:
                    p._sparse_grad = None
                if getattr(p, "_row_grad_coef", None) is not None:
                    p._row_grad_coef = None
                if getattr(p, "_lowp_grad", None) is not None:
                    p._lowp_grad = None

    @torch.no_grad()
    def materialize_grads(self) -> None:
        """Turn factored weight gradients into ordinary dense `.grad` tensors (for gradient clipping,
        the grad-norm diagnostic, or a different optimiser)."""
        for group in self.param_groups:
            fold_row_grad_coef(group["params"])
            for p in group["params"]:
                sg = getattr(p, "_sparse_grad", None)
                if sg is None:
                    continue
                rows, bias = sg.dense()
                p.grad = _grad_like(p, rows.to(p.dtype))
                if bias is not None:
                    sg.bias_param.grad = bias.view(sg.bias_param.shape).to(sg.bias_param.dtype)
                p._sparse_grad = None

    def _state(self, p):
        st = self.state[p]
        if len(st) == 0:
            st["step"] = torch.zeros((), dtype=torch.float32)
            st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
        return st

    # ---- checkpoint interchange with torch.optim.Adam (trainer.py:198-209, 272-278) ----
    def state_dict(self):
        """torch.optim.Adam's layout: `step`, `exp_avg`, `exp_avg_sq` per parameter index, the two moments as
        contiguous tensors of the parameter's logical shape (a feature-major W_E's moments leave as [d, F])."""
        return _contiguous_moments(super().state_dict())

    def load_state_dict(self, state_dict):
        """Accepts a torch.optim.Adam state dict (or this class's own): the moments are brought to each parameter's
        memory layout, which the update kernels address as one flat array together with the parameter."""
        super().load_state_dict(state_dict)
        _relayout_loaded_state(self, step_on_device=False)

    def _by_products(self, p, pv):
        """(role, bf16 shadow buffer or None, row-norm buffer or None) for the two weight matrices."""
        role = self._roles.get(id(p))
        shadow = norm_out = None
        if role is not None and pv.ndim == 2:
            shadow = self._model.get_derived_buffer(f"{role}.bf16")
            if role == "W_D" and pv.shape[1] % 4 == 0:
                norm_out = self._model.get_derived_buffer("W_D.norm")
                if norm_out is None:
                    norm_out = torch.empty(pv.shape[0], dtype=torch.float32, device=p.device)
        return role, shadow, norm_out

    def _publish(self, p, role, shadow, norm_out):
        # the kernel wrote through raw pointers: move the version counter like an in-place op would
        torch.autograd.graph.increment_version(p)
        if role is not None:
            if shadow is not None:
                self._model.set_derived(f"{role}.bf16", p, shadow)
            if norm_out is not None:
                self._model.set_derived("W_D.norm", p, norm_out)

    def _step_row_blocks(self, group, p, sg, st, pv, mv, vv, acc) -> None:
        """A weight whose [rows, d] view is updated block by block (a cross-layer transcoder's stacked layers):
        one kernel per block with a factored gradient, a plain zero-gradient Adam pass over rows no block covers."""
        b1, b2 = group["betas"]
        # a row is as long as the dense operand's rows: the last axis of the storage (a cross-layer transcoder's layers),
        # or several trailing axes taken together (a crosscoder's encoder, stored [F, H, d] with rows of H d)
        d = int(_pieces(sg)[0][1].dense_operand.shape[1])
        if pv.numel() % d != 0 or not pv.is_contiguous():
            raise NotImplementedError("the factored gradient's rows do not tile the parameter's storage")
        p2, m2, v2 = pv.reshape(-1, d), mv.reshape(-1, d), vv.reshape(-1, d)
        role = self._roles.get(id(p))
        shadow = self._model.get_derived_buffer(f"{role}.bf16") if role is not None else None
        if shadow is not None and (shadow.numel() != p2.numel() or shadow.dtype != torch.bfloat16):
            shadow = None
        sh2 = shadow.view(-1, d) if shadow is not None else None
        bias_param = getattr(sg, "bias_param", None)
        bias_buf = torch.zeros(p2.shape[0], dtype=torch.float32, device=p.device) if bias_param is not None else None
        # a decoder group held as one block (a cross-layer transcoder's W_D[j]) also yields its row norms
        want_norm = (role is not None and (role == "W_D" or role.startswith("W_D.")) and not hasattr(sg, "pieces") and d % 4 == 0
                     and hasattr(self._model, "set_derived"))
        norm_buf = None
        if want_norm:
            norm_buf = self._model.get_derived_buffer(f"{role}.norm")
            if norm_buf is None or norm_buf.numel() != p2.shape[0]:
                norm_buf = torch.empty(p2.shape[0], dtype=torch.float32, device=p.device)
        step = int(st["step"].item())
        covered = 0
        for r0, piece in sorted(_pieces(sg), key=lambda rp: rp[0]):
            n = piece.n_features
            if r0 != covered:
                raise NotImplementedError("row blocks of a factored gradient must tile the parameter")
            sums_out = None
            if acc is not None:
                if piece.sq_nnz is not None:
                    acc += piece.sq_nnz if piece.scale is None else torch.stack(
                        [piece.sq_nnz[0] * piece.scale.double().square().reshape(()), piece.sq_nnz[1]])
                else:
                    sums_out = acc
            ops.adam_step_sparse_rows(piece.fi, piece.coef, piece.dense_operand, p2[r0:r0 + n], m2[r0:r0 + n], v2[r0:r0 + n],
                                      lr=group["lr"], beta1=b1, beta2=b2, eps=group["eps"], step=step,
                                      shadow_bf16=None if sh2 is None else sh2[r0:r0 + n],
                                      row_norm_out=None if norm_buf is None else norm_buf[r0:r0 + n],
                                      bias_grad_out=None if bias_buf is None else bias_buf[r0:r0 + n],
                                      grad_scale=piece.scale, grad_sq_nnz_acc=sums_out, extra=piece.extra)
            covered = r0 + n
        if covered != p2.shape[0]:
            raise NotImplementedError("row blocks of a factored gradient must tile the parameter")
        if bias_buf is not None:
            g = bias_buf.view(bias_param.shape).to(bias_param.dtype)
            bias_param.grad = g if bias_param.grad is None else bias_param.grad + g
        p._sparse_grad = None
        torch.autograd.graph.increment_version(p)
        if shadow is not None:
            self._model.set_derived(f"{role}.bf16", p, shadow)
        if norm_buf is not None:
            self._model.set_derived(f"{role}.norm", p, norm_buf)

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        req, acc, wanted = self._norm_request, None, ()
        self._norm_request = None
        if req is not None:
            fold_row_grad_coef(req[0], keep_factored=True)   # the norm is over the element-wise gradient
            wanted = {id(p) for p in req[0]}
            acc = torch.zeros(2, dtype=torch.float64, device=req[1].device)
        # pass 1: weights whose gradient arrives in factored form (also yields the encoder-bias gradient)
        deferred = []
        for group in self.param_groups:
            for p in group["params"]:
                if getattr(p, "_sparse_grad", None) is not None:
                    deferred.append((group, p))
        # the decoder goes last so that, when overlapped, it has the stream's tail to itself
        deferred.sort(key=lambda gp: self._roles.get(id(gp[1])) == "W_D")
        for group, p in deferred:
            b1, b2 = group["betas"]
            sg = p._sparse_grad
            if p.grad is not None:
                raise RuntimeError("parameter has both a dense and a factored gradient")
            st = self._state(p)
            st["step"] += 1
            pv = _flat_view(p)
            mv, vv = _flat_view(st["exp_avg"]), _flat_view(st["exp_avg_sq"])
            if hasattr(sg, "pieces") or pv.ndim != 2:
                self._step_row_blocks(group, p, sg, st, pv, mv, vv, acc if id(p) in wanted else None)
                continue
            role, shadow, norm_out = self._by_products(p, pv)
            row_coef = getattr(p, "_row_grad_coef", None)     # the gradient through the row norm, added where rows are rebuilt
            if row_coef is not None and (p.dtype != torch.float32 or sg.sq_nnz is not None):
                raise RuntimeError("a row-norm gradient term cannot join this factored gradient")
            p._row_grad_coef = None
            bias_out = None
            if sg.bias_param is not None:
                bias_out = torch.empty(pv.shape[0], dtype=torch.float32, device=p.device)
            sums_out = None
            if id(p) in wanted:
                if sg.sq_nnz is not None:     # already reduced by a direct norm call: reuse
                    acc += sg.sq_nnz if sg.scale is None else torch.stack(
                        [sg.sq_nnz[0] * sg.scale.double().square().reshape(()), sg.sq_nnz[1]])
                else:
                    sums_out = acc
            side = None
            if self._overlap and role == "W_D" and bias_out is None:
                if self._side_stream is None:
                    self._side_stream = torch.cuda.Stream(device=p.device)
                side = self._side_stream
                side.wait_stream(torch.cuda.current_stream(p.device))
                extra_t = () if sg.extra is None else (sg.extra.row_map, sg.extra.rows, sg.extra.bias)
                for t in (sg.fi.feat_ptr, sg.fi.feat_slot, sg.fi.slot_tok, sg.coef, sg.dense_operand, sg.scale, *extra_t):
                    if t is not None:
                        t.record_stream(side)  # step-local tensors: keep their memory until the side stream is done
            with torch.cuda.stream(side) if side is not None else _null_ctx():
                ops.adam_step_sparse_rows(sg.fi, sg.coef, sg.dense_operand, pv, mv, vv, lr=group["lr"], beta1=b1, beta2=b2,
                                          eps=group["eps"], step=int(st["step"].item()), shadow_bf16=shadow,
                                          row_norm_out=norm_out, bias_grad_out=bias_out, grad_scale=sg.scale,
                                          grad_sq_nnz_acc=sums_out, extra=sg.extra, row_grad_coef=row_coef)
                if side is not None:
                    ev = torch.cuda.Event()
                    ev.record(side)
            if bias_out is not None:
                bias_out = bias_out.to(sg.bias_param.dtype)
                sg.bias_param.grad = bias_out if sg.bias_param.grad is None else sg.bias_param.grad + bias_out
            p._sparse_grad = None
            self._publish(p, role, shadow, norm_out)
            if side is not None:
                self._model.set_pending_update(ev)
        if req is not None:
            dense = [p.grad for p in req[0] if p.grad is not None]
            if dense:
                acc = acc + _dense_sq_nnz(dense)
            req[1].copy_(acc[0].sqrt() / acc[1].sqrt())
        # pass 2: everything with a dense gradient
        for group in self.param_groups:
            b1, b2 = group["betas"]
            for p in group["params"]:
                row_coef, lowp = getattr(p, "_row_grad_coef", None), getattr(p, "_lowp_grad", None)
                if lowp is not None and (p.grad is not None or tuple(lowp.shape) != tuple(_flat_view(p).shape)
                                         or not lowp.is_contiguous()):
                    fold_row_grad_coef([p])     # a second, fp32 gradient as well (or an unexpected layout): one dense sum
                    row_coef = lowp = None
                if row_coef is not None and ((p.grad is None and lowp is None) or p.ndim != 2 or p.shape[1] % 4 != 0
                                             or not p.is_contiguous() or (p.grad is not None and not p.grad.is_contiguous())):
                    fold_row_grad_coef([p])     # no row-wise kernel for this layout: add the term to the gradient
                    row_coef = lowp = None
                if p.grad is None and lowp is None:
                    continue
                if p.dtype not in (torch.float32, torch.bfloat16):
                    raise TypeError("HipAdam updates fp32 or bf16 parameters")
                st = self._state(p)
                st["step"] += 1
                pv = _flat_view(p)
                same_layout = lambda t: _flat_view(t) if t.stride() == p.stride() else None  # noqa: E731
                mv, vv = same_layout(st["exp_avg"]), same_layout(st["exp_avg_sq"])
                gv = lowp if lowp is not None else same_layout(p.grad)
                if gv is None:
                    gv = p.grad.permute(_flat_order(p)).contiguous()
                assert mv is not None and vv is not None, "optimizer state must share the parameter's layout"
                role, shadow, norm_out = self._by_products(p, pv)
                ops.adam_step(pv, gv, mv, vv, lr=group["lr"], beta1=b1, beta2=b2, eps=group["eps"],
                              step=int(st["step"].item()), shadow_bf16=shadow, row_norm_out=norm_out,
                              row_len=pv.shape[1] if (norm_out is not None or row_coef is not None) else 0,
                              row_grad_coef=row_coef)
                p._row_grad_coef = p._lowp_grad = None
                self._publish(p, role, shadow, norm_out)
        return loss


class HipSparseAdam(Optimizer):
    """SparseAdam of the reference (src/llamascopium/optim.py:142-254) with the per-parameter update in
    one kernel: moments decay everywhere, gradient contributions and the parameter move only where
    the gradient is non-zero, a parameter whose gradient is entirely zero is skipped (its step counter
    too).  That test runs on the device, so `step()` never synchronises.  Factored weight gradients
    are materialised first (the masked update needs the element-wise gradient)."""

    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8, weight_decay: float = 0, model=None):
        if lr < 0.0 or eps < 0.0 or not (0.0 <= betas[0] < 1.0) or not (0.0 <= betas[1] < 1.0) or weight_decay < 0.0:
            raise ValueError("invalid SparseAdam hyper-parameters")
        if weight_decay != 0:
            raise NotImplementedError("weight decay is not part of the kernel (the reference's trainer never sets it)")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self._model = model

    def state_dict(self):
        return _contiguous_moments(super().state_dict())

    def load_state_dict(self, state_dict):
        super().load_state_dict(state_dict)
        _relayout_loaded_state(self, step_on_device=True)

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            b1, b2 = group["betas"]
            for p in group["params"]:
                sg = getattr(p, "_sparse_grad", None)
                if sg is not None:
                    rows, bias = sg.dense()
                    p.grad = _grad_like(p, rows)
                    if bias is not None:
                        sg.bias_param.grad = bias.view(sg.bias_param.shape)
                    p._sparse_grad = None
        for group in self.param_groups:
            b1, b2 = group["betas"]
            for p in group["params"]:
                if p.grad is None:
                    continue
                st = self.state[p]
                if len(st) == 0:
                    st["step"] = torch.zeros(1, dtype=torch.float32, device=p.device)
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                pv = _flat_view(p)
                gv = _flat_view(p.grad) if p.grad.stride() == p.stride() else p.grad.permute(_flat_order(p)).contiguous()
                ops.sparse_adam_step(pv, gv, _flat_view(st["exp_avg"]), _flat_view(st["exp_avg_sq"]), st["step"],
                                     lr=group["lr"], beta1=b1, beta2=b2, eps=group["eps"])
                torch.autograd.graph.increment_version(p)
        return loss


def fold_row_grad_coef(params, keep_factored: bool = False) -> None:
    """Bring what the backward left on a weight for HipAdam into its dense fp32 `.grad`, for consumers of the
    element-wise gradient (norm, clipping, SparseAdam): a bf16 gradient over the parameter's storage
    (`_lowp_grad`, widened), and the row-norm gradient (`_row_grad_coef`: d n / n per row, added as
    coef[:, None] * W).  HipAdam.step otherwise takes both inside its update kernel."""
    for p in params:
        lowp = getattr(p, "_lowp_grad", None)
        if lowp is not None:
            term = _grad_like(p, lowp.to(p.dtype))
            p.grad = term if p.grad is None else p.grad + term
            p._lowp_grad = None
        coef = getattr(p, "_row_grad_coef", None)
        if coef is None:
            continue
        sg = getattr(p, "_sparse_grad", None)
        if sg is not None:
            if keep_factored and not hasattr(sg, "pieces"):
                continue        # HipAdam's factored pass adds the term to the rows it rebuilds
            # an element-wise consumer of a gradient that is factored AND has a row-norm term: both become dense
            rows, bias = sg.dense()
            p.grad = _grad_like(p, rows.to(p.dtype))
            if bias is not None:
                g = bias.view(sg.bias_param.shape).to(sg.bias_param.dtype)
                sg.bias_param.grad = g if sg.bias_param.grad is None else sg.bias_param.grad + g
            p._sparse_grad = None
        term = (coef.view(-1, *([1] * (p.ndim - 1))) * p.detach()).to(p.dtype)
        p.grad = term if p.grad is None else p.grad + term
        p._row_grad_coef = None


def _grad_sq_nnz(params) -> torch.Tensor:
    """device double[2] = (sum g^2, #non-zero g) over dense `.grad`s and factored weight gradients alike.
    A factored gradient is reduced by a kernel that rebuilds its rows in registers; the bias gradient it
    carries is produced on the way and becomes an ordinary `.grad` (so it is counted, clipped and stepped
    like any other).  The sums are cached (on the factored gradient; on a dense gradient tensor together with
    its version counter): the second norm of a step, the after-clipping diagnostic, launches almost nothing."""
    params = list(params)
    fold_row_grad_coef(params)
    parts = []
    for p in params:
        whole = getattr(p, "_sparse_grad", None)
        if whole is None:
            continue
        bias_param = getattr(whole, "bias_param", None)
        bias_buf = None
        for r0, sg in _pieces(whole):
            if sg.sq_nnz is None:
                own = torch.zeros(2, dtype=torch.float64, device=p.device)
                bias_out = None
                if bias_param is not None:
                    if bias_buf is None:
                        bias_buf = torch.zeros(bias_param.numel(), dtype=torch.float32, device=p.device)
                    bias_out = bias_buf[r0:r0 + sg.n_features]
                ops.sparse_rows_grad_sq_nnz(sg.fi, sg.coef, sg.dense_operand, own, bias_grad_out=bias_out, extra=sg.extra)
                sg.sq_nnz = own
            own = sg.sq_nnz
            if sg.scale is not None:
                own = torch.stack([own[0] * sg.scale.double().square().reshape(()), own[1]])
            parts.append(own)
        if bias_buf is not None:
            g = bias_buf.view(bias_param.shape).to(bias_param.dtype)
            bias_param.grad = g if bias_param.grad is None else bias_param.grad + g
            whole.bias_param = None
            for _, sg in _pieces(whole):
                sg.bias_param = None
    dense = [p.grad for p in params if p.grad is not None]
    if dense:
        parts.append(_dense_sq_nnz(dense))
    assert parts, "No gradients found"
    return parts[0] if len(parts) == 1 else torch.stack(parts).sum(0)


_dense_cache: dict = {"refs": (), "versions": (), "sums": None}


def _dense_sq_nnz(grads) -> torch.Tensor:
    """Joint (sum g^2, #non-zero) of a list of dense gradients, remembered while the same tensor objects
    stay unmodified (weak references and version counters decide)."""
    refs, versions = _dense_cache["refs"], _dense_cache["versions"]
    if len(refs) == len(grads) and all(r() is g and v == g._version for r, v, g in zip(refs, versions, grads)):
        return _dense_cache["sums"]
    sums = ops.grad_sq_nnz(grads)
    _dense_cache.update(refs=tuple(weakref.ref(g) for g in grads), versions=tuple(g._version for g in grads), sums=sums)
    return sums


def compute_grad_norm(params) -> torch.Tensor:
    """||g||_2 over all gradients divided by sqrt(number of non-zero gradient entries)
    (src/llamascopium/optim.py:257-277), as a device scalar.  Dense and factored gradients both count."""
    acc = _grad_sq_nnz(params)
    return (acc[0].sqrt() / acc[1].sqrt()).to(torch.float32)


def clip_grad_norm(params, max_norm: float) -> torch.Tensor:
    """src/llamascopium/optim.py:280-292 without the host round trip: gradients are scaled by
    max_norm / (norm + 1e-6) when the norm exceeds max_norm, decided on the device.  A factored weight
    gradient is not rewritten: the factor is attached to it and applied where its rows are formed."""
    params = list(params)   # not filtered yet: a bias gradient carried by a factored weight gradient appears below
    norm = compute_grad_norm(params)
    if max_norm != float("inf"):
        factor = torch.where(norm > max_norm, max_norm / (norm + 1e-6), torch.ones_like(norm))
        for p in params:
            if p.grad is not None:
                p.grad.mul_(factor)
            whole = getattr(p, "_sparse_grad", None)
            if whole is not None:
                for _, sg in _pieces(whole):
                    sg.scale = factor.reshape(1) if sg.scale is None else sg.scale * factor
    return norm
