"""Base class of the sparse-dictionary models on the HIP path.

Mirrors the public surface of the reference's `SparseDictionary`
(src/llamascopium/models/sparse_dictionary.py:217-1127) for the parts that sit on the train
step: `encode` / `decode` / `forward` / `compute_loss`, activation normalisation, the activation
callable stored at `self.activation_function`, `set_current_k`, `get_parameters`, and the
state-dict key names.  Checkpoint I/O to hubs, DTensor sharding and database hooks are not part
of this path.
"""

from __future__ import annotations

import math
from typing import Any, Callable, Optional

import torch
from torch import nn

from .activation_functions import JumpReLU, batch_topk_dense, topk_dense
from .config import SAE_TYPE_TO_MODEL_CLASS, SparseDictionaryConfig


CHECKPOINT_VERSION = "lm-saes-amd-1"


def apply_token_mask(t: torch.Tensor, n_token_dims: int, mask: Optional[torch.Tensor], reduction: str = "sum"):
    """Reduce the leading token dims (batch[, context]) of `t`, optionally weighted by a 0/1 mask.
    Same results as utils/tensor_specs.py:64-84."""
    dims = tuple(range(n_token_dims))
    if mask is None:
        if not dims:
            return t
        return t.sum(dim=dims) if reduction == "sum" else t.mean(dim=dims)
    assert tuple(mask.shape) == tuple(t.shape[:n_token_dims]), (
        f"Mask has shape {tuple(mask.shape)}, but input tensor has token part of shape {tuple(t.shape[:n_token_dims])}"
    )
    m = mask.to(t).reshape(*mask.shape, *([1] * (t.ndim - n_token_dims)))
    out = (t * m).sum(dim=dims)
    return out / mask.sum() if reduction == "mean" else out


class LazyDict(dict):
    """dict whose listed entries are computed on first access (dense [B, F] views of the sparse
    code are only materialised for callers that actually read them)."""

    _PENDING = object()

    def __init__(self, eager: dict, lazy: dict[str, Callable[[], Any]]):
        super().__init__(eager)
        self._lazy = dict(lazy)
        for k in lazy:
            dict.__setitem__(self, k, LazyDict._PENDING)

    def _resolve(self, k):
        v = dict.__getitem__(self, k)
        if v is LazyDict._PENDING:
            v = self._lazy.pop(k)()
            dict.__setitem__(self, k, v)
        return v

    def __getitem__(self, k):
        return self._resolve(k)

    def get(self, k, default=None):
        return self._resolve(k) if k in self else default

    def items(self):
        return [(k, self._resolve(k)) for k in self.keys()]

    def values(self):
        return [self._resolve(k) for k in self.keys()]


class SparseDictionary(nn.Module):
    def __init__(self, cfg: SparseDictionaryConfig, device_mesh=None):
        super().__init__()
        if device_mesh is not None:
            raise NotImplementedError("single-GPU build: device meshes are not supported")
        self.cfg = cfg
        self.current_k = cfg.top_k
        self.dataset_average_activation_norm: dict[str, float] | None = None
        self.device_mesh = None
        self.activation_function = self.activation_function_factory(None)
        # derived operands (bf16 shadows, row norms) keyed by name -> (param version, tensor)
        self._derived: dict[str, tuple[int, torch.Tensor]] = {}

    # ---- derived operands, refreshed when the parameter's version counter moves ----
    def _derive(self, name: str, param: torch.Tensor, make) -> torch.Tensor:
        ver = param._version
        hit = self._derived.get(name)
        if hit is not None and hit[0] == ver and hit[1].device == param.device:
            return hit[1]
        with torch.no_grad():
            t = make(hit[1] if hit is not None and hit[1].device == param.device else None)
        self._derived[name] = (ver, t)
        return t

    def set_derived(self, name: str, param: torch.Tensor, tensor: torch.Tensor) -> None:
        """Called by the fused optimiser after it wrote a fresh shadow / norm itself."""
        self._derived[name] = (param._version, tensor)

    def get_derived_buffer(self, name: str) -> Optional[torch.Tensor]:
        hit = self._derived.get(name)
        return None if hit is None else hit[1]

    # ---- small state setters (sparse_dictionary.py:248-260) ----
    @torch.no_grad()
    def set_dataset_average_activation_norm(self, dataset_average_activation_norm: dict[str, float]):
        self.dataset_average_activation_norm = dataset_average_activation_norm

    @torch.no_grad()
    def set_current_k(self, current_k: int):
        self.current_k = current_k

    # ---- activation factory (sparse_dictionary.py:713-796) ----
    def activation_function_factory(self, device_mesh=None):
        act = self.cfg.act_fn.lower()
        assert act in ["relu", "topk", "jumprelu", "batchtopk"], f"Not implemented activation function {self.cfg.act_fn}"
        if act == "relu":
            return lambda x: x * x.gt(0).to(x.dtype)
        if act == "jumprelu":
            return JumpReLU(self.cfg.jumprelu_threshold_window, shape=(self.cfg.d_sae,), device=self.cfg.device,
                            dtype=self.cfg.dtype)
        if act == "topk":
            def topk_activation(x: torch.Tensor):
                if x.is_cuda:
                    return topk_dense(x, self.current_k)
                raise RuntimeError("the TopK activation runs on the GPU only (no CPU fallback in this build)")
            return topk_activation

        def batch_topk(x: torch.Tensor):
            shape = None
            if x.ndim == 3:
                shape = (x.size(0), x.size(1))
                x = x.flatten(end_dim=1)
            out = batch_topk_dense(x, self.current_k * x.size(0))
            return out.unflatten(0, shape) if shape is not None else out
        return batch_topk

    @torch.no_grad()
    def init_parameters(self, **kwargs):
        if self.cfg.act_fn.lower() == "jumprelu":
            self.activation_function.log_jumprelu_threshold.data.fill_(kwargs["init_log_jumprelu_threshold_value"])

    # ---- activation normalisation (sparse_dictionary.py:427-499) ----
    def compute_norm_factor(self, x: torch.Tensor, hook_point: str) -> torch.Tensor:
        mode = self.cfg.norm_activation
        assert mode in ["token-wise", "batch-wise", "dataset-wise", "inference"], f"Not implemented norm_activation {mode}"
        if mode == "token-wise":
            return math.sqrt(self.cfg.d_model) / torch.norm(x, 2, dim=-1, keepdim=True)
        if mode == "batch-wise":
            return math.sqrt(self.cfg.d_model) / torch.norm(x, 2, dim=-1, keepdim=True).mean(dim=-2, keepdim=True)
        if mode == "dataset-wise":
            assert self.dataset_average_activation_norm is not None, (
                "dataset_average_activation_norm must be provided from Initializer"
            )
            return self._scalar(math.sqrt(self.cfg.d_model) / self.dataset_average_activation_norm[hook_point], x)
        return self._scalar(1.0, x)

    def _scalar(self, value: float, like: torch.Tensor) -> torch.Tensor:
        """0-dim tensor of `value` on like's device in like's dtype, built once (a host-to-device copy per call otherwise)."""
        cache = self.__dict__.setdefault("_scalar_cache", {})
        key = (value, like.device, like.dtype)
        t = cache.get(key)
        if t is None:
            if len(cache) > 64:
                cache.clear()
            t = cache[key] = torch.tensor(value, device=like.device, dtype=like.dtype)
        return t

    def normalize_activations(self, batch: dict[str, torch.Tensor], *, return_scale_factor: bool = False):
        hooks = self.cfg.associated_hook_points
        if self.cfg.norm_activation == "inference" and not return_scale_factor:
            return dict(batch)    # every factor is the constant 1: no pass over the activations
        scale = {k: self.compute_norm_factor(v, hook_point=k) for k, v in batch.items() if k in hooks}
        out = {k: (v * scale[k] if k in scale else v) for k, v in batch.items()}
        return (out, scale) if return_scale_factor else out

    def denormalize_activations(self, batch, scale_factors):
        return {k: v / scale_factors[k] for k, v in batch.items()}

    # ---- optimiser groups (sparse_dictionary.py:501-510) ----
    def log_statistics(self) -> dict[str, Any]:
        """models/sparse_dictionary.py:698-711: weight-norm means, the current k, the mean JumpReLU threshold."""
        out: dict[str, Any] = {}
        if hasattr(self, "encoder_norm") and hasattr(self, "decoder_norm"):
            with torch.no_grad():
                out["metrics/encoder_norm"] = self.encoder_norm().mean().item()
                out["metrics/decoder_norm"] = self.decoder_norm().mean().item()
                if self.cfg.use_decoder_bias and hasattr(self, "decoder_bias_norm"):
                    out["metrics/decoder_bias_norm"] = self.decoder_bias_norm().mean().item()
        if "topk" in self.cfg.act_fn:
            out["sparsity/k"] = self.current_k
        if isinstance(self.activation_function, JumpReLU):
            out["metrics/mean_jumprelu_threshold"] = self.activation_function.log_jumprelu_threshold.detach().exp().mean().item()
        return out

    def compute_training_metrics(self, **kwargs) -> dict[str, float]:
        """Model-specific training metrics (models/sparse_dictionary.py:1029-1039); none for the base class."""
        return {}

    def get_parameters(self) -> list[dict[str, Any]]:
        jr = list(self.activation_function.parameters()) if isinstance(self.activation_function, JumpReLU) else []
        others = [p for p in self.parameters() if not any(p is q for q in jr)]
        return [{"params": others, "name": "others"}, {"params": jr, "name": "jumprelu"}]

    # ---- state dict with the reference's extra scalars (sparse_dictionary.py:262-278, 512-523) ----
    @torch.no_grad()
    def full_state_dict(self) -> dict[str, torch.Tensor]:
        sd = {k: v.contiguous() for k, v in self.state_dict().items()}
        for hp in self.cfg.associated_hook_points:
            if self.dataset_average_activation_norm is not None:
                sd[f"dataset_average_activation_norm.{hp}"] = torch.tensor(
                    self.dataset_average_activation_norm[hp], device=self.cfg.device, dtype=self.cfg.dtype)
            else:
                sd[f"dataset_average_activation_norm.{hp}"] = torch.empty((), device=self.cfg.device, dtype=self.cfg.dtype)
        return sd

    def load_full_state_dict(self, state_dict: dict[str, torch.Tensor], strict: bool = True) -> None:
        norm_keys = [k for k in state_dict if k.startswith("dataset_average_activation_norm.")]
        if norm_keys:
            self.set_dataset_average_activation_norm({k.split(".", 1)[1]: state_dict[k].item() for k in norm_keys})
            state_dict = {k: v for k, v in state_dict.items() if k not in norm_keys}
        self.load_state_dict(state_dict, strict=strict)

    @classmethod
    def from_config(cls, cfg: SparseDictionaryConfig, device_mesh=None):
        if cls is SparseDictionary:
            cls = SAE_TYPE_TO_MODEL_CLASS[cfg.sae_type]
        if cfg.sae_pretrained_name_or_path is not None:
            return cls.from_pretrained(cfg.sae_pretrained_name_or_path, strict_loading=cfg.strict_loading,
                                       device=cfg.device, dtype=cfg.dtype)
        return cls(cfg, device_mesh)

    # ---- checkpoint files in the reference's format (sparse_dictionary.py:280-331, 558-665) ----
    @torch.no_grad()
    def save_checkpoint(self, ckpt_path) -> None:
        """`.safetensors`: the full state dict (reference key names and shapes, W_E as [d_model, d_sae]
        row-major, plus the `dataset_average_activation_norm.*` scalars) with a `version` metadata entry;
        `.pt`: `{"sae": state_dict, "version": ...}`."""
        import os

        sd = {k: v.detach().contiguous() for k, v in self.full_state_dict().items()}
        suffix = os.path.splitext(str(ckpt_path))[1]
        if suffix == ".safetensors":
            import safetensors.torch as safe

            safe.save_file({k: v.cpu() for k, v in sd.items()}, str(ckpt_path), {"version": CHECKPOINT_VERSION})
        elif suffix == ".pt":
            torch.save({"sae": sd, "version": CHECKPOINT_VERSION}, str(ckpt_path))
        else:
            raise ValueError(f"Invalid checkpoint path {ckpt_path}. Currently only supports .safetensors and .pt formats.")

    @torch.no_grad()
    def save_pretrained(self, save_path, fold_activation_scale: bool = False) -> None:
        import os

        os.makedirs(str(save_path), exist_ok=True)
        if fold_activation_scale:
            assert hasattr(self, "standardize_parameters_of_dataset_norm"), (
                f"{type(self).__name__} does not support dataset norm standardization")
            self.standardize_parameters_of_dataset_norm()
        self.save_checkpoint(os.path.join(str(save_path), "sae_weights.safetensors"))

    @classmethod
    def from_local(cls, path: str, device_mesh=None, strict_loading: bool = True, fold_activation_scale: bool = False,
                   **kwargs):
        """Load `<path>/config.json` and the first weights file found in the reference's priority order
        (sae_weights, checkpoints/pruned, checkpoints/final; safetensors before pt); `path` may also name
        a weights file directly.  The `.pt` form is read with `weights_only=True`."""
        import os

        path = str(path)
        cfg = SparseDictionaryConfig.from_pretrained(path, strict_loading=strict_loading, **kwargs)
        cfg.sae_pretrained_name_or_path = None
        model = cls.from_config(cfg, device_mesh=device_mesh)
        if path.endswith((".pt", ".safetensors")):
            ckpt_path = path
        else:
            for rel in ("sae_weights.safetensors", "sae_weights.pt", "checkpoints/pruned.safetensors", "checkpoints/pruned.pt",
                        "checkpoints/final.safetensors", "checkpoints/final.pt"):
                ckpt_path = os.path.join(path, rel)
                if os.path.exists(ckpt_path):
                    break
            else:
                raise FileNotFoundError(f"Pretrained model not found at {path}")
        if ckpt_path.endswith(".safetensors"):
            import safetensors.torch as safe

            state_dict = safe.load_file(ckpt_path, device=cfg.device)
        else:
            state_dict = torch.load(ckpt_path, map_location=cfg.device, weights_only=True)["sae"]
        model.load_full_state_dict(state_dict, strict=strict_loading)
        if fold_activation_scale:
            assert hasattr(model, "standardize_parameters_of_dataset_norm"), (
                f"{type(model).__name__} does not support dataset norm standardization")
            model.standardize_parameters_of_dataset_norm()
        return model

    @classmethod
    def from_pretrained(cls, pretrained_name_or_path: str, *, device_mesh=None, fold_activation_scale: bool = False,
                        strict_loading: bool = True, **kwargs):
        """Local directories and files only: hub repositories and SAELens names are outside this path."""
        import os

        if not os.path.exists(str(pretrained_name_or_path)):
            raise ValueError(f"{pretrained_name_or_path!r} is not a local path; hub downloads are not part of this library")
        return cls.from_local(str(pretrained_name_or_path), device_mesh=device_mesh, strict_loading=strict_loading,
                              fold_activation_scale=fold_activation_scale, **kwargs)

    def _sparse_decode_allowed(self, feature_acts: torch.Tensor) -> bool:
        """Whether `decode` may send dense activations through the sparse decoder kernels (models that set
        `sparse_api_decode`).  Their backward returns the activation gradient at the non-zero entries only, as the
        reference's sparse operator does (kernels/kernels.py:563): exact for TopK-family and ReLU activations, whose own
        backward passes nothing else on, but a JumpReLU's threshold gradient also reads entries just below the
        threshold, so a JumpReLU dictionary takes the route only where no gradient is asked of the activations."""
        if not (getattr(self, "sparse_api_decode", False) and feature_acts.is_cuda):
            return False
        needs_grad = torch.is_grad_enabled() and feature_acts.requires_grad
        return not (needs_grad and isinstance(self.activation_function, JumpReLU))

    # ---- to be provided by subclasses ----
    def encode(self, x, return_hidden_pre: bool = False, **kwargs):
        raise NotImplementedError

    def decode(self, feature_acts, **kwargs):
        raise NotImplementedError

    def prepare_input(self, batch, **kwargs):
        raise NotImplementedError

    def prepare_label(self, batch, **kwargs):
        raise NotImplementedError

    def forward(self, x, encoder_kwargs: dict = {}, decoder_kwargs: dict = {}):
        return self.decode(self.encode(x, **encoder_kwargs), **decoder_kwargs)

    # ---- generic loss: the reference's op sequence (sparse_dictionary.py:840-1007) over dense
    # tensors.  Subclasses route the configurations their fused kernels cover away from it. ----
    def compute_loss(
        self,
        batch: dict[str, torch.Tensor],
        label: Optional[torch.Tensor] = None,
        *,
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
        **kwargs,
    ):
        x, enc_kw, dec_kw = self.prepare_input(batch)
        label = self.prepare_label(batch, **kwargs)
        mask = batch.get("mask")
        feature_acts, hidden_pre = self.encode(x, return_hidden_pre=True, **enc_kw)
        reconstructed = self.decode(feature_acts, **dec_kw)
        ntd = label.ndim - 1

        l_rec = apply_token_mask((reconstructed - label).pow(2).sum(dim=-1), ntd, mask, "mean")
        loss_dict: dict[str, Optional[torch.Tensor]] = {"l_rec": l_rec}
        loss = l_rec

        if sparsity_loss_type is not None:
            n = self.decoder_norm()
            if sparsity_loss_type == "power":
                l_s = torch.norm(feature_acts * n, p=p, dim=-1)
            elif sparsity_loss_type == "tanh":
                l_s = torch.tanh(tanh_stretch_coefficient * feature_acts * n).sum(dim=-1)
            elif sparsity_loss_type == "tanh-quad":
                score = torch.tanh(tanh_stretch_coefficient * feature_acts * n)
                freq = score.mean(dim=tuple(range(score.ndim - 1)))
                l_s = (freq * (1 + freq / frequency_scale)).sum(dim=-1)
            else:
                raise ValueError(f"sparsity_loss_type f{sparsity_loss_type} not supported.")
            l_s = l1_coefficient * l_s
            loss_dict["l_s"] = l_s
            loss = loss + apply_token_mask(l_s, min(ntd, l_s.ndim), mask if l_s.ndim else None, "mean")
        else:
            loss_dict["l_s"] = None

        if lp_coefficient > 0.0 and isinstance(self.activation_function, JumpReLU):
            theta = self.activation_function.get_jumprelu_threshold()
            l_p = lp_coefficient * (torch.nn.functional.relu(theta - hidden_pre) * self.decoder_norm()).sum(dim=-1)
            l_p = apply_token_mask(l_p, ntd, mask, "mean")
            loss_dict["l_p"] = l_p
            loss = loss + l_p
        else:
            loss_dict["l_p"] = None

        if auxk_coefficient > 0.0:
            assert update_dead_statistics is not None, "update_dead_statistics must be set when auxk_coefficient > 0.0"
            specs = ("batch", "sae") if feature_acts.ndim == 2 else ("batch", "context", "sae")
            is_dead = update_dead_statistics(feature_acts, mask, specs)
            e = label - reconstructed
            current_k = self.current_k
            self.current_k = min(k_aux, int(is_dead.sum().item()))
            if self.current_k > 0:
                n = self.decoder_norm() if self.cfg.sparsity_include_decoder_norm else None
                dead_hidden_pre = hidden_pre * is_dead * n if n is not None else hidden_pre * is_dead
                dead_acts = self.activation_function(dead_hidden_pre)
                if n is not None:
                    dead_acts = dead_acts / n
                aux_rec = dead_acts @ self.W_D
                l_aux = apply_token_mask(auxk_coefficient * (e - aux_rec).pow(2).sum(dim=-1), ntd, mask, "mean")
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
            "loss": loss, **loss_dict, "label": label, "mask": mask,
            "n_tokens": batch["tokens"].numel() if mask is None else int(mask.sum().item()),
            "feature_acts": feature_acts, "reconstructed": reconstructed, "hidden_pre": hidden_pre,
            "l1_coefficient": l1_coefficient, "lp_coefficient": lp_coefficient, "auxk_coefficient": auxk_coefficient,
        }
