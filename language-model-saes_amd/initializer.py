"""Start-up initialisation of a sparse dictionary: uniform weights, encoder from the decoder transpose,
decoder bias from the mean label, and the coarse-then-fine grid search over decoder norms that picks the
norm with the lowest initial reconstruction error (src/llamascopium/initializer.py:30-293).

The grid search is 70 forward passes of `compute_loss` on one batch; on the GPU they run through the same
fused kernels as training (encoder GEMM, select, sparse decode + MSE), without gradients.  Initialisers that
copy weights from a host language model (Lorsa from attention heads, transcoders from an MLP, active-subspace
SVD) are not part of this path.
"""

from __future__ import annotations

import warnings
from typing import Iterable, List, Literal, Optional

import torch
from pydantic import BaseModel

from .config import SparseDictionaryConfig
from .sparse_dictionary import SparseDictionary


class InitializerConfig(BaseModel):
    bias_init_method: Literal["all_zero", "geometric_median"] = "all_zero"
    decoder_uniform_bound: float = 1.0
    encoder_uniform_bound: float = 1.0
    init_encoder_with_decoder_transpose: bool = True
    init_encoder_with_decoder_transpose_factor: float = 1.0
    init_log_jumprelu_threshold_value: Optional[float] = None
    grid_search_init_norm: bool = False
    init_encoder_bias_with_mean_hidden_pre: bool = False
    init_search: Optional[bool] = None   # accepted and ignored, as the reference's own tests still pass it


def calculate_activation_norm(activation_stream: Iterable[dict], hook_points: list[str], batch_num: int = 8) -> dict[str, float]:
    """Mean L2 norm of the activation vectors of each hook point over the first `batch_num` batches
    (utils/misc.py:122-159)."""
    assert len(hook_points) > 0, "No hook points provided"
    norms: dict[str, list[torch.Tensor]] = {}
    it = iter(activation_stream)
    while batch_num > 0:
        try:
            batch = next(it)
        except StopIteration:
            warnings.warn(f"Activation stream ended prematurely. {batch_num} batches not processed.")
            break
        for key in hook_points:
            norms.setdefault(key, []).append(batch[key].norm(p=2, dim=-1).reshape(-1))
        batch_num -= 1
    return {k: torch.cat(v).mean().item() for k, v in norms.items()}


class Initializer:
    def __init__(self, cfg: InitializerConfig):
        self.cfg = cfg
        self.best_norm: Optional[float] = None   # what the last grid search settled on

    @torch.no_grad()
    def initialize_parameters(self, sae: SparseDictionary):
        sae.init_parameters(encoder_uniform_bound=self.cfg.encoder_uniform_bound,
                            decoder_uniform_bound=self.cfg.decoder_uniform_bound,
                            init_log_jumprelu_threshold_value=self.cfg.init_log_jumprelu_threshold_value)
        if self.cfg.init_encoder_with_decoder_transpose:
            assert hasattr(sae, "init_encoder_with_decoder_transpose"), (
                f"{type(sae).__name__} does not support encoder initialization from decoder")
            sae.init_encoder_with_decoder_transpose(self.cfg.init_encoder_with_decoder_transpose_factor)
        return sae

    def _init_encoder_side(self, sae: SparseDictionary, batch: dict) -> None:
        if self.cfg.init_encoder_with_decoder_transpose:
            assert hasattr(sae, "init_encoder_with_decoder_transpose"), (
                f"{type(sae).__name__} does not support encoder initialization from decoder")
            sae.init_encoder_with_decoder_transpose(self.cfg.init_encoder_with_decoder_transpose_factor)
        if self.cfg.init_encoder_bias_with_mean_hidden_pre:
            assert hasattr(sae, "init_encoder_bias_with_mean_hidden_pre"), (
                f"{type(sae).__name__} does not support encoder bias initialization")
            sae.init_encoder_bias_with_mean_hidden_pre(batch)

    @torch.no_grad()
    def grid_search_best_init_norm(self, sae: SparseDictionary, batch: dict, search_range: List[float]) -> float:
        """initializer.py:115-137: reconstruction error of `batch` with the decoder rows set to each norm in
        turn (the encoder re-derived from it each time); returns the first norm with the lowest error."""
        assert hasattr(sae, "set_decoder_to_fixed_norm"), f"{type(sae).__name__} does not support norm constraints"
        losses: dict[float, float] = {}
        dev_type = next(sae.parameters()).device.type
        for norm in search_range:
            sae.set_decoder_to_fixed_norm(norm, force_exact=True)
            self._init_encoder_side(sae, batch)
            with torch.autocast(device_type=dev_type, dtype=sae.cfg.dtype, enabled=sae.cfg.dtype != torch.float32):
                mse = sae.compute_loss(batch)["l_rec"].mean().item()
            losses[norm] = mse
        return min(losses, key=losses.get)  # type: ignore[arg-type]

    @torch.no_grad()
    def initialization_search(self, sae: SparseDictionary, activation_batch: dict):
        batch = sae.normalize_activations(activation_batch)
        if self.cfg.bias_init_method == "geometric_median":
            assert sae.b_D is not None, "Decoder bias should exist if use_decoder_bias is True"
            # a cross-layer transcoder has one bias per layer (a list of vectors, or one [layers, d] tensor)
            if hasattr(sae.cfg, "hook_points_out") and (not torch.is_tensor(sae.b_D) or sae.b_D.ndim == 2):
                for i, hp in enumerate(sae.cfg.hook_points_out):
                    sae.b_D[i].copy_(batch[hp].mean(0))
            elif hasattr(sae.cfg, "hook_point_out"):
                label = sae.prepare_label(batch)
                sae.b_D.copy_(label.mean(dim=list(range(batch[sae.cfg.hook_point_out].ndim - 1))))
            else:
                raise ValueError(
                    f"Bias initialization method {self.cfg.bias_init_method} is not supported for {sae.cfg.sae_type}")
        if self.cfg.grid_search_init_norm:
            coarse = self.grid_search_best_init_norm(sae, batch, torch.linspace(0.1, 5.0, 50).numpy().tolist())
            fine = self.grid_search_best_init_norm(sae, batch, torch.linspace(coarse - 0.09, coarse + 0.1, 20).numpy().tolist())
            self.best_norm = fine
            sae.set_decoder_to_fixed_norm(fine, force_exact=True)
        self._init_encoder_side(sae, batch)
        return sae

    def initialize_sae_from_config(self, cfg: SparseDictionaryConfig, activation_stream: Optional[Iterable[dict]] = None,
                                   activation_norm: Optional[dict[str, float]] = None, device_mesh=None):
        sae = SparseDictionary.from_config(cfg, device_mesh=device_mesh)
        if cfg.sae_pretrained_name_or_path is not None:
            return sae
        sae = self.initialize_parameters(sae)
        if sae.cfg.norm_activation == "dataset-wise":
            if activation_norm is None:
                assert activation_stream is not None, "Activation iterator must be provided for dataset-wise normalization"
                activation_norm = calculate_activation_norm(activation_stream, cfg.associated_hook_points)
            sae.set_dataset_average_activation_norm(activation_norm)
        assert activation_stream is not None, "Activation iterator must be provided for initialization search"
        activation_batch = next(iter(activation_stream))
        return self.initialization_search(sae, activation_batch)
