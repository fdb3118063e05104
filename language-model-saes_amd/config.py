"""Configuration objects of the sparse-dictionary models.

Field names, defaults and the `sae_type` registry follow the reference
(src/llamascopium/config.py:19-40, models/sparse_dictionary.py:90-214, models/sae.py:32-49)
so that a reference `config.json` loads unchanged.
"""

from __future__ import annotations

from typing import Annotated, Literal, Optional

import torch
from pydantic import BaseModel, BeforeValidator, ConfigDict, Field, PlainSerializer

_DTYPES = {
    "torch.float32": torch.float32, "float32": torch.float32, "fp32": torch.float32,
    "torch.bfloat16": torch.bfloat16, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "torch.float16": torch.float16, "float16": torch.float16,
    "torch.float64": torch.float64, "float64": torch.float64,
}


def str_to_dtype(v):
    if isinstance(v, str):
        if v not in _DTYPES:
            raise ValueError(f"unknown dtype string {v!r}")
        return _DTYPES[v]
    return v


TorchDtype = Annotated[torch.dtype, BeforeValidator(str_to_dtype), PlainSerializer(lambda d: str(d))]


class BaseModelConfig(BaseModel):
    model_config = ConfigDict(arbitrary_types_allowed=True)
    device: str = Field(default="cpu", exclude=True)
    dtype: TorchDtype = Field(default=torch.float32, exclude=True, validate_default=False)


SAE_TYPE_TO_CONFIG_CLASS: dict[str, type] = {}
SAE_TYPE_TO_MODEL_CLASS: dict[str, type] = {}


def register_sae_config(name: str):
    def deco(cls):
        SAE_TYPE_TO_CONFIG_CLASS[name] = cls
        return cls
    return deco


def register_sae_model(name: str):
    def deco(cls):
        SAE_TYPE_TO_MODEL_CLASS[name] = cls
        return cls
    return deco


class SparseDictionaryConfig(BaseModelConfig):
    sae_type: str
    d_model: int
    expansion_factor: float
    use_decoder_bias: bool = True
    act_fn: Literal["relu", "jumprelu", "topk", "batchtopk", "batchlayertopk", "layertopk"] = "relu"
    norm_activation: Literal["token-wise", "batch-wise", "dataset-wise", "inference"] = "dataset-wise"
    sparsity_include_decoder_norm: bool = True
    top_k: int = 50
    sae_pretrained_name_or_path: Optional[str] = None
    strict_loading: bool = True
    # Kept for config compatibility.  The reference's flag selects its Triton SpMM; here the
    # HIP kernels are the only GPU path, so the flag does not change what runs.
    use_triton_kernel: bool = False
    sparsity_threshold_for_triton_spmm_kernel: float = 0.996
    jumprelu_threshold_window: float = 2.0

    @property
    def d_sae(self) -> int:
        return int(self.d_model * self.expansion_factor)

    @property
    def associated_hook_points(self) -> list[str]:
        raise NotImplementedError

    @property
    def hooks_in(self) -> list[str]:
        raise NotImplementedError

    @property
    def hooks_out(self) -> list[str]:
        raise NotImplementedError


@register_sae_config("sae")
class SAEConfig(SparseDictionaryConfig):
    sae_type: str = "sae"
    hook_point_in: str
    hook_point_out: str
    use_glu_encoder: bool = False

    @property
    def associated_hook_points(self) -> list[str]:
        return [self.hook_point_in, self.hook_point_out]

    @property
    def hooks_in(self) -> list[str]:
        return [self.hook_point_in]

    @property
    def hooks_out(self) -> list[str]:
        return [self.hook_point_out]
