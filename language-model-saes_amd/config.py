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

    @classmethod
    def from_pretrained(cls, pretrained_name_or_path: str, strict_loading: bool = True, **kwargs):
        """Read `<path>/config.json` as the reference writes it (models/sparse_dictionary.py:156-186) and build
        the config class its `sae_type` names; `kwargs` (device, dtype, ...) override the file.  A path to a
        weights file stands for its directory.  Hub names are not resolved here."""
        import json
        import os

        root = pretrained_name_or_path
        if os.path.isfile(root):
            root = os.path.dirname(root)
            if os.path.basename(root) == "checkpoints" and not os.path.exists(os.path.join(root, "config.json")):
                root = os.path.dirname(root)
        path = os.path.join(root, "config.json")
        if not os.path.exists(path):
            raise FileNotFoundError(f"no config.json under {root!r} (only local directories are supported)")
        with open(path, "r") as f:
            d = json.load(f)
        d["sae_pretrained_name_or_path"] = pretrained_name_or_path
        d["strict_loading"] = strict_loading
        if cls is SparseDictionaryConfig:
            cls = SAE_TYPE_TO_CONFIG_CLASS[d["sae_type"]]
        return cls.model_validate({**d, **kwargs})

    def save_hyperparameters(self, sae_path, remove_loading_info: bool = True) -> None:
        """Write `<sae_path>/config.json` (models/sparse_dictionary.py:188-196)."""
        import json
        import os

        assert os.path.exists(sae_path), f"{sae_path} does not exist. Unable to save hyperparameters."
        d = self.model_dump()
        if remove_loading_info:
            d.pop("sae_pretrained_name_or_path", None)
            d.pop("strict_loading", None)
        with open(os.path.join(sae_path, "config.json"), "w") as f:
            json.dump(d, f, indent=4)

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


@register_sae_config("crosscoder")
class CrosscoderConfig(SparseDictionaryConfig):
    """models/crosscoder.py:60-81: one head per hook point; reads and writes the same hook points."""

    sae_type: str = "crosscoder"
    hook_points: list[str]

    @property
    def associated_hook_points(self) -> list[str]:
        return self.hook_points

    @property
    def hooks_in(self) -> list[str]:
        return self.hook_points

    @property
    def hooks_out(self) -> list[str]:
        return self.hook_points

    @property
    def n_heads(self) -> int:
        return len(self.hook_points)


@register_sae_config("clt")
class CLTConfig(SparseDictionaryConfig):
    """models/clt.py:67-121: L encoders, L(L+1)/2 decoders (layer i writes to layers i..L-1)."""

    sae_type: str = "clt"
    act_fn: Literal["relu", "jumprelu", "topk", "batchtopk", "batchlayertopk", "layertopk"] = "relu"
    init_cross_layer_decoder_all_zero: bool = False
    hook_points_in: list[str]
    hook_points_out: list[str]
    # Kept for config compatibility: the reference switches its decode to torch CSR matrices with these;
    # here the sparse decode kernel is used whenever the activation is of the TopK family.
    decode_with_csr: bool = False
    sparsity_threshold_for_csr: float = 0.05

    @property
    def n_layers(self) -> int:
        return len(self.hook_points_in)

    @property
    def n_decoders(self) -> int:
        return self.n_layers * (self.n_layers + 1) // 2

    @property
    def associated_hook_points(self) -> list[str]:
        return self.hook_points_in + self.hook_points_out

    @property
    def hooks_in(self) -> list[str]:
        return self.hook_points_in

    @property
    def hooks_out(self) -> list[str]:
        return self.hook_points_out

    def model_post_init(self, __context):
        super().model_post_init(__context)
        assert len(self.hook_points_in) == len(self.hook_points_out), "Number of input and output hook points must match"


@register_sae_config("lorsa")
class LorsaConfig(SparseDictionaryConfig):
    """models/lorsa.py:45-106: every dictionary feature is a rank-1 value/output head; groups of
    d_sae / n_qk_heads features share one query/key head."""

    sae_type: str = "lorsa"
    hook_point_in: str
    hook_point_out: str
    n_qk_heads: int
    d_qk_head: int
    positional_embedding_type: Literal["rotary", "none"] = "rotary"
    rotary_dim: int
    rotary_base: int = 10000
    rotary_adjacent_pairs: bool = True
    rotary_scale: int = 1
    use_NTK_by_parts_rope: bool = False
    NTK_by_parts_factor: float = 1.0
    NTK_by_parts_low_freq_factor: float = 1.0
    NTK_by_parts_high_freq_factor: float = 1.0
    old_context_len: int = 2048
    n_ctx: int
    attn_scale: Optional[float] = None
    use_post_qk_ln: bool = False
    normalization_type: Optional[Literal["LN", "RMS"]] = None
    eps: float = 1e-6

    @property
    def n_ov_heads(self) -> int:
        return self.d_sae

    @property
    def ov_group_size(self) -> int:
        return self.n_ov_heads // self.n_qk_heads

    @property
    def associated_hook_points(self) -> list[str]:
        return [self.hook_point_in, self.hook_point_out]

    @property
    def hooks_in(self) -> list[str]:
        return [self.hook_point_in]

    @property
    def hooks_out(self) -> list[str]:
        return [self.hook_point_out]

    def model_post_init(self, __context):
        super().model_post_init(__context)
        assert self.hook_point_in is not None and self.hook_point_out is not None, "hook_point_in and hook_point_out must be set"
        assert self.hook_point_in != self.hook_point_out, "hook_point_in and hook_point_out must be different"
        assert self.n_ov_heads % self.n_qk_heads == 0, "n_ov_heads must be divisible by n_qk_heads"
        if self.attn_scale is None:
            self.attn_scale = self.d_qk_head ** 0.5
