"""MI355X-native SAE train-step path (HIP kernels behind the Llamascopium module API).

The directory name is not a Python identifier; load it under the alias `lm_saes_amd`
(see `__graft_entry__.load_package`).
"""

from . import _lib, ops  # noqa: F401
from .ops import FeatureIndex, SparseCode  # noqa: F401

__all__ = ["_lib", "ops", "SparseCode", "FeatureIndex"]

from .config import SAEConfig, SparseDictionaryConfig  # noqa: E402,F401
from .activation_functions import JumpReLU  # noqa: E402,F401
from .sparse_dictionary import SparseDictionary  # noqa: E402,F401
from .sae import SparseAutoEncoder  # noqa: E402,F401
from .optim import HipAdam  # noqa: E402,F401

__all__ += ["SAEConfig", "SparseDictionaryConfig", "JumpReLU", "SparseDictionary", "SparseAutoEncoder", "HipAdam"]

from .optim import HipSparseAdam, clip_grad_norm, compute_grad_norm  # noqa: E402,F401
from .trainer import Trainer, TrainerConfig, get_scheduler  # noqa: E402,F401

__all__ += ["HipSparseAdam", "clip_grad_norm", "compute_grad_norm", "Trainer", "TrainerConfig", "get_scheduler"]

from .config import CLTConfig, CrosscoderConfig, LorsaConfig  # noqa: E402,F401
from .crosscoder import Crosscoder  # noqa: E402,F401
from .clt import CrossLayerTranscoder  # noqa: E402,F401
from .lorsa import LowRankSparseAttention  # noqa: E402,F401

__all__ += ["CrosscoderConfig", "CLTConfig", "LorsaConfig", "Crosscoder", "CrossLayerTranscoder", "LowRankSparseAttention"]

from . import kernels, metrics  # noqa: E402,F401
from .activation import (  # noqa: E402,F401
    ActivationBatchler, ActivationTransformer, ActivationWriter, ActivationWriterConfig, BufferShuffleConfig,
    CachedActivationLoader, ChunkInfo, cached_activation_stream,
)
from .initializer import Initializer, InitializerConfig, calculate_activation_norm  # noqa: E402,F401

__all__ += ["metrics", "ActivationBatchler", "ActivationTransformer", "ActivationWriter", "ActivationWriterConfig",
            "BufferShuffleConfig", "CachedActivationLoader", "ChunkInfo", "cached_activation_stream", "Initializer",
            "InitializerConfig", "calculate_activation_norm"]
