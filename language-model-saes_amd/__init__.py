"""MI355X-native SAE train-step path (HIP kernels behind the Llamascopium module API).

The directory name is not a Python identifier; load it under the alias `lm_saes_amd`
(see `__graft_entry__.load_package`).
"""

from . import _lib, ops  # noqa: F401
from .ops import FeatureIndex, SparseCode  # noqa: F401

__all__ = ["_lib", "ops", "SparseCode", "FeatureIndex"]
