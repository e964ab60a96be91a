"""MI355X-native execution path of a sparse Mixture-of-Experts layer.

The class surface mirrors louislichen/SPARSE's ``DistributedSparseMoeBlock``
(utils/eval_core.py:4408-4440, :16418-16563); the kernels live in
``sparse_amd/csrc/libsparse_hip.so`` behind the C ABI of ``include/sparse_hip.h``.
"""
from .context import DistEnv, Metrics, SparseContext  # noqa: F401
from .block import DistributedSparseMoeBlock  # noqa: F401
from .methods import METHODS, method_settings, residency_config  # noqa: F401

__all__ = ["DistEnv", "Metrics", "SparseContext", "DistributedSparseMoeBlock", "METHODS", "method_settings",
           "residency_config"]
