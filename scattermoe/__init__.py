"""`import scattermoe` compatibility: the same module tree as shawntan/scattermoe, served by scattermoe_amd."""
import importlib
import sys

import scattermoe_amd as _impl
from scattermoe_amd import *  # noqa: F401,F403
from scattermoe_amd import flatten_sort_count, parallel_linear, ParallelExperts, parallel_experts, kernels, mlp, utils

__all__ = list(_impl.__all__)

for _name in ("parallel_experts", "kernels", "kernels.ops", "kernels.single", "mlp", "utils", "utils.replace_moe"):
    try:
        sys.modules[__name__ + "." + _name] = importlib.import_module("scattermoe_amd." + _name)
    except Exception:      # utils.* needs transformers' model classes only when they exist
        pass
