"""scattermoe_amd — ScatterMoE for MI355X (gfx950): the Python surface of shawntan/scattermoe over
hand-written HIP kernels (reference package root: scattermoe/__init__.py:1-15)."""
import os

from .parallel_experts import flatten_sort_count, flatten_and_sort, parallel_linear, ParallelExperts
from . import parallel_experts
from . import kernels
from . import mlp

if os.environ.get("SCATTERMOE_NO_HF_PATCH", "0") != "1":
    from . import utils
else:  # the submodule stays importable on demand; only the import-time Hugging Face patching is skipped
    utils = None

__all__ = [
    "flatten_sort_count",
    "flatten_and_sort",
    "parallel_linear",
    "ParallelExperts",
    "parallel_experts",
    "kernels",
    "mlp",
    "utils",
]
