"""MI355X-native scatter / segment / gather reductions with torch_scatter's API.

``import pytorch_scatter_amd as torch_scatter`` gives the function surface of
the reference package (torch_scatter/__init__.py:67-94). Importing registers
``torch.ops.torch_scatter.*`` from ``_torch_scatter_hip.so``, which runs
hand-written gfx950 kernels through the C ABI of ``libts_hip.so``. Both
libraries are built in-tree (``make -C pytorch_scatter_amd/csrc all torch``).
There is no CPU implementation here: inputs must live on the GPU.
"""
import os

import torch

__version__ = "0.1.0"

_HERE = os.path.dirname(os.path.abspath(__file__))
_OPS_LIB = os.path.join(_HERE, "_torch_scatter_hip.so")
_KERNEL_LIB = os.path.join(_HERE, "libts_hip.so")

for _path in (_KERNEL_LIB, _OPS_LIB):
    if not os.path.exists(_path):
        raise ImportError(
            f"{_path} is missing: build the HIP extension first "
            "(`make -C pytorch_scatter_amd/csrc -j8 all torch` or "
            "`python -c 'import __graft_entry__ as g; g.build()'`). "
            "This package has no CPU or pure-PyTorch fallback.")

# the reference loads one library per op family (torch_scatter/__init__.py:9-16);
# here a single library registers all 16 operators
torch.ops.load_library(_OPS_LIB)

hip_version = torch.ops.torch_scatter.cuda_version()  # HIP_VERSION of the build

from .index_format import (SortedIndex, index_to_indptr, indptr_to_index,  # noqa: E402
                           scatter_sorted)
from .index_reuse import (disable_index_reuse, enable_index_reuse,  # noqa: E402
                          index_reuse_enabled)
from .scatter import (scatter, scatter_add, scatter_max, scatter_mean,  # noqa: E402
                      scatter_min, scatter_mul, scatter_sum)
from .segment_coo import (gather_coo, segment_add_coo, segment_coo,  # noqa: E402
                          segment_max_coo, segment_mean_coo, segment_min_coo,
                          segment_sum_coo)
from .segment_csr import (gather_csr, segment_add_csr, segment_csr,  # noqa: E402
                          segment_max_csr, segment_mean_csr, segment_min_csr,
                          segment_sum_csr)
from .composite import (scatter_log_softmax, scatter_logsumexp,  # noqa: E402
                        scatter_softmax, scatter_std)

__all__ = [
    "scatter_sum", "scatter_add", "scatter_mul", "scatter_mean", "scatter_min",
    "scatter_max", "scatter",
    "segment_sum_csr", "segment_add_csr", "segment_mean_csr", "segment_min_csr",
    "segment_max_csr", "segment_csr", "gather_csr",
    "segment_sum_coo", "segment_add_coo", "segment_mean_coo", "segment_min_coo",
    "segment_max_coo", "segment_coo", "gather_coo",
    "scatter_std", "scatter_logsumexp", "scatter_softmax", "scatter_log_softmax",
    "SortedIndex", "index_to_indptr", "indptr_to_index", "scatter_sorted",
    "enable_index_reuse", "disable_index_reuse", "index_reuse_enabled",
    "hip_version", "__version__",
]
