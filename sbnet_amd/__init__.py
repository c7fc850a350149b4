"""sbnet_amd: MI355X (gfx950) implementation of Sparse Blocks Network's three custom ops.

`reduce_mask`, `sparse_gather`, `sparse_scatter` and `sparse_scatter_var` keep the reference's op
names and arguments (the gather and the copying scatter are differentiable, with the reference's
gradient definitions); they call hand-written HIP kernels through the C ABI of libsbnet_amd.so
(include/sbnet_amd.h).  Importing the package does not load the library; the first op call does,
and raises if it has not been built.
"""
from .block_params import (BlockParams, calc_block_params, calc_block_params_res_block,  # noqa: F401
                           calc_block_count_covering)
from .ops import (HipError, InvalidArgument, ReduceMaskResult, reduce_mask, release_workspaces,  # noqa: F401
                  sparse_gather, sparse_scatter, sparse_scatter_var)
from .autograd import SparseGatherFunction, SparseScatterFunction  # noqa: F401

__all__ = [
    "reduce_mask", "sparse_gather", "sparse_scatter", "sparse_scatter_var", "ReduceMaskResult",
    "InvalidArgument", "HipError", "release_workspaces", "SparseGatherFunction", "SparseScatterFunction", "BlockParams", "calc_block_params", "calc_block_params_res_block",
    "calc_block_count_covering",
]
