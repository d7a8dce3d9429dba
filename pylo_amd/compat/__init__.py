"""Modules with the names and call signatures of the reference's three extension modules
(``celo2_cuda_kernel``, ``cuda_lo``, ``velo_cuda_kernel``; pylo/csrc/*.cu, bound with pybind11), on
the single-tensor entry points of ``libpylo_mi355.so``.

They exist so that code written against the reference's per-tensor kernels keeps working::

    from pylo_amd.compat import celo2_cuda_kernel        # instead of: import celo2_cuda_kernel
    celo2_cuda_kernel.celo2_kernel(g, p, m, v, fac_r, fac_c, row_factor, col_factor, second_moment,
                                   w_in, b_in, w_h, b_h, w_out, b_out, step_out, exp_mult, dc, dr, vector_like)

``install()`` registers them in ``sys.modules`` under the reference's bare names.  The optimizer classes
of ``pylo_amd`` do not use these calls: they go through the multi-tensor plans, which also fuse the
accumulator updates.  Tensors must be contiguous float32 CUDA tensors (the reference dispatches on
dtype; here anything else raises).  Launches go to torch's current stream.
"""

import sys

from . import celo2_cuda_kernel, cuda_lo, velo_cuda_kernel

__all__ = ["celo2_cuda_kernel", "cuda_lo", "velo_cuda_kernel", "install"]


def install() -> None:
    """Make ``import celo2_cuda_kernel`` / ``cuda_lo`` / ``velo_cuda_kernel`` resolve to these modules."""
    for mod in (celo2_cuda_kernel, cuda_lo, velo_cuda_kernel):
        sys.modules.setdefault(mod.__name__.rsplit(".", 1)[1], mod)
