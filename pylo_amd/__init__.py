"""pylo_amd: the fused learned-optimizer step of PyLO, native to MI355X (gfx950).

Public names mirror ``pylo``: the meta-network containers and the ``*_CUDA`` optimizer
classes (here backed by hand-written HIP kernels behind a C ABI; there is no fallback path).
"""

from .models import CELO2MLP, MetaMLP, VeLOMLP, VeLORNN
from .optim import *  # noqa: F401,F403
from .optim import __all__ as _optim_all

__all__ = ["MetaMLP", "VeLOMLP", "VeLORNN", "CELO2MLP"] + list(_optim_all)
