"""Fused learned-optimizer classes (same public names as ``pylo.optim``)."""

from .AdafacLO_cuda import AdafacLO_CUDA
from .CELO2_cuda import CELO2_CUDA
from .ELO_CELO2_cuda import ELO_CELO2_CUDA
from .ELO_cuda import ELO_CUDA
from .MuLO_cuda import MuLO_CUDA
from .velo_cuda import VeLO_CUDA

ELO_CELO2 = ELO_CELO2_CUDA
CELO2 = CELO2_CUDA
ELO = ELO_CUDA
MuLO = MuLO_CUDA
VeLO = VeLO_CUDA
AdafacLO = AdafacLO_CUDA

__all__ = ["ELO_CELO2_CUDA", "ELO_CELO2", "CELO2_CUDA", "CELO2", "ELO_CUDA", "ELO", "MuLO_CUDA", "MuLO", "VeLO_CUDA", "VeLO", "AdafacLO_CUDA", "AdafacLO"]
