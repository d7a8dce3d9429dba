"""ELO_CUDA (Adafactor-MLP learned optimizer) on MI355X: AdafacLO's multi-tensor HIP step with ELO's
gradient conditioning and update rule.

Drop-in for pylo/optim/ELO_cuda.py:55-288: same constructor, ``step()``, ``param_groups`` keys
(``lr, exp_mult, weight_decay, clip_grad, clip_norm``) and per-parameter state (``step`` float64 CPU
scalar, ``exp_avg (3,*s)``, ``exp_avg_sq (*s)``, ``exp_avg_sq_r``, ``exp_avg_sq_c``).  What ELO changes
against AdafacLO (pylo/optim/ELO_naive.py:127-238):

* the accumulator decays are used as given, clamped to [0, 1] (no offset re-parameterisation);
* optional clipping by the global gradient norm, then ``torch.nan_to_num`` of every gradient: both run
  inside the kernels (``clip_norm`` column, tensor flags ``PYLO_F_GLOBAL_NORM | PYLO_F_NAN_TO_NUM``
  with ``clip_val = FLT_MAX``), so no gradient is copied;
* ``p -= lr * (step + weight_decay * p)`` with the pre-step parameter (``PYLO_F_WD_PRESTEP``); the
  reference's CUDA class snapshots ``p`` for this (ELO_cuda.py:244-247,285-286), here it is one fused
  expression in the apply pass.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch.optim import Optimizer

from .. import _lib
from ..models import MetaMLP, pack_metamlp
from .AdafacLO_cuda import AdafacLO_CUDA

_FLT_MAX = float(torch.finfo(torch.float32).max)


class ELO_CUDA(AdafacLO_CUDA):
    _PLAN_FLAGS = _lib.F_NAN_TO_NUM | _lib.F_WD_PRESTEP | _lib.F_GLOBAL_NORM

    def __init__(
        self,
        params,
        lr=0.001,
        exp_mult=0.001,
        weight_decay=0.0,
        hidden_size=32,
        hidden_layers=1,
        initial_momentum_decays=(0.9, 0.99, 0.999),
        initial_rms_decays=(0.999,),
        initial_adafactor_decays=(0.9, 0.99, 0.999),
        clip_grad=False,
        clip_norm=1.0,
        hf_key: Optional[str] = "DiamondXL/elo",
        checkpoint_path: Optional[str] = None,
        network: Optional[MetaMLP] = None,
        capturable: bool = False,
    ):
        if not torch.cuda.is_available():
            raise RuntimeError("ELO_CUDA requires a GPU (torch.cuda.is_available() is False).")
        self.capturable = bool(capturable)
        _lib.load()
        defaults = dict(lr=lr, exp_mult=exp_mult, weight_decay=weight_decay, clip_grad=clip_grad,
                        clip_norm=clip_norm)
        Optimizer.__init__(self, params, defaults)
        first = next(p for g in self.param_groups for p in g["params"])
        self.device = first.device if first.is_cuda else torch.device("cuda", torch.cuda.current_device())

        def raw(v):
            return torch.clamp(torch.tensor(v, dtype=torch.float32, device=self.device), 0.0, 1.0)

        self.beta_m, self.beta_rms, self.beta_adafactor = (raw(initial_momentum_decays), raw(initial_rms_decays),
                                                           raw(initial_adafactor_decays))
        if (self.beta_m.numel(), self.beta_rms.numel(), self.beta_adafactor.numel()) != (3, 1, 3):
            raise ValueError("the fused step supports 3 momentum decays, 1 rms decay and 3 adafactor decays")
        # precedence as in ELO_cuda.py:119-133: explicit network > local checkpoint > hub id > fresh
        if network is None:
            if checkpoint_path is not None:
                network = MetaMLP(input_size=39, hidden_size=hidden_size, hidden_layers=hidden_layers)
                network.load_state_dict(torch.load(checkpoint_path, map_location="cpu", weights_only=True))
            elif hf_key is not None:
                network = MetaMLP.from_pretrained(hf_key)
            else:
                network = MetaMLP(input_size=39, hidden_size=hidden_size, hidden_layers=hidden_layers)
        self.network = network.to(self.device)
        for prm in self.network.parameters():
            prm.requires_grad = False
        net = self.network.network
        if not (hasattr(net, "input") and hasattr(net, "linear_0") and hasattr(net, "output")) \
                or hasattr(net, "linear_1"):
            raise ValueError("ELO_CUDA kernel only supports hidden_layers=1 (39->32->32->2).")
        self._net = pack_metamlp(self.network).to(self.device)     # raises on any other geometry
        self._decays = _lib.make_decays(self.beta_m.tolist(), float(self.beta_rms[0]), self.beta_adafactor.tolist())
        self._plan = None
        self._plan_key = None

    def _norm_flags(self):
        return 0        # global-norm clipping (ELO_cuda.py:153-161): _PLAN_FLAGS

    def _scalars(self, group):
        return dict(lr=group["lr"], weight_decay=group["weight_decay"], exp_mult=group["exp_mult"], step_mult=1.0,
                    clip_norm=group["clip_norm"] if group["clip_grad"] else 0.0, clip_val=_FLT_MAX)
