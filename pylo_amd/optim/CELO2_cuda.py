"""CELO2_CUDA on MI355X: the reference's CELO2 optimizer on the same multi-tensor HIP step as
ELO_CELO2_CUDA.

Drop-in for pylo/optim/CELO2_cuda.py:54-345: same constructor defaults (``weight_decay=0``,
``adam_lr_mult=1``, ``clip_grad=False``, ``adam_betas``, ``adam_eps``, ``hf_key="DiamondXL/celo2"``),
``param_groups`` keys and per-parameter state.  The only arithmetic difference from ELO-CELO2 is
the AdamW branch of 1-D / embedding tensors (pylo/optim/CELO2_cuda.py:234-253): it keeps its own
moments ``exp_avg`` / ``exp_avg_sq`` with its own decays and a per-parameter ``adam_step`` counter,
and adds ``adam_eps`` outside the square root.  In the library that is the tensor flag
``PYLO_F_ADAM_INDEP`` plus three fields of ``PyloDecays``.
"""

from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import _lib
from ..models import CELO2MLP
from .ELO_CELO2_cuda import ELO_CELO2_CUDA


class CELO2_CUDA(ELO_CELO2_CUDA):
    """Inference-time CELO2: CELO2 MLP steps for >=2-D tensors, independent-moment AdamW for 1-D
    tensors and ``is_embedding`` groups."""

    _ADAM_FLAG = _lib.F_ADAM_INDEP

    def __init__(
        self,
        params,
        lr=1e-3,
        weight_decay=0.0,
        adam_lr_mult=1.0,
        adam_weight_decay=None,
        adam_betas=(0.9, 0.95),
        adam_eps=1e-8,
        use_adamw_for_1d=True,
        orthogonalize=True,
        clip_grad=False,
        clip_norm=1.0,
        ff_hidden_size=8,
        ff_hidden_layers=2,
        initial_momentum_decays=(0.9, 0.99, 0.999),
        initial_rms_decays=(0.95,),
        initial_adafactor_decays=(0.9, 0.99, 0.999),
        exp_mult=0.0,
        rmsmult=1.0,
        param_scale_mult=False,
        ns_coeffs=(3.4445, -4.7750, 2.0315),
        ns_iters=5,
        ns_eps=1e-8,
        grad_clip_val=1000.0,
        hf_key: Optional[str] = "DiamondXL/celo2",
        checkpoint_path: Optional[str] = None,
        network: Optional[CELO2MLP] = None,
        capturable: bool = False,
    ):
        super().__init__(
            params, lr=lr, weight_decay=weight_decay, clip_grad=clip_grad, clip_norm=clip_norm,
            adam_lr_mult=adam_lr_mult, adam_weight_decay=adam_weight_decay,
            use_adamw_for_1d=use_adamw_for_1d, orthogonalize=orthogonalize,
            ff_hidden_size=ff_hidden_size, ff_hidden_layers=ff_hidden_layers,
            initial_momentum_decays=initial_momentum_decays, initial_rms_decays=initial_rms_decays,
            initial_adafactor_decays=initial_adafactor_decays, exp_mult=exp_mult, rmsmult=rmsmult,
            param_scale_mult=param_scale_mult, ns_coeffs=ns_coeffs, ns_iters=ns_iters, ns_eps=ns_eps,
            grad_clip_val=grad_clip_val, hf_key=hf_key, checkpoint_path=checkpoint_path, network=network,
            capturable=capturable)
        self.adam_beta1, self.adam_beta2 = (float(b) for b in adam_betas)
        self.adam_eps = adam_eps
        self._decays = _lib.make_decays(self.beta_m.tolist(), float(self.beta_rms[-1]), self.beta_fac.tolist(),
                                        adam_betas=(self.adam_beta1, self.adam_beta2), adam_eps=adam_eps)

    def _init_state(self, state, p, adam):
        if not adam:
            return super()._init_state(state, p, adam)
        state["exp_avg"] = torch.zeros_like(p)
        state["exp_avg_sq"] = torch.zeros_like(p)
        state["adam_step"] = 0

    # pylo/optim/CELO2_cuda.py:241-251: the counter is per parameter and advances only on steps in
    # which the parameter has a gradient
    def _adam_row(self, group, state):
        if not self.capturable:
            state["adam_step"] += 1
        t = state["adam_step"]
        return (state["exp_avg"].data_ptr(), state["exp_avg_sq"].data_ptr(),
                1.0 - self.adam_beta1 ** t, 1.0 - self.adam_beta2 ** t)

    # device-side counters (capturable=True): one per AdamW parameter
    def _step_values(self, tensors):
        return [self.state[p].get("adam_step", 0) if a else 0 for _g, p, a in tensors]

    def _step_betas(self):
        return self.adam_beta1, self.adam_beta2

    def _store_step_values(self, tensors, values):
        for (_g, p, a), v in zip(tensors, values):
            if a and "adam_step" in self.state[p]:
                self.state[p]["adam_step"] = v

    def _adam_corrections_fast(self, fast, per_group):
        steps = fast.get("adam_states")
        if steps is None:
            steps = fast["adam_states"] = [self.state[p] for p, a in zip(fast["params"], fast["adam"]) if a]
        t = np.zeros(len(fast["params"]), dtype=np.float64)
        for s in steps:
            s["adam_step"] += 1
        t[fast["adam"]] = [s["adam_step"] for s in steps]
        adam = fast["adam"]
        return (np.where(adam, 1.0 - self.adam_beta1 ** t, 0.0),
                np.where(adam, 1.0 - self.adam_beta2 ** t, 0.0))
