"""AdafacLO_CUDA (small_fc_lopt) on MI355X: one multi-tensor HIP step per optimizer step.

Drop-in for pylo/optim/AdafacLO_cuda.py:76-407: same constructor and ``step()``, per-parameter state
``step`` (float64 CPU scalar), ``exp_avg (3,*s)``, ``exp_avg_sq (*s)``, ``exp_avg_sq_r``,
``exp_avg_sq_c``.  Arithmetic follows the naive class (pylo/optim/AdafacLO_naive.py:187-311); in
particular ``row_col_mean`` averages over the 2nd-largest parameter dim (the reference's CUDA class
reduces the decay axis instead, AdafacLO_cuda.py:342-343), and 1-D tensors use
``m * (v + 1e-6)^-1/2`` for the last feature group (AdafacLO_naive.py:298).
"""

from __future__ import annotations

from typing import Optional, Union

import torch
from torch.optim import Optimizer

from .. import _lib
from ..models import MetaMLP, pack_metamlp


def _factored_dims(shape):
    """(dc, dr): 2nd-largest and largest dim, ties by index (AdafacLO_cuda.py:52-73 with
    min_dim_size_to_factor=1)."""
    if len(shape) < 2:
        return None
    order = sorted(range(len(shape)), key=lambda i: (shape[i], i))
    return order[-2], order[-1]


def _decays(initial, offsets, device):
    """clip(1 - exp(10 * (log(1 - d0) / 10 + offset)), 0, 1) in fp32 (AdafacLO_cuda.py:29-34,153-173)."""
    off = offsets if torch.is_tensor(offsets) else torch.tensor(offsets, device=device)
    par = torch.log(1 - torch.tensor(initial, device=device)) / 10.0 + off.to(device)
    return torch.clip(1 - torch.exp(par * 10.0), 0.0, 1.0)


class AdafacLO_CUDA(Optimizer):
    _PLAN_FLAGS = 0      # PyloTensorShape.flags of every tensor
    # capturable=True: the per-parameter step counters live on the device and ``step()`` can be recorded
    # into a HIP graph (torch.cuda.graph) and replayed; ``state[p]["step"]`` is then refreshed by
    # ``state_dict()`` / ``sync_step_counters()`` only.  The reference has no such mode.
    capturable = False
    _dev_steps = None

    def __init__(
        self,
        params,
        lr: float = 1.0,
        min_dim_size_to_factor: int = 32,
        decay_rate: float = 0.8,
        decay_offset: int = 0,
        beta2_cap: float = 0.999,
        initial_momentum_decays=(0.9, 0.99, 0.999),
        initial_rms_decays=(0.999,),
        initial_adafactor_decays=(0.9, 0.99, 0.999),
        momentum_decays=[0.15216392, 0.14245212, 0.06812963],
        rms_decays=[0.01079706],
        adafactor_decays=[0.18621896, -0.10864615, -0.06185547],
        momentum_dtype: Union[str, torch.dtype] = torch.float32,
        eps: Optional[float] = None,
        weight_decay: float = 0.0,
        clipping_threshold: Optional[float] = None,
        max_grad_norm: Optional[float] = None,
        unscaled_wd: bool = False,
        step_mult: float = 0.01,
        exp_mult: float = 0.001,
        load_from_file: Optional[str] = None,
        *,
        foreach: Optional[bool] = False,
        hf_key: Optional[str] = "btherien/mulo",
        network: Optional[MetaMLP] = None,
        capturable: bool = False,
    ):
        if not torch.cuda.is_available():
            raise RuntimeError("AdafacLO_CUDA requires a GPU (torch.cuda.is_available() is False).")
        self.capturable = bool(capturable)
        _lib.load()
        if isinstance(momentum_dtype, str):
            momentum_dtype = {"float16": torch.float16, "bfloat16": torch.bfloat16,
                              "float32": torch.float32}[momentum_dtype]
        if momentum_dtype != torch.float32:
            raise NotImplementedError("the fused step keeps momentum in float32")
        if foreach:
            raise NotImplementedError("foreach=True is not implemented (neither is it in the reference)")
        defaults = dict(lr=lr, min_dim_size_to_factor=min_dim_size_to_factor, decay_rate=decay_rate,
                        decay_offset=decay_offset, beta2_cap=beta2_cap, momentum_dtype=momentum_dtype, eps=eps,
                        weight_decay=weight_decay, clipping_threshold=clipping_threshold,
                        max_grad_norm=max_grad_norm, unscaled_wd=unscaled_wd, foreach=foreach)
        super().__init__(params, defaults)
        first = next(p for g in self.param_groups for p in g["params"])
        self.device = first.device if first.is_cuda else torch.device("cuda", torch.cuda.current_device())
        self.metamlp = (network if network is not None else MetaMLP.from_pretrained(hf_key)).to(self.device)
        if load_from_file:
            loaded = torch.load(load_from_file, map_location=self.device, weights_only=True)
            self.metamlp.load_state_dict(loaded["state_dict"])
            momentum_decays = loaded["decays"]["momentum_decays"]
            rms_decays = loaded["decays"]["rms_decays"]
            adafactor_decays = loaded["decays"]["adafactor_decays"]
        for prm in self.metamlp.parameters():
            prm.requires_grad = False
        self.beta_m = _decays(initial_momentum_decays, momentum_decays, self.device)
        self.beta_rms = _decays(initial_rms_decays, rms_decays, self.device)
        self.beta_adafactor = _decays(initial_adafactor_decays, adafactor_decays, self.device)
        self.step_mult = step_mult
        self.exp_mult = exp_mult
        self._net = pack_metamlp(self.metamlp).to(self.device)
        self._decays = _lib.make_decays(self.beta_m.tolist(), float(self.beta_rms[0]),
                                        self.beta_adafactor.tolist())
        self._plan = None
        self._plan_key = None

    def _init_state(self, state, p):
        """pylo/optim/AdafacLO_cuda.py:227-256"""
        shape = tuple(p.shape)
        state["step"] = torch.tensor(0.0, dtype=torch.float64)
        fd = _factored_dims(shape)
        if fd is not None:
            dc, dr = fd
            r_shape, c_shape = list(shape), list(shape)
            r_shape[dr] = 1
            c_shape[dc] = 1
            state["exp_avg_sq_r"] = torch.zeros([3] + r_shape, device=self.device)
            state["exp_avg_sq_c"] = torch.zeros([3] + c_shape, device=self.device)
        else:
            state["exp_avg_sq_r"] = torch.zeros((3,) + shape, device=self.device)
            state["exp_avg_sq_c"] = state["exp_avg_sq_r"]      # the reference keeps two identical copies
        state["exp_avg_sq"] = torch.zeros(shape, device=self.device)
        state["exp_avg"] = torch.zeros((3,) + shape, device=self.device)

    def _ensure_plan(self, tensors):
        flags = self._PLAN_FLAGS | self._norm_flags()
        key = (flags,) + tuple((tuple(p.shape), p.dtype) for _, p in tensors)
        if key == self._plan_key:
            return
        for _, p in tensors:
            if not p.is_cuda or p.device != self.device or not p.is_contiguous():
                raise TypeError("AdafacLO_CUDA: parameters must be contiguous tensors on the optimizer's GPU")
        if self._plan is not None:
            self._plan.close()
        # parameters and gradients may be float16 / bfloat16 / float64 (the reference's kernels dispatch on the
        # element type, learned_optimizer.cu:338,364); the accumulators stay float32
        self._plan = _lib.Plan(_lib.KIND_ADAFAC, [tuple(p.shape) for _, p in tensors],
                               [flags | _lib.store_flag(p, "AdafacLO_CUDA") for _, p in tensors], self.device)
        self._plan_key = key
        if self.capturable:
            self._reset_device_steps(tensors)

    # ------------------------------------------------------------------ device-side step counters
    def _reset_device_steps(self, tensors):
        values = [int(self.state[p]["step"]) if "step" in self.state[p] else 0 for _, p in tensors]
        if self._dev_steps is None or self._dev_steps.numel() != len(tensors):
            self._dev_steps = torch.zeros(len(tensors), dtype=torch.int32, device=self.device)
        self._dev_steps.copy_(torch.tensor(values, dtype=torch.int32))   # in place: graphs keep the pointer
        self._plan.device_steps(self._dev_steps)
        self._plan.pinned_table(0)        # handed out now, not while a capture is open

    def sync_step_counters(self):
        """capturable mode: read the device counters back into ``state[p]["step"]`` (waits for the GPU)."""
        if self.capturable and self._dev_steps is not None and self._plan is not None:
            values = self._dev_steps.tolist()
            tensors = [(g, p) for g in self.param_groups for p in g["params"]]
            for (_, p), v in zip(tensors, values):
                if "step" in self.state[p]:
                    self.state[p]["step"] = torch.tensor(float(v), dtype=torch.float64)

    def refresh_graph_tables(self):
        """capturable mode: copy the groups' learning rates and weight decays into the pinned table
        that a recorded ``step()`` reads, e.g. after a scheduler step.  Call it while no replay is in
        flight."""
        if not self.capturable or self._plan is None:
            return
        table = self._plan.pinned_table(0)
        for i, (group, _p) in enumerate((g, p) for g in self.param_groups for p in g["params"]):
            for k, v in self._scalars(group).items():
                table[k][i] = v

    def state_dict(self):
        self.sync_step_counters()
        return super().state_dict()

    def load_state_dict(self, state_dict):
        out = super().load_state_dict(state_dict)
        if self.capturable and self._plan is not None:
            self._reset_device_steps([(g, p) for g in self.param_groups for p in g["params"]])
        return out

    def _norm_flags(self):
        """``max_grad_norm`` bounds every parameter's own gradient norm (AdafacLO_naive.py:199-200 and
        AdafacLO_cuda.py:214-215 call ``torch.nn.utils.clip_grad_norm_`` per parameter): the fused step takes the
        norms from its statistics pass and scales the gradients as it reads them (PYLO_F_TENSOR_NORM), so nothing
        is launched per parameter.  Unlike the reference, ``p.grad`` itself is left as it was."""
        on = any(g["max_grad_norm"] is not None for g in self.param_groups)
        return _lib.F_TENSOR_NORM if on else 0

    def _scalars(self, group):
        """Per-tensor scalar columns of the argument table."""
        mx = group["max_grad_norm"]
        return dict(lr=group["lr"], weight_decay=group["weight_decay"], exp_mult=self.exp_mult,
                    step_mult=self.step_mult, clip_norm=0.0 if mx is None else float(mx))

    @torch.no_grad()
    def step(self, loss=None):
        tensors = [(g, p) for g in self.param_groups for p in g["params"]]
        self._ensure_plan(tensors)
        plan = self._plan
        n = len(tensors)
        keys = ("grad", "param", "mom", "rms", "fac_r", "fac_c", "fac_v")
        cols = {k: [0] * n for k in keys}
        fl = {k: [0.0] * n for k in ("lr", "weight_decay", "exp_mult", "step_mult", "clip_norm", "clip_val", "bc1")}
        keep = []
        step_fed = None
        for i, (group, p) in enumerate(tensors):
            g = p.grad
            if g is None:
                continue
            if g.is_sparse:
                raise RuntimeError("Sparse gradients not supported")
            if g.dtype != p.dtype:
                raise TypeError("AdafacLO_CUDA: a gradient must have its parameter's dtype")
            if not g.is_contiguous():
                g = g.contiguous()
                keep.append(g)
            state = self.state[p]
            if len(state) == 0:
                self._init_state(state, p)
            if not self.capturable:     # else counted on the device
                state["step"] += 1
            # the time features take each parameter's own counter (pylo/optim/AdafacLO_cuda.py:304-305,400):
            # one that sat steps out lags behind the others
            s0 = float(state["step"]) - 1.0 if not self.capturable else 0.0
            fl["bc1"][i] = s0
            if step_fed is None:
                step_fed = s0
            elif step_fed != s0:
                step_fed = -1.0      # counters differ: the library reads them per tensor
            cols["grad"][i], cols["param"][i] = g.data_ptr(), p.data_ptr()
            cols["mom"][i], cols["rms"][i] = state["exp_avg"].data_ptr(), state["exp_avg_sq"].data_ptr()
            if _factored_dims(tuple(p.shape)) is None:
                cols["fac_v"][i] = state["exp_avg_sq_r"].data_ptr()
            else:
                cols["fac_r"][i] = state["exp_avg_sq_r"].data_ptr()
                cols["fac_c"][i] = state["exp_avg_sq_c"].data_ptr()
            for k, v in self._scalars(group).items():
                fl[k][i] = v
        if step_fed is None:
            return loss
        args = plan.args
        for k, v in cols.items():
            args[k] = v
        for k, v in fl.items():
            args[k] = v
        table = None
        if self.capturable and torch.cuda.is_current_stream_capturing():
            # the recorded call reads the plan's pinned table in place on every replay
            table = plan.pinned_table(0)
            table[:] = args
        with torch.cuda.device(self.device):
            plan.adafac_step(self._decays, self._net, step_fed, torch.cuda.current_stream(self.device).cuda_stream,
                             args=table)
        del keep
        return loss
