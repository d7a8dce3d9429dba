"""ELO_CELO2_CUDA on MI355X: the reference's ELO-CELO2 optimizer with its per-tensor Python
loop and CUDA extension replaced by one multi-tensor HIP step.

Drop-in for pylo/optim/ELO_CELO2_cuda.py:39-298: same constructor, ``step()``,
``param_groups`` keys and per-parameter state (``mom (3,*s)``, ``rms (*s)``, ``fac_r``,
``fac_c``).  What differs is *where* the work happens: gradient clipping, every
accumulator update, the 1-D AdamW branch and the feature/MLP pass of all tensors run in one
call into ``libpylo_mi355.so`` (seven launches); a second call orthogonalises the steps of all
matrices (Newton-Schulz as matrix-pipe products of the library's own; the slices of a tensor with more
than two dims each in LDS), normalises them and updates the parameters.  Arithmetic follows the
reference's naive class (pylo/optim/ELO_CELO2_naive.py:126-306), also where the reference's CUDA class
differs or fails: tensors with more than two dims normalise features and steps per slice of the last two
dims, and ``use_adamw_for_1d=False`` sends 1-D tensors through the MLP with a per-element accumulator
(state ``fac_v (3,*s)``).
"""

from __future__ import annotations

from typing import Optional

import os

import numpy as np
import torch
from torch.optim import Optimizer

from .. import _lib
from ..models import CELO2MLP, pack_celo2

_IN, _HID = 30, 8


def newton_schulz(x: torch.Tensor, coeffs, iters: int, eps: float) -> torch.Tensor:
    """Quintic Newton-Schulz over the last two dims (pylo/optim/CELO2_naive.py:59-73).  A leading
    batch dim runs as strided-batched library GEMMs with the scalings folded into them.  The reference
    transposes tall matrices so that the Gram matrix is the small one; the same products are taken
    here on the untransposed matrix (A = X^T X, X <- c0 X + X B), which keeps the result contiguous."""
    if x.dim() > 3:     # more leading dims: one batch of matrices
        return newton_schulz(x.reshape((-1,) + tuple(x.shape[-2:])), coeffs, iters, eps).reshape(x.shape)
    tall = x.shape[-2] > x.shape[-1]
    if x.dim() == 3 and x.is_cuda:
        # Frobenius norms through the multi-tensor kernels: a reduction to one value per matrix runs on a
        # handful of blocks (0.27 ms for a 50257 x 768 matrix), the multi-tensor one on all of them
        norm = torch.stack(torch._foreach_norm(list(x.unbind(0)))).view(-1, 1, 1)
    else:
        norm = torch.linalg.norm(x, dim=(-2, -1), keepdim=True)
    x = x / (norm + eps)
    c0, c1, c2 = coeffs
    if x.dim() == 3:
        split = _gram_split(x.shape[-2] if tall else x.shape[-1], min(x.shape[-2:]), x.shape[0])
        eye_c1 = torch.eye(min(x.shape[-2:]), device=x.device, dtype=x.dtype) * c1
        for _ in range(iters):
            xt = x.transpose(-2, -1)
            if split > 1 and tall:
                # Gram matrix of a very tall matrix (an embedding: 50257 x 768): one GEMM with a 768 x 768
                # output and a reduction 50257 long leaves most of the GPU idle; the rows are cut into
                # `split` slabs whose Gram matrices are one batched GEMM, added up afterwards
                xs = x.reshape(x.shape[0] * split, x.shape[1] // split, x.shape[2])
                a = torch.bmm(xs.transpose(-2, -1), xs).view(x.shape[0], split, x.shape[2], x.shape[2]).sum(1)
            else:
                a = torch.bmm(xt, x) if tall else torch.bmm(x, xt)
            # c1 A + c2 A A = (c2 A + c1 I) A and c0 X + B X = (B + c0 I) X: the scalings ride on the
            # diagonals of the small matrices, so every product is a plain GEMM (a GEMM that accumulates
            # into c0 X first copies X, half a gigabyte per iteration on this parameter set)
            a2 = torch.add(eye_c1, a, alpha=c2)      # c2 A + c1 I in one pass
            b = torch.bmm(a2, a)
            b.diagonal(dim1=-2, dim2=-1).add_(c0)
            x = torch.bmm(x, b) if tall else torch.bmm(b, x)
        return x
    for _ in range(iters):
        xt = x.transpose(-2, -1)
        a = xt @ x if tall else x @ xt
        b = c1 * a + c2 * (a @ a)
        x = c0 * x + (x @ b if tall else b @ x)
    return x


class _ns_blas:
    """The torch path of Newton-Schulz (shapes the library's own kernels do not take) with torch's BLAS choice
    left alone.  ``PYLO_MI355_NS_BLAS=rocblas`` in the environment opts in to rocBLAS for the duration of the
    block (on 768 .. 3072 wide matrices in batches of 12 its fp32 kernels run at 122 TFLOP/s where hipBLASLt's
    choices give 110); that switch is process-wide in torch, so it is never made unasked."""

    def __enter__(self):
        self.prev = None
        if os.environ.get("PYLO_MI355_NS_BLAS", "default") == "rocblas":
            self.prev = torch.backends.cuda.preferred_blas_library()
            torch.backends.cuda.preferred_blas_library("cublas")      # torch's name for rocBLAS
        return self

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.backends.cuda.preferred_blas_library(self.prev)
        return False


def _gram_split(k: int, small: int, batch: int) -> int:
    """Number of slabs to cut a reduction of length k into for the Gram product of `batch` matrices whose
    other dim is `small`: 1 unless the reduction is long against the output and the batch is too small to
    fill the GPU by itself; else the largest divisor of k up to 64 that leaves slabs of 512 or more."""
    if batch * small * small >= 8 * 1024 * 1024 or k < 16 * small or k < 8192:
        return 1
    for s in range(64, 1, -1):
        if k % s == 0 and k // s >= 512:
            return s
    return 1


_WATCH_ALL = 512   # parameter lists up to this length have every state tensor checked for replacement each step


class ELO_CELO2_CUDA(Optimizer):
    """Inference-time ELO-CELO2: CELO2 MLP steps for >=2-D tensors, shared-accumulator AdamW for
    1-D tensors and ``is_embedding`` groups."""

    _ADAM_FLAG = _lib.F_ADAM

    def __init__(
        self,
        params,
        lr=1e-3,
        weight_decay=0.1,
        clip_grad=True,
        clip_norm=1.0,
        adam_lr_mult=20.0,
        adam_weight_decay=None,
        use_adamw_for_1d=True,
        orthogonalize=True,
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
        hf_key: Optional[str] = "DiamondXL/elo-celo2",
        checkpoint_path: Optional[str] = None,
        network: Optional[CELO2MLP] = None,
        capturable: bool = False,
    ):
        if not torch.cuda.is_available():
            raise RuntimeError("ELO_CELO2_CUDA requires a GPU (torch.cuda.is_available() is False).")
        # capturable: step counters live on the device and ``step()`` can be recorded into a HIP graph
        # (torch.cuda.graph) and replayed; ``group["step"]`` is then refreshed by ``state_dict()`` /
        # ``sync_step_counters()`` only.  The reference has no such mode.
        self.capturable = bool(capturable)
        self._dev_steps = None
        _lib.load()
        defaults = dict(
            lr=lr, weight_decay=weight_decay, adam_lr_mult=adam_lr_mult,
            adam_weight_decay=weight_decay if adam_weight_decay is None else adam_weight_decay,
            use_adamw_for_1d=use_adamw_for_1d, orthogonalize=orthogonalize, clip_grad=clip_grad,
            clip_norm=clip_norm, exp_mult=exp_mult, rmsmult=rmsmult,
            param_scale_mult=param_scale_mult, grad_clip_val=grad_clip_val, is_embedding=False)
        super().__init__(params, defaults)
        first = next(p for g in self.param_groups for p in g["params"])
        self.device = first.device if first.is_cuda else torch.device("cuda", torch.cuda.current_device())

        def decays(v):
            return torch.clamp(torch.tensor(v, dtype=torch.float32, device=self.device), 0.0, 1.0)

        self.beta_m, self.beta_rms, self.beta_fac = (decays(initial_momentum_decays),
                                                      decays(initial_rms_decays),
                                                      decays(initial_adafactor_decays))
        self.n_mom, self.n_rms, self.n_fac = (self.beta_m.numel(), self.beta_rms.numel(),
                                              self.beta_fac.numel())
        if (self.n_mom, self.n_fac) != (3, 3) or self.n_rms < 1:
            raise ValueError("the fused step supports 3 momentum decays, 3 adafactor decays and >=1 rms decay")
        self.ns_coeffs = tuple(float(c) for c in ns_coeffs)
        self.ns_iters, self.ns_eps = ns_iters, ns_eps

        if network is None:
            if checkpoint_path is not None:
                network = CELO2MLP(hidden_size=ff_hidden_size, hidden_layers=ff_hidden_layers)
                network.load_state_dict(torch.load(checkpoint_path, map_location="cpu"))
            elif hf_key is not None:
                network = CELO2MLP.from_pretrained(hf_key)
            else:
                network = CELO2MLP(hidden_size=ff_hidden_size, hidden_layers=ff_hidden_layers)
        self.network = network.to(self.device)
        if sum(self.network.feature_dims) != _IN:
            raise ValueError(f"ELO_CELO2_CUDA kernel expects feature_dims summing to {_IN}, "
                             f"got {sum(self.network.feature_dims)}.")
        if self.network.hidden_size != _HID or len(self.network.dense_w) != 2:
            raise ValueError("ELO_CELO2_CUDA kernel only supports ff_hidden_size=8, ff_hidden_layers=2.")
        if self.network.activation != "relu" or self.network.output_size != 3:
            raise ValueError("ELO_CELO2_CUDA kernel only supports relu activation and output_size=3.")
        self._mlp = pack_celo2(self.network).to(self.device)
        bm, bf = self.beta_m.tolist(), self.beta_fac.tolist()
        self._decays = _lib.make_decays(bm, float(self.beta_rms[-1]), bf)
        # host copies: reading an element of a device tensor synchronises with the GPU
        self._adam_b1, self._adam_b2 = float(bm[0]), float(self.beta_rms[-1])
        self._plan = None
        self._plan_key = None
        self._fast_taken = False
        self._fin_fast = None
        self._lib_ns = os.environ.get("PYLO_MI355_NS", "lib") != "torch"

    # ------------------------------------------------------------------ plan
    def _tensors(self):
        out = []
        for group in self.param_groups:
            for p in group["params"]:
                # ELO_CELO2_naive.py:291-292: AdamW for tensors with fewer than two dims and for
                # is_embedding groups, unless the group turns that off
                adam = (p.dim() <= 1 or group["is_embedding"]) and group["use_adamw_for_1d"]
                out.append((group, p, adam))
        return out

    def _ensure_plan(self, tensors):
        # the plan reserves Newton-Schulz workspace (12 bytes per element) only for the tensors whose group
        # orthogonalises through the library
        no_ns = [not (group["orthogonalize"] and self._lib_ns and self.ns_iters > 0) for group, _p, _a in tensors]
        key = tuple((tuple(p.shape), adam, p.dtype, skip) for (_, p, adam), skip in zip(tensors, no_ns))
        if key == self._plan_key:
            return
        for _, p, _a in tensors:
            if not p.is_cuda or p.device != self.device:
                raise RuntimeError("ELO_CELO2_CUDA: every parameter must live on the optimizer's GPU")
            if not p.is_contiguous():
                raise TypeError("ELO_CELO2_CUDA: parameters must be contiguous tensors")
        if self._plan is not None:
            self._plan.close()
        shapes = [tuple(p.shape) for _, p, _a in tensors]
        # parameters and gradients may be float16 / bfloat16 / float64 (the reference's kernel dispatches on the
        # element type, celo2_kernel.cu:314,328); accumulators and raw steps stay float32 (ELO_CELO2_cuda.py:167-177)
        flags = [(self._ADAM_FLAG if adam else 0) | _lib.store_flag(p, type(self).__name__) |
                 (_lib.F_NO_ORTHOGONALIZE if skip else 0) for (_, p, adam), skip in zip(tensors, no_ns)]
        self._plan = _lib.Plan(_lib.KIND_CELO2, shapes, flags, self.device)
        self._plan_key = key
        # Raw steps of the MLP tensors: tensors of one parameter group and one shape share a
        # contiguous (count, *shape) buffer (what the torch products of Newton-Schulz run batched over).
        buckets = {}
        for i, (group, p, adam) in enumerate(tensors):
            if not adam:
                buckets.setdefault((id(group), tuple(p.shape)), []).append(i)
        self._raw = [None] * len(tensors)
        self._raw_groups = []
        for (_gid, shape), idx in buckets.items():
            buf = torch.empty((len(idx),) + shape, dtype=torch.float32, device=self.device)
            for j, i in enumerate(idx):
                self._raw[i] = buf[j]
            self._raw_groups.append((buf, idx))
        self._fin_args = np.zeros(len(tensors), dtype=_lib.ARGS_DTYPE)
        self._fin_fast = None
        # 0: torch products; 1: the library's tiled products (ns_iters > 0); 2: its per-slice launches (any ns_iters)
        self._ns_ok = [self._plan.orthogonalize_supported(i) for i in range(len(tensors))]
        if self.capturable:
            self._reset_device_steps(tensors)

    # ------------------------------------------------------------------ device-side step counters
    def _step_values(self, tensors):
        return [g.get("step", 0) for g, _p, _a in tensors]

    def _step_betas(self):
        return self._adam_b1, self._adam_b2

    def _store_step_values(self, tensors, values):
        for (g, _p, _a), v in zip(tensors, values):
            g["step"] = v

    def _reset_device_steps(self, tensors):
        values = torch.tensor(self._step_values(tensors), dtype=torch.int32)
        if self._dev_steps is None or self._dev_steps.numel() != len(tensors):
            self._dev_steps = torch.zeros(len(tensors), dtype=torch.int32, device=self.device)
        self._dev_steps.copy_(values)       # in place: a recorded graph keeps pointing at this tensor
        beta1, beta2 = self._step_betas()
        self._plan.device_steps(self._dev_steps, beta1, beta2)
        self._plan.pinned_table(0), self._plan.pinned_table(1)   # handed out now, not while a capture is open

    def sync_step_counters(self):
        """capturable mode: read the device counters back into ``group["step"]`` (waits for the GPU)."""
        if self.capturable and self._dev_steps is not None and self._plan is not None:
            self._store_step_values(self._tensors(), self._dev_steps.tolist())

    def state_dict(self):
        self.sync_step_counters()
        return super().state_dict()

    def refresh_graph_tables(self):
        """capturable mode: copy the groups' learning rates and weight decays into the pinned tables
        that a recorded ``step()`` reads, e.g. after a scheduler step.  Call it while no replay is in
        flight.  Tensors that the recorded step finishes with torch operations (more than two dims)
        keep the values they were recorded with."""
        if not self.capturable or self._plan is None:
            return
        step_tab, fin_tab = self._plan.pinned_table(0), self._plan.pinned_table(1)
        for i, (group, _p, adam) in enumerate(self._tensors()):
            if adam:
                step_tab["lr"][i] = group["adam_lr_mult"] * group["lr"]
                step_tab["weight_decay"][i] = group["adam_weight_decay"]
            elif fin_tab["grad"][i]:
                fin_tab["lr"][i], fin_tab["weight_decay"][i] = group["lr"], group["weight_decay"]
                fin_tab["step_mult"][i] = group["rmsmult"]

    def _capturing(self):
        return self.capturable and torch.cuda.is_current_stream_capturing()

    def _launch_step(self):
        plan = self._plan
        table = None
        if self._capturing():
            # the recorded call reads the plan's pinned table in place on every replay
            table = plan.pinned_table(0)
            table[:] = plan.args
        with torch.cuda.device(self.device):
            plan.celo2_step(self._decays, self._mlp, torch.cuda.current_stream(self.device).cuda_stream, args=table)

    def _init_state(self, state, p, adam):
        shape = tuple(p.shape)
        state["mom"] = torch.zeros((self.n_mom,) + shape, device=self.device)
        state["rms"] = torch.zeros(shape, device=self.device)
        if p.dim() >= 2:
            dc, dr = _factored_dims_host(shape)
            r_shape, c_shape = list(shape), list(shape)
            r_shape[dr] = 1
            c_shape[dc] = 1
            state["fac_r"] = torch.zeros([self.n_fac] + r_shape, device=self.device)
            state["fac_c"] = torch.zeros([self.n_fac] + c_shape, device=self.device)
        elif not adam:   # the MLP on a tensor with fewer than two dims: per-element Adafactor accumulator
            state["fac_v"] = torch.zeros((self.n_fac,) + shape, device=self.device)

    # ------------------------------------------------------------------ step
    @torch.no_grad()
    def step(self, loss=None):
        tensors = self.fused_step()
        self.finish_step(tensors)
        return loss

    # The argument table of the library call has one row per tensor.  Building it costs ~20 us of
    # Python per tensor; after a step in which every tensor had a dense contiguous fp32 gradient the
    # static columns (state pointers, output slices) are kept and only gradients, parameter pointers and
    # the per-group scalars are refreshed, which keeps the host ahead of a ~1.7 ms GPU step.
    def load_state_dict(self, state_dict):
        self._fast = None
        out = super().load_state_dict(state_dict)
        if self.capturable and self._plan is not None:
            self._reset_device_steps(self._tensors())
        return out

    def add_param_group(self, param_group):
        self._fast = None
        return super().add_param_group(param_group)

    # AdamW branch: which two moment buffers a tensor uses and its bias corrections this step
    def _adam_row(self, group, state):
        t = group.get("step", 0)
        return (state["mom"].data_ptr(), state["rms"].data_ptr(), 1.0 - self._adam_b1 ** t,
                1.0 - self._adam_b2 ** t)

    def _adam_corrections_fast(self, fast, per_group):
        beta1, beta2 = self._adam_b1, self._adam_b2
        adam = fast["adam"]
        return (np.where(adam, per_group(lambda g: 1.0 - beta1 ** g["step"]), 0.0),
                np.where(adam, per_group(lambda g: 1.0 - beta2 ** g["step"]), 0.0))

    def _fused_step_fast(self, fast):
        grads = [p.grad for p in fast["params"]]
        for g in grads:     # a dense gradient has its parameter's dtype (torch enforces it on assignment)
            if g is None or g.layout is not torch.strided or not g.is_contiguous():
                return None
        groups = self.param_groups
        if len(groups) != fast["n_groups"] or len(self.state) != fast["n_state"]:
            return None
        for st, key, t in fast["alive"]:
            if st.get(key) is not t:      # a state tensor was replaced: the cached pointers are stale
                return None
        if fast["routing"] != [(g["use_adamw_for_1d"], g["is_embedding"]) for g in groups]:
            return None                   # a group changed which branch its tensors take: new plan
        if not self.capturable:
            for group in groups:
                group["step"] = group.get("step", 0) + 1
        gidx, adam = fast["gidx"], fast["adam"]

        def per_group(fn):
            return np.asarray([fn(g) for g in groups], dtype=np.float64)[gidx]

        args = self._plan.args
        args["grad"] = [g.data_ptr() for g in grads]
        args["param"] = [p.data_ptr() for p in fast["params"]]
        args["clip_norm"] = per_group(lambda g: g["clip_norm"] if g["clip_grad"] else 0.0)
        args["clip_val"] = per_group(lambda g: g["grad_clip_val"])
        args["exp_mult"] = per_group(lambda g: g["exp_mult"])
        args["lr"] = np.where(adam, per_group(lambda g: g["adam_lr_mult"] * g["lr"]), 0.0)
        args["weight_decay"] = np.where(adam, per_group(lambda g: g["adam_weight_decay"]), 0.0)
        if not self.capturable:     # else the library derives them from its device counters
            args["bc1"], args["bc2"] = self._adam_corrections_fast(fast, per_group)
        self._launch_step()
        self._fast_taken = True
        return fast["tensors"]

    @torch.no_grad()
    def fused_step(self):
        """Everything up to the raw per-element step: one call into the HIP library."""
        fast = getattr(self, "_fast", None)
        if fast is not None and self._plan is not None:
            done = self._fused_step_fast(fast)
            if done is not None:
                return done
            self._fast = None
        self._fast_taken = False
        tensors = self._tensors()
        self._ensure_plan(tensors)
        plan = self._plan
        if not self.capturable:
            for group in self.param_groups:
                group["step"] = group.get("step", 0) + 1
        n = len(tensors)
        cols = {k: [0] * n for k in ("grad", "param", "mom", "rms", "fac_r", "fac_c", "fac_v", "step_out")}
        fl = {k: [0.0] * n for k in ("lr", "weight_decay", "clip_norm", "clip_val", "exp_mult", "bc1", "bc2")}
        keep = []   # contiguous copies of non-contiguous grads must outlive the launch
        for i, (group, p, adam) in enumerate(tensors):
            g = p.grad
            if g is None:
                continue
            if g.is_sparse:
                raise RuntimeError("ELO_CELO2_CUDA does not support sparse gradients")
            if g.dtype != p.dtype:
                raise TypeError("ELO_CELO2_CUDA: a gradient must have its parameter's dtype")
            if not g.is_contiguous():
                g = g.contiguous()
                keep.append(g)
            state = self.state[p]
            if len(state) == 0:
                self._init_state(state, p, adam)
            cols["grad"][i], cols["param"][i] = g.data_ptr(), p.data_ptr()
            fl["clip_norm"][i] = group["clip_norm"] if group["clip_grad"] else 0.0
            fl["clip_val"][i] = group["grad_clip_val"]
            fl["exp_mult"][i] = group["exp_mult"]
            if adam:
                cols["mom"][i], cols["rms"][i], fl["bc1"][i], fl["bc2"][i] = self._adam_row(group, state)
                fl["lr"][i] = group["adam_lr_mult"] * group["lr"]
                fl["weight_decay"][i] = group["adam_weight_decay"]
            else:
                cols["mom"][i], cols["rms"][i] = state["mom"].data_ptr(), state["rms"].data_ptr()
                if p.dim() >= 2:
                    cols["fac_r"][i], cols["fac_c"][i] = state["fac_r"].data_ptr(), state["fac_c"].data_ptr()
                else:
                    cols["fac_v"][i] = state["fac_v"].data_ptr()
                cols["step_out"][i] = self._raw[i].data_ptr()
        args = plan.args
        for k, v in cols.items():
            args[k] = v
        for k, v in fl.items():
            args[k] = v
        self._launch_step()
        if not keep and all(p.grad is not None for _, p, _a in tensors):
            index = {id(g): i for i, g in enumerate(self.param_groups)}
            # the cached rows point into the state tensors: hold them, and notice a replaced or cleared one.
            # Every state tensor of every parameter is watched (a few hundred identity checks a step for a
            # transformer's parameter list); beyond _WATCH_ALL parameters only the first state tensor of each
            # is, because the walk then costs milliseconds a step: there, state tensors must be updated in place
            # or through load_state_dict().
            def watched(state):
                items = [(k, t) for k, t in state.items() if torch.is_tensor(t) and t.dim() > 0]
                return items if len(tensors) <= _WATCH_ALL else items[:1]
            alive = [(self.state[p], k, t) for _, p, _a in tensors for k, t in watched(self.state[p])]
            self._fast = dict(tensors=tensors, params=[p for _, p, _a in tensors], n_groups=len(self.param_groups),
                              n_state=len(self.state), alive=alive,
                              routing=[(g["use_adamw_for_1d"], g["is_embedding"]) for g in self.param_groups],
                              gidx=np.asarray([index[id(g)] for g, _p, _a in tensors], dtype=np.int64),
                              adam=np.asarray([a for _g, _p, a in tensors], dtype=bool))
        del keep
        return tensors

    @torch.no_grad()
    def finish_step(self, tensors):
        """Newton-Schulz, RMS normalisation and the parameter update of the MLP tensors
        (pylo/optim/ELO_CELO2_cuda.py:288-296).  Matrices are orthogonalised by the library's own matrix-pipe
        kernels inside the finishing call (fp32 accuracy on the fp16 matrix instructions, any two dims; with
        ``PYLO_MI355_NS_F32=1`` the fp32 matrix instructions, dims that are multiples of 4); tensors with more
        than two dims slice by slice of their last two dims, small slices in launches that hold a slice in
        registers or LDS, large ones as matrices of the same products.  Batched torch products remain for what the
        library leaves to the caller (zero iterations on a matrix, the fp32 instructions' other shapes) and for
        everything with ``PYLO_MI355_NS=torch`` in the environment, for comparisons."""
        self._finish_step(tensors)

    # The finishing call's table has one row per tensor as well.  When the step went through the cached rows of
    # the fused call (every tensor has a gradient) and the library finishes every MLP tensor itself (no
    # param_scale_mult, no torch products), its static columns are kept too and a step refreshes parameter pointers and the groups' scalars with a few array operations, whatever the
    # number of tensors.
    def _fin_fast_key(self):
        return (self.ns_iters, self._lib_ns,
                tuple((g["orthogonalize"], g["param_scale_mult"]) for g in self.param_groups))

    def _build_fin_fast(self, tensors):
        if any(g["param_scale_mult"] for g in self.param_groups):
            return None
        idx, flags = [], []
        for i, (group, p, adam) in enumerate(tensors):
            if adam:
                continue
            orth = bool(group["orthogonalize"]) and p.dim() >= 2
            # (zero iterations still divide by the Frobenius norm, which the normaliser's epsilon sees: the
            # per-slice launches do that, the tiled products leave it to torch)
            if orth and not (self._lib_ns and (self._ns_ok[i] == 2 or (self._ns_ok[i] == 1 and self.ns_iters > 0))):
                return None
            idx.append(i)
            flags.append(_lib.ARG_ORTHOGONALIZE if orth else 0)
        if not idx:
            return None
        idx = np.asarray(idx, dtype=np.int64)
        fin = self._fin_args
        fin[:] = 0
        fin["grad"][idx] = 1          # "takes part"; the gradient itself is not read
        fin["step_out"][idx] = [self._raw[i].data_ptr() for i in idx]
        fin["flags"][idx] = flags
        return dict(key=self._fin_fast_key(), idx=idx, gidx=self._fast["gidx"][idx])

    def _finish_step_fast(self, ff):
        groups = self.param_groups
        fin, idx, gidx = self._fin_args, ff["idx"], ff["gidx"]
        fin["param"][idx] = self._plan.args["param"][idx]
        fin["lr"][idx] = np.asarray([g["lr"] for g in groups], dtype=np.float64)[gidx]
        fin["weight_decay"][idx] = np.asarray([g["weight_decay"] for g in groups], dtype=np.float64)[gidx]
        fin["step_mult"][idx] = np.asarray([g["rmsmult"] for g in groups], dtype=np.float64)[gidx]
        if self._capturing():
            table = self._plan.pinned_table(1)
            table[:] = fin
            fin = table
        with torch.cuda.device(self.device):
            self._plan.celo2_orthogonalize_finish(fin, self.ns_coeffs, self.ns_iters, self.ns_eps,
                                                  torch.cuda.current_stream(self.device).cuda_stream)

    def _finish_step(self, tensors):
        if getattr(self, "_fast", None) is not None and self._fast_taken:
            ff = getattr(self, "_fin_fast", None)
            if ff is None or ff["key"] != self._fin_fast_key():
                ff = self._fin_fast = self._build_fin_fast(tensors) or dict(key=self._fin_fast_key(), idx=None)
            if ff["idx"] is not None:
                return self._finish_step_fast(ff)
        self._fin_fast = None      # the general path below rewrites the table
        fin = self._fin_args
        fin["grad"] = 0
        fin["flags"] = 0
        lib_ns = self._lib_ns
        keep, any_fin = [], False   # post-Newton-Schulz matrices must outlive the launch
        for buf, idx in self._raw_groups:
            group = tensors[idx[0]][0]
            ps = [tensors[i][1] for i in idx]
            # a tensor that sits this step out keeps its row out of the table (its raw step is stale or unset; the
            # bucket-wide torch operations below run over it and nobody reads the result)
            present = [p.grad is not None for p in ps]
            if not any(present):
                continue
            step = buf
            nd = buf.dim() - 1
            if group["param_scale_mult"]:
                n = ps[0].numel()
                sq = torch.stack(torch._foreach_norm([p.float() for p in ps] if ps[0].dtype != torch.float32 else ps)) ** 2 / n
                step = step.mul_(torch.sqrt(sq + 1e-9).view([-1] + [1] * nd))   # the raw steps are scratch
            flag = 0
            # more than two dims: Newton-Schulz and the normaliser are per slice of the last two dims
            # (ELO_CELO2_naive.py:217-218,235), in the library too
            if group["orthogonalize"] and nd >= 2:
                ok = min(self._ns_ok[i] for i in idx)
                if lib_ns and (ok == 2 or (ok == 1 and self.ns_iters > 0)):
                    flag = _lib.ARG_ORTHOGONALIZE
                else:
                    with _ns_blas():
                        step = newton_schulz(step, self.ns_coeffs, self.ns_iters, self.ns_eps)
            step = step.contiguous()
            keep.append(step)
            base, stride = step.data_ptr(), step[0].numel() * 4
            for j, i in enumerate(idx):
                if not present[j]:
                    continue
                fin["grad"][i] = 1          # "takes part"; the gradient itself is not read
                fin["param"][i] = ps[j].data_ptr()
                fin["step_out"][i] = base + j * stride
                fin["lr"][i] = group["lr"]
                fin["weight_decay"][i] = group["weight_decay"]
                fin["step_mult"][i] = group["rmsmult"]
                fin["flags"][i] = flag
            any_fin = True
        if any_fin:
            if self._capturing():
                table = self._plan.pinned_table(1)
                table[:] = fin
                fin = table
            with torch.cuda.device(self.device):
                self._plan.celo2_orthogonalize_finish(fin, self.ns_coeffs, self.ns_iters, self.ns_eps,
                                                      torch.cuda.current_stream(self.device).cuda_stream)
        del keep


def _factored_dims_host(shape):
    """(dc, dr) as pylo/optim/CELO2_naive.py:42-47: 2nd-largest and largest dim, ties by index."""
    order = sorted(range(len(shape)), key=lambda i: (shape[i], i))
    return order[-2], order[-1]
