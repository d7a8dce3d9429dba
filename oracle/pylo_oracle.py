"""CPU (torch fp32) restatement of the reference's *naive* learned-optimizer steps.

TEST INFRASTRUCTURE ONLY -- imported by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``; never by the product package.

The reference ships two implementations of every optimizer: ``*_naive`` (pure
PyTorch, runs on CPU) and ``*_CUDA`` (needs its CUDA extension).  They disagree in
a few corners (1-D epsilons, a reduction axis in AdafacLO_cuda.py:342-343, N-D
indexing, ``param_scale_mult``); this file follows the **naive** classes, which
are the only ones that can run without CUDA, and keeps optimizer state in the
**CUDA classes' layout** (decay axis leading) so it can be compared entry by
entry with what the HIP path leaves in ``optimizer.state``.

Pins (see tests/test_oracle_*.py): golden trajectories written from the
reference's naive classes (tests/golden/), closed forms of the EMAs from zero
state, ``torch.optim.AdamW`` for the 1-D branch, ``torch.nn.LSTMCell`` with
permuted gates for the LSTM, fp64 brute force for Newton-Schulz and the feature
list, ``numpy.argsort`` for ``factored_dims``.

``AdafacOracle(per_param_step=True)`` restates the CUDA class's per-parameter step counter
(AdafacLO_cuda.py:304-305,400); the CUDA class cannot run here and the naive class counts per group, so
no golden trajectory covers a parameter that sat steps out.  The switch is pinned by a property instead
(tests/test_oracle_pins.py): AdafacLO tensors do not interact, so such a parameter must end bit-exactly
where a single-parameter run fed only the steps it took part in ends.  ``AdafacOracle(max_grad_norm=...)``
(norm clipping of every gradient by itself) is pinned by a golden trajectory of the naive class with that
argument (tests/golden/adafac_max_norm.npz).  Nothing here is unpinned.

Parameters stored as float16 / bfloat16 / float64 need no code of their own: the contract is the float32
step on the widened values with the result rounded into the storage type, so the tests feed these classes
widened inputs and round.  (Of the reference's naive classes, ELO_CELO2_naive and CELO2_naive raise a dtype
error on any parameter that is not float32 and all of them on float64; AdafacLO_naive, ELO_naive and
VeLO_naive run on 16-bit parameters with float32 accumulators and a few operations, g*g among them, in the
16-bit type.)

Every function cites the reference lines it restates.
"""

from __future__ import annotations

import math
import time
from typing import Dict, List, Optional, Sequence, Tuple

import torch

F32 = torch.float32


# ----------------------------------------------------------------------------
# shared helpers
# ----------------------------------------------------------------------------
def factored_dims(shape: Sequence[int]) -> Optional[Tuple[int, int]]:
    """(dc, dr) = (index of 2nd-largest dim, index of largest dim); ties keep index order.

    pylo/optim/CELO2_naive.py:42-47, pylo/optim/AdafacLO_naive.py:95-99
    (``np.argsort`` on <=16 entries is an insertion sort, hence stable).
    """
    if len(shape) < 2:
        return None
    order = sorted(range(len(shape)), key=lambda i: (shape[i], i))
    return order[-2], order[-1]


def factored_dims_velo(shape: Sequence[int]) -> Optional[Tuple[int, int]]:
    """VeLO's variant: equal top-two dims are returned swapped, except 4-D (0, 1).

    pylo/optim/Velo_naive.py:85-95 (= pylo/optim/velo_cuda.py:121-131)
    """
    if len(shape) < 2:
        return None
    order = sorted(range(len(shape)), key=lambda i: (shape[i], i))
    a, b = order[-2], order[-1]
    if shape[a] == shape[b] and not (len(shape) == 4 and a == 0 and b == 1):
        return b, a
    return a, b


def safe_rsqrt(x: torch.Tensor) -> torch.Tensor:
    """pylo/optim/CELO2_naive.py:50-51"""
    return torch.rsqrt(torch.clamp(x, min=1e-9))


def rms_normalize(x: torch.Tensor, dims: Sequence[int], eps: float) -> torch.Tensor:
    """x * rsqrt(eps + mean(x^2) over dims).  pylo/optim/CELO2_naive.py:54-56 (eps 1e-9),
    pylo/optim/Velo_naive.py:80-82 and pylo/optim/AdafacLO_naive.py:90-92 (eps 1e-5)."""
    ms = torch.mean(x * x, dim=list(dims), keepdim=True)
    return x * torch.rsqrt(eps + ms)


def newton_schulz(x: torch.Tensor, coeffs=(3.4445, -4.7750, 2.0315), iters: int = 5,
                  eps: float = 1e-8) -> torch.Tensor:
    """Quintic Newton-Schulz orthogonalisation over the last two dims.

    pylo/optim/CELO2_naive.py:59-73
    """
    flip = x.shape[-2] > x.shape[-1]
    if flip:
        x = x.transpose(-2, -1)
    x = x / (torch.linalg.norm(x, dim=(-2, -1), keepdim=True) + eps)
    c0, c1, c2 = coeffs
    for _ in range(iters):
        a = x @ x.transpose(-2, -1)
        b = c1 * a + c2 * (a @ a)
        x = c0 * x + b @ x
    return x.transpose(-2, -1) if flip else x


def decay_from_offsets(initial: Sequence[float], offsets: Sequence[float]) -> torch.Tensor:
    """clip(1 - exp(10 * (log(1 - d0) / 10 + offset)), 0, 1) in fp32.

    pylo/optim/Velo_naive.py:98-103,246-260; pylo/optim/AdafacLO_naive.py:102-107,144-164
    """
    d0 = torch.tensor(list(initial), dtype=F32)
    off = torch.tensor(list(offsets), dtype=F32)
    par = torch.log(1 - d0) / 10.0 + off
    return torch.clip(1 - torch.exp(par * 10.0), 0.0, 1.0)


def _to_double(obj):
    """Recursively converts floating tensors held in dicts / lists / tuples to fp64."""
    if torch.is_tensor(obj):
        return obj.double() if obj.is_floating_point() else obj
    if isinstance(obj, dict):
        return {k: _to_double(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return type(obj)(_to_double(v) for v in obj)
    return obj


def _bview(beta: torch.Tensor, ndim: int) -> torch.Tensor:
    return beta.view([-1] + [1] * ndim)


def _ema_(acc: torch.Tensor, beta: torch.Tensor, new: torch.Tensor) -> None:
    """acc <- beta*acc + (1-beta)*new  (the naive classes' form, not ``lerp_``).

    pylo/optim/ELO_CELO2_naive.py:145,149; Velo_naive.py:419-420; AdafacLO_naive.py:239-240
    """
    acc.mul_(beta).add_((1 - beta) * new)


def _factored_update(state: Dict[str, torch.Tensor], g: torch.Tensor, beta: torch.Tensor,
                     dc: int, dr: int, key_r: str, key_c: str):
    """Adafactor row/col accumulators + row/col factors; returns (row_factor, col_factor).

    ``state[key_r]``: mean of g^2 over ``dr`` (shape (3,*s) with dr->1);
    ``state[key_c]``: mean over ``dc``.
    pylo/optim/ELO_CELO2_naive.py:152-166 (identical in Velo_naive.py:46-58 and
    AdafacLO_naive.py:54-68)
    """
    nd = g.dim()
    b = _bview(beta, nd)
    q = g * g + 1e-30
    state[key_r] = b * state[key_r] + (1 - b) * q.mean(dim=dr, keepdim=True)[None]
    state[key_c] = b * state[key_c] + (1 - b) * q.mean(dim=dc, keepdim=True)[None]
    return _row_col_factors(state[key_r], state[key_c], dc)


def _row_col_factors(fac_r: torch.Tensor, fac_c: torch.Tensor, dc: int):
    """row_factor = safe_rsqrt(fac_r / (mean over the dc axis + 1e-9)), col_factor = safe_rsqrt(fac_c).

    pylo/optim/ELO_CELO2_naive.py:161-164,210-213
    """
    row_col_mean = fac_r.mean(dim=dc + 1, keepdim=True)
    return safe_rsqrt(fac_r / (row_col_mean + 1e-9)), safe_rsqrt(fac_c)


# ----------------------------------------------------------------------------
# ELO-CELO2
# ----------------------------------------------------------------------------
CELO2_FEATURE_DIMS = (1, 1, 1, 3, 1, 3, 1, 3, 1, 3, 3, 3, 3, 3)  # pylo/models/CELO2_MLP.py:25


def celo2_mlp(groups: List[torch.Tensor], sd: Dict[str, torch.Tensor]) -> torch.Tensor:
    """Split-input MLP; ``groups[i]`` has shape (k_i, *shape); returns (*shape, 3).

    pylo/models/CELO2_MLP.py:100-123 (weights stored (in, out), ``x @ w``)
    """
    o = None
    for i, x in enumerate(groups):
        t = x.movedim(0, -1) @ sd[f"w0.{i}"]
        o = t if o is None else o + t
    o = torch.relu(o + sd["b0"])
    o = torch.relu(o @ sd["dense_w.0"] + sd["dense_b.0"])
    return o @ sd["dense_w.1"] + sd["dense_b.1"]


def celo2_feature_groups(p, g, mom, rms, fac_r, fac_c, row_factor, col_factor):
    """The 14 CELO2 feature groups (30 channels), decay axis leading, un-normalised.

    pylo/optim/ELO_CELO2_naive.py:180-215
    """
    rs = torch.rsqrt(rms + 1e-8)
    full = (3,) + tuple(p.shape)
    rowf = fac_r.expand(full)
    colf = fac_c.expand(full)
    return [
        g[None],
        torch.clamp(g, -0.1, 0.1)[None],
        p[None],
        mom,
        rms[None],
        mom * rs[None],
        rs[None],
        g[None] * row_factor * col_factor,
        (g * rs)[None],
        rowf,
        colf,
        torch.rsqrt(rowf + 1e-8),
        torch.rsqrt(colf + 1e-8),
        mom * row_factor * col_factor,
    ]


class EloCelo2Oracle:
    """ELO_CELO2_naive.step restated (pylo/optim/ELO_CELO2_naive.py:261-306).

    ``net`` is a CELO2MLP state_dict (keys w0.0..w0.13, b0, dense_w.0/1, dense_b.0/1).
    State per tensor: ``mom (3,*s)``, ``rms (*s)``, ``fac_r``, ``fac_c`` (>=2-D only) -- the
    layout of ELO_CELO2_cuda.py:165-177.
    """

    def __init__(self, params: List[torch.Tensor], net: Dict[str, torch.Tensor], lr=1e-3,
                 weight_decay=0.1, clip_grad=True, clip_norm=1.0, adam_lr_mult=1.0,
                 adam_weight_decay=None, use_adamw_for_1d=True, orthogonalize=True,
                 momentum_decays=(0.9, 0.99, 0.999), rms_decays=(0.95,),
                 adafactor_decays=(0.9, 0.99, 0.999), exp_mult=0.0, rmsmult=1.0,
                 param_scale_mult=False, ns_coeffs=(3.4445, -4.7750, 2.0315), ns_iters=5,
                 ns_eps=1e-8, grad_clip_val=1000.0, is_embedding: Sequence[bool] = (), device="cpu",
                 independent_adam=None):
        # independent_adam = (beta1, beta2, eps): the AdamW branch keeps its own exp_avg / exp_avg_sq /
        # adam_step per tensor as CELO2_naive does (pylo/optim/CELO2_naive.py:263-283) instead of
        # reading mom[0] / rms of the shared accumulators.
        self.independent_adam = independent_adam
        self.params = params
        self.device = torch.device(device)
        self.net = {k: v.detach().to(F32).to(self.device) for k, v in net.items()}
        self.h = dict(lr=lr, weight_decay=weight_decay, clip_grad=clip_grad, clip_norm=clip_norm,
                      adam_lr_mult=adam_lr_mult,
                      adam_weight_decay=weight_decay if adam_weight_decay is None else adam_weight_decay,
                      use_adamw_for_1d=use_adamw_for_1d, orthogonalize=orthogonalize,
                      exp_mult=exp_mult, rmsmult=rmsmult, param_scale_mult=param_scale_mult,
                      grad_clip_val=grad_clip_val)
        dv = self.device
        self.beta_m = torch.tensor(momentum_decays, dtype=F32, device=dv)
        self.beta_rms = torch.clamp(torch.tensor(rms_decays, dtype=F32, device=dv), 0.0, 1.0)
        self.beta_fac = torch.clamp(torch.tensor(adafactor_decays, dtype=F32, device=dv), 0.0, 1.0)
        self.ns = (tuple(float(c) for c in ns_coeffs), ns_iters, ns_eps)
        self.is_embedding = list(is_embedding) or [False] * len(params)
        self.t = 0
        self.finish_seconds = 0.0     # time spent in finish_step (NS / normalise / apply), for bench.py
        self.state: List[Dict[str, torch.Tensor]] = []
        for p in params:
            s = tuple(p.shape)
            st = {"mom": torch.zeros((3,) + s, device=dv), "rms": torch.zeros(s, device=dv)}
            fd = factored_dims(s)
            if fd is not None:
                dc, dr = fd
                rs_, cs_ = list(s), list(s)
                rs_[dr] = 1
                cs_[dc] = 1
                st["fac_r"] = torch.zeros([3] + rs_, device=dv)
                st["fac_c"] = torch.zeros([3] + cs_, device=dv)
            elif not use_adamw_for_1d:
                st["fac_v"] = torch.zeros((3,) + s, device=dv)     # ELO_CELO2_naive.py:254-256
            self.state.append(st)

    def double_(self):
        """Evaluate everything in fp64 from here on (the decays keep their fp32 values): the
        reference formulas without fp32 rounding, for checks at sizes where fp32 PyTorch reductions
        are themselves less accurate than the tolerance.  ``self.params`` must then be fp64 tensors."""
        self.net, self.state = _to_double(self.net), _to_double(self.state)
        self.beta_m, self.beta_rms, self.beta_fac = self.beta_m.double(), self.beta_rms.double(), self.beta_fac.double()
        return self

    def grad_scale(self, grads) -> float:
        """clip_norm / max(global_norm, clip_norm).  pylo/optim/ELO_CELO2_naive.py:126-135"""
        total = torch.zeros((), device=self.device)
        for g in grads:
            if g is not None:
                total = total + g.detach().float().pow(2).sum()
        denom = torch.clamp(torch.sqrt(total), min=self.h["clip_norm"])
        return (self.h["clip_norm"] / denom).item() if denom > 0 else 1.0

    def raw_step(self, i: int, p: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
        """Accumulator update + features + MLP: direction * exp(magnitude * exp_mult).

        This is what the reference's fused kernel writes to ``step_out``
        (pylo/csrc/celo2_kernel.cu:203-282); pylo/optim/ELO_CELO2_naive.py:173-229.
        """
        st = self.state[i]
        nd = p.dim()
        _ema_(st["mom"], _bview(self.beta_m, nd), g[None])
        _ema_(st["rms"], self.beta_rms[-1], g * g)
        fd = factored_dims(tuple(p.shape))
        if fd is not None:
            dc, dr = fd
            rf, cf = _factored_update(st, g, self.beta_fac, dc, dr, "fac_r", "fac_c")
            groups = celo2_feature_groups(p, g, st["mom"], st["rms"], st["fac_r"], st["fac_c"], rf, cf)
        else:
            # fewer than two dims on the MLP path (use_adamw_for_1d=False): the accumulator is per
            # element and only the first nine feature groups exist; the split first layer adds up
            # the groups it is given (ELO_CELO2_naive.py:166-169,180-191; CELO2_MLP.py:100-110)
            b = _bview(self.beta_fac, nd)
            st["fac_v"] = b * st["fac_v"] + (1 - b) * (g * g + 1e-30)[None]
            rs = torch.rsqrt(st["rms"] + 1e-8)
            groups = [g[None], torch.clamp(g, -0.1, 0.1)[None], p[None], st["mom"], st["rms"][None],
                      st["mom"] * rs[None], rs[None], g[None] * safe_rsqrt(st["fac_v"] + 1e-9), (g * rs)[None]]
        axes = [nd - 1, nd] if nd >= 2 else [nd]      # last two param dims (decay axis leads)
        groups = [rms_normalize(x, axes, 1e-9) for x in groups]
        out = celo2_mlp(groups, self.net)
        step = out[..., 0] * torch.exp(out[..., 1] * self.h["exp_mult"])
        if self.h["param_scale_mult"]:
            step = out[..., 0] * (torch.sqrt(torch.mean(p * p) + 1e-9)
                                  * torch.exp(out[..., 1] * self.h["exp_mult"]))
        return step

    def finish_step(self, p: torch.Tensor, step: torch.Tensor) -> None:
        """NS -> RMS-normalise over last two dims -> rmsmult -> p -= lr (step + wd p).

        pylo/optim/ELO_CELO2_naive.py:231-237,305
        """
        h = self.h
        nd = p.dim()
        if h["orthogonalize"] and step.dim() >= 2:
            step = newton_schulz(step, *self.ns)
        step = rms_normalize(step, list(range(nd))[-2:], 1e-9) * h["rmsmult"]
        p.add_(step + h["weight_decay"] * p, alpha=-h["lr"])

    @torch.no_grad()
    def step(self, grads: List[Optional[torch.Tensor]], keep_raw: Optional[dict] = None) -> None:
        h = self.h
        scale = self.grad_scale(grads) if h["clip_grad"] else 1.0
        self.t += 1
        t = self.t
        beta1 = float(self.beta_m[0])
        beta2 = float(self.beta_rms[-1])
        adam_lr = h["adam_lr_mult"] * h["lr"]
        for i, (p, g) in enumerate(zip(self.params, grads)):
            if g is None:
                continue
            if scale != 1.0:
                g = g * scale
            g = torch.clamp(g, -h["grad_clip_val"], h["grad_clip_val"])
            if h["use_adamw_for_1d"] and (p.dim() <= 1 or self.is_embedding[i]) and self.independent_adam:
                b1, b2, eps = self.independent_adam
                st = self.state[i]
                if "exp_avg" not in st:
                    st["exp_avg"], st["exp_avg_sq"], st["adam_step"] = torch.zeros_like(p), torch.zeros_like(p), 0
                st["adam_step"] += 1
                ta = st["adam_step"]
                st["exp_avg"].mul_(b1).add_(g, alpha=1 - b1)
                st["exp_avg_sq"].mul_(b2).addcmul_(g, g, value=1 - b2)
                m_hat = st["exp_avg"] / (1.0 - b1 ** ta)
                v_hat = st["exp_avg_sq"] / (1.0 - b2 ** ta)
                p.add_(m_hat / (torch.sqrt(v_hat) + eps) + h["adam_weight_decay"] * p, alpha=-adam_lr)
            elif h["use_adamw_for_1d"] and (p.dim() <= 1 or self.is_embedding[i]):
                st = self.state[i]
                _ema_(st["mom"], _bview(self.beta_m, p.dim()), g[None])
                _ema_(st["rms"], self.beta_rms[-1], g * g)
                # The naive class also advances the Adafactor accumulators of a tensor routed
                # to AdamW (ELO_CELO2_naive.py:298); ELO_CELO2_cuda.py:246-253 does not.  They
                # never reach the parameters on this branch, so they are left untouched here.
                m_hat = st["mom"][0] / (1.0 - beta1 ** t)
                v_hat = st["rms"] / (1.0 - beta2 ** t)
                upd = m_hat / (torch.sqrt(v_hat) + 1e-8)
                p.add_(upd + h["adam_weight_decay"] * p, alpha=-adam_lr)
            else:
                raw = self.raw_step(i, p, g)
                if keep_raw is not None:
                    keep_raw[i] = raw.clone()
                t0 = time.perf_counter()
                self.finish_step(p, raw)
                self.finish_seconds += time.perf_counter() - t0


# ----------------------------------------------------------------------------
# VeLO
# ----------------------------------------------------------------------------
def clip_log_abs(v: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """pylo/optim/Velo_naive.py:110-112"""
    return torch.clamp(torch.log(1e-8 + torch.abs(v * scale)), -5, 5) * 0.5


def fractional_tanh_embed(x: float) -> torch.Tensor:
    """pylo/optim/Velo_naive.py:119-126"""
    ts = torch.tensor([0.03, 0.1, 0.2, 0.4, 0.6, 0.8, 0.9, 1.0, 1.1], dtype=F32)
    return torch.stack([torch.tanh((x - t) * 10) for t in ts])


def tanh_time_embedding(step: float) -> torch.Tensor:
    """pylo/optim/AdafacLO_naive.py:81-87"""
    ts = torch.tensor([1, 3, 10, 30, 100, 300, 1000, 3000, 10000, 30000, 100000], dtype=F32)
    return torch.tanh(torch.tensor(step, dtype=F32) / ts - 1.0)


class LossAccumulators:
    """pylo/optim/Velo_naive.py:129-175"""

    def __init__(self, num_steps: int):
        half = torch.logspace(1, torch.log10(torch.tensor(num_steps, dtype=F32)), 10)
        self.decays = torch.exp(-1.0 / half)
        self.means = torch.zeros(10)
        self.iteration = torch.tensor(0, dtype=torch.int32)
        self.running_min = 999999999999.0 * torch.ones(10)

    def update(self, loss: torch.Tensor) -> None:
        d = self.decays
        cor = self.means / (1 - d ** (self.iteration + 1))
        approx_max = torch.where(self.iteration == 0, loss, torch.max(cor))
        loss = torch.minimum(torch.abs(approx_max) * 2, loss)
        self.means = self.means * d + loss * (1.0 - d)
        cor = self.means / (1 - d ** (self.iteration + 1))
        self.running_min = torch.minimum(self.running_min, cor)
        self.iteration = self.iteration + 1

    def features(self) -> torch.Tensor:
        cor = self.means / (1 - self.decays ** self.iteration)
        hi, lo, rmin = cor[1:], cor[:-1], self.running_min[:-1]
        f = torch.clamp((lo - rmin) / torch.maximum(torch.tensor(1e-8), hi - rmin) - 1.0, -1, 1)
        return torch.where(self.iteration <= 2, f * 0, f)


def velo_tensor_features(p, mom, rms, fraction_trained: float, loss_features) -> torch.Tensor:
    """30 LSTM input features of one tensor; ``mom (3,*s)``, ``rms (1,*s)`` are the accumulators
    *before* this step's update.  Layout: fraction(9) | loss(9) | mean_rms(1) | rank one-hot(5) |
    var_m(3) | var_rms(3), where "var_rms" subtracts mean_m (sic).

    pylo/optim/Velo_naive.py:178-206 (alphabetical key order :204)
    """
    nu = torch.rsqrt(torch.clamp(torch.mean(p ** 2), min=1e-9))
    m = mom * nu
    r = rms * nu
    axes = list(range(1, p.dim() + 1))
    mean_m = torch.mean(m, dim=axes, keepdim=True)
    var_m = torch.mean((m - mean_m) ** 2, dim=axes)
    mean_rms = torch.mean(r, dim=axes, keepdim=True)
    var_rms = torch.mean((r - mean_m) ** 2, dim=axes)
    rank = torch.zeros(5)
    rank[sum(1 for d in p.shape if d > 1)] = 1.0
    return torch.cat([
        fractional_tanh_embed(fraction_trained),
        loss_features,
        clip_log_abs(mean_rms.view(-1), 10.0),
        rank,
        clip_log_abs(var_m, 10.0),
        clip_log_abs(var_rms, 10.0),
    ])


def velo_rnn(x: torch.Tensor, h: torch.Tensor, c: torch.Tensor, sd: Dict[str, torch.Tensor]):
    """Mixing layer + one LSTM cell step + heads.  Returns (controls [T,256], lr_mult [T], h, c).

    pylo/models/VeLO_RNN.py:110-135 (mix), :43-66 (cell; gate order i, g, f, o; forget +1)
    """
    lin = lambda name, v: v @ sd[name + ".weight"].t() + sd[name + ".bias"]
    mix = torch.relu(lin("mix_layer2", x))
    x2 = lin("final_mix_layer", x) + torch.max(mix, dim=0, keepdim=True)[0]
    gates = lin("lstm.linear", torch.cat((x2, h), dim=-1))
    i, g, f, o = gates.chunk(4, -1)
    c = torch.sigmoid(f + 1) * c + torch.sigmoid(i) * torch.tanh(g)
    h = torch.sigmoid(o) * torch.tanh(c)
    return lin("rnn_to_controls", h), torch.squeeze(lin("step_size", h), -1), h, c


VELO_BANK_KEYS = ("input_weights_", "input_bias_", "hidden_weights_.0", "hidden_bias_.0",
                  "output_weights_", "output_bias_")


def velo_mix_bank(control: torch.Tensor, sd: Dict[str, torch.Tensor]) -> List[torch.Tensor]:
    """100 * mean_i(control_i * bank_i) for the six arrays.  pylo/models/VeLO_MLP.py:92-126"""
    out = []
    for k in VELO_BANK_KEYS:
        bank = sd[k]
        cw = control.view([-1] + [1] * (bank.dim() - 1))
        out.append((cw * bank).mean(0) * 100.0)
    return out


def lo_feature_groups_1d(g, mom, rms, fac_v, rs_eps: float, fac_mom_eps: float):
    """Un-normalised groups shared by VeLO / AdafacLO for a non-factored tensor, except the
    leading g / clip / p groups.  ``fac_v (3,*s)`` already updated.

    pylo/optim/Velo_naive.py:60-68,439-451,478-488; pylo/optim/AdafacLO_naive.py:70-78,289-299
    """
    rs = torch.rsqrt(rms + rs_eps)
    fac_g = g[None] * safe_rsqrt(fac_v + 1e-9)
    fac_mom = mom * torch.pow(fac_v + fac_mom_eps, -0.5)
    return rs, fac_g, fac_v, fac_v, torch.rsqrt(fac_v + 1e-8), torch.rsqrt(fac_v + 1e-8), fac_mom


def velo_feature_groups(p, g, mom, rms, fac_row, fac_col, row_factor, col_factor):
    """The 30 un-normalised VeLO channels as groups with a leading channel axis; ``fac_col is None``
    marks a non-factored tensor whose accumulator ``fac_row`` is ``fac_vec_v (3,*s)``.

    pylo/optim/Velo_naive.py:421-488 (the order of pylo/csrc/velo_kernel.cu:124-162)
    """
    if fac_col is not None:
        rs = torch.rsqrt(rms + 1e-6)
        full = (3,) + tuple(p.shape)
        rowf, colf = fac_row.expand(full), fac_col.expand(full)
        tail = [g[None] * row_factor * col_factor, (g * rs)[None], rowf, colf,
                torch.rsqrt(rowf + 1e-8), torch.rsqrt(colf + 1e-8), mom * row_factor * col_factor]
    else:
        rs, fac_g, a, b_, c_, d_, fac_mom = lo_feature_groups_1d(g, mom, rms, fac_row, 1e-6, 0.0)
        tail = [fac_g, (g * rs)[None], a, b_, c_, d_, fac_mom]
    return [g[None], torch.clip(g, -0.1, 0.1)[None], p[None], mom, rms[None], mom * rs[None], rs[None]] + tail


def velo_element_mlp(groups, weights):
    """Normalise every channel over the whole tensor (eps 1e-5) and run the tensor's 30 -> 4 -> 4 -> 3
    MLP, weights stored (out, in); returns (*shape, 3).  pylo/optim/Velo_naive.py:489-497"""
    nd = groups[0].dim() - 1
    axes = list(range(1, nd + 1))
    x30 = torch.cat([rms_normalize(v, axes, 1e-5) for v in groups], dim=0)   # (30,*s)
    w_in, b_in, w_h, b_h, w_out, b_out = weights
    hcur = torch.relu(x30.movedim(0, -1) @ w_in.t() + b_in)
    hcur = torch.relu(hcur @ w_h.t() + b_h)
    return hcur @ w_out.t() + b_out


def adafac_feature_groups(p, g, mom, rms, fac_r, fac_c, row_factor, col_factor):
    """The 28 un-normalised AdafacLO channels; ``fac_c is None`` marks a non-factored tensor whose
    accumulator ``fac_r`` is ``(3,*s)``.

    pylo/optim/AdafacLO_naive.py:262-299 (the order of pylo/csrc/learned_optimizer.cu:59-97)
    """
    if fac_c is not None:
        rs = torch.rsqrt(rms + 1e-6)
        full = (3,) + tuple(p.shape)
        rowf, colf = fac_r.expand(full), fac_c.expand(full)
        tail = [g[None] * row_factor * col_factor, rowf, colf, torch.rsqrt(rowf + 1e-8),
                torch.rsqrt(colf + 1e-8), mom * row_factor * col_factor]
    else:
        rs, fac_g, a, b_, c_, d_, fac_mom = lo_feature_groups_1d(g, mom, rms, fac_r, 1e-6, 1e-6)
        tail = [fac_g, a, b_, c_, d_, fac_mom]
    return [g[None], p[None], mom, rms[None], mom * rs[None], rs[None]] + tail


def adafac_element_mlp(groups, tfeat, sd):
    """Normalise the 28 channels over the whole tensor (eps 1e-5), append the 11 time features and run
    the 39 -> 32 -> 32 -> 2 MetaMLP; returns (*shape, 2).  pylo/optim/AdafacLO_naive.py:300-307"""
    shape = tuple(groups[0].shape[1:])
    nd = len(shape)
    x28 = rms_normalize(torch.cat(groups, dim=0), list(range(1, nd + 1)), 1e-5)
    x = torch.cat([x28.movedim(0, -1), tfeat.expand(shape + (11,))], dim=-1)
    hcur = torch.relu(x @ sd["network.input.weight"].t() + sd["network.input.bias"])
    hcur = torch.relu(hcur @ sd["network.linear_0.weight"].t() + sd["network.linear_0.bias"])
    return hcur @ sd["network.output.weight"].t() + sd["network.output.bias"]


class VeloOracle:
    """VeLO_naive.step restated (pylo/optim/Velo_naive.py:384-503).

    ``rnn`` / ``mlp`` are VeLORNN / VeLOMLP state_dicts.  State layout follows
    velo_cuda.py:366-387: ``mom (3,*s)``, ``rms (1,*s)``, ``fac_vec_row``, ``fac_vec_col``,
    ``fac_vec_v``.
    """

    def __init__(self, params, rnn, mlp, lr=1e-3, exp_mult=0.001, step_mult=0.001,
                 num_steps=10000, weight_decay=0.0,
                 initial_momentum_decays=(0.9, 0.99, 0.999), initial_rms_decays=(0.999,),
                 initial_adafactor_decays=(0.9, 0.99, 0.999),
                 momentum_decays=(0.0, 0.0, 0.0), rms_decays=(0.0,), adafactor_decays=(0.0, 0.0, 0.0),
                 device="cpu"):
        self.params = params
        self.device = torch.device(device)
        with torch.device(self.device):
            self._init(params, rnn, mlp, lr, exp_mult, step_mult, num_steps, weight_decay,
                       initial_momentum_decays, initial_rms_decays, initial_adafactor_decays,
                       momentum_decays, rms_decays, adafactor_decays)

    def _init(self, params, rnn, mlp, lr, exp_mult, step_mult, num_steps, weight_decay,
              initial_momentum_decays, initial_rms_decays, initial_adafactor_decays,
              momentum_decays, rms_decays, adafactor_decays):
        self.rnn = {k: v.detach().to(F32).to(self.device) for k, v in rnn.items()}
        self.mlp = {k: v.detach().to(F32).to(self.device) for k, v in mlp.items()}
        self.lr, self.exp_mult, self.step_mult = lr, exp_mult, step_mult
        self.weight_decay, self.num_steps = weight_decay, num_steps
        self.beta_m = decay_from_offsets(initial_momentum_decays, momentum_decays)
        self.beta_rms = decay_from_offsets(initial_rms_decays, rms_decays)
        self.beta_fac = decay_from_offsets(initial_adafactor_decays, adafactor_decays)
        self.loss = LossAccumulators(num_steps)
        self.t = 0
        T = len(params)
        self.h = self.rnn["lstm_init_state.0"].repeat(T, 1)
        self.c = self.rnn["lstm_init_state.1"].repeat(T, 1)
        self.state = []
        for p in params:
            s = tuple(p.shape)
            st = {"mom": torch.zeros((3,) + s), "rms": torch.zeros((1,) + s)}
            fd = factored_dims_velo(s)
            if fd is not None:
                dc, dr = fd
                r_, c_ = list(s), list(s)
                r_[dr] = 1
                c_[dc] = 1
                st["fac_vec_row"] = torch.zeros([3] + r_)
                st["fac_vec_col"] = torch.zeros([3] + c_)
            else:
                st["fac_vec_v"] = torch.zeros((3,) + s)
            self.state.append(st)
        self.last_controls = None
        self.last_lr_mult = None
        self.last_rnn_in = None

    def double_(self):
        """fp64 evaluation, see EloCelo2Oracle.double_."""
        self.rnn, self.mlp, self.state = _to_double(self.rnn), _to_double(self.mlp), _to_double(self.state)
        self.beta_m, self.beta_rms, self.beta_fac = self.beta_m.double(), self.beta_rms.double(), self.beta_fac.double()
        self.h, self.c = self.h.double(), self.c.double()
        self.loss.decays, self.loss.means, self.loss.running_min = (
            self.loss.decays.double(), self.loss.means.double(), self.loss.running_min.double())
        self.dtype = torch.float64
        return self

    @torch.no_grad()
    def step(self, grads: List[torch.Tensor], loss: torch.Tensor) -> None:
        with torch.device(self.device):
            self._step(grads, loss)

    def _step(self, grads, loss):
        self.loss.update(loss.detach().to(getattr(self, "dtype", F32)).to(self.device))
        loss_feats = self.loss.features()
        frac = self.t / self.num_steps
        feats = []
        for p, st in zip(self.params, self.state):
            feats.append(velo_tensor_features(p, st["mom"], st["rms"], frac, loss_feats))
        x = torch.flip(torch.stack(feats), [0])                         # Velo_naive.py:349-350
        controls, lr_mult, self.h, self.c = velo_rnn(x, self.h, self.c, self.rnn)
        self.last_controls, self.last_lr_mult, self.last_rnn_in = controls, lr_mult, x
        self.t += 1
        for i, (p, g, st) in enumerate(zip(self.params, grads, self.state)):
            if g is None:
                continue
            g = torch.clip(g, -1000.0, 1000.0)
            nd = p.dim()
            _ema_(st["mom"], _bview(self.beta_m, nd), g[None])
            _ema_(st["rms"], _bview(self.beta_rms, nd), (g * g)[None])
            rms = st["rms"][0]
            fd = factored_dims_velo(tuple(p.shape))
            if fd is not None:
                dc, dr = fd
                rf, cf = _factored_update(st, g, self.beta_fac, dc, dr, "fac_vec_row", "fac_vec_col")
                groups = velo_feature_groups(p, g, st["mom"], rms, st["fac_vec_row"], st["fac_vec_col"], rf, cf)
            else:
                b = _bview(self.beta_fac, nd)
                st["fac_vec_v"] = b * st["fac_vec_v"] + (1 - b) * (g * g + 1e-30)[None]
                groups = velo_feature_groups(p, g, st["mom"], rms, st["fac_vec_v"], None, None, None)
            out = velo_element_mlp(groups, velo_mix_bank(controls[-(1 + i)], self.mlp))
            param_scale = torch.sqrt(torch.mean(p ** 2) + 1e-9)
            step = param_scale * (out[..., 0] * torch.exp(out[..., 1] * self.exp_mult) * self.step_mult)
            step = lr_mult[-(1 + i)] * step
            p.add_(step, alpha=-self.lr)
            if self.weight_decay > 0:
                p.add_(p, alpha=-self.weight_decay * self.lr)


# ----------------------------------------------------------------------------
# AdafacLO (small_fc_lopt)
# ----------------------------------------------------------------------------
class AdafacOracle:
    """AdafacLO_naive.step restated (pylo/optim/AdafacLO_naive.py:187-311).

    ``net`` is a MetaMLP state_dict (``network.input.weight`` (32,39) ...; torch.nn.Linear
    layout, pylo/models/Meta_MLP.py:29-54).  State layout follows AdafacLO_cuda.py:227-256:
    ``exp_avg (3,*s)``, ``exp_avg_sq (*s)``, ``exp_avg_sq_r``, ``exp_avg_sq_c``.
    """

    def __init__(self, params, net, lr=1.0, exp_mult=0.001, step_mult=0.01, weight_decay=0.0,
                 initial_momentum_decays=(0.9, 0.99, 0.999), initial_rms_decays=(0.999,),
                 initial_adafactor_decays=(0.9, 0.99, 0.999),
                 momentum_decays=(0.15216392, 0.14245212, 0.06812963),
                 rms_decays=(0.01079706,),
                 adafactor_decays=(0.18621896, -0.10864615, -0.06185547), device="cpu",
                 per_param_step=False, max_grad_norm=None):
        self.max_grad_norm = max_grad_norm
        # per_param_step: the time features follow each parameter's own step counter, as the CUDA
        # class keeps it (AdafacLO_cuda.py:304-305,400), instead of the group's counter of the naive
        # class (AdafacLO_naive.py:194-197,226); the two differ only for a parameter that sat steps out.
        self.per_param_step = per_param_step
        self.steps = [0] * len(params)
        self.params = params
        dv = self.device = torch.device(device)
        self.net = {k: v.detach().to(F32).to(dv) for k, v in net.items()}
        self.lr, self.exp_mult, self.step_mult, self.weight_decay = lr, exp_mult, step_mult, weight_decay
        self.beta_m = decay_from_offsets(initial_momentum_decays, momentum_decays).to(dv)
        self.beta_rms = decay_from_offsets(initial_rms_decays, rms_decays).to(dv)
        self.beta_fac = decay_from_offsets(initial_adafactor_decays, adafactor_decays).to(dv)
        self.t = 0
        self.state = []
        for p in params:
            s = tuple(p.shape)
            st = {"exp_avg": torch.zeros((3,) + s, device=dv), "exp_avg_sq": torch.zeros(s, device=dv)}
            fd = factored_dims(s)
            if fd is not None:
                dc, dr = fd
                r_, c_ = list(s), list(s)
                r_[dr] = 1
                c_[dc] = 1
                st["exp_avg_sq_r"] = torch.zeros([3] + r_, device=dv)
                st["exp_avg_sq_c"] = torch.zeros([3] + c_, device=dv)
            else:
                st["exp_avg_sq_r"] = torch.zeros((3,) + s, device=dv)      # the (3,n) vector accumulator
                st["exp_avg_sq_c"] = st["exp_avg_sq_r"]
            self.state.append(st)

    def double_(self):
        """fp64 evaluation, see EloCelo2Oracle.double_."""
        self.net, self.state = _to_double(self.net), _to_double(self.state)
        self.beta_m, self.beta_rms, self.beta_fac = self.beta_m.double(), self.beta_rms.double(), self.beta_fac.double()
        for st in self.state:                      # keep the 1-D alias
            if st["exp_avg_sq_r"].dim() == st["exp_avg"].dim() and st["exp_avg_sq_r"].shape == st["exp_avg"].shape:
                st["exp_avg_sq_c"] = st["exp_avg_sq_r"]
        return self

    def condition_grads(self, grads):
        """``max_grad_norm``: every gradient is clipped against its own 2-norm before anything else sees it
        (AdafacLO_naive.py:199-200, ``torch.nn.utils.clip_grad_norm_(p, max_grad_norm)`` on one parameter:
        the factor is ``min(1, max_norm / (norm + 1e-6))``).  The caller's tensors are left as they are."""
        if self.max_grad_norm is None:
            return grads
        out = []
        for g in grads:
            if g is not None:
                coef = self.max_grad_norm / (torch.linalg.vector_norm(g) + 1e-6)
                g = g * torch.clamp(coef, max=1.0)
            out.append(g)
        return out

    def apply(self, p: torch.Tensor, unit_step: torch.Tensor) -> None:
        """pylo/optim/AdafacLO_naive.py:305-310 (`unit_step` = direction * exp(magnitude * exp_mult))"""
        p.add_(unit_step * self.step_mult, alpha=-self.lr)
        if self.weight_decay > 0:
            p.add_(p, alpha=-self.weight_decay * self.lr)

    @torch.no_grad()
    def step(self, grads: List[Optional[torch.Tensor]]) -> None:
        self.t += 1
        tfeat = tanh_time_embedding(self.t - 1).to(self.device)
        sd = self.net
        grads = self.condition_grads(grads)
        for i, (p, g, st) in enumerate(zip(self.params, grads, self.state)):
            if g is None:
                continue
            self.steps[i] += 1
            if self.per_param_step:
                tfeat = tanh_time_embedding(self.steps[i] - 1).to(self.device)
            nd = p.dim()
            mom = st["exp_avg"]
            _ema_(mom, _bview(self.beta_m, nd), g[None])
            _ema_(st["exp_avg_sq"], self.beta_rms[0], g * g)
            rms = st["exp_avg_sq"]
            fd = factored_dims(tuple(p.shape))
            if fd is not None:
                dc, dr = fd
                rf, cf = _factored_update(st, g, self.beta_fac, dc, dr, "exp_avg_sq_r", "exp_avg_sq_c")
                groups = adafac_feature_groups(p, g, mom, rms, st["exp_avg_sq_r"], st["exp_avg_sq_c"], rf, cf)
            else:
                b = _bview(self.beta_fac, nd)
                st["exp_avg_sq_r"] = b * st["exp_avg_sq_r"] + (1 - b) * (g * g + 1e-30)[None]
                st["exp_avg_sq_c"] = st["exp_avg_sq_r"]
                groups = adafac_feature_groups(p, g, mom, rms, st["exp_avg_sq_r"], None, None, None)
            out = adafac_element_mlp(groups, tfeat, sd)
            self.apply(p, out[..., 0] * torch.exp(out[..., 1] * self.exp_mult))


class EloOracle(AdafacOracle):
    """ELO_naive.step restated (pylo/optim/ELO_naive.py:127-238): the AdafacLO feature set and MLP with
    the accumulator decays used as given (:76-99, no offset re-parameterisation), optional global-norm
    clipping followed by ``nan_to_num`` of every gradient (:118-125,141-146), and the update
    ``p -= lr * (step + weight_decay * p)`` against the pre-step parameter (:236-237).  State in
    ELO_cuda.py:162-178's layout, which is AdafacLO_cuda's."""

    def __init__(self, params, net, lr=1e-3, exp_mult=0.001, weight_decay=0.0,
                 initial_momentum_decays=(0.9, 0.99, 0.999), initial_rms_decays=(0.999,),
                 initial_adafactor_decays=(0.9, 0.99, 0.999), clip_grad=False, clip_norm=1.0, device="cpu"):
        super().__init__(params, net, lr=lr, exp_mult=exp_mult, step_mult=1.0, weight_decay=weight_decay,
                         device=device)
        dv = self.device

        def raw(v):
            return torch.clamp(torch.tensor(v, dtype=F32, device=dv), 0.0, 1.0)

        self.beta_m, self.beta_rms, self.beta_fac = (raw(initial_momentum_decays), raw(initial_rms_decays),
                                                     raw(initial_adafactor_decays))
        self.clip_grad, self.clip_norm = clip_grad, clip_norm

    def condition_grads(self, grads):
        scale = 1.0
        if self.clip_grad:
            total = torch.zeros((), device=self.device)
            for g in grads:
                if g is not None:
                    total = total + g.detach().float().pow(2).sum()
            denom = torch.clamp(torch.sqrt(total), min=self.clip_norm)
            scale = (self.clip_norm / denom).item() if denom > 0 else 1.0
        out = []
        for g in grads:
            if g is not None:
                if scale != 1.0:
                    g = g * scale
                g = torch.nan_to_num(g)
            out.append(g)
        return out

    def apply(self, p: torch.Tensor, unit_step: torch.Tensor) -> None:
        p.add_(unit_step + self.weight_decay * p, alpha=-self.lr)
