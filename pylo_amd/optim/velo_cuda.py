"""VeLO_CUDA on MI355X: one multi-tensor HIP step instead of the reference's per-tensor loop.

Drop-in for pylo/optim/velo_cuda.py:255-755: same constructor, ``step(loss)``, per-parameter
state (``layer_idx``, ``mom (3,*s)``, ``rms (1,*s)``, ``fac_vec_row``, ``fac_vec_col``,
``fac_vec_v``, ``rank_onehot``) and the extended ``state_dict`` (``loss_buffer``,
``lstm_hidden_state``, ``num_steps``).  Loss features, the per-tensor LSTM features, the LSTM
itself, bank mixing, every accumulator update and the per-element MLP run inside
``pylo_mi355_velo_step`` (12 launches, no host synchronisation -- the reference calls ``.item()``
once per tensor).  Arithmetic follows the naive class (pylo/optim/Velo_naive.py:384-503).
"""

from __future__ import annotations

import ctypes as C

import numpy as np
import torch
import torch.nn.functional as F
from torch.optim import Optimizer

from .. import _lib
from ..models import VeLOMLP, VeLORNN, pack_velo_bank


def factored_dims(shape):
    """(dc, dr): 2nd-largest and largest dim; an equal pair is swapped except 4-D (0, 1)
    (pylo/optim/velo_cuda.py:121-131)."""
    if len(shape) < 2:
        return None
    order = sorted(range(len(shape)), key=lambda i: (shape[i], i))
    a, b = order[-2], order[-1]
    if shape[a] == shape[b] and not (len(shape) == 4 and a == 0 and b == 1):
        return b, a
    return a, b


def _decays(initial, offsets, device):
    """clip(1 - exp(10 * (log(1 - d0) / 10 + offset)), 0, 1), in fp32 (velo_cuda.py:134-139,293-310)."""
    d0 = torch.tensor(initial, device=device)
    par = torch.log(1 - d0) / 10.0 + torch.tensor(offsets, device=device)
    return torch.clip(1 - torch.exp(par * 10.0), 0.0, 1.0)


_FRAC_TS = (0.03, 0.1, 0.2, 0.4, 0.6, 0.8, 0.9, 1.0, 1.1)


def fractional_tanh_embed(x: float) -> torch.Tensor:
    """tanh((x - ts) * 10) for the 9 fixed timescales (velo_cuda.py:155-162)."""
    return torch.tanh((x - torch.tensor(_FRAC_TS, dtype=torch.float32)) * 10)


class VeLO_CUDA(Optimizer):
    def __init__(
        self,
        params,
        momentum_decays=[0.0, 0.0, 0.0],
        rms_decays=[0.0],
        adafactor_decays=[0.0, 0.0, 0.0],
        lr=1e-3,
        exp_mult=0.001,
        step_mult=0.001,
        input_size=30,
        hidden_size=4,
        hidden_layers=1,
        initial_momentum_decays=(0.9, 0.99, 0.999),
        lstm_input_size=30,
        lstm_hidden_size=512,
        param_inits=256,
        num_steps=10000,
        initial_rms_decays=(0.999,),
        initial_adafactor_decays=(0.9, 0.99, 0.999),
        concat_weights=True,
        make_separate_weights=False,
        split_weights=False,
        weight_decay=0.0,
        clip_grad=False,
        mup_lrs=None,
        hf_key_rnn="Pauljanson002/VeLO_RNN",
        hf_key_mlp="Pauljanson002/VeLO_MLP",
        legacy=False,
        rnn: VeLORNN = None,
        mlp: VeLOMLP = None,
        capturable: bool = False,
    ):
        # capturable: the per-group step counters live on the device and ``step(loss)`` can be recorded
        # into a HIP graph (torch.cuda.graph) and replayed; ``group["step"]`` is then refreshed by
        # ``state_dict()`` / ``sync_step_counters()`` only.  The reference has no such mode.
        self.capturable = bool(capturable)
        self._dev_steps = None
        if legacy:
            raise NotImplementedError("legacy=True (the pure-PyTorch parameter loop) is not provided")
        if not torch.cuda.is_available():
            raise RuntimeError("VeLO_CUDA requires a GPU (torch.cuda.is_available() is False).")
        _lib.load()
        params = list(params)
        probe = params[0]
        if isinstance(probe, dict):
            probe["params"] = list(probe["params"])
            probe = probe["params"][0]
        self.device = probe.device
        if not probe.is_cuda:
            raise RuntimeError("VeLO_CUDA: parameters must live on a GPU")
        clip_mom = _decays(initial_momentum_decays, momentum_decays, self.device)
        clip_rms = _decays(initial_rms_decays, rms_decays, self.device)
        clip_fac = _decays(initial_adafactor_decays, adafactor_decays, self.device)
        defaults = dict(
            lr=lr, exp_mult=exp_mult, step_mult=step_mult, initial_momentum_decays=clip_mom,
            lstm_hidden_size=lstm_hidden_size, initial_rms_decays=clip_rms,
            initial_adafactor_decays=clip_fac, param_inits=param_inits, concat_weights=concat_weights,
            make_separate_weights=make_separate_weights, input_size=input_size, hidden_size=hidden_size,
            hidden_layers=hidden_layers, split_weights=split_weights, clip_grad=clip_grad, mup_lrs=mup_lrs,
            weight_decay=weight_decay, legacy=legacy)
        super().__init__(params, defaults)
        self.legacy = legacy
        self.num_steps = num_steps
        self.loss_buffer = self._init_loss_buffer(num_steps)
        self.rnn = (rnn if rnn is not None else VeLORNN.from_pretrained(hf_key_rnn)).to(self.device)
        self.network_stack = (mlp if mlp is not None else VeLOMLP.from_pretrained(hf_key_mlp)).to(self.device)
        self.lstm_init_state = self.rnn.lstm_init_state
        for net in (self.rnn, self.network_stack):
            for prm in net.parameters():
                prm.requires_grad = False
        if self.network_stack.hidden_layers != 1 or tuple(self.network_stack.input_weights.shape) != (4, 30) \
                or self.network_stack.output_weights.shape[0] != 3:
            raise ValueError("VeLO_CUDA kernel only supports the 30 -> 4 -> 4 -> 3 per-element MLP")
        if not self.rnn.mix_layers:
            raise ValueError("VeLO_CUDA kernel needs mix_layers=True")
        self._pack_networks()
        self.init_state()
        self._plan = None
        self._plan_key = None

    # ------------------------------------------------------------------ state
    def _init_loss_buffer(self, num_steps):
        """pylo/optim/velo_cuda.py:170-181"""
        halflife = torch.logspace(1, torch.log10(torch.tensor(num_steps, dtype=torch.float32)), 10)
        decays = torch.exp(-1.0 / halflife)
        return {
            "means": torch.zeros(10, dtype=torch.float32, device=self.device),
            "iteration": torch.tensor(0, dtype=torch.int32, device=self.device),
            "running_min": 999999999999.0 * torch.ones(10, dtype=torch.float32, device=self.device),
            "decays": decays.to(self.device),
        }

    @torch.no_grad()
    def init_state(self):
        """pylo/optim/velo_cuda.py:356-387"""
        layer_idx = 0
        for group in self.param_groups:
            group["step"] = 0
            for p in group["params"]:
                if p.requires_grad is False:
                    continue
                state = self.state[p]
                shape = tuple(p.shape)
                if len(state) == 0:
                    state["layer_idx"] = layer_idx
                    state["mom"] = torch.zeros((3,) + shape, device=self.device)
                    state["rms"] = torch.zeros((1,) + shape, device=self.device)
                    fd = factored_dims(shape)
                    empty = torch.tensor([], dtype=torch.float32, device=self.device)
                    if fd is not None:
                        dc, dr = fd
                        r_shape, c_shape = list(shape), list(shape)
                        r_shape[dr] = 1
                        c_shape[dc] = 1
                        state["fac_vec_row"] = torch.zeros([3] + r_shape, device=self.device)
                        state["fac_vec_col"] = torch.zeros([3] + c_shape, device=self.device)
                        state["fac_vec_v"] = empty
                    else:
                        state["fac_vec_row"], state["fac_vec_col"] = empty, empty.clone()
                        state["fac_vec_v"] = torch.zeros((3,) + shape, device=self.device)
                    n_rank = sum(1 for dim in shape if dim > 1)
                    state["rank_onehot"] = F.one_hot(torch.tensor(n_rank), num_classes=5).float().to(self.device)
                layer_idx += 1
        self.lstm_hidden_state = (
            self.lstm_init_state[0].detach().repeat(layer_idx, 1).to(self.device).contiguous(),
            self.lstm_init_state[1].detach().repeat(layer_idx, 1).to(self.device).contiguous(),
        )

    # ------------------------------------------------------------------ device-side step counters
    def _reset_device_steps(self):
        values = [0] * _lib.MAX_GROUPS
        for gi, group in enumerate(self.param_groups):
            values[gi] = int(group["step"])
        if self._dev_steps is None:
            self._dev_steps = torch.zeros(_lib.MAX_GROUPS, dtype=torch.int32, device=self.device)
        self._dev_steps.copy_(torch.tensor(values, dtype=torch.int32))   # in place: graphs keep the pointer
        self._plan.device_steps(self._dev_steps, num_steps=float(self.num_steps))
        self._plan.pinned_table(0)        # handed out now, not while a capture is open

    def sync_step_counters(self):
        """capturable mode: read the device counters back into ``group["step"]`` (waits for the GPU)."""
        if self.capturable and self._dev_steps is not None and self._plan is not None:
            values = self._dev_steps.tolist()
            for gi, group in enumerate(self.param_groups):
                group["step"] = values[gi]

    def refresh_graph_tables(self):
        """capturable mode: copy the groups' lr / weight_decay / exp_mult / step_mult into the pinned
        table that a recorded ``step()`` reads, e.g. after a scheduler step.  Call it while no replay
        is in flight."""
        if not self.capturable or self._plan is None:
            return
        table = self._plan.pinned_table(0)
        for i, (_gi, group, _p) in enumerate(self._tensors()):
            for k in ("lr", "weight_decay", "exp_mult", "step_mult"):
                table[k][i] = group[k]

    def state_dict(self):
        self.sync_step_counters()
        sd = super().state_dict()
        sd["loss_buffer"] = self.loss_buffer
        sd["lstm_hidden_state"] = self.lstm_hidden_state
        sd["num_steps"] = self.num_steps
        return sd

    def load_state_dict(self, state_dict):
        self._fast = None
        loss_buffer = state_dict.pop("loss_buffer")
        lstm_hidden_state = state_dict.pop("lstm_hidden_state")
        num_steps = state_dict.pop("num_steps")
        super().load_state_dict(state_dict)
        self.loss_buffer = {k: (v.to(self.device) if torch.is_tensor(v) else v) for k, v in loss_buffer.items()}
        self.lstm_hidden_state = tuple(t.to(self.device).contiguous() for t in lstm_hidden_state)
        self.num_steps = num_steps
        if self.capturable and self._plan is not None:
            self._reset_device_steps()

    # ------------------------------------------------------------------ networks
    def _pack_networks(self):
        """Device copies of the LSTM / bank weights in the (in, out) layout the kernels read."""
        r = self.rnn

        def t(w):
            return w.detach().float().t().contiguous().to(self.device)

        def v(b):
            return b.detach().float().contiguous().to(self.device)

        def gates_last(w):
            # (4H, 2H) with gate blocks i, g, f, o -> (2H, H, 4): a unit's four gate weights side by side
            h4, k2 = w.shape
            return w.detach().float().reshape(4, h4 // 4, k2).permute(2, 1, 0).contiguous().to(self.device)

        self._w = dict(
            mix2_wt=t(r.mix_layer2.weight), mix2_b=v(r.mix_layer2.bias),
            fmix_wt=t(r.final_mix_layer.weight), fmix_b=v(r.final_mix_layer.bias),
            lstm_wt=gates_last(r.lstm.linear.weight), lstm_b=v(r.lstm.linear.bias),
            ctrl_wt=t(r.rnn_to_controls.weight), ctrl_b=v(r.rnn_to_controls.bias),
            lr_w=v(r.step_size.weight.reshape(-1)), lr_b=v(r.step_size.bias),
            bank=pack_velo_bank(self.network_stack).to(self.device))
        H = r.lstm.linear.weight.shape[0] // 4
        K = r.rnn_to_controls.weight.shape[0]
        if self._w["bank"].shape != (K, 159):
            raise ValueError("VeLOMLP bank size does not match the LSTM's control width")
        if H % 64 != 0 or H > 1024:
            raise ValueError("VeLO_CUDA kernel needs an LSTM width that is a multiple of 64, at most 1024")
        nets = _lib.VeloNets()
        for k, w in self._w.items():
            setattr(nets, k, w.data_ptr())
        nets.hidden, nets.n_bank = H, K
        self._nets = nets
        self._H, self._K = H, K

    # ------------------------------------------------------------------ step
    def _tensors(self):
        out = []
        for gi, group in enumerate(self.param_groups):
            for p in group["params"]:
                if p.requires_grad is False:
                    continue
                out.append((gi, group, p))
        return out

    def _ensure_plan(self, tensors):
        key = tuple((tuple(p.shape), p.dtype) for _, _, p in tensors)
        if key == self._plan_key:
            return
        if len(self.param_groups) > _lib.MAX_GROUPS:
            raise ValueError(f"VeLO_CUDA supports at most {_lib.MAX_GROUPS} parameter groups")
        for _, _, p in tensors:
            if not p.is_cuda or p.device != self.device or not p.is_contiguous():
                raise TypeError("VeLO_CUDA: parameters must be contiguous tensors on the optimizer's GPU")
        if self._plan is not None:
            self._plan.close()
        # parameters and gradients may be float16 / bfloat16 / float64 (the reference's kernels dispatch on the
        # element type, velo_kernel.cu:405,427); the accumulators stay float32
        self._plan = _lib.Plan(_lib.KIND_VELO, [tuple(p.shape) for _, _, p in tensors],
                               [_lib.store_flag(p, "VeLO_CUDA") for _, _, p in tensors], self.device)
        self._plan_key = key
        if self.capturable:
            self._reset_device_steps()

    @torch.no_grad()
    def step(self, loss):
        tensors = self._tensors()
        self._ensure_plan(tensors)
        plan = self._plan
        n = len(tensors)
        bad = plan.statistics_stale()
        if bad:
            # the device-side guard of the carried sums (see invalidate_statistics) caught a parameter that was
            # written from outside between two steps: that step's update of the tensor is NaN
            self.invalidate_statistics()
            raise RuntimeError(
                f"VeLO_CUDA: parameter {bad - 1} was written between two steps in a way the optimizer does not see "
                "(through .data or by a custom kernel) and the step after it ran on the LSTM input statistics "
                "carried over from before the write; that step's update of the tensor was set to NaN. Call "
                "invalidate_statistics() after such writes, or write through in-place torch operations on the "
                "parameter itself.")
        if self.lstm_hidden_state[0].shape[0] != n:
            raise RuntimeError("VeLO_CUDA: the LSTM state does not match the number of parameters")
        if not torch.is_tensor(loss):
            loss = torch.tensor(float(loss))
        loss_dev = loss.detach().to(device=self.device, dtype=torch.float32).reshape(1)

        st = _lib.VeloStep()
        for gi, group in enumerate(self.param_groups):
            frac = fractional_tanh_embed(group["step"] / self.num_steps).tolist()
            for q in range(9):
                st.frac[gi][q] = frac[q]
        if not self.capturable:     # else counted on the device, which also forms the time features
            for group in self.param_groups:
                group["step"] += 1

        fast = getattr(self, "_fast", None)
        if fast is not None and (fast["key"] is not self._plan_key or len(self.state) != fast["n_state"]):
            fast = self._fast = None
        fl = {k: [0.0] * n for k in ("lr", "weight_decay", "clip_val", "exp_mult", "step_mult")}
        grp = [0] * n
        keep = []
        if fast is not None:
            # static columns (state pointers, group index) are still in the table from an earlier
            # step: refresh gradient / parameter pointers and the per-group scalars only
            grads = [p.grad for _, _, p in tensors]
            for g in grads:     # a dense gradient has its parameter's dtype (torch enforces it on assignment)
                if g is None or g.layout is not torch.strided or not g.is_contiguous():
                    fast = self._fast = None
                    break
        if fast is not None:
            for state, key, t, version in fast["alive"]:
                # a state tensor was replaced (the cached pointers are stale) or written in place through torch
                # (the carried sums over mom / rms are): the library's own writes do not count in `_version`
                if state.get(key) is not t or t._version != version:
                    fast = self._fast = None
                    break
            else:
                # a parameter object was swapped, or written in place through torch since the last step
                # (the library's own writes do not count in `_version`)
                if any(a is not p or v != p._version for a, v, (_, _, p) in zip(fast["params"], fast["versions"], tensors)):
                    fast = self._fast = None
        if fast is not None:
            args = plan.args
            gidx = fast["gidx"]
            args["grad"] = [g.data_ptr() for g in grads]
            args["param"] = [p.data_ptr() for _, _, p in tensors]
            for k in ("lr", "weight_decay", "exp_mult", "step_mult"):
                args[k] = np.asarray([g[k] for g in self.param_groups], dtype=np.float64)[gidx]
            tensors_slow = ()
        else:
            keys = ("grad", "param", "mom", "rms", "fac_r", "fac_c", "fac_v")
            cols = {k: [0] * n for k in keys}
            tensors_slow = tensors
        for i, (gi, group, p) in enumerate(tensors_slow):
            g = p.grad
            if g is None:
                raise RuntimeError("VeLO_CUDA.step: every parameter needs a gradient")
            if g.dtype != p.dtype or g.is_sparse:
                raise TypeError("VeLO_CUDA: gradients must be dense and of their parameter's dtype")
            if not g.is_contiguous():
                g = g.contiguous()
                keep.append(g)
            state = self.state[p]
            if state["layer_idx"] != i:
                raise RuntimeError("VeLO_CUDA: parameter order changed since init_state()")
            cols["grad"][i], cols["param"][i] = g.data_ptr(), p.data_ptr()
            cols["mom"][i], cols["rms"][i] = state["mom"].data_ptr(), state["rms"].data_ptr()
            if factored_dims(tuple(p.shape)) is None:
                cols["fac_v"][i] = state["fac_vec_v"].data_ptr()
            else:
                cols["fac_r"][i] = state["fac_vec_row"].data_ptr()
                cols["fac_c"][i] = state["fac_vec_col"].data_ptr()
            fl["lr"][i], fl["weight_decay"][i] = group["lr"], group["weight_decay"]
            fl["clip_val"][i] = 1000.0
            fl["exp_mult"][i], fl["step_mult"][i] = group["exp_mult"], group["step_mult"]
            grp[i] = gi
        if fast is None:
            # anything that sends the step down this path (first step, a loaded checkpoint, a replaced
            # state tensor or parameter, a parameter written in place) may have changed what the LSTM's
            # input sums are taken over: the library takes them from the tensors again
            plan.invalidate_statistics()
            args = plan.args
            for k, v in cols.items():
                args[k] = v
            for k, v in fl.items():
                args[k] = v
            args["group"] = grp
            if not keep:
                # every accumulator of every parameter is watched for replacement (a few hundred identity checks
                # a step); beyond 512 parameters only the two whose sums are carried from step to step, because
                # the walk then costs milliseconds a step: there, the factored accumulators must be updated in
                # place or through load_state_dict()
                keys = ("mom", "rms", "fac_vec_row", "fac_vec_col", "fac_vec_v") if n <= 512 else ("mom", "rms")
                alive = [(self.state[p], k, self.state[p][k], self.state[p][k]._version) for _, _, p in tensors for k in keys]
                self._fast = dict(key=self._plan_key, n_state=len(self.state), alive=alive,
                                  params=[p for _, _, p in tensors], versions=[p._version for _, _, p in tensors],
                                  gidx=np.asarray(grp, dtype=np.int64))

        h, c = self.lstm_hidden_state
        lb = self.loss_buffer
        st.lstm_h, st.lstm_c = h.data_ptr(), c.data_ptr()
        st.loss_means, st.loss_running_min = lb["means"].data_ptr(), lb["running_min"].data_ptr()
        st.loss_decays, st.loss_iteration = lb["decays"].data_ptr(), lb["iteration"].data_ptr()
        st.loss = loss_dev.data_ptr()
        st.controls_out = st.lr_mult_out = None
        table = None
        if self.capturable and torch.cuda.is_current_stream_capturing():
            # the recorded call reads the plan's pinned table in place on every replay
            table = plan.pinned_table(0)
            table[:] = plan.args
        with torch.cuda.device(self.device):
            plan.velo_step(self._decays_struct(), self._nets, st,
                           torch.cuda.current_stream(self.device).cuda_stream, args=table)
        del keep, loss_dev
        return

    def invalidate_statistics(self):
        """Call after writing parameters or ``mom`` / ``rms`` state tensors in a way the optimizer cannot see
        (through ``.data`` or a custom kernel): the next step then reads every tensor for the LSTM's input
        statistics, as the reference does on every step, instead of using the sums the previous step left.

        What the optimizer sees by itself: a parameter or state tensor object that was replaced, in-place torch
        operations on a parameter or on ``mom`` / ``rms`` (their version counters), ``load_state_dict``.  What it
        catches after the fact: a parameter written through ``.data`` or by a custom kernel.  The statistics
        items of every step re-sum p^2 of every tensor (they read the parameter anyway) and compare it with the
        carried sum; on a mismatch that step's update of the tensor is NaN and the next ``step()`` whose call
        sees the flag raises ``RuntimeError`` (the flag is read without waiting for the GPU, so up to the steps
        in flight later).  Not caught: writes to ``mom`` / ``rms`` through ``.data``."""
        self._fast = None
        if self._plan is not None:
            self._plan.invalidate_statistics()

    def _decays_struct(self):
        g0 = self.param_groups[0]
        key = (id(g0["initial_momentum_decays"]), id(g0["initial_rms_decays"]), id(g0["initial_adafactor_decays"]))
        if getattr(self, "_dec_key", None) != key:
            self._dec = _lib.make_decays(g0["initial_momentum_decays"].tolist(),
                                         float(g0["initial_rms_decays"][0]),
                                         g0["initial_adafactor_decays"].tolist())
            self._dec_key = key
        return self._dec
