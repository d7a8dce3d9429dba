"""VeLO's fused element pass (``k_velo_elem``) and the statistics it carries from step to step.

From its second step on a VeLO plan takes the per-tensor LSTM's input sums (over parameters, momenta and rms
as they stand before the step, velo_cuda.py:213-252) from what the previous step's apply items summed up over
the values they wrote, runs the LSTM next to the gradient sums and the statistics and apply items as one launch.
Checked here: the trajectory against the oracle and against the same library with every pass a launch of its
own (``PYLO_MI355_SLAB_ELEMS=0``), with slab parameters shrunk until small tensors span many slabs, are cut into
pieces and apply items wait on their flags; and that a write to parameters or state from outside is noticed
(in-place torch operations, replaced tensors, a loaded checkpoint) or can be announced
(``invalidate_statistics()`` after a write through ``.data``).
"""

import contextlib
import copy
import os

import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6
SHAPES = [(256, 384), (384,), (640, 128), (128, 640), (37, 101), (1024, 256), (96, 64), (64,), (1,), (512, 512),
          (32, 16, 3, 3), (1, 1, 48), (130, 128), (2048, 128)]


@contextlib.contextmanager
def _env(**kw):
    old = {k: os.environ.get(k) for k in kw}
    os.environ.update({k: str(v) for k, v in kw.items()})
    try:
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def _nets():
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(3)
    rnn = VeLORNN(lstm_hidden_size=128, param_inits=64)
    with torch.no_grad():
        rnn.lstm_init_state[0].normal_(0, 0.1)
        rnn.lstm_init_state[1].normal_(0, 0.1)
    return rnn, VeLOMLP(param_inits=64)


def _grads(gen, t):
    return [torch.randn(s, generator=gen) * 10.0 ** (-(i % 4)) for i, s in enumerate(SHAPES)]


def _run(env, steps=5, hook=None, compare=True):
    """Library trajectory next to the oracle's; `hook(t, opt, gpu, cpu)` runs between steps on both."""
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA

    rnn, mlp = _nets()
    gen = torch.Generator().manual_seed(17)
    init = [torch.randn(s, generator=gen) * 0.3 for s in SHAPES]
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    kw = dict(lr=1e-2, num_steps=50, weight_decay=1e-3)
    orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), **kw)
    with _env(**env):
        opt = VeLO_CUDA(gpu, rnn=copy.deepcopy(rnn), mlp=copy.deepcopy(mlp), **kw)
        names = None
        for t in range(steps):
            grads = _grads(gen, t)
            loss = torch.tensor(1.5 - 0.2 * t)
            for p, g in zip(gpu, grads):
                p.grad = g.cuda()
            orc.step(grads, loss)
            opt.step(loss.cuda())
            torch.cuda.synchronize()
            names = opt._plan.launch_names()
            checks = [("h", opt.lstm_hidden_state[0], orc.h), ("c", opt.lstm_hidden_state[1], orc.c)]
            for i, p in enumerate(gpu):
                checks += [(f"param{i}", p, cpu[i]), (f"mom{i}", opt.state[p]["mom"], orc.state[i]["mom"]),
                           (f"rms{i}", opt.state[p]["rms"], orc.state[i]["rms"])]
            for tag, got, ref in checks if compare else ():
                e = max_err(got, ref, REL, ABS)
                assert e <= 1.0, (env, t, tag, e)
            if hook is not None:
                opt = hook(t, opt, gpu, cpu, orc) or opt
    return gpu, names


@pytest.mark.parametrize("env", [
    {},
    {"PYLO_MI355_SLAB_ELEMS": 40000, "PYLO_MI355_KEEP_ELEMS": 10 ** 9},
    {"PYLO_MI355_SLAB_ELEMS": 40000, "PYLO_MI355_KEEP_ELEMS": 100000, "PYLO_MI355_SLAB_DEPTH": 1},
    {"PYLO_MI355_SLAB_ELEMS": 9000, "PYLO_MI355_KEEP_ELEMS": 20000, "PYLO_MI355_SLAB_DEPTH": 3},
    {"PYLO_MI355_SLAB_ELEMS": 10 ** 9, "PYLO_MI355_SLAB_DEPTH": 1},
])
def test_fused_pass_with_carried_statistics_follows_the_oracle(env):
    got, names = _run(env)
    assert "k_velo_elem" in names
    ref, ref_names = _run({"PYLO_MI355_SLAB_ELEMS": 0})
    assert "k_velo_apply" in ref_names
    for a, b in zip(got, ref):
        assert max_err(a, b, REL, ABS) <= 1.0


def test_writes_from_outside_are_noticed_or_can_be_announced():
    def hook(t, opt, gpu, cpu, orc):
        with torch.no_grad():
            if t == 1:        # in-place torch operation on a parameter: seen through its version counter
                gpu[0].mul_(1.5)
                cpu[0].mul_(1.5)
            if t == 2:        # through .data: invisible, so it is announced
                gpu[5].data.mul_(0.5)
                cpu[5].mul_(0.5)
                gpu[2].data.add_(0.25)
                cpu[2].add_(0.25)
                opt.invalidate_statistics()
            if t == 3:        # a state tensor replaced by a modified copy
                st = opt.state[gpu[3]]
                st["mom"] = st["mom"] * 2.0
                st["rms"] = st["rms"] * 3.0
                orc.state[3]["mom"] *= 2.0
                orc.state[3]["rms"] *= 3.0
        return None

    _run({}, steps=6, hook=hook)


def test_unannounced_write_through_data_is_loud():
    """A parameter scaled through ``.data`` between two steps, not announced: the device-side guard of the carried
    sums (sum p^2 re-taken by the statistics items) poisons that tensor's step and the next ``step()`` raises.  With
    the write announced (test above) the run follows the oracle."""
    seen = {}

    def hook(t, opt, gpu, cpu, orc):
        with torch.no_grad():
            if t == 2:
                gpu[5].data.mul_(0.5)
                cpu[5].mul_(0.5)
        if t == 3:
            torch.cuda.synchronize()
            seen["nan"] = bool(torch.isnan(gpu[5]).any())
            seen["others_finite"] = all(bool(torch.isfinite(p).all()) for i, p in enumerate(gpu) if i != 5)
            seen["flag"] = opt._plan.statistics_stale()
        return None

    with pytest.raises(RuntimeError, match="parameter 5 was written between two steps"):
        _run({}, steps=6, hook=hook, compare=False)
    assert seen == {"nan": True, "others_finite": True, "flag": 6}


def test_checkpoint_loaded_between_steps():
    from pylo_amd import VeLO_CUDA

    saved = {}

    def hook(t, opt, gpu, cpu, orc):
        if t == 1:
            saved["opt"] = copy.deepcopy(opt.state_dict())
            saved["params"] = [p.detach().clone() for p in gpu]
            saved["orc"] = (copy.deepcopy(orc.state), [c.clone() for c in cpu], orc.h.clone(), orc.c.clone(),
                            copy.deepcopy(orc.loss), orc.t)
        if t == 3:        # back to the state after step 1, on both sides
            with torch.no_grad():
                for p, v in zip(gpu, saved["params"]):
                    p.copy_(v)
            opt.load_state_dict(saved["opt"])
            state, params, h, c, loss, tt = saved["orc"]
            orc.state = copy.deepcopy(state)
            for cp, v in zip(cpu, params):
                cp.copy_(v)
            orc.h, orc.c, orc.loss, orc.t = h.clone(), c.clone(), copy.deepcopy(loss), tt
        return None

    _run({}, steps=6, hook=hook)
