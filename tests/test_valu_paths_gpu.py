"""The all-VALU kernels over linear chunks, kept next to the matrix-pipe kernels and selected with
PYLO_MI355_VALU_MLP=1 when a plan is created: same parity bar (rel 1e-5 / abs 1e-6 against the oracle) on
shapes that the default build walks column-resident."""

import copy

import pytest
import torch

from golden_io import step_keeping_raw, max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6
SHAPES = [(70, 384), (33, 128), (256, 516), (130, 192), (37, 101), (300,), (3, 64)]


def _inputs(seed, scale=0.3):
    gen = torch.Generator().manual_seed(seed)
    init = [torch.randn(s, generator=gen) * scale for s in SHAPES]
    grads = [[torch.randn(s, generator=gen) * (10.0 ** (-(i % 3))) for i, s in enumerate(SHAPES)] for _ in range(3)]
    return init, grads


def test_celo2_valu(monkeypatch):
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    monkeypatch.setenv("PYLO_MI355_VALU_MLP", "1")
    torch.manual_seed(1)
    net = CELO2MLP()
    init, grads = _inputs(3)
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cfg = dict(lr=1e-2, exp_mult=0.01, adam_lr_mult=20.0)
    orc = O.EloCelo2Oracle(cpu, net.state_dict(), **cfg)
    opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
    for t in range(3):
        raw = {}
        for p, g in zip(gpu, grads[t]):
            p.grad = g.cuda()
        orc.step(grads[t], keep_raw=raw)
        kept = step_keeping_raw(opt)
        for i, r in raw.items():
            assert max_err(kept[i], r, REL, ABS) <= 1.0, ("raw", t, i)
        for i, p in enumerate(gpu):
            for k, v in orc.state[i].items():
                assert max_err(opt.state[p][k], v, REL, ABS) <= 1.0, (t, i, k)
            p.data.copy_(cpu[i])


def test_velo_valu(monkeypatch):
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    monkeypatch.setenv("PYLO_MI355_VALU_MLP", "1")
    torch.manual_seed(2)
    rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
    init, grads = _inputs(4)
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), lr=1e-2, num_steps=20)
    opt = VeLO_CUDA(gpu, lr=1e-2, num_steps=20, rnn=copy.deepcopy(rnn), mlp=copy.deepcopy(mlp))
    for t in range(3):
        loss = torch.tensor(2.0 - 0.3 * t)
        for p, g in zip(gpu, grads[t]):
            p.grad = g.cuda()
        orc.step(grads[t], loss)
        opt.step(loss)
        for i, p in enumerate(gpu):
            assert max_err(p, cpu[i], REL, ABS) <= 1.0, (t, i)


@pytest.mark.parametrize("switch", ["PYLO_MI355_VALU_MLP", "PYLO_MI355_ADAFAC_F32"])
def test_adafac_valu(monkeypatch, switch):
    """AdafacLO's element MLP runs on the fp16 matrix instructions by default (operands split into two
    fp16 planes, three products per fp32 product); PYLO_MI355_ADAFAC_F32=1 keeps it on the fp32 matrix
    instructions, PYLO_MI355_VALU_MLP=1 on the vector pipe."""
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    monkeypatch.setenv(switch, "1")
    torch.manual_seed(3)
    net = MetaMLP(39, 32, 1)
    init, grads = _inputs(5)
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    orc = O.AdafacOracle(cpu, net.state_dict(), lr=0.5, weight_decay=1e-3)
    opt = AdafacLO_CUDA(gpu, lr=0.5, weight_decay=1e-3, network=copy.deepcopy(net))
    for t in range(3):
        for p, g in zip(gpu, grads[t]):
            p.grad = g.cuda()
        orc.step(grads[t])
        opt.step()
        for i, p in enumerate(gpu):
            assert max_err(p, cpu[i], REL, ABS) <= 1.0, (t, i)
            for k in ("exp_avg", "exp_avg_sq", "exp_avg_sq_r", "exp_avg_sq_c"):
                assert max_err(opt.state[p][k], orc.state[i][k], REL, ABS) <= 1.0, (t, i, k)


def test_adafac_matrix_pipes_against_fp64(monkeypatch):
    """The split-fp16 MLP gives up no accuracy: the parameter steps of both matrix-pipe variants against the
    oracle evaluated in fp64, relative to the error the fp32 oracle itself makes (both stay below it)."""
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(3)
    net = MetaMLP(39, 32, 1)
    shapes = [(256, 512), (96, 1024)]
    gen = torch.Generator().manual_seed(8)
    init = [torch.randn(s, generator=gen) * 0.01 for s in shapes]     # small against the step: p's own rounding stays out of the way
    grads = [torch.randn(s, generator=gen) * 0.1 for s in shapes]
    ref64 = [v.double().cuda() for v in init]
    ref32 = [v.clone().cuda() for v in init]
    kw = dict(lr=1.0, step_mult=1.0, exp_mult=0.1)
    O.AdafacOracle(ref64, net.state_dict(), device="cuda", **kw).double_().step([g.double().cuda() for g in grads])
    O.AdafacOracle(ref32, net.state_dict(), device="cuda", **kw).step([g.cuda() for g in grads])
    own = max(float((a.double() - b).abs().max()) for a, b in zip(ref32, ref64))
    errs = {}
    for name, env in (("fp16x2", "0"), ("fp32", "1")):
        monkeypatch.setenv("PYLO_MI355_ADAFAC_F32", env)
        gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
        opt = AdafacLO_CUDA(gpu, network=copy.deepcopy(net), **kw)
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        opt.step()
        torch.cuda.synchronize()
        errs[name] = max(float((p.detach().double() - b).abs().max()) for p, b in zip(gpu, ref64))
    print("max |p - fp64 oracle|: fp32 oracle", own, " HIP", errs)
    assert errs["fp16x2"] <= 1.5 * max(own, errs["fp32"]), (errs, own)


def test_adafac_fp16_planes_keep_their_range():
    """The default element MLP splits its operands into fp16 planes, which want numbers of order one: gradients of
    1e-12 next to a single outlier ten thousand times the rest (raw features from 1e-24 to 1e12, normalised features up
    to the square root of the element count, hidden values in the thousands) must come out finite and as close to the
    fp64 evaluation as the fp32 matrix instructions and the fp32 oracle bring them (lr = step_mult = 1: the step
    itself is what is compared)."""
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(4)
    net = MetaMLP(39, 32, 1)
    shapes = [(256, 512), (128, 1024), (64, 2048)]
    gen = torch.Generator().manual_seed(9)
    init = [torch.randn(s, generator=gen) * 0.01 for s in shapes]
    grads = [torch.randn(shapes[0], generator=gen) * 1e-12, torch.randn(shapes[1], generator=gen) * 1e-3,
             torch.randn(shapes[2], generator=gen) * 10.0]
    grads[0][7, 11] = 1e-8           # ten thousand times its neighbours
    grads[1][100, 5] = 50.0
    grads[2][3, 2000] = 2e5
    kw = dict(lr=1.0, step_mult=1.0, exp_mult=0.1)
    ref64 = [v.double().cuda() for v in init]
    ref32 = [v.clone().cuda() for v in init]
    O.AdafacOracle(ref64, net.state_dict(), device="cuda", **kw).double_().step([g.double().cuda() for g in grads])
    O.AdafacOracle(ref32, net.state_dict(), device="cuda", **kw).step([g.cuda() for g in grads])
    outs = {}
    for name, env in (("fp16x2", "0"), ("fp32", "1")):
        mp = pytest.MonkeyPatch()
        mp.setenv("PYLO_MI355_ADAFAC_F32", env)
        try:
            gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
            opt = AdafacLO_CUDA(gpu, network=copy.deepcopy(net), **kw)
            for p, g in zip(gpu, grads):
                p.grad = g.cuda()
            opt.step()
            torch.cuda.synchronize()
            outs[name] = [p.detach().clone() for p in gpu]
        finally:
            mp.undo()
    for i in range(len(shapes)):
        own = float((ref32[i].double() - ref64[i]).abs().max())
        e = {name: float((outs[name][i].double() - ref64[i]).abs().max()) for name in outs}
        size = float((ref64[i] - init[i].double().cuda()).abs().max())
        print(shapes[i], "largest step", size, "max |p - fp64 oracle|: fp32 oracle", own, " HIP", e)
        assert torch.isfinite(outs["fp16x2"][i]).all(), i
        assert e["fp16x2"] <= 2.0 * max(own, e["fp32"]) + 1e-7 * size, (i, e, own)
