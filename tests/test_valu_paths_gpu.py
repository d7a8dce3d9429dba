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


def test_adafac_valu(monkeypatch):
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    monkeypatch.setenv("PYLO_MI355_VALU_MLP", "1")
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
