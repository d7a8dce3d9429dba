"""Scalar (0-dim) and empty parameters through the five optimizer classes: a 0-dim parameter behaves
like a one-element vector (compared with the oracle run on shape (1,)), empty tensors are carried
along without touching memory.  VeLO mixes information across tensors (the LSTM's max-pool over
rows), so its empty-tensor case is only checked for finiteness: the reference itself yields NaN there
(means over zero elements)."""

import copy

import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6
SHAPES = [(), (0,), (0, 5), (4, 0), (16, 8), (1, 1), (5,)]
AS_ORACLE = [(1,), None, None, None, (16, 8), (1, 1), (5,)]


def _run(make_opt, make_orc, shapes=SHAPES, as_oracle=AS_ORACLE, loss=None, compare=True):
    gen = torch.Generator().manual_seed(1)
    init = [torch.randn(s, generator=gen) for s in shapes]
    grads = [[torch.randn(s, generator=gen) for s in shapes] for _ in range(3)]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    keep = [i for i, r in enumerate(as_oracle) if r is not None]
    cpu = [init[i].clone().reshape(as_oracle[i]) for i in keep]
    opt, orc = make_opt(gpu), make_orc(cpu)
    for t in range(3):
        for p, g in zip(gpu, grads[t]):
            p.grad = g.cuda()
        cg = [grads[t][i].reshape(as_oracle[i]) for i in keep]
        if loss is None:
            opt.step()
            orc.step(cg)
        else:
            opt.step(loss)
            orc.step(cg, loss)
    torch.cuda.synchronize()
    for i, c in zip(keep, cpu):
        assert bool(torch.isfinite(gpu[i]).all())
        assert not torch.equal(gpu[i].detach().cpu().reshape(c.shape), init[i].reshape(c.shape))   # it moved
        if compare:
            e = max_err(gpu[i].detach().reshape(c.shape), c, REL, ABS)
            assert e <= 1.0, (i, shapes[i], e)


def test_celo2_family():
    from oracle import pylo_oracle as O
    from pylo_amd import CELO2_CUDA, ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(1)
    net = CELO2MLP()
    _run(lambda g: ELO_CELO2_CUDA(g, lr=1e-2, network=net, hf_key=None, adam_lr_mult=1.0),
         lambda c: O.EloCelo2Oracle(c, net.state_dict(), lr=1e-2))
    _run(lambda g: CELO2_CUDA(g, lr=1e-2, network=net, hf_key=None),
         lambda c: O.EloCelo2Oracle(c, net.state_dict(), lr=1e-2, weight_decay=0.0, clip_grad=False,
                                    independent_adam=(0.9, 0.95, 1e-8)))


def test_adafac_family():
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA, ELO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(2)
    net = MetaMLP(39, 32, 1)
    _run(lambda g: AdafacLO_CUDA(g, lr=0.5, network=copy.deepcopy(net)),
         lambda c: O.AdafacOracle(c, net.state_dict(), lr=0.5))
    _run(lambda g: ELO_CUDA(g, lr=1e-2, network=copy.deepcopy(net), hf_key=None, clip_grad=True),
         lambda c: O.EloOracle(c, net.state_dict(), lr=1e-2, clip_grad=True))


def test_velo():
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(3)
    rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
    kw = dict(lr=1e-1, step_mult=0.1, num_steps=10)

    def make_opt(g):
        return VeLO_CUDA(g, rnn=copy.deepcopy(rnn), mlp=copy.deepcopy(mlp), **kw)

    def make_orc(c):
        return O.VeloOracle(c, rnn.state_dict(), mlp.state_dict(), **kw)

    loss = torch.tensor(1.0)
    _run(make_opt, make_orc, shapes=[(), (16, 8), (1, 1), (5,)], as_oracle=[(1,), (16, 8), (1, 1), (5,)], loss=loss)
    _run(make_opt, make_orc, loss=loss, compare=False)      # with empty tensors: runs, stays finite
