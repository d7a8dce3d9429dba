"""Seeded random parameter sets through whole optimizer steps against the oracle: one to nine tensors of one to five
dims (single elements, vectors, ragged and tile-sized matrices, convolution kernels, size-1 dims), random group
settings (clipping, orthogonalisation, iteration counts, weight decay, the MLP on vectors, param_scale_mult), a
gradient missing now and then.  Three steps a set; parameters at rel 1e-5 / abs 1e-6 after every step.  ELO-CELO2
parameters are re-synchronised after each step: five Newton-Schulz iterations amplify the fp32 rounding of the raw
step of a nearly singular 3 x 3 slice by up to 3.4445^5 in any fp32 evaluation, and free-running sets would compound
that.
"""

import copy
import random

import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6


def _shape(rng, wide):
    k = rng.random()
    if k < 0.2:
        return (rng.choice([1, 2, 7, 64, 300, 1000, 4097]),)
    if k < 0.6:
        return (rng.choice([1, 2, 3, 5, 8, 16, 33, 64, 100, 128, 130, 256, 300, 513]),
                rng.choice([1, 2, 4, 7, 16, 31, 64, 96, 128, 200, 256, 384, 1000] + ([1024] if wide else [])))
    if k < 0.85:
        return (rng.choice([1, 2, 3, 8, 16]), rng.choice([1, 2, 4, 8]), rng.choice([1, 3, 5, 7]), rng.choice([1, 3, 5, 7]))
    if k < 0.95:
        return (rng.choice([1, 2, 5]), rng.choice([1, 8, 16, 40, 64, 130]), rng.choice([1, 4, 16, 33, 64, 128, 140]))
    return (rng.choice([2, 3]), rng.choice([1, 2]), rng.choice([1, 2, 3]), rng.choice([2, 3, 9]), rng.choice([1, 4, 6]))


@pytest.mark.parametrize("block", range(4))
def test_elo_celo2_random_sets(block):
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    worst = 0.0
    for seed in range(40 * block, 40 * block + 40):
        rng = random.Random(seed)
        torch.manual_seed(seed)
        net = CELO2MLP()
        shapes = [_shape(rng, False) for _ in range(rng.randint(1, 9))]
        cfg = dict(lr=rng.choice([1e-3, 3e-4]), weight_decay=rng.choice([0.0, 0.1]), adam_lr_mult=rng.choice([1.0, 20.0]),
                   orthogonalize=rng.random() < 0.8, use_adamw_for_1d=rng.random() < 0.7,
                   ns_iters=rng.choice([5, 5, 5, 3, 1, 0, 4]), exp_mult=rng.choice([0.0, 0.01]),
                   clip_grad=rng.random() < 0.7, param_scale_mult=rng.random() < 0.15)
        gen = torch.Generator(device="cuda").manual_seed(seed)
        init = [torch.randn(s, generator=gen, device="cuda") * 0.05 for s in shapes]
        ref = [v.double() for v in init]
        gpu = [torch.nn.Parameter(v.clone()) for v in init]
        orc = O.EloCelo2Oracle(ref, net.state_dict(), device="cuda", **cfg).double_()
        opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
        for t in range(3):
            grads = [None if (t > 0 and rng.random() < 0.05)
                     else torch.randn(s, generator=gen, device="cuda") * 10.0 ** (-rng.randint(0, 3)) for s in shapes]
            for p, g in zip(gpu, grads):
                p.grad = g
            orc.step([None if g is None else g.double() for g in grads])
            opt.step()
            for i, p in enumerate(gpu):
                e = max_err(p, ref[i], REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (seed, t, i, shapes, cfg, e)
                p.data.copy_(ref[i].float())
    print("ELO-CELO2 random sets, worst err/tol", worst)


@pytest.mark.parametrize("which", ["velo", "adafac"])
def test_velo_and_adafac_random_sets(which):
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA, VeLO_CUDA
    from pylo_amd.models import MetaMLP, VeLOMLP, VeLORNN

    worst = 0.0
    for seed in range(60):
        rng = random.Random(1000 + seed)
        torch.manual_seed(seed)
        shapes = [_shape(rng, True) for _ in range(rng.randint(1, 8))]
        if which == "velo":   # one-hot rank feature of five classes (velo_cuda.py:174): at most four dims larger than one
            shapes = [s for s in shapes if sum(d > 1 for d in s) < 5] or [(8, 8)]
        gen = torch.Generator().manual_seed(seed)
        init = [torch.randn(s, generator=gen) * 0.05 for s in shapes]
        cpu = [v.clone() for v in init]
        gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
        if which == "velo":
            rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
            kw = dict(lr=rng.choice([1e-2, 1e-3]), num_steps=rng.choice([20, 1000]), weight_decay=rng.choice([0.0, 0.01]))
            orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), **kw)
            opt = VeLO_CUDA(gpu, rnn=copy.deepcopy(rnn), mlp=copy.deepcopy(mlp), **kw)
        else:
            net = MetaMLP(39, 32, 1)
            kw = dict(lr=rng.choice([0.5, 1.0]), weight_decay=rng.choice([0.0, 1e-3]))
            orc = O.AdafacOracle(cpu, net.state_dict(), per_param_step=True, **kw)
            opt = AdafacLO_CUDA(gpu, network=copy.deepcopy(net), **kw)
        for t in range(3):
            grads = [torch.randn(s, generator=gen) * 10.0 ** (-rng.randint(0, 3)) for s in shapes]
            for p, g in zip(gpu, grads):
                p.grad = g.cuda()
            if which == "velo":
                loss = torch.tensor(2.0 - 0.3 * t)
                orc.step(grads, loss)
                opt.step(loss)
            else:
                orc.step(grads)
                opt.step()
            for i, p in enumerate(gpu):
                e = max_err(p, cpu[i], REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (which, seed, t, i, shapes, kw, e)
    print(which, "random sets, worst err/tol", worst)
