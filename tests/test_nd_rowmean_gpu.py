"""row_col_mean of tensors with more than two dims: the mean of the row accumulator over the axis of
the second-largest dim, one value per slice.  The V0 kernel tabulates it per block in three ways (a thread
per slice for a short axis, a wave per slice for a long one, per entry when a block would touch more than
1024 slices); each shape below lands in one of them, with the axis last or in the middle of the row
vector.  AdafacLO and VeLO against the oracle, two steps, rel 1e-5 / abs 1e-6 on parameters and the
row / column accumulators."""

import copy

import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6
SHAPES = [
    (64, 3, 16, 16),     # axis of 16, last in the row vector: a thread per slice
    (48, 16, 3),         # axis of 16 with stride 3
    (300, 3, 256),       # axis of 256, last: a wave per slice
    (130, 100, 7),       # axis of 100 with stride 7
    (34, 33, 32, 35),    # axis of 34 with stride 33 * 32 = 1056 slices per block: per entry
]


@pytest.mark.parametrize("which", ["adafac", "velo"])
def test_nd_row_col_mean_paths(which):
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA, VeLO_CUDA
    from pylo_amd.models import MetaMLP, VeLOMLP, VeLORNN

    torch.manual_seed(2)
    gen = torch.Generator().manual_seed(5)
    init = [torch.randn(s, generator=gen) * 0.1 for s in SHAPES]
    grads = [[torch.randn(s, generator=gen) * 0.05 * (1 + torch.rand(s[-1], generator=gen)) for s in SHAPES]
             for _ in range(2)]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cpu = [v.clone() for v in init]
    if which == "adafac":
        net = MetaMLP(39, 32, 1)
        opt = AdafacLO_CUDA(gpu, lr=0.5, network=copy.deepcopy(net), hf_key=None)
        orc = O.AdafacOracle(cpu, net.state_dict(), lr=0.5)
        keys, okeys, loss = ("exp_avg_sq_r", "exp_avg_sq_c"), ("exp_avg_sq_r", "exp_avg_sq_c"), None
    else:
        rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
        opt = VeLO_CUDA(gpu, lr=1e-2, num_steps=10, rnn=copy.deepcopy(rnn), mlp=copy.deepcopy(mlp))
        orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), lr=1e-2, num_steps=10)
        keys, okeys, loss = ("fac_vec_row", "fac_vec_col"), ("fac_vec_row", "fac_vec_col"), torch.tensor(0.7)
    for t in range(2):
        for p, g in zip(gpu, grads[t]):
            p.grad = g.cuda()
        cg = [g.clone() for g in grads[t]]
        if loss is None:
            opt.step()
            orc.step(cg)
        else:
            opt.step(loss)
            orc.step(cg, loss)
        torch.cuda.synchronize()
        for i, (p, c) in enumerate(zip(gpu, cpu)):
            assert max_err(p.detach().cpu(), c, REL, ABS) <= 1.0, (which, t, i, SHAPES[i])
            for k, ok in zip(keys, okeys):
                assert max_err(opt.state[p][k].cpu(), orc.state[i][ok], REL, ABS) <= 1.0, (which, t, i, k)
