"""GPU parity of the fused AdafacLO step (HIP, through the C ABI) against the golden trajectories
of the reference's naive class and against the CPU oracle on larger / odd shapes.

Tolerance: rel 1e-5 / abs 1e-6 on parameters and every accumulator, every step.  The reference has
no numerical test of its `cuda_lo` kernel for AdafacLO (only a resume test).
"""

import copy

import pytest
import torch

from golden_io import Golden, max_err, trailing_to_keepdim

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6


@pytest.mark.parametrize("name", ["adafac_small", "adafac_small_wd", "adafac_max_norm"])
def test_adafac_matches_reference_golden(name):
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    G = Golden(name)
    meta, shapes = G.meta, G.shapes
    net = MetaMLP(39, 32, 1)
    net.load_state_dict(G.state_dict("net"))
    gpu = [torch.nn.Parameter(G.t(f"init/{i}").cuda()) for i in range(len(shapes))]
    # adafac_max_norm: max_grad_norm=1.0, per-parameter norm clipping inside the fused step
    opt = AdafacLO_CUDA(gpu, lr=meta["lr"], weight_decay=meta["weight_decay"], network=net, **(meta.get("extra") or {}))
    worst = 0.0
    for t in range(meta["n_steps"]):
        for i, p in enumerate(gpu):
            p.grad = G.t(f"grad{t}/{i}").cuda()
        opt.step()
        for i, p in enumerate(gpu):
            st = opt.state[p]
            checks = [("param", p, G.t(f"step{t}/param/{i}")), ("exp_avg", st["exp_avg"], G.t(f"step{t}/exp_avg/{i}")),
                      ("exp_avg_sq", st["exp_avg_sq"], G.t(f"step{t}/exp_avg_sq/{i}"))]
            if len(shapes[i]) < 2:
                checks.append(("fac_v", st["exp_avg_sq_r"], G.t(f"step{t}/fac_vec_v/{i}")))
            else:
                dc, dr = O.factored_dims(shapes[i])
                checks.append(("row", st["exp_avg_sq_r"],
                               trailing_to_keepdim(G.t(f"step{t}/fac_vec_row_trailing/{i}"), dr)))
                checks.append(("col", st["exp_avg_sq_c"],
                               trailing_to_keepdim(G.t(f"step{t}/fac_vec_col_trailing/{i}"), dc)))
            for tag, got, ref in checks:
                e = max_err(got, ref, REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (name, t, i, tag, e)
    print(name, "worst err/tol", worst)


@pytest.mark.parametrize("max_norm", [None, 0.7, "second group only"])
def test_adafac_matches_oracle_mixed_shapes(max_norm):
    """max_norm: ``max_grad_norm`` of the class (every gradient clipped against its own norm inside the fused step;
    gradient norms here run from 0.003 to 360, so some tensors are scaled and some are not), for all parameters or
    for the second of two parameter groups only."""
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(9)
    net = MetaMLP(39, 32, 1)
    shapes = [(256, 516), (516, 256), (300, 260), (37, 101), (32, 16, 3, 3), (1, 1, 48), (1000,), (7,), (64, 64),
              (70, 384), (33, 128), (1, 128), (130, 192), (3, 64)]  # column-resident walks (128 / 64 columns a wave)
    gen = torch.Generator().manual_seed(23)
    init = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    if max_norm == "second group only":
        half = len(shapes) // 2
        orc = O.AdafacOracle(cpu, net.state_dict(), lr=0.5, weight_decay=1e-3, max_grad_norm=0.7)
        clip = orc.condition_grads
        orc.condition_grads = lambda gs: gs[:half] + clip(gs[half:])
        groups = [{"params": gpu[:half]}, {"params": gpu[half:], "max_grad_norm": 0.7}]
        opt = AdafacLO_CUDA(groups, lr=0.5, weight_decay=1e-3, network=copy.deepcopy(net))
    else:
        orc = O.AdafacOracle(cpu, net.state_dict(), lr=0.5, weight_decay=1e-3, max_grad_norm=max_norm)
        opt = AdafacLO_CUDA(gpu, lr=0.5, weight_decay=1e-3, network=copy.deepcopy(net), max_grad_norm=max_norm)
    worst = 0.0
    for t in range(5):
        grads = [torch.randn(s, generator=gen) * (10.0 ** (-(i % 4))) for i, s in enumerate(shapes)]
        if t == 4:
            grads[3] = None      # a tensor without gradient is skipped
        for p, g in zip(gpu, grads):
            p.grad = None if g is None else g.cuda()
        orc.step(grads)
        opt.step()
        for p, g in zip(gpu, grads):     # the fused step scales what it reads, never the caller's buffer
            assert g is None or torch.equal(p.grad.cpu(), g)
        for i, p in enumerate(gpu):
            st, so = opt.state[p], orc.state[i]
            checks = [("param", p, cpu[i])]
            if len(st):
                checks += [("exp_avg", st["exp_avg"], so["exp_avg"]), ("exp_avg_sq", st["exp_avg_sq"], so["exp_avg_sq"]),
                           ("r", st["exp_avg_sq_r"], so["exp_avg_sq_r"]), ("c", st["exp_avg_sq_c"], so["exp_avg_sq_c"])]
            for tag, got, ref in checks:
                e = max_err(got, ref, REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (t, i, tag, e)
    print("adafac mixed worst err/tol", worst)


def test_parameter_that_sat_steps_out_keeps_its_own_step_counter():
    """AdafacLO_cuda.py:304-305,400: the time features come from each parameter's own ``state["step"]``;
    a parameter without gradient on some steps lags behind and the call carries per-tensor counters."""
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(12)
    net = MetaMLP(39, 32, 1)
    shapes = [(40, 128), (24, 20), (50,), (3, 4, 5)]
    gen = torch.Generator().manual_seed(5)
    init = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    orc = O.AdafacOracle(cpu, net.state_dict(), lr=0.5, per_param_step=True)
    opt = AdafacLO_CUDA(gpu, lr=0.5, network=copy.deepcopy(net))
    for t in range(6):
        grads = [torch.randn(s, generator=gen) * 0.1 for s in shapes]
        if t in (1, 2):
            grads[0] = None
        if t == 3:
            grads[2] = grads[3] = None
        for p, g in zip(gpu, grads):
            p.grad = None if g is None else g.cuda()
        orc.step(grads)
        opt.step()
        for i, p in enumerate(gpu):
            assert float(opt.state[p]["step"]) == orc.steps[i]
            e = max_err(p, cpu[i], REL, ABS)
            assert e <= 1.0, (t, i, e)
    assert [float(opt.state[p]["step"]) for p in gpu] == [4.0, 6.0, 5.0, 5.0]


def test_adafac_state_dict_resume():
    """tests/test_optimizer_resume.py:19-164"""
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(4)
    net = MetaMLP(39, 32, 1)
    shapes = [(24, 16), (16,)]
    gen = torch.Generator().manual_seed(2)
    init = [torch.randn(s, generator=gen) for s in shapes]
    grads = [[torch.randn(s, generator=gen).cuda() for s in shapes] for _ in range(8)]

    def run(params, opt, ts):
        for t in ts:
            for p, g in zip(params, grads[t]):
                p.grad = g.clone()
            opt.step()

    a = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    oa = AdafacLO_CUDA(a, lr=1.0, network=net)
    run(a, oa, range(4))
    sd = copy.deepcopy(oa.state_dict())
    snap = [p.detach().clone() for p in a]
    run(a, oa, range(4, 8))
    b = [torch.nn.Parameter(v.clone()) for v in snap]
    ob = AdafacLO_CUDA(b, lr=1.0, network=net)
    ob.load_state_dict(sd)
    run(b, ob, range(4, 8))
    for x, y in zip(a, b):
        assert torch.max(torch.abs(x - y)).item() < 1e-6
    st = oa.state[a[0]]
    assert set(st.keys()) == {"step", "exp_avg_sq_r", "exp_avg_sq_c", "exp_avg_sq", "exp_avg"}
    assert st["exp_avg"].shape == (3, 24, 16) and st["exp_avg_sq_r"].shape == (3, 1, 16)
    assert st["step"].dtype == torch.float64 and float(st["step"]) == 8.0


def test_mulo_wrapper_runs_the_fused_step_with_per_group_learning_rates():
    """MuLO_CUDA (pylo/optim/MuLO_cuda.py:12-61) = AdafacLO_CUDA over groups split by muP width multiplier
    with lr / multiplier: same parameters, bit for bit, as AdafacLO_CUDA given those groups directly."""
    from pylo_amd import AdafacLO_CUDA, MuLO_CUDA
    from pylo_amd.models import MetaMLP

    class Inf:
        def __init__(self, n, w):
            self.n, self.w = n, w

        def ninf(self):
            return self.n

        def width_mult(self):
            return self.w

    torch.manual_seed(2)
    net = MetaMLP(39, 32, 1)
    shapes, infs = [(40, 128), (24, 20), (50,), (16, 16)], [Inf(2, 4.0), Inf(2, 2.0), Inf(1, 1.0), Inf(2, 4.0)]
    gen = torch.Generator().manual_seed(8)
    init = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
    grads = [[torch.randn(s, generator=gen).cuda() * 0.1 for s in shapes] for _ in range(3)]
    a = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    for p, i in zip(a, infs):
        p.infshape = i
    oa = MuLO_CUDA(a, lr=0.8, network=copy.deepcopy(net))
    assert [g["lr"] for g in oa.param_groups] == [0.2, 0.4, 0.8]
    b = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    ob = AdafacLO_CUDA([dict(params=[b[0], b[3]], lr=0.2), dict(params=[b[1]], lr=0.4), dict(params=[b[2]], lr=0.8)],
                       lr=0.8, network=copy.deepcopy(net))
    for t in range(3):
        for ps in (a, b):
            for p, g in zip(ps, grads[t]):
                p.grad = g.clone()
        oa.step()
        ob.step()
    for x, y, v in zip(a, b, init):
        assert torch.equal(x, y)
        assert not torch.equal(x.cpu(), v)


@pytest.mark.parametrize("cls_name", ["AdafacLO_CUDA", "ELO_CUDA"])
def test_convolution_kernels_walked_as_matrices(cls_name):
    """(O, I, k, ..) tensors whose two largest dims are the leading ones take the column-resident apply pass as the
    matrix (O, I * k..): one statistics vector is indexed by the matrix column, the other by (row, column mod k..).
    Covered: O > I, O < I, O == I (the tie goes to I), one and three trailing dims, a size-1 dim in between, rows
    that do not fill the last tile; (8, 128, 3, 64) and (32, 16, 3, 3) stay on the generic path (factored dims
    not leading / I * k * k not a multiple of 64)."""
    from oracle import pylo_oracle as O
    import pylo_amd
    from pylo_amd.models import MetaMLP

    torch.manual_seed(5)
    net = MetaMLP(39, 32, 1)
    shapes = [(64, 64, 3, 3), (96, 128, 3, 3), (128, 64, 3, 3), (40, 64, 5), (256, 32, 2, 2, 2), (8, 128, 3, 64),
              (130, 64, 1, 3), (32, 16, 3, 3), (64, 128)]
    gen = torch.Generator().manual_seed(31)
    init = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    if cls_name == "ELO_CUDA":
        kw = dict(lr=1e-2, weight_decay=0.05, exp_mult=0.01, clip_grad=True, clip_norm=2.0)
        orc = O.EloOracle(cpu, net.state_dict(), **kw)
        opt = pylo_amd.ELO_CUDA(gpu, network=copy.deepcopy(net), hf_key=None, **kw)
    else:
        orc = O.AdafacOracle(cpu, net.state_dict(), lr=0.5, weight_decay=1e-3)
        opt = pylo_amd.AdafacLO_CUDA(gpu, lr=0.5, weight_decay=1e-3, network=copy.deepcopy(net))
    worst = 0.0
    for t in range(4):
        grads = [torch.randn(s, generator=gen) * (10.0 ** (-(i % 3))) for i, s in enumerate(shapes)]
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        orc.step(grads)
        opt.step()
        for i, p in enumerate(gpu):
            st, so = opt.state[p], orc.state[i]
            checks = [("param", p, cpu[i]), ("exp_avg", st["exp_avg"], so["exp_avg"]),
                      ("exp_avg_sq", st["exp_avg_sq"], so["exp_avg_sq"]),
                      ("r", st["exp_avg_sq_r"], so["exp_avg_sq_r"]), ("c", st["exp_avg_sq_c"], so["exp_avg_sq_c"])]
            for tag, got, ref in checks:
                e = max_err(got, ref, REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (cls_name, t, i, shapes[i], tag, e)
    print(cls_name, "convolution kernels worst err/tol", worst)
