"""GPU parity of ELO_CUDA (HIP, through the C ABI): AdafacLO's kernels with ELO's raw decays, global-norm
clipping, ``nan_to_num`` and update rule, against golden trajectories of the reference's ELO_naive and
against the CPU oracle on larger / odd shapes.

Tolerance: rel 1e-5 / abs 1e-6 on parameters and every accumulator, every step (the reference's own
check of its CUDA class, tests/test_elo_cuda.py, compares parameters at 1e-4).
"""

import copy

import pytest
import torch

from golden_io import Golden, max_err, trailing_to_keepdim

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6


@pytest.mark.parametrize("name", ["elo_small", "elo_small_nan"])
def test_elo_matches_reference_golden(name):
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CUDA
    from pylo_amd.models import MetaMLP

    G = Golden(name)
    meta, shapes = G.meta, G.shapes
    net = MetaMLP(39, 32, 1)
    net.load_state_dict(G.state_dict("net"))
    gpu = [torch.nn.Parameter(G.t(f"init/{i}").cuda()) for i in range(len(shapes))]
    extra = {k: (tuple(v) if isinstance(v, list) else v) for k, v in meta["extra"].items()}
    opt = ELO_CUDA(gpu, lr=meta["lr"], weight_decay=meta["weight_decay"], network=net, hf_key=None, **extra)
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
            assert float(st["step"]) == t + 1
    print(name, "worst err/tol", worst)


@pytest.mark.parametrize("clip", [True, False])
def test_elo_matches_oracle_mixed_shapes(clip):
    """Every walk of the AdafacLO kernels (column-resident, chunked 2-D, N-D, 1-D), NaN and infinite
    gradient elements, a tensor without gradient; with clipping the global norm is NaN on the steps that
    carry a NaN (scale 1, ELO_naive.py:118-125) and the exact re-reduction runs on the others."""
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(9)
    net = MetaMLP(39, 32, 1)
    shapes = [(256, 516), (516, 256), (37, 101), (32, 16, 3, 3), (1, 1, 48), (1000,), (7,), (64, 64),
              (70, 384), (33, 128), (130, 192), (3, 64)]
    gen = torch.Generator().manual_seed(29)
    init = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cfg = dict(lr=1e-2, weight_decay=0.03, exp_mult=0.01, clip_grad=clip, clip_norm=3.0,
               initial_momentum_decays=(0.5, 0.9, 0.99), initial_rms_decays=(0.9,),
               initial_adafactor_decays=(0.8, 0.95, 0.999))
    orc = O.EloOracle(cpu, net.state_dict(), **cfg)
    opt = ELO_CUDA(gpu, network=copy.deepcopy(net), hf_key=None, **cfg)
    worst = 0.0
    for t in range(5):
        grads = [torch.randn(s, generator=gen) * (10.0 ** (-(i % 3))) for i, s in enumerate(shapes)]
        if t == 1:                                  # NaNs in every kind of walk
            for i in (0, 2, 3, 5, 8):
                grads[i].view(-1)[[1, grads[i].numel() // 2, grads[i].numel() - 1]] = float("nan")
        if t == 3 and clip:                         # an infinity: the clip scale is 0 and every gradient becomes 0
            grads[1].view(-1)[17] = float("inf")
        if t == 4:
            grads[2] = None
        for p, g in zip(gpu, grads):
            p.grad = None if g is None else g.cuda()
        orc.step(grads)
        opt.step()
        for i, p in enumerate(gpu):
            st, so = opt.state[p], orc.state[i]
            checks = [("param", p, cpu[i]), ("exp_avg", st["exp_avg"], so["exp_avg"]),
                      ("exp_avg_sq", st["exp_avg_sq"], so["exp_avg_sq"]),
                      ("r", st["exp_avg_sq_r"], so["exp_avg_sq_r"]), ("c", st["exp_avg_sq_c"], so["exp_avg_sq_c"])]
            for tag, got, ref in checks:
                assert bool(torch.isfinite(ref).all()), (t, i, tag)
                e = max_err(got, ref, REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (clip, t, i, tag, e)
    print("elo mixed worst err/tol", worst)


def test_elo_gradients_are_left_untouched_and_plain_adafac_plans_reject_clipping():
    from pylo_amd import _lib, ELO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(1)
    net = MetaMLP(39, 32, 1)
    p = torch.nn.Parameter(torch.randn(40, 128).cuda())
    g = torch.randn(40, 128).cuda() * 10
    g[3, 5] = float("nan")
    p.grad = g.clone()
    opt = ELO_CUDA([p], network=net, hf_key=None, clip_grad=True, clip_norm=1.0)
    opt.step()
    torch.cuda.synchronize()
    assert torch.equal(torch.nan_to_num(p.grad, nan=123.0), torch.nan_to_num(g, nan=123.0))   # not scaled in place
    assert bool(torch.isfinite(p).all())
    plan = _lib.Plan(_lib.KIND_ADAFAC, [(40, 128)], [0], p.device)
    plan.args["grad"], plan.args["param"] = g.data_ptr(), p.data_ptr()
    st = opt.state[p]
    plan.args["mom"], plan.args["rms"] = st["exp_avg"].data_ptr(), st["exp_avg_sq"].data_ptr()
    plan.args["fac_r"], plan.args["fac_c"] = st["exp_avg_sq_r"].data_ptr(), st["exp_avg_sq_c"].data_ptr()
    plan.args["clip_norm"] = 1.0
    with pytest.raises(RuntimeError, match="PYLO_F_GLOBAL_NORM"):
        plan.adafac_step(opt._decays, opt._net, 0.0, torch.cuda.current_stream().cuda_stream)
