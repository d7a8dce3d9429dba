"""GPU parity of the fused VeLO step (HIP, through the C ABI) against the golden trajectories of
the reference's naive class and against the CPU oracle at the full LSTM size.

Tolerance: rel 1e-5 / abs 1e-6 on parameters, every accumulator and the LSTM state, every step.
The reference itself has no numerical test of its VeLO kernel (tests/test_velo_cuda.py only checks
that one step does not raise).
"""

import copy

import pytest
import torch

from golden_io import Golden, max_err, trailing_to_keepdim

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6


def _nets_from_golden(G):
    from pylo_amd.models import VeLOMLP, VeLORNN

    rnn = VeLORNN(lstm_hidden_size=G.meta["lstm_hidden"], param_inits=G.meta["param_inits"])
    rnn.load_state_dict(G.state_dict("rnn"))
    mlp = VeLOMLP(param_inits=G.meta["param_inits"])
    mlp.load_state_dict(G.state_dict("mlp"))
    return rnn, mlp


@pytest.mark.parametrize("name", ["velo_small", "velo_small_wd"])
def test_velo_matches_reference_golden(name):
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA

    G = Golden(name)
    meta, shapes = G.meta, G.shapes
    rnn, mlp = _nets_from_golden(G)
    gpu = [torch.nn.Parameter(G.t(f"init/{i}").cuda()) for i in range(len(shapes))]
    opt = VeLO_CUDA(gpu, lr=meta["lr"], num_steps=meta["num_steps"], weight_decay=meta["weight_decay"],
                    rnn=rnn, mlp=mlp)
    worst = 0.0
    for t in range(meta["n_steps"]):
        for i, p in enumerate(gpu):
            p.grad = G.t(f"grad{t}/{i}").cuda()
        opt.step(G.t(f"loss{t}").cuda())
        checks = [("lstm_h", opt.lstm_hidden_state[0], G.t(f"step{t}/lstm_h")),
                  ("lstm_c", opt.lstm_hidden_state[1], G.t(f"step{t}/lstm_c"))]
        for i, p in enumerate(gpu):
            st = opt.state[p]
            checks += [(f"param{i}", p, G.t(f"step{t}/param/{i}")), (f"mom{i}", st["mom"], G.t(f"step{t}/mom/{i}")),
                       (f"rms{i}", st["rms"], G.t(f"step{t}/rms/{i}"))]
            if len(shapes[i]) < 2:
                checks.append((f"fac_v{i}", st["fac_vec_v"], G.t(f"step{t}/fac_vec_v/{i}")))
            else:
                dc, dr = O.factored_dims_velo(shapes[i])
                checks.append((f"row{i}", st["fac_vec_row"],
                               trailing_to_keepdim(G.t(f"step{t}/fac_vec_row_trailing/{i}"), dr)))
                checks.append((f"col{i}", st["fac_vec_col"],
                               trailing_to_keepdim(G.t(f"step{t}/fac_vec_col_trailing/{i}"), dc)))
        for tag, got, ref in checks:
            e = max_err(got, ref, REL, ABS)
            worst = max(worst, e)
            assert e <= 1.0, (name, t, tag, e)
    print(name, "worst err/tol", worst)


def test_velo_matches_oracle_full_size():
    """Full 512-wide LSTM / 256-entry bank, mixed shapes (tiled 2-D both orientations, dword path,
    conv-like N-D, vectors, a scalar), 5 steps, per-step comparison of everything."""
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(3)
    rnn = VeLORNN()
    with torch.no_grad():
        rnn.lstm_init_state[0].normal_(0, 0.1)
        rnn.lstm_init_state[1].normal_(0, 0.1)
    mlp = VeLOMLP()
    shapes = [(70, 384), (33, 128), (1, 128), (130, 192),  # column-resident walk: ragged row ranges, one row
              (256, 1028), (1028, 256), (300, 260), (37, 101), (32, 16, 3, 3), (1, 1, 48), (1000,), (7,), (1,),
              (64, 64), (2, 3, 64, 64)]
    gen = torch.Generator().manual_seed(17)
    init = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    kw = dict(lr=1e-2, num_steps=50, weight_decay=1e-3)
    orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), **kw)
    opt = VeLO_CUDA(gpu, rnn=copy.deepcopy(rnn), mlp=copy.deepcopy(mlp), **kw)
    worst = 0.0
    for t in range(5):
        grads = [torch.randn(s, generator=gen) * (10.0 ** (-(i % 4))) for i, s in enumerate(shapes)]
        loss = torch.tensor(1.5 - 0.2 * t)
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        orc.step(grads, loss)
        opt.step(loss.cuda())
        checks = [("h", opt.lstm_hidden_state[0], orc.h), ("c", opt.lstm_hidden_state[1], orc.c)]
        for i, p in enumerate(gpu):
            st, so = opt.state[p], orc.state[i]
            checks += [(f"param{i}", p, cpu[i]), (f"mom{i}", st["mom"], so["mom"]), (f"rms{i}", st["rms"], so["rms"])]
            for k in ("fac_vec_row", "fac_vec_col", "fac_vec_v"):
                if k in so:
                    checks.append((f"{k}{i}", st[k], so[k]))
        for tag, got, ref in checks:
            e = max_err(got, ref, REL, ABS)
            worst = max(worst, e)
            assert e <= 1.0, (t, tag, e)
    print("velo full-size worst err/tol", worst)


def test_velo_state_dict_resume():
    """Checkpoint round trip incl. loss_buffer / lstm_hidden_state / num_steps
    (tests/test_optimizer_resume.py:19-164)."""
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(5)
    rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
    shapes = [(24, 16), (16,), (8, 24)]
    gen = torch.Generator().manual_seed(2)
    init = [torch.randn(s, generator=gen) for s in shapes]
    grads = [[torch.randn(s, generator=gen).cuda() for s in shapes] for _ in range(8)]

    def run(params, opt, ts):
        for t in ts:
            for p, g in zip(params, grads[t]):
                p.grad = g.clone()
            opt.step(torch.tensor(2.0 / (1 + t)).cuda())

    a = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    oa = VeLO_CUDA(a, lr=1e-2, num_steps=20, rnn=rnn, mlp=mlp)
    run(a, oa, range(4))
    sd = copy.deepcopy(oa.state_dict())
    assert {"loss_buffer", "lstm_hidden_state", "num_steps"} <= set(sd.keys())
    snap = [p.detach().clone() for p in a]
    run(a, oa, range(4, 8))
    b = [torch.nn.Parameter(v.clone()) for v in snap]
    ob = VeLO_CUDA(b, lr=1e-2, num_steps=20, rnn=rnn, mlp=mlp)
    ob.load_state_dict(sd)
    run(b, ob, range(4, 8))
    for x, y in zip(a, b):
        assert torch.max(torch.abs(x - y)).item() < 1e-6
    st = oa.state[a[0]]
    assert st["mom"].shape == (3, 24, 16) and st["rms"].shape == (1, 24, 16)
    assert st["fac_vec_row"].shape == (3, 1, 16) and st["fac_vec_col"].shape == (3, 24, 1)
    assert oa.state[a[1]]["fac_vec_v"].shape == (3, 16)


def test_velo_replaced_state_tensor_is_picked_up():
    """A state tensor swapped for a copy between steps is the one the next step updates (the argument
    table cached between calls must notice), with the trajectory unchanged."""
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(6)
    rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
    shapes = [(24, 16), (16,), (8, 24)]
    gen = torch.Generator().manual_seed(3)
    init = [torch.randn(s, generator=gen) for s in shapes]
    grads = [[torch.randn(s, generator=gen).cuda() for s in shapes] for _ in range(6)]

    def run(swap):
        ps = [torch.nn.Parameter(v.clone().cuda()) for v in init]
        opt = VeLO_CUDA(ps, lr=1e-2, num_steps=20, rnn=rnn, mlp=mlp)
        for t in range(6):
            for p, g in zip(ps, grads[t]):
                p.grad = g.clone()
            opt.step(torch.tensor(2.0 / (1 + t)).cuda())
            if swap and t == 2:
                for p in ps:
                    for k, v in list(opt.state[p].items()):
                        if torch.is_tensor(v):
                            opt.state[p][k] = v.clone()
                            v.fill_(float("nan"))
        return ps

    # Not bit for bit: the step after the swap takes the LSTM's input sums from the tensors again (fp32
    # partial sums around the tensors' first elements), the undisturbed run from what its previous step
    # carried over (fp64 around the first elements of a step earlier); both are the same sums up to rounding.
    for x, y in zip(run(False), run(True)):
        assert torch.isfinite(y).all()
        assert max_err(y, x, REL, ABS) <= 1.0


def test_velo_variance_features_where_the_spread_is_tiny():
    """The LSTM sees log-variances of the momentum / rms accumulators of every tensor.  A one-element
    tensor, or one whose gradient is the same for every element, has variance exactly zero in the
    reference (the feature sits at its lower clamp); large gradients on a small parameter make that a
    cancellation of order 1e2 in single precision unless the sums are shifted.  The LSTM mixes tensors
    through a max-pool, so one wrong row shows in every tensor's state."""
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(4)
    rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
    shapes = [(1, 1), (1,), (6, 40), (33,), (129, 257)]
    gen = torch.Generator().manual_seed(8)
    init = [torch.randn(s, generator=gen) * 0.01 for s in shapes]
    grads = []
    for t in range(4):
        gs = [torch.randn(s, generator=gen) * 30.0 for s in shapes]
        gs[2] = torch.full(shapes[2], 17.0 + t)          # the same gradient for every element
        gs[3] = torch.full(shapes[3], -250.0) + torch.randn(shapes[3], generator=gen) * 1e-3
        grads.append(gs)
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cpu = [v.clone() for v in init]
    opt = VeLO_CUDA(gpu, lr=1e-2, num_steps=10, rnn=rnn, mlp=mlp)
    orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), lr=1e-2, num_steps=10)
    loss = torch.tensor(1.0)
    for t in range(4):
        for p, g in zip(gpu, grads[t]):
            p.grad = g.cuda()
        opt.step(loss)
        orc.step([g.clone() for g in grads[t]], loss)
        torch.cuda.synchronize()
        assert max_err(opt.lstm_hidden_state[0].cpu(), orc.h, REL, ABS) <= 1.0, (t, "h")
        assert max_err(opt.lstm_hidden_state[1].cpu(), orc.c, REL, ABS) <= 1.0, (t, "c")
        for i, (p, c) in enumerate(zip(gpu, cpu)):
            assert max_err(p.detach().cpu(), c, REL, ABS) <= 1.0, (t, i)


def test_velo_loss_accumulators_follow_the_reference():
    """The ten loss EMAs, their running minima and the iteration counter (Velo_naive.py:129-175) over a
    loss sequence with a spike (clipped to twice the largest corrected mean), a plateau and a rise; the
    nine loss features feed the LSTM from the third step on, so its state is compared as well."""
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(9)
    rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
    shapes = [(12, 20), (20,)]
    gen = torch.Generator().manual_seed(3)
    init = [torch.randn(s, generator=gen) * 0.1 for s in shapes]
    losses = [2.3, 1.9, 1.7, 40.0, 1.5, 1.5, 1.5, 0.9, 1.2, 2.0, 0.05, 0.04]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cpu = [v.clone() for v in init]
    opt = VeLO_CUDA(gpu, lr=1e-2, num_steps=30, rnn=rnn, mlp=mlp)
    orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), lr=1e-2, num_steps=30)
    for t, lv in enumerate(losses):
        grads = [torch.randn(s, generator=gen) * 0.1 for s in shapes]
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        loss = torch.tensor(lv)
        opt.step(loss.cuda())
        orc.step(grads, loss)
        torch.cuda.synchronize()
        lb = opt.loss_buffer
        assert int(lb["iteration"]) == int(orc.loss.iteration) == t + 1
        assert max_err(lb["means"].cpu(), orc.loss.means, REL, ABS) <= 1.0, (t, "means")
        assert max_err(lb["running_min"].cpu(), orc.loss.running_min, REL, ABS) <= 1.0, (t, "running_min")
        assert max_err(opt.lstm_hidden_state[0].cpu(), orc.h, REL, ABS) <= 1.0, (t, "h")
        assert max_err(opt.lstm_hidden_state[1].cpu(), orc.c, REL, ABS) <= 1.0, (t, "c")
        for i, (p, c) in enumerate(zip(gpu, cpu)):
            assert max_err(p.detach().cpu(), c, REL, ABS) <= 1.0, (t, i)
