"""Steps recorded into a HIP graph (``capturable=True``): the step counters live on the device and the
recorded call reads the plan's pinned argument table in place, so replays need no host work.

Every replay is checked against an ordinary optimizer stepping eagerly on the same gradients
(rel 1e-5 / abs 1e-6 on the parameters), with eager work and synchronisations between the replays.
"""

import copy

import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6


def _celo2_net(seed):
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(seed)
    return CELO2MLP()


def _close(a, b, tag):
    for i, (x, y) in enumerate(zip(a, b)):
        e = max_err(x.detach().cpu(), y.detach().cpu(), REL, ABS)
        assert e <= 1.0, (tag, i, e)


def _graph_vs_eager(make_opt, step, shapes, n_warm=2, n_replay=4, seed=0):
    """make_opt(params, capturable) -> optimizer; step(opt) runs one step.  Returns both optimizers."""
    gen = torch.Generator().manual_seed(seed)
    init = [torch.randn(s, generator=gen) * 0.1 for s in shapes]
    grads = [[torch.randn(s, generator=gen) * 0.05 for s in shapes] for _ in range(n_warm + n_replay)]
    ref_p = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cap_p = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    ref, cap = make_opt(ref_p, False), make_opt(cap_p, True)
    for p in cap_p:
        p.grad = torch.zeros_like(p)              # static gradient buffers, refilled in place

    def feed(t):
        for p, q, g in zip(ref_p, cap_p, grads[t]):
            g = g.cuda()
            p.grad = g.clone()
            q.grad.copy_(g)

    side = torch.cuda.Stream()
    for t in range(n_warm):                       # eager steps of the capturable optimizer
        feed(t)
        step(ref)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(cap)
        torch.cuda.current_stream().wait_stream(side)
        _close(cap_p, ref_p, f"eager {t}")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(cap)
    _close(cap_p, ref_p, "capture must not run the step")
    for t in range(n_warm, n_warm + n_replay):
        feed(t)
        step(ref)
        graph.replay()
        torch.cuda.synchronize()
        _close(cap_p, ref_p, f"replay {t}")
        _ = sum(float(p.detach().sum()) for p in cap_p)    # eager work and a synchronisation between replays
    return ref, cap, n_warm + n_replay


@pytest.mark.parametrize("whole_step", [False, True, "tall"])
def test_elo_celo2_step_replays_from_a_graph(whole_step):
    from pylo_amd import ELO_CELO2_CUDA

    net = _celo2_net(3)
    shapes = [(96, 64), (64,), (64, 160), (160,), (33, 7)]
    if whole_step == "tall":
        # a very tall matrix: Newton-Schulz takes its Gram product over 25 row slabs and adds them up with a
        # library reduction, the Frobenius norm runs over a million elements -- both inside the graph
        shapes = [(16400, 64), (64,)]
        whole_step = True

    def make(params, capturable):
        return ELO_CELO2_CUDA(params, lr=1e-2, weight_decay=0.05, network=net, hf_key=None,
                              orthogonalize=whole_step, capturable=capturable)

    ref, cap, n = _graph_vs_eager(make, lambda o: o.step(), shapes)
    assert cap.state_dict()["param_groups"][0]["step"] == n == ref.param_groups[0]["step"]


def test_celo2_independent_adam_counters_on_the_device():
    from pylo_amd import CELO2_CUDA

    net = _celo2_net(4)
    shapes = [(48, 40), (40,), (40, 24), (24,)]

    def make(params, capturable):
        return CELO2_CUDA(params, lr=1e-2, weight_decay=0.01, adam_lr_mult=3.0, network=net, hf_key=None,
                          orthogonalize=False, capturable=capturable)

    ref, cap, n = _graph_vs_eager(make, lambda o: o.step(), shapes)
    cap.sync_step_counters()
    p1 = cap.param_groups[0]["params"][1]
    assert cap.state[p1]["adam_step"] == n == ref.state[ref.param_groups[0]["params"][1]]["adam_step"]


def test_capturable_checkpoint_resumes_the_counters():
    """state_dict() of a capturable optimizer carries the device counters; loading it into a fresh one
    continues the trajectory (bias corrections depend on the count)."""
    from pylo_amd import ELO_CELO2_CUDA

    net = _celo2_net(5)
    shapes = [(32, 24), (24,)]
    gen = torch.Generator().manual_seed(1)
    init = [torch.randn(s, generator=gen) * 0.1 for s in shapes]
    grads = [[(torch.randn(s, generator=gen) * 0.05).cuda() for s in shapes] for _ in range(6)]

    def run(opt, params, ts):
        for t in ts:
            for p, g in zip(params, grads[t]):
                p.grad = g.clone()
            opt.step()

    a = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    oa = ELO_CELO2_CUDA(a, lr=1e-2, network=net, hf_key=None, capturable=True)
    run(oa, a, range(3))
    sd = copy.deepcopy(oa.state_dict())        # load_state_dict keeps same-device tensors by reference
    assert sd["param_groups"][0]["step"] == 3
    b = [torch.nn.Parameter(p.detach().clone()) for p in a]
    ob = ELO_CELO2_CUDA(b, lr=1e-2, network=net, hf_key=None, capturable=True)
    ob.load_state_dict(sd)
    c = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    oc = ELO_CELO2_CUDA(c, lr=1e-2, network=net, hf_key=None)          # host-side counters, 6 steps
    run(oc, c, range(6))
    run(oa, a, range(3, 6))
    run(ob, b, range(3, 6))
    _close(a, c, "device counters vs host counters")
    _close(b, c, "resumed")


def test_velo_step_replays_from_a_graph():
    """The time features (tanh embedding of step / num_steps), the loss EMAs and the LSTM state all
    advance on the device; the loss is read from a static device scalar."""
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(8)
    rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
    shapes = [(40, 24), (24,), (8, 3, 5, 5), (24, 56)]
    loss = torch.zeros((), device="cuda")
    losses = iter([2.0, 1.7, 1.5, 1.45, 1.2, 1.1])

    def make(params, capturable):
        return VeLO_CUDA(params, lr=1e-2, num_steps=20, weight_decay=0.01, rnn=rnn, mlp=mlp, capturable=capturable)

    def step(opt):
        # the reference optimizer steps first in every round and draws the loss; the capturable one reuses it
        if not opt.capturable:
            loss.fill_(next(losses))
        opt.step(loss)

    ref, cap, n = _graph_vs_eager(make, step, shapes)
    assert cap.state_dict()["param_groups"][0]["step"] == n == ref.param_groups[0]["step"]
    for a, b in zip(cap.lstm_hidden_state, ref.lstm_hidden_state):
        assert max_err(a.cpu(), b.cpu(), REL, ABS) <= 1.0


@pytest.mark.parametrize("which", ["adafac", "adafac max_grad_norm", "elo"])
def test_adafac_family_step_replays_from_a_graph(which):
    from pylo_amd import AdafacLO_CUDA, ELO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(9)
    net = MetaMLP(39, 32, 1)
    shapes = [(48, 40), (40,), (6, 4, 3, 3), (40, 72)]

    def make(params, capturable):
        if which.startswith("adafac"):      # with max_grad_norm every tensor is clipped against its own norm in the call
            return AdafacLO_CUDA(params, lr=0.5, weight_decay=0.01, network=net, hf_key=None, capturable=capturable,
                                 max_grad_norm=0.3 if "max_grad_norm" in which else None)
        return ELO_CUDA(params, lr=1e-2, weight_decay=0.01, clip_grad=True, clip_norm=0.5, network=net, hf_key=None,
                        capturable=capturable)

    ref, cap, n = _graph_vs_eager(make, lambda o: o.step(), shapes)
    cap.sync_step_counters()
    p0 = cap.param_groups[0]["params"][0]
    assert float(cap.state[p0]["step"]) == n == float(ref.state[ref.param_groups[0]["params"][0]]["step"])


@pytest.mark.parametrize("which", ["elo_celo2", "velo", "adafac"])
def test_learning_rate_change_between_replays(which):
    """A scheduler step between replays reaches the recorded step through the pinned tables."""
    from pylo_amd import AdafacLO_CUDA, ELO_CELO2_CUDA, VeLO_CUDA
    from pylo_amd.models import MetaMLP, VeLOMLP, VeLORNN

    torch.manual_seed(10)
    shapes = [(40, 24), (24,), (24, 56)]
    loss = torch.tensor(1.3, device="cuda")
    if which == "elo_celo2":
        net = _celo2_net(6)
        make = lambda ps, cap: ELO_CELO2_CUDA(ps, lr=1e-2, network=net, hf_key=None, capturable=cap)
        step = lambda o: o.step()
    elif which == "velo":
        rnn, mlp = VeLORNN(lstm_hidden_size=64, param_inits=32), VeLOMLP(param_inits=32)
        make = lambda ps, cap: VeLO_CUDA(ps, lr=1e-2, num_steps=20, rnn=rnn, mlp=mlp, capturable=cap)
        step = lambda o: o.step(loss)
    else:
        net = MetaMLP(39, 32, 1)
        make = lambda ps, cap: AdafacLO_CUDA(ps, lr=0.5, network=net, hf_key=None, capturable=cap)
        step = lambda o: o.step()
    gen = torch.Generator().manual_seed(2)
    init = [torch.randn(s, generator=gen) * 0.1 for s in shapes]
    grads = [[(torch.randn(s, generator=gen) * 0.05).cuda() for s in shapes] for _ in range(5)]
    ref_p = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cap_p = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    ref, cap = make(ref_p, False), make(cap_p, True)
    for p in cap_p:
        p.grad = torch.zeros_like(p)
    graph = None
    for t in range(5):
        for p, q, g in zip(ref_p, cap_p, grads[t]):
            p.grad = g.clone()
            q.grad.copy_(g)
        if t >= 3:                                   # the schedule: a third of the rate from step 3 on
            for o in (ref, cap):
                o.param_groups[0]["lr"] = o.defaults["lr"] / 3
            cap.refresh_graph_tables()
        step(ref)
        if t == 0:
            step(cap)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step(cap)
        else:
            graph.replay()
        torch.cuda.synchronize()
        _close(cap_p, ref_p, f"{which} step {t}")
