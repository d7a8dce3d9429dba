"""GPU parity of CELO2_CUDA (HIP, through the C ABI): the ELO-CELO2 kernels with the independent-moment
AdamW branch of pylo/optim/CELO2_cuda.py:234-253, against the golden trajectories of the reference's
CELO2_naive and against the CPU oracle.

Tolerance: rel 1e-5 / abs 1e-6 (``max_err <= 1``) on parameters and every state after every step.
"""

import copy

import pytest
import torch

from golden_io import step_keeping_raw, Golden, max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6


@pytest.mark.parametrize("name", ["celo2_small", "celo2_small_defaults"])
def test_full_step_matches_reference_golden(name):
    from pylo_amd import CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    G = Golden(name)
    shapes = G.shapes
    net = CELO2MLP()
    net.load_state_dict(G.state_dict("net"))
    gpu = [torch.nn.Parameter(G.t(f"init/{i}").cuda()) for i in range(len(shapes))]
    cfg = dict(G.meta["cfg"])
    if "adam_betas" in cfg:
        cfg["adam_betas"] = tuple(cfg["adam_betas"])
    opt = CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
    worst = 0.0
    for t in range(G.meta["n_steps"]):
        for i, p in enumerate(gpu):
            p.grad = G.t(f"grad{t}/{i}").cuda()
        opt.step()
        for i, p in enumerate(gpu):
            keys = ["param"] + (["mom", "rms", "fac_r", "fac_c"] if p.dim() >= 2 else ["exp_avg", "exp_avg_sq"])
            for k in keys:
                got = p if k == "param" else opt.state[p][k]
                e = max_err(got, G.t(f"step{t}/{k}/{i}"), REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (name, t, i, k, e)
            if p.dim() <= 1:
                assert opt.state[p]["adam_step"] == t + 1
                assert set(opt.state[p].keys()) == {"exp_avg", "exp_avg_sq", "adam_step"}
    print(name, "worst err/tol", worst)


def test_adam_branch_matches_oracle_with_embedding_missing_grad_and_clipping():
    """Non-default AdamW decays and eps, an is_embedding group, global-norm clipping plus the value
    clamp, a parameter that skips every other step (its adam_step counter must lag), wide 1-D tensors
    on the vector path; accumulators, raw steps and AdamW parameters every step."""
    from oracle import pylo_oracle as O
    from pylo_amd import CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(3)
    net = CELO2MLP()
    shapes = [(48, 40), (4099,), (64, 16), (16,), (70, 384), (1,), (12288,)]
    emb = [False, False, True, False, False, False, False]
    gen = torch.Generator().manual_seed(21)
    init = [torch.randn(s, generator=gen) for s in shapes]
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    betas, eps = (0.8, 0.97), 1e-6
    cfg = dict(lr=1e-2, weight_decay=0.05, adam_weight_decay=0.02, adam_lr_mult=3.0, clip_grad=True,
               clip_norm=5.0, grad_clip_val=2.0)
    orc = O.EloCelo2Oracle(cpu, net.state_dict(), is_embedding=emb, independent_adam=(*betas, eps), **cfg)
    plain = [p for p, e in zip(gpu, emb) if not e]
    embp = [p for p, e in zip(gpu, emb) if e]
    opt = CELO2_CUDA([{"params": plain}, {"params": embp, "is_embedding": True}], network=net, hf_key=None,
                     adam_betas=betas, adam_eps=eps, **cfg)
    order = [i for i, e in enumerate(emb) if not e] + [i for i, e in enumerate(emb) if e]
    for t in range(6):
        grads = [torch.randn(s, generator=gen) * 1.5 for s in shapes]
        if t % 2 == 1:
            grads[3] = None
        raw = {}
        for p, g in zip(gpu, grads):
            p.grad = None if g is None else g.cuda()
        orc.step(grads, keep_raw=raw)
        kept = step_keeping_raw(opt)
        for i, p in enumerate(gpu):
            st, ost = opt.state[p], orc.state[i]
            adam = p.dim() <= 1 or emb[i]
            for k in (("exp_avg", "exp_avg_sq") if adam else ("mom", "rms", "fac_r", "fac_c")):
                e = max_err(st[k], ost[k], REL, ABS)
                assert e <= 1.0, (t, i, k, e)
            if adam:
                assert st["adam_step"] == ost["adam_step"], (t, i)
                e = max_err(p, cpu[i], REL, ABS)
                assert e <= 1.0, ("adam param", t, i, e)
        assert opt.state[gpu[3]]["adam_step"] == (t + 2) // 2
        for i, r in raw.items():
            assert max_err(kept[order.index(i)], r, REL, ABS) <= 1.0, ("raw", t, i)
        for pc, pg in zip(cpu, gpu):
            pg.data.copy_(pc)


def test_cached_argument_rows_keep_the_per_parameter_counter():
    """Steps after the first reuse cached argument rows; the bias corrections must still follow each
    parameter's own adam_step, also after a state_dict round trip (tests/test_celo2.py:122-167)."""
    from pylo_amd import CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(5)
    net = CELO2MLP()
    shapes = [(32, 24), (24,), (24, 8), (300,)]
    gen = torch.Generator().manual_seed(2)
    init = [torch.randn(s, generator=gen) for s in shapes]
    grads = [[torch.randn(s, generator=gen).cuda() for s in shapes] for _ in range(8)]

    def run(params, opt, ts):
        for t in ts:
            for p, g in zip(params, grads[t]):
                p.grad = g.clone()
            opt.step()

    a = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    oa = CELO2_CUDA(a, lr=1e-2, network=net, hf_key=None)
    run(a, oa, range(4))
    assert oa._fast is not None                      # the cached path was in use
    sd = copy.deepcopy(oa.state_dict())
    snap = [p.detach().clone() for p in a]
    run(a, oa, range(4, 8))
    b = [torch.nn.Parameter(v.clone()) for v in snap]
    ob = CELO2_CUDA(b, lr=1e-2, network=net, hf_key=None)
    ob.load_state_dict(sd)
    run(b, ob, range(4, 8))
    for x, y in zip(a, b):
        assert torch.max(torch.abs(x - y)).item() < 1e-5
    assert oa.state[a[1]]["adam_step"] == 8 and ob.state[b[1]]["adam_step"] == 8

    # the same eight steps without the cache (dropped before every step) give the same parameters
    c = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    oc = CELO2_CUDA(c, lr=1e-2, network=net, hf_key=None)
    for t in range(8):
        oc._fast = None
        run(c, oc, [t])
    for x, y in zip(a, c):
        assert torch.equal(x, y)
