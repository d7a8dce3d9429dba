"""GPU parity of the fused ELO-CELO2 step (HIP, through the C ABI) against the CPU oracle and the
golden trajectories of the reference's naive class.

Tolerance everywhere: rel 1e-5 / abs 1e-6 (``max_err <= 1``), on parameters and on every
optimizer state after every step.  Modelled on the reference's own CUDA-vs-naive harness
(tests/test_celo2_cuda.py:41-71).
"""

import copy

import pytest
import torch

from golden_io import step_keeping_raw, Golden, max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6


def _mk(shapes, seed, std=1.0):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randn(s, generator=gen) * std for s in shapes], gen


def _net(seed=1):
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(seed)
    return CELO2MLP()


def _pair(shapes, init, net, cfg, is_embedding=None):
    """(oracle, hip optimizer, cpu params, gpu params) fed identical inputs."""
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA

    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    emb = is_embedding or [False] * len(shapes)
    ocfg = dict(cfg)
    ocfg.setdefault("adam_lr_mult", 20.0)
    orc = O.EloCelo2Oracle(cpu, net.state_dict(), is_embedding=emb, **ocfg)
    plain = [p for p, e in zip(gpu, emb) if not e]
    embp = [p for p, e in zip(gpu, emb) if e]
    groups = [{"params": plain}] + ([{"params": embp, "is_embedding": True}] if embp else [])
    opt = ELO_CELO2_CUDA(groups, network=net, hf_key=None, **cfg)
    return orc, opt, cpu, gpu


def _check_states(opt, orc, gpu, t, tag=""):
    for i, p in enumerate(gpu):
        st = opt.state[p]
        for k in ("mom", "rms", "fac_r", "fac_c"):
            if k in orc.state[i] and k in st and not (orc.is_embedding[i] and k.startswith("fac")):
                e = max_err(st[k], orc.state[i][k], REL, ABS)
                assert e <= 1.0, (tag, t, i, k, e)


@pytest.mark.parametrize("shapes,gscale,cfg", [
    ([(64, 32), (32, 64), (32,), (48, 24)], 3.0, dict(lr=1e-2)),                       # clip active
    ([(64, 32), (32, 64), (32,), (24, 24)], 1e-3, dict(lr=1e-3, exp_mult=0.01)),       # clip inactive, exp
    ([(40, 56), (7,)], 0.5, dict(lr=1e-2, clip_grad=False, adam_lr_mult=1.0)),
    ([(37, 4099), (4099, 37), (5, 3), (1, 9), (1,), (130, 1)], 0.1, dict(lr=1e-3)),    # dword path, ragged
    ([(256, 1028), (1028, 256), (300, 260)], 2.0, dict(lr=1e-3)),                      # several tiles
    # column-resident walk (row length a multiple of 128): ragged row ranges, a single row, a
    # task count that does not fill the last block, next to narrow tensors on the chunked path
    ([(70, 384), (33, 128), (1, 128), (2100, 256), (300,), (64, 130)], 1.0, dict(lr=1e-3, exp_mult=0.01)),
])
def test_fused_kernel_matches_oracle_per_step(shapes, gscale, cfg):
    """Raw step (what celo2_kernel.cu writes to step_out) and all accumulators, every step, with
    the parameters re-synchronised from the oracle so only the fused kernels are compared."""
    net = _net()
    init, gen = _mk(shapes, 5)
    orc, opt, cpu, gpu = _pair(shapes, init, net, cfg)
    for t in range(6):
        grads = [torch.randn(s, generator=gen) * gscale for s in shapes]
        raw = {}
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        orc.step(grads, keep_raw=raw)
        kept = step_keeping_raw(opt)
        torch.cuda.synchronize()
        _check_states(opt, orc, gpu, t)
        for i, r in raw.items():
            e = max_err(kept[i], r, REL, ABS)
            assert e <= 1.0, ("raw step", t, i, shapes[i], e)
        for i, (pc, pg) in enumerate(zip(cpu, gpu)):
            if pc.dim() <= 1:
                assert max_err(pg, pc, REL, ABS) <= 1.0, ("adam param", t, i)
            pg.data.copy_(pc)


@pytest.mark.parametrize("name", ["elo_celo2_small_clip", "elo_celo2_small_noclip_exp",
                                  "elo_celo2_small_noortho", "elo_celo2_nd", "elo_celo2_mlp1d"])
def test_full_step_matches_reference_golden(name):
    """Whole step() trajectories (NS, normalise, apply included) against the reference's naive class."""
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    G = Golden(name)
    shapes = G.shapes
    net = CELO2MLP()
    net.load_state_dict(G.state_dict("net"))
    gpu = [torch.nn.Parameter(G.t(f"init/{i}").cuda()) for i in range(len(shapes))]
    cfg = dict(G.meta["cfg"])
    cfg.setdefault("adam_lr_mult", 1.0)          # the naive class's default
    opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
    worst = 0.0
    for t in range(G.meta["n_steps"]):
        for i, p in enumerate(gpu):
            p.grad = G.t(f"grad{t}/{i}").cuda()
        opt.step()
        for i, p in enumerate(gpu):
            keys = ["param", "mom", "rms"] + (["fac_r", "fac_c"] if p.dim() >= 2 else [])
            if p.dim() < 2 and not cfg.get("use_adamw_for_1d", True):
                keys.append("fac_v")          # the MLP on a 1-D tensor keeps a per-element accumulator
            for k in keys:
                got = p if k == "param" else opt.state[p][k]
                e = max_err(got, G.t(f"step{t}/{k}/{i}"), REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (name, t, i, k, e)
    print(name, "worst err/tol", worst)


@pytest.mark.parametrize("adam_1d", [True, False])
def test_tensors_with_more_than_two_dims_and_mlp_on_1d(adam_1d):
    """Per-slice normalisers (last two dims) on N-D tensors: short slices walked by one lane (3x3, 5x5),
    long ones by a wave (4x70, 40x33), next to 2-D tensors on the ordinary passes; with
    use_adamw_for_1d=False the 1-D tensors take the MLP with their per-element accumulator.  Raw steps,
    accumulators and whole-step parameters against the oracle, clipping active."""
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA

    shapes = [(32, 16, 3, 3), (8, 4, 70), (3, 40, 33), (5, 5, 5, 5), (300,), (64, 32), (2, 1, 7), (1,), (40, 128),
              (2, 3, 4, 2, 3)]
    net = _net(5)
    init, gen = _mk(shapes, 17)
    cfg = dict(lr=1e-2, exp_mult=0.01, clip_norm=4.0, use_adamw_for_1d=adam_1d, adam_lr_mult=2.0)
    cpu = [v.clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    orc = O.EloCelo2Oracle(cpu, net.state_dict(), **cfg)
    opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
    worst = 0.0
    for t in range(5):
        grads = [torch.randn(s, generator=gen) * (0.3 if i % 2 else 3.0) for i, s in enumerate(shapes)]
        if t == 3:
            grads[1] = None
        raw = {}
        for p, g in zip(gpu, grads):
            p.grad = None if g is None else g.cuda()
        orc.step(grads, keep_raw=raw)
        kept = step_keeping_raw(opt)
        for i, r in raw.items():
            e = max_err(kept[i], r, REL, ABS)
            worst = max(worst, e)
            assert e <= 1.0, ("raw step", adam_1d, t, i, shapes[i], e)
        for i, p in enumerate(gpu):
            for k, v in orc.state[i].items():
                if k in opt.state[p]:
                    e = max_err(opt.state[p][k], v, REL, ABS)
                    assert e <= 1.0, (adam_1d, t, i, k, e)
            e = max_err(p, cpu[i], REL, ABS)
            assert e <= 1.0, ("param", adam_1d, t, i, shapes[i], e)
            p.data.copy_(cpu[i])
        assert ("fac_v" in opt.state[gpu[4]]) == (not adam_1d)
    print("nd / 1-d mlp worst raw err/tol", worst)


def test_config1_trajectory():
    """BASELINE config 1: 1024x1024 weight + 1024 bias, 10 steps, params and states every step,
    against the golden samples of the reference's naive class."""
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    G = Golden("elo_celo2_cfg1")
    meta = G.meta
    shapes = G.shapes
    net = CELO2MLP()
    net.load_state_dict(G.state_dict("net"))
    gen = torch.Generator().manual_seed(meta["seed"])
    init = [torch.randn(s, generator=gen) * meta["init_std"] for s in shapes]
    gpu = [torch.nn.Parameter(v.cuda()) for v in init]
    opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **meta["cfg"])
    worst = 0.0
    for t in range(meta["n_steps"]):
        for p, s in zip(gpu, shapes):
            p.grad = (torch.randn(s, generator=gen) * meta["grad_scale"]).cuda()
        opt.step()
        for i, p in enumerate(gpu):
            keys = ["param", "mom", "rms"] + (["fac_r", "fac_c"] if p.dim() >= 2 else [])
            for k in keys:
                got = p if k == "param" else opt.state[p][k]
                e = max_err(got.reshape(-1)[::meta["sample"]].cpu(), G.t(f"step{t}/{k}/{i}/sample"), REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (t, i, k, e)
    print("cfg1 worst err/tol", worst)


def test_clamp_fallback_and_embedding_group_and_missing_grad():
    """|g| > grad_clip_val with global-norm clipping on (exact re-reduction pass), an is_embedding
    group routed to AdamW, and a parameter without gradient."""
    shapes = [(48, 40), (40, 48), (64, 16), (16,), (12, 20)]
    emb = [False, False, True, False, False]
    net = _net(3)
    init, gen = _mk(shapes, 9)
    cfg = dict(lr=1e-2, grad_clip_val=2.0, clip_norm=1000.0)
    orc, opt, cpu, gpu = _pair(shapes, init, net, cfg, is_embedding=emb)
    order = [0, 1, 3, 4, 2]   # param order inside the HIP optimizer: plain group, then embedding group
    for t in range(4):
        grads = [torch.randn(s, generator=gen) * 30.0 for s in shapes]
        grads[4] = None if t % 2 == 1 else grads[4]
        raw = {}
        for p, g in zip(gpu, grads):
            p.grad = None if g is None else g.cuda()
        orc.step(grads, keep_raw=raw)
        kept = step_keeping_raw(opt)
        _check_states(opt, orc, [gpu[i] for i in range(len(gpu))], t, "fallback")
        for i, r in raw.items():
            assert max_err(kept[order.index(i)], r, REL, ABS) <= 1.0, ("raw", t, i)
        for i, (pc, pg) in enumerate(zip(cpu, gpu)):
            if pc.dim() <= 1 or emb[i]:
                assert max_err(pg, pc, REL, ABS) <= 1.0, ("adam", t, i)
            pg.data.copy_(pc)


def test_state_dict_resume():
    """state_dict -> load_state_dict reproduces the continuation (tests/test_celo2.py:122-167)."""
    from pylo_amd import ELO_CELO2_CUDA

    shapes = [(32, 24), (24,), (24, 8)]
    net = _net(7)
    init, gen = _mk(shapes, 11)
    grads = [[torch.randn(s, generator=gen).cuda() for s in shapes] for _ in range(8)]

    def run(params, opt, ts):
        for t in ts:
            for p, g in zip(params, grads[t]):
                p.grad = g.clone()
            opt.step()

    a = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    oa = ELO_CELO2_CUDA(a, lr=1e-2, network=net, hf_key=None)
    run(a, oa, range(4))
    sd = copy.deepcopy(oa.state_dict())   # the reference test serialises to disk here
    snap = [p.detach().clone() for p in a]
    run(a, oa, range(4, 8))
    b = [torch.nn.Parameter(v.clone()) for v in snap]
    ob = ELO_CELO2_CUDA(b, lr=1e-2, network=net, hf_key=None)
    ob.load_state_dict(sd)
    run(b, ob, range(4, 8))
    for x, y in zip(a, b):
        assert torch.max(torch.abs(x - y)).item() < 1e-5
    assert set(oa.state[a[0]].keys()) == {"mom", "rms", "fac_r", "fac_c"}
    assert oa.state[a[0]]["mom"].shape == (3, 32, 24) and oa.state[a[0]]["fac_r"].shape == (3, 1, 24)
    assert set(oa.state[a[1]].keys()) == {"mom", "rms"}


def test_runs_on_the_callers_stream():
    """The library enqueues on torch's current stream (the reference launches on the legacy default
    stream): stepping under a side stream gives bit-identical parameters, and work queued on that stream
    before the step is ordered before it."""
    from pylo_amd import ELO_CELO2_CUDA

    shapes = [(70, 384), (48, 40), (40,)]
    net = _net(2)
    init, gen = _mk(shapes, 4)
    grads = [[torch.randn(s, generator=gen) for s in shapes] for _ in range(3)]

    def run(stream):
        ps = [torch.nn.Parameter(v.clone().cuda()) for v in init]
        opt = ELO_CELO2_CUDA(ps, lr=1e-2, network=net, hf_key=None)
        gs = [[g.cuda() for g in step] for step in grads]
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            for t in range(3):
                for p, g in zip(ps, gs[t]):
                    p.grad = g * 1.0          # produced on the same stream right before the step
                opt.step()
        stream.synchronize()
        return [p.detach().clone() for p in ps]

    a = run(torch.cuda.current_stream())
    b = run(torch.cuda.Stream())
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_replaced_state_tensor_is_picked_up():
    """The step caches its argument table between calls; a state tensor swapped for a copy (what a
    user-side checkpoint restore or a dtype/device round trip does) must be the one updated from then
    on, with the trajectory unchanged."""
    from pylo_amd import ELO_CELO2_CUDA

    shapes = [(40, 24), (24,), (24, 8)]
    net = _net(3)
    init, gen = _mk(shapes, 9)
    grads = [[torch.randn(s, generator=gen).cuda() for s in shapes] for _ in range(6)]

    def run(swap):
        ps = [torch.nn.Parameter(v.clone().cuda()) for v in init]
        opt = ELO_CELO2_CUDA(ps, lr=1e-2, network=net, hf_key=None)
        for t in range(6):
            for p, g in zip(ps, grads[t]):
                p.grad = g.clone()
            opt.step()
            if swap and t == 2:
                for p in ps:
                    for k, v in list(opt.state[p].items()):
                        if torch.is_tensor(v):
                            opt.state[p][k] = v.clone()
                            v.fill_(float("nan"))      # the old storage must not be read again
        return ps, opt

    a, _ = run(False)
    b, ob = run(True)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    assert all(bool(torch.isfinite(v).all()) for p in b for v in ob.state[p].values() if torch.is_tensor(v))


def test_replaced_state_tensors_are_noticed():
    """The step caches device pointers of the state tensors between calls; a state tensor swapped for another
    object (any of them, not only the first) must be picked up by the next step, which then updates the new
    tensor and leaves the orphaned one alone."""
    net = _net()
    shapes = [(64, 32), (32,), (48, 24)]
    init, gen = _mk(shapes, 9)
    orc, opt, cpu, gpu = _pair(shapes, init, net, dict(lr=1e-2))
    for t in range(4):
        grads = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        orphans = []
        if t == 2:      # after two steps on the fast path
            for p in gpu:
                st = opt.state[p]
                for k in ("rms", "fac_c") if "fac_c" in st else ("rms",):
                    orphans.append((st[k], st[k].clone()))
                    st[k] = st[k].clone()
        orc.step(grads)
        opt.step()
        torch.cuda.synchronize()
        _check_states(opt, orc, gpu, t, "after swap" if t >= 2 else "")
        for old, before in orphans:
            assert torch.equal(old, before)
        for pc, pg in zip(cpu, gpu):
            assert max_err(pg, pc, REL, ABS) <= 1.0, t
