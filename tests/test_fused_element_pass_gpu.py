"""The fused element pass of ELO-CELO2 (``k_celo2_elem``: statistics, folding and apply items of all
tensors in one launch, slab by slab, with the folded weights handed from block to block while the kernel
runs) against the same passes as launches of their own (``PYLO_MI355_SLAB_ELEMS=0``) and against the oracle.

The slab parameters are read from the environment at plan creation, so the tests shrink them until small
tensors span many slabs, are cut into pieces (the path of a tensor too large to stay cached: streamed
statistics, apply items last to first) and until a tensor's apply items directly follow its statistics
items (depth 1: blocks that find the flag not yet raised and wait).
"""

import contextlib
import os

import pytest
import torch

from golden_io import max_err, step_keeping_raw

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6
SHAPES = [(256, 384), (384,), (640, 128), (128, 640), (37, 4099), (1024, 256), (96, 64), (64,), (512, 512),
          (3, 4, 5), (130, 128), (2048, 128)]


@contextlib.contextmanager
def _env(**kw):
    old = {k: os.environ.get(k) for k in kw}
    os.environ.update({k: str(v) for k, v in kw.items()})
    try:
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def _run(env, steps=3, seed=0, shapes=SHAPES):
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(1)
    net = CELO2MLP()
    gen = torch.Generator(device="cuda").manual_seed(seed)
    params = [torch.nn.Parameter(torch.randn(s, generator=gen, device="cuda") * 0.05) for s in shapes]
    with _env(**env):
        opt = ELO_CELO2_CUDA(params, lr=1e-3, weight_decay=0.1, adam_lr_mult=20.0, network=net, hf_key=None,
                             exp_mult=0.01)
        raws = []
        for t in range(steps):
            for i, p in enumerate(params):
                p.grad = torch.randn(p.shape, generator=gen, device="cuda") * 10.0 ** (-1 - i % 3)
            raws.append(step_keeping_raw(opt))
        names = opt._plan.launch_names()
    torch.cuda.synchronize()
    return params, opt, raws, names


@pytest.mark.parametrize("env", [
    {},                                                                                   # defaults
    {"PYLO_MI355_SLAB_ELEMS": 40000, "PYLO_MI355_KEEP_ELEMS": 10 ** 9},                   # many slabs
    {"PYLO_MI355_SLAB_ELEMS": 40000, "PYLO_MI355_KEEP_ELEMS": 100000},                    # pieces, reversed apply
    {"PYLO_MI355_SLAB_ELEMS": 40000, "PYLO_MI355_KEEP_ELEMS": 100000, "PYLO_MI355_SLAB_DEPTH": 1},
    {"PYLO_MI355_SLAB_ELEMS": 9000, "PYLO_MI355_KEEP_ELEMS": 20000, "PYLO_MI355_SLAB_DEPTH": 1},
    {"PYLO_MI355_SLAB_ELEMS": 10 ** 9, "PYLO_MI355_SLAB_DEPTH": 1},                       # one slab: every apply block may wait
    {"PYLO_MI355_SLAB_ELEMS": 40000, "PYLO_MI355_VALU_MLP": 1},                           # all-VALU kernels
])
def test_fused_pass_equals_separate_passes(env):
    ref_env = {"PYLO_MI355_SLAB_ELEMS": 0}
    if "PYLO_MI355_VALU_MLP" in env:           # same arithmetic on both sides
        ref_env["PYLO_MI355_VALU_MLP"] = env["PYLO_MI355_VALU_MLP"]
    ref_p, ref_opt, ref_raw, ref_names = _run(ref_env)
    got_p, got_opt, got_raw, names = _run(env)
    assert "k_celo2_elem" in names and "k_celo2_apply" in ref_names
    worst = 0.0
    for t in range(len(ref_raw)):
        for i, (a, b) in enumerate(zip(got_raw[t], ref_raw[t])):
            if a is None:
                assert b is None
                continue
            assert torch.isfinite(a).all(), (t, i)
            # the two differ in the order in which a tensor's rows of fp64 partial sums are added
            e = max_err(a, b, 1e-6, 1e-8)
            worst = max(worst, e)
            assert e <= 1.0, (env, t, i, SHAPES[i], e)
    for i, (a, b) in enumerate(zip(got_p, ref_p)):
        assert max_err(a, b, 1e-6, 1e-8) <= 1.0, (env, i)
        for k in ("mom", "rms", "fac_r", "fac_c"):
            if k in ref_opt.state[b]:
                assert torch.equal(got_opt.state[a][k], ref_opt.state[b][k]), (env, i, k)
    print("fused vs separate passes: worst err (rel 1e-6 / abs 1e-8 units)", worst)


def test_fused_pass_is_bit_reproducible_and_matches_oracle():
    from oracle import pylo_oracle as O
    from pylo_amd.models import CELO2MLP

    env = {"PYLO_MI355_SLAB_ELEMS": 30000, "PYLO_MI355_KEEP_ELEMS": 150000}
    p1, o1, raw1, _ = _run(env, steps=2, seed=5)
    p2, o2, raw2, _ = _run(env, steps=2, seed=5)
    for t in range(2):
        for a, b in zip(raw1[t], raw2[t]):
            assert (a is None and b is None) or torch.equal(a, b)
    for a, b in zip(p1, p2):
        assert torch.equal(a, b)
    # and the oracle on the same inputs
    torch.manual_seed(1)
    net = CELO2MLP()
    gen = torch.Generator(device="cuda").manual_seed(5)
    init = [torch.randn(s, generator=gen, device="cuda") * 0.05 for s in SHAPES]
    ref = [v.cpu().clone() for v in init]
    orc = O.EloCelo2Oracle(ref, net.state_dict(), lr=1e-3, weight_decay=0.1, adam_lr_mult=20.0, exp_mult=0.01)
    for t in range(2):
        grads = [torch.randn(p.shape, generator=gen, device="cuda") * 10.0 ** (-1 - i % 3) for i, p in enumerate(init)]
        orc.step([g.cpu() for g in grads])
    for i, (a, b) in enumerate(zip(p1, ref)):
        assert max_err(a, b, REL, ABS) <= 1.0, (i, SHAPES[i])


def test_tensor_without_gradient_neither_counts_nor_waits():
    """A tensor that sits a step out has no statistics blocks that count in and no apply blocks that wait."""
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(1)
    net = CELO2MLP()
    gen = torch.Generator(device="cuda").manual_seed(2)
    with _env(PYLO_MI355_SLAB_ELEMS=20000, PYLO_MI355_SLAB_DEPTH=1):
        params = [torch.nn.Parameter(torch.randn(s, generator=gen, device="cuda") * 0.05) for s in SHAPES[:6]]
        opt = ELO_CELO2_CUDA(params, lr=1e-3, network=net, hf_key=None)
        for t in range(4):
            before = [p.detach().clone() for p in params]
            for i, p in enumerate(params):
                p.grad = None if (t + i) % 3 == 0 else torch.randn(p.shape, generator=gen, device="cuda") * 0.01
            opt.step()
            torch.cuda.synchronize()
            for i, p in enumerate(params):
                assert torch.isfinite(p).all()
                assert torch.equal(p, before[i]) == ((t + i) % 3 == 0), (t, i)
