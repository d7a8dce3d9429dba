"""The library's own Newton-Schulz kernels (``pylo_mi355_celo2_orthogonalize_finish``: symmetric products on
tiles on and above the diagonal, split Gram product of very tall matrices, scalings folded into the first
iteration) against the oracle's literal formula (pylo/optim/CELO2_naive.py:59-73) evaluated in fp64, through
whole optimizer steps.  The orthogonalised, normalised step is recovered from the parameter update,
``p_new = p_old - lr (s + wd p_old)``, and held to 2e-4 of its RMS (the library's fp32 products sit at
2e-5 .. 5e-5, the same as the batched torch products they replace); parameters at rel 1e-5 / abs 1e-6.
"""

import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

LR, WD = 1e-2, 0.1


def _run(shapes, steps=2, seed=0, **kw):
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(1)
    net = CELO2MLP()
    gen = torch.Generator(device="cuda").manual_seed(seed)
    init = [torch.randn(s, generator=gen, device="cuda") * 0.05 for s in shapes]
    ref = [v.double() for v in init]
    gpu = [torch.nn.Parameter(v.clone()) for v in init]
    cfg = dict(lr=LR, weight_decay=WD, adam_lr_mult=20.0)
    cfg.update(kw)
    orc = O.EloCelo2Oracle(ref, net.state_dict(), device="cuda", **cfg).double_()
    opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
    worst = 0.0
    for t in range(steps):
        before = [(p.detach().clone(), r.clone()) for p, r in zip(gpu, ref)]
        grads = [torch.randn(s, generator=gen, device="cuda") * 10.0 ** (-1 - i % 3) for i, s in enumerate(shapes)]
        for p, g in zip(gpu, grads):
            p.grad = g
        orc.step([g.double() for g in grads])
        opt.step()
        torch.cuda.synchronize()
        for i, p in enumerate(gpu):
            assert torch.isfinite(p).all(), (t, i, shapes[i])
            assert max_err(p, ref[i], 1e-5, 1e-6) <= 1.0, (t, i, shapes[i])
            if p.dim() == 2:
                got = (before[i][0].double() - p.detach().double()) / LR - WD * before[i][0].double()
                want = (before[i][1] - ref[i]) / LR - WD * before[i][1]
                rms = float(want.pow(2).mean().sqrt())
                quant = float(before[i][0].abs().max()) * 2.0 ** -23 / LR     # fp32 parameters quantise the recovered step
                e = float((got - want).abs().max()) / rms
                worst = max(worst, e)
                assert e <= 2e-4 + 2 * quant / rms, (t, i, shapes[i], e)
    return opt, worst


@pytest.mark.parametrize("pipe", ["fp16x2", "fp32"])
def test_library_kernels_take_these_shapes(pipe, monkeypatch):
    if pipe == "fp32":
        monkeypatch.setenv("PYLO_MI355_NS_F32", "1")
    shapes = [(256, 384), (384, 256), (128, 128), (132, 260), (260, 132), (4, 8), (8, 4), (36, 36), (1, 64), (64, 1),
              (130, 6), (6, 130), (10, 12), (12, 10), (9, 16), (16, 9), (37, 131), (131, 37), (1, 1), (3, 5)]
    opt, _ = _run(shapes, steps=2)
    if pipe == "fp16x2":
        # the split-fp16 kernels take any two dims
        assert all(opt._ns_ok), opt._ns_ok
        return
    # fp32 kernels: the last dim and the smaller dim must be multiples of 4; everything else goes through torch
    for s, got in zip(shapes, opt._ns_ok):
        r, c = s
        assert got == (c % 4 == 0 and min(r, c) % 4 == 0), s
    assert opt._ns_ok[:8] == [True] * 8 and not any(opt._ns_ok[8:])


@pytest.mark.parametrize("shapes", [
    [(256, 384), (384, 256), (128, 128), (768,)],                       # whole tiles
    [(132, 260), (260, 132), (4, 8), (8, 4), (36, 36), (200, 4)],        # ragged tiles, a single MFMA column
    [(8201, 128), (128, 8200), (16385, 64)],                             # split Gram product, odd reduction length
    [(130, 6), (6, 130), (9, 16), (64, 64)],                             # dims that are not multiples of 4 (fp32 kernels: torch)
    [(37, 4099), (4099, 37), (255, 257), (129, 129), (1, 300), (300, 1), (2, 3)],   # odd dims, single rows and columns
    [(300, 260), (300, 260), (300, 260), (64,)],                         # a bucket of equal shapes
])
@pytest.mark.parametrize("pipe", ["fp16x2", "fp16x2-literal", "fp16x2-chains-3,2", "fp32"])
def test_library_newton_schulz_matches_oracle(shapes, pipe, monkeypatch):
    """The sets of product kernels: the default (operands split into two scaled fp16 planes, three fp16 matrix
    products per fp32 product, two iterations sharing one Gram product and one update), the same with one Gram product and
    one update per iteration (PYLO_MI355_NS_PAIRS=0), with a chain of three iterations and one of two
    (PYLO_MI355_NS_CHAINS="3,2"), and the fp32 matrix instructions (PYLO_MI355_NS_F32=1, read at plan creation)."""
    if pipe == "fp32":
        monkeypatch.setenv("PYLO_MI355_NS_F32", "1")
    if pipe == "fp16x2-literal":
        monkeypatch.setenv("PYLO_MI355_NS_PAIRS", "0")
    if pipe.startswith("fp16x2-chains-"):
        monkeypatch.setenv("PYLO_MI355_NS_CHAINS", pipe.rsplit("-", 1)[1])   # three iterations, then two, per Gram product
    _, worst = _run(shapes, steps=2, seed=len(shapes))
    print("orthogonalised step err / rms", worst)


@pytest.mark.parametrize("iters", [0, 1, 2, 4])
@pytest.mark.parametrize("pipe", ["fp16x2", "fp32"])
def test_iteration_counts_and_result_buffer(iters, pipe, monkeypatch):
    """fp32 kernels: an even number of iterations leaves the result in the raw-step buffer, an odd one in the
    workspace; split-fp16 kernels: the last update writes fp32 over the raw step whatever the count."""
    if pipe == "fp32":
        monkeypatch.setenv("PYLO_MI355_NS_F32", "1")
    _run([(256, 384), (384, 256), (132, 260)], steps=2, ns_iters=iters)


def _orthogonalise_direct(mats, iters=5, coeffs=(3.4445, -4.775, 2.0315)):
    """rms_normalize(newton_schulz(x)) of every matrix through the finishing call alone: p = 0, lr = -1."""
    import numpy as np

    from pylo_amd import _lib

    shapes = [tuple(x.shape) for x in mats]
    plan = _lib.Plan(_lib.KIND_CELO2, shapes, [0] * len(shapes), torch.device("cuda:0"))
    steps = [x.clone().contiguous() for x in mats]
    params = [torch.zeros_like(x) for x in mats]
    fin = np.zeros(len(mats), dtype=_lib.ARGS_DTYPE)
    for i in range(len(mats)):
        fin["grad"][i], fin["param"][i], fin["step_out"][i] = 1, params[i].data_ptr(), steps[i].data_ptr()
        fin["lr"][i], fin["weight_decay"][i], fin["step_mult"][i] = -1.0, 0.0, 1.0
        fin["flags"][i] = _lib.ARG_ORTHOGONALIZE
    plan.celo2_orthogonalize_finish(fin, coeffs, iters, 1e-8, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    plan.close()
    return params


def _reference_direct(x, iters=5, dtype=torch.float64, coeffs=(3.4445, -4.775, 2.0315)):
    """The literal formula (pylo/optim/CELO2_naive.py:59-73) and the RMS normaliser, in fp64 or, as the reference
    runs it, in fp32 torch products."""
    c0, c1, c2 = coeffs
    x = x.to(dtype)
    t = x.shape[0] > x.shape[1]
    if t:
        x = x.T
    x = x / (x.norm() + 1e-8)
    for _ in range(iters):
        a = x @ x.T
        x = c0 * x + (c1 * a + c2 * (a @ a)) @ x
    if t:
        x = x.T
    return x * torch.rsqrt(1e-9 + (x * x).mean())


@pytest.mark.parametrize("chains,floor", [("2,2,1", 5e-5), ("1,1,1,1,1", 5e-5), ("3,2", 2e-4)])
def test_spectra_with_a_dominant_direction(chains, floor, monkeypatch):
    """Matrices whose singular values span several decades (one dominant direction over a flat or a decaying
    rest): where a Gram matrix loses its small eigenvalues to rounding and five iterations amplify what the first
    ones round off.  On such input the formula in fp32 torch products -- what the reference runs -- is itself
    1e-4 .. 5e-3 of the result's RMS away from its fp64 evaluation; the library's kernels, with two iterations
    sharing one Gram product (the default, PYLO_MI355_NS_CHAINS="2,2,1") or with one Gram product per iteration,
    must be no further away than 1.5 times that (plus 5e-5, the level of well-conditioned inputs).  Three iterations
    in the first chain (the faster, opt-in "3,2") pay up to 1e-4 on a dominant direction over a flat rest of equal
    weight: held to 2e-4 here."""
    monkeypatch.setenv("PYLO_MI355_NS_CHAINS", chains)
    pairs = chains
    gen = torch.Generator(device="cuda").manual_seed(5)
    rnd = lambda *s: torch.randn(*s, generator=gen, device="cuda")
    mats = []
    for (r, c), rest in (((256, 384), 5e-3), ((384, 256), 5e-3), ((768, 768), 1e-3), ((130, 1000), 1e-4),
                         ((256, 2048), 3e-2), ((256, 384), 1.0), ((768, 3072), 1.0), ((130, 1000), 1.0),
                         ((384, 256), 0.3)):
        u, v = rnd(r, 1), rnd(1, c)
        mats.append(u @ v / (u.norm() * v.norm()) + rest * rnd(r, c) / (r * c) ** 0.5)
    q1, _ = torch.linalg.qr(rnd(256, 256))
    q2, _ = torch.linalg.qr(rnd(512, 256))
    mats.append((q1 * torch.logspace(0, -4, 256, device="cuda")) @ q2.T)     # singular values 1 .. 1e-4
    mats.append(rnd(768, 768))
    got = _orthogonalise_direct(mats)
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    rows = []
    try:
        for x, y in zip(mats, got):
            want = _reference_direct(x)
            e = float((y.double() - want).abs().max())       # the result has unit RMS
            e32 = float((_reference_direct(x, dtype=torch.float32).double() - want).abs().max())
            rows.append((tuple(x.shape), e, e32))
            assert e <= 1.5 * e32 + floor, rows[-1]
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    print("chains", pairs, "(shape, library error / rms, fp32 torch formula error / rms):", rows)


@pytest.mark.parametrize("coeffs,iters", [((1.5, -0.5, 0.0), 8), ((1.875, -1.25, 0.375), 6), ((3.0, -3.2, 1.2), 5),
                                          ((3.4445, -4.775, 2.0315), 9), ((2.0, -1.0, 0.0), 3), ((0.5, 0.0, 0.0), 4)])
def test_other_coefficients_and_iteration_counts(coeffs, iters):
    """The operand planes are fp16 numbers scaled by powers of two that the library derives from the coefficients
    (bounds on the singular values of everything the iteration forms): other polynomials than the reference's
    default -- the cubic and quintic Newton-Schulz iterations, one that overshoots (sigma up to 1.09 for 2 - x),
    one that only shrinks -- and other iteration counts must come out as close to the fp64 formula as the
    reference's fp32 torch products do (1.5 times their error plus the level of well-conditioned inputs).  Where
    the polynomial does not amplify rounding the library's 23-bit operands show: 3 .. 12 times the fp32 formula's
    error, 1e-5 of the result's RMS at most."""
    gen = torch.Generator(device="cuda").manual_seed(17)
    rnd = lambda *s: torch.randn(*s, generator=gen, device="cuda")
    u, v = rnd(300, 1), rnd(1, 520)
    mats = [rnd(256, 384), rnd(384, 256), rnd(130, 1000), rnd(768, 768), rnd(1, 700), rnd(64, 64),
            u @ v / (u.norm() * v.norm()) + 0.05 * rnd(300, 520) / (300 * 520) ** 0.5]
    got = _orthogonalise_direct(mats, iters=iters, coeffs=coeffs)
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    rows = []
    try:
        for x, y in zip(mats, got):
            want = _reference_direct(x, iters=iters, coeffs=coeffs)
            assert torch.isfinite(y).all(), tuple(x.shape)
            e = float((y.double() - want).abs().max())
            e32 = float((_reference_direct(x, iters=iters, dtype=torch.float32, coeffs=coeffs).double() - want).abs().max())
            rows.append((tuple(x.shape), e, e32))
            assert e <= 1.5 * e32 + 5e-5, rows[-1]
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    print("coefficients", coeffs, "iterations", iters, "(shape, library error / rms, fp32 torch formula error / rms):", rows)


def test_a_nan_stays_a_nan_and_stays_in_its_matrix():
    """A NaN in one raw step makes that matrix's result NaN, as the formula does (its norm is NaN), instead of being
    clamped into the fp16 planes' range as a finite number; the other matrices of the call are what they are
    without it."""
    gen = torch.Generator(device="cuda").manual_seed(23)
    mats = [torch.randn(s, generator=gen, device="cuda") for s in ((256, 384), (130, 260), (384, 128))]
    clean = _orthogonalise_direct(mats)
    mats[1][3, 5] = float("nan")
    got = _orthogonalise_direct(mats)
    assert torch.isnan(got[1]).all()
    assert torch.equal(got[0], clean[0]) and torch.equal(got[2], clean[2])
    assert torch.isfinite(clean[1]).all()


def test_chain_length_chosen_per_matrix(monkeypatch):
    """PYLO_MI355_NS_ADAPTIVE=1: the first chain takes three iterations for the matrices whose A = X X^T has
    ||A||_F^2 <= (16 / 196)^2 (no direction holds more than 8 % of the step's squared norm: what three chained
    iterations add to the error is then no more than what a pair adds on any matrix) and two for the others.  The
    choice is made on the device, matrix by matrix; each result is bit-identical to that of the fixed schedule
    it amounts to, "3,2" or "2,2,1"."""
    gen = torch.Generator(device="cuda").manual_seed(5)
    rnd = lambda *s: torch.randn(*s, generator=gen, device="cuda")

    def dominant(r, c, rest):
        u, v = rnd(r, 1), rnd(1, c)
        return u @ v / (u.norm() * v.norm()) + rest * rnd(r, c) / (r * c) ** 0.5

    mats = [rnd(768, 3072), dominant(256, 384, 1.0), rnd(768, 768), dominant(130, 1000, 1.0), rnd(64, 64), rnd(8300, 160),
            dominant(8300, 160, 0.3), rnd(200, 150), rnd(12, 160)]
    longer = [True, False, True, False, False, True, False, False, False]
    for x, want in zip(mats, longer):
        a = (x / x.norm()).double()
        a = a @ a.T if x.shape[0] <= x.shape[1] else a.T @ a
        assert (float((a * a).sum()) <= (16 / 196) ** 2) == want, tuple(x.shape)
    monkeypatch.setenv("PYLO_MI355_NS_ADAPTIVE", "1")
    chosen = _orthogonalise_direct(mats)
    monkeypatch.delenv("PYLO_MI355_NS_ADAPTIVE")
    monkeypatch.setenv("PYLO_MI355_NS_CHAINS", "2,2,1")
    pairs = _orthogonalise_direct(mats)
    monkeypatch.setenv("PYLO_MI355_NS_CHAINS", "3,2")
    three = _orthogonalise_direct(mats)
    monkeypatch.delenv("PYLO_MI355_NS_CHAINS")
    default = _orthogonalise_direct(mats)
    for x, c, p, t, d, want in zip(mats, chosen, pairs, three, default, longer):
        assert torch.equal(c, t if want else p), tuple(x.shape)
        assert torch.equal(d, p), tuple(x.shape)            # the default: pairs
    # other odd counts: a chain of three alone, and three followed by pairs
    for iters in (3, 7):
        monkeypatch.setenv("PYLO_MI355_NS_ADAPTIVE", "1")
        got = _orthogonalise_direct(mats, iters)
        monkeypatch.delenv("PYLO_MI355_NS_ADAPTIVE")
        ref = _orthogonalise_direct(mats, iters)
        for x, y, z, want in zip(mats, got, ref, longer):
            e = float((y.double() - _reference_direct(x, iters)).abs().max())
            assert e <= 1e-4, (iters, tuple(x.shape), e)
            assert torch.equal(y, z) == (not want), (iters, tuple(x.shape))


def test_workspace_budget_and_unflagged_tensors(monkeypatch):
    """The operand planes live only during a matrix's own products: under a small PYLO_MI355_NS_WORKSPACE_MB the
    matrices run in batches that share the memory (same arithmetic, bit-identical parameters, smaller workspace);
    a group that does not orthogonalise reserves none."""
    shapes = [(300, 260), (132, 260), (260, 132), (8201, 128), (37, 131), (256, 384), (64,), (129, 129), (96, 1024)]
    opt_all, _ = _run(shapes, steps=2, seed=3)
    monkeypatch.setenv("PYLO_MI355_NS_WORKSPACE_MB", "4")
    opt_few, _ = _run(shapes, steps=2, seed=3)
    monkeypatch.delenv("PYLO_MI355_NS_WORKSPACE_MB")
    assert opt_few._plan.workspace.numel() < 0.7 * opt_all._plan.workspace.numel()
    for group_a, group_b in zip(opt_all.param_groups, opt_few.param_groups):
        for a, b in zip(group_a["params"], group_b["params"]):
            assert torch.equal(a, b)
    opt_none, _ = _run(shapes, steps=1, seed=3, orthogonalize=False)
    assert opt_none._plan.workspace.numel() < 0.3 * opt_all._plan.workspace.numel()
    assert not any(opt_none._ns_ok)


def test_groups_without_orthogonalisation_and_with_param_scale():
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP
    from oracle import pylo_oracle as O

    _run([(256, 384), (132, 260), (64,)], orthogonalize=False)
    _run([(256, 384), (132, 260), (64,)], param_scale_mult=True)
    _run([(256, 384), (132, 260), (64,)], ns_coeffs=(3.0, -3.2, 1.2), ns_eps=1e-6)
    # a tensor of a bucket sits a step out: its row stays out of the finishing table, the bucket's others go through
    torch.manual_seed(1)
    net = CELO2MLP()
    shapes = [(256, 128), (256, 128), (128, 256)]
    gen = torch.Generator(device="cuda").manual_seed(4)
    init = [torch.randn(s, generator=gen, device="cuda") * 0.05 for s in shapes]
    ref = [v.double() for v in init]
    gpu = [torch.nn.Parameter(v.clone()) for v in init]
    orc = O.EloCelo2Oracle(ref, net.state_dict(), lr=LR, weight_decay=WD, device="cuda").double_()
    opt = ELO_CELO2_CUDA(gpu, lr=LR, weight_decay=WD, network=net, hf_key=None)
    for t in range(3):
        grads = [None if (t == 1 and i == 1) else torch.randn(s, generator=gen, device="cuda") * 0.01
                 for i, s in enumerate(shapes)]
        for p, g in zip(gpu, grads):
            p.grad = g
        orc.step([None if g is None else g.double() for g in grads])
        opt.step()
        for i, p in enumerate(gpu):
            assert max_err(p, ref[i], 1e-5, 1e-6) <= 1.0, (t, i)


def test_flag_on_an_unsupported_tensor_is_refused(monkeypatch):
    import numpy as np

    from pylo_amd import _lib

    monkeypatch.setenv("PYLO_MI355_NS_F32", "1")   # the fp32 kernels refuse dims that are not multiples of 4
    plan = _lib.Plan(_lib.KIND_CELO2, [(130, 6), (64, 64)], [0, 0], torch.device("cuda:0"))
    assert not plan.orthogonalize_supported(0) and plan.orthogonalize_supported(1)
    x = torch.zeros(130 * 6 + 64 * 64, device="cuda")
    fin = np.zeros(2, dtype=_lib.ARGS_DTYPE)
    fin["grad"], fin["param"], fin["step_out"] = 1, x.data_ptr(), x.data_ptr()
    fin["flags"][0] = _lib.ARG_ORTHOGONALIZE
    with pytest.raises(RuntimeError, match="cannot orthogonalise"):
        plan.celo2_orthogonalize_finish(fin, (3.4445, -4.775, 2.0315), 5, 1e-8, 0)
    plan.close()
