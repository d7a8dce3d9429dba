"""Tensors with more than two dims in ``pylo_mi355_celo2_orthogonalize_finish`` / ``pylo_mi355_celo2_finish``:
Newton-Schulz, the normaliser and the parameter update per slice of the last two dims
(pylo/optim/CELO2_naive.py:59-73 "over the last two dims"; pylo/optim/ELO_CELO2_naive.py:231-235).  Small slices
are held in LDS or registers by one lane, a wave or a block from the raw step to the parameter; larger ones are
matrices of the tiled products like any 2-D tensor, each with its own norm and normaliser.  Against the literal
formula in fp64 slice by slice through the C-ABI, and through whole optimizer steps against the oracle
(parameters at rel 1e-5 / abs 1e-6).
"""

import numpy as np
import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

COEFFS = (3.4445, -4.775, 2.0315)

# (shape, lanes that own a slice)
SHAPES = [((32, 16, 3, 3), 1), ((6, 4, 1, 1), 1), ((5, 4, 8), 1), ((3, 8, 4), 1), ((2, 1, 7), 1), ((5, 5, 5, 5), 1),
          ((4, 6, 6), 1), ((70, 7, 7), 1), ((3, 2, 100), 1), ((130, 3, 3), 1),
          ((7, 16, 16), 64), ((2, 3, 4, 70), 64), ((3, 70, 4), 64), ((5, 8, 8), 64),
          ((3, 40, 33), 256), ((2, 64, 128), 256), ((2, 128, 64), 256), ((1, 2, 33, 200), 256)]
# slices for the tiled products
LARGE = [(2, 128, 128), (3, 64, 300), (2, 300, 64), (2, 2, 130, 201), (1, 8300, 40)]


def _formula(x, iters, dtype=torch.float64, orthogonalise=True):
    """orthogonalize_via_newton_schulz and the normaliser over the last two dims, batched over the leading ones."""
    c0, c1, c2 = COEFFS
    x = x.to(dtype)
    if orthogonalise:
        t = x.shape[-2] > x.shape[-1]
        if t:
            x = x.transpose(-2, -1)
        x = x / (torch.linalg.norm(x, dim=(-2, -1), keepdim=True) + 1e-8)
        for _ in range(iters):
            a = x @ x.transpose(-2, -1)
            x = c0 * x + (c1 * a + c2 * (a @ a)) @ x
        if t:
            x = x.transpose(-2, -1)
    return x * torch.rsqrt(1e-9 + (x * x).mean(dim=(-2, -1), keepdim=True))


def _finish_direct(mats, iters, flag=True, entry="orthogonalize_finish"):
    from pylo_amd import _lib

    shapes = [tuple(x.shape) for x in mats]
    plan = _lib.Plan(_lib.KIND_CELO2, shapes, [0] * len(shapes), torch.device("cuda:0"))
    assert all(plan.finish_supported(i) and plan.orthogonalize_supported(i) for i in range(len(mats)))
    per_slice = [plan.orthogonalize_supported(i) == 2 for i in range(len(mats))]
    steps = [x.clone().contiguous() for x in mats]
    params = [torch.zeros_like(x) for x in mats]
    fin = np.zeros(len(mats), dtype=_lib.ARGS_DTYPE)
    for i in range(len(mats)):
        fin["grad"][i], fin["param"][i], fin["step_out"][i] = 1, params[i].data_ptr(), steps[i].data_ptr()
        fin["lr"][i], fin["weight_decay"][i], fin["step_mult"][i] = -1.0, 0.0, 1.0
        fin["flags"][i] = _lib.ARG_ORTHOGONALIZE if flag else 0
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "finish":
        plan.celo2_finish(fin, stream)
    else:
        plan.celo2_orthogonalize_finish(fin, COEFFS, iters, 1e-8, stream)
    torch.cuda.synchronize()
    plan.close()
    for x, s, small in zip(mats, steps, per_slice):
        if small:
            assert torch.equal(x, s)      # the per-slice launches leave the raw step as it was
    return params


@pytest.mark.parametrize("iters", [5, 1, 0])
def test_slices_against_the_formula_in_fp64(iters):
    """With p = 0, lr = -1 the parameter is the normalised, orthogonalised step (unit RMS per slice).  A slice of a
    few elements can be nearly singular, where five iterations amplify rounding by up to 3.4445^5: the bar is the
    error of the same formula in fp32 torch products times 1.5, plus 5e-5."""
    gen = torch.Generator(device="cuda").manual_seed(11 + iters)
    shapes = [s for s, _l in SHAPES] + (LARGE if iters > 0 else [])
    mats = [torch.randn(s, generator=gen, device="cuda") * 10.0 ** (-(i % 4)) for i, s in enumerate(shapes)]
    got = _finish_direct(mats, iters)
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    rows = []
    try:
        for x, y in zip(mats, got):
            want = _formula(x, iters)
            e = float((y.double() - want).abs().max())
            e32 = float((_formula(x, iters, torch.float32).double() - want).abs().max())
            rows.append((tuple(x.shape), e, e32))
            assert e <= 1.5 * e32 + 5e-5, rows[-1]
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    print("iters", iters, "(shape, library error, fp32 torch formula error):", rows)


@pytest.mark.parametrize("entry", ["finish", "orthogonalize_finish"])
def test_slices_without_the_flag_are_normalised_only(entry):
    gen = torch.Generator(device="cuda").manual_seed(3)
    mats = [torch.randn(s, generator=gen, device="cuda") * 0.1 for s in [s for s, _l in SHAPES] + LARGE]
    # pylo_mi355_celo2_finish ignores the flag; the other entry point honours its absence
    got = _finish_direct(mats, 5, flag=(entry == "finish"), entry=entry)
    for x, y in zip(mats, got):
        want = _formula(x, 0, orthogonalise=False)
        assert float((y.double() - want).abs().max()) <= 2e-6, tuple(x.shape)


def test_which_kernels_take_a_tensor_and_what_is_refused():
    from pylo_amd import _lib

    shapes = [s for s, _l in SHAPES] + LARGE + [(64, 64), (64,)]
    flags = [0] * (len(shapes) - 1) + [_lib.F_ADAM]
    plan = _lib.Plan(_lib.KIND_CELO2, shapes, flags, torch.device("cuda:0"))
    n, k = len(SHAPES), len(LARGE)
    assert all(plan.finish_supported(i) for i in range(n + k + 1)) and not plan.finish_supported(n + k + 1)
    assert [plan.orthogonalize_supported(i) for i in range(n + k + 2)] == [2] * n + [1] * k + [1, 0]
    # zero iterations: the per-slice launches divide by the norm, the tiled products refuse the flag
    x = torch.zeros(2 * 128 * 128, device="cuda")
    fin = np.zeros(len(shapes), dtype=_lib.ARGS_DTYPE)
    fin["grad"][n], fin["param"][n], fin["step_out"][n] = 1, x.data_ptr(), x.data_ptr()
    fin["flags"][n] = _lib.ARG_ORTHOGONALIZE
    with pytest.raises(RuntimeError, match="ns_iters = 0"):
        plan.celo2_orthogonalize_finish(fin, COEFFS, 0, 1e-8, 0)
    plan.close()
    # a shape flagged as never orthogonalised: finished per slice, the flag refused
    flags = [_lib.F_NO_ORTHOGONALIZE, 0, _lib.F_NO_ORTHOGONALIZE]
    plan = _lib.Plan(_lib.KIND_CELO2, [(4, 3, 3), (4, 3, 3), (2, 128, 128)], flags, torch.device("cuda:0"))
    assert [plan.orthogonalize_supported(i) for i in range(3)] == [0, 2, 0]
    assert all(plan.finish_supported(i) for i in range(3))
    for i, msg in ((0, "PYLO_F_NO_ORTHOGONALIZE"), (2, "cannot orthogonalise")):
        fin = np.zeros(3, dtype=_lib.ARGS_DTYPE)
        fin["grad"][i], fin["param"][i], fin["step_out"][i] = 1, x.data_ptr(), x.data_ptr()
        fin["flags"][i] = _lib.ARG_ORTHOGONALIZE
        with pytest.raises(RuntimeError, match=msg):
            plan.celo2_orthogonalize_finish(fin, COEFFS, 5, 1e-8, 0)
    plan.close()


def test_fp32_matrix_instructions_leave_large_slices_to_the_caller(monkeypatch):
    """PYLO_MI355_NS_F32=1: the fp32 product kernels take 2-D tensors only; the class orthogonalises large slices
    with torch products and the library still normalises and applies them per slice."""
    from pylo_amd import _lib

    monkeypatch.setenv("PYLO_MI355_NS_F32", "1")
    plan = _lib.Plan(_lib.KIND_CELO2, [(2, 128, 128), (4, 3, 3), (64, 64)], [0, 0, 0], torch.device("cuda:0"))
    assert [plan.orthogonalize_supported(i) for i in range(3)] == [0, 2, 1]
    assert all(plan.finish_supported(i) for i in range(3))
    plan.close()
    test_whole_steps_against_the_oracle(dict(), True, False)


def test_short_slices_of_every_length_class_against_the_oracle():
    """The feature pass of short slices (one lane per slice, staged through LDS in blocks of several groups of 64
    slices; slices of one element straight from memory) over every class of slice length, with slice counts that
    leave the last group and the last block ragged: accumulators, raw steps and parameters through whole
    free-running steps against the fp64 oracle."""
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(2)
    net = CELO2MLP()
    # slices x length: 1480 x 1, 63 x 1, 577 x 2, 450 x 4, 300 x 6, 200 x 9, 273 x 16, 77 x 25, 70 x 32
    shapes = [(40, 37, 1, 1), (9, 7, 1, 1), (577, 1, 2), (9, 50, 2, 2), (20, 15, 2, 3), (8, 25, 3, 3), (21, 13, 4, 4),
              (7, 11, 5, 5), (10, 7, 4, 8), (48, 64)]
    gen = torch.Generator(device="cuda").manual_seed(31)
    init = [torch.randn(s, generator=gen, device="cuda") * 0.05 for s in shapes]
    ref = [v.double() for v in init]
    gpu = [torch.nn.Parameter(v.clone()) for v in init]
    cfg = dict(lr=1e-3, weight_decay=0.1, adam_lr_mult=20.0)
    orc = O.EloCelo2Oracle(ref, net.state_dict(), device="cuda", **cfg).double_()
    opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
    for t in range(3):
        grads = [torch.randn(s, generator=gen, device="cuda") * 10.0 ** (-1 - i % 3) for i, s in enumerate(shapes)]
        for p, g in zip(gpu, grads):
            p.grad = g
        orc.step([g.double() for g in grads])
        opt.step()
        torch.cuda.synchronize()
        for i, p in enumerate(gpu):
            assert max_err(p, ref[i], 1e-5, 1e-6) <= 1.0, (t, i, shapes[i])
            st = opt.state[p]
            for key in ("mom", "rms"):
                if key in st and key in orc.state[i]:
                    assert max_err(st[key], orc.state[i][key], 1e-5, 1e-6) <= 1.0, (t, i, shapes[i], key)


@pytest.mark.parametrize("kw,with_large_slices,cached_table", [
    (dict(), False, True), (dict(), True, True), (dict(ns_iters=0), True, False),
    (dict(orthogonalize=False), True, True), (dict(param_scale_mult=True), False, False)])
def test_whole_steps_against_the_oracle(kw, with_large_slices, cached_table):
    """ELO_CELO2_CUDA.step() on convolution-shaped tensors next to matrices and vectors, free-running for four
    steps against the fp64 oracle, with and without a tensor whose slices go to the tiled products.  When the
    library finishes every tensor itself the finishing table is the cached one (no per-step Python over the
    tensors); zero iterations on a matrix or param_scale_mult take the general path.
    lr = 1e-3: among 512 random 3 x 3 slices some are nearly singular, where five iterations amplify the fp32
    rounding of the raw step by up to 3.4445^5 in any fp32 evaluation (the accuracy of the orthogonalised step
    itself is held by test_slices_against_the_formula_in_fp64)."""
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(1)
    net = CELO2MLP()
    shapes = [(32, 16, 3, 3), (7, 16, 16), (256, 384), (64,), (3, 40, 33), (2, 64, 128), (6, 4, 1, 1), (5, 4, 8)]
    if with_large_slices:
        shapes += [(2, 128, 128), (3, 64, 300)]
    gen = torch.Generator(device="cuda").manual_seed(21)
    init = [torch.randn(s, generator=gen, device="cuda") * 0.05 for s in shapes]
    ref = [v.double() for v in init]
    gpu = [torch.nn.Parameter(v.clone()) for v in init]
    cfg = dict(lr=1e-3, weight_decay=0.1, adam_lr_mult=20.0)
    cfg.update(kw)
    orc = O.EloCelo2Oracle(ref, net.state_dict(), device="cuda", **cfg).double_()
    opt = ELO_CELO2_CUDA(gpu, network=net, hf_key=None, **cfg)
    for t in range(4):
        grads = [torch.randn(s, generator=gen, device="cuda") * 10.0 ** (-1 - i % 3) for i, s in enumerate(shapes)]
        for p, g in zip(gpu, grads):
            p.grad = g
        orc.step([g.double() for g in grads])
        opt.step()
        torch.cuda.synchronize()
        for i, p in enumerate(gpu):
            assert max_err(p, ref[i], 1e-5, 1e-6) <= 1.0, (kw, t, i, shapes[i])
    cached = getattr(opt, "_fin_fast", None)
    assert (cached is not None and cached["idx"] is not None) == cached_table
