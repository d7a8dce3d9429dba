"""Parameters and gradients stored as float16, bfloat16 or float64 (PYLO_F_STORE_*), through the optimizer
classes and the C ABI.

The reference's kernels are instantiated per element type and widen to float on load, compute in float and
narrow on store (celo2_kernel.cu:70-75,280,314; velo_kernel.cu:405; learned_optimizer.cu:338); its classes keep
the accumulators in float32 (ELO_CELO2_cuda.py:167-177).  The contract checked here is the same: a step on a
tagged tensor is the float32 step on the widened values, with the updated parameter rounded to nearest-even
into its storage type.  The checker is therefore the float32 oracle fed the widened gradients, whose
parameters are rounded into the storage type after every step:

* accumulators (float32 on both sides): rel 1e-5 / abs 1e-6, every step;
* float64 parameters: rel 1e-5 / abs 1e-6;
* 16-bit parameters: the oracle's value rounded into the type, compared in units of the type's spacing.  Two
  float32 results that agree to rel 1e-5 round to different neighbours where a rounding boundary lies between
  them, for a share of the elements of about 1e-5 / (relative spacing): up to 0.3 % in bfloat16 (spacing
  2^-8), 1 % .. 2 % in float16 (2^-11).  The bar: no element further than ONE spacing away (the spacing at
  1e-3 for values nearer zero), and not bit-identical at most 0.1 % (bfloat16) or 0.3 % (float16) of the
  values above 1e-3, or one element of a small tensor: the float32 steps agree to about 1e-6, ten times
  closer than the tolerance.  Each step starts from identical parameters (the oracle's are set to the
  buffer's contents after the comparison); the accumulators run free.

What the reference's own naive classes do with such parameters (mixed float16/float32 torch arithmetic where
they run at all) is held, loosely, in tests/test_storage_types_golden_gpu.py.
"""

import copy

import pytest
import torch

from golden_io import max_err

pytestmark = pytest.mark.gpu

REL, ABS = 1e-5, 1e-6
DTYPES = [torch.bfloat16, torch.float16, torch.float64]


def _widen(t):
    """What the kernels compute with: the stored value as float32 (float64 is rounded, as static_cast<float> does)."""
    return t.detach().float().cpu()


def _spacing(x, dtype):
    """Distance between neighbouring values of `dtype` at |x| (taken at 1e-3 for smaller values: next to zero
    the spacing falls below the float32 error of the step itself)."""
    bits = {torch.bfloat16: 7, torch.float16: 10}[dtype]
    mag = x.double().abs().clamp_min(1e-3)
    return torch.pow(2.0, torch.floor(torch.log2(mag)) - bits)


def _check_param(got, want32, dtype, where):
    assert got.dtype == dtype, where
    assert torch.isfinite(got).all(), where
    if dtype == torch.float64:
        # the kernels store a float32 result: every stored value is float32-representable
        assert torch.equal(got.detach().cpu(), got.detach().float().double().cpu()), where
        e = max_err(got, want32, REL, ABS)
        assert e <= 1.0, (where, e)
        want32.copy_(got.detach().float().cpu())
        return
    g = got.detach().cpu().reshape(-1)
    w = want32.to(dtype).reshape(-1)
    d = (g.double() - w.double()).abs() / _spacing(w, dtype)
    assert float(d.max()) <= 1.0, (where, float(d.max()))
    differ = int(((g != w) & (w.float().abs() > 1e-3)).sum())
    share = 1e-3 if dtype == torch.bfloat16 else 3e-3
    assert differ <= max(1, int(g.numel() * share)), (where, differ, g.numel())
    want32.copy_(got.detach().float().cpu().reshape(want32.shape))


def _grads(shapes, gen, dtype, scales):
    out = []
    for i, s in enumerate(shapes):
        g = (torch.randn(s, generator=gen) * scales[i % len(scales)]).to(dtype)
        out.append(g)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
def test_elo_celo2_steps_on_stored_types(dtype):
    """Whole ELO_CELO2_CUDA.step(): matrices (column walk, linear chunks, ragged), a tensor with more than two
    dims (the per-slice launch), AdamW vectors, an is_embedding group; one tensor stays float32 (mixed plan)."""
    from oracle import pylo_oracle as O
    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    torch.manual_seed(1)
    net = CELO2MLP()
    shapes = [(64, 256), (130, 36), (37, 41), (96,), (8, 3, 12, 20), (48, 64), (1, 128), (200,)]
    emb = [False, False, False, False, False, True, False, False]
    keep32 = {2}
    gen = torch.Generator().manual_seed(7)
    dts = [torch.float32 if i in keep32 else dtype for i in range(len(shapes))]
    init = [(torch.randn(s, generator=gen) * 0.3).to(dt) for s, dt in zip(shapes, dts)]
    cpu = [_widen(v).clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    cfg = dict(lr=1e-2, weight_decay=0.05, exp_mult=0.01)
    orc = O.EloCelo2Oracle(cpu, net.state_dict(), is_embedding=emb, adam_lr_mult=20.0, **cfg)
    plain = [p for p, e in zip(gpu, emb) if not e]
    embp = [p for p, e in zip(gpu, emb) if e]
    opt = ELO_CELO2_CUDA([{"params": plain}, {"params": embp, "is_embedding": True}], network=net, hf_key=None, **cfg)
    for t in range(4):
        grads = [g.to(dt) for g, dt in zip(_grads(shapes, gen, torch.float32, (1.0, 0.1, 3.0)), dts)]
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        orc.step([_widen(g) for g in grads])
        opt.step()
        torch.cuda.synchronize()
        for i, p in enumerate(gpu):
            st = opt.state[p]
            for k in ("mom", "rms", "fac_r", "fac_c"):
                if k in orc.state[i] and k in st and not (emb[i] and k.startswith("fac")):
                    assert st[k].dtype == torch.float32
                    e = max_err(st[k], orc.state[i][k], REL, ABS)
                    assert e <= 1.0, (dtype, t, i, k, e)
            if dts[i] == torch.float32:
                assert max_err(p, cpu[i], REL, ABS) <= 1.0, (dtype, t, i)
            else:
                _check_param(p, cpu[i], dtype, (str(dtype), t, i, shapes[i]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_velo_steps_on_stored_types(dtype):
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    torch.manual_seed(3)
    rnn = VeLORNN(lstm_hidden_size=64, param_inits=32)
    with torch.no_grad():
        rnn.lstm_init_state[0].normal_(0, 0.1)
        rnn.lstm_init_state[1].normal_(0, 0.1)
    mlp = VeLOMLP(param_inits=32)
    shapes = [(70, 384), (130, 36), (37, 41), (96,), (8, 3, 5, 5), (1, 1, 48), (1,), (64, 64)]
    gen = torch.Generator().manual_seed(11)
    init = [(torch.randn(s, generator=gen) * 0.3).to(dtype) for s in shapes]
    cpu = [_widen(v).clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    kw = dict(lr=1e-2, num_steps=50, weight_decay=1e-3)
    orc = O.VeloOracle(cpu, rnn.state_dict(), mlp.state_dict(), **kw)
    opt = VeLO_CUDA(gpu, rnn=copy.deepcopy(rnn), mlp=copy.deepcopy(mlp), **kw)
    for t in range(4):
        grads = _grads(shapes, gen, dtype, (1.0, 0.1, 0.01))
        loss = torch.tensor(1.5 - 0.2 * t)
        for p, g in zip(gpu, grads):
            p.grad = g.cuda()
        orc.step([_widen(g) for g in grads], loss)
        opt.step(loss.cuda())
        torch.cuda.synchronize()
        for tag, got, ref in (("h", opt.lstm_hidden_state[0], orc.h), ("c", opt.lstm_hidden_state[1], orc.c)):
            assert max_err(got, ref, REL, ABS) <= 1.0, (dtype, t, tag)
        for i, p in enumerate(gpu):
            st, so = opt.state[p], orc.state[i]
            for k in ("mom", "rms", "fac_vec_row", "fac_vec_col", "fac_vec_v"):
                if k in so:
                    assert st[k].dtype == torch.float32
                    e = max_err(st[k], so[k], REL, ABS)
                    assert e <= 1.0, (dtype, t, i, k, e)
            _check_param(p, cpu[i], dtype, (str(dtype), t, i, shapes[i]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_adafac_steps_on_stored_types(dtype):
    from oracle import pylo_oracle as O
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    torch.manual_seed(9)
    net = MetaMLP(39, 32, 1)
    shapes = [(70, 384), (130, 36), (37, 41), (96,), (8, 3, 5, 5), (3, 64), (64, 64)]
    gen = torch.Generator().manual_seed(23)
    init = [(torch.randn(s, generator=gen) * 0.3).to(dtype) for s in shapes]
    cpu = [_widen(v).clone() for v in init]
    gpu = [torch.nn.Parameter(v.clone().cuda()) for v in init]
    orc = O.AdafacOracle(cpu, net.state_dict(), lr=0.05, weight_decay=1e-3, per_param_step=True)
    opt = AdafacLO_CUDA(gpu, lr=0.05, weight_decay=1e-3, network=copy.deepcopy(net))
    for t in range(4):
        grads = _grads(shapes, gen, dtype, (1.0, 0.1, 0.01))
        if t == 2:
            grads[1] = None      # a tensor that sits a step out keeps its buffer untouched
        before = gpu[1].detach().clone()
        for p, g in zip(gpu, grads):
            p.grad = None if g is None else g.cuda()
        orc.step([None if g is None else _widen(g) for g in grads])
        opt.step()
        torch.cuda.synchronize()
        if t == 2:
            assert torch.equal(gpu[1].detach(), before)
        for i, p in enumerate(gpu):
            st, so = opt.state[p], orc.state[i]
            for k in ("exp_avg", "exp_avg_sq", "exp_avg_sq_r", "exp_avg_sq_c"):
                assert st[k].dtype == torch.float32
                e = max_err(st[k], so[k], REL, ABS)
                assert e <= 1.0, (dtype, t, i, k, e)
            _check_param(p, cpu[i], dtype, (str(dtype), t, i, shapes[i]))


def test_unsupported_storage_type_is_refused():
    from pylo_amd import AdafacLO_CUDA
    from pylo_amd.models import MetaMLP

    p = torch.nn.Parameter(torch.zeros(8, 8, device="cuda", dtype=torch.complex64))
    opt = AdafacLO_CUDA([p], lr=0.1, network=MetaMLP(39, 32, 1))
    p.grad = torch.zeros_like(p)
    with pytest.raises(TypeError, match="float32, float16, bfloat16 or float64"):
        opt.step()
