"""16-bit parameters against what the reference's own naive classes do with them.

AdafacLO_naive, ELO_naive and VeLO_naive run on float16 / bfloat16 parameters (ELO_CELO2_naive and CELO2_naive
raise a dtype error on anything but float32, every naive class does on float64): the accumulators are float32
and torch's type promotion decides the rest, so ``g ** 2`` and the row / column means over it are rounded to
the 16-bit type before they enter the float32 accumulators, and the two-stage weight decay rounds the parameter
twice (AdafacLO_naive.py:238-239,306-309).  The library follows the reference's *kernels* instead (widen, compute
in float32, narrow once: learned_optimizer.cu:34-98,296-299), which is strictly more accurate, so these golden
trajectories (tests/golden/{adafac_bf16,elo_f16,velo_bf16}.npz, written by tests/golden/make_golden.py from the
naive classes) can only be met to the 16-bit type's own resolution:

* momentum accumulators take no 16-bit operation in AdafacLO_naive and VeLO_naive: rel 1e-5 / abs 1e-6; ELO_naive
  scales the gradient by the clip factor in the 16-bit type first (ELO_naive.py:205-207): rel 2^-7;
* second-moment and factored accumulators: rel 2^-7 (their inputs were rounded at 2^-9 / 2^-12 relative);
* parameters: within two spacings of the storage type, six in ten bit-identical (with AdafacLO's lr of 0.5 a
  step differing in its third digit moves one parameter in five across a bfloat16 rounding boundary; VeLO's
  trajectory comes out bit-identical).

The exact contract of the stored types is tested in tests/test_storage_types_gpu.py.
"""

import pytest
import torch

from golden_io import Golden, max_err, trailing_to_keepdim

pytestmark = pytest.mark.gpu

DT = {"float16": torch.float16, "bfloat16": torch.bfloat16}
LOOSE = 2.0 ** -7


def _check_param(got, want, dtype, where):
    bits = {torch.bfloat16: 7, torch.float16: 10}[dtype]
    g, w = got.detach().float().cpu().reshape(-1).double(), want.reshape(-1).double()
    spacing = torch.pow(2.0, torch.floor(torch.log2(w.abs().clamp_min(1e-2))) - bits)
    d = (g - w).abs() / spacing
    assert float(d.max()) <= 2.0, (where, float(d.max()))
    same = float((g == w).double().mean())
    assert same >= 0.6 or g.numel() < 50, (where, same)
    return same


def _adafac_like(name, cls_name):
    from oracle import pylo_oracle as O
    import pylo_amd
    from pylo_amd.models import MetaMLP

    G = Golden(name)
    meta, shapes = G.meta, G.shapes
    dtype = DT[meta["dtype"]]
    net = MetaMLP(39, 32, 1)
    net.load_state_dict(G.state_dict("net"))
    gpu = [torch.nn.Parameter(G.t(f"init/{i}").to(dtype).cuda()) for i in range(len(shapes))]
    extra = {k: (tuple(v) if isinstance(v, list) else v) for k, v in (meta["extra"] or {}).items()}
    kw = dict(hf_key=None) if cls_name == "ELO_CUDA" else {}
    opt = getattr(pylo_amd, cls_name)(gpu, lr=meta["lr"], weight_decay=meta["weight_decay"], network=net, **kw, **extra)
    worst_same = 1.0
    for t in range(meta["n_steps"]):
        for i, p in enumerate(gpu):
            p.grad = G.t(f"grad{t}/{i}").to(dtype).cuda()
        opt.step()
        for i, p in enumerate(gpu):
            st = opt.state[p]
            # (a momentum near zero is a difference of terms that each carry the 16-bit rounding of g * scale)
            rel, ab = (LOOSE, 1e-5) if extra.get("clip_grad") else (1e-5, 1e-6)
            assert max_err(st["exp_avg"], G.t(f"step{t}/exp_avg/{i}"), rel, ab) <= 1.0, (name, t, i, "exp_avg")
            checks = [("exp_avg_sq", st["exp_avg_sq"], G.t(f"step{t}/exp_avg_sq/{i}"))]
            if len(shapes[i]) < 2:
                checks.append(("fac_v", st["exp_avg_sq_r"], G.t(f"step{t}/fac_vec_v/{i}")))
            else:
                dc, dr = O.factored_dims(shapes[i])
                checks.append(("row", st["exp_avg_sq_r"], trailing_to_keepdim(G.t(f"step{t}/fac_vec_row_trailing/{i}"), dr)))
                checks.append(("col", st["exp_avg_sq_c"], trailing_to_keepdim(G.t(f"step{t}/fac_vec_col_trailing/{i}"), dc)))
            for tag, got, ref in checks:
                e = max_err(got, ref, LOOSE, 1e-7)
                assert e <= 1.0, (name, t, i, tag, e)
            worst_same = min(worst_same, _check_param(p, G.t(f"step{t}/param/{i}"), dtype, (name, t, i)))
            # each step from the reference's own parameters: a rounding that fell the other way is not carried along
            p.data.copy_(G.t(f"step{t}/param/{i}").to(dtype))
    print(name, "least share of bit-identical parameters", worst_same)


def test_adafaclo_on_bfloat16_parameters_against_the_naive_class():
    _adafac_like("adafac_bf16", "AdafacLO_CUDA")


def test_elo_on_float16_parameters_against_the_naive_class():
    _adafac_like("elo_f16", "ELO_CUDA")


def test_velo_on_bfloat16_parameters_against_the_naive_class():
    from oracle import pylo_oracle as O
    from pylo_amd import VeLO_CUDA
    from pylo_amd.models import VeLOMLP, VeLORNN

    G = Golden("velo_bf16")
    meta, shapes = G.meta, G.shapes
    dtype = DT[meta["dtype"]]
    rnn = VeLORNN(lstm_hidden_size=meta["lstm_hidden"], param_inits=meta["param_inits"])
    rnn.load_state_dict(G.state_dict("rnn"))
    mlp = VeLOMLP(param_inits=meta["param_inits"])
    mlp.load_state_dict(G.state_dict("mlp"))
    gpu = [torch.nn.Parameter(G.t(f"init/{i}").to(dtype).cuda()) for i in range(len(shapes))]
    opt = VeLO_CUDA(gpu, lr=meta["lr"], num_steps=meta["num_steps"], weight_decay=meta["weight_decay"], rnn=rnn, mlp=mlp)
    worst_same = 1.0
    for t in range(meta["n_steps"]):
        for i, p in enumerate(gpu):
            p.grad = G.t(f"grad{t}/{i}").to(dtype).cuda()
        opt.step(G.t(f"loss{t}").cuda())
        # the LSTM sees the tensors through variances and means of the accumulators: 16-bit resolution of its inputs
        for tag, got in (("lstm_h", opt.lstm_hidden_state[0]), ("lstm_c", opt.lstm_hidden_state[1])):
            assert max_err(got, G.t(f"step{t}/{tag}"), LOOSE, 1e-3) <= 1.0, (t, tag)
        for i, p in enumerate(gpu):
            st = opt.state[p]
            assert max_err(st["mom"], G.t(f"step{t}/mom/{i}"), 1e-5, 1e-6) <= 1.0, (t, i, "mom")
            checks = [("rms", st["rms"], G.t(f"step{t}/rms/{i}"))]
            if len(shapes[i]) < 2:
                checks.append(("fac_v", st["fac_vec_v"], G.t(f"step{t}/fac_vec_v/{i}")))
            else:
                dc, dr = O.factored_dims_velo(shapes[i])
                checks.append(("row", st["fac_vec_row"], trailing_to_keepdim(G.t(f"step{t}/fac_vec_row_trailing/{i}"), dr)))
                checks.append(("col", st["fac_vec_col"], trailing_to_keepdim(G.t(f"step{t}/fac_vec_col_trailing/{i}"), dc)))
            for tag, got, ref in checks:
                e = max_err(got, ref, LOOSE, 1e-7)
                assert e <= 1.0, (t, i, tag, e)
            worst_same = min(worst_same, _check_param(p, G.t(f"step{t}/param/{i}"), dtype, ("velo_bf16", t, i)))
            p.data.copy_(G.t(f"step{t}/param/{i}").to(dtype))
    print("velo_bf16 least share of bit-identical parameters", worst_same)
