"""Independent pins of the oracle's building blocks (CPU): closed forms, library routines and fp64
brute force chosen so that a dropped term, a wrong sign or index, or a transposed operand fails.
The whole-step trajectories are pinned separately by tests/test_oracle_golden.py.
"""

import itertools
import math

import numpy as np
import pytest
import torch

from oracle import pylo_oracle as O


# ---------------------------------------------------------------- factored_dims
CONFIG_SHAPES = [(768, 768), (3072, 768), (768, 3072), (768, 2304), (50257, 768), (1024, 768), (768, 3, 16, 16),
                 (1, 1, 768), (197, 768), (768, 1000), (2048, 256), (2048, 5632), (5632, 2048), (32000, 2048),
                 (37, 4099), (4099, 37), (3, 4, 5), (6, 6), (2, 3, 64, 64), (5, 5, 3, 3)]


@pytest.mark.parametrize("shape", CONFIG_SHAPES)
def test_factored_dims_against_numpy_argsort(shape):
    # The reference calls np.argsort(shape) with the default kind (CELO2_naive.py:46), which is not
    # stable: for equal dims numpy 2.2 on x86 returns e.g. [3, 2, 1, 0] for (64, 64, 3, 3).  The
    # reference's own AdafacLO_cuda.py:70 sorts (size, index) pairs, i.e. stably; that order is the
    # one pinned here.  For every shape without equal top-two dims the two agree.
    order = np.argsort(shape, kind="stable")
    assert O.factored_dims(shape) == (int(order[-2]), int(order[-1]))
    top = sorted(shape)[-2:]
    if top[0] != top[1]:
        dflt = np.argsort(shape)
        assert O.factored_dims(shape) == (int(dflt[-2]), int(dflt[-1]))
    a, b = int(order[-2]), int(order[-1])
    if shape[a] == shape[b] and not (len(shape) == 4 and a == 0 and b == 1):
        a, b = b, a                                   # Velo_naive.py:89-93
    assert O.factored_dims_velo(shape) == (a, b)


def test_factored_dims_known_table():
    assert O.factored_dims((768, 768)) == (0, 1) and O.factored_dims_velo((768, 768)) == (1, 0)
    assert O.factored_dims((3072, 768)) == (1, 0)
    assert O.factored_dims_velo((768, 3, 16, 16)) == (3, 0)
    assert O.factored_dims_velo((1, 1, 768)) == (1, 2)
    assert O.factored_dims((7,)) is None


# ---------------------------------------------------------------- accumulators from zero state
def _celo2(shapes, **kw):
    torch.manual_seed(0)
    from pylo_amd.models import CELO2MLP
    params = [torch.randn(s) * 0.1 for s in shapes]
    return params, O.EloCelo2Oracle(params, CELO2MLP().state_dict(), **kw)


def test_ema_closed_forms_first_step_and_constant_gradient():
    params, orc = _celo2([(6, 4)], clip_grad=False)
    g = torch.randn(6, 4, dtype=torch.float64).float()
    orc.step([g.clone()])
    st = orc.state[0]
    one_minus = lambda b: 1 - torch.tensor(b, dtype=torch.float32)     # 1 - beta is formed in fp32
    for k, b in enumerate((0.9, 0.99, 0.999)):
        assert torch.allclose(st["mom"][k], one_minus(b) * g, rtol=2e-6, atol=0)
    assert torch.allclose(st["rms"], one_minus(0.95) * g * g, rtol=2e-6, atol=0)
    # dims: sizes (6,4) -> dc = 1 (size 4), dr = 0 (size 6): fac_r averages over dim 0
    assert torch.allclose(st["fac_r"][0], one_minus(0.9) * ((g * g).mean(0, keepdim=True) + 1e-30), rtol=3e-6)
    assert torch.allclose(st["fac_c"][2], one_minus(0.999) * ((g * g).mean(1, keepdim=True) + 1e-30), rtol=3e-6)
    assert st["fac_r"].shape == (3, 1, 4) and st["fac_c"].shape == (3, 6, 1)
    for _ in range(9):                                 # t = 10 steps of the same gradient: (1 - beta^t) g
        orc.step([g.clone()])
    assert torch.allclose(orc.state[0]["mom"][1], (1 - 0.99 ** 10) * g, rtol=2e-5)


def test_row_col_factors_invariants():
    torch.manual_seed(1)
    fac_r = torch.rand(3, 1, 7) + 0.1
    fac_c = torch.rand(3, 5, 1) + 0.1
    rf, cf = O._row_col_factors(fac_r, fac_c, dc=1)
    # row_factor = rsqrt(r_i / mean r): mean(1 / rf^2) = 1 up to the 1e-9 guard
    assert torch.allclose((1 / rf ** 2).mean(dim=2), torch.ones(3, 1), atol=1e-6)
    assert torch.allclose(cf, fac_c ** -0.5, rtol=1e-6)
    # clamps: tiny accumulators hit max(., 1e-9)
    rf2, cf2 = O._row_col_factors(torch.full((3, 1, 2), 1e-20), torch.full((3, 2, 1), 1e-20), dc=1)
    assert torch.allclose(cf2, torch.full((3, 2, 1), 1e-9 ** -0.5))
    assert torch.isfinite(rf2).all()


# ---------------------------------------------------------------- features, brute force
def test_celo2_feature_list_brute_force():
    """30 channels of a 2x3 and a 3x2 tensor against a scalar transcription of the channel list
    (pylo/csrc/celo2_kernel.cu:86-124) in fp64."""
    for shape in [(2, 3), (3, 2)]:
        torch.manual_seed(2)
        p, g = torch.randn(shape), torch.randn(shape)
        mom, rms = torch.randn((3,) + shape), torch.rand(shape)
        dc, dr = O.factored_dims(shape)
        rs_, cs_ = list(shape), list(shape)
        rs_[dr], cs_[dc] = 1, 1
        fac_r, fac_c = torch.rand([3] + rs_) + 0.1, torch.rand([3] + cs_) + 0.1
        rf, cf = O._row_col_factors(fac_r, fac_c, dc)
        groups = O.celo2_feature_groups(p, g, mom, rms, fac_r, fac_c, rf, cf)
        got = torch.cat(groups, dim=0)
        assert got.shape[0] == 30
        for i, j in itertools.product(range(shape[0]), range(shape[1])):
            idx = (i, j)
            ci, ri = idx[dc], idx[dr]          # fac_r is indexed by the dc coordinate, fac_c by the dr one
            G, P, R = float(g[idx]), float(p[idx]), float(rms[idx])
            M = [float(mom[k][idx]) for k in range(3)]
            rs = 1 / math.sqrt(R + 1e-8)
            fr = [float(fac_r[k].reshape(-1)[ci]) for k in range(3)]
            fc = [float(fac_c[k].reshape(-1)[ri]) for k in range(3)]
            rcm = [float(fac_r[k].mean()) for k in range(3)]
            rfk = [1 / math.sqrt(max(fr[k] / (rcm[k] + 1e-9), 1e-9)) for k in range(3)]
            cfk = [1 / math.sqrt(max(fc[k], 1e-9)) for k in range(3)]
            want = [G, min(max(G, -0.1), 0.1), P] + M + [R] + [m * rs for m in M] + [rs] + \
                   [G * rfk[k] * cfk[k] for k in range(3)] + [G * rs] + fr + fc + \
                   [1 / math.sqrt(v + 1e-8) for v in fr] + [1 / math.sqrt(v + 1e-8) for v in fc] + \
                   [M[k] * rfk[k] * cfk[k] for k in range(3)]
            assert np.allclose(got[(slice(None),) + idx].numpy(), np.array(want), rtol=2e-5, atol=1e-7), (shape, idx)


def test_rms_normalize_closed_form():
    x = torch.randn(4, 5, 6)
    y = O.rms_normalize(x, [1, 2], 1e-9)
    ms = (x * x).mean(dim=(1, 2))
    assert torch.allclose((y * y).mean(dim=(1, 2)), ms / (ms + 1e-9), rtol=1e-5)


# ---------------------------------------------------------------- MLPs reduce to matmul chains
def test_celo2_mlp_equals_concatenated_matmul():
    from pylo_amd.models import CELO2MLP
    torch.manual_seed(3)
    net = CELO2MLP()
    sd = net.state_dict()
    groups = [torch.randn(k, 5, 7) for k in O.CELO2_FEATURE_DIMS]
    x = torch.cat(groups, 0).movedim(0, -1)                          # (5,7,30)
    w = torch.cat([sd[f"w0.{i}"] for i in range(14)], 0)             # (30,8), CELO2_cuda.py:169-177
    h = torch.relu(x @ w + sd["b0"])
    h = torch.relu(h @ sd["dense_w.0"] + sd["dense_b.0"])
    want = h @ sd["dense_w.1"] + sd["dense_b.1"]
    assert torch.allclose(O.celo2_mlp(groups, sd), want, rtol=1e-5, atol=1e-6)
    assert torch.allclose(net([g.movedim(0, -1) for g in groups]), want, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- Newton-Schulz
def test_newton_schulz_fp64_brute_force_and_symmetry():
    torch.manual_seed(4)
    x = torch.randn(3, 5, dtype=torch.float64)
    c0, c1, c2 = 3.4445, -4.7750, 2.0315
    y = (x / (np.linalg.norm(x.numpy()) + 1e-8)).numpy()
    for _ in range(5):
        a = y @ y.T
        y = c0 * y + (c1 * a + c2 * a @ a) @ y
    got = O.newton_schulz(x)
    assert np.allclose(got.numpy(), y, rtol=1e-12)
    assert torch.allclose(O.newton_schulz(x.t()), got.t(), rtol=1e-12)        # NS(X^T) = NS(X)^T
    s = torch.linalg.svdvals(O.newton_schulz(torch.randn(16, 32, dtype=torch.float64)))
    assert s.min() > 0.3 and s.max() < 1.3                                     # pushed towards 1


# ---------------------------------------------------------------- 1-D branch = torch.optim.AdamW
def test_adamw_branch_equals_torch_adamw():
    torch.manual_seed(5)
    p0 = torch.randn(9)
    params, orc = _celo2([(9,)], clip_grad=False, lr=1e-2, adam_lr_mult=3.0, weight_decay=0.1)
    params[0].copy_(p0)
    q = torch.nn.Parameter(p0.clone())
    ref = torch.optim.AdamW([q], lr=3e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for _ in range(6):
        g = torch.randn(9)
        orc.step([g.clone()])
        q.grad = g.clone()
        ref.step()
    # torch applies decay before the Adam update and puts eps on sqrt(v)/sqrt(bc2): same to first order
    assert torch.allclose(params[0], q.detach(), rtol=2e-4, atol=2e-5)


def test_global_norm_clip_matches_clip_grad_norm():
    torch.manual_seed(6)
    gs = [torch.randn(4, 3) * 3, torch.randn(5) * 3]
    params, orc = _celo2([(4, 3), (5,)], clip_norm=1.0)
    scale = orc.grad_scale(gs)
    ps = [torch.nn.Parameter(torch.zeros_like(g)) for g in gs]
    for p, g in zip(ps, gs):
        p.grad = g.clone()
    total = torch.nn.utils.clip_grad_norm_(ps, 1.0)
    assert abs(scale - 1.0 / float(total)) < 1e-6
    assert torch.allclose(ps[0].grad, gs[0] * scale, rtol=1e-5)
    assert orc.grad_scale([g * 1e-3 for g in gs]) == 1.0               # below the threshold: no scaling


# ---------------------------------------------------------------- VeLO pieces
def test_lstm_cell_equals_torch_lstmcell_with_permuted_gates():
    torch.manual_seed(7)
    H, K, T = 16, 8, 5
    from pylo_amd.models import VeLORNN
    rnn = VeLORNN(lstm_hidden_size=H, param_inits=K)
    sd = rnn.state_dict()
    x = torch.randn(T, 30)
    h, c = torch.randn(T, H), torch.randn(T, H)
    ctrl, lr_mult, h2, c2 = O.velo_rnn(x, h, c, sd)
    mix = torch.relu(x @ sd["mix_layer2.weight"].t() + sd["mix_layer2.bias"]).max(0, keepdim=True)[0]
    x2 = x @ sd["final_mix_layer.weight"].t() + sd["final_mix_layer.bias"] + mix
    cell = torch.nn.LSTMCell(H, H)
    W, b = sd["lstm.linear.weight"], sd["lstm.linear.bias"].clone()
    i_, g_, f_, o_ = W.chunk(4, 0)
    bi, bg, bf, bo = b.chunk(4, 0)
    Wt = torch.cat([i_, f_, g_, o_], 0)                 # torch order: i, f, g, o
    with torch.no_grad():
        cell.weight_ih.copy_(Wt[:, :H])
        cell.weight_hh.copy_(Wt[:, H:])
        cell.bias_ih.copy_(torch.cat([bi, bf + 1.0, bg, bo]))
        cell.bias_hh.zero_()
        hw, cw = cell(x2, (h, c))
    assert torch.allclose(h2, hw, atol=1e-6) and torch.allclose(c2, cw, atol=1e-6)
    assert torch.allclose(ctrl, hw @ sd["rnn_to_controls.weight"].t() + sd["rnn_to_controls.bias"], atol=1e-6)
    assert lr_mult.shape == (T,)


def test_bank_mixing_is_einsum():
    torch.manual_seed(8)
    from pylo_amd.models import VeLOMLP
    mlp = VeLOMLP(param_inits=12)
    sd = mlp.state_dict()
    ctrl = torch.randn(12)
    mixed = O.velo_mix_bank(ctrl, sd)
    for k, got in zip(O.VELO_BANK_KEYS, mixed):
        want = torch.einsum("i,i...->...", ctrl.double(), sd[k].double()) * 100.0 / 12
        assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-4)
    mlp.update_params(ctrl)
    assert torch.allclose(mlp.input_weights, mixed[0], rtol=1e-6)


def test_scalar_closed_forms():
    assert torch.allclose(O.clip_log_abs(torch.tensor([0.0, 1.0, 1e9])),
                          torch.tensor([0.5 * -5.0, 0.5 * math.log(1 + 1e-8), 2.5]))
    assert torch.allclose(O.fractional_tanh_embed(0.4)[3], torch.tensor(0.0))
    assert torch.allclose(O.tanh_time_embedding(3.0)[1], torch.tensor(0.0))
    assert torch.allclose(O.tanh_time_embedding(0.0), torch.full((11,), math.tanh(-1.0)))
    d = O.decay_from_offsets((0.9, 0.99, 0.999), (0.0, 0.0, 0.0))
    assert torch.allclose(d, torch.tensor([0.9, 0.99, 0.999]), atol=1e-6)
    d2 = O.decay_from_offsets((0.9,), (0.1,))
    assert abs(float(d2) - (1 - math.exp(math.log(0.1) + 1.0))) < 1e-6


def test_loss_accumulators_closed_forms():
    acc = O.LossAccumulators(100)
    assert torch.allclose(acc.decays[0], torch.exp(torch.tensor(-0.1))) and acc.decays.shape == (10,)
    for t in range(3):
        acc.update(torch.tensor(2.0))
    # constant loss: every bias-corrected mean equals the loss, so numerators and features are 0 - 1 -> clamp
    cor = acc.means / (1 - acc.decays ** 3)
    assert torch.allclose(cor, torch.full((10,), 2.0), rtol=1e-5)
    f = acc.features()
    assert f.shape == (9,) and torch.all((f >= -1) & (f <= 1))
    acc2 = O.LossAccumulators(100)
    acc2.update(torch.tensor(1.0))
    assert torch.all(acc2.features() == 0)              # iteration <= 2 -> zeros
    acc2.update(torch.tensor(1000.0))                    # clipped to 2 * max corrected mean = 2
    cor2 = acc2.means / (1 - acc2.decays ** 2)
    assert float(cor2.max()) <= 2.0 + 1e-5


# ---------------------------------------------------------------- per-parameter step counters (AdafacLO)
def test_adafac_per_param_step_equals_single_parameter_runs():
    """AdafacLO_cuda.py:304-305,400: every parameter's time features follow its own step counter.
    AdafacLO tensors do not interact, so the switch is fixed by a property that needs no second
    implementation: a parameter that sat steps out must end exactly where a single-parameter run, fed
    only the steps it took part in (and counting per group, the golden-pinned default), ends."""
    from pylo_amd.models import MetaMLP

    torch.manual_seed(21)
    net = MetaMLP(39, 32, 1).state_dict()
    shapes = [(6, 10), (7,), (3, 4, 5)]
    gen = torch.Generator().manual_seed(9)
    init = [torch.randn(s, generator=gen) * 0.3 for s in shapes]
    sat_out = {0: {1, 2}, 1: {4}, 2: set()}          # parameter -> steps without a gradient
    steps = 6
    grads = [[None if t in sat_out[i] else torch.randn(s, generator=gen) * 0.1 for i, s in enumerate(shapes)]
             for t in range(steps)]
    both = [v.clone() for v in init]
    orc = O.AdafacOracle(both, net, lr=0.5, per_param_step=True)
    for t in range(steps):
        orc.step(grads[t])
    assert orc.steps == [4, 5, 6]
    for i in range(len(shapes)):
        alone = [init[i].clone()]
        solo = O.AdafacOracle(alone, net, lr=0.5)     # per group: t counts the calls it received
        for t in range(steps):
            if grads[t][i] is not None:
                solo.step([grads[t][i]])
        assert torch.equal(both[i], alone[0]), i
        for k in ("exp_avg", "exp_avg_sq", "exp_avg_sq_r", "exp_avg_sq_c"):
            assert torch.equal(orc.state[i][k], solo.state[0][k]), (i, k)
    # and the switch matters: counting per group moves the lagging parameter elsewhere
    grp = [v.clone() for v in init]
    orc_g = O.AdafacOracle(grp, net, lr=0.5)
    for t in range(steps):
        orc_g.step(grads[t])
    assert not torch.equal(grp[0], both[0]) and torch.equal(grp[2], both[2])
