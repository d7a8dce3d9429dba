"""The oracle against golden trajectories written from the reference's naive classes.

Tolerance: rel 1e-5 / abs 1e-6 on parameters and every optimizer state after every
step (``max_err <= 1``), the bar the north star sets for the HIP path itself.
"""

import numpy as np
import pytest
import torch

from oracle import pylo_oracle as O
from golden_io import Golden, max_err, trailing_to_keepdim

REL, ABS = 1e-5, 1e-6


def _regen_inputs(meta):
    gen = torch.Generator().manual_seed(meta["seed"])
    shapes = [tuple(s) for s in meta["shapes"]]
    init = [torch.randn(s, generator=gen) * meta["init_std"] for s in shapes]
    grads = [[torch.randn(s, generator=gen) * meta["grad_scale"] for s in shapes]
             for _ in range(meta["n_steps"])]
    return init, grads


@pytest.mark.parametrize("name", ["elo_celo2_small_clip", "elo_celo2_small_noclip_exp",
                                  "elo_celo2_small_noortho", "elo_celo2_cfg1", "elo_celo2_nd",
                                  "elo_celo2_mlp1d"])
def test_elo_celo2_oracle_matches_reference(name):
    G = Golden(name)
    meta = G.meta
    shapes = G.shapes
    if meta["full"]:
        init = [G.t(f"init/{i}") for i in range(len(shapes))]
        grads = [[G.t(f"grad{t}/{i}") for i in range(len(shapes))] for t in range(meta["n_steps"])]
    else:
        init, grads = _regen_inputs(meta)
    params = [v.clone() for v in init]
    cfg = dict(meta["cfg"])
    cfg.setdefault("adam_lr_mult", 1.0)
    opt = O.EloCelo2Oracle(params, G.state_dict("net"), **cfg)
    worst = 0.0
    for t in range(meta["n_steps"]):
        opt.step(grads[t])
        for i, p in enumerate(params):
            got = {"param": p, "mom": opt.state[i]["mom"], "rms": opt.state[i]["rms"]}
            if p.dim() >= 2:
                got["fac_r"], got["fac_c"] = opt.state[i]["fac_r"], opt.state[i]["fac_c"]
            elif not cfg.get("use_adamw_for_1d", True):
                got["fac_v"] = opt.state[i]["fac_v"]
            for k, v in got.items():
                if meta["full"]:
                    e = max_err(v, G.t(f"step{t}/{k}/{i}"), REL, ABS)
                else:
                    e = max_err(v.reshape(-1)[::meta["sample"]], G.t(f"step{t}/{k}/{i}/sample"), REL, ABS)
                    nrm = float(torch.linalg.norm(v.double()))
                    ref = float(G.t(f"step{t}/{k}/{i}/norm"))
                    assert abs(nrm - ref) <= 1e-6 * ref + 1e-12, (t, k, i, nrm, ref)
                worst = max(worst, e)
                assert e <= 1.0, (name, t, k, i, e)
    print(name, "worst err / tol =", worst)


@pytest.mark.parametrize("name", ["celo2_small", "celo2_small_defaults"])
def test_celo2_oracle_matches_reference(name):
    """CELO2_naive: the ELO-CELO2 arithmetic with independent AdamW moments on the AdamW branch."""
    G = Golden(name)
    meta, shapes = G.meta, G.shapes
    init = [G.t(f"init/{i}") for i in range(len(shapes))]
    params = [v.clone() for v in init]
    cfg = dict(meta["cfg"])
    betas, eps = cfg.pop("adam_betas", (0.9, 0.95)), cfg.pop("adam_eps", 1e-8)
    for k, v in dict(weight_decay=0.0, clip_grad=False, adam_lr_mult=1.0).items():   # CELO2_naive defaults
        cfg.setdefault(k, v)
    opt = O.EloCelo2Oracle(params, G.state_dict("net"), independent_adam=(betas[0], betas[1], eps), **cfg)
    worst = 0.0
    for t in range(meta["n_steps"]):
        opt.step([G.t(f"grad{t}/{i}") for i in range(len(shapes))])
        for i, p in enumerate(params):
            st = opt.state[i]
            if p.dim() >= 2:
                got = {"param": p, "mom": st["mom"], "rms": st["rms"], "fac_r": st["fac_r"], "fac_c": st["fac_c"]}
            else:
                got = {"param": p, "exp_avg": st["exp_avg"], "exp_avg_sq": st["exp_avg_sq"]}
            for k, v in got.items():
                e = max_err(v, G.t(f"step{t}/{k}/{i}"), REL, ABS)
                worst = max(worst, e)
                assert e <= 1.0, (name, t, k, i, e)
    print(name, "worst err / tol =", worst)


@pytest.mark.parametrize("name", ["velo_small", "velo_small_wd"])
def test_velo_oracle_matches_reference(name):
    G = Golden(name)
    meta = G.meta
    shapes = G.shapes
    params = [G.t(f"init/{i}").clone() for i in range(len(shapes))]
    opt = O.VeloOracle(params, G.state_dict("rnn"), G.state_dict("mlp"), lr=meta["lr"],
                       num_steps=meta["num_steps"], weight_decay=meta["weight_decay"])
    for t in range(meta["n_steps"]):
        grads = [G.t(f"grad{t}/{i}") for i in range(len(shapes))]
        opt.step(grads, G.t(f"loss{t}"))
        assert max_err(opt.h, G.t(f"step{t}/lstm_h"), REL, ABS) <= 1.0, (t, "h")
        assert max_err(opt.c, G.t(f"step{t}/lstm_c"), REL, ABS) <= 1.0, (t, "c")
        for i, p in enumerate(params):
            st = opt.state[i]
            assert max_err(p, G.t(f"step{t}/param/{i}"), REL, ABS) <= 1.0, (t, i, "param")
            assert max_err(st["mom"], G.t(f"step{t}/mom/{i}"), REL, ABS) <= 1.0, (t, i, "mom")
            assert max_err(st["rms"], G.t(f"step{t}/rms/{i}"), REL, ABS) <= 1.0, (t, i, "rms")
            if "fac_vec_v" in st:
                assert max_err(st["fac_vec_v"], G.t(f"step{t}/fac_vec_v/{i}"), REL, ABS) <= 1.0
            else:
                dc, dr = O.factored_dims_velo(shapes[i])
                ref_r = trailing_to_keepdim(G.t(f"step{t}/fac_vec_row_trailing/{i}"), dr)
                ref_c = trailing_to_keepdim(G.t(f"step{t}/fac_vec_col_trailing/{i}"), dc)
                assert max_err(st["fac_vec_row"], ref_r, REL, ABS) <= 1.0, (t, i, "row")
                assert max_err(st["fac_vec_col"], ref_c, REL, ABS) <= 1.0, (t, i, "col")


@pytest.mark.parametrize("name", ["adafac_small", "adafac_small_wd", "adafac_max_norm"])
def test_adafac_oracle_matches_reference(name):
    G = Golden(name)
    meta = G.meta
    shapes = G.shapes
    params = [G.t(f"init/{i}").clone() for i in range(len(shapes))]
    opt = O.AdafacOracle(params, G.state_dict("net"), lr=meta["lr"], weight_decay=meta["weight_decay"],
                         **(meta.get("extra") or {}))
    for t in range(meta["n_steps"]):
        grads = [G.t(f"grad{t}/{i}") for i in range(len(shapes))]
        opt.step(grads)
        for i, p in enumerate(params):
            st = opt.state[i]
            assert max_err(p, G.t(f"step{t}/param/{i}"), REL, ABS) <= 1.0, (t, i, "param")
            assert max_err(st["exp_avg"], G.t(f"step{t}/exp_avg/{i}"), REL, ABS) <= 1.0, (t, i)
            assert max_err(st["exp_avg_sq"], G.t(f"step{t}/exp_avg_sq/{i}"), REL, ABS) <= 1.0, (t, i)
            if len(shapes[i]) < 2:
                assert max_err(st["exp_avg_sq_r"], G.t(f"step{t}/fac_vec_v/{i}"), REL, ABS) <= 1.0
            else:
                dc, dr = O.factored_dims(shapes[i])
                ref_r = trailing_to_keepdim(G.t(f"step{t}/fac_vec_row_trailing/{i}"), dr)
                ref_c = trailing_to_keepdim(G.t(f"step{t}/fac_vec_col_trailing/{i}"), dc)
                assert max_err(st["exp_avg_sq_r"], ref_r, REL, ABS) <= 1.0, (t, i, "row")
                assert max_err(st["exp_avg_sq_c"], ref_c, REL, ABS) <= 1.0, (t, i, "col")


@pytest.mark.parametrize("name", ["elo_small", "elo_small_nan"])
def test_elo_oracle_matches_reference(name):
    """ELO_naive: raw decays, global-norm clipping, NaN gradients zeroed, pre-step weight decay."""
    G = Golden(name)
    meta = G.meta
    shapes = G.shapes
    params = [G.t(f"init/{i}").clone() for i in range(len(shapes))]
    opt = O.EloOracle(params, G.state_dict("net"), lr=meta["lr"], weight_decay=meta["weight_decay"], **meta["extra"])
    saw_nan = False
    for t in range(meta["n_steps"]):
        grads = [G.t(f"grad{t}/{i}") for i in range(len(shapes))]
        saw_nan |= any(bool(torch.isnan(g).any()) for g in grads)
        opt.step(grads)
        for i, p in enumerate(params):
            st = opt.state[i]
            assert max_err(p, G.t(f"step{t}/param/{i}"), REL, ABS) <= 1.0, (t, i, "param")
            assert max_err(st["exp_avg"], G.t(f"step{t}/exp_avg/{i}"), REL, ABS) <= 1.0, (t, i)
            assert max_err(st["exp_avg_sq"], G.t(f"step{t}/exp_avg_sq/{i}"), REL, ABS) <= 1.0, (t, i)
            if len(shapes[i]) < 2:
                assert max_err(st["exp_avg_sq_r"], G.t(f"step{t}/fac_vec_v/{i}"), REL, ABS) <= 1.0
            else:
                dc, dr = O.factored_dims(shapes[i])
                ref_r = trailing_to_keepdim(G.t(f"step{t}/fac_vec_row_trailing/{i}"), dr)
                ref_c = trailing_to_keepdim(G.t(f"step{t}/fac_vec_col_trailing/{i}"), dc)
                assert max_err(st["exp_avg_sq_r"], ref_r, REL, ABS) <= 1.0, (t, i, "row")
                assert max_err(st["exp_avg_sq_c"], ref_c, REL, ABS) <= 1.0, (t, i, "col")
    assert saw_nan == (name == "elo_small_nan")
    assert all(bool(torch.isfinite(p).all()) for p in params)


def test_constructor_rng_order_matches_reference():
    """Freshly constructed product meta-nets under seed 1234 have the reference's weights."""
    from pylo_amd import models as M

    G = Golden("ctor_checksums")
    for cls, args in (("CELO2MLP", ()), ("MetaMLP", (39, 32, 1)), ("VeLOMLP", ()), ("VeLORNN", ())):
        torch.manual_seed(G.meta["seed"])
        mod = getattr(M, cls)(*args)
        sd = mod.state_dict()
        ref_keys = sorted(k.split("/", 1)[1] for k in G._z.files if k.startswith(cls + "/"))
        assert sorted(sd.keys()) == ref_keys, cls
        for k, v in sd.items():
            ref = G.t(f"{cls}/{k}").numpy()
            d = v.double()
            got = np.array([float(d.sum()), float((d * d).sum()), v.numel()])
            assert np.allclose(got, ref, rtol=1e-12, atol=1e-12), (cls, k, got, ref)
