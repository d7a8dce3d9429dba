"""The theta converters (scripts/convert_celo2_checkpoint.py:53-84, scripts/convert_elo_checkpoint.py:46-66):
a synthetic Haiku-layout tree, evaluated with numpy as Haiku evaluates it (``x @ w + b`` with (in, out)
matrices), must give the same outputs as the converted torch container; the converted container packs
into the kernels' weight block; files written by the CLI load back through ``from_pretrained``.
"""

import numpy as np
import pytest
import torch

from pylo_amd import convert
from pylo_amd.models import CELO2_FEATURE_DIMS, CELO2MLP, MetaMLP, pack_celo2, pack_metamlp


def _celo2_tree(rng):
    mod = {f"w0__{i}": rng.standard_normal((k, 8)).astype(np.float32) for i, k in enumerate(CELO2_FEATURE_DIMS)}
    mod.update(b0=rng.standard_normal(8).astype(np.float32),
               w1=rng.standard_normal((8, 8)).astype(np.float32), b1=rng.standard_normal(8).astype(np.float32),
               w2=rng.standard_normal((8, 3)).astype(np.float32), b2=rng.standard_normal(3).astype(np.float32))
    return {"ff_mod_stack": {"celo2_mlp": mod}}, mod


def _elo_tree(rng):
    mod = dict(w0=rng.standard_normal((39, 32)).astype(np.float32), b0=rng.standard_normal(32).astype(np.float32),
               w1=rng.standard_normal((32, 32)).astype(np.float32), b1=rng.standard_normal(32).astype(np.float32),
               w2=rng.standard_normal((32, 2)).astype(np.float32), b2=rng.standard_normal(2).astype(np.float32))
    return {"nn": {"mlp": mod}}, mod


def test_celo2_theta_keeps_in_out_layout():
    rng = np.random.default_rng(0)
    tree, mod = _celo2_tree(rng)
    net = convert.celo2_from_theta(tree)
    xs = [rng.standard_normal((5, k)).astype(np.float32) for k in CELO2_FEATURE_DIMS]
    h = sum(x.astype(np.float64) @ mod[f"w0__{i}"] for i, x in enumerate(xs)) + mod["b0"]
    h = np.maximum(h, 0)
    h = np.maximum(h @ mod["w1"] + mod["b1"], 0)
    ref = h @ mod["w2"] + mod["b2"]
    got = net([torch.from_numpy(x) for x in xs]).detach().numpy()
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)
    for i in range(len(CELO2_FEATURE_DIMS)):
        assert torch.equal(net.w0[i], torch.from_numpy(mod[f"w0__{i}"]))      # no transpose
    packed = pack_celo2(net)
    assert packed.numel() == 347
    np.testing.assert_array_equal(packed[:240].reshape(30, 8).numpy(),
                                  np.concatenate([mod[f"w0__{i}"] for i in range(len(CELO2_FEATURE_DIMS))]))


def test_elo_theta_is_transposed_into_linear_layout():
    rng = np.random.default_rng(1)
    tree, mod = _elo_tree(rng)
    net = convert.metamlp_from_theta(tree)
    x = rng.standard_normal((7, 39)).astype(np.float32)
    h = np.maximum(x.astype(np.float64) @ mod["w0"] + mod["b0"], 0)
    h = np.maximum(h @ mod["w1"] + mod["b1"], 0)
    ref = h @ mod["w2"] + mod["b2"]
    np.testing.assert_allclose(net(torch.from_numpy(x)).detach().numpy(), ref, rtol=1e-5, atol=1e-5)
    assert torch.equal(net.network.input.weight, torch.from_numpy(mod["w0"]).t())
    assert pack_metamlp(net).numel() == 2466


def test_errors_name_the_leaf():
    rng = np.random.default_rng(2)
    tree, mod = _celo2_tree(rng)
    del mod["w0__3"]
    with pytest.raises(KeyError, match="w0__3"):
        convert.celo2_from_theta(tree)
    tree, mod = _elo_tree(rng)
    mod["w1"] = mod["w1"][:, :5]
    with pytest.raises(ValueError, match="linear_0.weight"):
        convert.metamlp_from_theta(tree)
    tree, _ = _elo_tree(rng)
    tree["other"] = {"w0": np.zeros((1, 1), np.float32)}
    with pytest.raises(ValueError, match="two leaves"):
        convert.metamlp_from_theta(tree)


def test_cli_round_trip(tmp_path):
    rng = np.random.default_rng(3)
    tree, _ = _celo2_tree(rng)
    np.savez(tmp_path / "theta.npz", **dict(convert.flatten(tree)))
    assert convert.main(["celo2", "--input", str(tmp_path / "theta.npz"), "--output", str(tmp_path / "celo2")]) == 0
    ref = convert.celo2_from_theta(tree)
    back = CELO2MLP.from_pretrained(str(tmp_path / "celo2"))
    for (k, a), (_, b) in zip(ref.state_dict().items(), back.state_dict().items()):
        assert torch.equal(a, b), k
    tree, _ = _elo_tree(rng)
    np.savez(tmp_path / "elo.npz", **dict(convert.flatten(tree)))
    assert convert.main(["elo", "--input", str(tmp_path / "elo.npz"), "--output", str(tmp_path / "elo.pt")]) == 0
    net = MetaMLP(39, 32, 1)
    net.load_state_dict(torch.load(tmp_path / "elo.pt", weights_only=True))
    assert torch.equal(net.network.output.bias, convert.metamlp_from_theta(tree).network.output.bias)
    with pytest.raises(ValueError, match="allow-pickle"):
        convert.load_tree(str(tmp_path / "x.pickle"))
