"""Meta-parameter trees of the JAX/Haiku learned optimizers -> the weight containers of this package.

Same layout rules as the reference's converters: CELO2's ``theta`` keeps Haiku's ``(in, out)``
matrices as they are (scripts/convert_celo2_checkpoint.py:53-84: ``w0__i -> w0.i``, ``b0``,
``w{j+1} / b{j+1} -> dense_w.j / dense_b.j``), ELO's dense MLP is transposed into
``torch.nn.Linear``'s ``(out, in)`` (scripts/convert_elo_checkpoint.py:46-66: ``w{j} / b{j}`` ->
``network.input, network.linear_*, network.output``).  A tree is any nesting of dicts whose leaves
are arrays; a leaf is found by the last component of its path.

    python -m pylo_amd.convert celo2 --input theta.npz --output celo2_dir
    python -m pylo_amd.convert elo   --input theta.npz --output elo_theta.pt

Inputs: ``.npz`` (flat ``a/b/leaf`` names, loaded without pickle) or ``.safetensors``; a ``.pickle``
checkpoint of the meta-training framework is only read with ``--allow-pickle`` (unpickling runs code
from the file: use it on your own checkpoints only).  Outputs: a ``.pt`` state_dict, as the reference
writes, or a directory in the ``config.json`` + ``model.safetensors`` format of ``from_pretrained``.
"""

from __future__ import annotations

import argparse
import os
from typing import Dict, Iterator, Tuple

import numpy as np
import torch

from .models import CELO2MLP, MetaMLP


def flatten(tree, prefix: str = "") -> Iterator[Tuple[str, np.ndarray]]:
    """(path, array) for every leaf of a nested dict."""
    if isinstance(tree, dict):
        for k, v in tree.items():
            yield from flatten(v, f"{prefix}/{k}" if prefix else str(k))
    else:
        yield prefix, np.asarray(tree)


def _leaves(tree) -> Dict[str, np.ndarray]:
    out = {}
    for name, arr in flatten(tree):
        key = name.split("/")[-1]
        if key in out:
            raise ValueError(f"two leaves are called {key!r}: pass the sub-tree of one network")
        out[key] = arr
    return out


def _put(sd, dst: str, leaves, src: str, transpose: bool = False) -> None:
    if src not in leaves:
        raise KeyError(f"the tree has no leaf {src!r} (needed for {dst})")
    t = torch.tensor(np.asarray(leaves[src]), dtype=torch.float32)
    if transpose:
        t = t.t().contiguous()
    if tuple(sd[dst].shape) != tuple(t.shape):
        raise ValueError(f"shape mismatch for {dst} <- {src}: {tuple(sd[dst].shape)} vs {tuple(t.shape)}")
    sd[dst] = t


def celo2_from_theta(tree, hidden_size: int = 8, hidden_layers: int = 2) -> CELO2MLP:
    leaves = _leaves(tree)
    model = CELO2MLP(hidden_size=hidden_size, hidden_layers=hidden_layers)
    sd = model.state_dict()
    for i in range(len(model.w0)):
        _put(sd, f"w0.{i}", leaves, f"w0__{i}")
    _put(sd, "b0", leaves, "b0")
    for j in range(len(model.dense_w)):
        _put(sd, f"dense_w.{j}", leaves, f"w{j + 1}")
        _put(sd, f"dense_b.{j}", leaves, f"b{j + 1}")
    model.load_state_dict(sd)
    return model


def metamlp_from_theta(tree, input_size: int = 39, hidden_size: int = 32, hidden_layers: int = 1) -> MetaMLP:
    leaves = _leaves(tree)
    model = MetaMLP(input_size=input_size, hidden_size=hidden_size, hidden_layers=hidden_layers)
    sd = model.state_dict()
    targets = ["network.input"] + [f"network.linear_{i}" for i in range(hidden_layers)] + ["network.output"]
    for j, dst in enumerate(targets):
        _put(sd, f"{dst}.weight", leaves, f"w{j}", transpose=True)
        _put(sd, f"{dst}.bias", leaves, f"b{j}")
    model.load_state_dict(sd)
    return model


def load_tree(path: str, allow_pickle: bool = False):
    if path.endswith(".npz"):
        with np.load(path, allow_pickle=False) as z:
            return {k: z[k] for k in z.files}
    if path.endswith(".safetensors"):
        from safetensors.numpy import load_file
        return load_file(path)
    if path.endswith((".pickle", ".pkl")):
        if not allow_pickle:
            raise ValueError("reading a pickle runs code from the file: pass --allow-pickle for your own checkpoints")
        import pickle
        with open(path, "rb") as f:
            return pickle.load(f)
    raise ValueError(f"unsupported input {path!r}: expected .npz, .safetensors or .pickle")


def save_model(model, path: str) -> None:
    if path.endswith((".pt", ".pth")):
        torch.save(model.state_dict(), path)
    else:
        os.makedirs(path, exist_ok=True)
        model.save_pretrained(path)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("kind", choices=["celo2", "elo"])
    ap.add_argument("--input", required=True)
    ap.add_argument("--output", required=True, help=".pt state_dict, or a directory for from_pretrained")
    ap.add_argument("--input-size", type=int, default=39)
    ap.add_argument("--hidden-size", type=int, default=None)
    ap.add_argument("--hidden-layers", type=int, default=None)
    ap.add_argument("--allow-pickle", action="store_true")
    a = ap.parse_args(argv)
    tree = load_tree(a.input, a.allow_pickle)
    if a.kind == "celo2":
        model = celo2_from_theta(tree, a.hidden_size or 8, a.hidden_layers or 2)
    else:
        model = metamlp_from_theta(tree, a.input_size, a.hidden_size or 32,
                                   1 if a.hidden_layers is None else a.hidden_layers)
    save_model(model, a.output)
    print(f"saved {type(model).__name__} ({sum(p.numel() for p in model.parameters())} parameters) to {a.output}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
