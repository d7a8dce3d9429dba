"""Helpers shared by the parity tests: golden-fixture loading and error metrics."""

import json
import os

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


class Golden:
    """One ``tests/golden/<name>.npz`` fixture (written by tests/golden/make_golden.py)."""

    def __init__(self, name):
        z = np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False)
        self.meta = json.loads(bytes(z["meta_json"]).decode())
        self._z = z

    def __contains__(self, key):
        return key in self._z.files

    def t(self, key) -> torch.Tensor:
        return torch.from_numpy(np.array(self._z[key]))

    def state_dict(self, prefix):
        pre = prefix + "/"
        return {k[len(pre):]: self.t(k) for k in self._z.files if k.startswith(pre)}

    @property
    def shapes(self):
        return [tuple(s) for s in self.meta["shapes"]]


def max_err(a: torch.Tensor, b: torch.Tensor, rel=1e-5, abs_=1e-6) -> float:
    """max over elements of |a-b| / (abs + rel*|b|): <= 1 means within rel/abs tolerance."""
    a = a.detach().double().cpu().reshape(-1)
    b = b.detach().double().cpu().reshape(-1)
    assert a.shape == b.shape, (a.shape, b.shape)
    if a.numel() == 0:
        return 0.0
    return float(torch.max(torch.abs(a - b) / (abs_ + rel * torch.abs(b))))


def trailing_to_keepdim(vec: torch.Tensor, drop_dim: int) -> torch.Tensor:
    """naive factored accumulator (param dims minus one, decay last) -> (3, *shape with dim->1)."""
    return vec.movedim(-1, 0).unsqueeze(drop_dim + 1)


def step_keeping_raw(opt):
    """``opt.step()`` of an ELO-CELO2-family optimizer, returning copies of the raw per-element steps (what
    celo2_kernel.cu:280 writes to ``step_out``) taken between the fused call and the finishing call, which
    orthogonalises in place and leaves intermediate results in those buffers."""
    tensors = opt.fused_step()
    kept = [None if r is None else r.clone() for r in opt._raw]
    opt.finish_step(tensors)
    return kept
