"""MuLO_CUDA's regrouping (pylo/optim/MuLO_cuda.py:12-61) with stand-in ``infshape`` objects: matrix-like
parameters split by width multiplier with lr / multiplier, vector-like ones kept at the group's lr,
defaults filled as mup.optim.process_param_groups does.  ``impl`` is replaced so that no GPU is needed.
"""

import pytest
import torch

from pylo_amd import MuLO_CUDA


class _Inf:
    def __init__(self, ninf, width=1.0):
        self._n, self._w = ninf, width

    def ninf(self):
        return self._n

    def width_mult(self):
        return self._w


def _p(shape, ninf, width=1.0):
    p = torch.nn.Parameter(torch.zeros(shape))
    p.infshape = _Inf(ninf, width)
    return p


def _capture(groups, **kwargs):
    return groups, kwargs


def test_split_by_width_multiplier():
    a, b, c = _p((8, 8), 2, 4.0), _p((8, 4), 2, 2.0), _p((8, 8), 2, 4.0)
    v, e = _p((8,), 1), _p((100, 8), 1, 4.0)          # bias; embedding with one infinite dim
    groups, kw = MuLO_CUDA([a, b, v, c, e], impl=_capture, lr=0.8, step_mult=0.02)
    assert kw == dict(lr=0.8, step_mult=0.02)
    assert [len(g["params"]) for g in groups] == [2, 1, 2]
    assert groups[0]["params"][0] is a and groups[0]["params"][1] is c and groups[0]["lr"] == pytest.approx(0.2)
    assert groups[1]["params"][0] is b and groups[1]["lr"] == pytest.approx(0.4)
    assert groups[2]["params"] == [v, e] and groups[2]["lr"] == 0.8
    assert all(g["weight_decay"] == 0.0 for g in groups)


def test_existing_groups_keep_their_options():
    a, v = _p((8, 8), 2, 2.0), _p((8,), 1)
    b = _p((4, 4), 2, 8.0)
    groups, _ = MuLO_CUDA([dict(params=[a, v], lr=1.0, weight_decay=0.1, tag="x"), dict(params=[b])],
                          impl=_capture, lr=0.5, weight_decay=0.01)
    assert [(g["lr"], g["weight_decay"], len(g["params"])) for g in groups] == \
        [(0.5, 0.1, 1), (1.0, 0.1, 1), (0.5 / 8.0, 0.01, 1), (0.5, 0.01, 0)]
    assert groups[0]["tag"] == "x" and "tag" not in groups[2]


def test_errors():
    with pytest.raises(AssertionError, match="set_base_shapes"):
        MuLO_CUDA([torch.nn.Parameter(torch.zeros(2, 2))], impl=_capture, lr=1.0)
    with pytest.raises(NotImplementedError, match="more than 2 inf"):
        MuLO_CUDA([_p((2, 2, 2), 3)], impl=_capture, lr=1.0)
    with pytest.raises(KeyError):
        MuLO_CUDA([_p((2, 2), 2)], impl=_capture)      # lr is required, as in mup
