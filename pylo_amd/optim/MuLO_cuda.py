"""MuLO_CUDA: the muP wrapper around the fused AdafacLO step (pylo/optim/MuLO_cuda.py:12-61).

Behaviour of the reference wrapper: inside every parameter group, parameters with two infinite
dimensions ("matrix-like") are regrouped by their muP width multiplier and the learning rate of each
such group is divided by the multiplier; all other parameters stay together at the group's learning
rate; three or more infinite dimensions are refused.  The regrouped list goes to ``AdafacLO_CUDA``
(or ``impl``).  Parameters carry ``infshape`` after ``mup.set_base_shapes``; only
``infshape.ninf()`` and ``infshape.width_mult()`` are read here, so the ``mup`` package (1.0.0 in the
reference's requirements) is not imported, and the defaults its ``process_param_groups`` fills in
(``lr`` from the keyword arguments, ``weight_decay`` 0 when absent) are set by ``_with_defaults``.
The fused step carries learning rates as per-tensor scalars: the split adds no launches.
"""

from __future__ import annotations

from .AdafacLO_cuda import AdafacLO_CUDA


def _with_defaults(params, kwargs):
    groups = list(params)
    if groups and not isinstance(groups[0], dict):
        groups = [dict(params=groups)]
    for group in groups:
        if "lr" not in group:
            group["lr"] = kwargs["lr"]
        group.setdefault("weight_decay", kwargs.get("weight_decay", 0.0))
    return groups


def _split_by_width(group):
    """[(options, params)]: one entry per width multiplier in order of first appearance, lr divided by
    it, then the vector-like parameters with the group's own options."""
    options = {k: v for k, v in group.items() if k != "params"}
    by_width, vectors = {}, []
    for p in group["params"]:
        shape = getattr(p, "infshape", None)
        if shape is None:
            raise AssertionError(f"A parameter with shape {tuple(p.shape)} does not have `infshape` attribute. "
                                 "Did you forget to call `mup.set_base_shapes` on the model?")
        n_inf = shape.ninf()
        if n_inf > 2:
            raise NotImplementedError("more than 2 inf dimensions")
        if n_inf == 2:
            by_width.setdefault(shape.width_mult(), []).append(p)
        else:
            vectors.append(p)
    out = [dict(options, lr=options["lr"] / width, params=ps) for width, ps in by_width.items()]
    out.append(dict(options, params=vectors))
    return out


def MuLO_CUDA(params, impl=AdafacLO_CUDA, **kwargs):
    groups = []
    for group in _with_defaults(params, kwargs):
        groups.extend(_split_by_width(group))
    return impl(groups, **kwargs)
