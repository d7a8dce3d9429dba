"""Shared argument handling of the single-tensor calls."""

from __future__ import annotations

import ctypes as C

import torch

from .. import _lib

_F = C.c_float
_P = C.c_void_p
_TAIL = [C.POINTER(C.c_int64), C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
_SIGS = {
    "pylo_mi355_celo2_kernel": [_P] * 16 + [_F] + _TAIL,
    "pylo_mi355_learned_optimizer_kernel": [_P] * 15 + [_F] * 6 + _TAIL,
    "pylo_mi355_velo_kernel_simple": [_P] * 15 + [_F] * 5 + _TAIL,
}
# the same calls with a leading element-type argument (what the reference's dispatch macro selects)
_SIGS.update({k + "_typed": [C.c_int] + v for k, v in list(_SIGS.items())})
_bound = set()


def entry(name: str):
    lib = _lib.load()
    fn = getattr(lib, name)
    if name not in _bound:
        fn.argtypes = _SIGS[name]
        fn.restype = C.c_int
        _bound.add(name)
    return fn


def pointers(who: str, device: torch.device, dtype: torch.dtype = torch.float32, **tensors) -> list:
    """Device pointers of contiguous tensors of `dtype` on `device` (``second_moment`` is always float32, as
    in the reference: celo2_kernel.cu:324); an empty tensor gives a null pointer (the reference passes nullptr
    for empty factor tensors, velo_kernel.cu:411-414)."""
    out = []
    for name, t in tensors.items():
        if not torch.is_tensor(t):
            raise TypeError(f"{who}: {name} must be a tensor")
        if t.numel() == 0:
            out.append(None)
            continue
        if not t.is_cuda or t.device != device:
            raise RuntimeError(f"{who}: {name} must live on {device}")
        want = torch.float32 if name == "second_moment" else dtype
        if t.dtype != want:
            raise TypeError(f"{who}: {name} must be {want} (got {t.dtype}); every array has the parameter's "
                            "element type, second_moment is float32")
        if not t.is_contiguous():
            raise RuntimeError(f"{who}: {name} must be contiguous")
        out.append(t.data_ptr())
    return out


def check_sizes(who: str, p: torch.Tensor, dc: int, dr: int, vector_like: int, n_stat: int, sizes: dict,
                weights: dict) -> None:
    """Element counts the kernels rely on (they index without bounds checks): per-element arrays, the
    three-decay accumulators, factor vectors with the dr / dc dim removed, `second_moment`, MLP arrays.
    `sizes` maps a name to (tensor, kind), kind in {"n", "3n", "row", "col", "stat"}."""
    n = p.numel()
    if vector_like:
        row = col = 3 * n
    else:
        if not (0 <= dc < p.dim() and 0 <= dr < p.dim()) or dc == dr:
            raise RuntimeError(f"{who}: dc / dr are not two dims of the tensor")
        row = 3 * n // max(p.shape[dr], 1)
        col = 3 * n // max(p.shape[dc], 1)
    want = {"n": n, "3n": 3 * n, "row": row, "col": col}
    for name, (t, kind) in sizes.items():
        if kind == "stat":
            if t.numel() < n_stat:
                raise RuntimeError(f"{who}: {name} needs at least {n_stat} elements")
        elif kind == "col" and vector_like:
            continue                      # not read for a vector-like tensor
        elif t.numel() != want[kind] and n > 0:
            raise RuntimeError(f"{who}: {name} has {t.numel()} elements, expected {want[kind]}")
    for name, (t, count) in weights.items():
        if t.numel() != count:
            raise RuntimeError(f"{who}: {name} has {t.numel()} elements, expected {count}")


def shape_args(p: torch.Tensor):
    arr = (C.c_int64 * max(p.dim(), 1))(*p.shape)
    return arr, p.dim()


def run(who: str, name: str, p: torch.Tensor, args: list) -> None:
    """Dispatch on the parameter's element type like the reference's AT_DISPATCH_FLOATING_TYPES_AND_HALF
    (celo2_kernel.cu:314): float32 takes the plain entry point, float16 / float64 (and bfloat16) the typed one."""
    with torch.cuda.device(p.device):
        stream = torch.cuda.current_stream(p.device).cuda_stream
        if p.dtype == torch.float32:
            _lib.check(entry(name)(*args, stream), who)
        else:
            _lib.check(entry(name + "_typed")(_lib.store_flag(p, who), *args, stream), who)
