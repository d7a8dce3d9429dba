"""ctypes binding of ``libpylo_mi355.so`` (the C ABI declared in include/pylo_mi355.h).

There is no fallback: if the library is missing or a call fails, a RuntimeError is raised.
"""

from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Sequence

import numpy as np
import torch

from .build import LIB_PATH

MAX_DIMS = 8
KIND_CELO2, KIND_VELO, KIND_ADAFAC = 0, 1, 2
F_ADAM = 1
F_ADAM_INDEP = 2
F_NO_ORTHOGONALIZE = 64   # CELO2: no Newton-Schulz workspace for this tensor
F_NAN_TO_NUM, F_WD_PRESTEP, F_GLOBAL_NORM, F_TENSOR_NORM = 4, 8, 16, 32
ARG_ORTHOGONALIZE = 1      # PyloTensorArgs.flags
# storage type of a tensor's grad / param buffers (PYLO_F_STORE_*); accumulators and arithmetic stay fp32
STORE_FLAG = {torch.float32: 0, torch.float16: 0x100, torch.bfloat16: 0x200, torch.float64: 0x300}


def store_flag(p: torch.Tensor, who: str) -> int:
    """The PYLO_F_STORE_* tag of a parameter; its gradient must have the same type (torch sees to that)."""
    try:
        return STORE_FLAG[p.dtype]
    except KeyError:
        raise TypeError(f"{who}: parameters must be float32, float16, bfloat16 or float64, got {p.dtype}") from None


class TensorShape(C.Structure):
    _fields_ = [("ndim", C.c_int32), ("flags", C.c_int32), ("shape", C.c_int64 * MAX_DIMS)]


class Decays(C.Structure):
    _fields_ = [("beta_m", C.c_float * 3), ("beta_rms", C.c_float), ("beta_fac", C.c_float * 3),
                ("adam_beta1", C.c_float), ("adam_beta2", C.c_float), ("adam_eps", C.c_float)]


# numpy mirror of PyloTensorArgs (8 pointers, 8 floats, 2 ints, no padding)
ARGS_DTYPE = np.dtype([
    ("grad", np.uint64), ("param", np.uint64), ("mom", np.uint64), ("rms", np.uint64),
    ("fac_r", np.uint64), ("fac_c", np.uint64), ("fac_v", np.uint64), ("step_out", np.uint64),
    ("lr", np.float32), ("weight_decay", np.float32), ("clip_norm", np.float32),
    ("clip_val", np.float32), ("exp_mult", np.float32), ("step_mult", np.float32),
    ("bc1", np.float32), ("bc2", np.float32), ("group", np.int32), ("flags", np.int32),
])
assert ARGS_DTYPE.itemsize == 104
MAX_GROUPS = 8


class VeloNets(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("mix2_wt", "mix2_b", "fmix_wt", "fmix_b", "lstm_wt", "lstm_b",
                                          "ctrl_wt", "ctrl_b", "lr_w", "lr_b", "bank")] + \
               [("hidden", C.c_int32), ("n_bank", C.c_int32)]


class VeloStep(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("lstm_h", "lstm_c", "loss_means", "loss_running_min", "loss_decays",
                                          "loss_iteration", "loss", "controls_out", "lr_mult_out")] + \
               [("frac", (C.c_float * 9) * MAX_GROUPS)]

_lib = None


class DeviceSteps(C.Structure):
    _fields_ = [("counters", C.c_void_p), ("beta1", C.c_double), ("beta2", C.c_double),
                ("num_steps", C.c_double)]


def load():
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m pylo_amd.build` "
            "(there is no non-HIP fallback for the fused optimizer step)")
    lib = C.CDLL(LIB_PATH)
    lib.pylo_mi355_abi_version.restype = C.c_int
    lib.pylo_mi355_last_error.restype = C.c_char_p
    lib.pylo_mi355_plan_workspace_bytes.argtypes = [C.c_int, C.POINTER(TensorShape), C.c_int,
                                                    C.POINTER(C.c_size_t)]
    lib.pylo_mi355_plan_create.argtypes = [C.c_int, C.POINTER(TensorShape), C.c_int, C.c_void_p,
                                           C.c_size_t, C.c_void_p, C.POINTER(C.c_void_p)]
    lib.pylo_mi355_plan_destroy.argtypes = [C.c_void_p]
    lib.pylo_mi355_plan_num_launches.argtypes = [C.c_void_p]
    lib.pylo_mi355_plan_factored_dims.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int),
                                                  C.POINTER(C.c_int)]
    lib.pylo_mi355_plan_timing_begin.argtypes = [C.c_void_p, C.c_int]
    lib.pylo_mi355_plan_timing_end.argtypes = [C.c_void_p, C.POINTER(C.c_float), C.c_int, C.POINTER(C.c_int)]
    lib.pylo_mi355_plan_launch_name.argtypes = [C.c_void_p, C.c_int]
    lib.pylo_mi355_plan_launch_name.restype = C.c_char_p
    lib.pylo_mi355_celo2_step.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(Decays), C.c_void_p,
                                          C.c_void_p]
    lib.pylo_mi355_celo2_finish.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    lib.pylo_mi355_celo2_orthogonalize_finish.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_float), C.c_int,
                                                         C.c_float, C.c_void_p]
    lib.pylo_mi355_plan_orthogonalize_supported.argtypes = [C.c_void_p, C.c_int]
    lib.pylo_mi355_plan_finish_supported.argtypes = [C.c_void_p, C.c_int]
    lib.pylo_mi355_velo_step.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(Decays), C.POINTER(VeloNets),
                                         C.POINTER(VeloStep), C.c_void_p]
    lib.pylo_mi355_adafac_step.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(Decays), C.c_void_p, C.c_float,
                                           C.c_void_p]
    lib.pylo_mi355_plan_invalidate_statistics.argtypes = [C.c_void_p]
    lib.pylo_mi355_plan_statistics_stale.argtypes = [C.c_void_p]
    lib.pylo_mi355_plan_arg_table.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_void_p)]
    lib.pylo_mi355_plan_device_steps.argtypes = [C.c_void_p, C.POINTER(DeviceSteps)]
    if lib.pylo_mi355_abi_version() != 9:
        raise RuntimeError("libpylo_mi355.so: ABI version mismatch, rebuild it")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: {load().pylo_mi355_last_error().decode()}")


def make_shapes(shapes: Sequence[Sequence[int]], flags: Sequence[int]):
    arr = (TensorShape * len(shapes))()
    for i, (s, f) in enumerate(zip(shapes, flags)):
        if len(s) > MAX_DIMS:
            raise ValueError(f"tensors with more than {MAX_DIMS} dims are not supported")
        arr[i].ndim = len(s)
        arr[i].flags = int(f)
        for j, v in enumerate(s):
            arr[i].shape[j] = int(v)
    return arr


def make_decays(beta_m, beta_rms, beta_fac, adam_betas=(0.9, 0.95), adam_eps=1e-8) -> Decays:
    d = Decays()
    d.adam_beta1, d.adam_beta2, d.adam_eps = float(adam_betas[0]), float(adam_betas[1]), float(adam_eps)
    for k in range(3):
        d.beta_m[k] = float(beta_m[k])
        d.beta_fac[k] = float(beta_fac[k])
    d.beta_rms = float(beta_rms)
    return d


class Plan:
    """A launch plan over a fixed list of tensor shapes; owns its device workspace."""

    def __init__(self, kind: int, shapes: Sequence[Sequence[int]], flags: Sequence[int],
                 device: torch.device):
        lib = load()
        self.kind = kind
        self.n = len(shapes)
        self._shapes = make_shapes(shapes, flags)
        nbytes = C.c_size_t(0)
        check(lib.pylo_mi355_plan_workspace_bytes(kind, self._shapes, self.n, C.byref(nbytes)),
              "plan_workspace_bytes")
        self.workspace = torch.empty(max(int(nbytes.value), 256), dtype=torch.uint8, device=device)
        handle = C.c_void_p()
        with torch.cuda.device(device):
            stream = torch.cuda.current_stream(device).cuda_stream
            check(lib.pylo_mi355_plan_create(kind, self._shapes, self.n, self.workspace.data_ptr(),
                                             self.workspace.numel(), stream, C.byref(handle)),
                  "plan_create")
        self._h = handle
        self.args = np.zeros(self.n, dtype=ARGS_DTYPE)

    def factored_dims(self, i: int):
        dc, dr = C.c_int(), C.c_int()
        check(load().pylo_mi355_plan_factored_dims(self._h, i, C.byref(dc), C.byref(dr)), "factored_dims")
        return (dc.value, dr.value) if dc.value >= 0 else None

    @property
    def num_launches(self) -> int:
        return load().pylo_mi355_plan_num_launches(self._h)

    def launch_names(self) -> List[str]:
        lib = load()
        return [lib.pylo_mi355_plan_launch_name(self._h, i).decode() for i in range(self.num_launches)]

    def timing_begin(self, max_steps: int) -> None:
        check(load().pylo_mi355_plan_timing_begin(self._h, max_steps), "timing_begin")
        self._timing_cap = max_steps * self.num_launches

    def timing_end(self) -> np.ndarray:
        """(steps, num_launches) array of launch durations in ms, measured with HIP events."""
        buf = (C.c_float * self._timing_cap)()
        steps = C.c_int(0)
        check(load().pylo_mi355_plan_timing_end(self._h, buf, self._timing_cap, C.byref(steps)), "timing_end")
        nl = self.num_launches
        return np.array(buf[:steps.value * nl], dtype=np.float64).reshape(steps.value, nl)

    def pinned_table(self, slot: int) -> np.ndarray:
        """The plan's own pinned argument table `slot` as a structured array.  A call given this
        array reads it in place when it runs on the device, which is what a HIP graph needs: every
        replay sees the table as it is then.  Do not write it while such a run may be in flight."""
        tabs = self.__dict__.setdefault("_tables", {})
        if slot not in tabs:
            ptr = C.c_void_p()
            check(load().pylo_mi355_plan_arg_table(self._h, slot, C.byref(ptr)), "plan_arg_table")
            buf = (C.c_char * (ARGS_DTYPE.itemsize * self.n)).from_address(ptr.value)
            tabs[slot] = np.frombuffer(buf, dtype=ARGS_DTYPE, count=self.n)
        return tabs[slot]

    def device_steps(self, counters: Optional[torch.Tensor], beta1: float = 0.0, beta2: float = 0.0,
                     num_steps: float = 1.0) -> None:
        """Keep the step counters in `counters` (int32, on the device; held by the plan) and let
        the library derive bias corrections / time features from them; None switches that off."""
        ds = DeviceSteps()
        if counters is not None:
            if counters.dtype != torch.int32 or not counters.is_cuda or not counters.is_contiguous():
                raise TypeError("step counters must be a contiguous int32 tensor on the GPU")
            ds.counters, ds.beta1, ds.beta2, ds.num_steps = counters.data_ptr(), beta1, beta2, num_steps
        check(load().pylo_mi355_plan_device_steps(self._h, C.byref(ds)), "plan_device_steps")
        self._counters = counters

    def _table_ptr(self, args: Optional[np.ndarray]) -> int:
        return (self.args if args is None else args).ctypes.data

    def celo2_step(self, decays: Decays, mlp: torch.Tensor, stream: int, args: Optional[np.ndarray] = None) -> None:
        check(load().pylo_mi355_celo2_step(self._h, self._table_ptr(args), C.byref(decays),
                                           mlp.data_ptr(), stream), "celo2_step")

    def celo2_finish(self, args: np.ndarray, stream: int) -> None:
        """Normalise + apply after Newton-Schulz; `args` is a table like `self.args` (own array)."""
        check(load().pylo_mi355_celo2_finish(self._h, args.ctypes.data, stream), "celo2_finish")

    def invalidate_statistics(self) -> None:
        """VeLO: parameters or accumulators were written by someone else since the plan's last step."""
        check(load().pylo_mi355_plan_invalidate_statistics(self._h), "plan_invalidate_statistics")

    def statistics_stale(self) -> int:
        """VeLO: 0, or 1 + the index of a tensor whose carried sum of p^2 did not match the tensor (no wait)."""
        return load().pylo_mi355_plan_statistics_stale(self._h)

    def orthogonalize_supported(self, i: int) -> int:
        """0: not by the library; 1: by the tiled products (ns_iters > 0); 2: by the per-slice launches (any ns_iters)."""
        return load().pylo_mi355_plan_orthogonalize_supported(self._h, i)

    def finish_supported(self, i: int) -> bool:
        return load().pylo_mi355_plan_finish_supported(self._h, i) == 1

    def celo2_orthogonalize_finish(self, args: np.ndarray, coeffs, iters: int, eps: float, stream: int) -> None:
        """Newton-Schulz on the tensors flagged in `args["flags"]`, then normalise + apply for all of them."""
        c = (C.c_float * 3)(*[float(v) for v in coeffs])
        check(load().pylo_mi355_celo2_orthogonalize_finish(self._h, args.ctypes.data, c, int(iters), float(eps), stream),
              "celo2_orthogonalize_finish")

    def velo_step(self, decays: Decays, nets: VeloNets, step: VeloStep, stream: int,
                  args: Optional[np.ndarray] = None) -> None:
        check(load().pylo_mi355_velo_step(self._h, self._table_ptr(args), C.byref(decays), C.byref(nets),
                                          C.byref(step), stream), "velo_step")

    def adafac_step(self, decays: Decays, net: torch.Tensor, step: float, stream: int,
                    args: Optional[np.ndarray] = None) -> None:
        check(load().pylo_mi355_adafac_step(self._h, self._table_ptr(args), C.byref(decays), net.data_ptr(),
                                            float(step), stream), "adafac_step")

    def close(self):
        self.__dict__.pop("_tables", None)     # views of pinned memory that dies with the plan
        if getattr(self, "_h", None):
            load().pylo_mi355_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
