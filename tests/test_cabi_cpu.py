"""The C-ABI library loads without a GPU and exports every symbol include/*.h declare (the boundary,
pylo_mi355.h, and the measurement instrumentation, pylo_mi355_bench.h);
host-only entry points (plan sizing, argument checks, error reporting) behave as documented."""

import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", n) for n in ("pylo_mi355.h", "pylo_mi355_bench.h")]


def _declared():
    text = "".join(open(h).read() for h in HEADERS)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pylo_mi355_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from pylo_amd import _lib

    lib = _lib.load()
    names = _declared()
    assert len(names) >= 12, names
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert lib.pylo_mi355_abi_version() == 9


def test_struct_sizes_match_header():
    from pylo_amd import _lib

    assert _lib.ARGS_DTYPE.itemsize == 8 * 8 + 8 * 4 + 2 * 4          # PyloTensorArgs
    assert C.sizeof(_lib.TensorShape) == 8 + 8 * 8
    assert C.sizeof(_lib.Decays) == 10 * 4            # 7 accumulator decays + adam_beta1/2, adam_eps
    assert C.sizeof(_lib.VeloNets) == 11 * 8 + 2 * 4
    assert C.sizeof(_lib.VeloStep) == 9 * 8 + 8 * 9 * 4


def test_workspace_sizing_and_error_paths_without_gpu():
    from pylo_amd import _lib

    lib = _lib.load()
    n = C.c_size_t(0)
    shapes = _lib.make_shapes([(50257, 768), (768,), (768, 2304)], [0, _lib.F_ADAM, 0])
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_CELO2, shapes, 3, C.byref(n)) == 0
    # partial sums and tables are a few % of the 154 MB tensor; the Newton-Schulz operand planes (two fp16
    # planes of X in both orientations, the second of them twice) add 12 bytes per matrix element
    n_mat = 50257 * 768 + 768 * 2304
    assert 12 * n_mat < n.value < 16 * n_mat
    # a CELO2 tensor with fewer than two dims and no AdamW flag takes the MLP (use_adamw_for_1d=False)
    mlp1d = _lib.make_shapes([(768,)], [0])
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_CELO2, mlp1d, 1, C.byref(n)) == 0
    # the independent-moment AdamW branch (CELO2_CUDA) is a tensor flag of its own
    indep = _lib.make_shapes([(768,), (64, 16)], [_lib.F_ADAM_INDEP, _lib.F_ADAM_INDEP])
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_CELO2, indep, 2, C.byref(n)) == 0
    # ELO_CUDA's tensor flags belong to AdafacLO plans; the global-norm flag is all-or-none
    elo = _lib.F_NAN_TO_NUM | _lib.F_WD_PRESTEP | _lib.F_GLOBAL_NORM
    ok = _lib.make_shapes([(64, 128), (128,), (4, 3, 5)], [elo, elo, elo])
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_ADAFAC, ok, 3, C.byref(n)) == 0
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_CELO2, ok, 1, C.byref(n)) != 0
    assert b"AdafacLO plans" in lib.pylo_mi355_last_error()
    for fl in ([elo, 0, elo], [0, elo, elo]):
        mixed = _lib.make_shapes([(64, 128), (128,), (4, 3, 5)], fl)
        assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_ADAFAC, mixed, 3, C.byref(n)) != 0
        assert b"PYLO_F_GLOBAL_NORM" in lib.pylo_mi355_last_error()
    # per-tensor norm clipping (AdafacLO's max_grad_norm): all-or-none too, AdafacLO plans only, and not together
    # with the global norm or nan_to_num
    tn = _lib.F_TENSOR_NORM
    ok = _lib.make_shapes([(64, 128), (128,), (4, 3, 5)], [tn, tn, tn])
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_ADAFAC, ok, 3, C.byref(n)) == 0
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_VELO, ok, 3, C.byref(n)) != 0
    assert b"AdafacLO plans" in lib.pylo_mi355_last_error()
    for fl, msg in (([tn, 0, tn], b"every tensor"), ([0, tn, tn], b"every tensor"),
                    ([tn | _lib.F_GLOBAL_NORM] * 3, b"does not combine"), ([tn | _lib.F_NAN_TO_NUM] * 3, b"does not combine")):
        bad = _lib.make_shapes([(64, 128), (128,), (4, 3, 5)], fl)
        assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_ADAFAC, bad, 3, C.byref(n)) != 0
        assert b"PYLO_F_TENSOR_NORM" in lib.pylo_mi355_last_error() and msg in lib.pylo_mi355_last_error()
    # tensors with more than two dims are fine for every kind
    nd = _lib.make_shapes([(768, 3, 16, 16)], [0])
    for kind in (_lib.KIND_VELO, _lib.KIND_ADAFAC, _lib.KIND_CELO2):
        assert lib.pylo_mi355_plan_workspace_bytes(kind, nd, 1, C.byref(n)) == 0
    # too large
    huge = _lib.make_shapes([(1 << 16, 1 << 16)], [0])
    assert lib.pylo_mi355_plan_workspace_bytes(_lib.KIND_VELO, huge, 1, C.byref(n)) != 0
    assert b"2^31" in lib.pylo_mi355_last_error()
    assert lib.pylo_mi355_plan_workspace_bytes(7, shapes, 3, C.byref(n)) != 0
    assert lib.pylo_mi355_plan_destroy(None) == 0
    # the graph-replay entry points refuse a null plan with a message instead of touching it
    table = C.c_void_p()
    assert lib.pylo_mi355_plan_arg_table(None, 0, C.byref(table)) != 0
    assert b"plan_arg_table" in lib.pylo_mi355_last_error()
    assert lib.pylo_mi355_plan_device_steps(None, None) != 0
    assert b"plan_device_steps" in lib.pylo_mi355_last_error()
    assert C.sizeof(_lib.DeviceSteps) == 8 + 3 * 8
    lib.pylo_mi355_stream_probe.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p]
    assert lib.pylo_mi355_stream_probe(None, None, 1024, 6, 5, 0, None) != 0
    assert b"stream_probe" in lib.pylo_mi355_last_error()


def test_optimizers_fail_loudly_without_gpu():
    import torch

    if torch.cuda.is_available():
        pytest.skip("this check is for GPU-less hosts")
    from pylo_amd import AdafacLO_CUDA, CELO2_CUDA, ELO_CELO2_CUDA, ELO_CUDA, VeLO_CUDA
    from pylo_amd.models import CELO2MLP, MetaMLP, VeLOMLP, VeLORNN

    p = [torch.nn.Parameter(torch.zeros(4, 4))]
    with pytest.raises(RuntimeError, match="requires a GPU"):
        ELO_CELO2_CUDA(p, network=CELO2MLP(), hf_key=None)
    with pytest.raises(RuntimeError, match="requires a GPU"):
        CELO2_CUDA(p, network=CELO2MLP(), hf_key=None)
    with pytest.raises(RuntimeError, match="requires a GPU"):
        VeLO_CUDA(p, rnn=VeLORNN(lstm_hidden_size=64, param_inits=8), mlp=VeLOMLP(param_inits=8))
    with pytest.raises(RuntimeError, match="requires a GPU"):
        AdafacLO_CUDA(p, network=MetaMLP(39, 32, 1))
    with pytest.raises(RuntimeError, match="requires a GPU"):
        ELO_CUDA(p, network=MetaMLP(39, 32, 1))


def test_weight_containers_round_trip_through_the_reference_file_format(tmp_path):
    """config.json + model.safetensors written by save_pretrained load back bit-identically, with
    the reference's parameter names."""
    import torch

    from pylo_amd.models import CELO2MLP, MetaMLP, VeLOMLP, VeLORNN

    torch.manual_seed(0)
    cases = [(CELO2MLP, {}), (MetaMLP, dict(input_size=39, hidden_size=32, hidden_layers=1)),
             (VeLOMLP, dict(param_inits=8)), (VeLORNN, dict(lstm_hidden_size=64, param_inits=8))]
    for cls, kw in cases:
        m = cls(**kw)
        d = tmp_path / cls.__name__
        m.save_pretrained(str(d))
        assert (d / "config.json").exists() and (d / "model.safetensors").exists()
        m2 = cls.from_pretrained(str(d))
        for (k1, v1), (k2, v2) in zip(m.state_dict().items(), m2.state_dict().items()):
            assert k1 == k2 and torch.equal(v1, v2), (cls.__name__, k1)
    keys = set(CELO2MLP().state_dict().keys())
    assert {"w0.0", "w0.13", "b0", "dense_w.0", "dense_b.1"} <= keys
    assert "network.linear_0.weight" in MetaMLP(39, 32, 1).state_dict()
    assert {"input_weights_", "hidden_weights_.0", "output_bias"} <= set(VeLOMLP(param_inits=4).state_dict())
    assert {"mix_layer1.weight", "lstm.linear.bias", "lstm_init_state.1", "step_size.weight"} <= \
        set(VeLORNN(lstm_hidden_size=64, param_inits=4).state_dict())


def test_reference_module_names_resolve_after_install():
    """``pylo_amd.compat.install()`` registers modules under the reference's extension-module names with
    its function names and argument lists (pylo/csrc/celo2_kernel.cu:352-357, learned_optimizer.cu:396-403,
    velo_kernel.cu:459-462)."""
    import importlib
    import inspect

    from pylo_amd import compat

    compat.install()
    want = {
        "celo2_cuda_kernel": ("celo2_kernel", 20),
        "cuda_lo": ("learned_optimizer_kernel", 24),
        "velo_cuda_kernel": ("velo_kernel_simple", 23),
    }
    for mod, (fn, nargs) in want.items():
        f = getattr(importlib.import_module(mod), fn)
        assert len(inspect.signature(f).parameters) == nargs, (mod, fn)
    import torch

    with pytest.raises((RuntimeError, TypeError)):       # CPU tensors are refused before anything is launched
        z = torch.zeros(4, 4)
        importlib.import_module("celo2_cuda_kernel").celo2_kernel(*([z] * 16), 0.0, 1, 0, 0)
