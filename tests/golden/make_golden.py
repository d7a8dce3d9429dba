"""Write golden trajectories from the reference's *naive* optimizer classes.

Run in the build container only (it needs /root/reference, which never travels):

    python tests/golden/make_golden.py

The reference package cannot be imported normally (``pylo/__init__.py`` pulls in
``mup``, which is not installed), so the handful of modules needed are loaded by
path under bare namespace packages.  The outputs are data only -- inputs, meta-net
weights and the parameters / optimizer states after every step -- stored as
``tests/golden/*.npz`` (numeric arrays, loaded with ``allow_pickle=False``).

What each fixture pins: whole-``step()`` trajectories of ELO_CELO2_naive,
VeLO_naive and AdafacLO_naive (op order, the var_rms quirk, tie rules, RNG order
of the seeded meta-net initialisers), which no closed form fixes.
"""

import json
import os
import sys
import tempfile
import types

import numpy as np
import torch

REF = os.environ.get("PYLO_REFERENCE", "/root/reference")
OUT = os.path.dirname(os.path.abspath(__file__))


def _load_reference():
    for name in ("pylo", "pylo.optim", "pylo.models"):
        mod = types.ModuleType(name)
        mod.__path__ = [os.path.join(REF, *name.split("."))]
        sys.modules[name] = mod
    import importlib
    m = importlib.import_module
    return dict(
        CELO2MLP=m("pylo.models.CELO2_MLP").CELO2MLP,
        MetaMLP=m("pylo.models.Meta_MLP").MetaMLP,
        VeLOMLP=m("pylo.models.VeLO_MLP").VeLOMLP,
        VeLORNN=m("pylo.models.VeLO_RNN").VeLORNN,
        ELO_CELO2_naive=m("pylo.optim.ELO_CELO2_naive").ELO_CELO2_naive,
        CELO2_naive=m("pylo.optim.CELO2_naive").CELO2_naive,
        VeLO_naive=m("pylo.optim.Velo_naive").VeLO_naive,
        AdafacLO_naive=m("pylo.optim.AdafacLO_naive").AdafacLO_naive,
        ELO_naive=m("pylo.optim.ELO_naive").ELO_naive,
    )


def _np(t):
    return t.detach().cpu().numpy().copy()


def _to_leading(t, p_dim):
    """naive state has the decay axis last; fixtures store it first (the CUDA classes' layout)."""
    return t.movedim(-1, 0) if t.dim() == p_dim + 1 else t


def _save(name, arrays, meta):
    arrays["meta_json"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    path = os.path.join(OUT, name + ".npz")
    np.savez_compressed(path, **arrays)
    print(f"{name}: {len(arrays)} arrays, {os.path.getsize(path) / 1024:.1f} KiB")


def _sd_arrays(prefix, module, arrays):
    for k, v in module.state_dict().items():
        arrays[f"{prefix}/{k}"] = _np(v)


# ------------------------------------------------------------------ ELO-CELO2
def celo2_case(R, name, shapes, n_steps, grad_scale, seed, cfg, net_seed=1, full=True, sample=4099,
               init_std=1.0, cls="ELO_CELO2_naive"):
    torch.manual_seed(net_seed)
    net = R["CELO2MLP"]()
    gen = torch.Generator().manual_seed(seed)
    init = [torch.randn(s, generator=gen) * init_std for s in shapes]
    params = [torch.nn.Parameter(v.clone()) for v in init]
    opt = R[cls](params, network=net, hf_key=None, **cfg)
    arrays = {}
    _sd_arrays("net", net, arrays)
    meta = dict(kind="elo_celo2" if cls == "ELO_CELO2_naive" else "celo2", shapes=[list(s) for s in shapes], n_steps=n_steps, cfg=cfg,
                grad_scale=grad_scale, seed=seed, net_seed=net_seed, full=full, sample=sample,
                init_std=init_std)
    if full:
        for i, v in enumerate(init):
            arrays[f"init/{i}"] = _np(v)
    for t in range(n_steps):
        grads = [torch.randn(s, generator=gen) * grad_scale for s in shapes]
        for p, g in zip(params, grads):
            p.grad = g.clone()
        opt.step()
        for i, p in enumerate(params):
            st = opt.state[p]
            if "exp_avg" in st:   # CELO2_naive: tensors on the AdamW branch keep their own two moments
                rec = {"param": p.detach(), "exp_avg": st["exp_avg"], "exp_avg_sq": st["exp_avg_sq"]}
            else:
                rec = {"param": p.detach(), "mom": _to_leading(st["mom"], p.dim()),
                       "rms": st["rms"][..., 0]}
            if "exp_avg" not in st and st["fac_vec_v"].numel():
                rec["fac_v"] = st["fac_vec_v"].movedim(-1, 0)
            if p.dim() >= 2 and "exp_avg" not in st:
                # naive fac_vec_row (mean over dr, decay last) -> (3,*s with dr->1)
                sorted_dims = np.argsort(p.shape)
                dc, dr = int(sorted_dims[-2]), int(sorted_dims[-1])
                rec["fac_r"] = st["fac_vec_row"].movedim(-1, 0).unsqueeze(dr + 1)
                rec["fac_c"] = st["fac_vec_col"].movedim(-1, 0).unsqueeze(dc + 1)
            for k, v in rec.items():
                if full:
                    arrays[f"step{t}/{k}/{i}"] = _np(v)
                    if k == "param":
                        arrays[f"grad{t}/{i}"] = _np(grads[i])
                else:
                    flat = v.reshape(-1)
                    arrays[f"step{t}/{k}/{i}/sample"] = _np(flat[::sample])
                    arrays[f"step{t}/{k}/{i}/norm"] = np.array(
                        [float(torch.linalg.norm(flat.double()))], dtype=np.float64)
    _save(name, arrays, meta)


# ---------------------------------------------------------------------- VeLO
_DTYPES = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def velo_case(R, name, shapes, n_steps, grad_scale, seed, num_steps, weight_decay, lr,
              lstm_hidden=64, param_inits=32, dtype="float32"):
    """`dtype`: the parameters' and gradients' element type.  The naive class keeps its accumulators in
    float32 and computes in whatever torch's type promotion gives; arrays are stored widened to float32."""
    dt = _DTYPES[dtype]
    # A reduced LSTM width / bank size keeps the fixture small; both classes read the sizes
    # from the saved config.json, and the arithmetic does not depend on them.
    torch.manual_seed(11)
    rnn = R["VeLORNN"](lstm_hidden_size=lstm_hidden, param_inits=param_inits)
    with torch.no_grad():                       # non-trivial initial LSTM state and lr head
        rnn.lstm_init_state[0].normal_(0, 0.1)
        rnn.lstm_init_state[1].normal_(0, 0.1)
    torch.manual_seed(12)
    mlp = R["VeLOMLP"](param_inits=param_inits)
    with torch.no_grad():                       # non-zero biases in the bank
        for n_, p_ in mlp.named_parameters():
            if "bias_" in n_:
                p_.normal_(0, 0.5)
    tmp = tempfile.mkdtemp()
    rnn.save_pretrained(os.path.join(tmp, "rnn"))
    mlp.save_pretrained(os.path.join(tmp, "mlp"))
    gen = torch.Generator().manual_seed(seed)
    init = [(torch.randn(s, generator=gen) * 0.5).to(dt) for s in shapes]
    params = [torch.nn.Parameter(v.clone()) for v in init]
    opt = R["VeLO_naive"](params, lr=lr, num_steps=num_steps, weight_decay=weight_decay,
                          hf_key_rnn=os.path.join(tmp, "rnn"), hf_key_mlp=os.path.join(tmp, "mlp"))
    arrays = {}
    _sd_arrays("rnn", rnn, arrays)
    _sd_arrays("mlp", mlp, arrays)
    meta = dict(kind="velo", shapes=[list(s) for s in shapes], n_steps=n_steps, seed=seed,
                num_steps=num_steps, weight_decay=weight_decay, lr=lr, grad_scale=grad_scale,
                lstm_hidden=lstm_hidden, param_inits=param_inits, dtype=dtype)
    for i, v in enumerate(init):
        arrays[f"init/{i}"] = _np(v.float())
    for t in range(n_steps):
        grads = [(torch.randn(s, generator=gen) * grad_scale).to(dt) for s in shapes]
        loss = torch.tensor(2.0 * np.exp(-t / 5.0) + 0.1 + 0.05 * ((t * 7) % 3), dtype=torch.float32)
        for p, g in zip(params, grads):
            p.grad = g.clone()
        opt.step(loss)
        arrays[f"loss{t}"] = _np(loss)
        arrays[f"step{t}/lstm_h"] = _np(opt.lstm_hidden_state[0])
        arrays[f"step{t}/lstm_c"] = _np(opt.lstm_hidden_state[1])
        for i, p in enumerate(params):
            st = opt.state[p]
            arrays[f"grad{t}/{i}"] = _np(grads[i].float())
            arrays[f"step{t}/param/{i}"] = _np(p.float())
            arrays[f"step{t}/mom/{i}"] = _np(st["mom"].movedim(-1, 0))
            arrays[f"step{t}/rms/{i}"] = _np(st["rms"].movedim(-1, 0))
            if st["fac_vec_v"].numel():
                arrays[f"step{t}/fac_vec_v/{i}"] = _np(st["fac_vec_v"].movedim(-1, 0))
            else:
                arrays[f"step{t}/fac_vec_row_trailing/{i}"] = _np(st["fac_vec_row"])
                arrays[f"step{t}/fac_vec_col_trailing/{i}"] = _np(st["fac_vec_col"])
    _save(name, arrays, meta)


# ------------------------------------------------------------------- AdafacLO
def adafac_case(R, name, shapes, n_steps, grad_scale, seed, weight_decay, lr, cls="AdafacLO_naive", extra=None,
                nan_at=(), dtype="float32"):
    """`extra`: further constructor arguments (ELO_naive: exp_mult, clip_grad, clip_norm, decays);
    `nan_at`: (step, tensor, flat index) triples where the gradient is NaN (ELO_naive zeroes them)."""
    torch.manual_seed(21)
    net = R["MetaMLP"](39, 32, 1)
    tmp = tempfile.mkdtemp()
    net.save_pretrained(os.path.join(tmp, "mlp"))
    gen = torch.Generator().manual_seed(seed)
    dt = _DTYPES[dtype]
    init = [(torch.randn(s, generator=gen) * 0.5).to(dt) for s in shapes]
    params = [torch.nn.Parameter(v.clone()) for v in init]
    extra = dict(extra or {})
    opt = R[cls](params, lr=lr, weight_decay=weight_decay, hf_key=os.path.join(tmp, "mlp"), **extra)
    arrays = {}
    _sd_arrays("net", net, arrays)
    meta = dict(kind="adafac" if cls == "AdafacLO_naive" else "elo", shapes=[list(s) for s in shapes],
                n_steps=n_steps, seed=seed, weight_decay=weight_decay, lr=lr, grad_scale=grad_scale, extra=extra,
                dtype=dtype)
    for i, v in enumerate(init):
        arrays[f"init/{i}"] = _np(v.float())
    for t in range(n_steps):
        grads = [(torch.randn(s, generator=gen) * grad_scale).to(dt) for s in shapes]
        for tt, ti, fi in nan_at:
            if tt == t:
                grads[ti].view(-1)[fi] = float("nan")
        for p, g in zip(params, grads):
            p.grad = g.clone()
        opt.step()
        for i, p in enumerate(params):
            st = opt.state[p]
            arrays[f"grad{t}/{i}"] = _np(grads[i].float())
            arrays[f"step{t}/param/{i}"] = _np(p.float())
            arrays[f"step{t}/exp_avg/{i}"] = _np(st["mom"].movedim(-1, 0))
            arrays[f"step{t}/exp_avg_sq/{i}"] = _np(st["rms"][..., 0])
            if st["fac_vec_v"].numel():
                arrays[f"step{t}/fac_vec_v/{i}"] = _np(st["fac_vec_v"].movedim(-1, 0))
            else:
                arrays[f"step{t}/fac_vec_row_trailing/{i}"] = _np(st["fac_vec_row"])
                arrays[f"step{t}/fac_vec_col_trailing/{i}"] = _np(st["fac_vec_col"])
    _save(name, arrays, meta)


def adafac_max_norm_case(R):
    """AdafacLO_naive with max_grad_norm (clip_grad_norm_ per parameter, AdafacLO_naive.py:199-200): gradients of
    N(0, 0.1) against a bound of 1.0 clip four tensors (norms 1.4 .. 3.8) and leave the two small ones alone."""
    adafac_case(R, "adafac_max_norm", [(20, 10), (20,), (40, 36), (6, 3, 4, 4), (16, 16), (3,)], 5, 0.1, 9,
                weight_decay=0.01, lr=0.5, extra=dict(max_grad_norm=1.0))


def ctor_checksums(R):
    """Sum and sum of squares (fp64) of every freshly constructed meta-net parameter under a fixed
    seed: pins the order in which the constructors draw from the RNG."""
    arrays = {}
    for cls, args in (("CELO2MLP", ()), ("MetaMLP", (39, 32, 1)), ("VeLOMLP", ()), ("VeLORNN", ())):
        torch.manual_seed(1234)
        mod = R[cls](*args)
        for k, v in mod.state_dict().items():
            d = v.double()
            arrays[f"{cls}/{k}"] = np.array([float(d.sum()), float((d * d).sum()), v.numel()])
    _save("ctor_checksums", arrays, dict(kind="ctor", seed=1234))


def stored_type_cases(R):
    """The naive classes on 16-bit parameters, where they run: AdafacLO_naive, ELO_naive and VeLO_naive keep
    float32 accumulators and let torch's type promotion decide the rest (g * g and the means over it are taken
    in the 16-bit type).  ELO_CELO2_naive and CELO2_naive raise a dtype error on any non-float32 parameter,
    and every naive class does on float64, so there is nothing to record for those."""
    adafac_case(R, "adafac_bf16", [(20, 10), (20,), (5, 20), (6, 3, 4, 4), (16, 16), (64, 128)], 5, 0.3, 51,
                weight_decay=0.01, lr=0.5, dtype="bfloat16")
    adafac_case(R, "elo_f16", [(20, 10), (20,), (6, 3, 4, 4), (40, 128)], 5, 0.3, 52, weight_decay=0.05, lr=1e-2,
                cls="ELO_naive", extra=dict(exp_mult=0.01, clip_grad=True, clip_norm=2.0), dtype="float16")
    velo_case(R, "velo_bf16", [(20, 10), (20,), (5, 20), (6, 3, 4, 4), (64, 128)], 5, 0.3, 53, num_steps=40,
              weight_decay=0.01, lr=1e-2, dtype="bfloat16")


def main():
    R = _load_reference()
    torch.set_num_threads(8)
    if "--stored-types-only" in sys.argv:
        return stored_type_cases(R)
    if "--max-norm-only" in sys.argv:
        return adafac_max_norm_case(R)
    # CELO2_naive (independent AdamW moments on 1-D tensors and is_embedding groups; CELO2_naive.py:263-283)
    celo2_case(R, "celo2_small", [(64, 32), (32, 64), (32,), (48, 24), (5,)], 8, 1.0, 12,
               dict(lr=1e-2, adam_lr_mult=3.0, weight_decay=0.02, adam_betas=(0.8, 0.9), adam_eps=1e-6,
                    clip_grad=True, clip_norm=2.0), cls="CELO2_naive")
    celo2_case(R, "celo2_small_defaults", [(40, 56), (7,), (24, 24)], 6, 0.1, 13, dict(lr=1e-3),
               cls="CELO2_naive")
    if "--celo2-only" in sys.argv:
        return
    # ELO_CELO2_naive on tensors with more than two dims (feature normalisers and Newton-Schulz per
    # slice of the last two dims) and with the MLP on 1-D tensors (use_adamw_for_1d=False)
    celo2_case(R, "elo_celo2_nd", [(6, 3, 4, 4), (2, 5, 3), (3, 16, 8), (12,), (20, 10), (4, 3, 70)], 6, 0.5, 41,
               dict(lr=1e-2, adam_lr_mult=5.0, exp_mult=0.01))
    celo2_case(R, "elo_celo2_mlp1d", [(20, 10), (12,), (5,), (200,), (3, 2, 2)], 6, 2.0, 42,
               dict(lr=1e-2, use_adamw_for_1d=False, clip_norm=3.0))
    if "--celo2-nd-only" in sys.argv:
        return
    # ELO_naive: AdafacLO's features and MLP, raw decays, global-norm clipping, nan_to_num, ELO update rule
    adafac_case(R, "elo_small", [(20, 10), (20,), (5, 20), (6, 3, 4, 4), (16, 16), (40, 128)], 6, 0.3, 31,
                weight_decay=0.05, lr=1e-2, cls="ELO_naive",
                extra=dict(exp_mult=0.01, clip_grad=True, clip_norm=2.0, initial_rms_decays=(0.99,)))
    adafac_case(R, "elo_small_nan", [(33, 17), (17,), (4, 3, 5)], 5, 1.0, 32, weight_decay=0.0, lr=1e-3,
                cls="ELO_naive", nan_at=((1, 0, 7), (1, 1, 3), (3, 2, 11), (3, 0, 100)))
    if "--elo-only" in sys.argv:
        return
    ctor_checksums(R)
    # shapes of the reference's own CUDA-vs-naive test (tests/test_celo2_cuda.py:38,116)
    celo2_case(R, "elo_celo2_small_clip", [(64, 32), (32, 64), (32,), (48, 24)], 10, 3.0, 2,
               dict(lr=1e-2, adam_lr_mult=20.0))
    celo2_case(R, "elo_celo2_small_noclip_exp", [(64, 32), (32, 64), (32,), (24, 24)], 10, 1e-3, 3,
               dict(lr=1e-3, adam_lr_mult=20.0, exp_mult=0.01, weight_decay=0.05, rmsmult=0.7))
    celo2_case(R, "elo_celo2_small_noortho", [(40, 56), (7,)], 8, 0.5, 4,
               dict(lr=1e-2, orthogonalize=False, clip_grad=False, adam_lr_mult=1.0))
    # BASELINE config 1: 1024x1024 weight + 1024 bias, N(0, 0.02) init, N(0, 1e-3) grads, 10 steps
    celo2_case(R, "elo_celo2_cfg1", [(1024, 1024), (1024,)], 10, 1e-3, 0,
               dict(lr=3.16e-4, weight_decay=0.1, adam_lr_mult=20.0), full=False, init_std=0.02)
    velo_case(R, "velo_small", [(20, 10), (20,), (5, 20), (5,), (6, 3, 4, 4), (16, 16), (1, 1, 12)],
              6, 0.3, 5, num_steps=40, weight_decay=0.0, lr=1e-2)
    velo_case(R, "velo_small_wd", [(33, 17), (17,)], 5, 2.0, 6, num_steps=10, weight_decay=0.01, lr=1e-3)
    adafac_case(R, "adafac_small", [(20, 10), (20,), (5, 20), (6, 3, 4, 4), (16, 16)], 6, 0.3, 7,
                weight_decay=0.0, lr=1.0)
    adafac_case(R, "adafac_small_wd", [(33, 17), (17,)], 5, 1e-3, 8, weight_decay=0.01, lr=0.5)
    adafac_max_norm_case(R)
    stored_type_cases(R)


if __name__ == "__main__":
    main()
