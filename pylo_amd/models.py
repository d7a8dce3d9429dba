"""Meta-network weight containers for the fused learned-optimizer step.

These modules exist to carry weights in the reference's on-disk format
(``config.json`` + ``model.safetensors`` via ``PyTorchModelHubMixin``) so that
``from_pretrained(<local dir>)`` / ``load_state_dict`` of reference-format files
work unchanged.  Parameter names, shapes, constructor kwargs and the order in
which the constructors draw from the RNG match the reference:

* ``MetaMLP``   -- pylo/models/Meta_MLP.py:29-54   (torch.nn.Linear layout, (out, in))
* ``CELO2MLP``  -- pylo/models/CELO2_MLP.py:50-123 (split first layer, (in, out) layout)
* ``VeLOMLP``   -- pylo/models/VeLO_MLP.py:41-142  (bank of ``param_inits`` weight sets)
* ``VeLORNN``   -- pylo/models/VeLO_RNN.py:16-135  (mixing layers + LSTM-512 + heads)

The optimizers never call ``forward`` on these modules: the weights are packed
into flat device buffers for the HIP kernels (see ``pack_*`` below).  ``forward``
is kept so the containers remain usable on their own.
"""

from __future__ import annotations

from collections import OrderedDict

import torch
import torch.nn as nn
import torch.nn.functional as F
from huggingface_hub import PyTorchModelHubMixin

CELO2_FEATURE_DIMS = (1, 1, 1, 3, 1, 3, 1, 3, 1, 3, 3, 3, 3, 3)

_HUB_KW = dict(license="apache-2.0", tags=["learned-optimizer"])


class MetaMLP(nn.Module, PyTorchModelHubMixin, **_HUB_KW):
    """input_size -> hidden (x hidden_layers+1) -> 2, ReLU between (AdafacLO / ELO / MuLO)."""

    def __init__(self, input_size, hidden_size, hidden_layers):
        super().__init__()
        layers = OrderedDict()
        layers["input"] = nn.Linear(input_size, hidden_size)
        layers["relu_input"] = nn.ReLU()
        for i in range(hidden_layers):
            layers[f"linear_{i}"] = nn.Linear(hidden_size, hidden_size)
            layers[f"relu_{i}"] = nn.ReLU()
        layers["output"] = nn.Linear(hidden_size, 2)
        self.network = nn.Sequential(layers)

    def forward(self, x):
        return self.network(x)


class CELO2MLP(nn.Module, PyTorchModelHubMixin, **_HUB_KW):
    """Split-input MLP of CELO2 / ELO-CELO2; weights are (in, out) and applied as ``x @ w``."""

    def __init__(self, feature_dims=CELO2_FEATURE_DIMS, hidden_size=8, hidden_layers=2,
                 output_size=3, activation="relu"):
        super().__init__()
        if activation not in ("relu", "tanh"):
            raise ValueError(f"Invalid MLP activation: {activation}")
        self.feature_dims = tuple(feature_dims)
        self.hidden_size = hidden_size
        self.hidden_layers = hidden_layers
        self.output_size = output_size
        self.activation = activation
        self.act_fn = torch.relu if activation == "relu" else torch.tanh
        self.w0 = nn.ParameterList(nn.Parameter(torch.empty(k, hidden_size)) for k in self.feature_dims)
        self.b0 = nn.Parameter(torch.zeros(hidden_size))
        widths = [hidden_size] * hidden_layers + [output_size]
        self.dense_w = nn.ParameterList()
        self.dense_b = nn.ParameterList()
        for fan_in, fan_out in zip(widths[:-1], widths[1:]):
            self.dense_w.append(nn.Parameter(torch.empty(fan_in, fan_out)))
            self.dense_b.append(nn.Parameter(torch.zeros(fan_out)))
        self.reset_parameters()

    def reset_parameters(self):
        """Truncated normal, std 1/sqrt(fan_in); fan_in of the split layer is the total width."""
        std0 = sum(self.feature_dims) ** -0.5
        for w in self.w0:
            nn.init.trunc_normal_(w, std=std0)
        for w in self.dense_w:
            nn.init.trunc_normal_(w, std=w.shape[0] ** -0.5)

    def forward(self, inps):
        acc = sum(x @ w for x, w in zip(inps, self.w0)) + self.b0
        acc = self.act_fn(acc)
        last = len(self.dense_w) - 1
        for i, (w, b) in enumerate(zip(self.dense_w, self.dense_b)):
            acc = acc @ w + b
            if i != last:
                acc = self.act_fn(acc)
        return acc


class VeLOMLP(nn.Module, PyTorchModelHubMixin, **_HUB_KW):
    """Bank of ``param_inits`` tiny MLPs (trailing underscore) plus the mixed working set."""

    def __init__(self, param_inits=256, input_size=30, hidden_size=4, hidden_layers=1, output_size=3):
        super().__init__()
        self.hidden_layers = hidden_layers

        def bank(*shape):
            return nn.Parameter(torch.randn(*shape))

        def zeros(*shape):
            return nn.Parameter(torch.zeros(*shape))

        for lead, suffix in (((param_inits,), "_"), ((), "")):
            setattr(self, "input_weights" + suffix, bank(*lead, hidden_size, input_size))
            setattr(self, "input_bias" + suffix, zeros(*lead, hidden_size))
            hw, hb = nn.ParameterList(), nn.ParameterList()
            for _ in range(hidden_layers):
                hw.append(bank(*lead, hidden_size, hidden_size))
                hb.append(zeros(*lead, hidden_size))
            setattr(self, "hidden_weights" + suffix, hw)
            setattr(self, "hidden_bias" + suffix, hb)
            setattr(self, "output_weights" + suffix, bank(*lead, output_size, hidden_size))
            setattr(self, "output_bias" + suffix, zeros(*lead, output_size))

    @staticmethod
    def _mix(control, bank):
        return (control.view([-1] + [1] * (bank.dim() - 1)) * bank).mean(0) * 100.0

    def update_params(self, control):
        """Working set <- 100 * mean_i(control_i * bank_i)."""
        self.input_weights.data.copy_(self._mix(control, self.input_weights_.data))
        self.input_bias.data.copy_(self._mix(control, self.input_bias_.data))
        for i in range(self.hidden_layers):
            self.hidden_weights[i].data.copy_(self._mix(control, self.hidden_weights_[i].data))
            self.hidden_bias[i].data.copy_(self._mix(control, self.hidden_bias_[i].data))
        self.output_weights.data.copy_(self._mix(control, self.output_weights_.data))
        self.output_bias.data.copy_(self._mix(control, self.output_bias_.data))

    def forward(self, x):
        x = F.relu(F.linear(x, self.input_weights, self.input_bias))
        for w, b in zip(self.hidden_weights, self.hidden_bias):
            x = F.relu(F.linear(x, w, b))
        return F.linear(x, self.output_weights, self.output_bias)


class _GateLSTM(nn.Module):
    """One Linear(2*in -> 4*hidden) producing gates in the order i, g, f, o; forget gate +1."""

    def __init__(self, input_size, hidden_size):
        super().__init__()
        self.linear = nn.Linear(2 * input_size, 4 * hidden_size)

    def forward(self, x, prev_state):
        h_prev, c_prev = prev_state
        i, g, f, o = self.linear(torch.cat((x, h_prev), dim=-1)).chunk(4, -1)
        c = torch.sigmoid(f + 1) * c_prev + torch.sigmoid(i) * torch.tanh(g)
        h = torch.sigmoid(o) * torch.tanh(c)
        return h, (h, c)


class VeLORNN(nn.Module, PyTorchModelHubMixin, **_HUB_KW):
    """Per-tensor LSTM of VeLO: features[T,30] -> (controls[T,param_inits], lr_mult[T], state)."""

    def __init__(self, input_size=30, lstm_hidden_size=512, param_inits=256, mix_layers=True):
        super().__init__()
        self.mix_layers = mix_layers
        self.mix_layer1 = nn.Linear(input_size, lstm_hidden_size)      # present in the files, unused
        self.mix_layer2 = nn.Linear(input_size, lstm_hidden_size)
        self.final_mix_layer = nn.Linear(input_size, lstm_hidden_size)
        self.lstm = _GateLSTM(lstm_hidden_size, lstm_hidden_size)
        self.rnn_to_controls = nn.Linear(lstm_hidden_size, param_inits)
        self.step_size = nn.Linear(lstm_hidden_size, 1)
        self.lstm_init_state = nn.ParameterList(
            nn.Parameter(torch.zeros(1, lstm_hidden_size)) for _ in range(2))

    def forward(self, x, state):
        if self.mix_layers:
            pooled = F.relu(self.mix_layer2(x)).max(dim=0, keepdim=True)[0]
            x = self.final_mix_layer(x) + pooled
        out, state = self.lstm(x, state)
        return self.rnn_to_controls(out), self.step_size(out).squeeze(-1), state


# ----------------------------------------------------------------------------
# flat fp32 packings handed to the kernels
# ----------------------------------------------------------------------------
def pack_celo2(net: CELO2MLP) -> torch.Tensor:
    """[w_in (30,8) | b_in 8 | w_h (8,8) | b_h 8 | w_out (8,3) | b_out 3] = 347 floats, (in,out)."""
    parts = [torch.cat([w.detach() for w in net.w0], dim=0), net.b0.detach(),
             net.dense_w[0].detach(), net.dense_b[0].detach(),
             net.dense_w[1].detach(), net.dense_b[1].detach()]
    return torch.cat([t.reshape(-1).float() for t in parts]).contiguous()


# AdafacLO's 28 features (g, p, m0..2, rms, m_k*rs, rs, fac_g_k, row_k, col_k, rsqrt(row_k), rsqrt(col_k),
# fac_mom_k; pylo/optim/AdafacLO_naive.py:261-300) in the kernels' 30-channel numbering, which also
# has clip(g) at 1 and g*rs at 14.
ADAFAC_CHANNELS = (0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 15, 16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26,
                   27, 28, 29)


def pack_metamlp(net: MetaMLP) -> torch.Tensor:
    """2466 floats, every matrix (in, out): w1 (30,32) in the 30-channel order (rows 1, 14 zero) | b1 32 |
    w_time (11,32) | w_h (32,32) | b_h 32 | w_o (32,2) | b_o 2."""
    seq = net.network
    w_in = seq.input.weight.detach().float()                 # (32, 39)
    if tuple(w_in.shape) != (32, 39) or not hasattr(seq, "linear_0") or hasattr(seq, "linear_1"):
        raise ValueError("the AdafacLO kernel supports MetaMLP(input_size=39, hidden_size=32, hidden_layers=1)")
    w1 = torch.zeros(30, 32, dtype=torch.float32, device=w_in.device)
    w1[list(ADAFAC_CHANNELS)] = w_in[:, :28].t()
    parts = [w1, seq.input.bias, w_in[:, 28:39].t(), seq.linear_0.weight.t(), seq.linear_0.bias,
             seq.output.weight.t(), seq.output.bias]
    return torch.cat([t.detach().float().reshape(-1) for t in parts]).contiguous()


def pack_velo_bank(net: VeLOMLP) -> torch.Tensor:
    """(param_inits, 159): per bank entry [W_in (4,30) | b_in 4 | W_h (4,4) | b_h 4 | W_out (3,4) | b_out 3]."""
    parts = [net.input_weights_, net.input_bias_, net.hidden_weights_[0], net.hidden_bias_[0],
             net.output_weights_, net.output_bias_]
    n = parts[0].shape[0]
    return torch.cat([t.detach().reshape(n, -1).float() for t in parts], dim=1).contiguous()
