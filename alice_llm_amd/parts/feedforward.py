"""Feed-forwards.  Gated MLP: down( act(gate x) * (up x) ), the activation on the gate branch
(llama3.rs:14519-14540); for Gemma 2 the activation is the tanh form of GELU
(llama3.rs:6183-6186).  A second gated form, "swish_limited", bounds both branches first:
g = min(gate x, limit), u = clamp(up x, -limit, limit), y = g * sigmoid(1.702 g) * (u + 1); a third, "silu", is
silu(gate x) * (up x) with silu(z) = z * sigmoid(z).  gate and up are stacked into one matrix at load so that one kernel reads
the input once and applies the activation and the product in its epilogue.

Dense MLP: down( act(up x) ), the activation as the epilogue of the first product; "relu_squared" is
max(z, 0)^2.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import FEED_FORWARDS, ParamSpec, Part, Precision
from .linear import Linear

# both forms are the gated epilogue of the matrix products; its parameter picks the form (0: tanh-GELU times up;
# a positive limit: the limited swish form; ops.GATED_SILU: silu times up)
_GATED_EPILOGUES = {"gelu_tanh": ops.EPI_GEGLU, "swish_limited": ops.EPI_GEGLU, "silu": ops.EPI_GEGLU}
_DEFAULT_NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, hidden_size: int, intermediate_size: int, activation: str,
                 limit: Optional[float] = None, tensor_names: Optional[Dict[str, str]] = None):
        if activation not in _GATED_EPILOGUES:
            raise ValueError(f"gated_mlp has no kernel for activation '{activation}'; "
                             f"available: {sorted(_GATED_EPILOGUES)}")
        if (activation == "swish_limited") != (limit is not None) or (limit is not None and not limit > 0):
            raise ValueError("gated_mlp: 'swish_limited' takes a positive limit, and only it does")
        self.precision = precision
        self.H, self.I = hidden_size, intermediate_size
        self.names = dict(_DEFAULT_NAMES, **(tensor_names or {}))
        self.gate_up = Linear(hidden_size, intermediate_size, precision, epilogue=_GATED_EPILOGUES[activation],
                              epi_param=ops.GATED_SILU if activation == "silu" else float(limit or 0.0))
        self.down = Linear(intermediate_size, hidden_size, precision)
        self._parts: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["gate"]: ParamSpec((self.I, self.H)),
                n["up"]: ParamSpec((self.I, self.H)),
                n["down"]: ParamSpec((self.H, self.I))}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name == self.names["down"]:
            self.down.load(tensor)
        elif name in (self.names["gate"], self.names["up"]):
            self._parts[name] = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        g, u = (self.precision.matrix(self._parts.pop(self.names[n])) for n in ("gate", "up"))
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.gate_up.load(torch.cat([g, u], dim=0))

    def weight_bytes(self) -> int:
        return self.gate_up.nbytes() + self.down.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.gate_up.accepts_fragment_input

    def forward(self, x, ctx) -> torch.Tensor:
        # decode steps: the gated product goes to the down projection in fragment order as well
        frag = (getattr(ctx, "fragment_activations", False) and self.down.accepts_fragment_input
                and self.gate_up.can_write_fragments(x.shape[0]))
        h = self.gate_up(x, self.precision.act, out_fragments=frag)
        return self.down(h, torch.float32, allow_partials=True)


# the activations of the ungated form are the matrix products' one-element epilogue; its parameter picks the function
_UNARY_EPILOGUES = {"relu_squared": (ops.EPI_SOFTCAP, ops.UNARY_RELU2)}


@FEED_FORWARDS.register("dense_mlp")
class DenseMLP(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, hidden_size: int, intermediate_size: int, activation: str,
                 tensor_names: Optional[Dict[str, str]] = None):
        if activation not in _UNARY_EPILOGUES:
            raise ValueError(f"dense_mlp has no kernel for activation '{activation}'; available: {sorted(_UNARY_EPILOGUES)}")
        self.precision = precision
        self.H, self.I = hidden_size, intermediate_size
        self.names = dict({"up": "up_proj.weight", "down": "down_proj.weight"}, **(tensor_names or {}))
        epi, param = _UNARY_EPILOGUES[activation]
        self.up = Linear(hidden_size, intermediate_size, precision, epilogue=epi, epi_param=param)
        self.down = Linear(intermediate_size, hidden_size, precision)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.names["up"]: ParamSpec((self.I, self.H)), self.names["down"]: ParamSpec((self.H, self.I))}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name == self.names["up"]:
            self.up.load(tensor)
        elif name == self.names["down"]:
            self.down.load(tensor)
        else:
            raise KeyError(name)

    def weight_bytes(self) -> int:
        return self.up.nbytes() + self.down.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.up.accepts_fragment_input

    def forward(self, x, ctx) -> torch.Tensor:
        return self.down(self.up(x, self.precision.act), torch.float32, allow_partials=True)
