"""A routed feed-forward: a token is served by `top` of `experts` small gated feed-forwards.

Router logits z = R h + r in 32-bit; the `top` best-scoring experts serve the token (of equal logits the lower index
wins) and are mixed by a softmax restricted to those `top` logits: y = sum_e w_e down_e(act(gate_e h) * (up_e h)).  Tensors: "router", "router.b", and "e<i>.gate", "e<i>.up", "e<i>.down" for every expert.

The experts' gate and up matrices are stacked into one matrix at load, and their down matrices side by side into
another.  Steps of few tokens, the 32-bit path and sizes that suit no tile: one gated product gives every expert's
middle activations, each is multiplied by its expert's weight of that token (zero where the token does not use the
expert), and one down projection over all of them is the weighted sum.  Steps of many tokens in bfloat16: the (token,
expert) pairs are put in expert order on the device and each pair meets its own expert's matrices only (grouped
products over the same stacked matrices).  Every kernel's launch depends on sizes only, never on which experts the
tokens chose.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import FEED_FORWARDS, ParamSpec, Part, Precision
from .linear import Linear

_GATED = {"gelu_tanh": 0.0, "silu": ops.GATED_SILU}
GROUPED_FROM_TOKENS = 128      # steps of this many tokens and more take the grouped products (bfloat16, sizes that suit the tiles);
                               # below, one pass over all experts' matrices is as fast or faster (measured at 16 experts, 2 a token)
MIDDLE_ELEMENTS = 1 << 28      # the most middle activations (tokens x experts x their width) that a step holds at a time


@FEED_FORWARDS.register("expert_mlp")
class ExpertMLP(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, hidden_size: int, intermediate_size: int, experts: int, top: int,
                 activation: str = "silu", router_bias: bool = True):
        if activation not in _GATED:
            raise ValueError(f"expert_mlp has no kernel for activation '{activation}'; available: {sorted(_GATED)}")
        if not 1 <= top <= experts <= ops.ROUTER_MAX_EXPERTS:
            raise ValueError(f"expert_mlp: 1 <= top <= experts <= {ops.ROUTER_MAX_EXPERTS}, found top {top} of {experts}")
        self.precision = precision
        self.H, self.F, self.E, self.top = hidden_size, int(intermediate_size), int(experts), int(top)
        self.router_bias = bool(router_bias)
        self.router = Linear(hidden_size, self.E, precision)
        self.gate_up = Linear(hidden_size, self.E * self.F, precision, epilogue=ops.EPI_GEGLU, epi_param=_GATED[activation])
        self.down = Linear(self.E * self.F, hidden_size, precision)
        self.bias: Optional[torch.Tensor] = None
        self._parts: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs: Dict[str, ParamSpec] = {}
        for e in range(self.E):
            specs[f"e{e}.gate"] = ParamSpec((self.F, self.H))
            specs[f"e{e}.up"] = ParamSpec((self.F, self.H))
            specs[f"e{e}.down"] = ParamSpec((self.H, self.F))
        specs["router"] = ParamSpec((self.E, self.H), init_std=0.1)
        if self.router_bias:
            specs["router.b"] = ParamSpec((self.E,), init_std=0.1)
        return specs

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name == "router":
            self.router.load(tensor)
        elif name == "router.b" and self.router_bias:
            self.bias = tensor.float().contiguous()
        elif name in self.param_specs():
            self._parts[name] = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        take = lambda what: [self.precision.matrix(self._parts.pop(f"e{e}.{what}")) for e in range(self.E)]
        gate, up, down = take("gate"), take("up"), take("down")
        if len({m.dtype for m in gate + up}) > 1:
            gate, up = [m.float() for m in gate], [m.float() for m in up]
        if len({m.dtype for m in down}) > 1:
            down = [m.float() for m in down]
        self.gate_up.load(torch.cat(gate + up, dim=0))       # [all gates; all ups]: the gated product's stacked matrix
        self.down.load(torch.cat(down, dim=1).contiguous())  # [W, E F]: the experts' columns side by side

    def weight_bytes(self) -> int:
        return self.router.nbytes() + self.gate_up.nbytes() + self.down.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return False

    def forward(self, x, ctx) -> torch.Tensor:
        T, dev = x.shape[0], self.down.weight.device
        logits = self.router(x, torch.float32)
        weights = torch.empty((T, self.E), dtype=torch.float32, device=dev)
        ops.route_topk(logits, self.bias, weights, self.top)
        if (T >= GROUPED_FROM_TOKENS and self.gate_up.layout == ops.LAYOUT_FRAG16 and self.down.layout == ops.LAYOUT_FRAG16
                and ops.expert_products_supported(x.dtype, self.H, self.F)):
            # enough tokens that the experts' products pay: each (token, expert) pair meets its own expert only
            out = torch.empty((T, self.H), dtype=torch.float32, device=dev)
            ops.expert_products(x, weights, self.gate_up.weight, self.down.weight, out, expert_width=self.F, top=self.top,
                                epi_param=self.gate_up.epi_param)
            return out
        rows = max(1, MIDDLE_ELEMENTS // (self.E * self.F))
        if T <= rows:
            return self._experts(x, weights, True)
        out = torch.empty((T, self.H), dtype=torch.float32, device=dev)      # a long step: the tokens in runs, so that the middle stays small
        for a in range(0, T, rows):
            out[a:a + rows] = self._experts(x[a:a + rows], weights[a:a + rows], False)
        return out

    def _experts(self, x, weights, allow_partials: bool) -> torch.Tensor:
        mid = self.gate_up(x, torch.float32)                 # every expert's middle activations, not yet rounded
        scaled = torch.empty(mid.shape, dtype=self.precision.act, device=mid.device)
        ops.scale_columns(mid, weights, scaled)
        return self.down(scaled, torch.float32, allow_partials=allow_partials)
