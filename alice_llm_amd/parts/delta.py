"""The gated-delta-rule mixer ("channel_delta"): a recurrent layer whose state per head is a matrix that is decayed per
key channel and corrected towards each new value.

With the mixer's input h: q = W_q h and k = W_k h (kv heads of size d), v = W_v h (heads of size P), each through a
short causal convolution per channel (`conv_taps` taps, the last the current token's, no bias) and silu; q and k are
made unit vectors per head, x / sqrt(sum x^2 + unit_eps), q also times d^(-1/2); beta = sigmoid(W_b h), one a head;
a decay per head and key channel g = exp(-exp(A_log) softplus(W_a2 (W_a1 h) + dt_bias)).  Per head (head h with the
q and k of kv head h // (heads / kv heads)):
    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q      (o is taken after the write).
Each head's o is divided by its root mean square (eps inside the root), multiplied by a weight of size P that the
heads share and by sigmoid(W_g2 (W_g1 h)), and goes through the output matrix.  S starts at zero, lives in 32-bit
in the cache's state rows, one per slot, beside the convolutions' last taps - 1 inputs, and both are carried from
step to step; decays, write strengths, unit vectors, the recurrence and the norm are 32-bit on both paths.

Head counts and sizes, taps, the widths of the two narrow middles and both eps are constructor arguments.  One fused
projection gives [q | k | v | b | W_a1 h | W_g1 h] in 32-bit; the second matrices are projections of their own.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import MIXERS, CacheNeed, ParamSpec, Part, Precision, StateNeed
from .linear import Linear

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "b": "b", "a1": "a1", "a2": "a2", "g1": "g1", "g2": "g2", "o": "o",
                  "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "dt_bias": "dt_bias", "A_log": "A_log", "norm": "norm"}


@MIXERS.register("channel_delta")
class ChannelDeltaMixer(Part):
    graph_safe = True
    graph_safe_prompts = True        # the kernels find each sequence's rows and state rows on the device

    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, num_heads: int, head_dim: int,
                 decay_rank: int, gate_rank: int, num_kv_heads: Optional[int] = None, value_head_dim: Optional[int] = None,
                 conv_taps: int = 4, norm_eps: float = 1e-6, unit_eps: float = 1e-6, tensor_names: Optional[Dict[str, str]] = None):
        self.precision = precision
        self.W, self.nH, self.d = hidden_size, num_heads, int(head_dim)
        self.nKV = num_heads if num_kv_heads is None else int(num_kv_heads)
        self.P = self.d if value_head_dim is None else int(value_head_dim)
        self.ra, self.rg, self.taps = int(decay_rank), int(gate_rank), int(conv_taps)
        self.eps, self.unit_eps = float(norm_eps), float(unit_eps)
        if min(self.nH, self.nKV, self.d, self.P, self.ra, self.rg) < 1 or self.nH % self.nKV:
            raise ValueError(f"channel_delta: heads {self.nH}, kv heads {self.nKV}, sizes {self.d} and {self.P}, middles {self.ra} and "
                             f"{self.rg}: at least 1, kv heads divide heads")
        if self.d > ops.RECURRENCE_MAX_KEY_DIM or not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"channel_delta: key size {self.d} beyond {ops.RECURRENCE_MAX_KEY_DIM} or taps {self.taps} outside "
                             f"1..{ops.SHORT_CONV_MAX_TAPS}: outside the range of the kernels")
        self.qk, self.vw = self.nKV * self.d, self.nH * self.P
        self.channels = 2 * self.qk + self.vw                                  # what the convolutions cover: q | k | v
        self.b_col = self.channels
        self.a_col = self.b_col + self.nH
        self.g_col = self.a_col + self.ra
        self.row = -(-(self.g_col + self.rg) // 4) * 4                         # rows of whole 16-byte units
        self.names = dict(_DEFAULT_NAMES, **(tensor_names or {}))
        self.proj = Linear(hidden_size, self.row, precision)
        self.decay = Linear(self.ra, self.nH * self.d, precision)
        self.gate = Linear(self.rg, self.vw, precision)
        self.o = Linear(self.vw, hidden_size, precision)
        self.small: Dict[str, torch.Tensor] = {}
        self.conv_w: Optional[torch.Tensor] = None
        self._parts: Dict[str, torch.Tensor] = {}

    def _order(self):
        return ["q", "k", "v", "b", "a1", "g1"]

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["q"]: ParamSpec((self.qk, self.W)), n["q_conv"]: ParamSpec((self.qk, self.taps), init_std=0.3),
                n["k"]: ParamSpec((self.qk, self.W)), n["k_conv"]: ParamSpec((self.qk, self.taps), init_std=0.3),
                n["v"]: ParamSpec((self.vw, self.W)), n["v_conv"]: ParamSpec((self.vw, self.taps), init_std=0.3),
                n["b"]: ParamSpec((self.nH, self.W)), n["A_log"]: ParamSpec((self.nH,), init_std=0.5),
                n["norm"]: ParamSpec((self.P,), init_std=0.3),
                n["a1"]: ParamSpec((self.ra, self.W)), n["a2"]: ParamSpec((self.nH * self.d, self.ra), init_std=0.3),
                n["dt_bias"]: ParamSpec((self.nH * self.d,), init_std=0.5),
                n["g1"]: ParamSpec((self.rg, self.W)), n["g2"]: ParamSpec((self.vw, self.rg), init_std=0.3),
                n["o"]: ParamSpec((self.W, self.vw))}

    def cache_need(self) -> CacheNeed:
        state = [StateNeed("S", (self.nH, self.d, self.P))]
        if self.taps > 1:
            state.append(StateNeed("conv", (self.channels, self.taps - 1)))
        return CacheNeed(state=tuple(state))

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        n = self.names
        if name == n["o"]:
            self.o.load(tensor)
        elif name == n["a2"]:
            self.decay.load(tensor)
        elif name == n["g2"]:
            self.gate.load(tensor)
        elif name in (n["dt_bias"], n["A_log"], n["norm"], n["q_conv"], n["k_conv"], n["v_conv"]):
            self.small[name] = tensor.float().contiguous()    # what enters the recurrence is 32-bit
        elif name in [n[c] for c in self._order()]:
            self._parts[name] = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        n = self.names
        mats = [self.precision.matrix(self._parts.pop(n[c])) for c in self._order()]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        w = torch.cat(mats, dim=0)
        if w.shape[0] < self.row:                             # the padding rows: zeros that nobody reads
            w = torch.cat([w, w.new_zeros(self.row - w.shape[0], w.shape[1])], dim=0)
        self.proj.load(w)
        self.conv_w = torch.cat([self.small.pop(n[c]) for c in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()

    def weight_bytes(self) -> int:
        return self.proj.nbytes() + self.decay.nbytes() + self.gate.nbytes() + self.o.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.proj.accepts_fragment_input

    def forward(self, x, ctx, cache) -> torch.Tensor:
        T, n, dev, act = x.shape[0], self.names, self.proj.weight.device, self.precision.act
        rows = self.proj(x, torch.float32)                   # [T, q | k | v | b | a | g], nothing rounded
        conv = torch.empty((T, self.channels), dtype=torch.float32, device=dev)
        ops.short_conv(rows, 0, self.conv_w, None, cache.state.get("conv"), conv, ctx)
        # the second matrices of the decay and of the gate: their operands in the activation dtype
        z = self.decay(rows[:, self.a_col:self.a_col + self.ra].to(act).contiguous(), torch.float32)
        gate = self.gate(rows[:, self.g_col:self.g_col + self.rg].to(act).contiguous(), torch.float32)
        beta = torch.empty((T, self.nH), dtype=torch.float32, device=dev)
        ops.delta_prepare(conv, self.qk, z, self.small[n["dt_bias"]], self.small[n["A_log"]], rows, self.b_col, beta,
                          qk_heads=self.nKV, heads=self.nH, head_dim=self.d, unit_eps=self.unit_eps, q_scale=self.d ** -0.5)
        o = torch.empty((T, self.vw), dtype=torch.float32, device=dev)
        ops.matrix_recurrence(conv, 0, conv, self.qk, conv, 2 * self.qk, z, beta, None, o, ctx, cache.state["S"],
                              heads=self.nH, qk_heads=self.nKV, head_dim=self.d, value_head_dim=self.P, delta=True,
                              decay_per_channel=True,
                              columns_per_wave=ops.recurrence_columns(getattr(ctx, "rounded_seqs", 0) or ctx.n_seqs, self.nH, self.d, self.P))
        out = torch.empty((T, self.vw), dtype=act, device=dev)
        ops.norm_gate(o, self.small[n["norm"]], out, parts=self.nH, eps=self.eps, weight_shared=True, gate=gate, gate_col=0,
                      gate_act="sigmoid")
        return self.o(out, torch.float32, allow_partials=True)
