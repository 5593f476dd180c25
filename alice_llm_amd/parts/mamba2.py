"""The state-space mixer ("mamba2"): a recurrent layer whose state per head is a matrix with one decay a token.

With the mixer's input h, one projection gives [z | x | B | C | dt] (z, x: heads * P; B, C: groups * N; dt: heads).
x, B and C pass a short causal convolution per channel (`conv_taps` taps, the last the current token's, with a bias)
and silu.  Then per head, with the step dt = softplus(dt + dt_bias) and the head's group's B and C:
    S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T   (S: N x P),     y_t = S_t^T C_t + D x_t.
y (heads concatenated) is multiplied by silu(z), RMS-normed in `norm_groups` equal parts, multiplied by a weight, and
goes through the output matrix.  S starts at zero, lives in 32-bit in the cache's state rows, one per slot, beside
the convolution's last taps - 1 inputs, and both are carried from step to step; the step sizes, the decays, the
recurrence and the norm are 32-bit on both paths, from a projection whose sums are never rounded.

Head count, head and state sizes, groups, taps and the norm's eps are constructor arguments.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import MIXERS, CacheNeed, ParamSpec, Part, Precision, StateNeed
from .linear import Linear

_DEFAULT_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log", "D": "D",
                  "norm": "norm", "o": "o"}


@MIXERS.register("mamba2")
class StateSpaceMixer(Part):
    graph_safe = True
    graph_safe_prompts = True        # the kernels find each sequence's rows and state rows on the device

    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, num_heads: int, value_head_dim: int,
                 state_dim: int, groups: int = 1, norm_groups: int = 1, conv_taps: int = 4, norm_eps: float = 1e-6,
                 tensor_names: Optional[Dict[str, str]] = None):
        self.precision = precision
        self.W, self.nH, self.P, self.N, self.G = hidden_size, num_heads, int(value_head_dim), int(state_dim), int(groups)
        self.norm_groups, self.taps, self.eps = int(norm_groups), int(conv_taps), float(norm_eps)
        if min(self.nH, self.P, self.N, self.G, self.norm_groups) < 1 or self.nH % self.G:
            raise ValueError(f"mamba2: heads {self.nH}, sizes {self.P} and {self.N}, groups {self.G}: at least 1, groups divide heads")
        if self.N > ops.RECURRENCE_MAX_KEY_DIM or not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"mamba2: state size {self.N} beyond {ops.RECURRENCE_MAX_KEY_DIM} or taps {self.taps} outside "
                             f"1..{ops.SHORT_CONV_MAX_TAPS}: outside the range of the kernels")
        self.inner = self.nH * self.P
        if self.inner % self.norm_groups:
            raise ValueError(f"mamba2: {self.norm_groups} norm groups must divide heads * value size {self.inner}")
        self.channels = self.inner + 2 * self.G * self.N                       # what the convolution covers: x | B | C
        self.cols = 2 * self.inner + 2 * self.G * self.N + self.nH             # z | x | B | C | dt
        self.dt_col = self.cols - self.nH
        self.row = -(-self.cols // 4) * 4                                      # rows of whole 16-byte units
        self.names = dict(_DEFAULT_NAMES, **(tensor_names or {}))
        self.proj = Linear(hidden_size, self.row, precision)
        self.o = Linear(self.inner, hidden_size, precision)
        self.small: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["in"]: ParamSpec((self.cols, self.W)), n["conv"]: ParamSpec((self.channels, self.taps), init_std=0.3),
                n["conv_bias"]: ParamSpec((self.channels,), init_std=0.1), n["dt_bias"]: ParamSpec((self.nH,), init_std=0.5),
                n["A_log"]: ParamSpec((self.nH,), init_std=0.5), n["D"]: ParamSpec((self.nH,), init_std=0.5),
                n["norm"]: ParamSpec((self.inner,), init_std=0.3), n["o"]: ParamSpec((self.W, self.inner))}

    def cache_need(self) -> CacheNeed:
        state = [StateNeed("S", (self.nH, self.N, self.P))]
        if self.taps > 1:
            state.append(StateNeed("conv", (self.channels, self.taps - 1)))
        return CacheNeed(state=tuple(state))

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        n = self.names
        if name == n["o"]:
            self.o.load(tensor)
        elif name == n["in"]:
            w = self.precision.matrix(tensor)
            if w.shape[0] < self.row:                         # the padding rows: zeros that nobody reads
                w = torch.cat([w, w.new_zeros(self.row - w.shape[0], w.shape[1])], dim=0)
            self.proj.load(w)
        elif name in (n["conv"], n["conv_bias"], n["dt_bias"], n["A_log"], n["D"], n["norm"]):
            self.small[name] = tensor.float().contiguous()    # what enters the recurrence is 32-bit
        else:
            raise KeyError(name)

    def weight_bytes(self) -> int:
        return self.proj.nbytes() + self.o.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.proj.accepts_fragment_input

    def forward(self, x, ctx, cache) -> torch.Tensor:
        T, n, dev = x.shape[0], self.names, self.proj.weight.device
        rows = self.proj(x, torch.float32)                   # [T, z | x | B | C | dt], nothing rounded
        conv = torch.empty((T, self.channels), dtype=torch.float32, device=dev)
        ops.short_conv(rows, self.inner, self.small[n["conv"]], self.small[n["conv_bias"]], cache.state.get("conv"), conv, ctx)
        step = torch.empty((T, self.nH), dtype=torch.float32, device=dev)
        decay = torch.empty_like(step)
        ops.ssm_prepare(rows, self.dt_col, self.small[n["dt_bias"]], self.small[n["A_log"]], step, decay)
        y = torch.empty((T, self.inner), dtype=torch.float32, device=dev)
        b_col = self.inner
        ops.matrix_recurrence(conv, b_col + self.G * self.N, conv, b_col, conv, 0, decay, step, self.small[n["D"]], y, ctx,
                              cache.state["S"], heads=self.nH, qk_heads=self.G, head_dim=self.N, value_head_dim=self.P,
                              delta=False, decay_per_channel=False,
                              columns_per_wave=ops.recurrence_columns(getattr(ctx, "rounded_seqs", 0) or ctx.n_seqs, self.nH, self.N, self.P))
        out = torch.empty((T, self.inner), dtype=self.precision.act, device=dev)
        ops.norm_gate(y, self.small[n["norm"]], out, parts=self.norm_groups, eps=self.eps, weight_shared=False,
                      gate=rows, gate_col=0, gate_act="silu")
        return self.o(out, torch.float32, allow_partials=True)
