"""Position encodings.  Rotary, half-split pairing (j, j + R/2) over the rotated width R:
angle = position * theta^(-2j/R) (llama3.rs:5367-5378; same pairing in src/rope.rs:12-27).

The angles' cosines and sines are tabulated once on the host in 64-bit and stored as 32-bit, so
the rotation itself is a 32-bit multiply-add in the kernel.  A position encoding serves the
attention mixer through `rotate_and_store`: rotate q and k, and put k and v into the cache in the
same pass, which saves one trip through memory for k.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..hip import ops
from .base import POSITIONS, Part, Precision


@POSITIONS.register("rope")
class RotaryEncoding(Part):
    graph_safe = True

    def __init__(self, precision: Precision, device, *, dim: int, theta: float, max_positions: int,
                 rotary_dim: Optional[int] = None):
        self.dim = dim
        self.rotary_dim = dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or self.rotary_dim > dim:
            raise ValueError(f"rotated width {self.rotary_dim} must be even and at most {dim}")
        self.theta = float(theta)
        self.max_positions = max_positions
        half = self.rotary_dim // 2
        j = torch.arange(half, dtype=torch.float64)
        inv_freq = self.theta ** (-2.0 * j / self.rotary_dim)
        ang = torch.arange(max_positions, dtype=torch.float64)[:, None] * inv_freq[None, :]
        self.cos = torch.cos(ang).to(torch.float32).to(device).contiguous()
        self.sin = torch.sin(ang).to(torch.float32).to(device).contiguous()

    def projection_row_order(self, num_heads: int, num_kv_heads: int, head_dim: int) -> Optional[torch.Tensor]:
        """A mixer that fuses its q, k and v projections may put the rows of every q and k head in pair order
        (rows j and j + d/2 at 2j and 2j + 1): the two elements of a rotated pair then leave the matrix product
        next to each other, in one lane of one tile, and the rotation can be its epilogue.  Returns the row
        permutation of the fused [q | k | v] matrix, or None where this does not apply (a partly rotated head).
        The mixer then passes pair_order=True to rotate_and_store."""
        if self.rotary_dim != head_dim or head_dim != self.dim or head_dim % 2:
            return None
        half = head_dim // 2
        one = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).flatten()      # 0, half, 1, half+1, ..
        heads = torch.arange(num_heads + num_kv_heads)[:, None] * head_dim + one[None, :]
        v0 = (num_heads + num_kv_heads) * head_dim
        return torch.cat([heads.flatten(), torch.arange(v0, v0 + num_kv_heads * head_dim)])

    def rotate_and_store(self, qkv: torch.Tensor, q_out: torch.Tensor, ctx, cache, *, num_heads: int,
                         num_kv_heads: int, head_dim: int, kv_layout: int = 0, pair_order: bool = False,
                         value_head_dim: Optional[int] = None) -> None:
        write = cache is not None and cache.writable
        ops.rope_cache_write(qkv, q_out, cache.k if write else None, cache.v if write else None,
                             self.cos, self.sin, ctx.positions, ctx.seq_of_token if write else None,
                             cache.block_table if write else None, num_heads=num_heads,
                             num_kv_heads=num_kv_heads, head_dim=head_dim, rotary_dim=self.rotary_dim,
                             max_position=ctx.max_position, kv_layout=kv_layout, interleaved=pair_order,
                             value_head_dim=value_head_dim)

    def project_rotate_store(self, proj, x, q_out: torch.Tensor, ctx, cache, *, num_heads: int, num_kv_heads: int,
                             head_dim: int, kv_layout: int, value_head_dim: Optional[int] = None) -> bool:
        """Projection (a Linear in the fragment layout with its rows in pair order), rotation and cache write as
        one kernel.  False where that kernel does not apply; the caller then takes the steps apart."""
        from .base import FragmentActs
        frag_in = isinstance(x, FragmentActs)
        if not (cache is not None and cache.writable and value_head_dim in (None, head_dim)
                and proj.layout == ops.LAYOUT_FRAG16 and proj.precision.act == torch.bfloat16 and head_dim % 16 == 0
                and (kv_layout == ops.KV_ROW or head_dim % 32 == 0)):
            return False
        ops.linear_rope_cache(x.data if frag_in else x, proj.weight, q_out, cache.k, cache.v, self.cos, self.sin,
                              ctx.positions, ctx.seq_of_token, cache.block_table, k_in=proj.k, num_heads=num_heads,
                              num_kv_heads=num_kv_heads, head_dim=head_dim, max_position=ctx.max_position,
                              kv_layout=kv_layout, rows=x.shape[0],
                              x_layout=ops.LAYOUT_FRAG16 if frag_in else ops.LAYOUT_ROW)
        return True


@POSITIONS.register("rope_pairs")
class RotaryPairs(Part):
    """Rotation in pairs of neighbouring dimensions (2i, 2i + 1), or of halves (i, i + R/2), over the first
    `rotary_dim` dimensions of every q and k head: the pair (u, v) at position p becomes
    (u cos a - v sin a, v cos a + u sin a), a = p * theta^(-2i / rotary_dim).  With `value_dim` the values are
    turned too, over all their dimensions and with frequencies of their own, theta^(-2m / value_dim), by their
    own position, and the attention kernel turns every head's output back by the query's position (so that a
    value enters the output turned by the distance).  The tables are made on the host in 64-bit and kept in
    32-bit; the attention mixer hands them to its kernels (`cos`, `sin`, `value_cos`, `value_sin`).

    `scaling` (factor s, original length L, fast, slow) stretches the frequencies of the q and k rotation for
    contexts beyond L, the slow ones most: with D(t) = R ln(L / (2 pi t)) / (2 ln theta), lo = max(floor D(fast), 0),
    hi = min(ceil D(slow), R - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the frequency becomes
    f_i / s * r_i + f_i (1 - r_i), and cos and sin are multiplied by 0.1 ln(s) + 1 (which the tables hold)."""
    graph_safe = True

    def __init__(self, precision: Precision, device, *, dim: int, theta: float, max_positions: int,
                 rotary_dim: Optional[int] = None, value_dim: Optional[int] = None, interleaved: bool = True,
                 scaling: Optional[dict] = None):
        self.dim = dim
        self.rotary_dim = dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= dim:
            raise ValueError(f"rotated width {self.rotary_dim} must be even and at most {dim}")
        if value_dim is not None and value_dim % 2:
            raise ValueError(f"turned values need an even size, found {value_dim}")
        self.theta, self.max_positions = float(theta), max_positions
        self.value_dim, self.interleaved = value_dim, bool(interleaved)
        self.scaling = None if not scaling else {k: float(scaling[k]) for k in ("factor", "original", "fast", "slow")}
        if self.scaling is not None and min(self.scaling.values()) <= 0:
            raise ValueError(f"stretched frequencies need positive factor, original, fast and slow, found {self.scaling}")
        self.cos, self.sin = self._tables(self.rotary_dim, device, self.scaling) if self.rotary_dim else (None, None)
        self.value_cos, self.value_sin = self._tables(value_dim, device) if value_dim else (None, None)

    def frequencies(self, width: int, scaling: Optional[dict] = None):
        """(the width / 2 frequencies in 64-bit, the factor of cos and sin)."""
        i = torch.arange(width // 2, dtype=torch.float64)
        f = self.theta ** (-2.0 * i / width)
        if scaling is None:
            return f, 1.0
        s, L = scaling["factor"], scaling["original"]
        at = lambda t: width * math.log(L / (2.0 * math.pi * t)) / (2.0 * math.log(self.theta))
        lo = max(math.floor(at(scaling["fast"])), 0)
        hi = min(math.ceil(at(scaling["slow"])), width - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / s * ramp + f * (1.0 - ramp), 0.1 * math.log(s) + 1.0

    def _tables(self, width: int, device, scaling: Optional[dict] = None):
        f, magnitude = self.frequencies(width, scaling)
        ang = torch.arange(self.max_positions, dtype=torch.float64)[:, None] * f[None, :]
        return ((torch.cos(ang) * magnitude).to(torch.float32).to(device).contiguous(),
                (torch.sin(ang) * magnitude).to(torch.float32).to(device).contiguous())


@POSITIONS.register("none")
class NoPositionEncoding(Part):
    graph_safe = True

    """No rotation: q passes through, k and v go to the cache unchanged."""

    def __init__(self, precision: Precision, device, **_):
        pass

    def rotate_and_store(self, qkv, q_out, ctx, cache, *, num_heads, num_kv_heads, head_dim, kv_layout=0,
                         value_head_dim=None) -> None:
        write = cache is not None and cache.writable
        ops.rope_cache_write(qkv, q_out, cache.k if write else None, cache.v if write else None, None, None,
                             ctx.positions, ctx.seq_of_token if write else None,
                             cache.block_table if write else None, num_heads=num_heads,
                             num_kv_heads=num_kv_heads, head_dim=head_dim, rotary_dim=0,
                             max_position=ctx.max_position, kv_layout=kv_layout, value_head_dim=value_head_dim)
