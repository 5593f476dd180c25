"""The latent attention mixer: every head's keys and values are linear maps of one latent row a token.

With h the mixer's input, H heads, d plain and r rotated query/key dimensions a head, values of dv, ranks A (queries)
and R (keys and values):

    a  = N(Dq h; wq)                       the query latent, RMS-normed                                    [A]
    q  = Uq a, head by head [d plain | r rotated]; the rotated part turned by the position
    [c' | kr'] = Dkv h;  c = N(c'; wc)     the latent [R];  kr = kr' turned by the position, one part for all heads [r]
    k_h(j) = [Uk_h c(j) | kr(j)],  v_h(j) = Uv_h c(j)
    score_h(i, j) = scale * q_h(i) . k_h(j),  keys max(0, i + 1 - window) .. i, softmax, output matrix on the heads

Only [c | kr] is cached: R + r numbers a token, whatever the number of heads, as the one "kv head" of a row-major
page.  The per-head maps move to the query's side, where they cost one small product a token instead of one a key:

    score_h(i, j) = scale * ((Uk_h^T q_h,plain(i)) . c(j) + q_h,rot(i) . kr(j))
    out_h(i)      = Uv_h (sum_j w_h(i, j) c(j))

so the attention itself runs with one shared key row of R + r dimensions whose first R are also the value.  Norms,
rotation, scores and softmax are 32-bit; products round as the run's other matrices do.  Ranks, head sizes, scale,
window and eps are constructor arguments; `position` names a "rope_pairs" table over the r rotated dimensions.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import MIXERS, CacheNeed, KVNeed, ParamSpec, Part, Precision
from .linear import Linear

_DEFAULT_NAMES = {"dq": "q_a_proj.weight", "dq_norm": "q_a_norm.weight", "uq": "q_b_proj.weight",
                  "dkv": "kv_a_proj.weight", "dkv_norm": "kv_a_norm.weight", "uk": "k_b_proj.weight",
                  "uv": "v_b_proj.weight", "o": "o_proj.weight"}


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    graph_safe = True

    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, num_heads: int, head_dim: int,
                 rot_dim: int, value_head_dim: int, q_rank: int, kv_rank: int, scale: float, norm_eps: float,
                 window: Optional[int] = None, position: Optional[str] = None,
                 tensor_names: Optional[Dict[str, str]] = None):
        if rot_dim % 2 or rot_dim < 0:
            raise ValueError(f"latent_attention: the rotated part ({rot_dim}) must be even")
        if (position is None) != (rot_dim == 0):
            raise ValueError("latent_attention: a rotated part needs a position encoding, and only it does")
        if not 1 <= kv_rank <= ops.LATENT_MAX_RANK:
            raise ValueError(f"latent_attention: kv_rank {kv_rank} is outside 1..{ops.LATENT_MAX_RANK}, the range of "
                             f"the latent attention kernels")
        self.precision = precision
        self.H, self.nH, self.d, self.r, self.dv = hidden_size, num_heads, head_dim, rot_dim, value_head_dim
        self.A, self.R = q_rank, kv_rank
        self.scale, self.eps, self.window = float(scale), float(norm_eps), window
        self.position = positions[position] if position is not None else None
        if self.position is not None and getattr(self.position, "rotary_dim", None) != rot_dim:
            raise ValueError("latent_attention: the position encoding must turn the whole rotated part")
        self.names = dict(_DEFAULT_NAMES, **(tensor_names or {}))
        # one product for both down projections: rows [a' (A) | c' (R) | kr' (r)], the sums kept in 32-bit for the norms
        self.down = Linear(hidden_size, q_rank + kv_rank + rot_dim, precision)
        self.uq = Linear(q_rank, num_heads * (head_dim + rot_dim), precision)
        self.o = Linear(num_heads * value_head_dim, hidden_size, precision)
        self.w_q_norm: Optional[torch.Tensor] = None
        self.w_kv_norm: Optional[torch.Tensor] = None
        self.uk_t: Optional[torch.Tensor] = None        # [H, d, R]: head h's map from its plain query to the latent's space
        self.uv_t: Optional[torch.Tensor] = None        # [H, R, dv]: head h's value map, transposed
        self.uk_mfma = self.uv_mfma = False             # True: kept as [H, outputs, inputs] for the matrix-core kernel
        self._parts: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n, H = self.names, self.nH
        return {n["dq"]: ParamSpec((self.A, self.H)), n["dq_norm"]: ParamSpec((self.A,), init_std=0.1),
                n["uq"]: ParamSpec((H * (self.d + self.r), self.A)),
                n["dkv"]: ParamSpec((self.R + self.r, self.H)), n["dkv_norm"]: ParamSpec((self.R,), init_std=0.1),
                n["uk"]: ParamSpec((H * self.d, self.R)), n["uv"]: ParamSpec((H * self.dv, self.R)),
                n["o"]: ParamSpec((self.H, H * self.dv))}

    def cache_need(self) -> CacheNeed:
        # one row a token, [c | kr]; its first R numbers are the value too, so the pages hold no values of their own
        return CacheNeed(kv=KVNeed(1, self.R + self.r, self.window, value_head_dim=0))

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        n = self.names
        if name == n["o"]:
            self.o.load(tensor)
        elif name == n["uq"]:
            self.uq.load(tensor)
        elif name == n["dq_norm"]:
            self.w_q_norm = tensor.float().contiguous()
        elif name == n["dkv_norm"]:
            self.w_kv_norm = tensor.float().contiguous()
        elif name in (n["dq"], n["dkv"], n["uk"], n["uv"]):
            self._parts[name] = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        n, p = self.names, self.precision
        dq, dkv = p.matrix(self._parts.pop(n["dq"])), p.matrix(self._parts.pop(n["dkv"]))
        if dq.dtype != dkv.dtype:
            dq, dkv = dq.float(), dkv.float()
        self.down.load(torch.cat([dq, dkv], dim=0))
        uk, uv = p.matrix(self._parts.pop(n["uk"])), p.matrix(self._parts.pop(n["uv"]))
        if p.full:
            uk, uv = uk.float(), uv.float()
        # y[n] = sum_k wt[k, n] x[k]: for the keys' map x is the plain query (k = d, n = R), and Uk_h is [d, R] as stored
        self.uk_t = uk.reshape(self.nH, self.d, self.R).contiguous()
        self.uv_t = uv.reshape(self.nH, self.dv, self.R).transpose(1, 2).contiguous()
        # the matrix-core kernel reads a head's matrix [outputs, inputs]: only one of the two forms is kept
        self.uk_mfma = self.uv_mfma = False
        if not p.full and uk.dtype == torch.bfloat16:
            if ops.heads_linear_mfma_supported(uk.dtype, self.R, self.d, self.r):
                self.uk_t, self.uk_mfma = self.uk_t.transpose(1, 2).contiguous(), True
            if ops.heads_linear_mfma_supported(uv.dtype, self.dv, self.R):
                self.uv_t, self.uv_mfma = self.uv_t.transpose(1, 2).contiguous(), True

    def weight_bytes(self) -> int:
        small = sum(t.numel() * t.element_size() for t in (self.uk_t, self.uv_t))
        return self.down.nbytes() + self.uq.nbytes() + self.o.nbytes() + small

    def forward(self, x, ctx, cache) -> torch.Tensor:
        """x: [T, H] in the activation dtype; returns the branch in float32 ([T, H] or partial sums)."""
        T, act, dev = x.shape[0], self.precision.act, x.device
        nH, d, r, R, dv = self.nH, self.d, self.r, self.R, self.dv
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos is not None else (None, None)
        rows = self.down(x, torch.float32)
        a = torch.empty((T, self.A), dtype=act, device=dev)
        write = cache is not None and cache.writable
        ops.latent_prepare(rows, self.w_q_norm, self.w_kv_norm, a, cache.k if write else None, ctx.positions,
                           ctx.seq_of_token if write else None, cache.block_table if write else None,
                           q_rank=self.A, kv_rank=R, rot_dim=r, eps=self.eps, cos=cos, sin=sin,
                           max_position=ctx.max_position)
        q = self.uq(a, act)                                        # [T, H * (d + r)]
        qk = torch.empty((T, nH * (R + r)), dtype=act, device=dev)
        (ops.heads_linear_mfma if self.uk_mfma else ops.heads_linear)(
            q, self.uk_t, qk, heads=nH, n=R, k=d, rot_dim=r, cos=cos, sin=sin, positions=ctx.positions,
            max_position=ctx.max_position)
        mixed = torch.empty((T, nH * R), dtype=act, device=dev)
        if not self.precision.full and ops.latent_tiled_supported(act, R, r):
            # single tokens: few query rows and many keys, so the keys are spread over blocks; how many is chosen from
            # the step's sizes as a captured step rounds them, so that an eager step of the same tokens adds alike
            longest = getattr(ctx, "rounded_context", 0) or ctx.max_context
            most = longest if self.window is None else min(longest, self.window)
            splits = ops.latent_tiled_splits(getattr(ctx, "rounded_seqs", 0) or T, nH, most) if ctx.is_decode else 1
            ops.latent_attention_tiled(qk, cache.k, mixed, ctx, cache.block_table, num_heads=nH, kv_rank=R, rot_dim=r,
                                       scale=self.scale, window=self.window, splits=splits, single_tokens=ctx.is_decode)
        else:
            ops.latent_attention(qk, cache.k, mixed, ctx, cache.block_table, num_heads=nH, kv_rank=R, rot_dim=r,
                                 scale=self.scale, window=self.window, full_precision=self.precision.full)
        out = torch.empty((T, nH * dv), dtype=act, device=dev)
        (ops.heads_linear_mfma if self.uv_mfma else ops.heads_linear)(mixed, self.uv_t, out, heads=nH, n=dv, k=R)
        return self.o(out, torch.float32, allow_partials=True)
