"""The attention mixer: grouped-query attention over the paged cache.

q, k, v projections (no biases), position encoding of q and k, k and v cached, then per query
head h with kv head h // (nH // nKV): score = (q . k) * scale, softcap cap * tanh(s / cap),
softmax over the keys max(0, pos + 1 - window) .. pos, weighted sum of v, output projection
(llama3.rs:14206-14217, 14307-14331, 5431-5451, 5622-5688, 14423).  Scale, softcap, window, head
counts and head size are constructor arguments; window None is global attention, softcap None
turns the tanh off.  A position term at the score stage is a constructor argument too:
score_bias_slopes, one slope a query head, adds slope * (key position - query position) to the
capped score (a linear distance bias; the 32-bit attention kernel over a row-major cache takes it,
in both dtypes).  Values may have a head size of their own (value_head_dim), and output_gate = "head" adds
one gate number a query head, projected from the mixer's input beside q, k and v: head h's output is
multiplied by sigmoid(gate_h) before the output projection.  tensor_names gives the local names of the
matrices (q, k, v, o, g) where a file names them otherwise.

Further constructor arguments, each off by default, make other attention mixers from the same part (they run
on the 32-bit attention kernel over a row-major cache in both dtypes, from a projection whose sums stay 32-bit
until the bias is added and the rotation done):
  bias            q, k and v have biases (the matrix's name + ".b"), added in the projection
  chunk           a query sees the keys of its own chunk of that many positions only, chunks counted from the
                  sequence's position 0 (the cache gives the pages of finished chunks back like a window's)
  keep_first      beside its window a query sees the first that many positions (the cache keeps their pages)
  sink            one learned number a head ("sink") whose exponential joins the softmax's denominator; it has no
                  key and no value.  "zero": the number is 0 for every head and no tensor is read (the denominator is
                  one more than the sum of the exponentials)
  qk_norm         "projection": q (all heads together) and k (likewise) are each divided by their root mean square over
                  the whole projection (qk_norm_eps inside the root) and multiplied by a weight of that length ("q_norm",
                  "k_norm"), after the bias and before the rotation
  output_bias     the output matrix has a bias ("o_bias")
  own_keys        False: the mixer has no k and v matrices (nor their biases and norm); it reads the keys and values that
                  another run of the schedule cached and brings its own queries, gate and output matrix
  talk            the heads' softmax weights are mixed by a learned matrix ("talk" [heads, heads]) before they meet
                  the values: weight_h <- sum_g talk[h, g] weight_g, head h keeping its own kv head's values
  output_gate     "elementwise": sigmoid of a projection of the mixer's input ("g" [heads * value size, width]) times
                  the concatenated heads
  output_scale    a constant factor of the mixer's output (applied to the gated heads; the output matrix is linear)
  position        a "rope_pairs" encoding: pairs of neighbouring dimensions, a rotated part of the head, and
                  values that are turned by their position and turned back at the output
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..hip import ops
from .base import MIXERS, CacheNeed, FragmentActs, KVNeed, ParamSpec, Part, Precision
from .linear import Linear


@MIXERS.register("attention")
class Attention(Part):
    graph_safe = True

    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, num_heads: int,
                 num_kv_heads: int, head_dim: int, scale: float, softcap: Optional[float] = None,
                 window: Optional[int] = None, position: Optional[str] = None,
                 score_bias_slopes: Optional[Sequence[float]] = None, value_head_dim: Optional[int] = None,
                 output_gate: Optional[str] = None, tensor_names: Optional[Dict[str, str]] = None,
                 bias: bool = False, chunk: Optional[int] = None, keep_first: int = 0, sink=False,
                 talk: bool = False, output_scale: float = 1.0, qk_norm: Optional[str] = None, qk_norm_eps: float = 1e-6,
                 output_bias: bool = False, own_keys: bool = True):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_kv_heads {num_kv_heads} must divide num_heads {num_heads}")
        if not 1 <= head_dim <= ops.ATTENTION_MAX_HEAD_DIM:
            # refused when the model is put together, not at its first step
            raise ValueError(f"attention: head_dim {head_dim} is outside 1..{ops.ATTENTION_MAX_HEAD_DIM}, the range "
                             f"of the attention kernels")
        self.precision = precision
        self.H, self.nH, self.nKV, self.d = hidden_size, num_heads, num_kv_heads, head_dim
        self.scale = float(scale)
        self.softcap = None if softcap is None else float(softcap)
        self.window = window
        if score_bias_slopes is not None and len(score_bias_slopes) != num_heads:
            raise ValueError(f"attention: {len(score_bias_slopes)} score bias slopes for {num_heads} heads")
        self.score_bias_slopes = None if score_bias_slopes is None else [float(v) for v in score_bias_slopes]
        self._slopes: Optional[torch.Tensor] = None
        self.position = positions[position] if position is not None else positions.get("none")
        if self.position is None:
            raise ValueError("attention needs a position encoding (use 'none' for no rotation)")
        self.dv = head_dim if value_head_dim is None else int(value_head_dim)
        if not 1 <= self.dv <= ops.ATTENTION_MAX_HEAD_DIM:
            raise ValueError(f"attention: value_head_dim {self.dv} is outside 1..{ops.ATTENTION_MAX_HEAD_DIM}")
        if output_gate not in (None, "head", "elementwise"):
            raise ValueError(f"attention: output_gate '{output_gate}' is not known (None, 'head' or 'elementwise')")
        if chunk is not None and (window is not None or chunk < 1):
            raise ValueError("attention: a chunk is at least 1 position and stands in the window's place")
        if keep_first < 0 or (keep_first and window is None):
            raise ValueError("attention: kept first positions go with a window")
        self.output_gate = output_gate
        self.n_gate = {None: 0, "head": num_heads, "elementwise": num_heads * self.dv}[output_gate]
        self.bias, self.chunk, self.keep_first = bool(bias), chunk, int(keep_first)
        if sink not in (False, True, None, "zero"):
            raise ValueError(f"attention: sink '{sink}' is not known (False, True or 'zero')")
        if qk_norm not in (None, "projection"):
            raise ValueError(f"attention: qk_norm '{qk_norm}' is not known (None or 'projection')")
        self.has_sink, self.has_talk, self.output_scale = bool(sink), bool(talk), float(output_scale)
        self.zero_sink = sink == "zero"
        self.qk_norm, self.qk_norm_eps = qk_norm, float(qk_norm_eps)
        self.output_bias, self.own_keys = bool(output_bias), bool(own_keys)
        pairs = getattr(self.position, "value_cos", "absent") != "absent"          # a rope_pairs encoding
        # the mixers made by the further arguments: float32 projection sums, bias and rotation in one kernel, the
        # 32-bit attention kernel with its further masks over a row-major cache
        self.extended = bool(bias or chunk or keep_first or sink or talk or output_gate == "elementwise"
                             or output_scale != 1.0 or pairs or qk_norm or output_bias or not own_keys)
        if self.extended and softcap is not None and talk:
            raise ValueError("attention: mixed heads take no softcap")
        self.names = dict({"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                           "g": "g_proj.weight", "sink": "sink", "talk": "talk", "q_norm": "q_norm.weight",
                           "k_norm": "k_norm.weight", "o_bias": "o_proj.bias"}, **(tensor_names or {}))
        self._bias_parts: Dict[str, torch.Tensor] = {}
        self.qkv_bias: Optional[torch.Tensor] = None
        self.sink: Optional[torch.Tensor] = None
        self.talk: Optional[torch.Tensor] = None
        self.q_dim = num_heads * head_dim
        # (a mixer without keys of its own has no k and v columns in its projection)
        self.kv_dim, self.v_dim = (num_kv_heads * head_dim, num_kv_heads * self.dv) if self.own_keys else (0, 0)
        self.o_in = num_heads * self.dv
        self.o_bias: Optional[torch.Tensor] = None
        self._norm_parts: Dict[str, torch.Tensor] = {}
        self.qk_norm_w: Optional[torch.Tensor] = None
        self._mats = "q" + ("kv" if self.own_keys else "") + ("g" if self.n_gate else "")
        # one fused projection: all q heads, the k heads, the v heads, then the gate numbers
        self.qkv = Linear(hidden_size, self.q_dim + self.kv_dim + self.v_dim + self.n_gate, precision)
        self.o = Linear(self.o_in, hidden_size, precision)
        # How this mixer lays keys and values out inside a page: the matrix-core kernels read a fragment
        # layout; every other case is row-major.  It depends on the arithmetic and the head size alone, so
        # that a run that reads another run's cache finds the layout it expects.
        self.kv_layout = (ops.KV_FRAGMENT if precision.name == "bfloat16" and precision.act == torch.bfloat16
                          and ops.library_ready() and ops.attention_mfma_supported(head_dim)
                          and score_bias_slopes is None and self.dv == head_dim and not self.extended else ops.KV_ROW)
        self._parts: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        specs = {n["q"]: ParamSpec((self.q_dim, self.H))}
        if self.own_keys:
            specs[n["k"]] = ParamSpec((self.kv_dim, self.H))
            specs[n["v"]] = ParamSpec((self.v_dim, self.H))
        specs[n["o"]] = ParamSpec((self.H, self.o_in))
        if self.n_gate:
            specs[n["g"]] = ParamSpec((self.n_gate, self.H))
        if self.bias:
            specs[n["q"] + ".b"] = ParamSpec((self.q_dim,), init_std=0.1)
            if self.own_keys:
                specs[n["k"] + ".b"] = ParamSpec((self.kv_dim,), init_std=0.1)
                specs[n["v"] + ".b"] = ParamSpec((self.v_dim,), init_std=0.1)
        if self.qk_norm:
            specs[n["q_norm"]] = ParamSpec((self.q_dim,), init_std=0.3)
            if self.own_keys:
                specs[n["k_norm"]] = ParamSpec((self.kv_dim,), init_std=0.3)
        if self.output_bias:
            specs[n["o_bias"]] = ParamSpec((self.H,), init_std=0.1)
        if self.has_sink and not self.zero_sink:
            specs[n["sink"]] = ParamSpec((self.nH,), init_std=1.0)
        if self.has_talk:
            specs[n["talk"]] = ParamSpec((self.nH, self.nH), init_std=0.3)
        return specs

    def cache_need(self) -> CacheNeed:
        # the fragment layout of the matrix-core kernels is written for pages of 64 positions
        page = ops.KV_FRAGMENT_PAGE if self.kv_layout == ops.KV_FRAGMENT else None
        # a chunk's keys lie at most chunk - 1 positions back: its pages go back to the pool like a window's
        return CacheNeed(kv=KVNeed(self.nKV, self.d, self.window if self.chunk is None else self.chunk, page_size=page,
                                   value_head_dim=None if self.dv == self.d else self.dv, keep_first=self.keep_first))

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name == self.names["o"]:
            self.o.load(tensor)
        elif name in [self.names[c] for c in self._mats]:
            self._parts[name] = tensor
        elif self.bias and name in [self.names[c] + ".b" for c in self._mats if c != "g"]:
            self._bias_parts[name] = tensor
        elif self.qk_norm and name in (self.names["q_norm"], self.names["k_norm"]):
            self._norm_parts[name] = tensor
        elif self.output_bias and name == self.names["o_bias"]:
            self.o_bias = tensor.float().contiguous()
        elif self.has_sink and not self.zero_sink and name == self.names["sink"]:
            self.sink = tensor.float().contiguous()
        elif self.has_talk and name == self.names["talk"]:
            self.talk = tensor.float().contiguous()
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        mats = [self.precision.matrix(self._parts.pop(self.names[c])) for c in self._mats]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]                # kept as stored, one of them in 32-bit: the fused matrix is 32-bit
        w = torch.cat(mats, dim=0)                          # rows: all q heads, then k heads, then v heads, then the gates
        # a position encoding may ask for the rows of the q and k heads in another order (rotated pairs next to
        # each other), so that its rotation can be the projection's epilogue
        order = getattr(self.position, "projection_row_order", lambda *a: None)(self.nH, self.nKV, self.d)
        self.pair_order = order is not None and self.dv == self.d and not self.n_gate and not self.extended
        if self.bias:
            self.qkv_bias = torch.cat([self._bias_parts.pop(self.names[c] + ".b").float() for c in self._mats if c != "g"]).contiguous()
        if self.qk_norm:
            self.qk_norm_w = torch.cat([self._norm_parts.pop(self.names[c]).float()
                                        for c in (("q_norm", "k_norm") if self.own_keys else ("q_norm",))]).contiguous()
        if self.zero_sink:
            self.sink = torch.zeros(self.nH, dtype=torch.float32, device=w.device)
        if self.pair_order:
            w = w[order.to(w.device)]
        self.qkv.load(w)
        if self.score_bias_slopes is not None:
            self._slopes = torch.tensor(self.score_bias_slopes, dtype=torch.float32, device=w.device)

    def weight_bytes(self) -> int:
        return self.qkv.nbytes() + self.o.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.qkv.accepts_fragment_input

    def forward(self, x, ctx, cache) -> torch.Tensor:
        """x: [T, H] in the activation dtype (a tensor, or FragmentActs in decode steps); returns the branch
        in float32 ([T, H] or partial sums)."""
        T = x.shape[0]
        if self.extended:
            return self._forward_extended(x, ctx, cache)
        q = torch.empty((T, self.q_dim), dtype=self.precision.act, device=x.device)
        geometry = dict(num_heads=self.nH, num_kv_heads=self.nKV, head_dim=self.d, kv_layout=self.kv_layout)
        if self.dv != self.d:
            geometry["value_head_dim"] = self.dv
        gate = None
        fused = self.pair_order and self.position.project_rotate_store(self.qkv, x, q, ctx, cache, **geometry)
        if not fused:
            qkv = self.qkv(x, self.precision.act)
            if self.n_gate:
                g0 = self.q_dim + self.kv_dim + self.v_dim
                gate = qkv[:, g0:g0 + self.n_gate]          # a column slice: the kernel reads it with the rows' stride
            if self.pair_order:
                self.position.rotate_and_store(qkv, q, ctx, cache, pair_order=True, **geometry)
            else:
                self.position.rotate_and_store(qkv, q, ctx, cache, **geometry)
        # Single tokens of at most 16 sequences whose keys are split over blocks: the output projection combines the
        # splits itself (one kernel fewer a layer).
        if (ctx.is_decode and self.kv_layout == ops.KV_FRAGMENT and self.o.layout == ops.LAYOUT_FRAG16
                and not self.n_gate and self.nH // self.nKV <= 16 and getattr(ctx, "fragment_activations", False)):
            splits = ops.decode_attention_splits(T, self.nKV, ctx.max_context, self.window)
            slices = ops.linear_parts_slices(T, self.o.n, self.nH, self.d, splits) if splits > 1 else 0
            if slices > 0:
                parts, _ = ops.attention_decode(q, cache.k, cache.v, None, ctx.context_lens, cache.block_table,
                                                num_heads=self.nH, max_context=ctx.max_context, scale=self.scale,
                                                softcap=self.softcap, window=self.window, splits=splits)
                y = torch.empty((slices, T, self.o.n), dtype=torch.float32, device=q.device)
                ops.linear_parts(parts, splits, self.o.weight, y, num_heads=self.nH, head_dim=self.d)
                return y if slices > 1 else y[0]
        # The matrix-core kernels' output goes to the output projection in fragment order.
        frag = (getattr(ctx, "fragment_activations", False) and self.kv_layout == ops.KV_FRAGMENT
                and self.o.accepts_fragment_input and FragmentActs.possible(self.precision, T, self.o_in))
        out = (FragmentActs.empty(T, self.o_in, q.device) if frag
               else torch.empty((T, self.o_in), dtype=q.dtype, device=q.device))
        ops.attention(q, cache.k, cache.v, out.data if frag else out, ctx, cache.block_table, num_heads=self.nH,
                      scale=self.scale, softcap=self.softcap, window=self.window, full_precision=self.precision.full,
                      kv_layout=self.kv_layout, out_layout=ops.LAYOUT_FRAG16 if frag else ops.LAYOUT_ROW,
                      bias_slopes=self._slopes, gate=gate)
        return self.o(out, torch.float32, allow_partials=True)

    def _forward_extended(self, x, ctx, cache) -> torch.Tensor:
        """The mixers made by the further constructor arguments (see the top of the file)."""
        T, act, dev = x.shape[0], self.precision.act, x.device
        rows = self.qkv(x, torch.float32)                     # [q | k | v | g], the sums as they are
        q = torch.empty((T, self.q_dim), dtype=act, device=dev)
        pos = self.position
        write = cache is not None and cache.writable
        if write and not self.own_keys:
            raise RuntimeError("attention: a mixer without keys of its own reads the cache of another run of the schedule")
        norm_w = self.qk_norm_w
        if norm_w is not None and self.own_keys and not write:
            norm_w = norm_w[:self.q_dim]                      # the keys are another run's: only the queries are normed here
        ops.qkv_prepare(rows, self.qkv_bias, q, cache.k if write else None, cache.v if write else None, ctx.positions,
                        ctx.seq_of_token if write else None, cache.block_table if write else None,
                        num_heads=self.nH, num_kv_heads=self.nKV, head_dim=self.d, value_head_dim=self.dv,
                        max_position=ctx.max_position, cos=getattr(pos, "cos", None), sin=getattr(pos, "sin", None),
                        rotary_dim=getattr(pos, "rotary_dim", 0), interleaved=getattr(pos, "interleaved", True),
                        value_cos=getattr(pos, "value_cos", None), value_sin=getattr(pos, "value_sin", None),
                        norm_weight=norm_w, norm_eps=self.qk_norm_eps)
        gate = None
        if self.n_gate:
            g0 = self.q_dim + self.kv_dim + self.v_dim
            gate = rows[:, g0:g0 + self.n_gate]
        out = torch.empty((T, self.o_in), dtype=act, device=dev)
        common = dict(num_heads=self.nH, scale=self.scale, window=self.window, chunk=self.chunk, keep_first=self.keep_first,
                      bias_slopes=self._slopes, sink=self.sink, value_cos=getattr(pos, "value_cos", None),
                      value_sin=getattr(pos, "value_sin", None))
        # steps with pieces of several tokens: the matrix-core kernel (bfloat16); steps of single tokens and the 32-bit
        # path: the 32-bit kernel (the choice must not depend on the sizes that a captured step rounds up)
        tiled = (not ctx.is_decode and self.softcap is None and not self.precision.full
                 and ops.attention_tiled_supported(act, self.d, self.dv))

        # single tokens: the kernel that splits the keys over blocks, where it takes the head sizes
        split = (not tiled and ctx.is_decode and self.softcap is None
                 and ops.attention_split_supported(act, self.nH, self.nKV, self.d, self.dv))
        if self.chunk is not None:
            most = min(ctx.max_context, self.chunk)
        elif self.window is not None:
            most = min(ctx.max_context, self.window + self.keep_first)
        else:
            most = ctx.max_context

        def attend(out_, per_, **more):
            if tiled:
                ops.attention_tiled(q, cache.k, cache.v, out_, ctx, cache.block_table, per_value_head=per_, **common, **more)
            elif split:
                ops.attention_split(q, cache.k, cache.v, out_, ctx.positions, ctx.seq_of_token, cache.block_table,
                                    per_value_head=per_, max_position=ctx.max_position, max_keys=most, **common, **more)
            else:
                ops.attention_masked(q, cache.k, cache.v, out_, ctx.positions, ctx.seq_of_token, cache.block_table,
                                     per_value_head=per_, softcap=self.softcap, max_position=ctx.max_position,
                                     full_precision=self.precision.full, **common, **more)
        if self.has_talk:
            # every head's weights on each kv head's values, then the mix of the heads with the gate behind it
            if self.output_gate == "head":
                raise NotImplementedError("attention: mixed heads take an elementwise gate or none")
            per = torch.empty((T, self.nH, self.nKV, self.dv), dtype=torch.float32, device=dev)
            attend(None, per)
            ops.mix_heads(per, self.talk, gate, out, full_precision=self.precision.full, out_scale=self.output_scale)
        else:
            attend(out, None, gate=gate, gate_per_element=self.output_gate == "elementwise", out_scale=self.output_scale)
        if self.o_bias is None:
            return self.o(out, torch.float32, allow_partials=True)
        y = self.o(out, torch.float32)
        ops.add_rows(y, None, self.o_bias)
        return y
