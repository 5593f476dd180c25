"""Vifirax: typed configuration from config.json, and its plan.

A decoder whose layers are written out one by one in config.json (`layers`: per layer its `type`, the sizes of
its `mixer` and its `mlp`, which may be null).  A sublayer reads the stream itself and its output is normed before
it is added: x += N_1(mixer(x)); x += N_2(ff(x)), N an RMS norm that multiplies by 1 + w for a stored weight w.  The
output head is the embedding matrix; the logits are multiplied by `logit_scale`.  Three mixer types:

  "attention"      grouped-query attention with biases on q, k, v and the output matrix; q and k each normed over the
                   whole projection (all heads at once) with a plain weight; the first `rot.dims` dimensions of the
                   q and k heads turned in halves (i, i + dims/2), with frequencies stretched by `rot.scaling`
                   (factor, original, fast, slow) and cos and sin multiplied by 0.1 ln(factor) + 1; every earlier key
                   visible; a softmax whose denominator carries an extra 1; one sigmoid gate number a head.  With
                   `kv_from: j` the layer has no keys and values of its own and reads the cache of layer j.
  "mamba2"         a state-space layer: one projection gives [z | x | B | C | dt]; x, B and C pass a short causal
                   convolution and silu; per head a matrix state with one decay a token; the read-out is gated by
                   silu(z) and then normed in `norm_groups` parts.
  "channel_delta"  a gated delta rule: q, k, v each through a short convolution and silu, q and k made unit vectors,
                   a decay per head and key channel from a projection through a narrow middle, a write strength
                   a head; the read-out is normed per head and gated by a sigmoid from a second narrow projection.

The feed-forward is gated by silu, either dense or routed: `router.experts` small ones, the `router.top` best-scoring
of which serve a token, mixed by a softmax restricted to their router logits.

Everything here is data for the builder: which registered part, with which constants, under which tensor names.
Sizes and constants come from config.json, and the sizes that only the tensors give (the widths of the narrow
middles) from their shapes (`with_tensor_shapes`).
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Dict, Mapping, Optional, Tuple

from .novotar import _obj
from .plan import ConfigError, LayerPlan, ModelPlan, PartSpec, ScheduleEntry, read_key, require

DEFAULT_MAX_POSITIONS = 65536        # the design has no position limit of its own; tables are sized by this
UNIT_EPS = 1e-6                      # inside the root of the unit vectors of "channel_delta"
MIXER_TYPES = ("attention", "mamba2", "channel_delta")


def _read_rot(m: Mapping[str, Any], where: str, dim: int):
    rot = _obj(m, "rot", where, optional=True)
    if rot is None:
        return None
    out = {"base": read_key(rot, "base", float), "dims": read_key(rot, "dims", int, dim), "scaling": None}
    sc = _obj(rot, "scaling", where + "rot: ", optional=True)
    if sc is not None:
        out["scaling"] = {"factor": read_key(sc, "factor", float), "original": read_key(sc, "original", float),
                          "fast": read_key(sc, "fast", float), "slow": read_key(sc, "slow", float)}
    return out


def _read_mlp(l: Mapping[str, Any], where: str):
    mlp = _obj(l, "mlp", where, optional=True)
    if mlp is None:
        return None
    kind = read_key(mlp, "kind", str, "dense")
    require(kind in ("dense", "moe"), f"{where}mlp kind '{kind}' has no feed-forward here (known: 'dense', 'moe')")
    if kind == "dense":
        return {"kind": kind, "ff": read_key(mlp, "ff", int)}
    expert, router = _obj(mlp, "expert", where + "mlp: "), _obj(mlp, "router", where + "mlp: ")
    return {"kind": kind, "expert": {"ff": read_key(expert, "ff", int)},
            "router": {"experts": read_key(router, "experts", int), "top": read_key(router, "top", int)}}


@dataclass(frozen=True)
class VifiraxConfig:
    vocab: int
    width: int
    layers: Tuple[Mapping[str, Any], ...]          # as config.json gives them, validated
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    max_positions: int = DEFAULT_MAX_POSITIONS
    torch_dtype: str = "bfloat16"

    architecture = "Vifirax"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "VifiraxConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        norm = _obj(d, "norm", "", optional=True) or {}
        cfg = cls(vocab=read_key(d, "vocab", int), width=read_key(d, "width", int),
                  layers=tuple(cls._read_layer(i, l) for i, l in enumerate(raw_layers)),
                  norm_eps=read_key(norm, "eps", float, 1e-6), logit_scale=read_key(d, "logit_scale", float, 1.0),
                  max_positions=read_key(d, "max_positions", int, DEFAULT_MAX_POSITIONS),
                  torch_dtype=read_key(d, "torch_dtype", str, "bfloat16"))
        cfg.validate()
        return cfg

    @staticmethod
    def _read_layer(i: int, l: Any) -> Dict[str, Any]:
        where = f"layers[{i}]: "
        if not isinstance(l, Mapping):
            raise ConfigError(f"config.json: {where}must be an object")
        kind = read_key(l, "type", str)
        require(kind in MIXER_TYPES, f"{where}type '{kind}' has no mixer here (known: {', '.join(MIXER_TYPES)})")
        m = _obj(l, "mixer", where)
        mw = where + "mixer: "
        if kind == "attention":
            heads, dim = read_key(m, "heads", int), read_key(m, "dim", int)
            out: Dict[str, Any] = {"heads": heads, "kv_heads": read_key(m, "kv_heads", int, heads), "dim": dim,
                                   "vdim": read_key(m, "vdim", int, dim), "scale": read_key(m, "scale", float),
                                   "rot": _read_rot(m, mw, dim), "kv_from": read_key(m, "kv_from", int, None, allow_none=True)}
        elif kind == "mamba2":
            heads = read_key(m, "heads", int)
            out = {"heads": heads, "vdim": read_key(m, "vdim", int), "state": read_key(m, "state", int),
                   "groups": read_key(m, "groups", int, 1), "norm_groups": read_key(m, "norm_groups", int, 1),
                   "conv": read_key(m, "conv", int)}
        else:
            heads, dim = read_key(m, "heads", int), read_key(m, "dim", int)
            out = {"heads": heads, "kv_heads": read_key(m, "kv_heads", int, heads), "dim": dim,
                   "vdim": read_key(m, "vdim", int, dim), "conv": read_key(m, "conv", int)}
            for k in ("decay_rank", "gate_rank"):          # not keys of the files: the tensors' shapes give them
                if read_key(m, k, int, 0):
                    out[k] = read_key(m, k, int)
        return {"type": kind, "mixer": out, "mlp": _read_mlp(l, where)}

    def validate(self) -> None:
        require(self.vocab >= 1 and self.width >= 1, "vocab and width must be at least 1")
        require(self.norm_eps > 0, "norm.eps must be positive")
        require(self.max_positions >= 1, "max_positions must be at least 1")
        for i, l in enumerate(self.layers):
            m, where = l["mixer"], f"layers[{i}].mixer"
            if l["type"] == "attention":
                require(min(m["heads"], m["kv_heads"], m["dim"], m["vdim"]) >= 1, f"{where}: heads, kv_heads, dim and vdim must be at least 1")
                require(m["heads"] % m["kv_heads"] == 0, f"{where}.kv_heads must divide heads")
                rot = m["rot"]
                require(rot is None or (rot["base"] > 0 and 0 <= rot["dims"] <= m["dim"] and rot["dims"] % 2 == 0),
                        f"{where}.rot: base must be positive, dims even and at most dim")
                sc = rot["scaling"] if rot else None
                require(sc is None or (sc["factor"] > 0 and sc["original"] > 0 and sc["fast"] > 0 and sc["slow"] > 0),
                        f"{where}.rot.scaling: factor, original, fast and slow must be positive")
                j = m["kv_from"]
                if j is not None:
                    require(0 <= j < i and self.layers[j]["type"] == "attention" and self.layers[j]["mixer"]["kv_from"] is None,
                            f"{where}.kv_from must name an earlier attention layer with keys and values of its own")
                    o = self.layers[j]["mixer"]
                    require((o["kv_heads"], o["dim"], o["vdim"]) == (m["kv_heads"], m["dim"], m["vdim"]),
                            f"{where}.kv_from: layer {j} has other key and value sizes")
            elif l["type"] == "mamba2":
                require(min(m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]) >= 1 and m["conv"] >= 1,
                        f"{where}: heads, vdim, state, groups, norm_groups and conv must be at least 1")
                require(m["heads"] % m["groups"] == 0, f"{where}.groups must divide heads")
                require((m["heads"] * m["vdim"]) % m["norm_groups"] == 0, f"{where}.norm_groups must divide heads * vdim")
            else:
                require(min(m["heads"], m["kv_heads"], m["dim"], m["vdim"]) >= 1 and m["conv"] >= 1,
                        f"{where}: heads, kv_heads, dim, vdim and conv must be at least 1")
                require(m["heads"] % m["kv_heads"] == 0, f"{where}.kv_heads must divide heads")
            mlp = l["mlp"]
            if mlp is not None and mlp["kind"] == "dense":
                require(mlp["ff"] >= 1, f"layers[{i}].mlp.ff must be at least 1")
            elif mlp is not None:
                r = mlp["router"]
                require(mlp["expert"]["ff"] >= 1 and 1 <= r["top"] <= r["experts"],
                        f"layers[{i}].mlp: expert.ff must be at least 1 and 1 <= router.top <= router.experts")
        require(self.torch_dtype in ("bfloat16", "float32"),
                f"torch_dtype must be 'bfloat16' or 'float32', found '{self.torch_dtype}'")

    def to_dict(self) -> dict:
        layers = []
        for l in self.layers:
            m = {k: v for k, v in _plain(l["mixer"]).items() if v is not None}
            if "rot" in m and m["rot"].get("scaling") is None:
                m["rot"] = {k: v for k, v in m["rot"].items() if k != "scaling"}
            layers.append({"type": l["type"], "mixer": m, "mlp": _plain(l["mlp"])})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale, "layers": layers,
                "max_positions": self.max_positions, "torch_dtype": self.torch_dtype}

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "VifiraxConfig":
        """The configuration with the sizes that only a folder's tensors give: the widths of the narrow middles of a
        "channel_delta" mixer's decay and gate projections are the rows of `l<i>.mix.a1` and `l<i>.mix.g1`."""
        layers = []
        for i, l in enumerate(self.layers):
            if l["type"] == "channel_delta":
                m = dict(l["mixer"])
                for key, name in (("decay_rank", f"l{i}.mix.a1"), ("gate_rank", f"l{i}.mix.g1")):
                    if key not in m and name in shapes and len(shapes[name]) == 2:
                        m[key] = int(shapes[name][0])
                l = dict(l, mixer=m)
            layers.append(l)
        return replace(self, layers=tuple(layers))

    # ------------------------------------------------------------------ the plan
    def _attention(self, m) -> PartSpec:
        shared = m["kv_from"] is not None
        names = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_norm": "q.norm", "k_norm": "k.norm", "o_bias": "o.b"}
        return PartSpec("attention", {
            "hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "value_head_dim": m["vdim"], "scale": m["scale"], "softcap": None, "window": None,
            "position": None if m["rot"] is None or not m["rot"]["dims"] else _rot_name(m),
            "bias": True, "output_bias": True, "sink": "zero", "output_gate": "head", "qk_norm": "projection",
            "qk_norm_eps": self.norm_eps, "own_keys": not shared, "tensor_names": names}, "mix")

    def _mamba2(self, m) -> PartSpec:
        return PartSpec("mamba2", {
            "hidden_size": self.width, "num_heads": m["heads"], "value_head_dim": m["vdim"], "state_dim": m["state"],
            "groups": m["groups"], "norm_groups": m["norm_groups"], "conv_taps": m["conv"], "norm_eps": self.norm_eps}, "mix")

    def _delta(self, i: int, m) -> PartSpec:
        for key, what in (("decay_rank", "decay"), ("gate_rank", "gate")):
            if key not in m:
                raise ConfigError(f"config.json: layers[{i}].mixer: the width of the {what} projection's middle is not known "
                                  f"(the tensors' shapes give it when a folder is loaded; '{key}' names it otherwise)")
        return PartSpec("channel_delta", {
            "hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "value_head_dim": m["vdim"], "conv_taps": m["conv"], "decay_rank": m["decay_rank"], "gate_rank": m["gate_rank"],
            "norm_eps": self.norm_eps, "unit_eps": UNIT_EPS}, "mix")

    def _ff(self, mlp) -> PartSpec:
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"hidden_size": self.width, "intermediate_size": mlp["ff"], "activation": "silu",
                                          "tensor_names": {"gate": "gate", "up": "up", "down": "down"}}, "mlp")
        return PartSpec("expert_mlp", {"hidden_size": self.width, "intermediate_size": mlp["expert"]["ff"],
                                       "experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
                                       "activation": "silu"}, "mlp")

    def plan(self) -> ModelPlan:
        W, eps = self.width, self.norm_eps
        norm = lambda name, scale=1.0: PartSpec("rmsnorm", {"dim": W, "eps": eps, "weight_offset": 1.0, "tensor_name": "",
                                                            "output_scale": scale}, name)
        layers, positions, schedule = [], {}, []
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            cache_from = None
            if l["type"] == "attention":
                mixer = self._attention(m)
                cache_from = m["kv_from"]
                if m["rot"] is not None and m["rot"]["dims"]:
                    rot = m["rot"]
                    positions[_rot_name(m)] = PartSpec("rope_pairs", {
                        "dim": m["dim"], "theta": rot["base"], "rotary_dim": rot["dims"], "value_dim": None,
                        "max_positions": self.max_positions, "interleaved": False, "scaling": rot["scaling"]})
            elif l["type"] == "mamba2":
                mixer = self._mamba2(m)
            else:
                mixer = self._delta(i, m)
            ff, norms = None, {"post_mixer": norm("norm1")}
            if l["mlp"] is not None:
                ff = self._ff(l["mlp"])
                norms["post_ff"] = norm("norm2")
            layers.append(LayerPlan(block="sandwich", mixer=mixer, feed_forward=ff, norms=norms, prefix=f"l{i}."))
            schedule.append(ScheduleEntry(i, cache_from=cache_from))
        # the logits' constant factor rides on the final norm's weight: the head is the embedding matrix as it is
        return ModelPlan(
            vocab_size=self.vocab, hidden_size=W, max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab, "dim": W, "scale": 1.0, "tensor_name": ""}, "embed"),
            positions=positions, layers=tuple(layers), schedule=tuple(schedule),
            final_norm=norm("final.norm", self.logit_scale),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "dim": W, "softcap": None, "tied_to": "embed"}, "head"),
            stop_token_ids=())


def _rot_name(m) -> str:
    """One table set per distinct (head size, rotated width, base, scaling)."""
    rot = m["rot"]
    sc = rot["scaling"]
    tail = "" if sc is None else "_" + "_".join(repr(sc[k]) for k in ("factor", "original", "fast", "slow"))
    return f"halves_{m['dim']}_{rot['dims']}_{rot['base']!r}{tail}"


def _plain(x):
    if isinstance(x, Mapping):
        return {k: _plain(v) for k, v in x.items()}
    return x
