"""Pefitar: typed configuration from config.json, and its plan.

A decoder whose layers are written out one by one in config.json (`layers`: per layer its `type`, the sizes of
its `mixer` and its `mlp`, which may be null), with a run of layers that is repeated with the same weights
(`loop`: start, stop, times; every pass keeps a cache of its own and nothing else happens between passes).
Every sublayer has a norm before and a norm after it, and its normed output enters the stream times a constant:
x += m * norm_b(sublayer(norm_a(x))), m = `residual_mult`.  The feed-forward is gated, down(silu(gate h) * (up h));
the output head is the embedding matrix, its logits capped by c * tanh(. / c), c = `logit_softcap`.  Two mixer
types:

  "attention"         grouped-query attention without biases, values of a size of their own; rotation of
                      neighbouring pairs over the first `rot.dims` dimensions of the q and k heads; every earlier
                      key visible; an elementwise sigmoid gate, projected from the mixer's input, on the
                      concatenated heads before the output matrix.
  "latent_attention"  queries through a normed latent of `q_rank` numbers; keys and values of all heads made from
                      one normed latent of `kv_rank` numbers a token, beside `rot_dim` rotated key dimensions that
                      all heads share; a head's query is [`dim` plain | `rot_dim` rotated]; a sliding window of
                      `mask.size` keys.  The cache holds the latent and the rotated part only.

Everything here is data for the builder: which registered part, with which constants, under which tensor names.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .novotar import _obj
from .plan import ConfigError, LayerPlan, ModelPlan, PartSpec, ScheduleEntry, read_key, require

DEFAULT_MAX_POSITIONS = 65536        # the design has no position limit of its own; tables are sized by this


def _read_rot(mixer: Mapping[str, Any], where: str, default_dims: int):
    rot = _obj(mixer, "rot", where, optional=True)
    if rot is None:
        return None
    return {"base": read_key(rot, "base", float), "dims": read_key(rot, "dims", int, default_dims)}


def _read_mask(mixer: Mapping[str, Any], where: str):
    mask = _obj(mixer, "mask", where, optional=True)
    return None if mask is None else {"size": read_key(mask, "size", int)}


@dataclass(frozen=True)
class PefitarConfig:
    vocab: int
    width: int
    layers: Tuple[Mapping[str, Any], ...]          # as config.json gives them, validated
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    logit_softcap: Optional[float] = None
    loop: Optional[Tuple[int, int, int]] = None    # (start, stop, times)
    max_positions: int = DEFAULT_MAX_POSITIONS
    torch_dtype: str = "bfloat16"

    architecture = "Pefitar"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "PefitarConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        norm = _obj(d, "norm", "", optional=True) or {}
        loop = _obj(d, "loop", "", optional=True)
        if loop is not None:
            loop = (read_key(loop, "start", int), read_key(loop, "stop", int), read_key(loop, "times", int))
        cfg = cls(vocab=read_key(d, "vocab", int), width=read_key(d, "width", int),
                  layers=tuple(cls._read_layer(i, l) for i, l in enumerate(raw_layers)),
                  norm_eps=read_key(norm, "eps", float, 1e-6), residual_mult=read_key(d, "residual_mult", float, 1.0),
                  logit_softcap=read_key(d, "logit_softcap", float, None, allow_none=True), loop=loop,
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
        require(kind in ("attention", "latent_attention"),
                f"{where}type '{kind}' has no mixer here (known: 'attention', 'latent_attention')")
        m = _obj(l, "mixer", where)
        mw = where + "mixer: "
        heads, dim = read_key(m, "heads", int), read_key(m, "dim", int)
        out: Dict[str, Any] = {"heads": heads, "dim": dim, "vdim": read_key(m, "vdim", int, dim),
                               "scale": read_key(m, "scale", float), "mask": _read_mask(m, mw)}
        if kind == "attention":
            out["kv_heads"] = read_key(m, "kv_heads", int, heads)
            out["rot"] = _read_rot(m, mw, dim)
        else:
            out["rot_dim"] = read_key(m, "rot_dim", int)
            out["q_rank"], out["kv_rank"] = read_key(m, "q_rank", int), read_key(m, "kv_rank", int)
            out["rot"] = _read_rot(m, mw, out["rot_dim"])
        mlp = _obj(l, "mlp", where, optional=True)
        out_mlp = None
        if mlp is not None:
            mk = read_key(mlp, "kind", str, "dense")
            require(mk == "dense", f"{where}mlp kind '{mk}' has no feed-forward here (known: 'dense')")
            out_mlp = {"kind": mk, "ff": read_key(mlp, "ff", int)}
        return {"type": kind, "mixer": out, "mlp": out_mlp}

    def validate(self) -> None:
        require(self.vocab >= 1 and self.width >= 1, "vocab and width must be at least 1")
        require(self.norm_eps > 0, "norm.eps must be positive")
        require(self.logit_softcap is None or self.logit_softcap > 0, "logit_softcap must be positive")
        require(self.max_positions >= 1, "max_positions must be at least 1")
        L = len(self.layers)
        if self.loop is not None:
            a, b, n = self.loop
            require(0 <= a < b <= L, f"loop start {a} and stop {b} must satisfy 0 <= start < stop <= {L}")
            require(n >= 1, f"loop times must be at least 1, found {n}")
        for i, l in enumerate(self.layers):
            m, where = l["mixer"], f"layers[{i}].mixer"
            require(min(m["heads"], m["dim"], m["vdim"]) >= 1, f"{where}: heads, dim and vdim must be at least 1")
            require(m["mask"] is None or m["mask"]["size"] >= 1, f"{where}.mask.size must be at least 1")
            rot = m["rot"]
            if l["type"] == "attention":
                require(m["kv_heads"] >= 1 and m["heads"] % m["kv_heads"] == 0, f"{where}.kv_heads must divide heads")
                require(rot is None or (rot["base"] > 0 and 0 <= rot["dims"] <= m["dim"] and rot["dims"] % 2 == 0),
                        f"{where}.rot: base must be positive, dims even and at most dim")
            else:
                require(m["q_rank"] >= 1 and m["kv_rank"] >= 1, f"{where}: q_rank and kv_rank must be at least 1")
                require(m["rot_dim"] >= 0 and m["rot_dim"] % 2 == 0, f"{where}.rot_dim must be even and not negative")
                require(m["rot_dim"] == 0 or rot is not None, f"{where}: rotated dimensions need 'rot'")
                require(rot is None or (rot["base"] > 0 and rot["dims"] == m["rot_dim"]),
                        f"{where}.rot: base must be positive and dims equal to rot_dim (the rotated part turns as a whole)")
            require(l["mlp"] is None or l["mlp"]["ff"] >= 1, f"layers[{i}].mlp.ff must be at least 1")
        require(self.torch_dtype in ("bfloat16", "float32"),
                f"torch_dtype must be 'bfloat16' or 'float32', found '{self.torch_dtype}'")

    def to_dict(self) -> dict:
        d: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                             "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
                             "layers": [_plain(l) for l in self.layers], "max_positions": self.max_positions,
                             "torch_dtype": self.torch_dtype}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        return d

    # ------------------------------------------------------------------ derived
    def layer_runs(self):
        """The layers in the order in which they run."""
        L = len(self.layers)
        if self.loop is None:
            return list(range(L))
        a, b, n = self.loop
        return list(range(a)) + list(range(a, b)) * n + list(range(b, L))

    # ------------------------------------------------------------------ the plan
    def _attention(self, m) -> PartSpec:
        return PartSpec("attention", {
            "hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "value_head_dim": m["vdim"], "scale": m["scale"], "softcap": None,
            "window": None if m["mask"] is None else m["mask"]["size"],
            "position": None if m["rot"] is None or not m["rot"]["dims"] else _rot_name(m["dim"], m["rot"]),
            "output_gate": "elementwise",
            "tensor_names": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g"}}, "mix")

    def _latent(self, m) -> PartSpec:
        return PartSpec("latent_attention", {
            "hidden_size": self.width, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
            "value_head_dim": m["vdim"], "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": m["scale"],
            "window": None if m["mask"] is None else m["mask"]["size"], "norm_eps": self.norm_eps,
            "position": None if not m["rot_dim"] else _rot_name(m["rot_dim"], m["rot"]),
            "tensor_names": {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm",
                             "uk": "uk", "uv": "uv", "o": "o"}}, "mix")

    def plan(self) -> ModelPlan:
        W, eps, mult = self.width, self.norm_eps, self.residual_mult
        # every norm keeps its weight in 32-bit: the ones behind a sublayer carry the stream's factor, and the fused
        # add-and-norm kernel meets one of them together with the next sublayer's
        norm = lambda name, scale=1.0: PartSpec("rmsnorm", {"dim": W, "eps": eps, "weight_offset": 0.0, "tensor_name": "",
                                                            "output_scale": scale, "keep_float32": True}, name)
        layers, positions = [], {}
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            if l["type"] == "attention":
                mixer = self._attention(m)
                head, rot = m["dim"], m["rot"]
            else:
                mixer = self._latent(m)
                head, rot = m["rot_dim"], m["rot"]
            if rot is not None and rot["dims"]:
                positions[_rot_name(head, rot)] = PartSpec("rope_pairs", {
                    "dim": head, "theta": rot["base"], "rotary_dim": rot["dims"], "value_dim": None,
                    "max_positions": self.max_positions, "interleaved": True})
            ff, norms = None, {"pre_mixer": norm("norm1"), "post_mixer": norm("norm1b", mult)}
            if l["mlp"] is not None:
                ff = PartSpec("gated_mlp", {"hidden_size": W, "intermediate_size": l["mlp"]["ff"], "activation": "silu",
                                            "tensor_names": {"gate": "gate", "up": "up", "down": "down"}}, "mlp")
                norms["pre_ff"] = norm("norm2")
                norms["post_ff"] = norm("norm2b", mult)
            layers.append(LayerPlan(block="sandwich", mixer=mixer, feed_forward=ff, norms=norms, prefix=f"l{i}."))
        return ModelPlan(
            vocab_size=self.vocab, hidden_size=W, max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab, "dim": W, "scale": 1.0, "tensor_name": ""}, "embed"),
            positions=positions, layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in self.layer_runs()),
            final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "dim": W, "softcap": self.logit_softcap,
                                      "tied_to": "embed"}, "head"),
            stop_token_ids=())


def _rot_name(head: int, rot) -> str:
    """One table set per distinct (head size, rotated width, base)."""
    return f"pairs_{head}_{rot['dims']}_{rot['base']!r}"


def _plain(x):
    if isinstance(x, Mapping):
        return {k: _plain(v) for k, v in x.items()}
    return x
