"""Shared by the tests: two tiny Gemma 2 configurations that differ in every size and option, model
folders with random weights in a temporary place, and comparison helpers."""
import json
import os
import tempfile

import torch

_COMMON = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", hidden_activation="gelu_pytorch_tanh",
               tie_word_embeddings=True, eos_token_id=1, bos_token_id=2)

# layers 2 / 3 (sliding, global / sliding, global, sliding), width 64 / 96, heads 4 / 6, kv heads 1 / 3
# (groups of 4 / 2), head size 16 / 24 (q width = width / != width), feed-forward 128 / 320, vocabulary
# 256 / 384, theta 1e4 / 5e5, window 8 / 6, score scale 16 (= head size) / 32 (!= head size),
# score cap 50 / 20, logit cap 30 / 15, eps 1e-6 / 1e-5.
TINY_A = dict(_COMMON, num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=1,
              head_dim=16, intermediate_size=128, vocab_size=256, rope_theta=10000.0, sliding_window=8,
              query_pre_attn_scalar=16, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
              rms_norm_eps=1e-6, max_position_embeddings=512)
TINY_B = dict(_COMMON, num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=3,
              head_dim=24, intermediate_size=320, vocab_size=384, rope_theta=500000.0, sliding_window=6,
              query_pre_attn_scalar=32, attn_logit_softcapping=20.0, final_logit_softcapping=15.0,
              rms_norm_eps=1e-5, max_position_embeddings=768)
# A third shape whose sizes suit the matrix-core kernels (head size 64, widths multiples of 32) but are
# no powers of two, with a window longer than a page.
TINY_C = dict(_COMMON, num_hidden_layers=4, hidden_size=160, num_attention_heads=6, num_key_value_heads=2,
              head_dim=64, intermediate_size=416, vocab_size=1000, rope_theta=20000.0, sliding_window=80,
              query_pre_attn_scalar=48, attn_logit_softcapping=12.0, final_logit_softcapping=9.0,
              rms_norm_eps=2e-6, max_position_embeddings=1024)
# The options that the published Gemma 2 configurations leave at their defaults, all turned the other way: a head with
# a matrix of its own, no caps, and the layers' kinds listed in config.json (global first, then two sliding layers).
TINY_D = dict(TINY_B, tie_word_embeddings=False, attn_logit_softcapping=None, final_logit_softcapping=None,
              layer_types=["full_attention", "sliding_attention", "sliding_attention"], sliding_window=5, hidden_size=80,
              num_attention_heads=4, num_key_value_heads=4, head_dim=32, query_pre_attn_scalar=32, vocab_size=130)
TINY = {"tiny-a": (TINY_A, 0), "tiny-b": (TINY_B, 1), "tiny-c": (TINY_C, 2), "tiny-d": (TINY_D, 3)}

_FOLDERS = {}
_TMP = None


def model_folder(name: str, stored: str = "bfloat16", hot: float = 1.0) -> str:
    """A folder with config.json and model.safetensors for a tiny configuration; made once per session.
    hot > 1 multiplies q/k and embedding weights so that scores and logits reach their caps."""
    global _TMP
    key = (name, stored, hot)
    if key in _FOLDERS:
        return _FOLDERS[key]
    import alice_llm_amd as alice
    if _TMP is None:
        _TMP = tempfile.TemporaryDirectory(prefix="alice_tests_")
    folder = os.path.join(_TMP.name, f"{name}-{stored}-{hot}")
    raw, seed = TINY[name]
    alice.write_random_model(folder, dict(raw), seed, {"bfloat16": torch.bfloat16, "float32": torch.float32}[stored])
    if hot != 1.0:
        from safetensors.torch import load_file, save_file
        path = os.path.join(folder, "model.safetensors")
        t = load_file(path)
        for k in t:
            if "q_proj" in k or "k_proj" in k or "embed_tokens" in k:
                t[k] = (t[k].float() * hot).to(t[k].dtype)
        save_file(t, path)
    _FOLDERS[key] = folder
    return folder


def write_marker_model(folder: str, raw: dict, seed: int, markers=(7, 8, 9)) -> None:
    """A model folder with random weights, edited so that the keys of the marker tokens stand out: every query scores
    them far above all other keys (one hidden feature that only the markers' embeddings have, read by one row of
    every key projection; a constant feature read by the matching row of every query projection; the pair sits in
    the rotation's slowest plane, so the score survives thousands of positions).  Among thousands of keys with nearly
    equal weights one key more or less changes nothing that a tolerance sees; one marker more or less does."""
    import alice_llm_amd as alice
    from safetensors.torch import load_file, save_file
    alice.write_random_model(folder, dict(raw), seed=seed)
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    d, nH, nKV = raw["head_dim"], raw["num_attention_heads"], raw["num_key_value_heads"]
    E = t["model.embed_tokens.weight"].float()
    E[:, 0] = 0.1                       # a feature every token has
    E[:, 1:2 + len(markers)] = 0.0
    for n, m in enumerate(markers):
        E[m, 1] = 0.5                   # one that only the markers have, which the keys read,
        E[m, 2 + n] = 0.5               # and one of its own for each marker, so that their values differ
    t["model.embed_tokens.weight"] = E.to(torch.bfloat16)
    j = d // 2 - 1                      # the slowest plane of the rotation: rows j and j + d/2 of a head
    for i in range(raw["num_hidden_layers"]):
        q = t[f"model.layers.{i}.self_attn.q_proj.weight"].float()
        k = t[f"model.layers.{i}.self_attn.k_proj.weight"].float()
        for h in range(nH):
            q[h * d + j, 0] += 2.0
        for h in range(nKV):
            k[h * d + j, 1] += 2.0
        t[f"model.layers.{i}.self_attn.q_proj.weight"] = q.to(torch.bfloat16)
        t[f"model.layers.{i}.self_attn.k_proj.weight"] = k.to(torch.bfloat16)
    save_file(t, path)


def plain_model(folder: str, dense: bool = False, device="cpu"):
    """dense: attention as one masked matrix product per head instead of key by key (the two forms are tested
    against each other); what sequences of thousands of tokens need."""
    from plain.gemma2_plain import PlainGemma2
    return PlainGemma2.from_folder(folder, dense=dense, device=device)


def random_tokens(vocab: int, n: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# Tolerances on logits, absolute, against the 64-bit plain implementation.
#   float32: sums of a few hundred 32-bit products and two dozen ops deep: errors stay near 1e-6 for
#            logits of order 1; 2e-5 leaves an order of magnitude.
#   bfloat16: activations are rounded to 8 bits of mantissa (relative 2^-9) between kernels; through a few
#            layers the logits (of order 1) carry errors of a few 1e-3 to 1e-2; a wrong mask, position or
#            head gives errors of order 0.1 to 1.
TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def max_err(a: torch.Tensor, b: torch.Tensor) -> float:
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


def model_from_tensors(cfg, tensors, dtype):
    """A model of the package filled with given tensors (by name, on the device), as the loader fills it from a folder."""
    from alice_llm_amd.api import Model
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.parts import Precision
    lm = CausalLM(cfg.plan(), Precision.of(dtype), next(iter(tensors.values())).device)
    for name in lm.param_specs():
        lm.assign(name, tensors[name])
    lm.finalize()
    return Model(cfg, lm)


# ------------------------------------------------------------------ Novotar: three small configurations
def _nv_layer(left, right, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


# A: a loop in the middle run twice, a token-side input, grouped kv heads, value heads twice the key size, a window
#    shorter than a page, one layer without a feed-forward.
# B: no loop, no token-side input, kv heads = heads, value size = key size, a window longer than a page, value heads
#    of the matrix memory that fit no tile (40), eps and embedding scale other than A's, limits that never bind.
# C: sizes that suit the matrix cores, a loop over every layer run three times, one kv head, window 100.
def _nv_a():
    le = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.3, "mask": {"size": 5}}
    ri = {"heads": 2, "dim": 16, "vdim": 32, "gate_cap": 8.0}
    mlp = {"kind": "dense", "ff": 96, "limit": 1.5}
    return {"architecture": "Novotar", "vocab": 97, "width": 64, "embedding": {"scale": 4.0}, "norm": {"eps": 1e-6},
            "layers": [_nv_layer(le, ri, mlp), _nv_layer(le, ri, None), _nv_layer(dict(le, mask={"size": 9}), ri, mlp)],
            "loop": {"start": 1, "stop": 3, "times": 2}, "token_side": {"dim": 8}}


def _nv_b():
    le = {"heads": 3, "kv_heads": 3, "dim": 24, "vdim": 24, "scale": 0.2, "mask": {"size": 70}}
    ri = {"heads": 3, "dim": 8, "vdim": 40, "gate_cap": 15.0}
    mlp = {"kind": "dense", "ff": 80, "limit": 50.0}
    return {"architecture": "Novotar", "vocab": 130, "width": 96, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
            "layers": [_nv_layer(le, ri, mlp), _nv_layer(le, dict(ri, heads=1, dim=32, vdim=16), mlp)]}


def _nv_c():
    le = {"heads": 4, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 100}}
    ri = {"heads": 2, "dim": 64, "vdim": 128, "gate_cap": 10.0}
    mlp = {"kind": "dense", "ff": 256, "limit": 3.0}
    return {"architecture": "Novotar", "vocab": 300, "width": 128, "embedding": {"scale": 8.0}, "norm": {"eps": 1e-6},
            "layers": [_nv_layer(le, ri, mlp), _nv_layer(le, ri, mlp)],
            "loop": {"start": 0, "stop": 2, "times": 3}, "token_side": {"dim": 16}}


# D: sizes that fit no tile anywhere (width 72, heads of 20 / 28 / 12, a side input of 5), one kv head for three
#    query heads, a loop over the first layer alone, a layer without a window.
def _nv_d():
    le = {"heads": 3, "kv_heads": 1, "dim": 20, "vdim": 28, "scale": 0.25, "mask": {"size": 33}}
    ri = {"heads": 2, "dim": 12, "vdim": 20, "gate_cap": 6.0}
    mlp = {"kind": "dense", "ff": 100, "limit": 2.5}
    free = {k: v for k, v in le.items() if k != "mask"}
    return {"architecture": "Novotar", "vocab": 61, "width": 72, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-6},
            "layers": [_nv_layer(le, ri, mlp), _nv_layer(free, ri, mlp)],
            "loop": {"start": 0, "stop": 1, "times": 2}, "token_side": {"dim": 5}}


NOVOTAR = {"nv-a": _nv_a, "nv-b": _nv_b, "nv-c": _nv_c, "nv-d": _nv_d}


def novotar_folder(name: str, seed: int = 0) -> str:
    """A model folder (config.json, model.safetensors in bfloat16) of a Novotar test configuration."""
    global _TMP
    key = ("novotar", name, seed)
    if key not in _FOLDERS:
        from safetensors.torch import save_file
        if _TMP is None:
            _TMP = tempfile.TemporaryDirectory(prefix="alice_tests_")
        folder = os.path.join(_TMP.name, f"{name}-{seed}")
        os.makedirs(folder, exist_ok=True)
        raw = NOVOTAR[name]()
        _, tensors = novotar_tensors(raw, seed)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(raw, f)
        save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
        _FOLDERS[key] = folder
    return _FOLDERS[key]


def novotar_tensors(raw: dict, seed: int):
    """Random tensors for a Novotar configuration, by name, in bfloat16 on the CPU: matrices N(0, gain^2 / inputs) with
    gains that make every mechanism matter (gates that open and close, limits that bind, scores of order 1), norm
    weights around 1."""
    import alice_llm_amd as alice
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.parts import Precision
    cfg = alice.config_from_dict(raw)
    specs = CausalLM(cfg.plan(), Precision.of("float32"), "cpu").param_specs()
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in specs.items():
        shape = tuple(spec.shape)
        r = torch.randn(shape, generator=g)
        if len(shape) == 1:
            t = r if name.endswith(".b") else 1.0 + 0.2 * r
        elif name in ("embed", "side.embed"):
            t = r * (0.5 if name == "embed" else 1.0)
        else:
            gain = 2.0 if name.endswith((".i", ".f", "left.q", "left.k", "left.g")) else 1.0
            t = r * gain / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return cfg, out


def novotar_pair(name: str, dtype: str, seed: int = 0, device="cuda"):
    """(the package's model, the plain model) on the same tensors."""
    from plain.novotar_plain import PlainNovotar
    raw = NOVOTAR[name]()
    cfg, tensors = novotar_tensors(raw, seed)
    plain = PlainNovotar(raw, {k: v.double() for k, v in tensors.items()})
    model = model_from_tensors(cfg, {k: v.to(device) for k, v in tensors.items()}, dtype)
    return model, plain


# --------------------------------------------------------------------------- Telulorn test configurations
# A: a loop in the middle run twice; grouped kv heads; value heads twice / half the key size; a chunk and a window
#    shorter than a page; a part of the head rotated; one layer without a feed-forward; side factors other than 1.
# B: no loop; kv heads = heads; sizes that fit no tile (width 72, heads of 20 / 28 / 12); the whole head rotated; a
#    window and a chunk longer than a page; tau 1; both side factors 1.
# C: sizes that suit the matrix cores; a loop over every layer run three times; one kv head; a chunk of exactly a
#    page; kept first positions that reach into the second page; value heads of the recurrence wider than 64.
# D: an attention layer first; a loop over the first layer alone; a layer without any mask or rotation and one whose
#    window keeps no first positions; keys of the recurrence wider than 128; three query heads a kv head.
def _tl_par(left, right, mlp, ls=1.0, rs=1.0):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def _tl_a():
    le = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.3, "mask": {"size": 7}}
    ri = {"heads": 2, "dim": 16, "vdim": 32, "tau": 4.0, "rank": 8}
    at = {"heads": 4, "kv_heads": 1, "dim": 32, "vdim": 16, "scale": 0.2, "mask": {"size": 9, "keep_first": 3},
          "rot": {"base": 100.0, "dims": 16}}
    mlp = {"kind": "dense", "ff": 96}
    return {"architecture": "Telulorn", "vocab": 97, "width": 64, "norm": {"eps": 1e-6},
            "layers": [_tl_par(le, ri, mlp, 0.8, 1.3), {"type": "attention", "mixer": at, "mlp": mlp}, _tl_par(le, ri, None, 1.5, 0.7)],
            "loop": {"start": 1, "stop": 3, "times": 2}}


def _tl_b():
    le = {"heads": 3, "kv_heads": 3, "dim": 20, "vdim": 28, "scale": 0.25, "mask": {"size": 100}}
    ri = {"heads": 3, "dim": 12, "vdim": 20, "tau": 1.0, "rank": 5}
    at = {"heads": 3, "kv_heads": 3, "dim": 20, "vdim": 20, "scale": 0.3, "mask": {"size": 70, "keep_first": 5},
          "rot": {"base": 10000.0, "dims": 20}}
    mlp = {"kind": "dense", "ff": 100}
    return {"architecture": "Telulorn", "vocab": 130, "width": 72, "norm": {"eps": 1e-5},
            "layers": [_tl_par(le, ri, mlp), {"type": "attention", "mixer": at, "mlp": mlp}]}


def _tl_c():
    le = {"heads": 4, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 64}}
    ri = {"heads": 2, "dim": 64, "vdim": 128, "tau": 16.0, "rank": 32}
    at = {"heads": 4, "kv_heads": 1, "dim": 64, "vdim": 128, "scale": 0.125, "mask": {"size": 40, "keep_first": 70},
          "rot": {"base": 500.0, "dims": 32}}
    mlp = {"kind": "dense", "ff": 256}
    return {"architecture": "Telulorn", "vocab": 300, "width": 128, "norm": {"eps": 1e-6},
            "layers": [{"type": "attention", "mixer": at, "mlp": mlp}, _tl_par(le, ri, mlp, 1.1, 0.9)],
            "loop": {"start": 0, "stop": 2, "times": 3}}


def _tl_d():
    le = {"heads": 3, "kv_heads": 1, "dim": 24, "vdim": 24, "scale": 0.2}
    ri = {"heads": 1, "dim": 136, "vdim": 24, "tau": 8.0, "rank": 3}
    at = {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.25, "mask": {"size": 33}, "rot": {"base": 50.0, "dims": 8}}
    free = {k: v for k, v in at.items() if k not in ("mask", "rot")}      # no mask and no rotation at all
    mlp = {"kind": "dense", "ff": 80}
    return {"architecture": "Telulorn", "vocab": 61, "width": 48, "norm": {"eps": 1e-6},
            "layers": [{"type": "attention", "mixer": at, "mlp": mlp}, _tl_par(le, ri, mlp, 1.2, 1.0),
                       {"type": "attention", "mixer": free, "mlp": None}],
            "loop": {"start": 0, "stop": 1, "times": 2}}


TELULORN = {"tl-a": _tl_a, "tl-b": _tl_b, "tl-c": _tl_c, "tl-d": _tl_d}


def telulorn_tensors(raw: dict, seed: int):
    """Random tensors for a Telulorn configuration, by name, in bfloat16 on the CPU: matrices N(0, gain^2 / inputs)
    with gains that make every mechanism matter (sharp softmaxes, gates that open and close, sinks of the scores'
    order, a head mix far from the identity, decays from fast to almost none), norm weights around 1."""
    import alice_llm_amd as alice
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.parts import Precision
    cfg = alice.config_from_dict(raw)
    specs = CausalLM(cfg.plan(), Precision.of("float32"), "cpu").param_specs()
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in specs.items():
        shape = tuple(spec.shape)
        r = torch.randn(shape, generator=g)
        if name.endswith(".sink"):
            t = 1.5 * r
        elif name.endswith("a2.b"):
            t = 2.0 + 3.0 * r                       # sigmoid(.)^(1/tau) from about 0.5 to almost 1
        elif name.endswith(".talk"):
            t = torch.eye(shape[0]) * 0.7 + 0.4 * r
        elif name == "loop.step":
            t = 0.3 * r
        elif len(shape) == 1:
            t = 0.5 * r if name.endswith(".b") else 1.0 + 0.2 * r
        elif name == "embed":
            t = r * 0.5
        else:
            gain = 2.5 if name.endswith((".q", ".k", ".g", ".a2")) else 1.0
            t = r * gain / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return cfg, out


def telulorn_pair(name: str, dtype: str, seed: int = 0, device="cuda"):
    """(the package's model, the plain model) on the same tensors."""
    from plain.telulorn_plain import PlainTelulorn
    raw = TELULORN[name]()
    cfg, tensors = telulorn_tensors(raw, seed)
    plain = PlainTelulorn(raw, tensors)
    model = model_from_tensors(cfg, {k: v.to(device) for k, v in tensors.items()}, dtype)
    return model, plain


def telulorn_folder(name: str, seed: int = 0) -> str:
    """A model folder (config.json without the decay projection's middle width, which the tensors give;
    model.safetensors in bfloat16) of a Telulorn test configuration."""
    global _TMP
    key = ("telulorn", name, seed)
    if key not in _FOLDERS:
        from safetensors.torch import save_file
        if _TMP is None:
            _TMP = tempfile.TemporaryDirectory(prefix="alice_tests_")
        folder = os.path.join(_TMP.name, f"{name}-{seed}")
        os.makedirs(folder, exist_ok=True)
        raw = TELULORN[name]()
        _, tensors = telulorn_tensors(raw, seed)
        for l in raw["layers"]:
            if l["type"] == "parallel":
                l["mixer"]["right"].pop("rank", None)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(raw, f)
        save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
        _FOLDERS[key] = folder
    return _FOLDERS[key]


# --------------------------------------------------------------------------- Pefitar test configurations
# A: a loop in the middle run twice; the latent layer's sizes all multiples of 8 and all different (query latent 40,
#    key/value latent 32, plain 16, rotated 8, values 24), a window shorter than a page; grouped kv heads with a part
#    of the head rotated; one layer without a feed-forward; stream factor 0.7.
# B: no loop; sizes that fit no tile (width 72, a latent of 44 beside 6 rotated dimensions, heads of 20 / 28); a window
#    longer than a page; kv heads = heads with the whole head rotated; stream factor 1; no logit cap.
# C: sizes that suit the matrix cores (latent 128 beside 32 rotated, values 64, heads of 64); a loop over every layer
#    run three times; a window of exactly a page; one kv head; values wider than keys.
# D: an attention layer first; a loop over the first layer alone; two latent layers that differ in every size, one
#    whose window is a single key and one without any window; three query heads a kv head.
def _pf_lat(heads, dim, rot, vdim, qr, kvr, scale, window, base=1000.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": qr, "kv_rank": kvr, "scale": scale,
         "rot": {"base": base, "dims": rot}}
    if window is not None:
        m["mask"] = {"size": window}
    return m


def _pf_a():
    lat = _pf_lat(4, 16, 8, 24, 40, 32, 0.3, 9, base=100.0)
    att = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.3, "rot": {"base": 100.0, "dims": 8}}
    mlp = {"kind": "dense", "ff": 96}
    return {"architecture": "Pefitar", "vocab": 97, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 0.7, "logit_softcap": 20.0,
            "layers": [{"type": "latent_attention", "mixer": lat, "mlp": mlp}, {"type": "attention", "mixer": att, "mlp": mlp},
                       {"type": "latent_attention", "mixer": lat, "mlp": None}],
            "loop": {"start": 1, "stop": 3, "times": 2}}


def _pf_b():
    lat = _pf_lat(3, 20, 6, 28, 36, 44, 0.25, 70, base=10000.0)
    att = {"heads": 3, "kv_heads": 3, "dim": 20, "vdim": 20, "scale": 0.3, "rot": {"base": 10000.0, "dims": 20}}
    mlp = {"kind": "dense", "ff": 100}
    return {"architecture": "Pefitar", "vocab": 130, "width": 72, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
            "layers": [{"type": "latent_attention", "mixer": lat, "mlp": mlp}, {"type": "attention", "mixer": att, "mlp": mlp}]}


def _pf_c():
    lat = _pf_lat(4, 32, 32, 64, 64, 128, 0.125, 64, base=500.0)
    att = {"heads": 4, "kv_heads": 1, "dim": 64, "vdim": 128, "scale": 0.125, "rot": {"base": 500.0, "dims": 32}}
    mlp = {"kind": "dense", "ff": 256}
    return {"architecture": "Pefitar", "vocab": 300, "width": 128, "norm": {"eps": 1e-6}, "residual_mult": 0.4, "logit_softcap": 25.0,
            "layers": [{"type": "attention", "mixer": att, "mlp": mlp}, {"type": "latent_attention", "mixer": lat, "mlp": mlp}],
            "loop": {"start": 0, "stop": 2, "times": 3}}


def _pf_d():
    att = {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.25, "rot": {"base": 50.0, "dims": 16}}
    one = _pf_lat(2, 8, 16, 40, 24, 16, 0.3, 1, base=50.0)
    free = _pf_lat(5, 24, 8, 8, 16, 56, 0.2, None, base=3000.0)
    mlp = {"kind": "dense", "ff": 80}
    return {"architecture": "Pefitar", "vocab": 61, "width": 48, "norm": {"eps": 1e-6}, "residual_mult": 1.3, "logit_softcap": 30.0,
            "layers": [{"type": "attention", "mixer": att, "mlp": mlp}, {"type": "latent_attention", "mixer": one, "mlp": mlp},
                       {"type": "latent_attention", "mixer": free, "mlp": None}],
            "loop": {"start": 0, "stop": 1, "times": 2}}


PEFITAR = {"pf-a": _pf_a, "pf-b": _pf_b, "pf-c": _pf_c, "pf-d": _pf_d}


def pefitar_tensors(raw: dict, seed: int):
    """Random tensors for a Pefitar configuration, by name, in bfloat16 on the CPU: matrices N(0, gain^2 / inputs) with
    gains that make softmaxes sharp and gates open and close; norm weights around 1."""
    import alice_llm_amd as alice
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.parts import Precision
    cfg = alice.config_from_dict(raw)
    specs = CausalLM(cfg.plan(), Precision.of("float32"), "cpu").param_specs()
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in specs.items():
        shape = tuple(spec.shape)
        r = torch.randn(shape, generator=g)
        if len(shape) == 1:
            t = 1.0 + 0.2 * r
        elif name == "embed":
            t = r * 0.5
        else:
            # every branch is normed again behind its sublayer, so a rounding inside it reaches the stream undamped:
            # the gains of the score's two sides are kept lower than the gate's
            gain = 2.5 if name.endswith(".g") else 1.6 if name.endswith((".q", ".k", ".uq", ".uk")) else 1.0
            t = r * gain / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return cfg, out


class PlainPefitar:
    """The plain model on given tensors: forward(tokens) -> logits [T, vocab] in 64-bit."""

    def __init__(self, raw, tensors):
        from plain import pefitar_plain
        self.P, self.c, self.t = pefitar_plain, raw, {k: v.double() for k, v in tensors.items()}

    @classmethod
    def from_folder(cls, folder):
        from plain import pefitar_plain
        return cls(*pefitar_plain.load_folder(folder))

    def forward(self, tokens, return_layers=False):
        return self.P.forward(self.c, self.t, tokens, return_stream=return_layers)

    def greedy(self, prompt, n):
        seq, out = list(prompt), []
        for _ in range(n):
            out.append(int(self.forward(seq)[-1].argmax()))
            seq.append(out[-1])
        return out


def pefitar_pair(name: str, dtype: str, seed: int = 0, device="cuda"):
    """(the package's model, the plain model) on the same tensors."""
    raw = PEFITAR[name]()
    cfg, tensors = pefitar_tensors(raw, seed)
    model = model_from_tensors(cfg, {k: v.to(device) for k, v in tensors.items()}, dtype)
    return model, PlainPefitar(raw, tensors)


def pefitar_folder(name: str, seed: int = 0) -> str:
    """A model folder (config.json, model.safetensors in bfloat16) of a Pefitar test configuration."""
    global _TMP
    key = ("pefitar", name, seed)
    if key not in _FOLDERS:
        from safetensors.torch import save_file
        if _TMP is None:
            _TMP = tempfile.TemporaryDirectory(prefix="alice_tests_")
        folder = os.path.join(_TMP.name, f"{name}-{seed}")
        os.makedirs(folder, exist_ok=True)
        raw = PEFITAR[name]()
        _, tensors = pefitar_tensors(raw, seed)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(raw, f)
        save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
        _FOLDERS[key] = folder
    return _FOLDERS[key]


# --------------------------------------------------------------------------- Vifirax test configurations
# A: a state-space layer first (grouped B and C, four norm parts); attention with grouped kv heads, values twice the key
#    size, a part of the head turned with stretched frequencies, a routed feed-forward (2 of 6); a delta-rule layer with
#    grouped q and k and no feed-forward; an attention layer that reads the second layer's keys.
# B: sizes that fit no tile (width 72, heads of 20 / 28 / 12); attention first with the whole head turned and no
#    stretching, kv heads = heads; a routed feed-forward that uses every expert and one that uses a single one; a
#    convolution of one tap (no convolution state); eps other than A's; no logit factor in the file.
# C: sizes that suit the matrix cores; a delta-rule layer first with one q/k head for two heads and values wider than
#    64; a state of 128 numbers a column; two attention layers that read another's keys, one without a feed-forward;
#    an attention layer with no rotation at all.
# D: two layers that read the first layer's keys; key sizes of the recurrences beyond 128; five taps; three query heads a
#    kv head; three norm parts; a single delta-rule head.
# E: no attention at all (the cache holds no pages); a group a head and a norm part a head; two experts, both for every token.
def _vx_rot(base, dims, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return rot


def _vx_moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _vx_a():
    at = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.6, "rot": _vx_rot(100.0, 8, (4.0, 16, 8.0, 1.0))}
    ss = {"heads": 4, "vdim": 16, "state": 8, "groups": 2, "norm_groups": 4, "conv": 4}
    de = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "conv": 2, "decay_rank": 6, "gate_rank": 5}
    return {"architecture": "Vifirax", "vocab": 97, "width": 64, "norm": {"eps": 1e-6}, "logit_scale": 0.37,
            "layers": [{"type": "mamba2", "mixer": ss, "mlp": {"kind": "dense", "ff": 96}},
                       {"type": "attention", "mixer": at, "mlp": _vx_moe(6, 2, 24)},
                       {"type": "channel_delta", "mixer": de, "mlp": None},
                       {"type": "attention", "mixer": dict(at, kv_from=1), "mlp": {"kind": "dense", "ff": 40}}]}


def _vx_b():
    at = {"heads": 3, "kv_heads": 3, "dim": 20, "vdim": 28, "scale": 0.5, "rot": _vx_rot(10000.0, 20)}
    de = {"heads": 3, "kv_heads": 3, "dim": 12, "vdim": 20, "conv": 3, "decay_rank": 7, "gate_rank": 3}
    ss = {"heads": 3, "vdim": 20, "state": 12, "groups": 3, "norm_groups": 1, "conv": 1}
    return {"architecture": "Vifirax", "vocab": 130, "width": 72, "norm": {"eps": 1e-5},
            "layers": [{"type": "attention", "mixer": at, "mlp": _vx_moe(5, 5, 18)},
                       {"type": "channel_delta", "mixer": de, "mlp": {"kind": "dense", "ff": 100}},
                       {"type": "mamba2", "mixer": ss, "mlp": _vx_moe(3, 1, 40)}]}


def _vx_c():
    at = {"heads": 4, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.25, "rot": _vx_rot(500.0, 32, (16.0, 64, 4.0, 0.5))}
    free = {"heads": 2, "kv_heads": 2, "dim": 128, "vdim": 32, "scale": 0.2}
    de = {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 128, "conv": 4, "decay_rank": 32, "gate_rank": 16}
    ss = {"heads": 4, "vdim": 64, "state": 128, "groups": 1, "norm_groups": 2, "conv": 4}
    dense = {"kind": "dense", "ff": 256}
    return {"architecture": "Vifirax", "vocab": 300, "width": 128, "norm": {"eps": 1e-6}, "logit_scale": 2.0,
            "layers": [{"type": "channel_delta", "mixer": de, "mlp": dense},
                       {"type": "attention", "mixer": at, "mlp": _vx_moe(8, 2, 64)},
                       {"type": "mamba2", "mixer": ss, "mlp": dense},
                       {"type": "attention", "mixer": dict(at, kv_from=1), "mlp": None},
                       {"type": "attention", "mixer": free, "mlp": dense},
                       {"type": "attention", "mixer": dict(at, kv_from=1), "mlp": _vx_moe(4, 3, 32)}]}


def _vx_d():
    at = {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.7, "rot": _vx_rot(50.0, 16, (2.0, 32, 2.0, 1.0))}
    ss = {"heads": 2, "vdim": 24, "state": 136, "groups": 1, "norm_groups": 3, "conv": 2}
    de = {"heads": 1, "kv_heads": 1, "dim": 136, "vdim": 24, "conv": 5, "decay_rank": 3, "gate_rank": 9}
    return {"architecture": "Vifirax", "vocab": 61, "width": 48, "norm": {"eps": 2e-6}, "logit_scale": 0.8,
            "layers": [{"type": "attention", "mixer": at, "mlp": None},
                       {"type": "attention", "mixer": dict(at, kv_from=0), "mlp": _vx_moe(4, 3, 16)},
                       {"type": "mamba2", "mixer": ss, "mlp": {"kind": "dense", "ff": 80}},
                       {"type": "attention", "mixer": dict(at, kv_from=0), "mlp": {"kind": "dense", "ff": 64}},
                       {"type": "channel_delta", "mixer": de, "mlp": _vx_moe(7, 2, 8)}]}


def _vx_e():
    ss = {"heads": 8, "vdim": 8, "state": 16, "groups": 4, "norm_groups": 2, "conv": 3}
    de = {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 40, "conv": 4, "decay_rank": 4, "gate_rank": 4}
    return {"architecture": "Vifirax", "vocab": 83, "width": 40, "norm": {"eps": 1e-6}, "logit_scale": 1.5,
            "layers": [{"type": "channel_delta", "mixer": de, "mlp": _vx_moe(2, 2, 24)},
                       {"type": "mamba2", "mixer": ss, "mlp": None},
                       {"type": "mamba2", "mixer": dict(ss, groups=8, norm_groups=8, conv=2), "mlp": {"kind": "dense", "ff": 56}}]}


VIFIRAX = {"vx-a": _vx_a, "vx-b": _vx_b, "vx-c": _vx_c, "vx-d": _vx_d, "vx-e": _vx_e}


def vifirax_tensors(raw: dict, seed: int):
    """Random tensors for a Vifirax configuration, by name, in bfloat16 on the CPU: matrices N(0, gain^2 / inputs) with
    gains that make every mechanism matter (sharp softmaxes, gates that open and close, routers that decide, decays
    from fast to almost none), layer norm weights around 0 (they enter as 1 + w) and the mixers' plain ones around 1."""
    import alice_llm_amd as alice
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.parts import Precision
    cfg = alice.config_from_dict(raw)
    specs = CausalLM(cfg.plan(), Precision.of("float32"), "cpu").param_specs()
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in specs.items():
        shape = tuple(spec.shape)
        r = torch.randn(shape, generator=g)
        last = name.rsplit(".", 1)[-1]
        if last == "A_log":
            t = -2.0 + 1.5 * r                      # rates from a few thousandths to about one
        elif last == "dt_bias":
            t = 0.5 * r
        elif last == "D":
            t = r
        elif last == "conv":
            t = 0.6 * r
        elif len(shape) == 1 and (last in ("norm1", "norm2") or name == "final.norm"):
            t = 0.2 * r
        elif len(shape) == 1:
            t = 0.5 * r if last == "b" else 1.0 + 0.2 * r
        elif name == "embed":
            t = r * 0.5
        else:
            gain = 2.5 if last in ("q", "k", "g", "a2", "g2", "router", "b") else 1.0
            t = r * gain / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return cfg, out


def vifirax_pair(name: str, dtype: str, seed: int = 0, device="cuda"):
    """(the package's model, the plain model) on the same tensors."""
    from plain.vifirax_plain import PlainVifirax
    raw = VIFIRAX[name]()
    cfg, tensors = vifirax_tensors(raw, seed)
    plain = PlainVifirax(raw, {k: v.double() for k, v in tensors.items()})
    model = model_from_tensors(cfg, {k: v.to(device) for k, v in tensors.items()}, dtype)
    return model, plain


def vifirax_folder(name: str, seed: int = 0) -> str:
    """A model folder (config.json without the widths of the narrow middles, which the tensors give; model.safetensors in
    bfloat16) of a Vifirax test configuration."""
    global _TMP
    key = ("vifirax", name, seed)
    if key not in _FOLDERS:
        from safetensors.torch import save_file
        if _TMP is None:
            _TMP = tempfile.TemporaryDirectory(prefix="alice_tests_")
        folder = os.path.join(_TMP.name, f"{name}-{seed}")
        os.makedirs(folder, exist_ok=True)
        raw = VIFIRAX[name]()
        _, tensors = vifirax_tensors(raw, seed)
        for l in raw["layers"]:
            l["mixer"].pop("decay_rank", None)
            l["mixer"].pop("gate_rank", None)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(raw, f)
        save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
        _FOLDERS[key] = folder
    return _FOLDERS[key]
