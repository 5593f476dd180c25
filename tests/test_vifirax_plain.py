"""Vifirax on the CPU: the configuration reader and its refusals, the plan (which parts with which constants, which
run reads whose cache), tensor names and shapes, the sizes that only tensors give, and the plain implementation's
own invariants (a recurrence and a convolution cut in two, stretched frequencies, the one in the softmax's
denominator, the router's choice, keys read from another layer)."""
import json
import math

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.engine.model import CausalLM
from alice_llm_amd.parts import Precision
from helpers import VIFIRAX, random_tokens, vifirax_tensors
from plain import vifirax_plain as P


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


# ------------------------------------------------------------------ configuration and plan

def test_architecture_is_found_by_its_key_and_round_trips():
    raw = VIFIRAX["vx-a"]()
    cfg = alice.config_from_dict(raw)
    assert type(cfg).__name__ == "VifiraxConfig" and "Vifirax" in alice.registered_architectures()
    assert alice.config_from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    plan = cfg.plan()
    assert [(e.layer, e.cache_from) for e in plan.schedule] == [(0, None), (1, None), (2, None), (3, 1)]
    assert [l.mixer.kind for l in plan.layers] == ["mamba2", "attention", "channel_delta", "attention"]
    assert [None if l.feed_forward is None else l.feed_forward.kind for l in plan.layers] == ["gated_mlp", "expert_mlp", None, "gated_mlp"]
    assert all(set(l.norms) == ({"post_mixer", "post_ff"} if l.feed_forward else {"post_mixer"}) for l in plan.layers)
    assert all(n.args["weight_offset"] == 1.0 for l in plan.layers for n in l.norms.values())
    at, shared = plan.layers[1].mixer.args, plan.layers[3].mixer.args
    assert at["own_keys"] and not shared["own_keys"] and at["sink"] == "zero" and at["qk_norm"] == "projection"
    assert at["output_gate"] == "head" and at["bias"] and at["output_bias"] and at["window"] is None
    assert at["position"] == shared["position"] and len(plan.positions) == 1
    rot = next(iter(plan.positions.values())).args
    assert rot["interleaved"] is False and rot["rotary_dim"] == 8 and rot["scaling"]["factor"] == 4.0
    assert plan.final_norm.args["output_scale"] == 0.37 and plan.head.args["tied_to"] == "embed"
    ex = plan.layers[1].feed_forward.args
    assert (ex["experts"], ex["top"], ex["intermediate_size"]) == (6, 2, 24)


def test_defaults_and_absent_keys():
    plan = alice.config_from_dict(VIFIRAX["vx-b"]()).plan()
    assert plan.final_norm.args["output_scale"] == 1.0
    assert next(iter(plan.positions.values())).args["scaling"] is None
    free = alice.config_from_dict(VIFIRAX["vx-c"]()).plan().layers[4].mixer.args
    assert free["position"] is None
    raw = VIFIRAX["vx-b"]()
    del raw["layers"][0]["mixer"]["kv_heads"], raw["layers"][0]["mixer"]["vdim"], raw["norm"]
    cfg = alice.config_from_dict(raw)
    assert cfg.layers[0]["mixer"]["kv_heads"] == 3 and cfg.layers[0]["mixer"]["vdim"] == 20 and cfg.norm_eps == 1e-6


@pytest.mark.parametrize("change,match", [
    (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda r: r["layers"][3]["mixer"].update(kv_from=2), "kv_from"),
    (lambda r: r["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
    (lambda r: r["layers"][3]["mixer"].update(dim=32), "kv_from"),
    (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=7), "rot"),
    (lambda r: r["layers"][1]["mixer"]["rot"]["scaling"].update(factor=0.0), "scaling"),
    (lambda r: r["layers"][0]["mixer"].update(groups=3), "groups"),
    (lambda r: r["layers"][0]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(top=7), "top"),
    (lambda r: r["layers"][2].update(type="conv"), "no mixer"),
    (lambda r: r["layers"][0]["mlp"].update(kind="sparse"), "no feed-forward"),
    (lambda r: r["layers"][2]["mixer"].pop("conv"), "conv"),
])
def test_refusals(change, match):
    raw = VIFIRAX["vx-a"]()
    change(raw)
    with pytest.raises(alice.ConfigError, match=match):
        alice.config_from_dict(raw)


def test_tensor_names_and_shapes():
    cfg = alice.config_from_dict(VIFIRAX["vx-a"]())
    specs = {k: tuple(v.shape) for k, v in CausalLM(cfg.plan(), Precision.of("float32"), "cpu").param_specs().items()}
    want = {"embed": (97, 64), "l0.norm1": (64,), "l0.norm2": (64,), "l0.mix.in": (2 * 64 + 2 * 16 + 4, 64), "l0.mix.conv": (96, 4),
            "l0.mix.conv.b": (96,), "l0.mix.dt_bias": (4,), "l0.mix.A_log": (4,), "l0.mix.D": (4,), "l0.mix.norm": (64,),
            "l0.mix.o": (64, 64), "l0.mlp.gate": (96, 64), "l0.mlp.down": (64, 96), "l1.mix.q": (64, 64), "l1.mix.q.b": (64,),
            "l1.mix.k": (32, 64), "l1.mix.k.b": (32,), "l1.mix.v": (64, 64), "l1.mix.v.b": (64,), "l1.mix.q.norm": (64,),
            "l1.mix.k.norm": (32,), "l1.mix.g": (4, 64), "l1.mix.o": (64, 128), "l1.mix.o.b": (64,), "l1.mlp.router": (6, 64),
            "l1.mlp.router.b": (6,), "l1.mlp.e5.gate": (24, 64), "l1.mlp.e0.down": (64, 24), "l2.mix.q": (32, 64),
            "l2.mix.q.conv": (32, 2), "l2.mix.k.conv": (32, 2), "l2.mix.v": (32, 64), "l2.mix.v.conv": (32, 2), "l2.mix.b": (4, 64),
            "l2.mix.A_log": (4,), "l2.mix.norm": (8,), "l2.mix.a1": (6, 64), "l2.mix.a2": (64, 6), "l2.mix.dt_bias": (64,),
            "l2.mix.g1": (5, 64), "l2.mix.g2": (32, 5), "l2.mix.o": (64, 32), "l3.mix.q": (64, 64), "l3.mix.q.norm": (64,),
            "l3.mix.g": (4, 64), "l3.mix.o.b": (64,), "final.norm": (64,)}
    for name, shape in want.items():
        assert specs.get(name) == shape, (name, specs.get(name))
    for absent in ("l2.norm2", "l3.mix.k", "l3.mix.v", "l3.mix.k.b", "l3.mix.v.b", "l3.mix.k.norm", "l1.mix.sink", "l1.mlp.e6.up", "head"):
        assert absent not in specs, absent
    # a single tap keeps no inputs
    needs = CausalLM(alice.config_from_dict(VIFIRAX["vx-b"]()).plan(), Precision.of("float32"), "cpu").cache_needs()
    assert [s.name for s in needs[2].state] == ["S"] and [s.name for s in needs[1].state] == ["S", "conv"]
    assert needs[1].state[1].shape == (3 * 12 * 2 + 3 * 20, 2)
    needs = CausalLM(cfg.plan(), Precision.of("float32"), "cpu").cache_needs()
    assert needs[3] is None and needs[1].kv.num_kv_heads == 2 and needs[1].kv.v_dim == 32 and needs[1].kv.window is None


def test_the_narrow_middles_come_from_the_tensors():
    raw = VIFIRAX["vx-a"]()
    del raw["layers"][2]["mixer"]["decay_rank"], raw["layers"][2]["mixer"]["gate_rank"]
    cfg = alice.config_from_dict(raw)
    with pytest.raises(alice.ConfigError, match="middle"):
        cfg.plan()
    full = cfg.with_tensor_shapes({"l2.mix.a1": (6, 64), "l2.mix.g1": (5, 64), "l0.mix.in": (164, 64)})
    args = full.plan().layers[2].mixer.args
    assert args["decay_rank"] == 6 and args["gate_rank"] == 5


# ------------------------------------------------------------------ the plain implementation's own invariants

def test_stretched_frequencies():
    f, m = P.stretched_frequencies(16, 100.0, None)
    assert m == 1.0 and torch.allclose(f, 100.0 ** (-torch.arange(8, dtype=torch.float64) / 8))
    s = {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0}
    g, m = P.stretched_frequencies(16, 100.0, s)
    assert m == pytest.approx(0.1 * math.log(4.0) + 1.0)
    D = lambda t: 16 * math.log(16 / (2 * math.pi * t)) / (2 * math.log(100.0))
    lo, hi = max(math.floor(D(8.0)), 0), min(math.ceil(D(1.0)), 15)
    assert (lo, hi) == (0, 2)
    assert g[0] == f[0] and g[1] == pytest.approx(float(f[1]) * (0.5 + 0.5 / 4)) and torch.allclose(g[2:], f[2:] / 4)
    # hi == lo: the ramp is a step
    g2, _ = P.stretched_frequencies(8, 10.0, {"factor": 2.0, "original": 63, "fast": 10.0, "slow": 10.0})
    f2, _ = P.stretched_frequencies(8, 10.0, None)
    assert g2[0] == f2[0] and torch.allclose(g2[1:], f2[1:] / 2)


def test_rotation_in_halves_keeps_lengths_and_the_rest():
    x = rnd(5, 3, 12, seed=1)
    f, _ = P.stretched_frequencies(8, 50.0, None)
    y = P.rotate_halves(x, torch.arange(5), f, 1.0)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.equal(y[0], x[0])
    assert torch.allclose((y[..., :8] ** 2).sum(-1), (x[..., :8] ** 2).sum(-1))
    assert torch.allclose(y[2, 1, 1] ** 2 + y[2, 1, 5] ** 2, x[2, 1, 1] ** 2 + x[2, 1, 5] ** 2)       # 1 is paired with 5
    y2 = P.rotate_halves(x, torch.arange(5), f, 1.3)
    assert torch.allclose(y2[..., :8], 1.3 * y[..., :8])


def test_one_more_in_the_denominator():
    s = rnd(4, 6, seed=2, scale=3.0)
    mask = torch.arange(6)[None, :] <= torch.arange(4)[:, None] + 2
    w = P.one_more_softmax(s, mask)
    e = torch.exp(s) * mask
    assert torch.allclose(w, e / (1 + e.sum(-1, keepdim=True)))
    assert float(P.one_more_softmax(torch.full((1, 3), -80.0, dtype=torch.float64), torch.ones(1, 3, dtype=torch.bool)).sum()) < 1e-30
    big = P.one_more_softmax(torch.tensor([[900.0, 0.0]], dtype=torch.float64), torch.ones(1, 2, dtype=torch.bool))
    assert float(big[0, 0]) == pytest.approx(1.0) and torch.isfinite(big).all()


def test_convolution_cut_in_two():
    x, w, b = rnd(11, 5, seed=3), rnd(5, 4, seed=4), rnd(5, seed=5)
    whole = P.causal_conv(x, w, b)
    assert torch.allclose(whole[0], x[0] * w[:, 3] + b) and torch.allclose(whole[1], x[1] * w[:, 3] + x[0] * w[:, 2] + b)
    for cut in (1, 2, 3, 7):
        pad = torch.cat([torch.zeros(3, 5, dtype=torch.float64), x[:cut]])[-3:]
        assert torch.allclose(P.causal_conv(x[cut:], w, b, pad), whole[cut:])


@pytest.mark.parametrize("kind", ["mamba2", "channel_delta"])
def test_recurrent_mixers_cut_in_pieces_carry_their_state(kind):
    raw = VIFIRAX["vx-a"]()
    i = 0 if kind == "mamba2" else 2
    _, tensors = vifirax_tensors(raw, 3)
    p = {k[len(f"l{i}.mix."):]: v.double() for k, v in tensors.items() if k.startswith(f"l{i}.mix.")}
    fn = P.mamba2_mixer if kind == "mamba2" else P.channel_delta_mixer
    h = rnd(23, 64, seed=6)
    whole = fn(h, p, raw["layers"][i]["mixer"], 1e-6)
    for cuts in ([1, 1, 2, 19], [22, 1], [3, 20]):
        state, outs, at = None, [], 0
        for c in cuts:
            o, state = fn(h[at:at + c], p, raw["layers"][i]["mixer"], 1e-6, state, return_state=True)
            outs.append(o)
            at += c
        assert torch.allclose(torch.cat(outs), whole, atol=1e-10), cuts


def test_delta_rule_replaces_what_a_key_held():
    """With no decay and full write strength, writing twice under one unit key leaves the second value only."""
    k = torch.zeros(2, 1, 4, dtype=torch.float64)
    k[:, 0, 1] = 1.0
    v = rnd(2, 1, 3, seed=7)
    o, S = P.delta_rule_scan(k, k, v, torch.ones(2, 1, 4, dtype=torch.float64), torch.ones(2, 1, dtype=torch.float64))
    assert torch.allclose(o, v) and torch.allclose(S[0, 1], v[1, 0]) and float(S[0, [0, 2, 3]].abs().max()) == 0.0


def test_router_choice_and_the_experts_mix():
    W, E, F = 16, 5, 6
    p = {"router": rnd(E, W, seed=8), "router.b": rnd(E, seed=9)}
    for e in range(E):
        p.update({f"e{e}.gate": rnd(F, W, seed=10 + e), f"e{e}.up": rnd(F, W, seed=20 + e), f"e{e}.down": rnd(W, F, seed=30 + e)})
    h = rnd(7, W, seed=40)
    z = h @ p["router"].T + p["router.b"]
    every = torch.stack([P.gated_ff(h, p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"]) for e in range(E)], dim=1)
    all_of_them = P.routed_ff(h, p, {"router": {"experts": E, "top": E}})
    assert torch.allclose(all_of_them, (torch.softmax(z, -1)[:, :, None] * every).sum(1))
    one = P.routed_ff(h, p, {"router": {"experts": E, "top": 1}})
    assert torch.allclose(one, every[torch.arange(7), z.argmax(-1)])


def test_a_layer_that_reads_anothers_keys_sees_them():
    """Changing the key matrix of the layer that owns the keys changes the reading layer's output from its own first
    sublayer on; the reading layer has no key tensors to change."""
    raw = VIFIRAX["vx-d"]()
    _, tensors = vifirax_tensors(raw, 4)
    t = {k: v.double() for k, v in tensors.items()}
    toks = random_tokens(61, 12, 1)
    base, layers = P.forward(raw, t, toks, return_layers=True)
    assert not any(k.startswith(("l1.mix.k", "l1.mix.v", "l3.mix.k")) for k in t)
    raw2 = VIFIRAX["vx-d"]()
    raw2["layers"][1]["mixer"] = dict(raw2["layers"][1]["mixer"], kv_from=None)
    with pytest.raises(KeyError):
        P.forward(raw2, t, toks)                                  # keys of its own would need tensors of its own
    t2 = dict(t)
    t2["l0.mix.v"] = t["l0.mix.v"] * 1.5
    _, layers2 = P.forward(raw, t2, toks, return_layers=True)
    assert not torch.allclose(layers2[0], layers[0]) and not torch.allclose(layers2[1], layers[1])
    assert base.shape == (12, 61)
