"""Pefitar on the CPU: the configuration reader, its defaults and refusals, the plan's order of layer runs, tensor
names and shapes, what the latent layers ask of the cache, and the plain implementation's own invariants (the latent
attention with the per-head maps on the query's side equals the one with keys and values made per head, the edges of
a window, the rotation's dependence on the distance alone, the gate, the loop, the stream's factor, the logit cap)."""
import json
import math

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.cache import Cache
from alice_llm_amd.config.plan import ConfigError
from alice_llm_amd.engine.model import CausalLM
from alice_llm_amd.parts import Precision
from helpers import PEFITAR, PlainPefitar, pefitar_tensors, random_tokens
from plain import pefitar_plain as P


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


# ------------------------------------------------------------------ configuration and plan

def test_architecture_is_found_by_its_key_and_round_trips():
    raw = PEFITAR["pf-a"]()
    cfg = alice.config_from_dict(raw)
    assert type(cfg).__name__ == "PefitarConfig" and "Pefitar" in alice.registered_architectures()
    assert alice.config_from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    assert cfg.layer_runs() == [0, 1, 2, 1, 2] == P.layer_runs(raw)
    plan = cfg.plan()
    assert [e.layer for e in plan.schedule] == [0, 1, 2, 1, 2] and all(e.before is None for e in plan.schedule)
    assert plan.layers[2].feed_forward is None and "pre_ff" not in plan.layers[2].norms
    lat, att = plan.layers[0].mixer, plan.layers[1].mixer
    assert lat.kind == "latent_attention" and att.kind == "attention"
    assert (lat.args["q_rank"], lat.args["kv_rank"], lat.args["rot_dim"], lat.args["window"]) == (40, 32, 8, 9)
    assert att.args["output_gate"] == "elementwise" and att.args["window"] is None and att.args["value_head_dim"] == 32
    assert plan.layers[0].norms["post_mixer"].args["output_scale"] == 0.7 and plan.layers[0].norms["pre_mixer"].args["output_scale"] == 1.0
    assert plan.head.args["tied_to"] == "embed" and plan.head.args["softcap"] == 20.0


@pytest.mark.parametrize("name", list(PEFITAR))
def test_order_of_layer_runs(name):
    raw = PEFITAR[name]()
    assert alice.config_from_dict(raw).layer_runs() == P.layer_runs(raw)


def test_defaults_and_absent_keys():
    raw = PEFITAR["pf-b"]()
    cfg = alice.config_from_dict(raw)
    plan = cfg.plan()
    assert cfg.loop is None and cfg.logit_softcap is None and plan.head.args["softcap"] is None
    assert plan.layers[1].mixer.args["num_kv_heads"] == 3
    raw["layers"][1]["mixer"].pop("kv_heads")
    raw["layers"][1]["mixer"].pop("vdim")
    raw["layers"][1]["mixer"]["rot"].pop("dims")
    again = alice.config_from_dict(raw).plan().layers[1].mixer.args
    assert again["num_kv_heads"] == 3 and again["value_head_dim"] == 20
    free = alice.config_from_dict(PEFITAR["pf-d"]()).plan().layers[2].mixer.args
    assert free["window"] is None
    # one rotation table for each distinct (rotated width, base)
    assert len(alice.config_from_dict(PEFITAR["pf-a"]()).plan().positions) == 2
    assert len(alice.config_from_dict(PEFITAR["pf-d"]()).plan().positions) == 2      # two layers turn 16 dimensions by base 50


@pytest.mark.parametrize("edit,match", [
    (lambda r: r["layers"][0].__setitem__("type", "recurrent"), "no mixer"),
    (lambda r: r["layers"][0]["mlp"].__setitem__("kind", "routed"), "feed-forward"),
    (lambda r: r["loop"].__setitem__("stop", 9), "loop"),
    (lambda r: r["loop"].__setitem__("times", 0), "times"),
    (lambda r: r["layers"][1]["mixer"].__setitem__("kv_heads", 3), "kv_heads"),
    (lambda r: r["layers"][0]["mixer"].__setitem__("rot_dim", 7), "rot_dim"),
    (lambda r: r["layers"][0]["mixer"]["rot"].__setitem__("dims", 4), "rot"),
    (lambda r: r["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "mask"),
    (lambda r: r["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda r: r.pop("vocab"), "vocab"),
])
def test_refusals(edit, match):
    raw = PEFITAR["pf-a"]()
    edit(raw)
    with pytest.raises(ConfigError, match=match):
        alice.config_from_dict(raw)


def test_tensor_names_and_shapes():
    cfg = alice.config_from_dict(PEFITAR["pf-a"]())
    specs = {k: tuple(v.shape) for k, v in CausalLM(cfg.plan(), Precision.of("float32"), "cpu").param_specs().items()}
    want = {"embed": (97, 64), "final.norm": (64,), "l0.norm1": (64,), "l0.norm1b": (64,), "l0.norm2": (64,), "l0.norm2b": (64,),
            "l0.mix.dq": (40, 64), "l0.mix.dq.norm": (40,), "l0.mix.uq": (4 * 24, 40), "l0.mix.dkv": (32 + 8, 64),
            "l0.mix.dkv.norm": (32,), "l0.mix.uk": (4 * 16, 32), "l0.mix.uv": (4 * 24, 32), "l0.mix.o": (64, 4 * 24),
            "l0.mlp.gate": (96, 64), "l0.mlp.up": (96, 64), "l0.mlp.down": (64, 96),
            "l1.mix.q": (64, 64), "l1.mix.k": (32, 64), "l1.mix.v": (64, 64), "l1.mix.g": (128, 64), "l1.mix.o": (64, 128),
            "l2.norm1": (64,), "l2.norm1b": (64,), "l2.mix.o": (64, 96)}
    for k, v in want.items():
        assert specs.get(k) == v, (k, specs.get(k))
    assert not any(k.startswith("l2.mlp") or k.startswith("l2.norm2") for k in specs) and "head" not in specs
    assert len(specs) == 2 + 15 + 12 + 10


def test_the_latent_layers_cache_one_row_a_token_and_every_run_has_its_own():
    cfg = alice.config_from_dict(PEFITAR["pf-a"]())
    lm = CausalLM(cfg.plan(), Precision.of("float32"), "cpu")
    needs = [l.block.mixer.cache_need().kv for l in lm.layers]
    assert (needs[0].num_kv_heads, needs[0].head_dim, needs[0].window, needs[0].value_head_dim) == (1, 32 + 8, 9, 0)
    assert (needs[1].num_kv_heads, needs[1].head_dim, needs[1].window, needs[1].value_head_dim) == (2, 16, None, 32)
    assert len(lm.plan.schedule) == 5                    # five runs, five caches: the loop's passes share weights only


# ------------------------------------------------------------------ the plain implementation's own invariants

def _latent_weights(W, H, d, r, dv, A, R, seed):
    return {"dq": rnd(A, W, seed=seed), "dq.norm": 1 + 0.1 * rnd(A, seed=seed + 1), "uq": rnd(H * (d + r), A, seed=seed + 2, scale=0.5),
            "dkv": rnd(R + r, W, seed=seed + 3), "dkv.norm": 1 + 0.1 * rnd(R, seed=seed + 4), "uk": rnd(H * d, R, seed=seed + 5, scale=0.5),
            "uv": rnd(H * dv, R, seed=seed + 6, scale=0.3), "o": rnd(W, H * dv, seed=seed + 7, scale=0.2)}


def test_latent_attention_with_the_maps_on_the_querys_side_equals_keys_and_values_a_head():
    """score_h(i, j) = (Uk_h^T q_h)(i) . c(j) + q_rot . kr and out_h = Uv_h sum_j w c(j): what the cache of latent rows
    rests on."""
    T, W, H, d, r, dv, A, R, eps, scale, size = 23, 20, 3, 6, 4, 5, 9, 7, 1e-6, 0.4, 6
    w = _latent_weights(W, H, d, r, dv, A, R, 1)
    m = {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "q_rank": A, "kv_rank": R, "scale": scale, "mask": {"size": size},
         "rot": {"base": 30.0, "dims": r}}
    h, pos = rnd(T, W, seed=2), torch.arange(T)
    ref = P.latent_attention(h, w, m, pos, eps)
    cq = P.rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).reshape(T, H, d + r)
    dkv = h @ w["dkv"].T
    c = P.rms_norm(dkv[:, :R], w["dkv.norm"], eps)
    kr = P.rotate_pairs(dkv[:, None, R:], pos, 30.0, r)[:, 0]
    qr = P.rotate_pairs(q[..., d:], pos, 30.0, r)
    uk, uv = w["uk"].reshape(H, d, R), w["uv"].reshape(H, dv, R)
    out = torch.zeros(T, H, dv, dtype=torch.float64)
    for hh in range(H):
        qa = q[:, hh, :d] @ uk[hh]                                            # [T, R]
        s = (qa @ c.T + qr[:, hh] @ kr.T) * scale
        s = s.masked_fill(~P.causal_mask(T, size), -math.inf)
        out[:, hh] = (torch.softmax(s, dim=1) @ c) @ uv[hh].T
    assert (out.reshape(T, H * dv) @ w["o"].T - ref).abs().max() < 1e-12


def test_window_edges_and_the_first_tokens():
    m = P.causal_mask(12, 4)
    assert m[7].nonzero().flatten().tolist() == [4, 5, 6, 7] and m[2].nonzero().flatten().tolist() == [0, 1, 2]
    assert m[0].nonzero().flatten().tolist() == [0] and P.causal_mask(5, 1).int().tolist() == torch.eye(5).int().tolist()
    assert P.causal_mask(6).int().tolist() == torch.tril(torch.ones(6, 6)).int().tolist()
    # a key that every query scores far above the rest: seen by the window's last query, lost by the next
    T, H, d, size = 20, 2, 4, 5
    q, k, v = rnd(T, H, d, seed=1), rnd(T, 1, d, seed=2), rnd(T, 1, 3, seed=3)
    q[:, :, 0], k[:, :, 0] = 3.0, 0.0
    k[6, :, 0] = 8.0
    out = P.softmax_attention(q, k, v, P.causal_mask(T, size), 1.0)
    assert (out[6 + size - 1] - v[6, 0]).abs().max() < 1e-3 and (out[6 + size] - v[6, 0]).abs().max() > 0.1


def test_rotation_turns_neighbouring_pairs_and_scores_depend_on_the_distance():
    x = rnd(1, 1, 8, seed=1)
    y = P.rotate_pairs(x.expand(5, 1, 8), torch.arange(5), 100.0, 4)
    assert (y[..., 4:] - x[..., 4:]).abs().max() == 0                         # the rest passes
    a1 = 3 * 100.0 ** (-2.0 / 4)
    assert abs(float(y[3, 0, 2]) - float(x[0, 0, 2] * math.cos(a1) - x[0, 0, 3] * math.sin(a1))) < 1e-12
    assert abs(float(y[3, 0, 3]) - float(x[0, 0, 3] * math.cos(a1) + x[0, 0, 2] * math.sin(a1))) < 1e-12
    q, k = rnd(1, 1, 6, seed=2), rnd(1, 1, 6, seed=3)
    dots = [float((P.rotate_pairs(q, torch.tensor([p + 4]), 50.0, 6) * P.rotate_pairs(k, torch.tensor([p]), 50.0, 6)).sum()) for p in (0, 9, 300)]
    assert max(dots) - min(dots) < 1e-9
    assert (P.rotate_pairs(x, torch.tensor([7]), 10.0, 0) - x).abs().max() == 0


def test_gated_attention_reads_the_gate_from_the_mixers_input_and_groups_heads():
    T, W, H, G, d, dv = 9, 10, 4, 2, 4, 3
    w = {"q": rnd(H * d, W, seed=1), "k": rnd(G * d, W, seed=2), "v": rnd(G * dv, W, seed=3), "g": rnd(H * dv, W, seed=4),
         "o": torch.eye(H * dv, dtype=torch.float64)}
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": 0.5, "rot": {"base": 10.0, "dims": 2}}
    h = rnd(T, W, seed=5)
    out = P.gated_attention(h, w, m, torch.arange(T))
    # the first token sees itself alone: its output is its own value, head by head of its group, times the gate
    v0 = (h[0] @ w["v"].T).reshape(G, dv)
    want = torch.stack([v0[hh // (H // G)] for hh in range(H)]).reshape(-1) * torch.sigmoid(h[0] @ w["g"].T)
    assert (out[0] - want).abs().max() < 1e-12
    closed = dict(w, g=torch.zeros_like(w["g"]))
    # a gate matrix of zeros halves every output element: what is left is the plain grouped attention
    half = P.gated_attention(h, closed, m, torch.arange(T))
    assert (half * 2 - P.softmax_attention(
        P.rotate_pairs((h @ w["q"].T).reshape(T, H, d), torch.arange(T), 10.0, 2),
        P.rotate_pairs((h @ w["k"].T).reshape(T, G, d), torch.arange(T), 10.0, 2),
        (h @ w["v"].T).reshape(T, G, dv), P.causal_mask(T), 0.5).reshape(T, -1)).abs().max() < 1e-12


def test_feed_forward_norm_and_cap():
    h, g, u, dn = rnd(3, 6, seed=1), rnd(8, 6, seed=2), rnd(8, 6, seed=3), rnd(6, 8, seed=4)
    z = h @ g.T
    assert (P.silu_gated_ff(h, g, u, dn) - ((z * torch.sigmoid(z)) * (h @ u.T)) @ dn.T).abs().max() < 1e-12
    x = rnd(2, 16, seed=5, scale=1e-4)
    n = P.rms_norm(x, torch.ones(16, dtype=torch.float64), 1e-6)
    assert float((n * n).mean(-1).max()) < 1.0                               # eps is inside the root
    assert (P.unit_rms(rnd(2, 16, seed=6), 0.0).pow(2).mean(-1) - 1).abs().max() < 1e-12


@pytest.mark.parametrize("name", ["pf-a", "pf-d"])
def test_loop_passes_share_weights_and_the_stream_factor_scales_every_branch(name):
    raw = PEFITAR[name]()
    _, tensors = pefitar_tensors(raw, 3)
    plain = PlainPefitar(raw, tensors)
    toks = random_tokens(raw["vocab"], 17, 2)
    lg, runs = plain.forward(toks, return_layers=True)
    assert runs.shape[0] == len(P.layer_runs(raw))
    cap = raw["logit_softcap"]
    assert float(lg.abs().max()) <= cap
    # unrolled by hand: the same layers written out with copied weights give the same logits
    a, b, n = raw["loop"]["start"], raw["loop"]["stop"], raw["loop"]["times"]
    order = P.layer_runs(raw)
    flat = dict(raw, layers=[raw["layers"][i] for i in order])
    flat.pop("loop")
    t2 = {k: v for k, v in plain.t.items() if not k.startswith("l")}
    for new, old in enumerate(order):
        for k, v in plain.t.items():
            if k.startswith(f"l{old}."):
                t2[f"l{new}." + k[len(f"l{old}."):]] = v
    assert (P.forward(flat, t2, toks) - lg).abs().max() < 1e-12
    # a prefix's logits do not depend on what follows
    assert (plain.forward(toks[:9]) - lg[:9]).abs().max() < 1e-9
