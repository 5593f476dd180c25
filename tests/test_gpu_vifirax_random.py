"""Seeded random Vifirax configurations and schedules against the plain implementation: every size and option drawn
(layer order, head counts and sizes, a rotated part with or without stretched frequencies, groups, taps, narrow
middles, experts and how many a token takes, layers without a feed-forward, layers that read another's keys), a
prompt whole, the same prompt in random pieces, and two unequal requests together that then go on by single tokens.
Most cases run in 32-bit, where every logit is held to the plain model's; every fourth runs in bfloat16 with dense
feed-forwards in the routed ones' places (a token whose router logits nearly tie takes another expert under bfloat16's
rounding, and layers with state carry that on; the fixed configurations cover routed layers in bfloat16).  A norm
part holds at least 8 numbers (a part of one number is the sign of its input, which no rounding survives near zero)."""
import random

import pytest
import torch

from helpers import model_from_tensors, random_tokens, vifirax_tensors
from plain.vifirax_plain import PlainVifirax
from test_gpu_vifirax import assert_close

pytestmark = pytest.mark.gpu


def _divisors(n):
    return [d for d in range(1, n + 1) if n % d == 0]


def draw_config(rng: random.Random, routed: bool = True) -> dict:
    width = rng.choice([40, 48, 64, 96, 136, 200, 256])
    layers, owners = [], []
    for i in range(rng.randint(2, 7)):
        kind = rng.choice(["attention", "mamba2", "channel_delta"])
        if kind == "attention":
            if owners and rng.random() < 0.4:
                j = rng.choice(owners)
                m = dict(layers[j]["mixer"], kv_from=j)
            else:
                heads = rng.choice([1, 2, 3, 4, 6, 8])
                dim = rng.choice([8, 16, 24, 40, 64, 96, 128])
                m = {"heads": heads, "kv_heads": rng.choice(_divisors(heads)), "dim": dim, "vdim": rng.choice([8, 16, 24, 40, 64, 96, 128]),
                     "scale": rng.uniform(0.3, 1.0)}
                if rng.random() < 0.85:
                    rot = {"base": rng.choice([50.0, 1e4, 2.5e5]), "dims": 2 * rng.randint(1, dim // 2)}
                    if rng.random() < 0.6:
                        rot["scaling"] = {"factor": rng.choice([2.0, 8.0, 32.0]), "original": rng.choice([8, 64, 2048]),
                                          "fast": rng.choice([4.0, 32.0]), "slow": rng.choice([0.5, 1.0, 2.0])}
                    m["rot"] = rot
                owners.append(i)
        elif kind == "mamba2":
            heads, vdim = rng.choice([1, 2, 4, 6, 8]), rng.choice([8, 16, 24, 32, 64])
            m = {"heads": heads, "vdim": vdim, "state": rng.choice([4, 8, 16, 24, 64, 128, 160]), "groups": rng.choice(_divisors(heads)),
                 "norm_groups": rng.choice([g for g in _divisors(heads * vdim) if g <= 16 and heads * vdim // g >= 8]), "conv": rng.randint(1, 5)}
        else:
            heads = rng.choice([1, 2, 3, 4, 6])
            m = {"heads": heads, "kv_heads": rng.choice(_divisors(heads)), "dim": rng.choice([8, 16, 32, 64, 96, 128, 192]),
                 "vdim": rng.choice([8, 16, 24, 40, 64, 128]), "conv": rng.randint(1, 5), "decay_rank": rng.randint(2, 32),
                 "gate_rank": rng.randint(2, 32)}
        r = rng.random()
        if r < 0.2:
            mlp = None
        elif r < 0.6 or not routed:
            mlp = {"kind": "dense", "ff": rng.choice([17, 32, 96, 160])}
        else:
            experts = rng.randint(1, 16)
            mlp = {"kind": "moe", "expert": {"ff": rng.choice([8, 16, 24, 64])}, "router": {"experts": experts, "top": rng.randint(1, min(4, experts))}}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    raw = {"architecture": "Vifirax", "vocab": rng.randint(50, 700), "width": width, "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        raw["logit_scale"] = rng.choice([0.25, 0.37, 1.0, 3.0])
    return raw


@pytest.mark.parametrize("seed", range(14))
def test_random_configuration(seed):
    rng = random.Random(1000 + seed)
    dtype = "bfloat16" if seed % 4 == 3 else "float32"
    raw = draw_config(rng, routed=dtype == "float32")
    cfg, tensors = vifirax_tensors(raw, seed)
    plain = PlainVifirax(raw, {k: v.double() for k, v in tensors.items()})
    model = model_from_tensors(cfg, {k: v.to("cuda") for k, v in tensors.items()}, dtype)
    V = raw["vocab"]
    eng = model.engine(max_tokens=1024, max_seqs=3)
    n = rng.randint(1, 200)
    toks = random_tokens(V, n, seed)
    ref = plain.forward(toks)
    s = eng.open(1)
    assert_close(eng.step(s, [toks], "all"), ref, dtype, ("whole", raw))
    eng.close(s)
    s, got, at = eng.open(1), [], 0
    while at < n:
        c = min(n - at, rng.choice([1, 2, 3, 17, 64, 70]))
        got.append(eng.step(s, [toks[at:at + c]], "all"))
        at += c
    eng.close(s)
    assert_close(torch.cat(got), ref, dtype, ("pieces", raw))
    lens, dec = [rng.randint(1, 90), rng.randint(1, 90)], [rng.randint(1, 12), rng.randint(1, 12)]
    seqs = [random_tokens(V, L + d, 50 + seed + i) for i, (L, d) in enumerate(zip(lens, dec))]
    refs = [plain.forward(t) for t in seqs]
    slots = eng.open(2)
    out = eng.step(slots, [t[:L] for t, L in zip(seqs, lens)], "last")
    rows = [[out[0]], [out[1]]]
    live = [0, 1]
    for step in range(max(dec)):
        live = [b for b in live if step < dec[b]]
        out = eng.step([slots[b] for b in live], [[seqs[b][lens[b] + step]] for b in live], "last")
        for r, b in enumerate(live):
            rows[b].append(out[r])
        for b in list(live):
            if step + 1 == dec[b]:
                eng.close([slots[b]])
    for b in range(2):
        assert_close(torch.stack(rows[b]), refs[b][lens[b] - 1:], dtype, ("together", b, raw))
    eng.cache.check_consistent()
