"""Vifirax on the GPU against the plain implementation, in 32-bit and in bfloat16: every mechanism alone (the short
convolution and its carried inputs, both matrix recurrences, the norm and gate behind them, the router, the routed
feed-forward, the projection norm with the rotation in halves and stretched frequencies, the softmax with one more
in its denominator), then the model through the engine: whole prompts, the stream after every layer, a prefix and
then single tokens, prompts in pieces down to two tokens, unequal batches against each request alone on slots and
pages that are used again, long decoding from the first token, captured against eager steps, and greedy generation,
the command line and trace replay through the package's own entry points."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.hip import ops
from alice_llm_amd.parts import FEED_FORWARDS, POSITIONS, Precision
from helpers import VIFIRAX, max_err, random_tokens, vifirax_folder, vifirax_pair
from plain import vifirax_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]
CASES = [(n, d) for n in VIFIRAX for d in DTYPES]
_PAIRS = {}


def pair(name, dtype):
    if (name, dtype) not in _PAIRS:
        _PAIRS[(name, dtype)] = vifirax_pair(name, dtype, seed=len(name) + 5)
    return _PAIRS[(name, dtype)]


def row_errors(got, ref):
    """Per row of logits: the root mean square of the difference (means taken off) over that of the row itself."""
    d = got.double().cpu() - ref.double().cpu()
    d = d - d.mean(-1, keepdim=True)
    r = ref.double().cpu() - ref.double().cpu().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / r.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def assert_close(got, ref, dtype, what=""):
    """The test models' weights make softmaxes sharp, gates open and close, routers decide and decays range from fast to
    almost none, so a rounding ahead of such a place is amplified.  32-bit: every logit within 1e-3 of the plain
    model's (relative to the largest logit) and the median row within 2e-5.  bfloat16: a row's error is measured as a
    whole (root mean square against the row's own): the rows' mean within 0.06 and nine rows in ten within 0.1 (of
    twenty rows and more; of fewer, every row but one within 0.3); a token whose router
    logits nearly tie may take another expert than the plain model's: it is among the tenth, or the one.  A wrong key, state
    or position moves most rows by 0.3 and more."""
    assert got.shape == ref.shape, what
    if dtype == "float32":
        scale = max(1.0, float(ref.abs().max()))
        e = (got.double().cpu() - ref.double().cpu()).abs().max(-1).values
        assert float(e.max()) < 1e-3 * scale and float(e.median()) < 2e-5 * scale, (what, float(e.max()), float(e.median()))
    else:
        e = row_errors(got, ref).sort().values
        many = e.numel() >= 20
        rest = e if many or e.numel() == 1 else e[:-1]
        assert (float(rest.mean()) < 0.06 or not many) and float(e.quantile(0.9) if many else rest.max()) < (0.1 if many else 0.3) and float(e.max()) < 1.0, \
            (what, float(e.max()), float(e.mean()))


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


class _Ctx:
    """What the recurrent kernels read of a step."""

    def __init__(self, lens, slots):
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        self.cu_seqlens = torch.tensor(cu, dtype=torch.int32, device=DEV)
        self.slots = torch.tensor(slots, dtype=torch.int32, device=DEV)
        self.seq_of_token = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(torch.int32).to(DEV)
        self.n_seqs = len(lens)


# Steps of three sequences on slots 2, 0 and 5 of six: unequal pieces down to one and two tokens, a sequence that sits a
# step out, and one that ends, after which its slot is cleared and used by a new sequence.
_STEPS = [([7, 1, 3], [0, 1, 2]), ([1, 1, 1], [0, 1, 2]), ([2, 40], [0, 2]), ([1, 1, 1], [0, 1, 2]), ([66, 5], [1, 0]),
          ([9, 2, 1], [3, 0, 2]), ([1, 1], [3, 0])]
_SLOTS = [2, 0, 5, 0]          # sequence 3 takes slot 0 after sequence 1, which ends with the fifth step


def _walk(total_of):
    """The steps above as (lens, sequence ids, slot ids, [(start, stop) of each sequence's piece])."""
    at = {}
    for lens, ids in _STEPS:
        yield lens, ids, [_SLOTS[i] for i in ids], [(at.get(i, 0), at.get(i, 0) + n) for i, n in zip(ids, lens)]
        for i, n in zip(ids, lens):
            at[i] = at.get(i, 0) + n


_TOTAL = {}
for _lens, _ids in _STEPS:
    for _i, _n in zip(_ids, _lens):
        _TOTAL[_i] = _TOTAL.get(_i, 0) + _n


# ------------------------------------------------------------------ mechanisms alone

@pytest.mark.parametrize("C,taps,col0,bias", [(37, 4, 3, True), (300, 2, 0, False), (64, 1, 5, True), (20, 5, 0, False), (9, 16, 1, True)])
def test_short_convolution_over_pieces_with_carried_inputs(C, taps, col0, bias):
    """The inputs just ahead of a piece come from the state row of the sequence's slot: pieces shorter than the taps,
    single tokens, a slot that is cleared and used again."""
    row_w = col0 + C + 2
    xs = {i: rnd(n, row_w, seed=10 + i) for i, n in _TOTAL.items()}
    w, b = rnd(C, taps, seed=1, scale=0.6), (rnd(C, seed=2) if bias else None)
    refs = {i: P.silu(P.causal_conv(x[:, col0:col0 + C].double(), w.double(), None if b is None else b.double())) for i, x in xs.items()}
    state = torch.full((6, C, taps - 1), 3.0, device=DEV) if taps > 1 else None
    if state is not None:
        state[[2, 0, 5]] = 0.0
    wd, bd = w.to(DEV), None if b is None else b.to(DEV)
    for step, (lens, ids, slots, spans) in enumerate(_walk(_TOTAL)):
        if step == 5 and state is not None:
            state[0] = 0.0                                      # a new sequence takes the slot
        rows = torch.cat([xs[i][a:e] for i, (a, e) in zip(ids, spans)]).to(DEV)
        out = torch.empty(rows.shape[0], C, device=DEV)
        ops.short_conv(rows, col0, wd, bd, state, out, _Ctx(lens, slots))
        at = 0
        for i, (a, e) in zip(ids, spans):
            assert max_err(out[at:at + e - a], refs[i][a:e]) < 1e-5, (step, i)
            at += e - a
    if state is not None:
        assert float((state[[1, 3, 4]] - 3.0).abs().max()) == 0.0          # rows of other slots are untouched
        tail = xs[2][_TOTAL[2] - (taps - 1):, col0:col0 + C] if _TOTAL[2] >= taps - 1 else None
        if tail is not None:
            assert max_err(state[5], tail.T) == 0.0


@pytest.mark.parametrize("delta", [False, True])
@pytest.mark.parametrize("cols", [0, 4, 8, 16])
@pytest.mark.parametrize("H,G,d,dv", [(4, 2, 8, 16), (3, 3, 12, 20), (2, 1, 64, 128), (1, 1, 136, 24), (2, 2, 200, 7), (6, 3, 1, 1)])
def test_matrix_recurrence_over_pieces_and_slots(delta, cols, H, G, d, dv):
    """Both recurrences against the plain scan, the state carried from step to step in the slots' rows; with the value
    columns a wave left to the launcher and fixed at each of its choices."""
    data = {}
    for i, n in _TOTAL.items():
        q, k = rnd(n, G * d, seed=20 + i), rnd(n, G * d, seed=30 + i)
        if delta:
            q = P.unit_vectors(q.view(n, G, d)).reshape(n, G * d)
            k = P.unit_vectors(k.view(n, G, d)).reshape(n, G * d)
        v = rnd(n, H * dv, seed=40 + i)
        decay = torch.sigmoid(rnd(n, H * d if delta else H, seed=50 + i, scale=2.0) + 2.0)
        b = torch.sigmoid(rnd(n, H, seed=60 + i)) * (1.0 if delta else 2.0)
        data[i] = (q.float(), k.float(), v, decay.float(), b.float())
    skip = None if delta else rnd(H, seed=3)
    per = H // G
    refs = {}
    for i, (q, k, v, decay, b) in data.items():
        n = q.shape[0]
        qh = q.double().view(n, G, d).repeat_interleave(per, dim=1)
        kh = k.double().view(n, G, d).repeat_interleave(per, dim=1)
        if delta:
            refs[i] = P.delta_rule_scan(qh, kh, v.double().view(n, H, dv), decay.double().view(n, H, d), b.double())
        else:
            # the plain scan takes rates and step sizes: exp(-exp(a) dt) = decay with a = 0 and dt = -ln(decay); the write's
            # factor is given apart by scaling the values
            dt = -torch.log(decay.double())
            u = v.double().view(n, H, dv) * (b.double() / dt)[:, :, None]
            y, S = P.state_space_scan(u, kh, qh, dt, torch.zeros(H, dtype=torch.float64), torch.zeros(H, dtype=torch.float64))
            refs[i] = (y + skip.double()[None, :, None] * v.double().view(n, H, dv), S)
    S = torch.full((6, H, d, dv), 3.0, device=DEV)
    S[[2, 0, 5]] = 0.0
    for step, (lens, ids, slots, spans) in enumerate(_walk(_TOTAL)):
        if step == 5:
            S[0] = 0.0
        cat = lambda j: torch.cat([data[i][j][a:e] for i, (a, e) in zip(ids, spans)]).to(DEV).contiguous()
        q, k, v, decay, b = (cat(j) for j in range(5))
        out = torch.empty(q.shape[0], H * dv, device=DEV)
        ops.matrix_recurrence(q, 0, k, 0, v, 0, decay, b, None if skip is None else skip.to(DEV), out, _Ctx(lens, slots), S,
                              heads=H, qk_heads=G, head_dim=d, value_head_dim=dv, delta=delta, decay_per_channel=delta,
                              columns_per_wave=cols)
        at = 0
        for i, (a, e) in zip(ids, spans):
            ref = refs[i][0][a:e].reshape(e - a, H * dv)
            assert max_err(out[at:at + e - a], ref) < 2e-4 * max(1.0, float(ref.abs().max())), (step, i)
            at += e - a
    for i, slot in ((0, 2), (2, 5), (3, 0)):
        assert max_err(S[slot], refs[i][1]) < 2e-4 * max(1.0, float(refs[i][1].abs().max())), i
    assert float((S[[1, 3, 4]] - 3.0).abs().max()) == 0.0


def test_a_far_token_is_kept_by_a_decay_of_one_and_lost_by_a_fast_one():
    """Delta rule, single tokens: the first token writes a value under two keys; 700 steps later, with write strength 0
    in between, the channel that does not decay still holds it and the one that decays by half a step has lost it."""
    H, d, dv, T = 1, 4, 8, 700
    S = torch.zeros(2, H, d, dv, device=DEV)
    val = torch.arange(1, dv + 1).float()
    outs = []
    for t in range(T):
        q, k = torch.zeros(1, d), torch.zeros(1, d)
        if t == 0:
            k[0, 0] = k[0, 1] = 1.0
        q[0, 0 if t % 2 else 1] = 1.0
        decay = torch.tensor([[1.0, 0.5, 1.0, 1.0]])
        b = torch.tensor([[1.0 if t == 0 else 0.0]])
        out = torch.empty(1, dv, device=DEV)
        ops.matrix_recurrence(q.to(DEV), 0, k.to(DEV), 0, val[None].to(DEV), 0, decay.to(DEV), b.to(DEV), None, out, _Ctx([1], [1]), S,
                              heads=H, qk_heads=1, head_dim=d, value_head_dim=dv, delta=True, decay_per_channel=True)
        outs.append(out[0].cpu())
    assert max_err(outs[-1], val) < 1e-6 and float(outs[-2].abs().max()) < 1e-30          # odd steps read channel 0, even ones channel 1
    assert max_err(outs[1], val) < 1e-6 and max_err(outs[2], val * 0.25) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,width,parts", [(5, 64, 4), (33, 60, 1), (7, 48, 3), (2, 1024, 2), (9, 24, 24)])
def test_norm_and_gate_behind_a_read_out(dtype, T, width, parts):
    act = Precision.of(dtype).act
    x, gate, eps = rnd(T, width, seed=1, scale=3.0), rnd(T, width + 5, seed=2, scale=2.0), 1e-5
    n = width // parts
    for shared, gate_act in ((False, "silu"), (True, "sigmoid"), (False, None)):
        w = rnd(n if shared else width, seed=3).abs() + 0.5
        y = x.double()
        g = gate.double()[:, 2:2 + width]
        if gate_act == "silu":
            y = y * P.silu(g)
        y = P.unit_rms(y.view(T, parts, n), eps) * (w.double() if shared else w.double().view(parts, n))
        y = y.reshape(T, width)
        if gate_act == "sigmoid":
            y = y * torch.sigmoid(g)
        out = torch.empty(T, width, dtype=act, device=DEV)
        ops.norm_gate(x.to(DEV), w.to(DEV), out, parts=parts, eps=eps, weight_shared=shared,
                      gate=None if gate_act is None else gate.to(DEV), gate_col=2, gate_act=gate_act)
        assert max_err(out, y) < (1e-5 if dtype == "float32" else 2e-2) * max(1.0, float(y.abs().max())), (shared, gate_act)


@pytest.mark.parametrize("T,E,top", [(9, 6, 2), (70, 16, 3), (3, 5, 5), (4, 3, 1), (2, 200, 8), (1, 1, 1)])
def test_router_takes_the_largest_and_weights_them_by_their_own_softmax(T, E, top):
    z, b = rnd(T, E, seed=1, scale=2.0), rnd(E, seed=2)
    if E > 2:
        z[0, 1] = z[0, 2] = 50.0                               # equal logits: the lower index first
        b[1] = b[2] = 0.0
    w = torch.empty(T, E, device=DEV)
    ops.route_topk(z.to(DEV), b.to(DEV), w, top)
    val, idx = torch.topk((z + b).double(), top, dim=-1)
    ref = torch.zeros(T, E, dtype=torch.float64).scatter_(1, idx, torch.softmax(val, dim=-1))
    if E > 2 and top == 1:
        ref[0] = 0.0
        ref[0, 1] = 1.0
    assert max_err(w, ref) < 1e-6
    assert int((w > 0).sum(dim=1).max()) <= top and max_err(w.sum(dim=1), torch.ones(T)) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,W,F,E,top", [(5, 64, 24, 6, 2), (70, 72, 18, 5, 5), (130, 128, 64, 8, 2), (33, 48, 7, 3, 1), (64, 40, 32, 4, 1),
                                         (300, 256, 96, 16, 3), (1000, 72, 64, 3, 3), (257, 136, 160, 33, 4)])
def test_routed_feed_forward(dtype, T, W, F, E, top):
    p = Precision.of(dtype)
    ff = FEED_FORWARDS.get("expert_mlp")(p, hidden_size=W, intermediate_size=F, experts=E, top=top, activation="silu")
    ws = {}
    for i, (n, s) in enumerate(ff.param_specs().items()):
        scale = 2.5 / W ** 0.5 if n == "router" else (0.5 if n == "router.b" else 0.15)
        ws[n] = rnd(*s.shape, seed=i, scale=scale).to(torch.bfloat16).to(DEV)
    assert set(ws) == {f"e{e}.{m}" for e in range(E) for m in ("gate", "up", "down")} | {"router", "router.b"}
    for n, t in ws.items():
        ff.assign(n, t)
    ff.finalize()
    x = rnd(T, W, seed=99).to(torch.bfloat16)                  # the router sees the same numbers on both paths
    ref = P.routed_ff(x.double(), {k: v.double().cpu() for k, v in ws.items()}, {"router": {"experts": E, "top": top}})
    from alice_llm_amd.parts import experts
    kept = experts.GROUPED_FROM_TOKENS
    try:
        for experts.GROUPED_FROM_TOKENS in (1, 10 ** 9, kept):  # the grouped products wherever they apply, never, and the part's own choice
            out = ff.forward(x.to(p.act).to(DEV), None)
            out = out.sum(0) if out.dim() == 3 else out
            assert max_err(out, ref) < (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max())), experts.GROUPED_FROM_TOKENS
    finally:
        experts.GROUPED_FROM_TOKENS = kept
    with pytest.raises(ValueError, match="top"):
        FEED_FORWARDS.get("expert_mlp")(p, hidden_size=W, intermediate_size=F, experts=E, top=E + 1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,R,scaling", [(4, 2, 16, 32, 8, (4.0, 16, 8.0, 1.0)), (3, 3, 20, 28, 20, None), (4, 1, 64, 64, 32, (16.0, 64, 4.0, 0.5)),
                                                (2, 2, 24, 8, 0, None), (6, 2, 16, 24, 16, (2.0, 32, 2.0, 1.0))])
def test_projection_norm_rotation_in_halves_and_cache_write(dtype, H, G, d, dv, R, scaling):
    """q (all heads together) and k (likewise) normed over the whole projection after the bias, then the first R
    dimensions of every head turned in halves with stretched frequencies; k and v land on scattered pages."""
    act = Precision.of(dtype).act
    T, page, eps, base = 70, 64, 1e-5, 300.0
    sc = None if scaling is None else dict(zip(("factor", "original", "fast", "slow"), scaling))
    width = H * d + G * d + G * dv + 3
    rows, bias = rnd(T, width, seed=1), rnd(width, seed=2, scale=0.5)
    wn = rnd(H * d + G * d, seed=3).abs() + 0.3
    pos = torch.arange(T)
    x = rows.double() + bias.double()
    q = P.unit_rms(x[:, :H * d], eps) * wn[:H * d].double()
    k = P.unit_rms(x[:, H * d:H * d + G * d], eps) * wn[H * d:].double()
    v = x[:, H * d + G * d:H * d + G * d + G * dv].view(T, G, dv)
    q, k = q.view(T, H, d), k.view(T, G, d)
    cos = sin = None
    if R:
        f, m = P.stretched_frequencies(R, base, sc)
        q, k = P.rotate_halves(q, pos, f, m), P.rotate_halves(k, pos, f, m)
        part = POSITIONS.get("rope_pairs")(Precision.of(dtype), DEV, dim=d, theta=base, max_positions=128, rotary_dim=R,
                                           interleaved=False, scaling=sc)
        cos, sin = part.cos, part.sin
        ang = pos.double()[:, None] * f[None, :]
        assert max_err(cos[:T], torch.cos(ang) * m) < 1e-6 and max_err(sin[:T], torch.sin(ang) * m) < 1e-6
    kp = torch.zeros(5, G, page, d, dtype=act, device=DEV)
    vp = torch.zeros(5, G, page, dv, dtype=act, device=DEV)
    bt = torch.tensor([[3, 1]], dtype=torch.int32, device=DEV)
    q_out = torch.empty(T, H * d, dtype=act, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    ops.qkv_prepare(rows.to(DEV), bias.to(DEV), q_out, kp, vp, pos.to(torch.int32).to(DEV), seq, bt, num_heads=H, num_kv_heads=G,
                    head_dim=d, value_head_dim=dv, max_position=T - 1, cos=cos, sin=sin, rotary_dim=R, interleaved=False,
                    norm_weight=wn.to(DEV), norm_eps=eps)
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert max_err(q_out, q.reshape(T, H * d)) < tol * float(q.abs().max())
    got_k = torch.cat([kp[3].permute(1, 0, 2), kp[1].permute(1, 0, 2)])[:T]
    got_v = torch.cat([vp[3].permute(1, 0, 2), vp[1].permute(1, 0, 2)])[:T]
    assert max_err(got_k, k) < tol * float(k.abs().max()) and max_err(got_v, v) < tol * float(v.abs().max())
    # queries alone (a mixer that reads another's keys): the same q from rows that hold no k and v
    q2 = torch.empty_like(q_out)
    ops.qkv_prepare(rows[:, :H * d + 1].contiguous().to(DEV), bias.to(DEV), q2, None, None, pos.to(torch.int32).to(DEV), None, None,
                    num_heads=H, num_kv_heads=G, head_dim=d, value_head_dim=dv, max_position=T - 1, cos=cos, sin=sin, rotary_dim=R,
                    interleaved=False, norm_weight=wn[:H * d].contiguous().to(DEV), norm_eps=eps)
    assert max_err(q2, q_out) == 0.0


def _paged(k, v, page, scatter_seed):
    """Keys [T, G, d] and values [T, G, dv] of one sequence put into scattered pages; returns pools and the table."""
    T, G, d = k.shape
    n = -(-T // page)
    order = torch.randperm(n + 3, generator=torch.Generator().manual_seed(scatter_seed))[:n] + 1
    kp = torch.full((n + 5, G, page, d), 7.0, dtype=k.dtype)
    vp = torch.full((n + 5, G, page, v.shape[-1]), -7.0, dtype=v.dtype)
    for t in range(T):
        kp[order[t // page], :, t % page] = k[t]
        vp[order[t // page], :, t % page] = v[t]
    return kp.to(DEV), vp.to(DEV), order.to(torch.int32)[None].to(DEV)


class _Step:
    def __init__(self, pieces, T):
        cu = [0]
        for a, b in pieces:
            cu.append(cu[-1] + b - a)
        self.positions = torch.cat([torch.arange(a, b) for a, b in pieces]).to(torch.int32).to(DEV)
        self.cu_seqlens = torch.tensor(cu, dtype=torch.int32, device=DEV)
        self.n_seqs, self.max_position, self.rows = len(pieces), T - 1, torch.cat([torch.arange(a, b) for a, b in pieces])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,T", [(4, 2, 24, 40, 300), (6, 1, 96, 96, 700), (3, 3, 20, 28, 130), (2, 1, 64, 128, 65)])
def test_far_key_and_the_one_in_the_denominator(dtype, H, G, d, dv, T):
    """One key near the start that late queries score far above the hundreds between; queries that score every key far
    below zero, whose output the one in the denominator takes almost all of; a query whose scores are all near zero
    (weights 1 / (keys + 1)); one gate number a head.  Prompts whole and in pieces, and single tokens, through every
    attention kernel that serves them."""
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    q, k, v = rnd(T, H, d, seed=1, scale=0.3), rnd(T, G, d, seed=2, scale=0.3), rnd(T, G, dv, seed=3)
    gate = rnd(T, H + 3, seed=4, scale=2.0)
    far = 2
    k[:, :, 0] = 0.0
    k[far, :, 0] = 8.0
    v[far] += 6.0
    q[:, :, 0] = 0.0
    q[T - 9:, :, 0] = 4.0                                       # the last queries look for the far key
    q[T // 2] = 0.0                                            # scores of exactly zero
    q[T // 2 + 1, :, 0] = -60.0                                 # and one that looks away from everything it could like
    k[: T // 2 + 2, :, 0] += 1.0
    k[far, :, 0] = 8.0
    q, k, v = (x.to(dt) for x in (q, k, v))
    mask = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    ref = torch.empty(T, H, dv, dtype=torch.float64)
    for h in range(H):
        g = h // (H // G)
        w = P.one_more_softmax((q[:, h].double() @ k[:, g].double().T) * 0.5, mask)
        ref[:, h] = (w @ v[:, g].double()) * torch.sigmoid(gate.double()[:, h:h + 1])
    assert float(ref[T // 2 + 1].abs().max()) < 1e-6 * float(ref.abs().max())       # the plain model's own check of the case
    kp, vp, bt = _paged(k, v, 64, 5)
    zero = torch.zeros(H, device=DEV)
    qd, gd = q.reshape(T, H * d).to(DEV), gate.to(DEV)
    common = dict(num_heads=H, scale=0.5, sink=zero)
    tol = (2e-5 if dtype == "float32" else 2e-2) * float(ref.abs().max())
    pos, seq = torch.arange(T, dtype=torch.int32, device=DEV), torch.zeros(T, dtype=torch.int32, device=DEV)
    out = torch.empty(T, H * dv, dtype=dt, device=DEV)
    ops.attention_masked(qd, kp, vp, out, pos, seq, bt, max_position=T - 1, full_precision=dtype == "float32", gate=gd, **common)
    assert max_err(out, ref.reshape(T, H * dv)) < tol
    if ops.attention_tiled_supported(dt, d, dv):
        cuts = sorted(c for c in {0, 2, 63, 66, T - 9, T - 7, T} if c <= T)
        for pieces in ([(0, T)], list(zip(cuts[:-1], cuts[1:]))):
            st = _Step(pieces, T)
            o2 = torch.empty(len(st.rows), H * dv, dtype=dt, device=DEV)
            ops.attention_tiled(qd[st.rows], kp, vp, o2, st, bt.expand(st.n_seqs, -1).contiguous(), gate=gd[st.rows], **common)
            assert max_err(o2, ref.reshape(T, H * dv)[st.rows]) < tol, pieces
    if ops.attention_split_supported(dt, H, G, d, dv):
        for t in (0, 1, far, T // 2, T // 2 + 1, 63, 64, T - 9, T - 1):
            o3 = torch.empty(1, H * dv, dtype=dt, device=DEV)
            ops.attention_split(qd[t:t + 1], kp, vp, o3, pos[t:t + 1], seq[:1], bt, max_position=t, max_keys=t + 1, gate=gd[t:t + 1], **common)
            assert max_err(o3[0], ref[t].reshape(H * dv)) < tol, t


# ------------------------------------------------------------------ the model through the engine

@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=512)
    V = plain.config["vocab"]
    for n, seed in ((1, 1), (2, 2), (9, 3), (64, 4), (65, 5), (200, 6)):
        toks = random_tokens(V, n, seed)
        ref = plain.forward(toks)
        s = eng.open(1)
        got = eng.step(s, [toks], "all")
        eng.close(s)
        assert_close(got, ref, dtype, n)
    eng.cache.check_consistent()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["vx-a", "vx-d"])
def test_residual_stream_after_every_layer(name, dtype):
    model, plain = pair(name, dtype)
    toks = random_tokens(plain.config["vocab"], 21, 8)
    _, runs = plain.forward(toks, return_layers=True)
    seen = []
    blocks = [l.block for l in model.lm.layers]
    olds = [b.forward for b in blocks]
    try:
        for b, old in zip(blocks, olds):
            def fwd(stream, ctx, cache, old=old):
                old(stream, ctx, cache)
                stream.flush()
                seen.append(stream.x.clone())
            b.forward = fwd
        eng = model.engine(max_tokens=64, use_graphs=False)
        s = eng.open(1)
        eng.step(s, [toks], "none")
        eng.close(s)
    finally:
        for b, old in zip(blocks, olds):
            b.forward = old
    assert len(seen) == runs.shape[0] == len(plain.config["layers"])
    for i, x in enumerate(seen):
        if dtype == "float32":
            assert max_err(x, runs[i]) < 2e-5 * float(runs[i].abs().max()), i
        else:
            e = row_errors(x, runs[i])
            assert float(e.mean()) < 0.03 and float(e.max()) < 0.3, (i, float(e.mean()), float(e.max()))


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefix_then_single_tokens_past_pages(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.config["vocab"], 190, 7)
    ref = plain.forward(toks)
    s = eng.open(1)
    got = [eng.step(s, [toks[:50]], "all")]                     # decoding crosses positions 64 and 128
    for t in toks[50:]:
        got.append(eng.step(s, [[t]], "last"))
    eng.close(s)
    assert_close(torch.cat(got), ref, dtype)


@pytest.mark.parametrize("name,dtype", CASES)
def test_prompt_in_pieces(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.config["vocab"], 180, 9)
    ref = plain.forward(toks)
    for cuts in ([2, 3, 7, 64, 1, 73, 30], [63, 2, 2, 113], [128, 52], [1, 1, 2, 176]):
        assert sum(cuts) == 180
        s = eng.open(1)
        got, at = [], 0
        for c in cuts:
            got.append(eng.step(s, [toks[at:at + c]], "all"))
            at += c
        eng.close(s)
        assert_close(torch.cat(got), ref, dtype, cuts)
    eng.cache.check_consistent()


@pytest.mark.parametrize("name,dtype", CASES)
def test_unequal_batch_against_each_alone_on_reused_slots(name, dtype):
    model, plain = pair(name, dtype)
    V = plain.config["vocab"]
    eng = model.engine(max_tokens=640, max_seqs=4)
    for rnd_ in range(2):                                       # the second round runs on slots and pages used before
        lens = [1, 66, 23, 130] if rnd_ == 0 else [70, 2, 129, 5]
        n_dec = [12, 30, 5, 20]
        seqs = [random_tokens(V, L + d, 20 + 10 * rnd_ + i) for i, (L, d) in enumerate(zip(lens, n_dec))]
        refs = [plain.forward(t) for t in seqs]
        slots = eng.open(4)
        if rnd_ == 1:
            slots = slots[::-1]
        got = [[] for _ in seqs]
        out = eng.step(slots, [t[:L] for t, L in zip(seqs, lens)], "last")
        for b in range(4):
            got[b].append(out[b])
        live = list(range(4))
        for step in range(max(n_dec)):
            live = [b for b in live if step < n_dec[b]]
            out = eng.step([slots[b] for b in live], [[seqs[b][lens[b] + step]] for b in live], "last")
            for r, b in enumerate(live):
                got[b].append(out[r])
            for b in list(live):
                if step + 1 == n_dec[b]:
                    eng.close([slots[b]])                       # shorter requests end earlier and give their slot back
        for b in range(4):
            ref = refs[b][lens[b] - 1:]
            assert_close(torch.stack(got[b]), ref, dtype, (rnd_, b))
        eng.cache.check_consistent()
    assert eng.cache.slots.n_free() == 4


@pytest.mark.parametrize("name,dtype", [("vx-a", "float32"), ("vx-b", "bfloat16"), ("vx-c", "float32"), ("vx-d", "bfloat16"), ("vx-e", "float32")])
def test_long_decoding_from_the_first_token(name, dtype):
    model, plain = pair(name, dtype)
    toks = random_tokens(plain.config["vocab"], 330, 11)
    ref = plain.forward(toks)
    eng = model.engine(max_tokens=384)
    s = eng.open(1)
    got = torch.cat([eng.step(s, [[t]], "last") for t in toks])
    eng.close(s)
    assert_close(got, ref, dtype)


@pytest.mark.parametrize("name", list(VIFIRAX))
def test_captured_steps_equal_eager_ones(name):
    model, plain = pair(name, "bfloat16")
    toks = [random_tokens(plain.config["vocab"], 40 + 9 * i, 30 + i) for i in range(3)]
    outs = []
    for graphs in (False, True):
        eng = model.engine(max_tokens=512, use_graphs=graphs)
        assert eng.use_graphs == graphs and (not graphs or eng.capture_prompts)
        slots = eng.open(3)
        rows = [eng.step(slots, [t[:20] for t in toks], "last")]
        for j in range(20, 40):
            rows.append(eng.step(slots, [[t[j]] for t in toks], "last"))
        # short pieces of several tokens: recorded at their second sighting
        for rep in range(3):
            eng.close(slots)
            slots = eng.open(3)
            rows.append(eng.step(slots, [t[:7] for t in toks], "last"))
        eng.close(slots)
        outs.append(torch.cat(rows))
    assert max_err(outs[0], outs[1]) < 1e-5


@pytest.mark.parametrize("name,dtype", CASES)
def test_greedy_generation_through_the_entry_point(name, dtype):
    model, plain = pair(name, dtype)
    V = plain.config["vocab"]
    prompts = [random_tokens(V, n, 40 + n) for n in (3, 17, 70)]
    res = model.generate(prompts, max_new_tokens=[10, 6, 12], stop_token_ids=[])
    for p, r, cap in zip(prompts, res, (10, 6, 12)):
        assert len(r.tokens) == cap
        seq = list(p)
        for tok in r.tokens:
            lg = plain.forward(seq)[-1]
            if dtype == "float32":
                assert float(lg.max() - lg[tok]) < 1e-4 * max(1.0, float(lg.abs().max())), "the chosen token is not the plain model's maximum"
            else:
                assert float(lg.max() - lg[tok]) < 0.15 * float(lg.std()) + 0.05
            seq.append(tok)
    model.release_engine()


# ------------------------------------------------------------------ a folder on disk: loader, command line, trace replay
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_of_a_folder(dtype, tmp_path):
    """bin/trace_run on a model folder whose config.json leaves the widths of the narrow middles to the tensors: prompts
    of unequal lengths as one batch, single tokens together, a request that ends early, one that starts later on the
    slot given back; rows asked for by index."""
    folder = vifirax_folder("vx-d", 5)
    plain = P.PlainVifirax.from_folder(folder)
    a, b, c = (random_tokens(61, n, 60 + n) for n in (70, 9, 40))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 64, 65]}, {"id": "b", "tokens": b[:7], "want": [6]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[66:67], "want": [0]}, {"id": "b", "tokens": b[7:8], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[67:68], "want": []}, {"id": "b", "tokens": b[8:9], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[68:69], "want": [0]}], "end": []},
             {"step": 4, "entries": [{"id": "c", "tokens": c[:38], "want": [37]}], "end": []},
             {"step": 5, "entries": [{"id": "c", "tokens": c[38:], "want": [0, 1]}], "end": ["c"]},
             {"step": 6, "entries": [{"id": "a", "tokens": a[69:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", "140"], input="".join(json.dumps(s) + "\n" for s in steps),
                          capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == [f"done {i}" for i in range(7)]
    ra, rb, rc = plain.forward(a), plain.forward(b), plain.forward(c)
    want = {0: torch.stack([ra[0], ra[64], ra[65], rb[6]]), 1: torch.stack([ra[66], rb[7]]), 2: rb[8][None], 3: ra[68][None],
            4: rc[37][None], 5: torch.stack([rc[38], rc[39]]), 6: ra[69][None]}
    got_all, want_all = [], []
    for i, w in want.items():
        got = torch.frombuffer(bytearray((out / f"{i}.f32").read_bytes()), dtype=torch.float32).view(-1, 61)
        assert got.shape == w.shape, i
        got_all.append(got)
        want_all.append(w)
    assert_close(torch.cat(got_all), torch.cat(want_all), dtype)


def test_command_line_generates_from_a_folder():
    folder = vifirax_folder("vx-a", 6)
    plain = P.PlainVifirax.from_folder(folder)
    proc = subprocess.run([sys.executable, "-m", "alice_llm_amd.generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", "5,9,11,60", "--prompt-ids", "3", "--max-tokens", "5"],
                          capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    for prompt in ([5, 9, 11, 60], [3]):
        ids = plain.greedy(prompt, 5)
        assert ",".join(str(i) for i in ids) in proc.stdout, (ids, proc.stdout[-500:])
