"""Pefitar on the GPU against the plain implementation, in 32-bit and in bfloat16: every mechanism alone (the rows of
the fused down projection to the query latent and the cache, a matrix a head with the rotated part behind it, the
attention over latent rows with its window, the gated attention with a far key, the feed-forward, the norm with the
stream's factor), then the model through the engine: whole prompts, the stream after every layer run, a prefix and
then single tokens, prompts in pieces down to two tokens, unequal batches against each request alone on slots and
pages that are used again, long decoding from the first token, captured against eager steps, and greedy generation,
the command line and trace replay through the package's own entry points."""
import json
import math
import os
import subprocess
import sys
import types

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.hip import ops
from alice_llm_amd.parts import FEED_FORWARDS, Precision
from helpers import PEFITAR, PlainPefitar, max_err, pefitar_folder, pefitar_pair, random_tokens
from plain import pefitar_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]
CASES = [(n, d) for n in PEFITAR for d in DTYPES]
_PAIRS = {}


def pair(name, dtype):
    if (name, dtype) not in _PAIRS:
        _PAIRS[(name, dtype)] = pefitar_pair(name, dtype, seed=len(name) + 5)
    return _PAIRS[(name, dtype)]


def row_errors(got, ref):
    """Per row of logits: the root mean square of the difference (means taken off) over that of the row itself."""
    d = got.double().cpu() - ref.double().cpu()
    d = d - d.mean(-1, keepdim=True)
    r = ref.double().cpu() - ref.double().cpu().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / r.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def assert_close(got, ref, dtype, what=""):
    """32-bit: every logit within 1e-3 of the plain model's (relative to the largest logit) and the median row within
    2e-5.  bfloat16: a row's error is measured as a whole (root mean square against the row's own): the rows' mean
    within 0.06 and nine rows in ten within 0.1 (of twenty rows and more; every row within 0.3 of fewer).  A wrong
    key, window or position moves most rows by 0.3 and more."""
    assert got.shape == ref.shape, what
    if dtype == "float32":
        scale = max(1.0, float(ref.abs().max()))
        e = (got.double().cpu() - ref.double().cpu()).abs().max(-1).values
        assert float(e.max()) < 1e-3 * scale and float(e.median()) < 2e-5 * scale, (what, float(e.max()), float(e.median()))
    else:
        e = row_errors(got, ref)
        many = e.numel() >= 20
        assert float(e.mean()) < 0.06 and float(e.quantile(0.9) if many else e.max()) < (0.1 if many else 0.3) and float(e.max()) < 1.0, \
            (what, float(e.max()), float(e.mean()))


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def tables(T, width, base):
    i = torch.arange(width // 2, dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * base ** (-2.0 * i / width)[None, :]
    return torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)


def torch_dtype(dtype):
    return torch.float32 if dtype == "float32" else torch.bfloat16


# ------------------------------------------------------------------ mechanisms alone

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("A,R,r,page", [(40, 32, 8, 64), (36, 44, 6, 64), (64, 128, 32, 16), (24, 16, 16, 64), (16, 56, 0, 48),
                                        (1, 1, 2, 64), (200, 520, 64, 64)])
def test_down_projection_rows_to_query_latent_and_cache(dtype, A, R, r, page):
    """Both norms with eps inside the root (rows of tiny numbers among them), the rotation of the shared key part in
    neighbouring pairs, and the write into scattered pages, for two sequences that start at other positions than 0."""
    dt, eps, base = torch_dtype(dtype), 1e-5, 100.0
    starts, lens = [60, 3], [10, 70]
    T = sum(lens)
    rows = rnd(T, A + R + r + 3, seed=1)
    rows[5] *= 1e-3                                         # eps matters here
    wq, wc = 1.0 + 0.3 * rnd(A, seed=2), 1.0 + 0.3 * rnd(R, seed=3)
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)])
    seq = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)])
    per = -(-80 // page)
    bt = (torch.randperm(2 * per + 2, generator=torch.Generator().manual_seed(4))[:2 * per] + 1).view(2, per).to(torch.int32)
    pool = torch.zeros(2 * per + 4, 1, page, R + r, dtype=dt, device=DEV)
    a = torch.empty(T, A, dtype=dt, device=DEV)
    c, s = tables(80, r, base) if r else (None, None)
    ops.latent_prepare(rows.to(DEV), wq.to(DEV), wc.to(DEV), a, pool, pos.to(torch.int32).to(DEV), seq.to(torch.int32).to(DEV),
                       bt.to(DEV), q_rank=A, kv_rank=R, rot_dim=r, eps=eps, cos=c, sin=s, max_position=79)
    x = rows.double()
    tol = 3e-6 if dtype == "float32" else 2e-2
    assert max_err(a, P.rms_norm(x[:, :A], wq.double(), eps)) < tol * 4
    lat = P.rms_norm(x[:, A:A + R], wc.double(), eps)
    kr = P.rotate_pairs(x[:, None, A + R:A + R + r], pos, base, r)[:, 0]
    want = torch.cat([lat, kr], dim=1)
    for t in range(T):
        page_id = int(bt[seq[t], pos[t] // page])
        assert max_err(pool[page_id, 0, pos[t] % page], want[t]) < tol * 4, t
    used = set(int(bt[seq[t], pos[t] // page]) for t in range(T))
    for p_ in range(pool.shape[0]):
        if p_ not in used:
            assert float(pool[p_].abs().max()) == 0.0, p_   # nothing beside its own places
    # without a cache to write (a layer that reads another's rows): the query latent alone
    a2 = torch.empty_like(a)
    ops.latent_prepare(rows.to(DEV), wq.to(DEV), wc.to(DEV), a2, None, pos.to(torch.int32).to(DEV), None, None,
                       q_rank=A, kv_rank=R, rot_dim=r, eps=eps, cos=c, sin=s, max_position=79)
    assert max_err(a2, a.double().cpu()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,n,k,r", [(1, 4, 32, 16, 8), (5, 3, 44, 20, 6), (17, 4, 128, 32, 32), (70, 2, 16, 8, 16), (300, 5, 56, 24, 0),
                                       (64, 4, 24, 32, 0), (65, 3, 28, 44, 0), (2, 1, 1, 1, 2), (9, 16, 512, 128, 64), (33, 2, 260, 72, 0)])
def test_a_matrix_a_head_with_the_rotated_part_behind_it(dtype, T, H, n, k, r):
    """y[t, h] = [M_h x[t, h, :k] | the r numbers behind them turned by the token's position]: the map of the plain query
    into the latent's space (with rotation) and the value map (without), by the plain kernel and, in bfloat16 where
    the sizes suit, by the matrix-core one."""
    dt, base = torch_dtype(dtype), 50.0
    x = rnd(T, H * (k + r), seed=1).to(dt)
    w = rnd(H, n, k, seed=2, scale=k ** -0.5).to(dt)
    pos = torch.randint(0, 500, (T,), generator=torch.Generator().manual_seed(3))
    c, s = tables(500, r, base) if r else (None, None)
    xs = x.double().view(T, H, k + r)
    ref = torch.cat([torch.einsum("thk,hnk->thn", xs[..., :k], w.double()), P.rotate_pairs(xs[..., k:], pos, base, r)], dim=-1)
    kw = dict(heads=H, n=n, k=k, rot_dim=r, cos=c, sin=s, positions=pos.to(torch.int32).to(DEV), max_position=499)
    tol = (2e-5 if dtype == "float32" else 2e-2) * max(1.0, float(ref.abs().max()))
    y = torch.full((T, H * (n + r)), 9.0, dtype=dt, device=DEV)
    ops.heads_linear(x.to(DEV), w.transpose(1, 2).contiguous().to(DEV), y, **kw)
    assert max_err(y.view(T, H, n + r), ref) < tol
    if ops.heads_linear_mfma_supported(dt, n, k, r):
        y2 = torch.full_like(y, 9.0)
        ops.heads_linear_mfma(x.to(DEV), w.to(DEV), y2, **kw)
        assert max_err(y2.view(T, H, n + r), ref) < tol
    else:
        assert dtype == "float32" or n % 4 or k % 8 or r % 8, "a size the matrix-core kernel was expected to take"


def _latent_pool(rows, page, lens, starts, seed):
    """The cached rows of several sequences put into scattered pages: rows[i] is [starts[i] + lens[i], D]."""
    per = [-(-(s + n) // page) for s, n in zip(starts, lens)]
    n_pages = sum(per) + 3
    order = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(seed)) + 1
    D = rows[0].shape[1]
    pool = torch.full((n_pages, 1, page, D), 7.0, dtype=rows[0].dtype)
    bt = torch.zeros(len(lens), max(per), dtype=torch.int32)
    at = 0
    for i, rws in enumerate(rows):
        for j in range(per[i]):
            bt[i, j] = order[at]
            chunk = rws[j * page:(j + 1) * page]
            pool[order[at], 0, :chunk.shape[0]] = chunk
            at += 1
    return pool.to(DEV), bt.to(DEV)


def _latent_ctx(lens, starts):
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)])
    seq = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)])
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    return types.SimpleNamespace(positions=pos.to(torch.int32).to(DEV), seq_of_token=seq.to(torch.int32).to(DEV),
                                 cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=DEV), n_seqs=len(lens),
                                 max_position=max(s + n for s, n in zip(starts, lens)) - 1)


def _latent_plain(q, rows, R, window, scale, start):
    """q [n, H, D] at positions start .. start + n - 1 over rows [start + n, D]: weights times the rows' first R numbers."""
    n, H, D = q.shape
    out = torch.zeros(n, H, R, dtype=torch.float64)
    for i in range(n):
        p = start + i
        lo = 0 if window is None else max(0, p + 1 - window)
        keys = rows[lo:p + 1].double()
        s = (q[i].double() @ keys.T) * scale
        out[i] = torch.softmax(s, dim=1) @ keys[:, :R]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,R,r,window,page,T", [(4, 32, 8, 9, 64, 150), (3, 44, 6, 70, 64, 200), (4, 128, 32, 64, 64, 200),
                                                 (2, 16, 16, 1, 64, 70), (5, 56, 8, None, 64, 700), (4, 64, 16, 65, 16, 150),
                                                 (2, 64, 0, 128, 48, 300), (16, 256, 32, 300, 64, 330)])
def test_attention_over_latent_rows_at_the_windows_edges_and_far_back(dtype, H, R, r, window, page, T):
    """Marker rows that every query scores far above the others: one just inside the window of one query and just
    outside that of the next (with no window: at position 3, hundreds of keys back), one at a page's last place.
    A whole prompt, the prompt in pieces around the edges as sequences of one step, and single tokens on the rows
    around every edge; by the 32-bit kernel and, in bfloat16 where the sizes suit, by the matrix-core one (single
    tokens also with the keys spread over blocks)."""
    dt, D, scale = torch_dtype(dtype), R + r, 0.5
    rows, q = rnd(T, D, seed=1, scale=0.4), rnd(T, H, D, seed=2, scale=0.4)
    q[:, :, 0], rows[:, 0] = 3.0, 0.0
    mark = 3 if window is None else max(1, T - 20 - window)
    rows[mark, 0] = 6.0                                     # the latent is the value too: the marker shows in column 0
    edge = page * ((T - 5) // page) - 1                     # a page's last place
    if edge != mark and edge > 0:
        rows[edge, 0] = 4.0
    rows, q = rows.to(dt), q.to(dt)
    ref = _latent_plain(q, rows, R, window, scale, 0)
    if window is not None and mark + window < T:
        assert (ref[mark + window - 1] - ref[mark + window]).abs().max() > 0.5          # the marker does show
    else:
        assert float(ref[T - 1, :, 0].min()) > 3.0                                      # the far key carries the last row
    edges = [e for e in ((mark + window if window else T - 1), (edge + window if window else edge + 1), edge + 1) if 0 < e < T]
    tol = 3e-5 if dtype == "float32" else 6e-2
    tiled = dtype == "bfloat16" and ops.latent_tiled_supported(dt, R, r)
    assert tiled or dtype == "float32" or R % 8 or r % 8, "sizes the matrix-core kernel was expected to take"
    # whole, and in pieces: each piece is a sequence of the step with its own copy of the rows up to its end
    cuts = sorted({0, T} | {p for e in edges for p in (e - 1, e, e + 2) if 0 < p < T})
    for pieces in ([(0, T)], list(zip(cuts[:-1], cuts[1:]))):
        lens, starts = [b - a for a, b in pieces], [a for a, b in pieces]
        pool, bt = _latent_pool([rows[:b] for a, b in pieces], page, lens, starts, 5)
        ctx = _latent_ctx(lens, starts)
        idx = torch.cat([torch.arange(a, b) for a, b in pieces])
        qs = q[idx].reshape(-1, H * D).contiguous().to(DEV)
        out = torch.empty(idx.numel(), H * R, dtype=dt, device=DEV)
        ops.latent_attention(qs, pool, out, ctx, bt, num_heads=H, kv_rank=R, rot_dim=r, scale=scale, window=window,
                             full_precision=dtype == "float32")
        assert max_err(out.view(-1, H, R), ref[idx]) < tol, len(pieces)
        if tiled:
            out2 = torch.full_like(out, 9.0)
            ops.latent_attention_tiled(qs, pool, out2, ctx, bt, num_heads=H, kv_rank=R, rot_dim=r, scale=scale, window=window)
            assert max_err(out2.view(-1, H, R), ref[idx]) < tol, ("tiled", len(pieces))
    # single tokens around every edge, each a sequence of its own, in one step
    singles = sorted({p for e in edges for p in (e - 1, e, e + 1) if 0 <= p < T} | {0, T - 1})
    pool, bt = _latent_pool([rows[:p + 1] for p in singles], page, [1] * len(singles), singles, 6)
    ctx = _latent_ctx([1] * len(singles), singles)
    qs = q[singles].reshape(-1, H * D).contiguous().to(DEV)
    out = torch.empty(len(singles), H * R, dtype=dt, device=DEV)
    ops.latent_attention(qs, pool, out, ctx, bt, num_heads=H, kv_rank=R, rot_dim=r, scale=scale, window=window,
                         full_precision=dtype == "float32")
    assert max_err(out.view(-1, H, R), ref[singles]) < tol, singles
    if tiled:
        most = T if window is None else min(T, window)
        # by the kernel of single tokens (the waves share a token's heads) and by the prompt kernel's mapping
        for splits, single in [(s_, w_) for s_ in sorted({1, 2, ops.latent_tiled_splits(len(singles), H, most)}) for w_ in (True, False)]:
            out2 = torch.full_like(out, 9.0)
            ops.latent_attention_tiled(qs, pool, out2, ctx, bt, num_heads=H, kv_rank=R, rot_dim=r, scale=scale, window=window,
                                       splits=splits, single_tokens=single)
            assert max_err(out2.view(-1, H, R), ref[singles]) < tol, ("tiled", splits, single)
        with pytest.raises(ops.HipLibraryError, match="single tokens"):         # two tokens of one sequence are no such step
            ops.latent_attention_tiled(qs[:2].contiguous(), pool, out[:2], _latent_ctx([2], [0]), bt, num_heads=H, kv_rank=R,
                                       rot_dim=r, scale=scale, window=window, single_tokens=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,T", [(8, 1, 64, 32, 700), (4, 2, 16, 32, 330), (3, 3, 20, 20, 200), (6, 2, 16, 24, 130)])
def test_gated_attention_finds_a_key_hundreds_of_tokens_back(dtype, H, G, d, dv, T):
    """Every earlier key is visible: a marker key at position 3 carries the last rows over hundreds of others; the
    elementwise gate (rows of a wider matrix) closes some output elements and opens others."""
    dt, page = torch_dtype(dtype), 64
    q, k, v = rnd(T, H, d, seed=1, scale=0.4), rnd(T, G, d, seed=2, scale=0.4), rnd(T, G, dv, seed=3)
    gate = rnd(T, H * dv + 5, seed=4, scale=3.0)
    q[:, :, 0], k[:, :, 0] = 3.0, 0.0
    k[3, :, 0] = 8.0
    v[3] += 5.0
    q, k, v = q.to(dt), k.to(dt), v.to(dt)
    ref = P.softmax_attention(q.double(), k.double(), v.double(), P.causal_mask(T), 0.5)
    assert float((ref[T - 1] - v[3].double().repeat_interleave(H // G, 0)).abs().max()) < 0.2
    ref = ref * torch.sigmoid(gate.double()[:, :H * dv]).view(T, H, dv)
    n = -(-T // page)
    order = torch.randperm(n + 3, generator=torch.Generator().manual_seed(5))[:n] + 1
    kp = torch.full((n + 5, G, page, d), 7.0, dtype=dt)
    vp = torch.full((n + 5, G, page, dv), -7.0, dtype=dt)
    for t in range(T):
        kp[order[t // page], :, t % page], vp[order[t // page], :, t % page] = k[t], v[t]
    kp, vp, bt = kp.to(DEV), vp.to(DEV), order.to(torch.int32)[None].to(DEV)
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    g = gate.to(DEV)
    tol = 3e-5 if dtype == "float32" else 8e-2
    for rows in (slice(0, T), slice(T - 1, T), slice(3, 4), slice(64, 65), slice(0, 1)):
        m = rows.stop - rows.start
        qs = q[rows].reshape(m, H * d).contiguous().to(DEV)
        out = torch.empty(m, H * dv, dtype=dt, device=DEV)
        ops.attention_masked(qs, kp, vp, out, pos[rows].contiguous(), seq[rows].contiguous(), bt, num_heads=H, scale=0.5,
                             max_position=T - 1, full_precision=dtype == "float32", gate=g[rows][:, :H * dv], gate_per_element=True)
        assert max_err(out.view(m, H, dv), ref[rows]) < tol, rows
        if ops.attention_split_supported(dt, H, G, d, dv):
            out2 = torch.full_like(out, 9.0)
            ops.attention_split(qs, kp, vp, out2, pos[rows].contiguous(), seq[rows].contiguous(), bt, num_heads=H, scale=0.5,
                                max_position=T - 1, max_keys=T, gate=g[rows][:, :H * dv], gate_per_element=True)
            assert max_err(out2.view(m, H, dv), ref[rows]) < tol, ("split", rows)
    if dtype == "bfloat16" and ops.attention_tiled_supported(dt, d, dv):
        for pieces in ([(0, T)], [(0, 2), (2, 4), (4, 65), (65, T - 1), (T - 1, T)]):
            idx = torch.cat([torch.arange(a, b) for a, b in pieces])
            cu = [0]
            for a, b in pieces:
                cu.append(cu[-1] + b - a)
            ctx = types.SimpleNamespace(positions=idx.to(torch.int32).to(DEV), cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=DEV),
                                        n_seqs=len(pieces), max_position=T - 1)
            out = torch.empty(T, H * dv, dtype=dt, device=DEV)
            ops.attention_tiled(q[idx].reshape(T, H * d).contiguous().to(DEV), kp, vp, out, ctx, bt.expand(len(pieces), -1).contiguous(),
                                num_heads=H, scale=0.5, gate=g[idx.to(DEV)][:, :H * dv], gate_per_element=True)
            assert max_err(out.view(T, H, dv), ref[idx]) < tol, len(pieces)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,W,I", [(5, 64, 96), (70, 72, 100), (300, 128, 256), (33, 48, 80), (1, 64, 96)])
def test_silu_gated_feed_forward(dtype, T, W, I):
    p = Precision.of(dtype)
    ff = FEED_FORWARDS.get("gated_mlp")(p, hidden_size=W, intermediate_size=I, activation="silu",
                                        tensor_names={"gate": "gate", "up": "up", "down": "down"})
    ws = {n: rnd(*s.shape, seed=i, scale=0.2).to(torch.bfloat16).to(DEV) for i, (n, s) in enumerate(ff.param_specs().items())}
    assert set(ws) == {"gate", "up", "down"}
    for n, t in ws.items():
        ff.assign(n, t)
    ff.finalize()
    x = rnd(T, W, seed=9, scale=2.0).to(p.act).to(DEV)
    out = ff.forward(x, None)
    out = out.sum(0) if out.dim() == 3 else out
    ref = P.silu_gated_ff(x.double().cpu(), ws["gate"].double().cpu(), ws["up"].double().cpu(), ws["down"].double().cpu())
    assert max_err(out, ref) < (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,W,mult", [(1, 64, 0.7), (9, 72, 1.0), (70, 100, 1.3), (300, 128, 0.4), (5, 2048, 0.25)])
def test_norms_around_a_sublayer_with_the_streams_factor(dtype, T, W, mult):
    """x + m N_b(branch) and then N_a of the sum, by the fused add-and-norm kernel and by the add alone: eps inside the
    root (a branch row of tiny numbers), weights stored in bfloat16 and kept in 32-bit with the factor folded in, the
    stream in 32-bit whatever the arithmetic."""
    from alice_llm_amd.parts import NORMS
    from alice_llm_amd.parts.stream import ResidualStream
    prec, eps = Precision.of(dtype), 1e-5
    behind = NORMS.get("rmsnorm")(prec, dim=W, eps=eps, tensor_name="", output_scale=mult, keep_float32=True)
    ahead = NORMS.get("rmsnorm")(prec, dim=W, eps=eps, tensor_name="", keep_float32=True)
    wb, wa = (1.0 + 0.3 * rnd(W, seed=1)).to(torch.bfloat16), (1.0 + 0.3 * rnd(W, seed=2)).to(torch.bfloat16)
    behind.assign("", wb.to(DEV))
    ahead.assign("", wa.to(DEV))
    assert behind.weight.dtype == torch.float32 and ahead.weight.dtype == torch.float32
    x, branch = rnd(T, W, seed=3, scale=2.0), rnd(T, W, seed=4, scale=5.0)
    branch[0] *= 1e-4
    want_x = x.double() + mult * P.rms_norm(branch.double(), wb.double(), eps)
    want_h = P.rms_norm(want_x, wa.double(), eps)
    for fused in (True, False):
        stream = ResidualStream(x.clone().to(DEV), prec)
        stream.push(branch.to(DEV), behind)
        if fused:
            h = stream.normed(ahead)
            assert max_err(h, want_h) < (3e-6 if dtype == "float32" else 2e-2) * 4
        stream.flush()
        assert stream.x.dtype == torch.float32 and max_err(stream.x, want_x) < 2e-5


# ------------------------------------------------------------------ the model through the engine

@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=512)
    V = plain.c["vocab"]
    for n, seed in ((1, 1), (2, 2), (9, 3), (10, 3), (64, 4), (65, 5), (200, 6)):
        toks = random_tokens(V, n, seed)
        ref = plain.forward(toks)
        s = eng.open(1)
        got = eng.step(s, [toks], "all")
        eng.close(s)
        assert_close(got, ref, dtype, n)
    eng.cache.check_consistent()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["pf-a", "pf-d"])
def test_residual_stream_after_every_layer_run(name, dtype):
    """The stream after each run of a layer (a looped layer counts each time), against the plain one: every norm, the
    stream's factor and each mixer in its place."""
    model, plain = pair(name, dtype)
    toks = random_tokens(plain.c["vocab"], 21, 8)
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
    assert len(seen) == runs.shape[0] == len(P.layer_runs(plain.c))
    assert seen[0].dtype == torch.float32                    # the stream is 32-bit in either arithmetic
    for i, x in enumerate(seen):
        assert max_err(x, runs[i]) < (2e-5 if dtype == "float32" else 5e-2) * float(runs[i].abs().max()), i


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefix_then_single_tokens_past_windows_and_pages(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.c["vocab"], 190, 7)
    ref = plain.forward(toks)
    s = eng.open(1)
    got = [eng.step(s, [toks[:50]], "all")]                     # decoding crosses positions 64 and 128 and every window's edge
    for t in toks[50:]:
        got.append(eng.step(s, [[t]], "last"))
    eng.close(s)
    assert_close(torch.cat(got), ref, dtype)
    eng.cache.check_consistent()


@pytest.mark.parametrize("name,dtype", CASES)
def test_prompt_in_pieces(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.c["vocab"], 180, 9)
    ref = plain.forward(toks)
    for cuts in ([2, 3, 7, 64, 1, 73, 30], [63, 2, 2, 113], [128, 52], [2] * 8 + [164]):
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
    V = plain.c["vocab"]
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


@pytest.mark.parametrize("name,dtype", [("pf-a", "float32"), ("pf-b", "bfloat16"), ("pf-c", "float32"), ("pf-c", "bfloat16"), ("pf-d", "bfloat16")])
def test_long_decoding_from_the_first_token(name, dtype):
    model, plain = pair(name, dtype)
    toks = random_tokens(plain.c["vocab"], 330, 11)
    ref = plain.forward(toks)
    eng = model.engine(max_tokens=384)
    s = eng.open(1)
    got = torch.cat([eng.step(s, [[t]], "last") for t in toks])
    eng.close(s)
    assert_close(got, ref, dtype)
    eng.cache.check_consistent()


def test_window_pages_go_back_to_the_pool_while_decoding():
    """A layer whose window lies pages behind the newest token holds no more pages than the window needs."""
    model, plain = pair("pf-a", "bfloat16")                     # windows of 9 keys beside an attention layer that keeps all
    eng = model.engine(max_tokens=1024)
    free0 = [g.n_free() for g in eng.cache.groups]
    s = eng.open(1)
    eng.step(s, [random_tokens(97, 300, 3)], "none")
    for t in random_tokens(97, 200, 4):
        eng.step(s, [[t]], "none")
    eng.cache.check_consistent()
    held = [a - g.n_free() for a, g in zip(free0, eng.cache.groups)]
    assert min(held) <= 2 and max(held) >= 500 // eng.page_size, held
    eng.close(s)
    assert [g.n_free() for g in eng.cache.groups] == free0


@pytest.mark.parametrize("name", list(PEFITAR))
def test_captured_steps_equal_eager_ones(name):
    model, plain = pair(name, "bfloat16")
    toks = [random_tokens(plain.c["vocab"], 40 + 9 * i, 30 + i) for i in range(3)]
    outs = []
    for graphs in (False, True):
        eng = model.engine(max_tokens=512, use_graphs=graphs)
        slots = eng.open(3)
        rows = [eng.step(slots, [t[:20] for t in toks], "last")]
        for j in range(20, 40):
            rows.append(eng.step(slots, [[t[j]] for t in toks], "last"))
        for rep in range(3):                                     # short pieces of several tokens: recorded at their second sighting
            eng.close(slots)
            slots = eng.open(3)
            rows.append(eng.step(slots, [t[:7] for t in toks], "last"))
        eng.close(slots)
        outs.append(torch.cat(rows))
    assert max_err(outs[0], outs[1]) < 1e-5


@pytest.mark.parametrize("name,dtype", CASES)
def test_greedy_generation_through_the_entry_point(name, dtype):
    model, plain = pair(name, dtype)
    V = plain.c["vocab"]
    prompts = [random_tokens(V, n, 40 + n) for n in (3, 17, 70)]
    res = model.generate(prompts, max_new_tokens=[10, 6, 12], stop_token_ids=[])
    for p, r, cap in zip(prompts, res, (10, 6, 12)):
        assert len(r.tokens) == cap
        seq = list(p)
        for tok in r.tokens:
            lg = plain.forward(seq)[-1]
            if dtype == "float32":
                assert float(lg.max() - lg[tok]) < 1e-4, "the chosen token is not the plain model's maximum"
            else:
                assert float(lg.max() - lg[tok]) < 0.15 * float(lg.std()) + 0.05
            seq.append(tok)
    model.release_engine()


# ------------------------------------------------------------------ a folder on disk: loader, command line, trace replay
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_of_a_folder(dtype, tmp_path):
    """bin/trace_run on a model folder: prompts of unequal lengths as one batch, single tokens together, a request
    that ends early, one that starts later on the slot given back; rows asked for by index."""
    folder = pefitar_folder("pf-d", 5)
    plain = PlainPefitar.from_folder(folder)
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
    folder = pefitar_folder("pf-a", 6)
    plain = PlainPefitar.from_folder(folder)
    proc = subprocess.run([sys.executable, "-m", "alice_llm_amd.generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", "5,9,11,60", "--prompt-ids", "3", "--max-tokens", "5"],
                          capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    for prompt in ([5, 9, 11, 60], [3]):
        ids = plain.greedy(prompt, 5)
        assert ",".join(str(i) for i in ids) in proc.stdout, (ids, proc.stdout[-500:])


# ------------------------------------------------------------------ configurations drawn at random

def _drawn_config(seed):
    """Layers, sizes and constants drawn from a seed: sizes that fit the matrix-core kernels and sizes that fit none,
    one head and many, every window from a single key to none, loops at the start, the end and over everything."""
    g = torch.Generator().manual_seed(1000 + seed)
    pick = lambda xs: xs[int(torch.randint(0, len(xs), (1,), generator=g))]
    n_layers = pick([1, 2, 3, 4])
    layers = []
    for _ in range(n_layers):
        base = pick([50.0, 1000.0, 30000.0, 500000.0])
        if pick([0, 1]):
            heads = pick([1, 2, 3, 4, 6, 8])
            kv = pick([k for k in (1, 2, 3, 4, 6, 8) if heads % k == 0])
            dim = pick([8, 12, 16, 24, 32, 40, 64])
            mixer = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": pick([8, 12, 20, 32, 48, 64]), "scale": pick([0.1, 0.2, dim ** -0.5]),
                     "rot": {"base": base, "dims": pick([d for d in (2, 4, 8, 12, 16, 32, 64) if d <= dim])}}
            if pick([0, 0, 1]):
                mixer["mask"] = {"size": pick([5, 64, 90])}
            kind = "attention"
        else:
            rot = pick([2, 4, 8, 16, 24, 32])
            mixer = {"heads": pick([1, 2, 3, 4, 5, 8]), "dim": pick([4, 7, 16, 24, 32, 48]), "rot_dim": rot, "vdim": pick([8, 20, 28, 48, 80]),
                     "q_rank": pick([16, 30, 64, 96]), "kv_rank": pick([24, 32, 50, 64, 96, 128]), "scale": pick([0.1, 0.15, 0.25]),
                     "rot": {"base": base, "dims": rot}}
            w = pick([None, 1, 2, 7, 31, 63, 64, 65, 70, 100, 129])
            if w is not None:
                mixer["mask"] = {"size": w}
            kind = "latent_attention"
        layers.append({"type": kind, "mixer": mixer, "mlp": None if pick([0, 0, 0, 1]) else {"kind": "dense", "ff": pick([40, 64, 100, 192])}})
    raw = {"architecture": "Pefitar", "vocab": pick([50, 97, 211, 300]), "width": pick([48, 64, 80, 100, 128]),
           "norm": {"eps": pick([1e-5, 1e-6])}, "residual_mult": pick([0.3, 0.5, 1.0, 1.4]), "layers": layers}
    if pick([0, 1]):
        raw["logit_softcap"] = pick([10.0, 30.0])
    if pick([0, 1, 1]):
        a = pick(list(range(n_layers)))
        raw["loop"] = {"start": a, "stop": pick(list(range(a + 1, n_layers + 1))), "times": pick([1, 2, 3])}
    return raw


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations_whole_in_pieces_and_token_by_token(seed, dtype):
    from helpers import model_from_tensors, pefitar_tensors
    raw = _drawn_config(seed)
    cfg, tensors = pefitar_tensors(raw, seed)
    model = model_from_tensors(cfg, {k: v.to(DEV) for k, v in tensors.items()}, dtype)
    plain = PlainPefitar(raw, tensors)
    toks = random_tokens(raw["vocab"], 150, seed)
    ref = plain.forward(toks)
    eng = model.engine(max_tokens=512, max_seqs=4)
    s = eng.open(1)
    assert_close(eng.step(s, [toks], "all"), ref, dtype, ("whole", raw))
    eng.close(s)
    s = eng.open(2)                                             # beside a second request of another length, then token by token
    other = random_tokens(raw["vocab"], 40, seed + 50)
    got = [eng.step(s, [toks[:3], other[:9]], "all")[:3], eng.step(s, [toks[3:70], other[9:11]], "all")[:67]]
    for j in range(70, 150):
        both = j - 70 < 29                                      # the second request ends after 29 single tokens
        got.append(eng.step(s if both else s[:1], [[toks[j]], [other[11 + j - 70]]] if both else [[toks[j]]], "last")[:1])
        if j - 70 == 28:
            eng.close(s[1:])
    eng.close(s[:1])
    assert_close(torch.cat(got), ref, dtype, ("pieces", raw))
    eng.cache.check_consistent()
