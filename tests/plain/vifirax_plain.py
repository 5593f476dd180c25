"""Plain, slow Vifirax for whole sequences: the oracle of the tests.

One function per mechanism, written from the design's equations; whole sequences, dense masks, token-by-token
recurrences, no cache, float64 by default, and no code shared with the package under test: it reads config.json
keys and safetensors tensor names itself.

The design in this file's notation (T tokens, width W, weights stored [out, in], y = x A^T):

  x        = E[token]
  layer    : x <- x + N_1(mix(x));  x <- x + N_2(ff(x))   (the sublayers read x itself; ff may be absent)
  N(y)     = y / sqrt(mean(y^2) + eps) * (1 + w)
  logits   = c * E N_f(x)                                   (c: logit_scale)

  mixer "attention":  q, k, v with biases; q and k each divided by the root mean square of the whole projection
             (all heads together) and multiplied by a weight of that length; the first R dimensions of every q
             and k head turned in the pairs (i, i + R/2) by p * f_i, cos and sin times m, with stretched
             frequencies f and the factor m of `stretched_frequencies`; scores q.k * scale over keys j <= i;
             weights exp(s_j) / (1 + sum_j exp(s_j)); head h times sigmoid((G x)_h); output matrix with bias.
             With `kv_from` the keys and values are the ones another layer made.
  mixer "mamba2":  [z | u | B | C | dt] = A_in x; (u, B, C) through a causal convolution of a few taps a channel
             with bias, then silu; dt = softplus(dt + b); per head S_t = exp(-exp(a) dt) S_(t-1) + dt B_t u_t^T,
             y_t = S_t^T C_t + D u_t; y * silu(z), normed in equal parts, times a weight; output matrix.
  mixer "channel_delta":  q, k, v each through a causal convolution without bias, then silu; q and k made unit
             vectors a head, q times d^(-1/2); beta = sigmoid(B x); a decay per head and key channel
             g = exp(-exp(a) softplus(A_2 A_1 x + b)); S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T;
             o = S^T q; o normed per head with a shared weight, times sigmoid(G_2 G_1 x); output matrix.
  ff "dense":  D (silu(G h) * (U h));   ff "moe": small gated feed-forwards; the `top` best-scoring by the router logits R h + r serve
             a token, mixed by a softmax restricted to those logits.
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

DT = torch.float64
UNIT_EPS = 1e-6          # inside the root of the unit vectors of "channel_delta"


# --------------------------------------------------------------------------- small formulas

def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * (1.0 + w)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def gated_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


# --------------------------------------------------------------------------- rotation

def stretched_frequencies(dims: int, base: float, scaling):
    """(f [dims/2], m): f_i = base^(-2i/dims); with scaling (factor s, original length L, fast, slow):
    D(t) = dims ln(L / (2 pi t)) / (2 ln base), lo = max(floor D(fast), 0), hi = min(ceil D(slow), dims - 1),
    r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), f_i <- f_i / s * r_i + f_i (1 - r_i), m = 0.1 ln s + 1."""
    i = torch.arange(dims // 2, dtype=DT)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    s, L = float(scaling["factor"]), float(scaling["original"])
    D = lambda t: dims * math.log(L / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(D(float(scaling["fast"]))), 0)
    hi = min(math.ceil(D(float(scaling["slow"]))), dims - 1)
    r = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s * r + f * (1 - r), 0.1 * math.log(s) + 1.0


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, m: float) -> torch.Tensor:
    """x: [T, heads, d]; dimension i < R/2 is paired with i + R/2 (R = 2 len(freqs)); the rest pass."""
    half = freqs.numel()
    ang = positions.to(DT)[:, None] * freqs[None, :]
    c, s = (torch.cos(ang) * m)[:, None, :], (torch.sin(ang) * m)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:2 * half]
    out[..., :half] = u * c - v * s
    out[..., half:2 * half] = v * c + u * s
    return out


# --------------------------------------------------------------------------- attention

def one_more_softmax(scores: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """Weights exp(s_j) / (1 + sum_j exp(s_j)) over the keys the mask allows (a key of score 0 without a value)."""
    s = scores.masked_fill(~mask, -math.inf)
    top = torch.clamp(s.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - top)
    return e / (torch.exp(-top) + e.sum(dim=-1, keepdim=True))


def attention_keys_values(h, p, m, eps, positions):
    """The keys (normed, turned) [T, G, d] and values [T, G, dv] that a layer makes and caches."""
    T, G, d, dv = h.shape[0], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
    k = h @ p["k"].T + p["k.b"]
    v = h @ p["v"].T + p["v.b"]
    k = unit_rms(k, eps) * p["k.norm"]
    rot = m.get("rot")
    k = k.view(T, G, d)
    if rot and rot.get("dims", d):
        f, mm = stretched_frequencies(rot.get("dims", d), rot["base"], rot.get("scaling"))
        k = rotate_halves(k, positions, f, mm)
    return k, v.view(T, G, dv)


def attention_mixer(h, p, m, eps, positions, kv):
    """kv: the (keys, values) of the whole sequence, this layer's own or another's."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
    q = h @ p["q"].T + p["q.b"]
    q = (unit_rms(q, eps) * p["q.norm"]).view(T, H, d)
    rot = m.get("rot")
    if rot and rot.get("dims", d):
        f, mm = stretched_frequencies(rot.get("dims", d), rot["base"], rot.get("scaling"))
        q = rotate_halves(q, positions, f, mm)
    k, v = kv
    n = k.shape[0]
    i = positions[:, None]
    mask = torch.arange(n)[None, :] <= i                         # the keys stand at positions 0 .. n - 1
    gate = torch.sigmoid(h @ p["g"].T)                           # [T, H]
    out = torch.empty(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        g = hh // (H // G)
        w = one_more_softmax((q[:, hh] @ k[:, g].T) * m["scale"], mask)
        out[:, hh] = (w @ v[:, g]) * gate[:, hh:hh + 1]
    return out.reshape(T, H * dv) @ p["o"].T + p["o.b"]


# --------------------------------------------------------------------------- convolution and recurrences

def causal_conv(x: torch.Tensor, w: torch.Tensor, bias=None, before=None) -> torch.Tensor:
    """x: [T, C]; w: [C, taps], the last column the current token's; zeros (or `before`, [taps - 1, C]) ahead."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.zeros(taps - 1, C, dtype=x.dtype) if before is None else before
    xp = torch.cat([pad, x], dim=0)
    y = torch.zeros(T, C, dtype=x.dtype)
    for j in range(taps):
        y = y + xp[j:j + T] * w[:, j][None, :]
    return y if bias is None else y + bias


def state_space_scan(u, B, C, dt, a_log, D, S0=None):
    """u: [T, H, P]; B, C: [T, H, N] (already given to their heads); dt: [T, H]; returns y [T, H, P] and S [H, N, P]."""
    T, H, P = u.shape
    S = torch.zeros(H, B.shape[-1], P, dtype=u.dtype) if S0 is None else S0.clone()
    y = torch.empty_like(u)
    rate = torch.exp(a_log)
    for t in range(T):
        S = torch.exp(-rate * dt[t])[:, None, None] * S + dt[t][:, None, None] * B[t][:, :, None] * u[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", S, C[t]) + D[:, None] * u[t]
    return y, S


def mamba2_mixer(h, p, m, eps, state=None, return_state=False):
    T, H, P, N, G = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    r = h @ p["in"].T
    z, xbc, dt = r[:, :inner], r[:, inner:2 * inner + 2 * G * N], r[:, 2 * inner + 2 * G * N:]
    before = None if state is None else state[0]
    conv_in = xbc if before is None else torch.cat([before, xbc], dim=0)
    xbc = silu(causal_conv(xbc, p["conv"], p["conv.b"], before))
    u = xbc[:, :inner].view(T, H, P)
    per = H // G
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(per, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(per, dim=1)
    dt = softplus(dt + p["dt_bias"])
    y, S = state_space_scan(u, B, C, dt, p["A_log"], p["D"], None if state is None else state[1])
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * p["norm"]
    out = y @ p["o"].T
    if return_state:
        taps = p["conv"].shape[1]
        full = torch.cat([torch.zeros(taps - 1, conv_in.shape[1], dtype=h.dtype), conv_in], dim=0)
        return out, (full[full.shape[0] - (taps - 1):], S)
    return out


def delta_rule_scan(q, k, v, g, beta, S0=None):
    """q, k, g: [T, H, d]; v: [T, H, dv]; beta: [T, H]: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=q.dtype) if S0 is None else S0.clone()
    o = torch.empty_like(v)
    for t in range(T):
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hdp,hd->hp", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        o[t] = torch.einsum("hdp,hd->hp", S, q[t])
    return o, S


def unit_vectors(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + UNIT_EPS)


def channel_delta_mixer(h, p, m, eps, state=None, return_state=False):
    T, H, G, d, P = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    raw = [h @ p[n].T for n in ("q", "k", "v")]
    before = [None] * 3 if state is None else state[0]
    q, k, v = (silu(causal_conv(x, p[n + ".conv"], None, b)) for x, n, b in zip(raw, ("q", "k", "v"), before))
    per = H // G
    q = (unit_vectors(q.view(T, G, d)) * d ** -0.5).repeat_interleave(per, dim=1)
    k = unit_vectors(k.view(T, G, d)).repeat_interleave(per, dim=1)
    v = v.view(T, H, P)
    beta = torch.sigmoid(h @ p["b"].T)
    rate = torch.exp(p["A_log"])[None, :, None]
    g = torch.exp(-rate * softplus((h @ p["a1"].T) @ p["a2"].T + p["dt_bias"]).view(T, H, d))
    o, S = delta_rule_scan(q, k, v, g, beta, None if state is None else state[1])
    o = unit_rms(o, eps) * p["norm"] * torch.sigmoid((h @ p["g1"].T) @ p["g2"].T).view(T, H, P)
    out = o.reshape(T, H * P) @ p["o"].T
    if return_state:
        tails = []
        for x, n, b in zip(raw, ("q", "k", "v"), before):
            taps = p[n + ".conv"].shape[1]
            full = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=h.dtype)] + ([] if b is None else [b]) + [x], dim=0)
            tails.append(full[full.shape[0] - (taps - 1):])
        return out, (tails, S)
    return out


# --------------------------------------------------------------------------- feed-forwards

def routed_ff(h, p, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ p["router"].T + p["router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    w = torch.softmax(val, dim=-1)
    out = torch.zeros(h.shape[0], p["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += w[t, j] * gated_ff(h[t:t + 1], p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"])[0]
    return out


def feed_forward(h, p, mlp):
    if mlp.get("kind", "dense") == "dense":
        return gated_ff(h, p["gate"], p["up"], p["down"])
    return routed_ff(h, p, mlp)


# --------------------------------------------------------------------------- the model

def sub(p: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in p.items() if k.startswith(prefix)}


def forward(config: dict, tensors: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of a whole sequence (and, if asked, the stream after every layer [layers, T, W])."""
    eps = config.get("norm", {}).get("eps", 1e-6)
    tok = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tok.numel())
    x = tensors["embed"][tok]
    made, after = {}, []
    for i, layer in enumerate(config["layers"]):
        p, m, kind = sub(tensors, f"l{i}."), layer["mixer"], layer["type"]
        pm = sub(p, "mix.")
        if kind == "attention":
            src = m.get("kv_from")
            if src is None:
                made[i] = attention_keys_values(x, pm, m, eps, positions)
            y = attention_mixer(x, pm, m, eps, positions, made[i if src is None else src])
        elif kind == "mamba2":
            y = mamba2_mixer(x, pm, m, eps)
        elif kind == "channel_delta":
            y = channel_delta_mixer(x, pm, m, eps)
        else:
            raise ValueError(kind)
        x = x + norm_one_plus(y, p["norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + norm_one_plus(feed_forward(x, sub(p, "mlp."), layer["mlp"]), p["norm2"], eps)
        after.append(x)
    logits = (norm_one_plus(x, tensors["final.norm"], eps) @ tensors["embed"].T) * config.get("logit_scale", 1.0)
    return (logits, torch.stack(after)) if return_layers else logits


# --------------------------------------------------------------------------- files

_DTYPES = {"F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "I32": (torch.int32, 4), "F64": (torch.float64, 8)}


def read_safetensors(path: str) -> dict:
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        dt, _ = _DTYPES[info["dtype"]]
        a, b = info["data_offsets"]
        t = torch.frombuffer(bytearray(data[a:b]), dtype=dt).reshape(info["shape"])
        out[name] = t.to(DT) if dt.is_floating_point else t
    return out


def read_model(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    return config, read_safetensors(os.path.join(folder, "model.safetensors"))


class PlainVifirax:
    def __init__(self, config: dict, tensors: dict):
        self.config, self.tensors = config, tensors

    @classmethod
    def from_folder(cls, folder: str) -> "PlainVifirax":
        return cls(*read_model(folder))

    def forward(self, tokens, return_layers: bool = False):
        return forward(self.config, self.tensors, tokens, return_layers)

    def greedy(self, prompt, n: int):
        seq, out = list(prompt), []
        for _ in range(n):
            tok = int(torch.argmax(self.forward(seq)[-1]))
            out.append(tok)
            seq.append(tok)
        return out
