"""Plain, slow Pefitar for whole sequences: the oracle of the tests.

One function per mechanism, written from the design's equations; whole sequences, dense masks, no cache,
float64 by default, and no code shared with the package under test: it reads config.json keys and
safetensors tensor names itself.

The design in this file's notation (T tokens, width W, weights stored [out, in], y = x A^T):

  x        = E[token]
  order    = layers 0..a-1, then (a..b-1) repeated n times, then b..L-1     (loop a, b, n)
  layer    : x <- x + m N_1b(mix(N_1(x)));  x <- x + m N_2b(ff(N_2(x)))    (ff may be absent; m a constant)
  N(x)     = x / sqrt(mean(x^2) + eps) * w
  ff(h)    = D (silu(G h) * (U h))
  logits   = c tanh(E N_f(x) / c)      (c: the logit cap; absent: no cap)

  mixer "attention": q, k, v without biases, H query heads on G key/value heads; the first R dimensions of the q
             and k heads rotated in pairs (2i, 2i+1) by p * base^(-2i/R); keys j <= i (or, with a window w,
             0 <= i - j < w); softmax of scale * q.k; the concatenated heads times sigmoid(A h); output matrix.
  mixer "latent_attention": cq = N(Dq h) (weight nq), q = Uq cq, per head [d plain | r rotated];
             Dkv h = [c' | kr], c = N(c') (weight nkv), kr rotated as one head shared by all heads;
             per head k = Uk c (d each), v = Uv c (dv each); score = scale (q_plain . k + q_rot . kr);
             window as above; softmax; output matrix on the concatenated heads.
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

DT = torch.float64


# --------------------------------------------------------------------------- small formulas

def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def silu_gated_ff(h, gate, up, down):
    g = h @ gate.T
    return ((g / (1.0 + torch.exp(-g))) * (h @ up.T)) @ down.T


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x: [T, heads, d]; the first `dims` dimensions of every head turn in pairs (2i, 2i + 1) by the angle
    position * base^(-2i / dims); the rest pass."""
    if dims == 0:
        return x.clone()
    i = torch.arange(dims // 2, dtype=x.dtype)
    ang = positions.to(x.dtype)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def causal_mask(T: int, size=None) -> torch.Tensor:
    """[T, T] bool: i sees j if j <= i and (size is None or i - j < size)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if size is not None:
        m = m & (i - j < size)
    return m


def softmax_attention(q, k, v, mask, scale: float) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv], mask [T, T]; head h reads kv head h // (H // G).  [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, -math.inf)
        e = torch.exp(s - s.max(dim=1, keepdim=True).values)
        out[:, h] = (e / e.sum(dim=1, keepdim=True)) @ v[:, g]
    return out


# --------------------------------------------------------------------------- the two mixers

def gated_attention(h, w, m, positions):
    """The mixer "attention".  h [T, W]; w: the mixer's tensors by local name; m: its config entry."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    G, dv = m.get("kv_heads", H), m.get("vdim", d)
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, G, d)
    v = (h @ w["v"].T).reshape(T, G, dv)
    rot = m.get("rot")
    if rot is not None:
        dims = rot.get("dims", d)
        q, k = rotate_pairs(q, positions, rot["base"], dims), rotate_pairs(k, positions, rot["base"], dims)
    mask = causal_mask(T, None if m.get("mask") is None else m["mask"]["size"])
    o = softmax_attention(q, k, v, mask, m["scale"]).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def latent_attention(h, w, m, positions, eps: float):
    """The mixer "latent_attention": every head's keys and values are made from one latent a token."""
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).reshape(T, H, d + r)
    q_plain, q_rot = q[..., :d], q[..., d:]
    dkv = h @ w["dkv"].T
    c = rms_norm(dkv[:, :rank], w["dkv.norm"], eps)
    base = m["rot"]["base"]
    k_rot = rotate_pairs(dkv[:, None, rank:], positions, base, r)                     # [T, 1, r], one for all heads
    q_rot = rotate_pairs(q_rot, positions, base, r)
    k_plain = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, dv)
    qf = torch.cat([q_plain, q_rot], dim=-1)
    kf = torch.cat([k_plain, k_rot.expand(T, H, r)], dim=-1)
    mask = causal_mask(T, None if m.get("mask") is None else m["mask"]["size"])
    o = softmax_attention(qf, kf, v, mask, m["scale"]).reshape(T, H * dv)
    return o @ w["o"].T


# --------------------------------------------------------------------------- the model

def layer_runs(cfg):
    L = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(L))
    a, b, n = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * n + list(range(b, L))


def forward(cfg, tensors, tokens, dtype=DT, return_stream=False):
    """Logits [T, vocab] of one whole sequence; with return_stream also the stream after every layer run."""
    W = {k: v.to(dtype) for k, v in tensors.items()}
    eps = float(cfg.get("norm", {}).get("eps", 1e-6))
    mult = float(cfg.get("residual_mult", 1.0))
    tok = torch.as_tensor(tokens, dtype=torch.long)
    T = tok.numel()
    pos = torch.arange(T)
    x = W["embed"][tok]
    streams = []
    for i in layer_runs(cfg):
        l = cfg["layers"][i]
        p = f"l{i}."
        w = {k[len(p) + 4:]: v for k, v in W.items() if k.startswith(p + "mix.")}
        h = rms_norm(x, W[p + "norm1"], eps)
        if l["type"] == "attention":
            y = gated_attention(h, w, l["mixer"], pos)
        elif l["type"] == "latent_attention":
            y = latent_attention(h, w, l["mixer"], pos, eps)
        else:
            raise ValueError(l["type"])
        x = x + mult * rms_norm(y, W[p + "norm1b"], eps)
        if l.get("mlp") is not None:
            h = rms_norm(x, W[p + "norm2"], eps)
            y = silu_gated_ff(h, W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"])
            x = x + mult * rms_norm(y, W[p + "norm2b"], eps)
        streams.append(x.clone())
    logits = rms_norm(x, W["final.norm"], eps) @ W["embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    if return_stream:
        return logits, torch.stack(streams)
    return logits


# --------------------------------------------------------------------------- files

_DTYPES = {"F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2), "I32": (torch.int32, 4),
           "F64": (torch.float64, 8)}


def read_safetensors(path):
    """name -> tensor, from the file format itself: 8 bytes of header length, a JSON header, the data."""
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        dt, _ = _DTYPES[info["dtype"]]
        a, b = info["data_offsets"]
        t = torch.frombuffer(bytearray(data[a:b]), dtype=dt) if b > a else torch.zeros(0, dtype=dt)
        out[name] = t.reshape(info["shape"]).clone()
    return out


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))
