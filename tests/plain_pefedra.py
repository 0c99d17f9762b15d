"""Plain float64 implementation of the Pefedra design: one function per mechanism, whole
sequences, nothing cached, no code shared with the engine.  ``weights``: tensors by checkpoint
name, float64; ``cfg``: the config.json dict.

Notation: x the stream [T, d]; n(x; w) = x / sqrt(mean(x^2) + eps) * w; positions count from 0.
"""
from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm(x, w, eps):
    return unit_rms(x, eps) * w


def gelu(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def token_shift(h, mu):
    """h[t] + (h[t-1] - h[t]) * mu, with zeros before the first token."""
    before = torch.zeros_like(h)
    before[1:] = h[:-1]
    return h + (before - h) * mu


def turn_halves(x, angle_pos, n_turn, base, divide=1.0):
    """x [T, heads, D]: the first ``n_turn`` elements of every head turn in pairs (i, i + n_turn/2)
    by angle_pos[t] * base^(-2i/n_turn) / divide; the rest stay."""
    half = n_turn // 2
    if half == 0:
        return x
    freq = torch.tensor([base ** (-2.0 * i / n_turn) / divide for i in range(half)], dtype=torch.float64)
    ang = angle_pos.to(torch.float64)[:, None, None] * freq[None, None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:n_turn]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., n_turn:]], dim=-1)


def window_mask(T, size):
    """[T, T] True where query i may read key j: 0 <= i - j < size (size None: every earlier key)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & (i - j < size)
    return ok


def softmax_attention(q, k, v, scale, mask):
    """q [T, D], k [T, D], v [T, Vd] of one head -> [T, Vd]."""
    s = (q @ k.T) * scale
    s = s.masked_fill(~mask, float("-inf"))
    return torch.softmax(s, dim=-1) @ v


def projections(W, p, h):
    return (h @ W[p + "q"].T + W[p + "q.b"], h @ W[p + "k"].T + W[p + "k.b"], h @ W[p + "v"].T + W[p + "v.b"])


def rotation_of(mx):
    rot = mx.get("rot")
    if rot is None:
        return 0, 1.0, 1.0
    return int(rot["dims"]), float(rot["base"]), float((rot.get("scaling") or {}).get("factor", 1.0))


def diff_lambda(W, p, diff):
    return math.exp(float((W[p + "lq1"] * W[p + "lk1"]).sum())) - math.exp(float((W[p + "lq2"] * W[p + "lk2"]).sum())) + diff


def differential_attention(W, p, h, mx, eps):
    """Mixer ``attention``: two score maps a head over the same values."""
    T = h.shape[0]
    H, G, D, Vd = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    pos = torch.arange(T)
    q, k, v = projections(W, p, h)
    n_turn, base, divide = rotation_of(mx)
    q = turn_halves(q.view(T, 2 * H, D), pos, n_turn, base, divide).view(T, H, 2, D)
    k = turn_halves(k.view(T, 2 * G, D), pos, n_turn, base, divide).view(T, G, 2, D)
    v = v.view(T, G, Vd)
    mask = window_mask(T, (mx.get("mask") or {}).get("size"))
    lam = diff_lambda(W, p, mx["diff"])
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        a1 = softmax_attention(q[:, hh, 0], k[:, g, 0], v[:, g], mx["scale"], mask)
        a2 = softmax_attention(q[:, hh, 1], k[:, g, 1], v[:, g], mx["scale"], mask)
        heads.append(unit_rms(a1 - lam * a2, eps) * (1.0 - mx["diff"]))
    return torch.cat(heads, dim=-1) @ W[p + "o"].T


def gated_attention(W, p, h, mx, eps):
    """Mixer ``attention_2``: norm over the whole q and k projections, values that turn with their
    position and are turned back at the query, a gate per head."""
    T = h.shape[0]
    H, G, D, Vd = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    pos = torch.arange(T)
    q, k, v = projections(W, p, h)
    q, k = norm(q, W[p + "q.norm"], eps), norm(k, W[p + "k.norm"], eps)
    n_turn, base, divide = rotation_of(mx)
    q = turn_halves(q.view(T, H, D), pos, n_turn, base, divide)
    k = turn_halves(k.view(T, G, D), pos, n_turn, base, divide)
    v = turn_halves(v.view(T, G, Vd), pos, Vd, base)                 # the keys' scaling does not apply
    mask = window_mask(T, (mx.get("mask") or {}).get("size"))
    gate = torch.sigmoid(h @ W[p + "g"].T)
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        o = softmax_attention(q[:, hh], k[:, g], v[:, g], mx["scale"], mask)
        o = turn_halves(o[:, None, :], -pos, Vd, base)[:, 0]
        heads.append(o * gate[:, hh:hh + 1])
    return torch.cat(heads, dim=-1) @ W[p + "o"].T


def feed_forward(W, p, h):
    return gelu(h @ W[p + "up"].T) @ W[p + "down"].T


MIXERS = {"attention": differential_attention, "attention_2": gated_attention}


def layer(cfg, W, i, x):
    """x + mixer(shift(n(x; norm1))) + ff(n(x; norm2))."""
    L, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    h = token_shift(norm(x, W[p + "norm1"], eps), W[p + "shift"])
    y = MIXERS[L["type"]](W, p + "mix.", h, L["mixer"], eps)
    if L.get("mlp") is not None:
        y = y + feed_forward(W, p + "mlp.", norm(x, W[p + "norm2"], eps))
    return x + y


def forward(cfg, W, tokens, upto=None):
    """Logits [T, vocab] of a whole sequence (``upto``: the stream after that many layers instead)."""
    x = W["embed"][torch.tensor(list(tokens), dtype=torch.long)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    for i in range(len(cfg["layers"]) if upto is None else upto):
        x = layer(cfg, W, i, x)
    if upto is not None:
        return x
    return norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T


def greedy(row):
    return int(torch.argmax(row))
