"""Plain, slow implementation of the Ravenex design, one function per mechanism, on whole
sequences in float64 on the CPU.  It shares no code with the engine: the tests hold the
engine's kernels, cache and scheduler against it.

Notation: d the model's width, H heads, n the unrotated and r the rotated query/key sizes of a
head, v the value size of a head, R the latent's size, W the window, m the residual multiplier.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_adjacent(x, positions, base, dims):
    """x [..., T, D]: pairs (2i, 2i+1) of the first ``dims`` elements turn by p * base^(-2i/dims)."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=F)
    ang = positions.to(F)[:, None] * base ** (-2.0 * i / dims)          # [T, dims/2]
    c, s = torch.cos(ang), torch.sin(ang)
    u, w = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - w * s
    out[..., 1:dims:2] = w * c + u * s
    return out


def latent_kv(h, w_dkv, w_norm, eps, R, rot, positions):
    """The latent c [T, R] and the rotated key part [T, r] that a layer caches."""
    z = h @ w_dkv.T
    c = norm(z[:, :R], w_norm, eps)
    kr = rotate_adjacent(z[:, R:], positions, rot["base"], rot["dims"])
    return c, kr


def window_mask(T, W):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = (j <= i)
    if W is not None:
        ok = ok & (i - j < W)
    return ok


def latent_attention(h, c, kr, w, mx, positions):
    """h [T, d] the mixer's input, (c, kr) the latent and rotated key part that it reads."""
    H, n, r, v = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"]
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, H, n + r)
    qn, qr = q[..., :n], q[..., n:]
    qr = rotate_adjacent(qr.transpose(0, 1), positions, mx["rot"]["base"], mx["rot"]["dims"]).transpose(0, 1)
    kn = (c @ w["uk"].T).view(T, H, n)
    val = (c @ w["uv"].T).view(T, H, v)
    s = torch.einsum("ihc,jhc->hij", qn, kn) + torch.einsum("ihc,jc->hij", qr, kr)
    s = s * mx["scale"]
    W = mx.get("mask", {}).get("size") if mx.get("mask") else None
    s = s.masked_fill(~window_mask(T, W)[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhc->ihc", p, val).reshape(T, H * v)
    return o @ w["o"].T


def dense_ff(h, w, act):
    return (act(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def router_choice(h, w_router, correction, top):
    """Scores s = sigmoid(W_r h); the ``top`` experts by s + correction (lowest index among equals);
    returns (experts [T, top], weights [T, top] = their s)."""
    s = torch.sigmoid(h @ w_router.T)
    choice = s + correction
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    return idx, torch.gather(s, 1, idx)


def moe_ff(h, w, mlp, experts=None):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    idx, wt = router_choice(h, w["router"], w["correction"], top)
    if experts is not None:                       # follow a given choice (ties at low precision)
        idx = experts
        wt = torch.gather(torch.sigmoid(h @ w["router"].T), 1, idx)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            we = {k: w[f"e{e}.{k}"] for k in ("gate", "up", "down")}
            out[t] += wt[t, j] * dense_ff(h[t:t + 1], we, silu)[0]
    if mlp.get("shared"):
        out = out + dense_ff(h, {k: w[f"shared.{k}"] for k in ("gate", "up", "down")}, silu)
    return out, idx


def token_side(x, tokens, side_embed, w, layer, dim, eps):
    e = side_embed[tokens][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ w["gate"].T) * e
    y = g @ w["proj"].T
    return rms(y, eps) * w["norm"]


def sub(weights, prefix):
    return {k[len(prefix):]: t for k, t in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, layers_out=None, experts=None, routing_out=None):
    """Logits [T, V] of a whole sequence.  ``layers_out`` (a list) receives the residual stream
    after every layer; ``experts``: {layer: [T, top]} to follow instead of the router's choice."""
    wt = {k: t.to(F) for k, t in weights.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    pos = torch.arange(T)
    x = wt["embed"][tokens]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        assert layer["type"] == "latent_attention"
        p = f"l{i}."
        mx = layer["mixer"]
        h = norm(x, wt[p + "norm1"], eps)
        mw = sub(wt, p + "mix.")
        if mx.get("kv_from") is None:
            kept[i] = latent_kv(h, mw["dkv"], mw["dkv.norm"], eps, mx["kv_rank"], mx["rot"], pos)
            c, kr = kept[i]
        else:
            c, kr = kept[mx["kv_from"]]
        a = latent_attention(h, c, kr, mw, mx, pos)
        x = x + m * norm(a, wt[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm(x, wt[p + "norm2"], eps)
            fw = sub(wt, p + "mlp.")
            if mlp["kind"] == "dense":
                f = dense_ff(h, fw, gelu_tanh)
            else:
                f, idx = moe_ff(h, fw, mlp, None if experts is None else experts.get(i))
                if routing_out is not None:
                    routing_out[i] = idx
            x = x + m * norm(f, wt[p + "norm2b"], eps)
        if cfg.get("token_side"):
            x = x + m * token_side(x, tokens, wt["side.embed"], sub(wt, p + "side."), i, cfg["token_side"]["dim"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm(x, wt["final.norm"], eps) @ wt["head"].T


def greedy(logits_row):
    return int(torch.argmax(logits_row))
