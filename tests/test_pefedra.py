"""The Pefedra design in the engine against the plain implementation (``plain_pefedra``): every
mechanism's kernel alone, whole prompts, decoding through the cache, portions down to two tokens,
mixed batches with pages and slots used again, window edges, far keys, the first tokens, generation."""
from __future__ import annotations

import copy
import math

import numpy as np
import pytest
import torch

import helpers as H
import plain_pefedra as plain


def _mixer(kind, heads, kv, dim, vdim, window, base=10000.0, dims=None, factor=None, scale=None, diff=0.3):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 1.0 / math.sqrt(dim),
         "rot": {"base": base, "dims": dim if dims is None else dims}}
    if factor is not None:
        m["rot"]["scaling"] = {"factor": factor}
    if window is not None:
        m["mask"] = {"size": window}
    if kind == "attention":
        m["diff"] = diff
    return m


def _layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# sizes that no fast kernel takes: odd widths, keys and values of unequal width, grouped heads, a part of
# the head that turns, scaled and unscaled frequencies in both kinds of mixer, a layer without feed-forward
SMALL = {"architecture": "Pefedra", "vocab": 96, "width": 40, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
         "layers": [_layer("attention_2", _mixer("attention_2", 4, 2, 12, 10, 9, dims=8), 56),
                    _layer("attention", _mixer("attention", 6, 3, 6, 14, 21, base=500.0, dims=4, factor=4.0, diff=0.4), 24),
                    _layer("attention_2", _mixer("attention_2", 3, 3, 8, 6, 5, base=100.0, factor=2.0, scale=0.4), None),
                    _layer("attention", _mixer("attention", 2, 1, 10, 8, 13, diff=0.7), 32),
                    _layer("attention_2", _mixer("attention_2", 2, 1, 16, 16, None, dims=6), 16)]}
# sizes that the matrix-unit kernels take in bfloat16 (keys and values of 64, pages of 32)
WIDE = {"architecture": "Pefedra", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
        "layers": [_layer("attention_2", _mixer("attention_2", 4, 2, 64, 64, 40, dims=32), 128),
                   _layer("attention", _mixer("attention", 4, 2, 64, 64, 72, base=20000.0, factor=4.0, diff=0.35), 192),
                   _layer("attention_2", _mixer("attention_2", 2, 2, 64, 64, None, base=1000.0), 64),
                   _layer("attention", _mixer("attention", 2, 1, 32, 64, 33, diff=0.2), 64)]}
# values that are 1 or equal where the other configurations have them apart
ONES = {"architecture": "Pefedra", "vocab": 50, "width": 24, "norm": {"eps": 1e-3}, "embedding": {"scale": 1.0},
        "layers": [_layer("attention", _mixer("attention", 1, 1, 4, 4, 1, dims=2, factor=1.0, diff=0.0), 8),
                   _layer("attention_2", _mixer("attention_2", 1, 1, 2, 2, 1, scale=1.0), 24),
                   _layer("attention_2", _mixer("attention_2", 5, 1, 4, 4, 2), None)]}
CONFIGS = {"small": SMALL, "wide": WIDE, "ones": ONES}
PAGE = {"small": 16, "wide": 32, "ones": 4}


def planted(cfg, seed, gain=3.0, std=0.08):
    """Random tensors with sharper attention (queries, the projection norm's weights), shifts of the size
    of the stream, biases and lambda vectors large enough to matter."""
    from spite_amd.weights.random_init import random_tensors
    t = random_tensors(cfg, seed, std)
    g = torch.Generator().manual_seed(seed)
    for name in list(t):
        if name.endswith(".mix.q") or name.endswith(".mix.q.norm"):
            t[name] = t[name] * gain
        if name.endswith(".shift"):
            t[name] = torch.rand(t[name].shape, generator=g)
        if name.endswith(".b"):
            t[name] = t[name] * 4.0
        if ".mix.l" in name:
            t[name] = torch.randn(t[name].shape, generator=g) * 0.5
        if name.endswith(".mix.g"):
            t[name] = t[name] * 8.0
    return t


def make_model(folder, cfg, seed, dtype, **kw):
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(folder), cfg, seed, dtype=dtype, overrides=planted(cfg, seed, **kw))
    return H.read_weights(str(folder))


def requests(vocab, lengths, seed):
    return {f"r{i}": H.random_tokens(vocab, n, seed + 13 * i) for i, n in enumerate(lengths)}


def plain_rows(cfg, weights, reqs):
    rows = {}
    for rid, toks in reqs.items():
        out = plain.forward(cfg, weights, toks).to(torch.float32).numpy()
        for i in range(len(toks)):
            rows[(rid, i)] = out[i]
    return rows


def engine(folder, dtype, name, **kw):
    from spite_amd import Engine
    kw.setdefault("page_size", PAGE[name])
    kw.setdefault("cache_tokens", 1024)
    kw.setdefault("max_requests", 4)
    return Engine(str(folder), dtype=dtype, device="cuda:0", **kw)


def poison(eng):
    """Every cache row and every state row holds NaN until it is written or cleared."""
    for g in eng.cache.groups:
        for half in g.halves():
            if half is not None and half.numel():
                half.fill_(float("nan"))
    for st in eng.cache.states.values():
        st.fill_(float("nan"))


def scale_of(rows):
    return max(float(np.abs(v).max()) for v in rows.values())


# ------------------------------------------------------------------------------------------ without a GPU
def test_registry_and_tensor_names():
    from spite_amd.config import read_config, PefedraConfig
    from spite_amd.engine.model import Model
    from spite_amd.engine.context import Env
    arch, cfg = read_config(SMALL)
    assert arch.name == "Pefedra" and isinstance(cfg, PefedraConfig)
    assert cfg.layers[1].mixer.rot_factor == 4.0 and cfg.layers[4].mixer.window is None and cfg.layers[2].mlp is None
    model = Model(arch.build_spec(cfg), Env(torch.float32, torch.device("cpu")))
    names = {n: ps.shape for n, ps, _, _ in model.tensor_plan()}
    assert {"embed", "final.norm", "head", "l0.mix.q.norm", "l0.mix.g", "l0.mix.q.b", "l1.mix.lq1", "l1.mix.lk2", "l1.shift",
            "l3.mlp.up", "l4.norm2"} <= set(names)
    assert "l2.norm2" not in names and "l2.mlp.up" not in names and "l1.mix.g" not in names and "l0.mix.lq1" not in names
    assert names["l1.mix.q"] == (6 * 2 * 6, 40) and names["l1.mix.k"] == (3 * 2 * 6, 40) and names["l1.mix.v"] == (3 * 14, 40)
    assert names["l0.mix.q.norm"] == (48,) and names["l0.mix.k.norm"] == (24,) and names["l0.mix.g"] == (4, 40)
    needs = model.cache_needs()
    # a layer's keys and values, then its shift's state row
    assert needs[2].kv.n_kv_heads == 6 and needs[2].kv.value_heads == 3 and needs[2].kv.head_dim == 6 and needs[2].kv.value_dim == 14
    assert needs[2].kv.visibility == "window" and needs[2].kv.span == 21 and needs[8].kv.visibility == "full"
    assert needs[3].kv is None and needs[3].state.shape == (40,)


def test_config_errors_are_collected():
    from spite_amd.config import read_config, ConfigError
    bad = copy.deepcopy(SMALL)
    del bad["width"]
    bad["layers"][0]["mixer"]["kv_heads"] = 3
    bad["layers"][1]["mixer"]["rot"]["dims"] = 7
    del bad["layers"][3]["mixer"]["diff"]
    bad["layers"][4]["type"] = "other"
    with pytest.raises(ConfigError) as e:
        read_config(bad)
    msg = str(e.value)
    assert "width" in msg and "kv_heads" in msg and "rot.dims" in msg and "diff" in msg and "type" in msg


def test_plain_mechanisms():
    ok = plain.window_mask(6, 3)
    assert ok[5].tolist() == [False, False, False, True, True, True] and ok[1].tolist() == [True, True] + [False] * 4
    x = torch.arange(8, dtype=torch.float64).view(1, 1, 8)
    assert torch.equal(plain.turn_halves(x, torch.tensor([0]), 4, 100.0), x)            # position 0 turns nothing
    y = plain.turn_halves(x, torch.tensor([3]), 4, 100.0)
    assert abs(float(y[0, 0, 0]) - (0 * math.cos(3.0) - 2 * math.sin(3.0))) < 1e-12 and torch.equal(y[0, 0, 4:], x[0, 0, 4:])
    assert abs(float(y[0, 0, 3]) - (3 * math.cos(0.3) + 1 * math.sin(0.3))) < 1e-12     # pair 1: 100^(-2/4) = 0.1
    back = plain.turn_halves(y, -torch.tensor([3]), 4, 100.0)
    assert float((back - x).abs().max()) < 1e-12
    assert float((plain.turn_halves(x, torch.tensor([8]), 4, 100.0, divide=4.0) - plain.turn_halves(x, torch.tensor([2]), 4, 100.0)).abs().max()) < 1e-12
    h = torch.tensor([[1.0, 2.0], [3.0, 6.0]], dtype=torch.float64)
    assert plain.token_shift(h, torch.tensor([0.5, 1.0], dtype=torch.float64)).tolist() == [[0.5, 0.0], [2.0, 2.0]]
    assert abs(float(plain.gelu(torch.tensor(1.0, dtype=torch.float64))) - 0.8413447460685429) < 1e-12


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d,lens", [(40, [5, 1, 2, 1]), (256, [1, 1, 1]), (7, [33])])
def test_token_shift_kernel(dtype, d, lens):
    """Portions and single tokens of several requests in two steps: the second step's first tokens read
    what the first step left, a fresh slot reads zeros, nobody reads another slot's row."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(d)
    dt = getattr(torch, dtype)
    n = len(lens)
    slots = [3, 0, 5, 2][:n]
    state = torch.full((6, d), float("nan"))
    state[slots] = 0.0
    state = state.cuda()
    mu = torch.rand(d, generator=g)
    seqs = [torch.randn(2 * L, d, generator=g) for L in lens]
    want = [plain.token_shift(s.double(), mu.double()) for s in seqs]
    for step in range(2):
        x = torch.cat([s[step * L:(step + 1) * L] for s, L in zip(seqs, lens)])
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
        seq_of = torch.tensor([i for i, L in enumerate(lens) for _ in range(L)], dtype=torch.int32)
        y = torch.empty(x.shape, dtype=dt, device="cuda:0")
        hipops.token_shift(x.cuda(), y, mu.cuda(), state, seq_of.cuda(), cu.cuda(), torch.tensor(slots, dtype=torch.int32).cuda())
        ref = torch.cat([w[step * L:(step + 1) * L] for w, L in zip(want, lens)])
        assert float((y.cpu().double() - ref).abs().max()) <= (1e-6 if dtype == "float32" else 2e-2)
    assert torch.equal(state[slots].cpu(), torch.stack([s[-1] for s in seqs]))
    assert bool(torch.isnan(state[[1, 4][:6 - n]]).all())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,n", [("float32", 1000), ("bfloat16", 4096), ("bfloat16", 37)])
def test_activation_and_scaled_embedding(dtype, n):
    from spite_amd.csrc import hipops
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(n)
    x = (torch.randn(n, generator=g) * 3).to(dt)
    y = x.cuda().clone()
    hipops.act_rows(y, "gelu")
    assert float((y.cpu().double() - plain.gelu(x.double())).abs().max()) <= (1e-6 if dtype == "float32" else 2e-2)
    table = torch.randn(11, 24, generator=g).to(dt)
    ids = torch.tensor([3, 10, 0, 3], dtype=torch.int32)
    h = torch.empty(4, 24, device="cuda:0")
    hipops.embed(ids.cuda(), table.cuda(), h, 12.5)
    assert torch.equal(h.cpu(), table[ids.long()].float() * 12.5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,M,N,K", [("float32", 9, 24, 40), ("bfloat16", 5, 64, 128), ("bfloat16", 100, 64, 128), ("bfloat16", 300, 1024, 256),
                                         ("bfloat16", 200, 48, 72), ("bfloat16", 7, 20, 40), ("bfloat16", 40, 96, 64)])
@pytest.mark.parametrize("act", ["gelu", "gelu_tanh", "silu"])
def test_products_with_an_activation(dtype, M, N, K, act):
    """act(x W^T) through every product kernel (in the epilogue where the kernel has one, else in a pass after it),
    and a plain product right after it on the same thread."""
    from spite_amd.parts.linear import linear, Weight
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(M + N)
    x = (torch.randn(M, K, generator=g)).to(dt)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K) * 2).to(dt)
    y = torch.empty(M, N, dtype=dt, device="cuda:0")
    W = Weight(w.cuda())
    linear(x.cuda(), W, y, act=act)
    z = x.double() @ w.double().T
    want = {"gelu": plain.gelu, "gelu_tanh": lambda v: 0.5 * v * (1 + torch.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))),
            "silu": lambda v: v * torch.sigmoid(v)}[act](z)
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert float((y.cpu().double() - want).abs().max()) <= tol * max(1.0, float(want.abs().max()))
    linear(x.cuda(), W, y)
    assert float((y.cpu().double() - z).abs().max()) <= tol * max(1.0, float(z.abs().max()))


def _paged(rows, ps, perm, n_pages, heads, width, transposed):
    """rows[i]: [t, heads, width] of request i -> pages (NaN where nothing was written) and the block table."""
    n = len(rows)
    table = torch.full((n, max(-(-r.shape[0] // ps) for r in rows) + 1), -1, dtype=torch.int32)
    pages = torch.full((n_pages, heads, width, ps) if transposed else (n_pages, heads, ps, width), float("nan"))
    for i, r in enumerate(rows):
        for b in range(-(-r.shape[0] // ps)):
            pg = perm[(i, b)]
            table[i, b] = pg
            chunk = r[b * ps:(b + 1) * ps]                      # [c, heads, width]
            if transposed:
                pages[pg, :, :, :chunk.shape[0]] = chunk.permute(1, 2, 0)
            else:
                pages[pg, :, :chunk.shape[0]] = chunk.permute(1, 0, 2)
    return pages, table


@pytest.mark.gpu
@pytest.mark.parametrize("HQ,GK,GV,D,Vd,ps,vis,span", [(6, 3, 3, 12, 10, 8, "window", 9), (12, 6, 3, 6, 14, 16, "window", 21),
                                                      (2, 2, 1, 32, 64, 4, "full", 0), (5, 1, 1, 4, 4, 4, "window", 1),
                                                      (4, 4, 2, 64, 64, 32, "window", 70)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_kernel(HQ, GK, GV, D, Vd, ps, vis, span, dtype):
    """Keys and values of unequal width and head count on a paged cache with scattered pages: single tokens
    beside portions, far keys, windows that end inside a page."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(HQ * D + Vd)
    dt = getattr(torch, dtype)
    starts, lens = [70, 0, 23, 0, 41], [1, 17, 40, 1, 2]
    totals = [s + c for s, c in zip(starts, lens)]
    keys = [torch.randn(t, GK, D, generator=g).to(dt).float() for t in totals]
    vals = [torch.randn(t, GV, Vd, generator=g).to(dt).float() for t in totals]
    n_pages = sum(-(-t // ps) for t in totals) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    perm = {(i, b): order.pop() for i, t in enumerate(totals) for b in range(-(-t // ps))}
    k_pages, table = _paged(keys, ps, perm, n_pages, GK, D, False)
    v_pages, _ = _paged(vals, ps, perm, n_pages, GV, Vd, True)
    T = sum(lens)
    q = (torch.randn(T, HQ, D, generator=g) * 2).to(dt).float()
    positions = torch.tensor([s + j for s, c in zip(starts, lens) for j in range(c)], dtype=torch.int32)
    seq = torch.tensor([i for i, c in enumerate(lens) for _ in range(c)], dtype=torch.int32)
    scale = 0.7 / math.sqrt(D)
    want = torch.zeros(T, HQ, Vd, dtype=torch.float64)
    for t in range(T):
        p, i = int(positions[t]), int(seq[t])
        lo = 0 if vis == "full" else max(0, p - span + 1)
        for h in range(HQ):
            gk = h // (HQ // GK)
            s = (keys[i][lo:p + 1, gk].double() @ q[t, h].double()) * scale
            want[t, h] = torch.softmax(s, 0) @ vals[i][lo:p + 1, gk % GV].double()
    tiled = dtype == "bfloat16" and D == Vd and D % 32 == 0 and ps % 32 == 0
    kp, vp = k_pages.to(dt).cuda(), v_pages.to(dt).cuda()
    if tiled:
        kp, vp = hipops.kv_operand_order(torch.nan_to_num(kp), torch.nan_to_num(vp))
    for out_dt in ({dt, torch.float32}):
        out = torch.full((T, HQ * Vd), float("nan"), dtype=out_dt, device="cuda:0")
        hipops.attn_wide(q.to(dt).cuda().view(T, HQ * D), kp, vp, out, positions.cuda(), seq.cuda(), table.cuda(), T, HQ, GK, GV, D, Vd,
                         ps, vis, span, scale, k_tiled=tiled, v_tiled=tiled)
        tol = 2e-5 if out_dt == torch.float32 else 2e-2
        assert float((out.cpu().double().view(T, HQ, Vd) - want).abs().max()) < tol * max(1.0, float(want.abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("HQ,GK,GV,D,Vd,rot,ps,norm,turn_v,extra", [(4, 2, 2, 12, 10, 8, 8, True, True, 4), (12, 6, 3, 6, 14, 4, 16, False, False, 0),
                                                                      (2, 1, 1, 64, 64, 64, 32, True, True, 14), (3, 3, 3, 5, 7, 0, 4, False, False, 1)])
def test_projection_to_cache_kernel(dtype, HQ, GK, GV, D, Vd, rot, ps, norm, turn_v, extra):
    """Bias, the norm over the whole q and k parts, the rotation of a head's leading part, turned values,
    and the places of keys and values in their pages; columns behind q, k and v are left alone."""
    from spite_amd.csrc import hipops
    if turn_v and Vd % 2:
        pytest.skip("values turn in pairs")
    g = torch.Generator().manual_seed(D + Vd)
    dt = getattr(torch, dtype)
    T, eps, base = 9, 1e-4, 300.0
    n = (HQ + GK) * D + GV * Vd
    row = torch.randn(T, n + extra, generator=g).to(dt)
    bias = torch.randn(n, generator=g)
    wq, wk = torch.rand(HQ * D, generator=g) + 0.5, torch.rand(GK * D, generator=g) + 0.5
    positions = torch.tensor([0, 1, 2, 100, 101, 7, 200, 5, 6], dtype=torch.int32)
    slots = torch.tensor([ps * 2 + 0, ps * 2 + 1, ps * 2 + 2, 1, 2, ps * 3 + ps - 1, 0, -1, ps + 3], dtype=torch.int32)
    x = row[:, :n].double() + bias.double()
    qq, kk, vv = x[:, :HQ * D], x[:, HQ * D:(HQ + GK) * D], x[:, (HQ + GK) * D:]
    if norm:
        qq, kk = plain.norm(qq, wq.double(), eps), plain.norm(kk, wk.double(), eps)
    qq = plain.turn_halves(qq.reshape(T, HQ, D), positions, rot, base, 2.0)
    kk = plain.turn_halves(kk.reshape(T, GK, D), positions, rot, base, 2.0)
    vv = vv.reshape(T, GV, Vd)
    if turn_v:
        vv = plain.turn_halves(vv, positions, Vd, base)
    f = lambda n_turn, div: torch.tensor([base ** (-2.0 * i / n_turn) / div for i in range(n_turn // 2)], dtype=torch.float64).float().cuda()
    n_pages = 5
    tiled = dtype == "bfloat16" and D == Vd and D % 32 == 0 and ps % 32 == 0
    kp = torch.zeros(n_pages, GK, ps, D, dtype=dt, device="cuda:0")
    vp = torch.zeros(n_pages, GV, Vd, ps, dtype=dt, device="cuda:0")
    q_out = torch.empty(T, HQ * D, dtype=dt, device="cuda:0")
    dev_row = row.cuda()
    hipops.qkv_prepare(dev_row, q_out, kp, vp, positions.cuda(), slots.cuda(), HQ, GK, GV, D, Vd, ps, bias=bias.cuda(),
                       norm_q=wq.cuda() if norm else None, norm_k=wk.cuda() if norm else None, eps=eps,
                       inv_freq=f(rot, 2.0) if rot else None, rot=rot, inv_freq_v=f(Vd, 1.0) if turn_v else None, k_tiled=tiled, v_tiled=tiled)
    assert torch.equal(dev_row.cpu(), row)
    tol = 2e-5 if dtype == "float32" else 3e-2
    assert float((q_out.cpu().double().view(T, HQ, D) - qq).abs().max()) < tol * max(1.0, float(qq.abs().max()))
    want_k, want_v = torch.zeros(n_pages, GK, ps, D, dtype=torch.float64), torch.zeros(n_pages, GV, Vd, ps, dtype=torch.float64)
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            want_k[s // ps, :, s % ps] = kk[t]
            want_v[s // ps, :, :, s % ps] = vv[t]
    if tiled:
        a, b = hipops.kv_operand_order(want_k.to(dt).cuda(), want_v.to(dt).cuda())
        want_k, want_v = a.cpu().double(), b.cpu().double()
    assert float((kp.cpu().double() - want_k).abs().max()) < tol * max(1.0, float(kk.abs().max()))
    assert float((vp.cpu().double() - want_v).abs().max()) < tol * max(1.0, float(vv.abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,ps", [("float32", 8), ("bfloat16", 32)])
def test_keys_stored_wider_than_they_are(dtype, ps):
    """Queries and keys of 32 elements stored 64 wide: their own elements first, zeros behind them, also where
    the page held something else before."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(5)
    dt = getattr(torch, dtype)
    T, HQ, GK, GV, D, Vd, Dp = 6, 4, 2, 1, 32, 64, 64
    n = (HQ + GK) * D + GV * Vd
    row = torch.randn(T, n, generator=g).to(dt)
    positions = torch.arange(T, dtype=torch.int32)
    slots = torch.tensor([ps + 3, ps + 4, 0, 1, 2 * ps - 1, 2 * ps], dtype=torch.int32)
    tiled = dtype == "bfloat16"
    kp = torch.full((3, GK, ps, Dp), float("nan"), dtype=dt, device="cuda:0")
    vp = torch.zeros(3, GV, Vd, ps, dtype=dt, device="cuda:0")
    q_out = torch.full((T, HQ * Dp), float("nan"), dtype=dt, device="cuda:0")
    hipops.qkv_prepare(row.cuda(), q_out, kp, vp, positions.cuda(), slots.cuda(), HQ, GK, GV, D, Vd, ps, k_tiled=tiled, v_tiled=tiled,
                       stored_dim=Dp)
    want_q = torch.zeros(T, HQ, Dp, dtype=dt)
    want_q[:, :, :D] = row[:, :HQ * D].view(T, HQ, D)
    assert torch.equal(q_out.cpu().view(T, HQ, Dp), want_q)
    want_k = torch.full((3, GK, ps, Dp), float("nan"), dtype=dt)
    for t in range(T):
        sl = int(slots[t])
        want_k[sl // ps, :, sl % ps, :D] = row[t, HQ * D:(HQ + GK) * D].view(GK, D)
        want_k[sl // ps, :, sl % ps, D:] = 0
    if tiled:
        want_k, _ = hipops.kv_operand_order(want_k.cuda(), vp)
    assert torch.equal(torch.nan_to_num(kp.cpu(), nan=-7.0), torch.nan_to_num(want_k.cpu(), nan=-7.0))


@pytest.mark.gpu
@pytest.mark.parametrize("hd,HQ,GK,GV", [(64, 8, 4, 2), (128, 4, 2, 1), (64, 2, 2, 2)])
def test_matrix_unit_kernels_with_fewer_value_heads(hd, HQ, GK, GV):
    """The prefill and decode kernels of the matrix units with value heads shared by several key heads, against
    the plain kernel on the same pages: portions, and single tokens far into their requests."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(hd + GV)
    ps, dev = 32, "cuda:0"
    starts, lens = [70, 0, 23], [40, 17, 100]
    totals = [s + c for s, c in zip(starts, lens)]
    n_pages = sum(-(-t // ps) for t in totals) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((3, 8), -1, dtype=torch.int32)
    for i, t in enumerate(totals):
        for b in range(-(-t // ps)):
            table[i, b] = order.pop()
    kp, vp = hipops.kv_operand_order(torch.randn(n_pages, GK, ps, hd, generator=g).bfloat16().to(dev),
                                     torch.randn(n_pages, GV, hd, ps, generator=g).bfloat16().to(dev))
    scale = 1.0 / math.sqrt(hd)
    for decode in (False, True):
        ln = [1, 1, 1] if decode else lens
        st = [t - 1 for t in totals] if decode else starts
        T = sum(ln)
        q = (torch.randn(T, HQ * hd, generator=g) * 1.5).bfloat16().to(dev)
        positions = torch.tensor([s + j for s, c in zip(st, ln) for j in range(c)], dtype=torch.int32, device=dev)
        seq = torch.tensor([i for i, c in enumerate(ln) for _ in range(c)], dtype=torch.int32, device=dev)
        cu = torch.tensor(np.concatenate([[0], np.cumsum(ln)]), dtype=torch.int32, device=dev)
        ref = torch.empty(T, HQ * hd, device=dev)
        hipops.attn_wide(q, kp, vp, ref, positions, seq, table.to(dev), T, HQ, GK, GV, hd, hd, ps, "window", 90, scale, k_tiled=True, v_tiled=True)
        out = torch.full((T, HQ * hd), float("nan"), dtype=torch.bfloat16, device=dev)
        if decode:
            n_splits = 2
            scratch = torch.empty(hipops.attn_decode_workspace(T, HQ, hd, n_splits) // 4, device=dev)
            hipops.attn_decode(q, kp, vp, out, scratch, positions, seq, table.to(dev), T, HQ, GK, hd, ps, "window", 90, scale, n_splits,
                               value_heads=GV)
        else:
            hipops.attn_prefill(q, kp, vp, out, positions, cu, np.asarray(ln), table.to(dev), HQ, GK, hd, ps, "window", 90, scale,
                                value_heads=GV)
        assert float((out.float() - ref).abs().max()) < 0.02 * float(ref.abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H_,Vd", [(3, 14), (4, 64), (1, 130)])
def test_attention_finish_kernel(dtype, H_, Vd):
    """Two maps combined and normed; values turned back with a gate taken from columns of a wider matrix."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(Vd)
    dt = getattr(torch, dtype)
    T, eps, lam, post, base = 7, 1e-3, 0.37, 0.6, 200.0
    tol = 1e-5 if dtype == "float32" else 2e-2
    for in_dt in {torch.float32, dt}:
        a = torch.randn(T, 2, H_, Vd, generator=g).to(in_dt)
        out = torch.empty(T, H_ * Vd, dtype=dt, device="cuda:0")
        hipops.attn_finish(a.cuda().view(T, -1), out, None, H_, Vd, maps=2, lam=lam, eps=eps, post=post)
        want = plain.unit_rms(a[:, 0].double() - lam * a[:, 1].double(), eps) * post
        assert float((out.cpu().double().view(T, H_, Vd) - want).abs().max()) < tol * 4
    a = torch.randn(T, H_, Vd, generator=g).to(dt)
    wide = torch.randn(T, 5 + H_ + 2, generator=g).to(dt)
    positions = torch.tensor([0, 1, 5, 90, 64, 3, 2], dtype=torch.int32)
    fv = torch.tensor([base ** (-2.0 * i / Vd) for i in range(Vd // 2)], dtype=torch.float64).float().cuda()
    out = torch.empty(T, H_ * Vd, dtype=dt, device="cuda:0")
    hipops.attn_finish(a.cuda().view(T, -1), out, positions.cuda(), H_, Vd, inv_freq_v=fv, gate=wide.cuda()[:, 5:5 + H_])
    want = plain.turn_halves(a.double(), -positions, Vd, base) * torch.sigmoid(wide[:, 5:5 + H_].double())[:, :, None]
    assert float((out.cpu().double().view(T, H_, Vd) - want).abs().max()) < tol * 4


# ------------------------------------------------------------------------------------------ the model in the engine
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            folder = tmp_path_factory.mktemp(f"pefedra_{name}_{dtype}")
            # milder weights for the 16-bit runs: with very sharp attention the rounding of a score moves the
            # logits by more than any tolerance that would still tell a wrong key
            kw = {} if dtype == "float32" else dict(gain=1.5, std=0.05)
            made[(name, dtype)] = (folder, make_model(folder, CONFIGS[name], seed=11 + len(name), dtype=dtype, **kw))
        return made[(name, dtype)]
    return get


LENGTHS = {"small": [1, 45, 23, 60, 2, 31, 17], "wide": [90, 1, 140, 33, 75], "ones": [30, 1, 44, 9]}


@pytest.mark.gpu
def test_every_layer_against_plain(models):
    """The stream after each layer of a whole prompt, in true 32-bit."""
    from spite_amd.engine.engine import StepEntry, StepMeta
    cfg = SMALL
    folder, weights = models("small", "float32")
    toks = H.random_tokens(cfg["vocab"], 37, 3)
    eng = engine(folder, "float32", "small")
    slot = eng.admit()
    eng.cache.reserve_all([(slot, len(toks))])
    meta = StepMeta(eng, [StepEntry(slot, toks, [0])])
    eng._step_ws.reset()
    m, state = eng.model, {}
    for u in range(m.n_units()):
        kind, _, i, _ = m._units[u]
        m.run_units(u, u + 1, state, meta.ctx, eng.cache, meta, eng._arenas, eng._step_ws)
        if kind == "stage" and m._units[u + 1][2] != i:
            x = state["h"].clone()
            for p in state["pending"]:
                x += p[:x.shape[0]]
            ref = plain.forward(cfg, weights, toks, upto=i + 1)
            assert float((x.cpu().double() - ref).abs().max()) <= 2e-5 * float(ref.abs().max()), f"layer {i}"


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["small", "wide", "ones"])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_float32_against_plain(models, name, schedule):
    """True 32-bit: every schedule gives the plain implementation's logits at every position.  Pools and state
    rows start poisoned and are small: pages and slots are used again in the mixed schedule."""
    cfg = CONFIGS[name]
    folder, weights = models(name, "float32")
    reqs = requests(cfg["vocab"], LENGTHS[name], 5)
    ref = plain_rows(cfg, weights, reqs)
    steps = {"whole": H.schedule_whole, "tail": lambda r: H.schedule_tail_one_by_one(r, tail=28),
             "portions": H.schedule_portions, "mixed": lambda r: H.schedule_mixed(r, seed=3, max_live=4)}[schedule](reqs)
    eng = engine(folder, "float32", name, cache_tokens=4 * (max(LENGTHS[name]) + PAGE[name]))
    poison(eng)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
    err, where = H.max_diff(got, ref)
    assert err <= 2e-4 * scale_of(ref), f"{err} at {where} (scale {scale_of(ref)})"
    assert all(eng.cache.free_pages(g) == eng.cache.total_pages(g) for g in range(eng.cache.n_groups()))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["small", "wide"])
def test_bfloat16_against_plain_and_itself(models, name):
    """bfloat16 through the serving kernels: whole prompts against the plain implementation, then the other
    schedules against the whole prompts."""
    cfg = CONFIGS[name]
    folder, weights = models(name, "bfloat16")
    reqs = requests(cfg["vocab"], LENGTHS[name], 8)
    eng = engine(folder, "bfloat16", name, cache_tokens=4 * (max(LENGTHS[name]) + PAGE[name]))
    poison(eng)
    whole = H.schedule_whole(reqs)
    rows = H.collect(whole, H.run_trace_inprocess(eng, whole), cfg["vocab"])
    ref = plain_rows(cfg, weights, reqs)
    scale = scale_of(ref)
    err, where = H.max_diff(rows, ref)
    assert err <= 0.05 * scale, f"{err} at {where} (scale {scale})"
    for steps in (H.schedule_tail_one_by_one(reqs, tail=28), H.schedule_portions(reqs), H.schedule_mixed(reqs, seed=4, max_live=4)):
        got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
        err, where = H.max_diff(got, rows)
        assert err <= 0.05 * scale, f"{err} at {where} (scale {scale})"


def _one_layer(kind, window, wide=False):
    if wide:
        mix = _mixer(kind, 4, 2, 64, 64, window, dims=32)
    else:
        mix = _mixer(kind, 3, 3, 12, 10, window, dims=8)
    return {"architecture": "Pefedra", "vocab": 64, "width": 128 if wide else 40, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
            "layers": [_layer(kind, mix, 32)]}


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["attention", "attention_2"])
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
@pytest.mark.parametrize("decoded", [False, True])
def test_window_edges(tmp_path, kind, dtype, wide, decoded):
    """One layer, a window of 11 over pages of 8 (32 in bfloat16).  The key at j is made of the tokens j and j - 1
    (the shift), so the logits at i do not move at all when token i - 12 changes and move when token i - 11
    does; in a prompt and when the positions are decoded one by one."""
    W = 11
    cfg = _one_layer(kind, W, wide=wide)
    make_model(tmp_path, cfg, seed=2, dtype=dtype, gain=3.0)
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=256, max_requests=2, device="cuda:0")
    base = H.random_tokens(64, 48, 1)

    def run(toks):
        reqs = {"a": toks}
        steps = H.schedule_tail_one_by_one(reqs, tail=30) if decoded else H.schedule_whole(reqs)
        return H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    ref = run(base)
    for i in (20, 31, 47):
        outside, inside = list(base), list(base)
        outside[i - W - 1] = (base[i - W - 1] + 7) % 64
        inside[i - W] = (base[i - W] + 7) % 64
        a, b = run(outside)[("a", i)], run(inside)[("a", i)]
        assert np.array_equal(a, ref[("a", i)]), f"position {i} sees the token {W + 1} back"
        assert float(np.abs(b - ref[("a", i)]).max()) > 1e-4 * float(np.abs(ref[("a", i)]).max()), f"position {i} misses the window's first key"


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_far_keys_and_long_decoding(tmp_path, kind):
    """Every earlier key is read (no window), attention is sharp, the prompt spans many small pages and more
    than a hundred tokens are decoded one by one: a lost key anywhere shows against the plain implementation."""
    cfg = _one_layer(kind, None)
    weights = make_model(tmp_path, cfg, seed=4, dtype="float32", gain=6.0)
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype="float32", page_size=8, cache_tokens=512, max_requests=2, device="cuda:0")
    poison(eng)
    reqs = {"a": H.random_tokens(64, 330, 6)}
    ref = plain_rows(cfg, weights, reqs)
    steps = H.schedule_tail_one_by_one(reqs, tail=130)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    err, where = H.max_diff(got, ref)
    assert err <= 2e-4 * scale_of(ref), f"{err} at {where}"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
def test_one_far_key_stands_out(tmp_path, dtype, wide):
    """One token, seen once at position 3, whose key every later query of the first score map scores far above all
    others (a query bias on an element that does not turn, and a key row along that token's normed embedding):
    hundreds of keys later, in the prompt and in decoded tokens, the result is that key's value.  Without it the
    logits are others altogether, which the test shows first."""
    cfg = _one_layer("attention", None, wide=wide)
    cfg["layers"][0]["mixer"]["scale"] = 0.25
    mx = cfg["layers"][0]["mixer"]
    Hh, G, D, d, special, gain = mx["heads"], mx["kv_heads"], mx["dim"], cfg["width"], 7, 5.0
    t = planted(cfg, 3, gain=1.0)
    t["l0.shift"] = torch.zeros(d)
    h = t["embed"][special].double() * cfg["embedding"]["scale"]
    h = plain.norm(h, t["l0.norm1"].double(), cfg["norm"]["eps"])
    u = (h / h.norm()).float()
    c0 = D - 1                                                     # behind the elements that turn
    for hh in range(Hh):
        t["l0.mix.q"][(hh * 2) * D + c0] = 0.0
        t["l0.mix.q.b"][(hh * 2) * D + c0] = gain
    for g in range(G):
        t["l0.mix.k"][(g * 2) * D + c0] = gain * u
        t["l0.mix.k.b"][(g * 2) * D + c0] = 0.0
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(tmp_path), cfg, 3, dtype=dtype, overrides=t)
    weights = H.read_weights(str(tmp_path))
    toks = [x if x != special else special + 1 for x in H.random_tokens(64, 330, 9)]
    toks[3] = special
    without = list(toks)
    without[3] = special + 1
    ref, other = plain.forward(cfg, weights, toks), plain.forward(cfg, weights, without)
    scale = float(ref.abs().max())
    assert float((ref[300:] - other[300:]).abs().max()) > 0.2 * scale          # the far key decides
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=512, max_requests=2, device="cuda:0")
    if wide:
        assert not eng.slow_paths, eng.slow_paths
    poison(eng)
    steps = H.schedule_tail_one_by_one({"a": toks}, tail=40)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    rows = {("a", i): ref[i].float().numpy() for i in range(len(toks))}
    err, where = H.max_diff(got, rows)
    assert err <= (2e-4 if dtype == "float32" else 0.05) * scale, f"{err} at {where} (scale {scale})"


@pytest.mark.gpu
def test_a_slot_used_again_starts_from_zeros(models):
    """A request that takes the slot (and the pages) of a finished one reads nothing of it: its first
    token's shift sees zeros, whatever the slot's state row held."""
    cfg = CONFIGS["small"]
    folder, weights = models("small", "float32")
    eng = engine(folder, "float32", "small", max_requests=1, cache_tokens=64)
    a, b = H.random_tokens(cfg["vocab"], 40, 1), H.random_tokens(cfg["vocab"], 25, 2)
    for toks in (a, b, a):
        steps = H.schedule_portions({"x": toks}, sizes=(1, 2, 9))
        got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
        ref = plain_rows(cfg, weights, {"x": toks})
        err, where = H.max_diff(got, ref)
        assert err <= 2e-4 * scale_of(ref), f"{err} at {where}"


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["small", "wide"])
def test_greedy_generation(models, name):
    """Through the engine's own entry point and scheduler: prompts of unequal length, more new tokens than the
    windows are long, in true 32-bit: the plain implementation's greedy tokens."""
    cfg = CONFIGS[name]
    folder, weights = models(name, "float32")
    prompts = [H.random_tokens(cfg["vocab"], n, 40 + n) for n in (1, 19, 7)]
    eng = engine(folder, "float32", name, cache_tokens=512, max_batch_tokens=16)
    n_new = 40 if name == "small" else 12
    got = eng.generate(prompts, max_tokens=n_new, temperature=0.0)
    for p, g in zip(prompts, got):
        toks = list(p)
        for k in range(n_new):
            last = plain.forward(cfg, weights, toks)[-1]
            top = torch.topk(last, 2).values
            if float(top[0] - top[1]) < 1e-3 * float(last.abs().max()):
                break                                              # a tie at 32-bit precision: what follows may differ
            assert g[k] == plain.greedy(last), f"token {k} of a prompt of {len(p)}"
            toks.append(g[k])
        assert k >= 5


@pytest.mark.gpu
def test_decode_steps_replay_graphs(models):
    """Decode steps of one shape are captured and replayed; every replay gives the eager logits (the shift's
    state rows move on inside the graph)."""
    cfg = CONFIGS["wide"]
    folder, _ = models("wide", "bfloat16")
    reqs = requests(cfg["vocab"], [40, 41], 21)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:20], "want": [19]} for r, t in reqs.items()], "end": []}]
    steps += [{"step": 1 + i, "entries": [{"id": r, "tokens": [t[20 + i]], "want": [0]} for r, t in reqs.items()], "end": []} for i in range(20)]
    outs = []
    for graphs in (False, True):
        eng = engine(folder, "bfloat16", "wide", graphs=graphs)
        outs.append(H.run_trace_inprocess(eng, copy.deepcopy(steps)))
        assert (eng.graph_replays > 10) == graphs
    for k in outs[0]:
        assert np.array_equal(outs[0][k], outs[1][k]), f"step {k}"


def random_config(seed, aligned=False):
    """A configuration drawn from a seed: layer count and order, heads, sizes, windows, bases, scaling and
    constants all vary; now and then a value is 1 or sizes are odd.  ``aligned``: sizes in multiples of 8,
    32 and 64, which the bfloat16 runs take on the matrix units in one kernel or another."""
    rng = np.random.RandomState(seed)
    pick = lambda *xs: xs[rng.randint(len(xs))]
    layers = []
    for _ in range(int(pick(1, 2, 3, 5))):
        kind = pick("attention", "attention_2")
        kv = int(pick(1, 2, 3))
        heads = kv * int(pick(1, 2, 4))
        if aligned:
            dim = int(pick(32, 64, 64, 128))
            vdim = int(pick(dim, dim, 32, 64))
            dims = int(pick(dim, dim // 2, 16))
            window = pick(None, 24, 72, 100)
            ff = pick(None, 64, 128, 200)
        else:
            dim = int(pick(2, 6, 8, 12, 16))
            vdim = int(pick(2, 4, 6, 10, 16)) if kind == "attention_2" else int(pick(3, 4, 5, 10, 16))      # (one value a head leaves a sign only)
            dims = int(pick(*[x for x in (2, 4, 6, 8, 12, 16) if x <= dim]))
            window = pick(None, 1, 2, 7, 16, 33, 64)
            ff = pick(None, 8, 20, 32)
        mix = _mixer(kind, heads, kv, dim, vdim, window, base=float(pick(100.0, 10000.0, 1e6)), dims=dims,
                     factor=pick(None, 1.0, 2.0, 4.0), scale=float(pick(0.1, 0.25, 0.5)), diff=float(pick(0.0, 0.2, 0.45, 0.8)))
        layers.append(_layer(kind, mix, ff))
    return {"architecture": "Pefedra", "vocab": int(pick(50, 128, 257)), "width": int(pick(64, 128, 192)) if aligned else int(pick(24, 37, 48, 64)),
            "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "embedding": {"scale": float(pick(1.0, 4.0, 10.0))}, "layers": layers}


@pytest.mark.gpu
@pytest.mark.parametrize("seed", list(range(8)) + list(range(100, 108)))
def test_random_configurations(tmp_path, seed):
    """Whatever the configuration says: true 32-bit against the plain implementation, whole prompts and a mixed
    schedule through small pages; then bfloat16 against itself across schedules and, loosely, against the plain
    implementation."""
    cfg = random_config(seed, aligned=seed >= 100)
    page = int(np.random.RandomState(seed + 100).choice([4, 16, 32, 64]))
    weights = make_model(tmp_path / "f32", cfg, seed=seed, dtype="float32", gain=2.0)
    reqs = requests(cfg["vocab"], [41, 1, 70, 2, 19], seed)
    ref = plain_rows(cfg, weights, reqs)
    from spite_amd import Engine
    eng = Engine(str(tmp_path / "f32"), dtype="float32", page_size=page, cache_tokens=4 * (70 + page), max_requests=4, device="cuda:0")
    poison(eng)
    for steps in (H.schedule_whole(reqs), H.schedule_mixed(reqs, seed=seed, max_live=4)):
        got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
        err, where = H.max_diff(got, ref)
        assert err <= 3e-4 * scale_of(ref), f"{err} at {where} (scale {scale_of(ref)}): {cfg}"
    del eng
    weights = make_model(tmp_path / "bf16", cfg, seed=seed, dtype="bfloat16", gain=1.5, std=0.05)
    eng = Engine(str(tmp_path / "bf16"), dtype="bfloat16", page_size=page, cache_tokens=4 * (70 + page), max_requests=4, device="cuda:0")
    poison(eng)
    whole = H.schedule_whole(reqs)
    rows = H.collect(whole, H.run_trace_inprocess(eng, whole), cfg["vocab"])
    ref = plain_rows(cfg, weights, reqs)
    scale = scale_of(ref)
    err, where = H.max_diff(rows, ref)
    assert err <= 0.08 * scale, f"{err} at {where} (scale {scale}): {cfg}"
    steps = H.schedule_mixed(reqs, seed=seed + 1, max_live=4)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
    err, where = H.max_diff(got, rows)
    assert err <= 0.08 * scale, f"{err} at {where} (scale {scale}): {cfg}"


@pytest.mark.gpu
def test_replay_program(models):
    """The replay program on a model folder, as a child process: a mixed schedule in true 32-bit gives the
    plain implementation's logits."""
    cfg = CONFIGS["small"]
    folder, weights = models("small", "float32")
    reqs = requests(cfg["vocab"], [30, 1, 47, 12, 22], 77)
    steps = H.schedule_mixed(reqs, seed=9, max_live=4)
    out = H.run_trace_program(str(folder), "float32", steps, max_tokens=4 * 64, extra=["--page-size", "16", "--max-requests", "4"])
    got = H.collect(steps, out, cfg["vocab"])
    ref = plain_rows(cfg, weights, reqs)
    err, where = H.max_diff(got, ref)
    assert err <= 2e-4 * scale_of(ref), f"{err} at {where}"
