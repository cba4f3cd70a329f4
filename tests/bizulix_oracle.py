"""Plain, slow float64 implementation of the Bizulix design, one function per mechanism.

It is the yardstick of the Bizulix tests and shares no code with the engine: it takes a config dict (the
layout of config.json) and a dict name -> torch tensor, runs one whole sequence at a time, and keeps no
cache (every position is recomputed from the full prefix).

Notation: n tokens, width E. Linear weights are [out, in]; y = x @ W.T.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def query_temperature(n, coef, every):
    p = torch.arange(n, dtype=F64)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def softcap(z, cap):
    return cap * torch.tanh(z / cap)


def attention_mixer(h, W, m):
    """h [n, E]; W: q, k, v, o. Causal softmax attention with grouped key/value heads, a position-dependent
    query multiplier and tanh-capped scores; no rotation."""
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].T).view(n, H, D)
    k = (h @ W["k"].T).view(n, G, D)
    v = (h @ W["v"].T).view(n, G, Dv)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(n, qt["coef"], qt["every"])[:, None, None]
    out = torch.zeros(n, H, Dv, dtype=F64)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if m.get("softcap"):
            s = softcap(s, m["softcap"])
        s = s.masked_fill(~mask, -math.inf)
        out[:, hd] = torch.softmax(s, -1) @ v[:, g]
    return out.reshape(n, H * Dv) @ W["o"].T


def rotate_half(x, dims, base):
    """x [n, heads, D]: dimension i < dims/2 is paired with i + dims/2; the rest passes unchanged."""
    n = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = torch.arange(n, dtype=F64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def retention_mixer(h, W, m, eps):
    """Linear attention with a fixed per-head decay, token by token: S <- d S + k v^T, o = S^T q."""
    n = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].T).view(n, H, D)
    k = (h @ W["k"].T).view(n, H, D)
    v = (h @ W["v"].T).view(n, H, Dv)
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, rot["dims"], rot["base"])
        k = rotate_half(k, rot["dims"], rot["base"])
    k = k * D ** -0.5
    o = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(n):
            S = m["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps).reshape(n, H * Dv)
    return (o * silu(h @ W["g"].T)) @ W["o"].T


def expert(h, W):
    return (silu(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def moe_ff(h, W, mlp):
    """W: router, router.b, e<i>.{gate,up,down}, shared.{gate,up,down,sg}."""
    n = h.shape[0]
    X, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ W["router"].T + W["router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    wt = torch.softmax(val, -1)
    y = torch.zeros(n, W["e0.down"].shape[0], dtype=F64)
    for t in range(n):
        for j in range(top):
            e = int(idx[t, j])
            y[t] += wt[t, j] * expert(h[t:t + 1], {k: W[f"e{e}.{k}"] for k in ("gate", "up", "down")})[0]
    if mlp.get("shared"):
        sh = expert(h, {k: W[f"shared.{k}"] for k in ("gate", "up", "down")})
        y = y + torch.sigmoid(h @ W["shared.sg"].T) * sh
    return y


def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in tensors.items() if k.startswith(prefix)}


def layer_runs(cfg):
    """Layer indices in the order they run, with the pass number of looped layers."""
    L = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, 0, False) for i in range(L)]
    a, b, t = loop["start"], loop["stop"], loop["times"]
    runs = [(i, 0, False) for i in range(a)]
    for p in range(t):
        runs += [(i, p, i == a) for i in range(a, b)]
    return runs + [(i, 0, False) for i in range(b, L)]


def forward(cfg, tensors, tokens):
    """logits [n, vocab] and the residual stream after every layer run [runs, n, E]."""
    T = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x0 = T["embed"][torch.tensor(tokens)]
    x = x0
    trail = []
    for i, _p, first_of_pass in layer_runs(cfg):
        if first_of_pass:
            x = torch.cat([x, x0], -1) @ T["loop.in"].T
        spec = cfg["layers"][i]
        pre = f"l{i}."
        h = layer_norm(x, T[pre + "norm1"], T[pre + "norm1.b"], eps)
        if spec["type"] == "attention":
            y = attention_mixer(h, sub(T, pre + "mix."), spec["mixer"])
        elif spec["type"] == "retention":
            y = retention_mixer(h, sub(T, pre + "mix."), spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        if spec.get("mlp"):
            y = y + moe_ff(h, sub(T, pre + "mlp."), spec["mlp"])
        x = x + cfg["residual_mult"] * y
        trail.append(x)
    z = layer_norm(x, T["final.norm"], T["final.norm.b"], eps) @ T["head"].T
    if cfg.get("logit_softcap"):
        z = softcap(z, cfg["logit_softcap"])
    return z, torch.stack(trail)
