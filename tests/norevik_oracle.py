"""Plain, slow float64 implementation of the Norevik design, one function per mechanism.

It is the yardstick of the Norevik tests and shares no code with the engine: it takes a config dict (the
layout of config.json) and a dict name -> torch tensor, runs one whole sequence at a time and keeps no cache
(attention looks at the full prefix, recurrences are walked token by token from a zero state).

Notation: n tokens, width E. Linear weights are [out, in]; y = x @ W.T. A layer is
x <- x + LN1(mixer(x)), then x <- x + LN2(ff(x)): the sublayers read the stream itself, the layer norm
(weight and bias) sits on their outputs.
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


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rotate_pairs(x, pos, dims, base):
    """x [n, ..., D]: dims (2i, 2i + 1), i < dims / 2, of the last axis turn by pos * base^(-2i / dims)."""
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    ang = pos.to(F64)[:, None] * f[None, :]
    while ang.dim() < x.dim():
        ang = ang.unsqueeze(1)
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# --------------------------------------------------------------------------------------------- mixers
def latent_attention_mixer(h, W, m, eps):
    """Keys and values of all heads come from one low-rank latent per token, c = rms_norm(first kv_rank rows of
    W_dkv h); the last rot_dim rows are a rotated key part that every head shares. Softmax with a per-head sink
    in the denominator, a sigmoid output gate."""
    n = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n)
    q = (h @ W["q"].T).view(n, H, D + R)
    qn, qr = q[..., :D], q[..., D:]
    dkv = h @ W["dkv"].T
    c = unit_rms(dkv[:, :C], eps) * W["dkv.norm"]
    kr = dkv[:, C:]
    rd, base = m["rot"]["dims"], m["rot"]["base"]
    qr = rotate_pairs(qr, pos, rd, base)
    kr = rotate_pairs(kr, pos, rd, base)
    kn = (c @ W["uk"].T).view(n, H, D)
    v = (c @ W["uv"].T).view(n, H, Dv)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    out = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        s = (qn[:, hd] @ kn[:, hd].T + qr[:, hd] @ kr.T) * m["scale"]
        s = s.masked_fill(~mask, -math.inf)
        sink = W["sink"][hd]
        mx = torch.maximum(s.max(-1, keepdim=True).values, sink)
        e = torch.exp(s - mx)
        p = e / (e.sum(-1, keepdim=True) + torch.exp(sink - mx))
        out[:, hd] = p @ v[:, hd]
    g = torch.sigmoid(h @ W["g"].T)
    return (out.reshape(n, H * Dv) * g) @ W["o"].T


def mlstm_mixer(h, W, m, eps):
    """Matrix memory with exponential gates kept stable by a running maximum that starts at 0."""
    n = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W["q"].T).view(n, H, D) * D ** -0.5
    k = (h @ W["k"].T).view(n, H, D)
    v = (h @ W["v"].T).view(n, H, Dv)
    ig = cap * torch.tanh((h @ W["i"].T + W["i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W["f"].T + W["f.b"]) / cap))
    out = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        nv = torch.zeros(D, dtype=F64)
        mm = torch.zeros((), dtype=F64)
        for t in range(n):
            mn = torch.maximum(fg[t, hd] + mm, ig[t, hd])
            a, b = torch.exp(fg[t, hd] + mm - mn), torch.exp(ig[t, hd] - mn)
            S = a * S + b * torch.outer(k[t, hd], v[t, hd])
            nv = a * nv + b * k[t, hd]
            mm = mn
            den = torch.maximum(torch.abs(nv @ q[t, hd]), torch.exp(-mm)) + 1e-6
            out[t, hd] = (S.T @ q[t, hd]) / den
    o = unit_rms(out, eps).reshape(n, H * Dv) * W["norm"]
    return (o * torch.sigmoid(h @ W["g"].T)) @ W["o"].T


def mamba2_mixer(h, W, m, eps):
    """Selective state space layer with a scalar decay per head (state N x vdim per head)."""
    n = h.shape[0]
    H, P, N, G, K, NG = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"]
    inner = H * P
    zx = h @ W["in"].T
    z, xbc, dt = zx[:, :inner], zx[:, inner:2 * inner + 2 * G * N], zx[:, 2 * inner + 2 * G * N:]
    pad = torch.cat([torch.zeros(K - 1, xbc.shape[1], dtype=F64), xbc], 0)
    conv = sum(pad[j:j + n] * W["conv"][:, j] for j in range(K)) + W["conv.b"]   # tap K-1 is the current token
    xbc = silu(conv)
    x = xbc[:, :inner].view(n, H, P)
    Bm = xbc[:, inner:inner + G * N].view(n, G, N)
    Cm = xbc[:, inner + G * N:].view(n, G, N)
    dt = softplus(dt + W["dt_bias"])
    A = -torch.exp(W["A_log"])
    y = torch.zeros(n, H, P, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(n):
            S = torch.exp(A[hd] * dt[t, hd]) * S + dt[t, hd] * torch.outer(Bm[t, g], x[t, hd])
            y[t, hd] = S.T @ Cm[t, g] + W["D"][hd] * x[t, hd]
    y = y.reshape(n, inner) * silu(z)
    y = unit_rms(y.view(n, NG, inner // NG), eps).reshape(n, inner) * W["norm"]
    return y @ W["o"].T


MIXERS = {"latent_attention": latent_attention_mixer, "mlstm": mlstm_mixer, "mamba2": mamba2_mixer}


# --------------------------------------------------------------------------------------------- feed-forward
def dense_ff(h, W):
    return torch.relu(h @ W["up"].T) ** 2 @ W["down"].T


def glu_expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, f):
    """Per token: the chosen outputs (ids < experts: real experts, the rest identity) and their weights."""
    r = f["router"]
    X, I, top = r["experts"], r.get("identity", 0), r["top"]
    s = torch.softmax(h @ W["router"].T, -1)              # over experts and identity experts together
    choice = s + W["correction"]
    gr = r.get("groups")
    if gr and gr["count"] > 1:
        per = (X + I) // gr["count"]
        best = choice.view(-1, gr["count"], per).max(-1).values
        keep = torch.topk(best, gr["keep"], dim=-1).indices
        ok = torch.zeros_like(best, dtype=torch.bool).scatter_(1, keep, True)
        choice = choice.masked_fill(~ok.repeat_interleave(per, dim=1), -math.inf)
    ids = torch.topk(choice, top, dim=-1).indices
    return ids, torch.gather(s, 1, ids)


def moe_ff(h, W, f):
    X = f["router"]["experts"]
    ids, wt = route(h, W, f)
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            y[t] += wt[t, j] * (glu_expert(h[t:t + 1], W, f"e{e}.")[0] if e < X else h[t])
    if f.get("shared"):
        y = y + glu_expert(h, W, "shared.")
    return y


# --------------------------------------------------------------------------------------------- model
def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens):
    """Logits [n, vocab] of every position and the residual stream after every layer [layers, n, E]."""
    eps = cfg["norm"]["eps"]
    T = {k: v.to(F64) for k, v in tensors.items()}
    x = T["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    trail = []
    for i, ent in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[ent["type"]](x, sub(tensors, p + "mix."), ent["mixer"], eps)
        x = x + layer_norm(y, T[p + "norm1"], T[p + "norm1.b"], eps)
        f = ent.get("mlp")
        if f:
            W = sub(tensors, p + "mlp.")
            y = dense_ff(x, W) if f["kind"] == "dense" else moe_ff(x, W, f)
            x = x + layer_norm(y, T[p + "norm2"], T[p + "norm2.b"], eps)
        trail.append(x.clone())
    z = layer_norm(x, T["final.norm"], T["final.norm.b"], eps) @ T["head"].T
    return z, torch.stack(trail)
