"""Plain, slow PyTorch rendering of the Rotutar decoder, one function per mechanism.

Everything runs token by token (or with explicit masks) in one precision (float64 by
default), straight from the equations; it shares nothing with the engine's model, cache or
kernels.  A model is a ``config`` dict (the keys of a Rotutar ``config.json``) and a dict of
tensors named as in its checkpoint.

Layer:   x <- x + N(m * sigmoid(R1 x + b1)),  m = mixer(x);   x <- x + N(f * sigmoid(R2 x + b2)),
f = ff(x).  N is an RMS norm taken separately over ``norm.groups`` equal parts of the vector.
"""
from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    T, n = x.shape
    return rms(x.view(T, groups, n // groups), eps).reshape(T, n) * w


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ windowed attention
def rotate(x, base, dims):
    """x [T, heads, dim]: channels (2i, 2i+1), i < dims/2, turned by t * base^(-2i/dims)."""
    T = x.shape[0]
    out = x.clone()
    for t in range(T):
        for i in range(dims // 2):
            a = t * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, :, 2 * i], x[t, :, 2 * i + 1]
            out[t, :, 2 * i] = u * c - v * s
            out[t, :, 2 * i + 1] = v * c + u * s
    return out


def window_attention(h, t, p, mx, eps):
    """Grouped-query attention, sliding window, softmax whose denominator holds exp(sink)."""
    H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = rms(h @ t[p + "q"].T, eps) * t[p + "q.norm"]
    k = rms(h @ t[p + "k"].T, eps) * t[p + "k.norm"]
    v = (h @ t[p + "v"].T).view(T, G, V)
    q = rotate(q.view(T, H, D), mx["rot"]["base"], mx["rot"]["dims"])
    k = rotate(k.view(T, G, D), mx["rot"]["base"], mx["rot"]["dims"])
    win = mx["mask"]["size"]
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for i in range(T):
        lo = max(0, i - win + 1)
        for hd in range(H):
            g = hd // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hd]) * mx["scale"]
            e = torch.exp(s)
            den = e.sum() + torch.exp(t[p + "sink"][hd])
            out[i, hd] = (e / den) @ v[lo:i + 1, g]
    return out.reshape(T, H * V) @ t[p + "o"].T


# ------------------------------------------------------------------ gated delta rule
def short_conv(x, w):
    """x [T, C], w [C, taps]: y[t] = sum_j w[:, taps-1-j] * x[t-j], with x[t] = 0 for t < 0."""
    T, C = x.shape
    K = w.shape[1]
    y = torch.zeros_like(x)
    for i in range(T):
        for j in range(K):
            if i - j >= 0:
                y[i] += w[:, K - 1 - j] * x[i - j]
    return y


def gated_delta(h, t, p, mx, eps):
    H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ t[p + "q"].T, t[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ t[p + "k"].T, t[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ t[p + "v"].T, t[p + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ t[p + "b"].T)                                      # [T, H]
    dt = torch.nn.functional.softplus((h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "dt_bias"],
                                      threshold=1e9).view(T, H, D)
    decay = torch.exp(-torch.exp(t[p + "A_log"])[None, :, None] * dt)           # [T, H, D]
    S = torch.zeros(H, D, V, dtype=h.dtype)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for i in range(T):
        for hd in range(H):
            g = hd // (H // G)
            Sh = decay[i, hd][:, None] * S[hd]
            u = beta[i, hd] * (v[i, hd] - Sh.T @ k[i, g])
            Sh = Sh + torch.outer(k[i, g], u)
            S[hd] = Sh
            o[i, hd] = Sh.T @ q[i, g]
    gate = torch.sigmoid((h @ t[p + "g1"].T) @ t[p + "g2"].T).view(T, H, V)
    o = rms(o, eps) * t[p + "norm"] * gate
    return o.reshape(T, H * V) @ t[p + "o"].T


def parallel(h, t, p, mx, eps):
    return mx["left_scale"] * window_attention(h, t, p + "left.", mx["left"], eps) \
        + mx["right_scale"] * gated_delta(h, t, p + "right.", mx["right"], eps)


# ------------------------------------------------------------------ HGRN2
def hgrn2(h, t, p, mx, eps):
    H, D, V = mx["heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = silu(h @ t[p + "q"].T).view(T, H, D)
    v = (h @ t[p + "v"].T).view(T, H, V)
    lower = t[p + "lower"]
    f = (lower + (1 - lower) * torch.sigmoid(h @ t[p + "f"].T + t[p + "f.b"])).view(T, H, D)
    S = torch.zeros(H, D, V, dtype=h.dtype)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for i in range(T):
        S = f[i][:, :, None] * S + (1 - f[i])[:, :, None] * v[i][:, None, :]
        o[i] = torch.einsum("hdv,hd->hv", S, q[i])
    o = rms(o, eps) * t[p + "norm"]
    return o.reshape(T, H * V) @ t[p + "o"].T


MIXERS = {"parallel": parallel, "hgrn2": hgrn2}


# ------------------------------------------------------------------ feed-forward
def dense_ff(h, t, p, ml):
    return (silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def route(z, r):
    """z [experts] router logits -> (chosen experts, their weights)."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(z)
    gc, keep = r["groups"]["count"], r["groups"]["keep"]
    per = E // gc
    gs = [sum(sorted(s[g * per:(g + 1) * per].tolist(), reverse=True)[:2]) for g in range(gc)]
    best = sorted(range(gc), key=lambda g: (-gs[g], g))[:keep]
    allowed = [e for e in range(E) if e // per in best]
    chosen = sorted(allowed, key=lambda e: (-float(s[e]), e))[:top]
    return chosen, [s[e] for e in chosen]


def moe_ff(h, t, p, ml):
    lim = ml["expert"]["limit"]
    out = torch.zeros_like(h)
    z = h @ t[p + "router"].T
    for i in range(h.shape[0]):
        chosen, w = route(z[i], ml["router"])
        for e, we in zip(chosen, w):
            pe = p + "e%d." % e
            g = torch.clamp(t[pe + "gate"] @ h[i], max=lim)
            u = torch.clamp(t[pe + "up"] @ h[i], -lim, lim)
            out[i] += we * (t[pe + "down"] @ (g * torch.sigmoid(1.702 * g) * (u + 1)))
    return out


# ------------------------------------------------------------------ model
def forward(config, tensors, tokens, return_layers=False, dtype=torch.float64):
    """Logits [T, vocab] of a whole sequence (and the residual stream after every layer)."""
    t = {k: v.to(dtype) for k, v in tensors.items()}
    eps, groups = config["norm"]["eps"], config["norm"]["groups"]
    x = t["embed"][torch.tensor(tokens)]
    layers = []
    for i, L in enumerate(config["layers"]):
        p = "l%d." % i
        m = MIXERS[L["type"]](x, t, p + "mix.", L["mixer"], eps)
        m = m * torch.sigmoid(x @ t[p + "rg1"].T + t[p + "rg1.b"])
        x = x + group_norm(m, t[p + "norm1"], groups, eps)
        if L.get("mlp"):
            ff = dense_ff if L["mlp"]["kind"] == "dense" else moe_ff
            f = ff(x, t, p + "mlp.", L["mlp"])
            f = f * torch.sigmoid(x @ t[p + "rg2"].T + t[p + "rg2.b"])
            x = x + group_norm(f, t[p + "norm2"], groups, eps)
        layers.append(x.clone())
    y = group_norm(x, t["final.norm"], groups, eps) @ t["head"].T
    cap = config.get("logit_softcap")
    if cap:
        y = cap * torch.tanh(y / cap)
    return (y, layers) if return_layers else y
