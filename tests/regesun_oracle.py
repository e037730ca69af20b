"""Plain, slow PyTorch rendering of the Regesun decoder, one function per mechanism.

Everything runs token by token (or with explicit masks) in one precision, straight from
the equations; it shares nothing with the engine's model, cache or kernels.  A model is a
``config`` dict (the keys of a Regesun ``config.json``) and a dict of tensors named as in
its checkpoint.
"""
from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def general_delta(h, t, p, mx, eps):
    """h [T, W] -> mixer output [T, W]; state per head is a dim x dim matrix from zero."""
    H, D = mx["heads"], mx["dim"]
    T = h.shape[0]
    r = (h @ t[p + "r"].T).view(T, H, D)
    k = (h @ t[p + "k"].T).view(T, H, D)
    v = (h @ t[p + "v"].T).view(T, H, D)
    lo = torch.tanh(h @ t[p + "w1"].T) @ t[p + "w2"].T + t[p + "w0"]
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(lo)).view(T, H, D)
    a = torch.sigmoid(h @ t[p + "a"].T + t[p + "a.b"]).view(T, H, D)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, D, D, dtype=h.dtype)
    out = torch.zeros(T, H, D, dtype=h.dtype)
    for i in range(T):
        uS = torch.einsum("hk,hkv->hv", u[i], S)
        S = w[i][:, :, None] * S - (a[i] * u[i])[:, :, None] * uS[:, None, :] \
            + k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hkv,hk->hv", S, r[i])
    o = rms(out, eps).reshape(T, H * D) * t[p + "norm"] * torch.sigmoid(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def mamba2(h, t, p, mx, eps):
    H, P, N, G, K = mx["heads"], mx["vdim"], mx["state"], mx["groups"], mx["conv"]
    ng = mx["norm_groups"]
    T = h.shape[0]
    inner = H * P
    zxbcdt = h @ t[p + "in"].T
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    cw, cb = t[p + "conv"], t[p + "conv.b"]
    pad = torch.cat([torch.zeros(K - 1, xbc.shape[1], dtype=h.dtype), xbc], 0)
    conv = torch.zeros_like(xbc)
    for i in range(T):
        conv[i] = (pad[i:i + K].T * cw).sum(-1) + cb
    conv = conv * torch.sigmoid(conv)
    x = conv[:, :inner].view(T, H, P)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    C = conv[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + t[p + "dt_bias"], threshold=1e9)
    A = -torch.exp(t[p + "A_log"])
    S = torch.zeros(H, N, P, dtype=h.dtype)
    y = torch.zeros(T, H, P, dtype=h.dtype)
    hg = H // G
    for i in range(T):
        for hh in range(H):
            g = hh // hg
            S[hh] = torch.exp(A[hh] * dt[i, hh]) * S[hh] + dt[i, hh] * B[i, g][:, None] * x[i, hh][None, :]
            y[i, hh] = S[hh].T @ C[i, g] + t[p + "D"][hh] * x[i, hh]
    y = y.reshape(T, inner) * (z * torch.sigmoid(z))
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * t[p + "norm"]
    return y @ t[p + "o"].T


def latent_attention(h, t, p, mx, eps):
    H, D, V, R = mx["heads"], mx["dim"], mx["vdim"], mx["kv_rank"]
    win, scale = mx["mask"]["size"], mx["scale"]
    T = h.shape[0]
    q = (h @ t[p + "q"].T).view(T, H, D)
    c = rms(h @ t[p + "dkv"].T, eps) * t[p + "dkv.norm"]
    k = (c @ t[p + "uk"].T).view(T, H, D)
    v = (c @ t[p + "uv"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for i in range(T):
        lo = max(0, i - win + 1)
        for hh in range(H):
            s = (k[lo:i + 1, hh] @ q[i, hh]) * scale
            sink = t[p + "sink"][hh]
            m = torch.maximum(s.max(), sink)
            e = torch.exp(s - m)
            den = e.sum() + torch.exp(sink - m)
            out[i, hh] = (e / den) @ v[lo:i + 1, hh]
    o = out.reshape(T, H * V) * torch.sigmoid(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def dense_ff(h, t, p, mlp):
    lim = mlp["limit"]
    g = torch.clamp(h @ t[p + "gate"].T, max=lim)
    u = torch.clamp(h @ t[p + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ t[p + "down"].T


MIXERS = {"general_delta": general_delta, "mamba2": mamba2, "latent_attention": latent_attention}


@torch.no_grad()
def forward(config, tensors, tokens, dtype=torch.float64, return_layers=False):
    """tokens (list) -> logits [T, vocab]; optionally also the residual after each layer."""
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    ids = torch.tensor(tokens, dtype=torch.long)
    x = t["embed"][ids] + t["pos"][:len(tokens)]
    layers = []
    for i, L in enumerate(config["layers"]):
        p = "l%d." % i
        m = MIXERS[L["type"]](rms(x, eps) * t[p + "norm1"], t, p + "mix.", L["mixer"], eps)
        x = x + rms(m, eps) * t[p + "norm1b"] * t[p + "ls1"]
        if L.get("mlp") is not None:
            f = dense_ff(rms(x, eps) * t[p + "norm2"], t, p + "mlp.", L["mlp"])
            x = x + rms(f, eps) * t[p + "norm2b"] * t[p + "ls2"]
        layers.append(x.clone())
    logits = (rms(x, eps) * t["final.norm"]) @ t["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits
