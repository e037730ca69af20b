"""Sequence-mixer ops: recurrent state layers (generalized delta rule, Mamba-2), latent
attention with a sliding window and a softmax sink, learned positions, and the norms and
pointwise steps around them.

GPU tensors always run the gfx950 kernels of ``csrc/seqmix`` (``libp2p_seqmix.so``, built on
first use when missing); CPU tensors run the PyTorch rendering of the same math, which is
the plumbing / scheduling path of CPU tests, never a fallback for GPU tensors.

Conventions shared by every op:
  * activations (``x``-like matrices that feed or leave matrix products) are bf16 or fp32;
    vector parameters, recurrent state, the residual stream and every reduction are fp32;
  * a step is a flat list of R token rows cut into E *entries* (one per sequence portion):
    ``ent`` int32 [E, 4] = (first row, rows, first position, state slot); a portion whose
    first position is 0 starts from a zero state, others continue the slot's state;
  * ``row_ent`` int32 [R] names each row's entry, ``pos`` int32 [R] its position.
"""
from __future__ import annotations

import ctypes
import math
import os
import threading

import torch

from . import _lib

c_int, c_long, c_float, c_void_p = ctypes.c_int, ctypes.c_long, ctypes.c_float, ctypes.c_void_p

_SIGS = {
    "p2p_sm_embed_pos": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                         c_void_p],
    "p2p_sm_rmsnorm": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                       c_void_p, c_int, c_int, c_int, c_float, c_void_p],
    "p2p_sm_norm_scale_add": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                              c_float, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "p2p_sm_gdelta_scan": [c_void_p] * 5 + [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                            c_int, c_float, c_int, c_void_p],
    "p2p_sm_gdelta_scan_chunked": [c_void_p] * 5 + [c_int, c_void_p, c_int, c_void_p, c_void_p,
                                                    c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                    c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                                                    c_float, c_int, c_void_p],
    "p2p_sm_mamba_scan_chunked": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                  c_int, c_void_p],
    "p2p_sm_mamba_conv": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_mamba_scan": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                          c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_mamba_tail": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_void_p],
    "p2p_sm_latent_attn": [c_void_p, c_long, c_long, c_void_p, c_void_p, c_int, c_void_p,
                           c_void_p, c_void_p, c_float, c_int, c_void_p, c_long, c_long, c_int,
                           c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_latent_attn_mfma": [c_void_p, c_long, c_long, c_void_p, c_void_p, c_int, c_void_p,
                                c_void_p, c_void_p, c_int, c_void_p, c_float, c_int, c_void_p,
                                c_long, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
    "p2p_sm_tanh": [c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_sigmoid_gate": [c_void_p, c_long, c_long, c_void_p, c_int, c_void_p, c_int, c_int,
                            c_int, c_int, c_int, c_void_p],
    "p2p_sm_ff_act": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_float, c_int,
                      c_void_p],
}

_lock = threading.Lock()
_so = None


def lib_path() -> str:
    from .. import _build

    return _build.SEQMIX_LIB


def lib():
    """Load (once) the sequence-mixer kernel library; build it first when it is missing.  A
    library that no build of the tree's sources produced is refused (build stamp)."""
    global _so
    if _so is not None:
        return _so
    with _lock:
        if _so is not None:
            return _so
        from .. import _build

        path = _build.SEQMIX_LIB
        if not os.path.exists(path):
            _build.build_seqmix(jobs=min(16, os.cpu_count() or 1))
        srcs, hdrs = _build.seqmix_sources()
        if srcs:
            import json

            try:
                with open(path + ".stamp") as f:
                    ok = json.load(f).get("sources_sha256") == _build.sources_digest(srcs + hdrs)
            except FileNotFoundError:
                ok = False
            if not ok and os.environ.get("P2P_ALLOW_STALE_LIB", "0") != "1":
                raise _lib.KernelError("%s was not built from the tree's csrc/seqmix -- rebuild "
                                       "with `python -m p2p_llm_chat_go_amd._build --only seqmix`"
                                       % path)
        L = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        for name, args in _SIGS.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = c_int
        _so = L
    return _so


def _st(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _f32(t) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise TypeError("activations are bfloat16 or float32, got %s" % t.dtype)


def _chk(err, name):
    if err != 0:
        raise _lib.KernelError("%s failed with hipError %d" % (name, err))


def _rows2d(t, name):
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError("%s must be a row-major 2-d view" % name)


def _vec(t, n, name):
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
        raise ValueError("%s must be a contiguous float32 vector of %d" % (name, n))


def _rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


# ------------------------------------------------------------------ embedding / norms
def embed_pos(embed, pos_table, ids, pos, out):
    """out[r] = embed[ids[r]] (+ pos_table[pos[r]]) as fp32 rows."""
    R, W = out.shape
    if not out.is_cuda:
        v = embed[ids.long()].float()
        if pos_table is not None:
            v = v + pos_table[pos.long()].float()
        out.copy_(v)
        return out
    assert out.dtype == torch.float32 and out.is_contiguous() and embed.shape[1] == W
    assert ids.dtype == torch.int32 and pos.dtype == torch.int32 and ids.numel() >= R
    assert embed.is_contiguous() and (pos_table is None or (pos_table.is_contiguous()
                                                           and pos_table.dtype == embed.dtype))
    _chk(lib().p2p_sm_embed_pos(embed.data_ptr(), _lib.ptr(pos_table), ids.data_ptr(),
                                pos.data_ptr(), out.data_ptr(), R, W, _f32(embed), _st(out)),
         "embed_pos")
    return out


def rmsnorm(x, w, eps, out, parts: int = 1, in_rows=None, out_rows=None):
    """out[o(r)] = x[i(r)] / sqrt(mean(x^2) + eps) * w, the mean taken over each of ``parts``
    equal parts of the row.  x: fp32 or activation type; out: activation type (or fp32).
    in_rows / out_rows: int32 row gathers / scatters (out row < 0: dropped)."""
    R = (in_rows if in_rows is not None else x).shape[0]
    n = x.shape[1]
    if not x.is_cuda:
        xs = x.float() if in_rows is None else x[in_rows.long()].float()
        v = _rms(xs.view(R, parts, n // parts), eps).reshape(R, n)
        if w is not None:
            v = v * w
        v = v.to(out.dtype)
        if out_rows is None:
            out[:R] = v
        else:
            keep = out_rows >= 0
            out[out_rows[keep].long()] = v[keep]
        return out
    _rows2d(x, "x")
    _rows2d(out, "out")
    if w is not None:
        _vec(w, n, "w")
    if n % parts:
        raise ValueError("row of %d does not split into %d parts" % (n, parts))
    assert out.shape[1] == n and (out_rows is not None or out.shape[0] >= R)
    _chk(lib().p2p_sm_rmsnorm(x.data_ptr(), x.stride(0), _f32(x), _lib.ptr(w), out.data_ptr(),
                              out.stride(0), _f32(out), _lib.ptr(in_rows), _lib.ptr(out_rows), R,
                              n, parts, eps, _st(x)), "rmsnorm")
    return out


def norm_scale_add(x, y, w, ls, eps, next_w=None, next_out=None):
    """x += y / sqrt(mean(y^2) + eps) * w * ls on the fp32 residual x (ls may be None).
    With next_w / next_out also the next sublayer's input in the same pass:
    next_out = x / sqrt(mean(x^2) + eps) * next_w from the updated rows."""
    R, n = x.shape
    if not x.is_cuda:
        v = _rms(y.float(), eps) * w
        if ls is not None:
            v = v * ls
        x += v
        if next_w is not None:
            next_out[:R] = (_rms(x, eps) * next_w).to(next_out.dtype)
        return x
    _rows2d(y, "y")
    assert x.dtype == torch.float32 and x.is_contiguous() and y.shape == x.shape
    _vec(w, n, "w")
    if ls is not None:
        _vec(ls, n, "ls")
    ldh = 0
    if next_w is not None:
        _vec(next_w, n, "next_w")
        _rows2d(next_out, "next_out")
        assert next_out.dtype == y.dtype and next_out.shape[1] == n and next_out.shape[0] >= R
        ldh = next_out.stride(0)
    _chk(lib().p2p_sm_norm_scale_add(x.data_ptr(), y.data_ptr(), y.stride(0), w.data_ptr(),
                                     _lib.ptr(ls), R, n, eps, _lib.ptr(next_w),
                                     _lib.ptr(next_out if next_w is not None else None), ldh,
                                     _f32(y), _st(x)), "norm_scale_add")
    return x


# ------------------------------------------------------------------ pointwise
def tanh_(x):
    if not x.is_cuda:
        x.copy_(torch.tanh(x.float()).to(x.dtype))
        return x
    _rows2d(x, "x")
    _chk(lib().p2p_sm_tanh(x.data_ptr(), x.stride(0), x.shape[1], x.shape[0], _f32(x), _st(x)),
         "tanh")
    return x


def sigmoid_gate(o, g, out, H: int, V: int):
    """out[r, h*V + v] = o[h, r, v] * sigmoid(g[r, h*V + v]); o is any [H, R, V] view whose
    last stride is 1."""
    R = g.shape[0]
    if not g.is_cuda:
        out.copy_((o.float().permute(1, 0, 2).reshape(R, H * V) * torch.sigmoid(g.float())).to(out.dtype))
        return out
    _rows2d(g, "g")
    _rows2d(out, "out")
    assert o.shape == (H, R, V) and o.stride(2) == 1 and o.dtype == g.dtype == out.dtype
    _chk(lib().p2p_sm_sigmoid_gate(o.data_ptr(), o.stride(0), o.stride(1), g.data_ptr(),
                                   g.stride(0), out.data_ptr(), out.stride(0), R, H, V, _f32(g),
                                   _st(g)), "sigmoid_gate")
    return out


def ff_act(gu, out, limit: float, alpha: float = 1.702):
    """[gate | up] -> min(gate, limit) * sigmoid(alpha * .) * (clamp(up, +-limit) + 1)."""
    R, F = out.shape
    if not gu.is_cuda:
        g = torch.clamp(gu[:, :F].float(), max=limit)
        u = torch.clamp(gu[:, F:].float(), -limit, limit)
        out.copy_((g * torch.sigmoid(alpha * g) * (u + 1)).to(out.dtype))
        return out
    _rows2d(gu, "gu")
    _rows2d(out, "out")
    assert gu.shape == (R, 2 * F) and gu.dtype == out.dtype
    _chk(lib().p2p_sm_ff_act(gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), R, F,
                             limit, alpha, _f32(gu), _st(gu)), "ff_act")
    return out


# ------------------------------------------------------------------ recurrences in chunks
# A portion of at least 2 * SCAN_CHUNK tokens is scanned in chunks of SCAN_CHUNK tokens that
# run side by side (local pass, chain over the chunks, output pass); shorter steps -- decode,
# small portions -- walk their tokens in one pass.  Both recurrences are linear in the state,
# so the chunked form computes the same sums in another order (fp32 throughout).
SCAN_CHUNK = int(os.environ.get("P2P_SCAN_CHUNK", "64"))


def scan_chunks(ent_host: list, chunk: int):
    """(chunks as entries [(row0, n, 1, chunk index)], per entry (first chunk, chunks, first
    position, slot)) as int32 tensors."""
    vent, cent = [], []
    for row0, n, start, slot in ent_host:
        c0 = len(vent)
        for r in range(row0, row0 + n, chunk):
            vent.append((r, min(chunk, row0 + n - r), 1, len(vent)))
        cent.append((c0, len(vent) - c0, start, slot))
    return torch.tensor(vent, dtype=torch.int32), torch.tensor(cent, dtype=torch.int32)


def _chunked(ent_host) -> bool:
    return SCAN_CHUNK > 0 and max(e[1] for e in ent_host) >= 2 * SCAN_CHUNK


# ------------------------------------------------------------------ generalized delta rule
GD_DECAY_SCALE = math.exp(-0.5)


def gdelta_scan(r, k, v, g, a, lo, w0, ab, normw, state, ent, ent_host, out, H: int, D: int,
                eps: float):
    """Generalized delta rule over the entries of a step, state carried in ``state`` slots.

    r, k, v, g, a: [R, H*D] views of one projection buffer (same row stride); lo [R, H*D] the
    decay logits before their bias w0; ab the removal-rate bias; normw the output weight.
    state fp32 [slots, H, D, D] (key index, value index).  ent_host: the entries as a list of
    (row0, n, start, slot) (the CPU path walks it; the kernel reads ``ent``)."""
    if not r.is_cuda:
        for row0, n, start, slot in ent_host:
            S = state[slot] if start > 0 else torch.zeros_like(state[slot])
            for t in range(row0, row0 + n):
                rr, kk, vv = (z[t].float().view(H, D) for z in (r, k, v))
                w = torch.exp(-GD_DECAY_SCALE * torch.sigmoid(lo[t].float() + w0)).view(H, D)
                aa = torch.sigmoid(a[t].float() + ab).view(H, D)
                u = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
                uS = torch.einsum("hk,hkv->hv", u, S)
                S = w[:, :, None] * S - (aa * u)[:, :, None] * uS[:, None, :] \
                    + kk[:, :, None] * vv[:, None, :]
                o = torch.einsum("hkv,hk->hv", S, rr)
                o = _rms(o, eps).reshape(H * D) * normw * torch.sigmoid(g[t].float())
                out[t] = o.to(out.dtype)
            state[slot] = S
        return out
    n = H * D
    for t_, nm in ((r, "r"), (k, "k"), (v, "v"), (g, "g"), (a, "a"), (lo, "lo"), (out, "out")):
        _rows2d(t_, nm)
        assert t_.shape[1] == n and t_.dtype == r.dtype, nm
    ld = r.stride(0)
    assert all(t_.stride(0) == ld for t_ in (k, v, g, a))
    for t_, nm in ((w0, "w0"), (ab, "ab"), (normw, "normw")):
        _vec(t_, n, nm)
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, D)
    E = ent.shape[0]
    assert ent.dtype == torch.int32 and ent.is_contiguous() and ent.shape[1] == 4
    if D > 256:
        raise ValueError("gdelta_scan: head size %d > 256" % D)
    if _chunked(ent_host):
        vent, cent = (t_.to(r.device) for t_ in scan_chunks(ent_host, SCAN_CHUNK))
        tmp = torch.empty(3, vent.shape[0], H, D, D, device=r.device, dtype=torch.float32)
        _chk(lib().p2p_sm_gdelta_scan_chunked(
            r.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), a.data_ptr(), ld,
            lo.data_ptr(), lo.stride(0), w0.data_ptr(), ab.data_ptr(), normw.data_ptr(),
            state.data_ptr(), tmp.data_ptr(), vent.data_ptr(), vent.shape[0], cent.data_ptr(), E,
            out.data_ptr(), out.stride(0), H, D, eps, _f32(r), _st(r)), "gdelta_scan_chunked")
        return out
    _chk(lib().p2p_sm_gdelta_scan(r.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(),
                                  a.data_ptr(), ld, lo.data_ptr(), lo.stride(0), w0.data_ptr(),
                                  ab.data_ptr(), normw.data_ptr(), state.data_ptr(),
                                  ent.data_ptr(), E, out.data_ptr(), out.stride(0), H, D, eps,
                                  _f32(r), _st(r)), "gdelta_scan")
    return out


# ------------------------------------------------------------------ Mamba-2
def mamba_conv(zx, xoff: int, cw, cb, tail, ent, ent_host, row_ent, out):
    """Causal per-channel convolution + bias + silu over channels [xoff, xoff + C) of zx.
    cw fp32 [C, K] (column K-1 multiplies the newest input), tail fp32 [slots, K-1, C] the raw inputs
    before each slot's next token (read only here; ``mamba_scan`` rolls it)."""
    R, C = out.shape
    K = cw.shape[1]
    if not zx.is_cuda:
        for row0, n, start, slot in ent_host:
            raw = zx[row0:row0 + n, xoff:xoff + C].float()
            prev = tail[slot] if start > 0 else torch.zeros(K - 1, C)
            pad = torch.cat([prev, raw], 0)
            acc = cb.clone().expand(n, C).clone()
            for kk in range(K):
                acc += pad[kk:kk + n] * cw[:, kk]
            out[row0:row0 + n] = acc * torch.sigmoid(acc)
        return out
    _rows2d(zx, "zx")
    assert out.dtype == torch.float32 and out.is_contiguous()
    assert cw.dtype == torch.float32 and cw.is_contiguous() and cw.shape[0] == C
    _vec(cb, C, "cb")
    assert tail.dtype == torch.float32 and tail.is_contiguous() and tail.shape[1:] == (K - 1, C)
    assert xoff + C <= zx.shape[1] and row_ent.dtype == torch.int32
    _chk(lib().p2p_sm_mamba_conv(zx.data_ptr(), zx.stride(0), xoff, cw.data_ptr(), cb.data_ptr(),
                                 tail.data_ptr(), ent.data_ptr(), row_ent.data_ptr(),
                                 out.data_ptr(), R, C, K, _f32(zx), _st(zx)), "mamba_conv")
    return out


def mamba_scan(conv, zx, xoff: int, dtoff: int, dt_bias, A_log, Dp, state, tail, ent, ent_host,
               y, H: int, P: int, N: int, G: int):
    """Selective state-space scan.  conv fp32 [R, H*P + 2*G*N] = silu(conv(x | B | C)); zx the
    input projection (z at column 0, raw x|B|C at xoff, dt at dtoff).  state fp32
    [slots, H, N, P].  Writes y * silu(z) as fp32 [R, H*P] and rolls the convolution tail."""
    R, C = conv.shape
    inner = H * P
    Km1 = tail.shape[1]
    if not conv.is_cuda:
        hg = H // G
        A = -torch.exp(A_log)
        for row0, n, start, slot in ent_host:
            S = state[slot] if start > 0 else torch.zeros_like(state[slot])
            for t in range(row0, row0 + n):
                x = conv[t, :inner].view(H, P)
                B = conv[t, inner:inner + G * N].view(G, N).repeat_interleave(hg, 0)
                Cc = conv[t, inner + G * N:].view(G, N).repeat_interleave(hg, 0)
                dt = torch.nn.functional.softplus(zx[t, dtoff:dtoff + H].float() + dt_bias,
                                                  threshold=1e9)
                S = torch.exp(A * dt)[:, None, None] * S + (dt[:, None] * B)[:, :, None] * x[:, None, :]
                yy = torch.einsum("hnp,hn->hp", S, Cc) + Dp[:, None] * x
                z = zx[t, :inner].float()
                y[t] = yy.reshape(inner) * (z * torch.sigmoid(z))
            state[slot] = S
            if Km1:
                raw = zx[row0:row0 + n, xoff:xoff + C].float()
                prev = tail[slot] if start > 0 else torch.zeros(Km1, C)
                tail[slot] = torch.cat([prev, raw], 0)[-Km1:]
        return y
    _rows2d(zx, "zx")
    assert conv.dtype == torch.float32 and conv.is_contiguous() and C == inner + 2 * G * N
    assert y.dtype == torch.float32 and y.is_contiguous() and y.shape == (R, inner)
    for t_, nm in ((dt_bias, "dt_bias"), (A_log, "A_log"), (Dp, "D")):
        _vec(t_, H, nm)
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, N, P)
    assert tail.dtype == torch.float32 and tail.is_contiguous() and tail.shape[2] == C
    assert dtoff + H <= zx.shape[1] and xoff + C <= zx.shape[1] and H % G == 0
    if N > 256 or P > 256:
        raise ValueError("mamba_scan: state %d / value %d sizes above 256" % (N, P))
    E = ent.shape[0]
    if _chunked(ent_host):
        vent, cent = (t_.to(zx.device) for t_ in scan_chunks(ent_host, SCAN_CHUNK))
        NV = vent.shape[0]
        tmp = torch.empty(NV, H, N, P, device=zx.device, dtype=torch.float32)
        decay = torch.empty(NV, H, device=zx.device, dtype=torch.float32)
        _chk(lib().p2p_sm_mamba_scan_chunked(
            conv.data_ptr(), C, zx.data_ptr(), zx.stride(0), xoff, dtoff, dt_bias.data_ptr(),
            A_log.data_ptr(), Dp.data_ptr(), state.data_ptr(), tmp.data_ptr(), decay.data_ptr(),
            vent.data_ptr(), NV, cent.data_ptr(), E, y.data_ptr(), H, P, N, G, _f32(zx),
            _st(zx)), "mamba_scan_chunked")
    else:
        _chk(lib().p2p_sm_mamba_scan(conv.data_ptr(), C, zx.data_ptr(), zx.stride(0), xoff, dtoff,
                                     dt_bias.data_ptr(), A_log.data_ptr(), Dp.data_ptr(),
                                     state.data_ptr(), tail.data_ptr(), ent.data_ptr(), E,
                                     y.data_ptr(), H, P, N, G, Km1 + 1, _f32(zx), _st(zx)),
             "mamba_scan")
    _chk(lib().p2p_sm_mamba_tail(zx.data_ptr(), zx.stride(0), xoff, tail.data_ptr(),
                                 ent.data_ptr(), E, C, Km1 + 1, _f32(zx), _st(zx)), "mamba_tail")
    return y


# ------------------------------------------------------------------ latent attention
def latent_attn_ok(H: int, rank: int) -> bool:
    """One head's query, a tile of 4 keys and the accumulators must fit a block."""
    return rank <= 32 * 256 and (rank + 4 * (rank + 1) + 4 + 3) * 4 <= 64 * 1024


def latent_rows_per_wave(H: int) -> int:
    """Rows of one sequence portion that a wavefront of the matrix-core kernel takes: its 16
    (row, head) pairs are RW rows x HS head slots, HS the power of two >= min(H, 16)."""
    hs = 1
    while hs < H and hs < 16:
        hs *= 2
    return 16 // hs


def make_units(ent_host: list, rows_per_wave: int) -> torch.Tensor:
    """int32 [U, 2] (first row, rows): the entries' rows cut into groups of at most
    ``rows_per_wave`` consecutive rows; a group never spans two entries."""
    u = [(r, min(rows_per_wave, row0 + n - r)) for row0, n, _s, _sl in ent_host
         for r in range(row0, row0 + n, rows_per_wave)]
    return torch.tensor(u, dtype=torch.int32).view(-1, 2)


def latent_mfma_ok(qa, cache) -> bool:
    """The matrix-core kernel serves bf16 activations with a latent size that is a multiple
    of 8 up to 512 and 16-byte aligned rows; everything else (and float32) runs the fp32
    kernel.  P2P_LATENT_MFMA=0 switches it off."""
    rank = qa.shape[2]
    return (qa.is_cuda and qa.dtype == torch.bfloat16 and rank % 8 == 0 and 8 <= rank <= 512
            and qa.stride(0) % 8 == 0 and qa.stride(1) % 8 == 0 and qa.data_ptr() % 16 == 0
            and cache.data_ptr() % 16 == 0 and os.environ.get("P2P_LATENT_MFMA", "1") != "0")


LATENT_SPLIT_BLOCKS = 512   # split windows while a step has fewer blocks than this


def latent_attn(qa, cache, block_tables, row_ent, pos, sink, scale: float, win: int, out,
                page: int, units=None, max_keys=None):
    """Windowed attention over cached latents with a softmax sink.

    qa [H, R, rank] (any strides, last = 1): the queries already carried into latent space
    (W_uk^T q per head); cache [tokens, rank] one layer's latent pool, token t of a sequence
    at block_tables[e, t // page] * page + t % page.  out [H, R, rank] = sum_j p_j c_j with
    p = softmax over {sink_h} U {scale * qa . c_j : 0 <= pos - j < win}, the sink term having
    no value.  units: ``make_units(entries, latent_rows_per_wave(H))`` on the device; with
    it, bf16 inputs run on the matrix cores (``latent_mfma_ok``).  max_keys: an upper bound of
    the keys any row sees (host side; lets a step of few rows split its windows)."""
    H, R, rank = qa.shape
    if not qa.is_cuda:
        bt = block_tables.long()
        for r in range(R):
            p = int(pos[r])
            lo = max(0, p - win + 1)
            j = torch.arange(lo, p + 1)
            tok = bt[int(row_ent[r])][j // page] * page + j % page
            c = cache[tok].float()                                  # [n, rank]
            s = (qa[:, r].float() @ c.T) * scale                    # [H, n]
            m = torch.maximum(s.max(-1).values, sink)
            e = torch.exp(s - m[:, None])
            den = e.sum(-1) + torch.exp(sink - m)
            out[:, r] = ((e / den[:, None]) @ c).to(out.dtype)
        return out
    assert qa.stride(2) == 1 and out.stride(2) == 1 and out.shape == qa.shape
    assert qa.dtype == cache.dtype == out.dtype
    assert cache.dim() == 2 and cache.is_contiguous() and cache.shape[1] == rank
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous()
    assert row_ent.dtype == torch.int32 and pos.dtype == torch.int32
    _vec(sink, H, "sink")
    if units is not None and latent_mfma_ok(qa, cache):
        assert units.dtype == torch.int32 and units.is_contiguous() and units.shape[1] == 2
        # few row groups with long windows (decode): cut every window into runs of key tiles
        # so that the step fills the chip; the runs are merged by a second small kernel
        U = units.shape[0]
        hg = -(-H // (16 // latent_rows_per_wave(H)))
        splits = 1
        if max_keys is not None and U * hg < LATENT_SPLIT_BLOCKS:
            splits = max(1, min(-(-min(max_keys, win) // 64), LATENT_SPLIT_BLOCKS // (U * hg), 64))
        part = None
        if splits > 1:
            L = lib()
            L.p2p_sm_latent_attn_mfma_ws.restype = c_long
            n = L.p2p_sm_latent_attn_mfma_ws(U, H, rank, splits)
            part = torch.empty(n, device=qa.device, dtype=torch.float32)
        _chk(lib().p2p_sm_latent_attn_mfma(qa.data_ptr(), qa.stride(0), qa.stride(1),
                                           cache.data_ptr(), block_tables.data_ptr(),
                                           block_tables.shape[1], row_ent.data_ptr(),
                                           pos.data_ptr(), units.data_ptr(), units.shape[0],
                                           sink.data_ptr(), scale, win, out.data_ptr(),
                                           out.stride(0), out.stride(1), H, rank, page, splits,
                                           _lib.ptr(part), _st(qa)),
             "latent_attn_mfma")
        return out
    if not latent_attn_ok(H, rank):
        raise ValueError("latent_attn: %d heads x latent %d exceed the kernel's tile" % (H, rank))
    _chk(lib().p2p_sm_latent_attn(qa.data_ptr(), qa.stride(0), qa.stride(1), cache.data_ptr(),
                                  block_tables.data_ptr(), block_tables.shape[1],
                                  row_ent.data_ptr(), pos.data_ptr(), sink.data_ptr(), scale,
                                  win, out.data_ptr(), out.stride(0), out.stride(1), R, H, rank,
                                  page, _f32(qa), _st(qa)), "latent_attn")
    return out
