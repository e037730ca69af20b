"""Hybrid decoders: a configurable stack of sequence mixers on an fp32 residual stream.

A model is a list of layers; each layer has one *mixer* (registered in ``MIXERS``) and
optionally a feed-forward, both wrapped as

    x <- x + scale * norm_b(sublayer(norm_a(x)))        (RMS norms, per-channel layer scale)

with learned absolute positions added to the token embedding.  Mixers:

  ``general_delta``     generalized delta rule: per head a D x D state with per-channel decay
                        and an in-context removal of the unit key direction;
  ``mamba2``            Mamba-2 selective state space (short causal convolution + scan);
  ``latent_attention``  attention over a cached low-rank latent per token (keys and values
                        are up-projections of it), causal sliding window, softmax with a
                        learned per-head sink, sigmoid output gate, no positional rotation.

"Regesun" is the design that stacks these three; its checkpoints are a ``config.json`` with
``architecture: "Regesun"`` and one safetensors file (``load_dir``).

One ``forward`` serves every step: a flat list of token rows cut into entries (portions of
prompts and single decoded tokens side by side, ``StepBatch``); attention layers read and
write the paged latent pool, recurrent layers their sequence's state slot
(``engine.seq_cache``).  Matrix products are vendor GEMMs (``torch.nn.functional.linear``,
bf16 with fp32 accumulation or true fp32); everything between them runs on the kernels of
``ops.seqmix``.  Sums over the residual, norms, scores, softmax, decays, gates of the
recurrences and the states stay in fp32 in both precisions.
"""
from __future__ import annotations

import dataclasses
import json
import os

import torch
import torch.nn.functional as F

from ..ops import PAGE
from ..ops import seqmix as sm


# ---------------------------------------------------------------------------- config
@dataclasses.dataclass(frozen=True)
class LayerSpec:
    kind: str
    mixer: dict
    mlp: dict | None


@dataclasses.dataclass(frozen=True)
class HybridConfig:
    name: str
    width: int
    vocab: int
    layers: tuple
    eps: float = 1e-5
    max_pos: int = 2048
    bos_id: int = 1
    eos_ids: tuple = ()
    is_moe: bool = False

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def hidden(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, c: dict, name: str | None = None) -> "HybridConfig":
        layers = tuple(LayerSpec(L["type"], dict(L["mixer"]), dict(L["mlp"]) if L.get("mlp") else None)
                       for L in c["layers"])
        for L in layers:
            if L.kind not in MIXERS:
                raise KeyError("unknown mixer %r (known: %s)" % (L.kind, ", ".join(sorted(MIXERS))))
            if L.mlp is not None and L.mlp.get("kind", "dense") != "dense":
                raise KeyError("unknown feed-forward kind %r" % L.mlp.get("kind"))
        eos = c.get("eos_token_id", ())
        eos = tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        return cls(name=name or str(c.get("architecture", "hybrid")).lower(), width=int(c["width"]),
                   vocab=int(c["vocab"]), layers=layers, eps=float(c["norm"]["eps"]),
                   max_pos=int(c["max_positions"]), bos_id=int(c.get("bos_token_id", 1)),
                   eos_ids=eos)

    def resolve(self, shapes: dict) -> "HybridConfig":
        """Fill the sizes that a config leaves to the checkpoint's tensor shapes (the rank of
        the generalized delta rule's decay projection).  shapes: tensor name -> shape."""
        layers = []
        for i, L in enumerate(self.layers):
            mx = dict(L.mixer)
            k = "l%d.mix.w1" % i
            if L.kind == "general_delta" and "decay_rank" not in mx and k in shapes:
                mx["decay_rank"] = int(tuple(shapes[k])[0])
            layers.append(LayerSpec(L.kind, mx, L.mlp))
        return dataclasses.replace(self, layers=tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": "Regesun", "width": self.width, "vocab": self.vocab,
                "max_positions": self.max_pos, "norm": {"eps": self.eps},
                "layers": [{"type": L.kind, "mixer": L.mixer, "mlp": L.mlp} for L in self.layers]}


def _vec(t, dev):
    return t.to(dev).float().contiguous()


# ---------------------------------------------------------------------------- step batch
class StepBatch:
    """Device-side description of one step (see ``ops.seqmix`` for the conventions).

    entries: list of (slot, pages, start, tokens) -- a sequence's state slot, its page list,
    the position of its first token in this step and the tokens.  want: per entry the
    indices (within its tokens) whose logits are needed."""

    def __init__(self, entries: list, want: list, device, min_pages: int = 1):
        host, meta = self.build_host(entries, want, min_pages)
        self._adopt(host.to(device), meta)

    @staticmethod
    def build_host(entries: list, want: list, min_pages: int = 1):
        """All of the step's metadata as one int32 host tensor + how to cut it."""
        ids, pos, row_ent, rows, ent, outs = [], [], [], [], [], []
        maxp = max([min_pages] + [len(e[1]) for e in entries])
        bt = torch.zeros(len(entries), maxp, dtype=torch.int32)
        r0 = 0
        for i, (slot, pages, start, toks) in enumerate(entries):
            n = len(toks)
            if n < 1:
                raise ValueError("an entry needs at least one token")
            if (start + n + PAGE - 1) // PAGE > len(pages):
                raise ValueError("entry %d: %d pages do not hold %d tokens" % (i, len(pages), start + n))
            bt[i, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
            ids += list(toks)
            pos += range(start, start + n)
            row_ent += [i] * n
            rows += [pages[p // PAGE] * PAGE + p % PAGE for p in range(start, start + n)]
            ent.append((r0, n, start, slot))
            outs += [r0 + w for w in want[i]]
            r0 += n
        parts = [torch.tensor(x, dtype=torch.int32).reshape(-1)
                 for x in (ids, pos, row_ent, rows, ent, outs or [0])] + [bt.reshape(-1)]
        meta = {"R": r0, "E": len(entries), "ent_host": ent, "n_out": len(outs),
                "max_pos": max(pos), "maxp": maxp, "sizes": [p.numel() for p in parts]}
        return torch.cat(parts), meta

    def _adopt(self, flat, meta):
        """flat: the device copy of ``build_host``'s tensor (one host -> device copy)."""
        self.flat, self.meta = flat, meta
        self.R, self.E = meta["R"], meta["E"]
        self.ent_host, self.n_out, self.max_pos = meta["ent_host"], meta["n_out"], meta["max_pos"]
        # most keys any row of this step can see; a batch that is reloaded for a captured
        # graph reports the whole width of its block tables instead
        self.max_keys = meta["max_pos"] + 1
        cut, o = [], 0
        for n in meta["sizes"]:
            cut.append(flat[o:o + n])
            o += n
        self.ids, self.pos, self.row_ent, self.cache_rows = cut[0], cut[1], cut[2], cut[3]
        self.ent = cut[4].view(-1, 4)
        self.out_rows = cut[5][:self.n_out]
        self.block_tables = cut[6].view(meta["E"], meta["maxp"])
        self._units = {}

    def reload(self, entries: list, want: list):
        """Same shape of step (rows, entries, wanted rows, table width), new contents, written
        into the device tensors this batch already has (a captured graph reads them)."""
        host, meta = self.build_host(entries, want, self.meta["maxp"])
        if meta["sizes"] != self.meta["sizes"] or meta["maxp"] != self.meta["maxp"]:
            raise ValueError("a reloaded step must have the shape of the captured one")
        self.flat.copy_(host, non_blocking=True)
        self.ent_host, self.max_pos = meta["ent_host"], meta["max_pos"]
        self.meta = meta

    def units(self, rows_per_wave: int):
        """Row groups for the matrix-core attention kernel (``ops.seqmix.make_units``)."""
        u = self._units.get(rows_per_wave)
        if u is None:
            u = self._units[rows_per_wave] = sm.make_units(self.ent_host, rows_per_wave).to(
                self.ids.device)
        return u


# ---------------------------------------------------------------------------- mixers
class Mixer:
    """One sequence mixer: weights + forward on a step.  ``cache_spec`` tells the sequence
    cache what the layer keeps between steps."""
    kind = ""

    def __init__(self, spec: dict, width: int, eps: float):
        self.spec, self.width, self.eps = spec, width, eps

    def tensor_shapes(self) -> dict:
        raise NotImplementedError

    def load(self, get, dtype, dev):
        raise NotImplementedError

    def cache_spec(self):
        return None

    def forward(self, h, b: StepBatch, cache, layer: int):
        raise NotImplementedError


class GeneralDelta(Mixer):
    kind = "general_delta"
    LOW_RANK = 32

    def tensor_shapes(self):
        n, W = self.spec["heads"] * self.spec["dim"], self.width
        lr = int(self.spec.get("decay_rank", self.LOW_RANK))
        return {"r": (n, W), "k": (n, W), "v": (n, W), "g": (n, W), "a": (n, W), "a.b": (n,),
                "w1": (lr, W), "w2": (n, lr), "w0": (n,), "norm": (n,), "o": (W, n)}

    def load(self, get, dtype, dev):
        self.H, self.D = int(self.spec["heads"]), int(self.spec["dim"])
        self.n = self.H * self.D
        # one projection for everything that reads the layer input: r | k | v | g | a | w1
        self.w_in = torch.cat([get(k) for k in ("r", "k", "v", "g", "a", "w1")], 0).to(dev, dtype).contiguous()
        self.w2 = get("w2").to(dev, dtype).contiguous()
        self.w0, self.ab, self.normw = _vec(get("w0"), dev), _vec(get("a.b"), dev), _vec(get("norm"), dev)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("state", {"S": (self.H, self.D, self.D)})

    def forward(self, h, b, cache, layer):
        n = self.n
        proj = F.linear(h, self.w_in)
        low = proj[:, 5 * n:]
        sm.tanh_(low)
        lo = F.linear(low, self.w2)
        out = torch.empty(b.R, n, device=h.device, dtype=h.dtype)
        sm.gdelta_scan(proj[:, 0:n], proj[:, n:2 * n], proj[:, 2 * n:3 * n], proj[:, 3 * n:4 * n],
                       proj[:, 4 * n:5 * n], lo, self.w0, self.ab, self.normw,
                       cache.state[layer]["S"], b.ent, b.ent_host, out, self.H, self.D, self.eps)
        return F.linear(out, self.wo)


class Mamba2(Mixer):
    kind = "mamba2"

    def _dims(self):
        s = self.spec
        self.H, self.P, self.N, self.G = int(s["heads"]), int(s["vdim"]), int(s["state"]), int(s["groups"])
        self.K, self.ng = int(s["conv"]), int(s.get("norm_groups", 1))
        self.inner = self.H * self.P
        self.C = self.inner + 2 * self.G * self.N

    def tensor_shapes(self):
        self._dims()
        return {"in": (2 * self.inner + 2 * self.G * self.N + self.H, self.width),
                "conv": (self.C, self.K), "conv.b": (self.C,), "dt_bias": (self.H,),
                "A_log": (self.H,), "D": (self.H,), "norm": (self.inner,),
                "o": (self.width, self.inner)}

    def load(self, get, dtype, dev):
        self._dims()
        if self.H % self.G or self.inner % self.ng:
            raise ValueError("mamba2: heads %d / groups %d / norm groups %d do not divide"
                             % (self.H, self.G, self.ng))
        self.w_in = get("in").to(dev, dtype).contiguous()
        self.cw, self.cb = _vec(get("conv"), dev), _vec(get("conv.b"), dev)
        self.dt_bias, self.A_log, self.Dp = (_vec(get(k), dev) for k in ("dt_bias", "A_log", "D"))
        self.normw = _vec(get("norm"), dev)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("state", {"S": (self.H, self.N, self.P), "tail": (self.K - 1, self.C)})

    def forward(self, h, b, cache, layer):
        st = cache.state[layer]
        zx = F.linear(h, self.w_in)
        conv = torch.empty(b.R, self.C, device=h.device, dtype=torch.float32)
        sm.mamba_conv(zx, self.inner, self.cw, self.cb, st["tail"], b.ent, b.ent_host, b.row_ent, conv)
        y = torch.empty(b.R, self.inner, device=h.device, dtype=torch.float32)
        sm.mamba_scan(conv, zx, self.inner, self.inner + self.C, self.dt_bias, self.A_log, self.Dp,
                      st["S"], st["tail"], b.ent, b.ent_host, y, self.H, self.P, self.N, self.G)
        yn = torch.empty(b.R, self.inner, device=h.device, dtype=h.dtype)
        sm.rmsnorm(y, self.normw, self.eps, yn, parts=self.ng)
        return F.linear(yn, self.wo)


class LatentAttention(Mixer):
    kind = "latent_attention"

    def _dims(self):
        s = self.spec
        self.H, self.D, self.V, self.rank = int(s["heads"]), int(s["dim"]), int(s["vdim"]), int(s["kv_rank"])
        self.win = int(s["mask"]["size"]) if s.get("mask") else 1 << 30
        self.scale = float(s["scale"]) if "scale" in s else self.D ** -0.5

    def tensor_shapes(self):
        self._dims()
        H, D, V, r, W = self.H, self.D, self.V, self.rank, self.width
        return {"q": (H * D, W), "dkv": (r, W), "dkv.norm": (r,), "uk": (H * D, r),
                "uv": (H * V, r), "sink": (H,), "g": (H * V, W), "o": (W, H * V)}

    def load(self, get, dtype, dev):
        self._dims()
        H, D, V, r = self.H, self.D, self.V, self.rank
        # one projection for everything that reads the layer input: q | latent | gate
        self.w_in = torch.cat([get("q"), get("dkv"), get("g")], 0).to(dev, dtype).contiguous()
        self.cnorm = _vec(get("dkv.norm"), dev)
        # keys and values are never formed: the query is carried into latent space with
        # W_uk (per head [D, rank]) and the attended latent leaves through W_uv^T
        self.uk = get("uk").to(dev, dtype).view(H, D, r).contiguous()
        self.uvt = get("uv").to(dev, dtype).view(H, V, r).transpose(1, 2).contiguous()
        self.sink = _vec(get("sink"), dev)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("paged", self.rank)

    def forward(self, h, b, cache, layer):
        H, D, V, r = self.H, self.D, self.V, self.rank
        pool = cache.paged[layer]
        proj = F.linear(h, self.w_in)
        sm.rmsnorm(proj[:, H * D:H * D + r], self.cnorm, self.eps, pool, out_rows=b.cache_rows)
        qa = torch.bmm(proj[:, :H * D].view(b.R, H, D).transpose(0, 1), self.uk)   # [H, R, rank]
        ol = torch.empty_like(qa)
        units = b.units(sm.latent_rows_per_wave(H)) if sm.latent_mfma_ok(qa, pool) else None
        sm.latent_attn(qa, pool, b.block_tables, b.row_ent, b.pos, self.sink, self.scale, self.win,
                       ol, PAGE, units=units, max_keys=b.max_keys)
        o = torch.bmm(ol, self.uvt)                                                # [H, R, V]
        gated = torch.empty(b.R, H * V, device=h.device, dtype=h.dtype)
        sm.sigmoid_gate(o, proj[:, H * D + r:], gated, H, V)
        return F.linear(gated, self.wo)


MIXERS = {c.kind: c for c in (GeneralDelta, Mamba2, LatentAttention)}


class DenseFF:
    """Clamped gated feed-forward (``ops.seqmix.ff_act``)."""

    def __init__(self, spec: dict, width: int):
        self.spec, self.width = spec, width
        self.F, self.limit = int(spec["ff"]), float(spec["limit"])

    def tensor_shapes(self):
        return {"gate": (self.F, self.width), "up": (self.F, self.width), "down": (self.width, self.F)}

    def load(self, get, dtype, dev):
        self.w_gu = torch.cat([get("gate"), get("up")], 0).to(dev, dtype).contiguous()
        self.w_down = get("down").to(dev, dtype).contiguous()

    def forward(self, h):
        gu = F.linear(h, self.w_gu)
        act = torch.empty(h.shape[0], self.F, device=h.device, dtype=h.dtype)
        sm.ff_act(gu, act, self.limit)
        return F.linear(act, self.w_down)


# ---------------------------------------------------------------------------- weights
class HybridLayer:
    def __init__(self, spec: LayerSpec, cfg: HybridConfig):
        self.mixer = MIXERS[spec.kind](spec.mixer, cfg.width, cfg.eps)
        self.ff = DenseFF(spec.mlp, cfg.width) if spec.mlp is not None else None
        self.norm1 = self.norm1b = self.ls1 = self.norm2 = self.norm2b = self.ls2 = None

    def tensor_shapes(self, W):
        d = {"norm1": (W,), "norm1b": (W,), "ls1": (W,)}
        d.update({"mix." + k: s for k, s in self.mixer.tensor_shapes().items()})
        if self.ff is not None:
            d.update({"norm2": (W,), "norm2b": (W,), "ls2": (W,)})
            d.update({"mlp." + k: s for k, s in self.ff.tensor_shapes().items()})
        return d


def tensor_shapes(cfg: HybridConfig) -> dict:
    """name -> shape of every tensor of a checkpoint of this config."""
    W = cfg.width
    d = {"embed": (cfg.vocab, W), "pos": (cfg.max_pos, W), "final.norm": (W,), "head": (cfg.vocab, W)}
    for i, spec in enumerate(cfg.layers):
        d.update({"l%d.%s" % (i, k): s for k, s in HybridLayer(spec, cfg).tensor_shapes(W).items()})
    return d


class HybridWeights:
    """The weight store: matrices in the activation dtype ([out, in], as stored), vectors in
    fp32.  ``dtype`` is torch.bfloat16 (serving) or torch.float32 (exact)."""

    def __init__(self, cfg: HybridConfig, sd, device, dtype=torch.bfloat16):
        cfg = cfg.resolve({k: v.shape for k, v in sd.items()})
        self.cfg, self.dtype = cfg, dtype
        dev = self.device = torch.device(device)
        want = tensor_shapes(cfg)
        for k, s in want.items():
            if k not in sd:
                raise KeyError("checkpoint lacks tensor %r" % k)
            if tuple(sd[k].shape) != tuple(s):
                raise ValueError("tensor %r has shape %s, the config gives %s" % (k, tuple(sd[k].shape), s))
        self.embed = sd["embed"].to(dev, dtype).contiguous()
        self.pos = sd["pos"].to(dev, dtype).contiguous()
        self.final_norm = _vec(sd["final.norm"], dev)
        self.head = sd["head"].to(dev, dtype).contiguous()
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            L = HybridLayer(spec, cfg)
            p = "l%d." % i
            L.mixer.load(lambda k, p=p: sd[p + "mix." + k], dtype, dev)
            L.norm1, L.norm1b, L.ls1 = (_vec(sd[p + k], dev) for k in ("norm1", "norm1b", "ls1"))
            if L.ff is not None:
                L.ff.load(lambda k, p=p: sd[p + "mlp." + k], dtype, dev)
                L.norm2, L.norm2b, L.ls2 = (_vec(sd[p + k], dev) for k in ("norm2", "norm2b", "ls2"))
            self.layers.append(L)

    @classmethod
    def random(cls, cfg: HybridConfig, device="cuda", seed: int = 0, dtype=torch.bfloat16):
        return cls(cfg, random_state_dict(cfg, seed), device, dtype)

    def cache_specs(self) -> list:
        return [L.mixer.cache_spec() for L in self.layers]


def random_state_dict(cfg: HybridConfig, seed: int = 0) -> dict:
    """A random checkpoint (bf16 values): projections ~ N(0, 1/in), gains near 1, decay and
    step parameters in the ranges where the recurrences neither vanish nor blow up."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for k, s in tensor_shapes(cfg).items():
        leaf = k.split(".", 1)[1] if k.startswith("l") and "." in k else k
        if len(s) == 2 and not leaf.endswith("mix.conv"):
            t = torch.randn(*s, generator=g) / (s[1] ** 0.5 if k not in ("embed", "pos") else 1.0)
        elif leaf.endswith("mix.conv"):
            t = torch.randn(*s, generator=g) * 0.5
        elif leaf.endswith(("norm1", "norm2", "norm1b", "norm2b", "mix.norm", "dkv.norm")) or k == "final.norm":
            t = 1.0 + 0.1 * torch.randn(*s, generator=g)
        elif leaf in ("ls1", "ls2"):
            t = 0.5 + 0.1 * torch.randn(*s, generator=g)
        elif leaf.endswith("A_log"):
            t = torch.rand(*s, generator=g) * 1.5 - 1.0
        elif leaf.endswith(("dt_bias", "mix.D")):
            t = torch.randn(*s, generator=g) * 0.5
        else:
            t = torch.randn(*s, generator=g) * 0.5
        sd[k] = t.to(torch.bfloat16)
    return sd


def load_dir(path: str, device="cuda", dtype=torch.bfloat16):
    """(config, weights) of a checkpoint folder: ``config.json`` + ``model.safetensors``."""
    from safetensors.torch import load_file

    with open(os.path.join(path, "config.json")) as f:
        cfg = HybridConfig.from_dict(json.load(f), name=os.path.basename(os.path.normpath(path)))
    sd = load_file(os.path.join(path, "model.safetensors"))
    w = HybridWeights(cfg, sd, device, dtype)
    return w.cfg, w


# ---------------------------------------------------------------------------- model
class HybridModel:
    def __init__(self, weights: HybridWeights, cache):
        self.w, self.cfg, self.cache = weights, weights.cfg, cache
        self.device, self.dtype = weights.device, weights.dtype

    @torch.no_grad()
    def forward(self, b: StepBatch, layer_out=None):
        """Run one step; returns fp32 logits [n_out, vocab] of the wanted rows (None when no
        row is wanted).  layer_out: optional list that receives the residual stream after
        every layer (debugging / layer-by-layer checks)."""
        cfg, w = self.cfg, self.w
        if b.max_pos >= cfg.max_pos:
            raise ValueError("position %d exceeds the model's %d positions" % (b.max_pos, cfg.max_pos))
        x = torch.empty(b.R, cfg.width, device=self.device, dtype=torch.float32)
        sm.embed_pos(w.embed, w.pos, b.ids, b.pos, x)
        h = torch.empty(b.R, cfg.width, device=self.device, dtype=self.dtype)
        # every post-sublayer pass (norm, layer scale, residual add) also forms the next
        # sublayer's normed input from the updated rows
        sm.rmsnorm(x, w.layers[0].norm1, cfg.eps, h)
        for i, L in enumerate(w.layers):
            after = w.layers[i + 1].norm1 if i + 1 < len(w.layers) else None
            m = L.mixer.forward(h, b, self.cache, i)
            sm.norm_scale_add(x, m, L.norm1b, L.ls1, cfg.eps,
                              next_w=L.norm2 if L.ff is not None else after, next_out=h)
            if L.ff is not None:
                sm.norm_scale_add(x, L.ff.forward(h), L.norm2b, L.ls2, cfg.eps, next_w=after,
                                  next_out=h)
            if layer_out is not None:
                layer_out.append(x.clone())
        if b.n_out == 0:
            return None
        hn = torch.empty(b.n_out, cfg.width, device=self.device, dtype=self.dtype)
        sm.rmsnorm(x, w.final_norm, cfg.eps, hn, in_rows=b.out_rows)
        return F.linear(hn, w.head).float()
