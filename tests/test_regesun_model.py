"""The Regesun hybrid model on the engine against the plain oracle (tests/regesun_oracle.py).

Every test builds its own small configuration and random checkpoint, runs the oracle once
over whole sequences in float64, and drives the engine's step function / generate / server
in float32 (and bfloat16 with a loose bound).  The CPU variants exercise the model, cache,
batching and scheduling code with the ops' PyTorch rendering; the ``gpu`` variants run the
same cases on the HIP kernels.
"""
import pytest
import torch

import regesun_oracle as O
from p2p_llm_chat_go_amd.engine.hybrid import HybridEngine
from p2p_llm_chat_go_amd.models import hybrid as Hy
from p2p_llm_chat_go_amd.ops import PAGE

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]

GD = {"type": "general_delta", "mixer": {"heads": 3, "dim": 16}, "mlp": None}
MB = {"type": "mamba2", "mixer": {"heads": 4, "vdim": 8, "state": 16, "groups": 2, "conv": 4,
                                  "norm_groups": 1}, "mlp": None}
LA = {"type": "latent_attention", "mixer": {"heads": 2, "dim": 16, "vdim": 24, "kv_rank": 32,
                                            "mask": {"size": 9}, "scale": 0.3},
      "mlp": {"kind": "dense", "ff": 80, "limit": 1.5}}


def make(layers, width=64, vocab=97, seed=0, max_pos=512, eps=1e-5):
    c = {"architecture": "Regesun", "width": width, "vocab": vocab, "max_positions": max_pos,
         "norm": {"eps": eps}, "layers": layers}
    cfg = Hy.HybridConfig.from_dict(c)
    return c, cfg, Hy.random_state_dict(cfg, seed)


def engine(cfg, sd, dev, dtype=torch.float32, pages=24, slots=4, **kw):
    return HybridEngine(cfg, Hy.HybridWeights(cfg, sd, dev, dtype), dev, kv_pages=pages,
                        num_slots=slots, max_batch=slots, **kw)


def toks(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, ref, tol=2e-4):
    """Difference of logits rows, mean removed, RMS over the vocabulary, relative to the
    RMS of the reference logits."""
    got, ref = got.detach().cpu().double(), ref.double()
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    scale = (ref - ref.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    err = (d.pow(2).mean(-1).sqrt() / scale).max().item()
    assert err < tol, "relative logits error %.3g" % err


def run_whole(eng, key, t):
    out = eng.step([(key, t, list(range(len(t))))])
    eng.release(key)
    return out


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("layer", [GD, MB, LA, dict(GD, mlp=LA["mlp"])],
                         ids=["general_delta", "mamba2", "latent_attention", "delta+ff"])
def test_single_mechanism(dev, layer):
    c, cfg, sd = make([layer], seed=3)
    t = toks(70, cfg.vocab, 1)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "a", t), ref)


@pytest.mark.parametrize("dev", DEVICES)
def test_layers_match_oracle(dev):
    c, cfg, sd = make([GD, MB, LA, MB, GD, LA], seed=4)
    t = toks(40, cfg.vocab, 2)
    ref, lay = O.forward(c, sd, t, return_layers=True)
    eng = engine(cfg, sd, dev)
    got = []
    out = eng.step([("a", t, list(range(len(t))))], return_layers=got)
    for i, x in enumerate(got):
        torch.testing.assert_close(x.cpu().double(), lay[i], rtol=1e-4, atol=1e-4, msg="layer %d" % i)
    close(out, ref)


# ------------------------------------------------------------------ other sizes
VARIANTS = {
    # one head / one group everywhere, two convolution taps, no window reached
    "ones": [{"type": "general_delta", "mixer": {"heads": 1, "dim": 24}, "mlp": None},
             {"type": "mamba2", "mixer": {"heads": 1, "vdim": 16, "state": 8, "groups": 1, "conv": 2,
                                          "norm_groups": 1}, "mlp": None},
             {"type": "latent_attention", "mixer": {"heads": 1, "dim": 8, "vdim": 8, "kv_rank": 16,
                                                    "mask": {"size": 1000}, "scale": 1.0},
              "mlp": None}],
    # a group per head, norm groups = heads, sizes not multiples of 16, value size < key size
    "odd": [{"type": "mamba2", "mixer": {"heads": 3, "vdim": 20, "state": 12, "groups": 3, "conv": 5,
                                         "norm_groups": 3}, "mlp": {"kind": "dense", "ff": 50, "limit": 0.7}},
            {"type": "latent_attention", "mixer": {"heads": 5, "dim": 12, "vdim": 4, "kv_rank": 20,
                                                   "mask": {"size": 1}, "scale": 0.05},
             "mlp": None},
            {"type": "general_delta", "mixer": {"heads": 2, "dim": 40}, "mlp": None}],
    # attention first, window of two, wide state
    "wide": [{"type": "latent_attention", "mixer": {"heads": 3, "dim": 8, "vdim": 16, "kv_rank": 72,
                                                    "mask": {"size": 2}, "scale": 0.5},
              "mlp": {"kind": "dense", "ff": 33, "limit": 3.0}},
             {"type": "mamba2", "mixer": {"heads": 2, "vdim": 72, "state": 80, "groups": 2, "conv": 3,
                                          "norm_groups": 2}, "mlp": None},
             {"type": "general_delta", "mixer": {"heads": 1, "dim": 72}, "mlp": None}],
}


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_sizes(dev, name):
    c, cfg, sd = make(VARIANTS[name], width=48 if name != "wide" else 100, vocab=61, seed=5, eps=1e-3)
    t = toks(75, cfg.vocab, 3)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    # first part as a prompt, the rest in portions of 1, 2 and 5 tokens
    cuts, at = [40, 1, 2, 5, 1, 1, 2, 23], 0
    outs = []
    for n in cuts:
        outs.append(eng.step([("a", t[at:at + n], list(range(n)))]))
        at += n
    close(torch.cat(outs), ref)


# ------------------------------------------------------------------ prefill vs decode, portions
@pytest.mark.parametrize("dev", DEVICES)
def test_prefill_decode_and_portions(dev):
    c, cfg, sd = make([MB, GD, LA, GD, MB, LA], seed=6)
    n = 2 * PAGE + 21                      # crosses two page borders, many windows
    t = toks(n, cfg.vocab, 4)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "w", t), ref)
    # token by token from the first token on
    outs = [eng.step([("d", [x], [0])]) for x in t]
    eng.release("d")
    close(torch.cat(outs), ref)
    # portions of changing size, down to two tokens and one, cut inside pages and windows
    for sizes in ([2] * 20 + [63, 1, 1, 2, 40, 3], [5, 59, 1, 64, 7, 2, 3, 8]):
        at, outs = 0, []
        for s in sizes:
            s = min(s, n - at)
            if s <= 0:
                break
            outs.append(eng.step([("p", t[at:at + s], list(range(s)))]))
            at += s
        if at < n:
            outs.append(eng.step([("p", t[at:], list(range(n - at)))]))
        eng.release("p")
        close(torch.cat(outs), ref)


# ------------------------------------------------------------------ batches, reuse of pages and slots
@pytest.mark.parametrize("dev", DEVICES)
def test_mixed_batches_and_reuse(dev):
    c, cfg, sd = make([GD, LA, MB, LA], seed=7)
    lens = [150, 9, 70, 1, 33, 130, 64, 65]
    reqs = {i: toks(n, cfg.vocab, 10 + i) for i, n in enumerate(lens)}
    refs = {i: O.forward(c, sd, t) for i, t in reqs.items()}
    # a pool that holds three of the long requests at most: pages and slots must come back
    eng = engine(cfg, sd, dev, pages=8, slots=3)
    got = {i: [] for i in reqs}
    at = {i: 0 for i in reqs}
    waiting, live, step = sorted(reqs), [], 0
    sizes = [7, 1, 30, 2, 1, 64, 3, 1, 1, 19]
    while waiting or live:
        while waiting and len(live) < 3:
            need = sum(-(-len(reqs[i]) // PAGE) for i in live) + -(-len(reqs[waiting[0]]) // PAGE)
            if need > 7:
                break
            live.append(waiting.pop(0))
        entries = []
        for j, i in enumerate(live):
            if (step + j) % 4 == 3 and len(live) > 1:
                continue                      # a request may sit a step out
            n = min(sizes[(step + 3 * j) % len(sizes)], len(reqs[i]) - at[i])
            entries.append((i, reqs[i][at[i]:at[i] + n], list(range(n))))
            at[i] += n
        out = eng.step(entries)
        o = 0
        for i, tk, w in entries:
            got[i].append(out[o:o + len(w)])
            o += len(w)
        for i in [i for i in live if at[i] == len(reqs[i])]:
            eng.release(i)
            live.remove(i)
        step += 1
    assert eng.cache.live == 0 and eng.cache.allocator.free_pages == 7 and eng.cache.slots.free_slots == 3
    for i in reqs:
        close(torch.cat(got[i]), refs[i])


@pytest.mark.parametrize("dev", DEVICES)
def test_first_tokens_in_a_used_slot(dev):
    """A sequence that starts in a slot and pages another one left behind sees none of it:
    zero state, zero inputs before the convolution's first tap, no keys before position 0."""
    c, cfg, sd = make([MB, GD, LA], seed=8)
    eng = engine(cfg, sd, dev, pages=3, slots=1)
    a, b = toks(100, cfg.vocab, 20), toks(5, cfg.vocab, 21)
    eng.step([("a", a, [])])
    eng.release("a")
    ref = O.forward(c, sd, b)
    outs = [eng.step([("b", [b[0]], [0])]), eng.step([("b", b[1:3], [0, 1])]), eng.step([("b", b[3:], [0, 1])])]
    close(torch.cat(outs), ref)


# ------------------------------------------------------------------ far keys, edges, long decoding
def slow_decay(sd, cfg):
    """Make the recurrences remember: decays near 1, small steps."""
    for i, L in enumerate(cfg.layers):
        p = "l%d.mix." % i
        if L.kind == "general_delta":
            sd[p + "w0"] = torch.full_like(sd[p + "w0"], -6.0)
            sd[p + "w2"] = sd[p + "w2"] * 0.1
        if L.kind == "mamba2":
            sd[p + "A_log"] = torch.full_like(sd[p + "A_log"], -5.0)
    return sd


@pytest.mark.parametrize("dev", DEVICES)
def test_far_tokens_and_long_decoding(dev):
    c, cfg, sd = make([GD, MB, LA], seed=9)
    sd = slow_decay(sd, cfg)
    n = 3 * PAGE + 10
    t = toks(n, cfg.vocab, 30)
    ref = O.forward(c, sd, t)
    # the early tokens matter at the end: changing token 2 moves the last logits
    t2 = list(t)
    t2[2] = (t[2] + 1) % cfg.vocab
    ref2 = O.forward(c, sd, t2)
    assert (ref[-1] - ref2[-1]).abs().max() > 1e-3
    eng = engine(cfg, sd, dev)
    outs = [eng.step([("a", t[:20], list(range(20)))])]
    outs += [eng.step([("a", [x], [0])]) for x in t[20:]]          # 180+ decoded tokens
    close(torch.cat(outs), ref)
    eng.release("a")
    outs = [eng.step([("b", t2[:20], [])])] + [eng.step([("b", [x], [0])]) for x in t2[20:]]
    close(torch.cat(outs[1:])[-1:], ref2[-1:])


def spike_model(win, hot, qtok, beta=25.0, seed=11):
    """One attention layer, no position vectors, whose query projection is rebuilt so that
    the query of token ``qtok`` scores ``beta`` against the key of token ``hot`` in every
    head and far less against other keys: where ``hot`` is visible it takes nearly all the
    weight, so a window that is one token off changes the output at once."""
    mx = {"heads": 2, "dim": 16, "vdim": 16, "kv_rank": 24, "mask": {"size": win}, "scale": 0.25}
    c, cfg, sd = make([{"type": "latent_attention", "mixer": mx, "mlp": None}], width=32, vocab=50,
                      seed=seed)
    sd["pos"] = torch.zeros_like(sd["pos"])
    f = lambda k: sd[k].double()
    eps = c["norm"]["eps"]
    h = lambda tok: O.rms(f("embed")[tok], eps) * f("l0.norm1")
    lat = O.rms(f("l0.mix.dkv") @ h(hot), eps) * f("l0.mix.dkv.norm")
    k = (f("l0.mix.uk") @ lat).view(mx["heads"], mx["dim"])
    want_q = (beta / mx["scale"]) * k / (k * k).sum(-1, keepdim=True)          # q . k_hot * scale = beta
    hq = h(qtok)
    sd["l0.mix.q"] = (want_q.reshape(-1, 1) * hq[None, :] / (hq @ hq)).to(torch.bfloat16)
    return c, cfg, sd


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("n,win", [(PAGE + 5, 6), (PAGE, PAGE), (2 * PAGE + 1, PAGE + 1),
                                   (2 * PAGE + 10, PAGE), (40, 2)])
def test_window_edges(dev, n, win):
    """Keys just inside and just outside the window, in a prompt and when decoding, with the
    window's far edge on and off a page border."""
    hot, qtok = 7, 11
    c, cfg, sd = spike_model(win, hot, qtok)
    g = torch.Generator().manual_seed(n * 1000 + win)
    t = torch.randint(0, cfg.vocab, (n,), generator=g).tolist()
    t = [x if x != hot else 8 for x in t]
    t[-1] = qtok
    base = O.forward(c, sd, t)
    for edge in (win - 1, win):               # just inside, just outside the last row's window
        if n - 1 - edge < 0:
            continue
        tt = list(t)
        tt[n - 1 - edge] = hot
        ref = O.forward(c, sd, tt)
        moved = (ref[-1] - base[-1]).abs().max().item()
        assert (moved > 0.05) == (edge == win - 1), "the oracle's window edge (%g)" % moved
        eng = engine(cfg, sd, dev)
        close(run_whole(eng, "w", tt), ref)
        k = min(5, n - 1)
        outs = [eng.step([("d", tt[:n - k], list(range(n - k)))])]
        outs += [eng.step([("d", [x], [0])]) for x in tt[n - k:]]
        close(torch.cat(outs), ref)
        eng.release("d")


@pytest.mark.parametrize("dev", DEVICES)
def test_sink_counts_once(dev):
    """A large sink takes most of the softmax weight; leaving it out, or scaling it, would
    change the output by a factor."""
    c, cfg, sd = spike_model(8, 7, 11, beta=3.0, seed=12)
    sd["l0.mix.sink"] = torch.tensor([4.0, -3.0]).to(torch.bfloat16)
    t = toks(20, cfg.vocab, 40)
    ref = O.forward(c, sd, t)
    sd0 = dict(sd)
    sd0["l0.mix.sink"] = torch.tensor([-30.0, -30.0]).to(torch.bfloat16)
    assert (O.forward(c, sd0, t) - ref).abs().max() > 1e-2
    close(run_whole(engine(cfg, sd, dev), "a", t), ref)


# ------------------------------------------------------------------ bf16 serving precision
@pytest.mark.parametrize("dev", DEVICES)
def test_bfloat16(dev):
    c, cfg, sd = make([GD, MB, LA, GD, MB, LA], width=128, vocab=200, seed=13)
    t = toks(PAGE + 30, cfg.vocab, 50)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev, dtype=torch.bfloat16)
    whole = run_whole(eng, "a", t)
    close(whole, ref, tol=0.08)
    outs = [eng.step([("b", t[:50], list(range(50)))])] + [eng.step([("b", [x], [0])]) for x in t[50:]]
    close(torch.cat(outs), ref, tol=0.08)


# ------------------------------------------------------------------ generation
def oracle_greedy(c, sd, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(c, sd, seq)[-1].argmax()))
    return seq[len(prompt):]


def near_tie(c, sd, prompt, got, n):
    """Greedy tokens equal the oracle's, or differ only where its top two logits tie."""
    seq = list(prompt)
    for tkn in got[:n]:
        lg = O.forward(c, sd, seq)[-1]
        assert tkn == int(lg.argmax()) or float(lg.max() - lg[tkn]) < 1e-3 * float(lg.abs().max())
        seq.append(tkn)


@pytest.mark.parametrize("dev", DEVICES)
def test_generate_greedy(dev):
    c, cfg, sd = make([GD, MB, LA], seed=14)
    prompts = [toks(n, cfg.vocab, 60 + n) for n in (12, 70, 3)]
    eng = engine(cfg, sd, dev, max_prefill_tokens=32)      # prompts are cut into portions
    res = eng.generate(prompts, max_new_tokens=12, stop_on_eos=False)
    for p, r in zip(prompts, res):
        assert len(r.tokens) == 12 and r.prompt_eval_count == len(p)
        near_tie(c, sd, p, r.tokens, 12)
    assert eng.cache.live == 0 and eng.cache.slots.free_slots == 4


@pytest.mark.parametrize("dev", DEVICES)
def test_server_scheduler_greedy(dev):
    """Through the continuous-batching server: the native scheduler owns the pages, requests
    arrive while others decode, state slots are handed back and used again."""
    native = pytest.importorskip("p2p_llm_chat_go_amd.native")
    try:
        native.load()
    except Exception as e:  # noqa: BLE001
        pytest.skip("native runtime not built: %s" % e)
    from p2p_llm_chat_go_amd.engine.sampling import SamplingParams
    from p2p_llm_chat_go_amd.engine.server import EngineServer

    c, cfg, sd = make([GD, MB, LA], seed=15)
    eng = engine(cfg, sd, dev, pages=40, slots=2, max_prefill_tokens=48)
    srv = EngineServer(eng, max_batch=2, decode_chunk=4)
    try:
        prompts = [toks(n, cfg.vocab, 80 + n) for n in (20, 5, 66, 9, 31)]
        futs = [srv.submit(p, SamplingParams(max_tokens=10, stop_on_eos=False)) for p in prompts]
        for p, f in zip(prompts, futs):
            r = f.result(timeout=120)
            assert len(r["tokens"]) == 10
            near_tie(c, sd, p, r["tokens"], 10)
        assert eng.cache.slots.free_slots == 2
    finally:
        srv.close()


@pytest.mark.gpu
def test_decode_graph_matches_eager():
    """Greedy decoding through the captured step graph, replayed many times with eager steps
    of other requests in between, gives the tokens of the eager engine."""
    c, cfg, sd = make([GD, MB, LA, MB], seed=16)
    prompts = [toks(n, cfg.vocab, 90 + n) for n in (70, 5, 33)]
    w = Hy.HybridWeights(cfg, sd, "cuda:0", torch.bfloat16)
    outs = []
    for graph in (True, False):
        eng = HybridEngine(cfg, w, "cuda:0", kv_pages=24, num_slots=4, max_batch=4, use_graph=graph)
        res = eng.generate(prompts, max_new_tokens=40, stop_on_eos=False)
        res2 = eng.generate(prompts[:2], max_new_tokens=70, stop_on_eos=False)
        outs.append([r.tokens for r in res + res2])
        assert bool(eng._graphs) == graph
    assert outs[0] == outs[1]
    for p, t in zip(prompts, outs[0]):
        assert len(t) == 40


def test_trace_runner_cli(tmp_path):
    """bin/trace_run on a saved checkpoint: steps on stdin, logits files and 'done' lines out,
    finished requests hand their pages and slot back (the pool is smaller than the sum)."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file

    c, cfg, sd = make([GD, MB, LA], seed=17)
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(c))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model / "model.safetensors"))
    a, b, d = toks(90, cfg.vocab, 1), toks(40, cfg.vocab, 2), toks(100, cfg.vocab, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:50], "want": [0, 49]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[50:88], "want": []},
                                {"id": "b", "tokens": b[:39], "want": [38]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[39:], "want": [0]},
                                {"id": "a", "tokens": a[88:], "want": [0, 1]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "d", "tokens": d, "want": [99]}], "end": ["d"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "192", "--device", "cpu"],
                       input="".join(json.dumps(x) + "\n" for x in steps), capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == ["done %d" % i for i in range(4)]
    ra, rb, rd = (O.forward(c, sd, t) for t in (a, b, d))
    got = {i: torch.from_numpy(np.fromfile(out / ("%d.f32" % i), dtype="<f4").reshape(-1, cfg.vocab))
           for i in (0, 1, 2, 3)}
    close(got[0], ra[[0, 49]])
    close(got[1], rb[[38]])
    close(got[2], torch.stack([rb[39], ra[88], ra[89]]))
    close(got[3], rd[[99]])


def test_config_roundtrip_and_errors():
    c, cfg, sd = make([GD, MB, LA])
    assert Hy.HybridConfig.from_dict(cfg.to_dict()).layers == cfg.layers
    assert set(Hy.tensor_shapes(cfg)) == set(sd)
    bad = dict(sd)
    bad["l0.mix.w2"] = bad["l0.mix.w2"][:, :3]
    with pytest.raises(ValueError):
        Hy.HybridWeights(cfg, bad, "cpu", torch.float32)
    with pytest.raises(KeyError):
        Hy.HybridConfig.from_dict(dict(c, layers=[{"type": "nope", "mixer": {}, "mlp": None}]))
    eng = engine(cfg, sd, "cpu", pages=2, slots=1)
    eng.step([("a", [1, 2, 3], [2])])
    with pytest.raises(MemoryError):
        eng.step([("b", [1], [0])])          # no second state slot
    with pytest.raises(MemoryError):
        eng.step([("a", [1] * PAGE, [])])    # no second page
