"""The Rotutar hybrid model on the engine against the plain oracle (tests/rotutar_oracle.py).

Every test builds its own small configuration and random checkpoint, runs the oracle once
over whole sequences in float64, and drives the engine's step function / generate / server
in float32 (and bfloat16 with a loose bound).  The CPU variants exercise the model, cache,
batching and scheduling code with the ops' PyTorch rendering; the ``gpu`` variants run the
same cases on the HIP kernels.
"""
import copy

import pytest
import torch

import rotutar_oracle as O
from p2p_llm_chat_go_amd.engine.hybrid import HybridEngine
from p2p_llm_chat_go_amd.models import hybrid as Hy
from p2p_llm_chat_go_amd.ops import PAGE

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]

DENSE = {"kind": "dense", "ff": 72}
MOE = {"kind": "moe", "expert": {"ff": 24, "limit": 1.2},
       "router": {"experts": 9, "top": 3, "groups": {"count": 3, "keep": 2}}}
HG = {"type": "hgrn2", "mixer": {"heads": 3, "dim": 12, "vdim": 20}, "mlp": None}
LEFT = {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "mask": {"size": 9},
        "rot": {"base": 300.0, "dims": 10}, "scale": 0.4}
RIGHT = {"heads": 4, "kv_heads": 2, "dim": 20, "vdim": 12, "conv": 4}
PA = {"type": "parallel", "mixer": {"left": LEFT, "right": RIGHT, "left_scale": 0.7, "right_scale": 1.2},
      "mlp": None}


def layer(base, mlp=None, **mixer):
    L = copy.deepcopy(base)
    L["mlp"] = copy.deepcopy(mlp)
    L["mixer"].update(copy.deepcopy(mixer))
    return L


def make(layers, width=48, vocab=97, seed=0, eps=1e-5, groups=3, cap=20.0):
    c = {"architecture": "Rotutar", "width": width, "vocab": vocab, "norm": {"eps": eps, "groups": groups},
         "layers": copy.deepcopy(layers)}
    if cap:
        c["logit_softcap"] = cap
    cfg = Hy.HybridConfig.from_dict(c)
    sd = Hy.random_state_dict(cfg, seed)
    cfg = cfg.resolve({k: v.shape for k, v in sd.items()})
    return c, cfg, sd


def engine(cfg, sd, dev, dtype=torch.float32, pages=24, slots=4, **kw):
    return HybridEngine(cfg, Hy.HybridWeights(cfg, sd, dev, dtype), dev, kv_pages=pages,
                        num_slots=slots, max_batch=slots, **kw)


def toks(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, ref, tol=2e-4, over=0.0):
    """Difference of logits rows, mean removed, RMS over the vocabulary, relative to the
    RMS of the reference logits.  over: share of rows that may exceed the bound (bf16 rounding
    can move a router's choice between two experts with nearly equal scores)."""
    got, ref = got.detach().cpu().double(), ref.double()
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    scale = (ref - ref.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    err = d.pow(2).mean(-1).sqrt() / scale
    bad = (err >= tol).double().mean().item()
    assert bad <= over, "relative logits error %.3g, %.3g of the rows over %g" % (err.max().item(), bad, tol)


def run_whole(eng, key, t):
    out = eng.step([(key, t, list(range(len(t))))])
    eng.release(key)
    return out


def run_cuts(eng, key, t, cuts):
    at, outs = 0, []
    for n in cuts:
        n = min(n, len(t) - at)
        if n <= 0:
            break
        outs.append(eng.step([(key, t[at:at + n], list(range(n)))]))
        at += n
    if at < len(t):
        outs.append(eng.step([(key, t[at:], list(range(len(t) - at)))]))
    eng.release(key)
    return torch.cat(outs)


# ------------------------------------------------------------------ each mechanism alone
ALONE = {
    "hgrn2": [HG],
    "window_attention": [layer(PA, right_scale=0.0)],
    "gated_delta": [layer(PA, left_scale=0.0)],
    "parallel": [PA],
    "dense_ff": [layer(HG, DENSE)],
    "moe_ff": [layer(HG, MOE)],
}


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("name", sorted(ALONE))
def test_single_mechanism(dev, name):
    c, cfg, sd = make(ALONE[name], seed=3)
    t = toks(70, cfg.vocab, 1)
    ref = O.forward(c, sd, t)
    close(run_whole(engine(cfg, sd, dev), "a", t), ref)


@pytest.mark.parametrize("dev", DEVICES)
def test_layers_match_oracle(dev):
    c, cfg, sd = make([layer(HG, DENSE), layer(PA, MOE), layer(HG, MOE), PA, layer(PA, DENSE)], seed=4)
    t = toks(40, cfg.vocab, 2)
    ref, lay = O.forward(c, sd, t, return_layers=True)
    eng = engine(cfg, sd, dev)
    got = []
    out = eng.step([("a", t, list(range(len(t))))], return_layers=got)
    assert len(got) == len(lay)
    for i, x in enumerate(got):
        torch.testing.assert_close(x.cpu().double(), lay[i], rtol=1e-4, atol=1e-4, msg="layer %d" % i)
    close(out, ref)


def test_oracle_pieces():
    """The oracle's own building blocks on cases that can be worked out by hand."""
    # routing: 2 blocks of 3 experts, ranked by their top-2 sums of sigmoids
    z = torch.tensor([4.0, -9.0, -9.0, 2.0, 2.1, -9.0], dtype=torch.float64)
    ch, w = O.route(z, {"experts": 6, "top": 2, "groups": {"count": 2, "keep": 1}})
    assert ch == [4, 3]                      # expert 0 is the largest but its group loses
    assert abs(float(w[0]) - float(torch.sigmoid(z[4]))) < 1e-12
    ch, _ = O.route(z, {"experts": 6, "top": 2, "groups": {"count": 2, "keep": 2}})
    assert ch == [0, 4]
    # rotation: a quarter turn per position on the first pair, base 1 -> angle = position
    x = torch.zeros(3, 1, 4, dtype=torch.float64)
    x[:, 0, 0] = 1.0
    x[:, 0, 2] = 5.0
    r = O.rotate(x, 1.0, 2)
    torch.testing.assert_close(r[2, 0, :2], torch.tensor([torch.cos(torch.tensor(2.0)), torch.sin(torch.tensor(2.0))],
                                                         dtype=torch.float64))
    assert float(r[2, 0, 2]) == 5.0
    # convolution: last column multiplies the current token
    y = O.short_conv(torch.tensor([[1.0], [10.0], [100.0]]), torch.tensor([[2.0, 3.0]]))
    assert y.flatten().tolist() == [3.0, 32.0, 320.0]
    # group norm: every part has unit mean square
    g = O.group_norm(torch.tensor([[3.0, 4.0, 0.1, 0.2]]), torch.ones(4), 2, 0.0)
    torch.testing.assert_close((g.view(2, 2) ** 2).mean(-1), torch.ones(2))


# ------------------------------------------------------------------ other sizes
VARIANTS = {
    # one head, one kv head, one norm group, one tap, one expert group, top 1, no cap, no window reached
    "ones": dict(groups=1, cap=0.0, layers=[
        layer(HG, {"kind": "moe", "expert": {"ff": 16, "limit": 0.8},
                   "router": {"experts": 4, "top": 1, "groups": {"count": 1, "keep": 1}}},
              heads=1, dim=24, vdim=8),
        layer(PA, None,
              left={"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "mask": {"size": 1000},
                    "rot": {"base": 10.0, "dims": 8}, "scale": 1.0},
              right={"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 16, "conv": 1})]),
    # sizes that are not multiples of 8 or 16, window of one, two taps, every group kept
    "odd": dict(groups=2, cap=7.0, layers=[
        layer(PA, {"kind": "moe", "expert": {"ff": 10, "limit": 3.0},
                   "router": {"experts": 6, "top": 4, "groups": {"count": 3, "keep": 3}}},
              left={"heads": 5, "kv_heads": 5, "dim": 6, "vdim": 10, "mask": {"size": 1},
                    "rot": {"base": 40000.0, "dims": 2}, "scale": 0.05},
              right={"heads": 6, "kv_heads": 3, "dim": 10, "vdim": 6, "conv": 2}),
        layer(HG, {"kind": "dense", "ff": 50}, heads=5, dim=6, vdim=4)]),
    # wide states, window of two, five taps, value size above key size
    "wide": dict(groups=5, cap=50.0, layers=[
        layer(HG, None, heads=1, dim=72, vdim=80),
        layer(PA, DENSE,
              left={"heads": 4, "kv_heads": 1, "dim": 40, "vdim": 72, "mask": {"size": 2},
                    "rot": {"base": 1000.0, "dims": 40}, "scale": 0.5},
              right={"heads": 2, "kv_heads": 1, "dim": 72, "vdim": 80, "conv": 5})]),
}


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_sizes(dev, name):
    v = VARIANTS[name]
    c, cfg, sd = make(v["layers"], width=40 if name != "wide" else 100, vocab=61, seed=5, eps=1e-3,
                      groups=v["groups"], cap=v["cap"])
    t = toks(75, cfg.vocab, 3)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    # first part as a prompt, the rest in portions of 1, 2 and 5 tokens
    close(run_cuts(eng, "a", t, [40, 1, 2, 5, 1, 1, 2, 23]), ref)


# ------------------------------------------------------------------ prefill vs decode, portions
@pytest.mark.parametrize("dev", DEVICES)
def test_prefill_decode_and_portions(dev):
    c, cfg, sd = make([layer(PA, MOE), layer(HG, DENSE), PA], seed=6)
    n = 2 * PAGE + 21                      # crosses two page borders, many windows
    t = toks(n, cfg.vocab, 4)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "w", t), ref)
    # token by token from the first token on
    close(run_cuts(eng, "d", t, [1] * n), ref)
    # portions of changing size, down to two tokens and one, cut inside pages and windows
    for sizes in ([2] * 20 + [63, 1, 1, 2, 40, 3], [5, 59, 1, 64, 7, 2, 3, 8]):
        close(run_cuts(eng, "p", t, sizes), ref)


# ------------------------------------------------------------------ batches, reuse of pages and slots
@pytest.mark.parametrize("dev", DEVICES)
def test_mixed_batches_and_reuse(dev):
    c, cfg, sd = make([layer(HG, MOE), layer(PA, DENSE), PA], seed=7)
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
    zero states, zero inputs before the convolutions' first tap, no keys before position 0."""
    c, cfg, sd = make([HG, PA, layer(HG, MOE)], seed=8)
    eng = engine(cfg, sd, dev, pages=3, slots=1)
    a, b = toks(100, cfg.vocab, 20), toks(7, cfg.vocab, 21)
    eng.step([("a", a, [])])
    eng.release("a")
    ref = O.forward(c, sd, b)
    outs = [eng.step([("b", [b[0]], [0])]), eng.step([("b", b[1:3], [0, 1])]), eng.step([("b", b[3:], [0, 1, 2, 3])])]
    close(torch.cat(outs), ref)


# ------------------------------------------------------------------ far tokens, long decoding
def long_memory(sd, cfg):
    """Make the recurrences remember: forget gates near 1, decays near 1."""
    for i, L in enumerate(cfg.layers):
        p = "l%d.mix." % i
        if L.kind == "hgrn2":
            sd[p + "lower"] = torch.full_like(sd[p + "lower"], 0.992)
        if L.kind == "parallel":
            sd[p + "right.A_log"] = torch.full_like(sd[p + "right.A_log"], -6.0)
    return sd


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("which", ["hgrn2", "gated_delta"])
def test_far_tokens_and_long_decoding(dev, which):
    layers = [HG, layer(HG, DENSE)] if which == "hgrn2" else [layer(PA, DENSE, left_scale=0.3)]
    c, cfg, sd = make(layers, seed=9)
    sd = long_memory(sd, cfg)
    n = 3 * PAGE + 10
    t = toks(n, cfg.vocab, 30)
    ref = O.forward(c, sd, t)
    # the early tokens matter at the end, far outside the attention window: changing token 2
    # moves the last logits
    t2 = list(t)
    t2[2] = (t[2] + 1) % cfg.vocab
    ref2 = O.forward(c, sd, t2)
    assert (ref[-1] - ref2[-1]).abs().max() > 1e-3
    eng = engine(cfg, sd, dev)
    close(run_cuts(eng, "a", t, [20] + [1] * (n - 20)), ref)          # 180+ decoded tokens
    got = run_cuts(eng, "b", t2, [20] + [1] * (n - 20))
    close(got[-1:], ref2[-1:])


# ------------------------------------------------------------------ window edges, sink
def spike_model(win, hot, qtok, beta=25.0, seed=11, rot_dims=2):
    """Attention alone (the other branch scaled by zero), whose query projection is rebuilt so
    that every query points along the unrotated part of the key of token ``hot``: where
    ``hot`` is visible it takes nearly all the softmax weight, so a window that is one token
    off changes the output at once."""
    left = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "mask": {"size": win},
            "rot": {"base": 100.0, "dims": rot_dims}, "scale": 1.0}
    c, cfg, sd = make([layer(PA, None, left=left, left_scale=1.0, right_scale=0.0)], width=32, vocab=50,
                      seed=seed, groups=1, cap=0.0)
    f = lambda k: sd[k].double()
    eps = c["norm"]["eps"]
    H, G, D = left["heads"], left["kv_heads"], left["dim"]
    sd["l0.mix.left.k.norm"] = torch.ones_like(sd["l0.mix.left.k.norm"])
    sd["l0.mix.left.q.norm"] = torch.ones_like(sd["l0.mix.left.q.norm"])
    k = O.rms(f("l0.mix.left.k") @ f("embed")[hot], eps).view(G, D).clone()
    k[:, :rot_dims] = 0.0
    target = k.repeat_interleave(H // G, 0).reshape(-1)                  # [H * D]
    xq = f("embed")[qtok]
    sd["l0.mix.left.q"] = (target[:, None] * xq[None, :] / (xq @ xq)).to(torch.bfloat16)
    qn = O.rms(target[None, :], eps).view(H, D)
    c["layers"][0]["mixer"]["left"]["scale"] = beta / float((qn[0] * k[0]).sum())
    cfg = Hy.HybridConfig.from_dict(c).resolve({k_: v.shape for k_, v in sd.items()})
    return c, cfg, sd


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("n,win", [(PAGE + 5, 6), (PAGE, PAGE), (2 * PAGE + 1, PAGE + 1),
                                   (2 * PAGE + 10, PAGE), (40, 2), (3 * PAGE, 100)])
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
        close(run_cuts(eng, "d", tt, [n - k] + [1] * k), ref)
        # the hot key decoded alone, the query in a portion of two
        close(run_cuts(eng, "e", tt, [max(1, n - 1 - edge), 1] + [2] * n), ref)


@pytest.mark.parametrize("dev", DEVICES)
def test_sink_counts_once(dev):
    """A large sink takes most of the softmax weight; leaving it out, or scaling it, would
    change the output by a factor."""
    c, cfg, sd = spike_model(8, 7, 11, beta=3.0, seed=12, rot_dims=8)
    sd["l0.mix.left.sink"] = torch.tensor([4.0, -3.0, 2.0, 0.5]).to(torch.bfloat16)
    t = toks(20, cfg.vocab, 40)
    ref = O.forward(c, sd, t)
    sd0 = dict(sd)
    sd0["l0.mix.left.sink"] = torch.full((4,), -30.0).to(torch.bfloat16)
    assert (O.forward(c, sd0, t) - ref).abs().max() > 1e-2
    close(run_whole(engine(cfg, sd, dev), "a", t), ref)


@pytest.mark.parametrize("dev", DEVICES)
def test_rotation_depends_on_distance_only(dev):
    """The same tokens behind a prefix that the window no longer sees and that leaves no state
    (recurrent branch off): the rotation cancels to relative positions, in the engine too."""
    left = dict(LEFT, mask={"size": 5}, rot={"base": 30.0, "dims": 16})
    c, cfg, sd = make([layer(PA, None, left=left, right_scale=0.0)], seed=21)
    a = toks(30, cfg.vocab, 22)
    shifted = toks(PAGE + 3, cfg.vocab, 23) + a
    ref = O.forward(c, sd, a)
    ref_s = O.forward(c, sd, shifted)
    torch.testing.assert_close(ref_s[-20:], ref[-20:], rtol=1e-9, atol=1e-9)
    got = run_cuts(engine(cfg, sd, dev), "s", shifted, [PAGE + 3, 7, 1, 1, 2])
    close(got[-20:], ref[-20:])


# ------------------------------------------------------------------ bf16 serving precision
@pytest.mark.parametrize("dev", DEVICES)
def test_bfloat16(dev):
    c, cfg, sd = make([layer(HG, DENSE, heads=4, dim=16, vdim=32),
                       layer(PA, DENSE, left=dict(LEFT, dim=32, vdim=32, rot={"base": 300.0, "dims": 32}),
                             right=dict(RIGHT, dim=32, vdim=16)),
                       layer(HG, MOE, heads=4, dim=16, vdim=32)], width=128, vocab=200, seed=13, groups=4)
    t = toks(PAGE + 30, cfg.vocab, 50)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev, dtype=torch.bfloat16)
    # the experts sit in the last layer only: a choice that rounding moves between two experts
    # with nearly equal scores then changes that row alone, not the states after it
    close(run_whole(eng, "a", t), ref, tol=0.08, over=0.1)
    close(run_cuts(eng, "b", t, [50] + [1] * 44), ref, tol=0.08, over=0.1)


# ------------------------------------------------------------------ generation
def near_tie(c, sd, prompt, got, n):
    """Greedy tokens equal the oracle's, or differ only where its top two logits tie."""
    seq = list(prompt)
    for tkn in got[:n]:
        lg = O.forward(c, sd, seq)[-1]
        assert tkn == int(lg.argmax()) or float(lg.max() - lg[tkn]) < 1e-3 * float(lg.abs().max())
        seq.append(tkn)


@pytest.mark.parametrize("dev", DEVICES)
def test_generate_greedy(dev):
    c, cfg, sd = make([layer(HG, MOE), layer(PA, DENSE)], seed=14)
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

    c, cfg, sd = make([layer(HG, DENSE), layer(PA, MOE)], seed=15)
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
    c, cfg, sd = make([layer(HG, MOE), layer(PA, DENSE), layer(PA, MOE)], width=64, seed=16, groups=4)
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

    import numpy as np
    from safetensors.torch import save_file

    c, cfg, sd = make([layer(HG, MOE), PA], seed=17)
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


def test_preset_through_registry(tmp_path):
    """The preset and a saved checkpoint both reach the hybrid engine through the registry."""
    import json

    from safetensors.torch import save_file

    from p2p_llm_chat_go_amd.models import registry
    from p2p_llm_chat_go_amd.models.config import get_config

    cfg = get_config("tiny-rotutar")
    assert cfg.design == "Rotutar" and cfg.is_moe and not cfg.traits.positions
    sd = Hy.random_state_dict(cfg, 3)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    assert registry.is_hybrid_dir(str(tmp_path)) and registry.supports_dtype(str(tmp_path), torch.float32)
    cfg2, w = registry.load_checkpoint(str(tmp_path), "cpu", torch.float32)
    assert cfg2.layers == cfg.resolve({k: v.shape for k, v in sd.items()}).layers
    eng = registry.make_engine(cfg2, w, "cpu", kv_pages=6, num_slots=2, max_batch=2, dtype=torch.float32)
    p = toks(9, cfg.vocab, 5)
    r = eng.generate([p], max_new_tokens=4, stop_on_eos=False)[0]
    near_tie(cfg.to_dict(), sd, p, r.tokens, 4)


def test_config_roundtrip_and_errors():
    c, cfg, sd = make([layer(HG, MOE), layer(PA, DENSE)])
    again = Hy.HybridConfig.from_dict(cfg.to_dict())
    assert again.layers == cfg.layers and again.design == "Rotutar" and again.norm_groups == 3
    assert again.logit_softcap == 20.0 and again.is_moe
    assert set(Hy.tensor_shapes(cfg)) == set(sd) and "pos" not in sd
    bad = dict(sd)
    bad["l1.mix.right.q.conv"] = bad["l1.mix.right.q.conv"][:, :2]
    with pytest.raises(ValueError):
        Hy.HybridWeights(cfg, bad, "cpu", torch.float32)
    with pytest.raises(KeyError):
        Hy.HybridConfig.from_dict(dict(c, layers=[{"type": "nope", "mixer": {}, "mlp": None}]))
    with pytest.raises(KeyError):
        Hy.HybridConfig.from_dict(dict(c, layers=[layer(HG, {"kind": "nope"})]))
    with pytest.raises(ValueError):
        Hy.HybridConfig.from_dict(dict(c, norm={"eps": 1e-5, "groups": 7}))
    with pytest.raises(ValueError):       # more experts chosen than the kept groups hold
        make([layer(HG, dict(MOE, router={"experts": 9, "top": 4, "groups": {"count": 3, "keep": 1}}))])
    eng = engine(cfg, sd, "cpu", pages=2, slots=1)
    eng.step([("a", [1, 2, 3], [2])])
    with pytest.raises(MemoryError):
        eng.step([("b", [1], [0])])          # no second state slot
    with pytest.raises(MemoryError):
        eng.step([("a", [1] * PAGE, [])])    # no second page
