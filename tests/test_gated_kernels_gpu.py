"""HIP kernels of the window-attention / gated-scan / expert ops of ops.seqmix against the
PyTorch rendering of the same ops (CPU tensors), in fp32 and bf16, at sizes that are not
multiples of the kernels' tiles, with several entries per step and state carried over a
second step."""
import pytest
import torch

from p2p_llm_chat_go_amd.ops import seqmix as sm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64


def _ents(lens, starts, slots):
    ent, r0 = [], 0
    for n, s, sl in zip(lens, starts, slots):
        ent.append((r0, n, s, sl))
        r0 += n
    row_ent = [i for i, e in enumerate(ent) for _ in range(e[1])]
    return ent, torch.tensor(ent, dtype=torch.int32), torch.tensor(row_ent, dtype=torch.int32), r0


def _tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-4, atol=2e-5)


def _d(*ts):
    return [t.to(DEV) for t in ts]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wide,parts", [(200, 1), (200, 5), (8200, 2)])
def test_embed_gate_norm_add(dt, wide, parts):
    g = torch.Generator().manual_seed(0)
    Vc, W, R = 50, wide, 21
    emb = torch.randn(Vc, W, generator=g).to(dt)
    ids = torch.randint(0, Vc, (R,), generator=g, dtype=torch.int32)
    x1, h1 = torch.empty(R, W), torch.empty(R, W, dtype=dt)
    x2, h2 = torch.empty(R, W, device=DEV), torch.empty(R, W, dtype=dt, device=DEV)
    sm.embed_rows(emb, ids, x1, h1)
    sm.embed_rows(emb.to(DEV), ids.to(DEV), x2, h2)
    torch.testing.assert_close(x2.cpu(), x1, rtol=0, atol=0)
    torch.testing.assert_close(h2.cpu(), h1, rtol=0, atol=0)
    big = torch.randn(R, 2 * W + 3, generator=g).to(dt)     # y and gate as column views
    gb, w = torch.randn(W, generator=g), torch.randn(W, generator=g)
    bigd = big.to(DEV)
    sm.gate_norm_add(x1, big[:, :W], big[:, W + 3:], gb, w, parts, 1e-5, next_out=h1)
    sm.gate_norm_add(x2, bigd[:, :W], bigd[:, W + 3:], gb.to(DEV), w.to(DEV), parts, 1e-5, next_out=h2)
    torch.testing.assert_close(x2.cpu(), x1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h2.cpu().float(), h1.float(), **_tol(dt))
    sm.gate_norm_add(x2, bigd[:, :W], bigd[:, W + 3:], gb.to(DEV), w.to(DEV), parts, 1e-5)
    sm.gate_norm_add(x1, big[:, :W], big[:, W + 3:], gb, w, parts, 1e-5)
    torch.testing.assert_close(x2.cpu(), x1, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_glu_softcap(dt):
    g = torch.Generator().manual_seed(1)
    R, Fd = 9, 70
    gu = (torch.randn(R, 2 * Fd, generator=g) * 2).to(dt)
    a = sm.glu_act(gu, torch.empty(R, Fd, dtype=dt))
    b = sm.glu_act(gu.to(DEV), torch.empty(R, Fd, dtype=dt, device=DEV))
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    y = (torch.randn(R, 333, generator=g) * 40).to(dt)
    a = sm.softcap(y, 25.0, torch.empty(R, 333))
    b = sm.softcap(y.to(DEV), 25.0, torch.empty(R, 333, device=DEV))
    torch.testing.assert_close(b.cpu(), a, rtol=1e-5, atol=1e-5)


ATTN_SHAPES = [
    # H, G, D, V, rotated channels, window
    (6, 2, 24, 40, 16, 37),      # three heads per key/value head, part of the head rotated
    (4, 4, 16, 8, 16, 1000),     # one head per key/value head, window never reached
    (5, 1, 40, 72, 0, 1),        # no rotation, window of one
    (16, 2, 80, 112, 80, 100),   # eight heads per key/value head
    (34, 2, 8, 16, 4, 70),       # more heads per key/value head than a wavefront's pairs
    (3, 1, 7, 5, 4, 11),         # odd sizes: the last channel of a head has no partner
]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V,rot,win", ATTN_SHAPES)
def test_window_attention(dt, H, G, D, V, rot, win):
    g = torch.Generator().manual_seed(2)
    # three sequences: a prompt from 0, a portion that continues at 150, one decoded token at 131
    lens, starts = [70, 9, 1], [0, 150, 131]
    ent, ent_t, row_ent, R = _ents(lens, starts, [0, 1, 2])
    pos = torch.tensor([s + i for n, s in zip(lens, starts) for i in range(n)], dtype=torch.int32)
    n_pages, maxp = 12, 3
    bt = torch.tensor([[3, 5, 0], [7, 2, 9], [1, 4, 8]], dtype=torch.int32)
    rows = torch.tensor([int(bt[e, p // PAGE]) * PAGE + p % PAGE
                         for e, (n, s) in enumerate(zip(lens, starts)) for p in range(s, s + n)],
                        dtype=torch.int32)
    pool = torch.randn(n_pages * PAGE, G * (D + V), generator=g).to(dt)
    nq, nk, nv = H * D, G * D, G * V
    proj = torch.randn(R, nq + nk + nv + 5, generator=g).to(dt)
    qw, kw = 1 + 0.1 * torch.randn(nq, generator=g), 1 + 0.1 * torch.randn(nk, generator=g)
    inv = sm.rope_inv_freq(3000.0, rot, "cpu")
    sink = torch.randn(H, generator=g)
    q1, q2 = torch.empty(R, nq, dtype=dt), torch.empty(R, nq, dtype=dt, device=DEV)
    pool2 = pool.to(DEV)
    sm.qk_norm_rope_store(proj, H, G, D, V, qw, kw, inv, pos, rows, pool, 1e-5, q1)
    sm.qk_norm_rope_store(proj.to(DEV), H, G, D, V, *_d(qw, kw, inv, pos, rows), pool2, 1e-5, q2)
    torch.testing.assert_close(q2.cpu().float(), q1.float(), **_tol(dt))
    torch.testing.assert_close(pool2.cpu().float(), pool.float(), **_tol(dt))
    pool2.copy_(pool)
    q2.copy_(q1)
    o1 = torch.empty(R, H * V + 8, dtype=dt)[:, 8:]
    sm.window_attn(q1, pool, bt, row_ent, pos, sink, 0.3, win, o1, PAGE, H, G, D, V, out_scale=0.7)
    for mfma in ([False, True] if dt == torch.bfloat16 else [False]):
        for max_keys in (None, 300):    # whole windows / windows cut into runs
            o2 = torch.empty(R, H * V + 8, dtype=dt, device=DEV)[:, 8:]
            units = None
            if mfma:
                if not sm.window_mfma_ok(q2, pool2, D, V):
                    assert D % 8 or V % 8    # only sizes off the 16-byte grid stay off the matrix cores
                    continue
                units = sm.make_units(ent, sm.window_rows_per_wave(H // G)).to(DEV)
            sm.window_attn(q2, pool2, *_d(bt, row_ent, pos, sink), 0.3, win, o2, PAGE, H, G, D, V,
                           units=units, max_keys=max_keys, out_scale=0.7)
            torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))


SCAN_SHAPES = [(3, 3, 20, 12), (4, 2, 56, 24), (2, 1, 40, 72), (1, 1, 130, 200), (6, 6, 8, 16)]


# portions walked token by token / long portions cut into chunks that run side by side
SCAN_LENS = [[37, 1, 5], [200, 3, 131]]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V", SCAN_SHAPES)
@pytest.mark.parametrize("lens", SCAN_LENS, ids=["short", "chunked"])
def test_hgrn2_scan(dt, H, G, D, V, lens):
    g = torch.Generator().manual_seed(3)
    n = H * D
    lower, fb, normw = torch.rand(n, generator=g) * 0.9, torch.randn(n, generator=g), \
        1 + 0.1 * torch.randn(V, generator=g)
    S1 = torch.randn(5, H, D, V, generator=g)
    S2 = S1.to(DEV)
    for starts in ([0, 7, 0], [lens[0], 8, lens[2]]):      # second step continues the first one's slots
        ent, ent_t, _re, R = _ents(lens, starts, [2, 0, 3])
        proj = torch.randn(R, 2 * n + H * V + 3, generator=g).to(dt)
        o1, o2 = torch.empty(R, H * V, dtype=dt), torch.empty(R, H * V, dtype=dt, device=DEV)
        sm.hgrn2_scan(proj, lower, fb, normw, S1, ent_t, ent, o1, H, D, V, 1e-5, out_scale=1.3)
        sm.hgrn2_scan(proj.to(DEV), *_d(lower, fb, normw), S2, ent_t.to(DEV), ent, o2, H, D, V, 1e-5,
                      out_scale=1.3)
        torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))
        torch.testing.assert_close(S2.cpu(), S1, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V", SCAN_SHAPES)
@pytest.mark.parametrize("taps", [1, 3])
@pytest.mark.parametrize("lens", SCAN_LENS, ids=["short", "chunked"])
def test_gated_delta_scan(dt, H, G, D, V, taps, lens):
    g = torch.Generator().manual_seed(4)
    C = 2 * G * D + H * V
    A_log, dt_bias = torch.rand(H, generator=g) * 1.5 - 1, torch.randn(H * D, generator=g) * 0.5
    normw = 1 + 0.1 * torch.randn(V, generator=g)
    cw, cb = torch.randn(C, taps, generator=g) * 0.5, torch.zeros(C)
    S1, tail1 = torch.randn(5, H, D, V, generator=g) * 0.1, torch.randn(5, taps - 1, C, generator=g)
    S2, tail2 = S1.to(DEV), tail1.to(DEV)
    for starts in ([0, 7, 0], [lens[0], 8, lens[2]]):
        ent, ent_t, row_ent, R = _ents(lens, starts, [2, 0, 3])
        big = torch.randn(R, C + H + H * D + H * V, generator=g).to(dt)
        bigd, entd = big.to(DEV), ent_t.to(DEV)
        c1, c2 = torch.empty(R, C), torch.empty(R, C, device=DEV)
        sm.mamba_conv(big, 0, cw, cb, tail1, ent_t, ent, row_ent, c1)
        sm.mamba_conv(bigd, 0, *_d(cw, cb), tail2, entd, ent, row_ent.to(DEV), c2)
        torch.testing.assert_close(c2.cpu(), c1, rtol=1e-4, atol=1e-5)
        sm.conv_tail_roll(big, 0, tail1, ent_t, ent, C)
        sm.conv_tail_roll(bigd, 0, tail2, entd, ent, C)
        torch.testing.assert_close(tail2.cpu(), tail1, rtol=0, atol=0)
        o1, o2 = torch.empty(R, H * V, dtype=dt), torch.empty(R, H * V, dtype=dt, device=DEV)
        a, b, gt = C + H, C, C + H + H * D
        sm.gated_delta_scan(c1, big[:, a:a + H * D], big[:, b:b + H], big[:, gt:], A_log, dt_bias,
                            normw, S1, ent_t, ent, o1, H, G, D, V, 1e-5, out_scale=0.9)
        sm.gated_delta_scan(c1.to(DEV), bigd[:, a:a + H * D], bigd[:, b:b + H], bigd[:, gt:],
                            *_d(A_log, dt_bias, normw), S2, entd, ent, o2, H, G, D, V, 1e-5,
                            out_scale=0.9)
        torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))
        torch.testing.assert_close(S2.cpu(), S1, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,groups,keep,top,W,Fd", [(12, 3, 2, 3, 72, 40), (8, 1, 1, 2, 64, 64),
                                                     (6, 6, 2, 2, 50, 33), (70, 7, 3, 5, 96, 24),
                                                     (5, 1, 1, 3, 40, 48)])
@pytest.mark.parametrize("R", [45, 300])     # few slots per expert / the large prompt tile
def test_experts(dt, E, groups, keep, top, W, Fd, R):
    g = torch.Generator().manual_seed(5)
    h = torch.randn(R, W, generator=g).to(dt)
    wr = torch.randn(E, W, generator=g) * 0.5
    res = []
    for dev in ("cpu", DEV):
        ids = torch.empty(R, top, dtype=torch.int32, device=dev)
        wts = torch.empty(R, top, device=dev)
        cnt = torch.empty(E, dtype=torch.int32, device=dev)
        rows = torch.full((E, R * top), -1, dtype=torch.int32, device=dev)
        sm.group_route(h.to(dev), wr.to(dev), top, groups, keep, ids, wts, cnt, rows)
        res.append((ids.cpu(), wts.cpu(), cnt.cpu(), rows.cpu()))
    (i1, w1, c1, r1), (i2, w2, c2, r2) = res
    # the same choice, except where two scores tie within rounding (then the weights agree)
    torch.testing.assert_close(w2, w1, rtol=1e-5, atol=1e-6)
    assert (i1 != i2).any(-1).float().mean() < 0.02
    assert int(c2.sum()) == R * top
    got = sorted(s_ for e in range(E) for s_ in r2[e, :int(c2[e])].tolist())
    assert got == list(range(R * top))           # every slot in exactly one expert's list
    for e in range(E):
        assert all(int(i2.reshape(-1)[s_]) == e for s_ in r2[e, :int(c2[e])].tolist())
    c1, r1 = c2, r2
    # grouped products through the device's own slot lists
    wg = (torch.randn(E, 2 * Fd, W, generator=g) / W ** 0.5).to(dt)
    wd = (torch.randn(E, W, Fd, generator=g) / Fd ** 0.5).to(dt)
    gu1, gu2 = torch.zeros(R * top, 2 * Fd, dtype=dt), torch.zeros(R * top, 2 * Fd, dtype=dt, device=DEV)
    sm.expert_gemm(h, top, wg, c1, r1, gu1, R * top)
    sm.expert_gemm(h.to(DEV), top, wg.to(DEV), c2.to(DEV), r2.to(DEV), gu2, R * top)
    torch.testing.assert_close(gu2.cpu().float(), gu1.float(), **_tol(dt))
    if Fd % 16 == 0:    # the activation in the first product's epilogue
        wi = sm.interleave_gate_up(wg[:, :Fd], wg[:, Fd:])
        a0 = sm.ff_act(gu1, torch.empty(R * top, Fd, dtype=dt), 0.9)
        a1 = sm.expert_gemm(h, top, wi, c1, r1, torch.zeros(R * top, Fd, dtype=dt), R * top, act_limit=0.9)
        a2 = sm.expert_gemm(h.to(DEV), top, wi.to(DEV), c2.to(DEV), r2.to(DEV),
                            torch.zeros(R * top, Fd, dtype=dt, device=DEV), R * top, act_limit=0.9)
        torch.testing.assert_close(a1.float(), a0.float(), **_tol(dt))
        torch.testing.assert_close(a2.cpu().float(), a1.float(), **_tol(dt))
    act = torch.randn(R * top, Fd, generator=g).to(dt)
    y1, y2 = torch.zeros(R * top, W, dtype=dt), torch.zeros(R * top, W, dtype=dt, device=DEV)
    sm.expert_gemm(act, 1, wd, c1, r1, y1, R * top)
    sm.expert_gemm(act.to(DEV), 1, wd.to(DEV), c2.to(DEV), r2.to(DEV), y2, R * top)
    torch.testing.assert_close(y2.cpu().float(), y1.float(), **_tol(dt))
    o1 = sm.expert_combine(y1, w1, torch.empty(R, W, dtype=dt))
    o2 = sm.expert_combine(y1.to(DEV), w1.to(DEV), torch.empty(R, W, dtype=dt, device=DEV))
    torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))
