"""HIP kernels of ops.seqmix against the PyTorch rendering of the same ops (CPU tensors),
in fp32 and bf16, at sizes that are not multiples of the kernels' tiles, with several
entries per step and state carried over a second step."""
import pytest
import torch

from p2p_llm_chat_go_amd.ops import seqmix as sm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ents(lens, starts, slots):
    ent, r0 = [], 0
    for n, s, sl in zip(lens, starts, slots):
        ent.append((r0, n, s, sl))
        r0 += n
    row_ent = [i for i, e in enumerate(ent) for _ in range(e[1])]
    return ent, torch.tensor(ent, dtype=torch.int32), torch.tensor(row_ent, dtype=torch.int32), r0


def _tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wide", [200, 4100])   # rows kept in registers / rows read twice
def test_embed_norms(dt, wide):
    g = torch.Generator().manual_seed(0)
    V, W, R = 50, wide, 37
    emb, ptab = torch.randn(V, W, generator=g).to(dt), torch.randn(64, W, generator=g).to(dt)
    ids = torch.randint(0, V, (R,), generator=g, dtype=torch.int32)
    pos = torch.randint(0, 64, (R,), generator=g, dtype=torch.int32)
    a = sm.embed_pos(emb, ptab, ids, pos, torch.empty(R, W))
    b = sm.embed_pos(emb.to(DEV), ptab.to(DEV), ids.to(DEV), pos.to(DEV), torch.empty(R, W, device=DEV))
    torch.testing.assert_close(b.cpu(), a, rtol=0, atol=0)
    w = torch.randn(W, generator=g)
    for parts in (1, 4) if wide % 4 == 0 else (1,):
        o1 = sm.rmsnorm(a, w, 1e-5, torch.empty(R, W, dtype=dt), parts=parts)
        o2 = sm.rmsnorm(b, w.to(DEV), 1e-5, torch.empty(R, W, dtype=dt, device=DEV), parts=parts)
        torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))
    # gather + scatter
    inr = torch.tensor([5, 0, 36], dtype=torch.int32)
    outr = torch.tensor([7, -1, 2], dtype=torch.int32)
    y = a.to(dt)
    o1 = sm.rmsnorm(y, w, 1e-5, torch.zeros(9, W, dtype=dt), in_rows=inr, out_rows=outr)
    o2 = sm.rmsnorm(y.to(DEV), w.to(DEV), 1e-5, torch.zeros(9, W, dtype=dt, device=DEV),
                    in_rows=inr.to(DEV), out_rows=outr.to(DEV))
    torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))
    ls = torch.randn(W, generator=g)
    x1 = sm.norm_scale_add(a.clone(), y, w, ls, 1e-5)
    x2 = sm.norm_scale_add(b.clone(), y.to(DEV), w.to(DEV), ls.to(DEV), 1e-5)
    torch.testing.assert_close(x2.cpu(), x1, rtol=1e-5, atol=1e-5)
    # ... and the next sublayer's normed input in the same pass
    w2 = torch.randn(W, generator=g)
    h1, h2 = torch.empty(R, W, dtype=dt), torch.empty(R, W, dtype=dt, device=DEV)
    x1 = sm.norm_scale_add(a.clone(), y, w, ls, 1e-5, next_w=w2, next_out=h1)
    x2 = sm.norm_scale_add(b.clone(), y.to(DEV), w.to(DEV), ls.to(DEV), 1e-5, next_w=w2.to(DEV), next_out=h2)
    torch.testing.assert_close(x2.cpu(), x1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h2.cpu().float(), h1.float(), **_tol(dt))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_pointwise(dt):
    g = torch.Generator().manual_seed(1)
    R, H, V, Fd = 9, 3, 20, 70
    x = torch.randn(R, 40, generator=g).to(dt)
    a = sm.tanh_(x[:, 10:33].clone())
    big = x.to(DEV)
    b = sm.tanh_(big[:, 10:33])
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    o, gt = torch.randn(H, R, V, generator=g).to(dt), torch.randn(R, H * V, generator=g).to(dt)
    a = sm.sigmoid_gate(o, gt, torch.empty(R, H * V, dtype=dt), H, V)
    b = sm.sigmoid_gate(o.to(DEV), gt.to(DEV), torch.empty(R, H * V, dtype=dt, device=DEV), H, V)
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    gu = (3 * torch.randn(R, 2 * Fd, generator=g)).to(dt)
    a = sm.ff_act(gu, torch.empty(R, Fd, dtype=dt), 1.75)
    b = sm.ff_act(gu.to(DEV), torch.empty(R, Fd, dtype=dt, device=DEV), 1.75)
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))


@pytest.fixture(params=[64, 8], ids=["onepass", "chunks8"])
def scan_chunk(request, monkeypatch):
    """Both forms of the recurrent scans: one pass over a portion, and chunks of 8 tokens
    side by side (used for portions of 16 tokens and more)."""
    monkeypatch.setattr(sm, "SCAN_CHUNK", request.param)
    return request.param


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D", [(2, 40), (3, 20), (1, 72), (2, 64), (1, 136), (2, 7)])
def test_gdelta(dt, H, D, scan_chunk):
    g = torch.Generator().manual_seed(2)
    n = H * D
    slots = 5
    w0, ab, nw = (torch.randn(n, generator=g) for _ in range(3))
    st_c = torch.zeros(slots, H, D, D)
    st_g = st_c.to(DEV)
    for lens, starts in (([40, 1, 7], [0, 0, 0]), ([3, 1, 35], [40, 1, 7])):
        ent_h, ent, row_ent, R = _ents(lens, starts, [3, 0, 4])
        proj = torch.randn(R, 5 * n + 3, generator=g).to(dt)
        lo = torch.randn(R, n, generator=g).to(dt)
        v5 = lambda p: [p[:, i * n:(i + 1) * n] for i in range(5)]
        a = sm.gdelta_scan(*v5(proj), lo, w0, ab, nw, st_c, ent, ent_h, torch.empty(R, n, dtype=dt), H, D, 1e-5)
        pg = proj.to(DEV)
        b = sm.gdelta_scan(*v5(pg), lo.to(DEV), w0.to(DEV), ab.to(DEV), nw.to(DEV), st_g, ent.to(DEV),
                           ent_h, torch.empty(R, n, dtype=dt, device=DEV), H, D, 1e-5)
        torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
        torch.testing.assert_close(st_g.cpu()[[3, 0, 4]], st_c[[3, 0, 4]], rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,P,N,G,K", [(6, 40, 24, 3, 3), (4, 24, 16, 1, 4), (2, 72, 80, 2, 2), (2, 200, 256, 1, 4), (8, 64, 128, 4, 4)])
def test_mamba(dt, H, P, N, G, K, scan_chunk):
    g = torch.Generator().manual_seed(3)
    inner, C = H * P, H * P + 2 * G * N
    slots = 4
    cw, cb = torch.randn(C, K, generator=g) * 0.5, torch.randn(C, generator=g) * 0.1
    dtb, Al, Dp = torch.randn(H, generator=g), torch.rand(H, generator=g) - 0.5, torch.randn(H, generator=g)
    S_c, T_c = torch.zeros(slots, H, N, P), torch.zeros(slots, K - 1, C)
    S_g, T_g = S_c.to(DEV), T_c.to(DEV)
    for lens, starts in (([1, 30, 2], [0, 0, 0]), ([1, 1, 33], [1, 30, 2]), ([5, 1, 1], [2, 31, 35])):
        ent_h, ent, row_ent, R = _ents(lens, starts, [2, 0, 3])
        zx = torch.randn(R, 2 * inner + 2 * G * N + H, generator=g).to(dt)
        c1 = sm.mamba_conv(zx, inner, cw, cb, T_c, ent, ent_h, row_ent, torch.empty(R, C))
        zg = zx.to(DEV)
        c2 = sm.mamba_conv(zg, inner, cw.to(DEV), cb.to(DEV), T_g, ent.to(DEV), ent_h, row_ent.to(DEV),
                           torch.empty(R, C, device=DEV))
        torch.testing.assert_close(c2.cpu(), c1, rtol=1e-4, atol=1e-5)
        y1 = sm.mamba_scan(c1, zx, inner, inner + C, dtb, Al, Dp, S_c, T_c, ent, ent_h, torch.empty(R, inner), H, P, N, G)
        y2 = sm.mamba_scan(c2, zg, inner, inner + C, dtb.to(DEV), Al.to(DEV), Dp.to(DEV), S_g, T_g, ent.to(DEV),
                           ent_h, torch.empty(R, inner, device=DEV), H, P, N, G)
        torch.testing.assert_close(y2.cpu(), y1, rtol=2e-4, atol=2e-4)
        torch.testing.assert_close(S_g.cpu()[[2, 0, 3]], S_c[[2, 0, 3]], rtol=2e-4, atol=2e-4)
        torch.testing.assert_close(T_g.cpu()[[2, 0, 3]], T_c[[2, 0, 3]], rtol=0, atol=0)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,rank,win", [(6, 120, 36), (3, 40, 7), (5, 96, 200), (16, 512, 33), (20, 64, 64), (1, 8, 3)])
def test_latent_attn(dt, H, rank, win):
    g = torch.Generator().manual_seed(4)
    page, npages = 64, 12
    cache = torch.randn(npages * page, rank, generator=g).to(dt)
    bt = torch.tensor([[3, 7, 1, 9], [2, 5, 0, 0]], dtype=torch.int32)
    # entry 0: rows at positions 100..139 (crosses a page border), entry 1: single token at 70
    pos = torch.tensor(list(range(100, 140)) + [70], dtype=torch.int32)
    row_ent = torch.tensor([0] * 40 + [1], dtype=torch.int32)
    R = pos.numel()
    qa = (torch.randn(R, H, rank, generator=g) * 0.3).to(dt).transpose(0, 1)   # strided [H, R, rank]
    sink = torch.randn(H, generator=g)
    a = sm.latent_attn(qa, cache, bt, row_ent, pos, sink, 0.2, win, torch.empty(H, R, rank, dtype=dt), page)
    b = sm.latent_attn(qa.to(DEV), cache.to(DEV), bt.to(DEV), row_ent.to(DEV), pos.to(DEV), sink.to(DEV), 0.2,
                       win, torch.empty(H, R, rank, dtype=dt, device=DEV), page)
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    if dt == torch.bfloat16:
        # the matrix-core kernel: queries as a contiguous [H, R, rank] tensor, row groups per wave
        qc = qa.contiguous().to(DEV)
        assert sm.latent_mfma_ok(qc, cache.to(DEV))
        units = sm.make_units([(0, 40, 100, 0), (40, 1, 70, 1)], sm.latent_rows_per_wave(H)).to(DEV)
        c = sm.latent_attn(qc, cache.to(DEV), bt.to(DEV), row_ent.to(DEV), pos.to(DEV), sink.to(DEV), 0.2,
                           win, torch.empty(H, R, rank, dtype=dt, device=DEV), page, units=units)
        torch.testing.assert_close(c.cpu().float(), a.float(), **_tol(dt))
        # few rows, long windows: every window cut into runs of key tiles and merged
        d = sm.latent_attn(qc, cache.to(DEV), bt.to(DEV), row_ent.to(DEV), pos.to(DEV), sink.to(DEV), 0.2,
                           win, torch.empty(H, R, rank, dtype=dt, device=DEV), page, units=units,
                           max_keys=140)
        torch.testing.assert_close(d.cpu().float(), a.float(), **_tol(dt))
