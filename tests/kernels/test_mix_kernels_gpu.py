"""gfx950 kernels of the layer-list models against the plain torch ops (fp32 and bf16)."""
import numpy as np
import pytest
import torch

from replisense_rfq_amd import ops
from replisense_rfq_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _tol(dt, wide=False):
    """wide: sums over up to 1024 fp32 terms in another order than torch's."""
    if dt == torch.float32:
        return dict(rtol=1e-4, atol=1e-4) if wide else dict(rtol=2e-5, atol=2e-5)
    return dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_embed_sinusoid(dt):
    g = torch.Generator().manual_seed(0)
    V, d, T = 97, 70, 33
    table = torch.randn(V, d, generator=g).to(dt)
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    pos = torch.randint(0, 3000, (T,), generator=g, dtype=torch.int32)
    inv = ops.sinusoid_inv_freq(d, "cpu")
    want = torch.empty(T, d)
    ref.embed_sinusoid(ids, pos, table, inv, 3.5, want)
    got = ops.embed_sinusoid(ids.to(DEV), pos.to(DEV), table.to(DEV), inv.to(DEV), 3.5)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=2e-4)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [48, 300, 1030])
def test_sandwich_norm(dt, d):
    g = torch.Generator().manual_seed(1)
    T = 7
    x = torch.randn(T, d, generator=g) * 5
    y = (torch.randn(T, d, generator=g) * 3).to(dt)
    wp, gn, wn = (torch.randn(d, generator=g) for _ in range(3))
    xr, want = x.clone(), torch.empty(T, d)
    ref.sandwich_norm(y, xr, wp, gn, wn, 1e-5, want)
    xg = x.to(DEV)
    got = ops.sandwich_norm(y.to(DEV), xg, wp.to(DEV), gn.to(DEV), wn.to(DEV), 1e-5)
    torch.testing.assert_close(xg.cpu(), xr, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5)
    want2 = torch.empty(T, d)
    ref.sandwich_norm(None, xr, None, None, wn, 1e-5, want2)
    got2 = ops.sandwich_norm(None, xg, None, None, wn.to(DEV), 1e-5)
    torch.testing.assert_close(got2.cpu(), want2, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_canon_conv_runs_and_state(dt, taps):
    """Three steps over two slots: a long run, runs shorter than the state, a reused slot."""
    g = torch.Generator().manual_seed(2)
    d, S, K = 40, 3, taps - 1
    w = torch.randn(d, taps, generator=g)
    st_c = torch.randn(2 * S, K, d, generator=g)          # garbage: a fresh slot must not read it
    st_g = st_c.to(DEV)
    gen = {0: 0, 2: 0}
    pos0 = {0: 0, 2: 0}
    for runs in ([(0, 6), (2, 1)], [(2, 1), (0, 1)], [(0, 2), (2, 4)], [(2, 1)]):
        rs, rb, rf, ps = [], [], [], []
        for slot, q in runs:
            for i in range(q):
                rs.append(slot * 2 + (gen[slot] & 1))
                rb.append(i)
                rf.append(q - 1 - i)
                ps.append(pos0[slot] + i)
            gen[slot] += 1
            pos0[slot] += q
        T = len(rs)
        h = torch.randn(T, d, generator=g)
        mk = lambda a: torch.tensor(a, dtype=torch.int32)  # noqa: E731
        want = torch.empty(T, d, dtype=dt)
        ref.canon_conv(h, w, st_c, mk(rs), mk(rb), mk(rf), mk(ps), want)
        got = torch.empty(T, d, dtype=dt, device=DEV)
        ops.canon_conv(h.to(DEV), w.to(DEV), st_g, mk(rs).to(DEV), mk(rb).to(DEV), mk(rf).to(DEV),
                       mk(ps).to(DEV), got)
        torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
    torch.testing.assert_close(st_g.cpu(), st_c, rtol=0, atol=0)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_glu_clamped(dt):
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn(5, 2 * 300, generator=g) * 3).to(dt)
    want = torch.empty(5, 300, dtype=dt)
    ref.glu_clamped(gu, 1.25, 1.702, want)
    got = ops.glu_clamped(gu.to(DEV), 1.25, 1.702)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


def _paged(dt, H, G, dim, vdim, lens, qlens, seed, BS=32):
    """Random paged caches (pages handed out in a shuffled order) and step metadata."""
    g = torch.Generator().manual_seed(seed)
    nblk = sum((n + BS - 1) // BS for n in lens) + 3
    perm = torch.randperm(nblk - 1, generator=g).tolist()
    maxb = max((n + BS - 1) // BS for n in lens) + 1
    bt = torch.full((len(lens), maxb), nblk - 1, dtype=torch.int32)
    for b, n in enumerate(lens):
        for i in range((n + BS - 1) // BS):
            bt[b, i] = perm.pop()
    kc = torch.randn(nblk, G, BS, dim, generator=g).to(dt)
    vc = torch.randn(nblk, G, BS, vdim, generator=g).to(dt)
    qs = np.concatenate([[0], np.cumsum(qlens)[:-1]]).astype(np.int32)
    meta = dict(bt=bt, q_start=torch.from_numpy(qs), q_len=torch.tensor(qlens, dtype=torch.int32),
                kv_len=torch.tensor(lens, dtype=torch.int32))
    return g, kc, vc, meta


CASES = [(8, 2, 64, 64, 72), (6, 3, 24, 40, 16), (3, 1, 16, 8, 0), (8, 8, 32, 32, 50),
         (5, 5, 72, 24, 33)]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dim,vdim,chunk", CASES)
@pytest.mark.parametrize("use_talk,use_sink", [(True, True), (False, False)])
def test_attn_talk_decode(dt, H, G, dim, vdim, chunk, use_talk, use_sink):
    lens, qlens = [1, 37, 260, 64, 130], [1, 5, 1, 32, 2]
    g, kc, vc, m = _paged(dt, H, G, dim, vdim, lens, qlens, 5)
    T = sum(qlens)
    qn = torch.randn(T, H, dim, generator=g)
    slopes = torch.rand(H, generator=g) * 0.2
    talk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g) if use_talk else None
    sink = torch.randn(H, generator=g) if use_sink else None
    want = torch.empty(T, H * vdim, dtype=dt)
    ref.attn_talk_decode(qn, kc, vc, m["bt"], m["q_start"], m["q_len"], m["kv_len"], want, slopes,
                         talk, sink, 0.2, chunk)
    got = torch.empty(T, H * vdim, dtype=dt, device=DEV)
    dv = lambda t: None if t is None else t.to(DEV)  # noqa: E731
    ops.attn_talk_decode(qn.to(DEV), kc.to(DEV), vc.to(DEV), m["bt"].to(DEV), m["q_start"].to(DEV),
                         m["q_len"].to(DEV), m["kv_len"].to(DEV), got, slopes.to(DEV), dv(talk),
                         dv(sink), 0.2, chunk)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dim,vdim,chunk", CASES + [(2, 2, 64, 64, 0), (8, 2, 128, 128, 96), (8, 8, 128, 128, 70), (32, 8, 128, 64, 0), (16, 4, 128, 32, 500)])
@pytest.mark.parametrize("mfma", [False, True, "grouped"])
def test_attn_mixq_prefill(dt, H, G, dim, vdim, chunk, mfma):
    if mfma and dt != torch.bfloat16:
        pytest.skip("the MFMA tiles are bf16")
    if mfma and not ops.mixq_mfma_ok(H, G, dim, vdim):
        pytest.skip("sizes outside the MFMA tiles")
    lens, qlens = [33, 300, 97, 64, 2], [33, 120, 40, 64, 2]
    g, kc, vc, m = _paged(dt, H, G, dim, vdim, lens, qlens, 6)
    T = sum(qlens)
    qn = torch.randn(T, H, dim, generator=g)
    ts = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)) * 0.2
    qmix = torch.einsum("hcr,tcrd->thcd", ts.view(H, G, H // G),
                        qn.view(T, G, H // G, dim)).reshape(T, H, G * dim).contiguous()
    slopes = torch.rand(H, generator=g) * 0.2
    sink = torch.randn(H, generator=g)
    ws, wq = [], []
    for b, q in enumerate(qlens):
        for c in range((q + 31) // 32):
            ws.append(b)
            wq.append(c)
    ws, wq = torch.tensor(ws, dtype=torch.int32), torch.tensor(wq, dtype=torch.int32)
    want = torch.empty(T, H * vdim, dtype=dt)
    # the MFMA kernel's query operand is the bf16 rounding of the mixed queries
    ref.attn_mixq_prefill(qmix.bfloat16().float() if mfma else qmix, kc, vc, m["bt"], m["q_start"],
                          m["q_len"], m["kv_len"], want, slopes, sink, chunk)
    got = torch.empty(T, H * vdim, dtype=dt, device=DEV)
    args = (kc.to(DEV), vc.to(DEV), m["bt"].to(DEV), m["q_start"].to(DEV), m["q_len"].to(DEV),
            m["kv_len"].to(DEV), ws.to(DEV), wq.to(DEV), got, slopes.to(DEV), sink.to(DEV), chunk)
    if mfma:
        ops.attn_mix_mfma(qn.to(DEV), ts.to(DEV), *args, grouped=mfma == "grouped")
    else:
        ops.attn_mixq_prefill(qmix.to(DEV), *args)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt, wide=True))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dim,vdim", [(4, 2, 64, 64), (6, 3, 24, 40), (5, 1, 16, 8)])
def test_head_norm_append(dt, H, G, dim, vdim):
    g = torch.Generator().manual_seed(7)
    T, BS, nblk, mix_from = 9, 32, 4, 3
    qkv = (torch.randn(T, H * dim + G * (dim + vdim), generator=g) * 2).to(dt)
    qw, kw = torch.randn(dim, generator=g), torch.randn(dim, generator=g)
    ts = torch.randn(H, H, generator=g)
    slots = torch.tensor([5, 37, -1, 64, 65, 66, 100, 2, 31], dtype=torch.int32)
    kc, vc = torch.zeros(nblk, G, BS, dim, dtype=dt), torch.zeros(nblk, G, BS, vdim, dtype=dt)
    qn, qm = torch.empty(T, H, dim), torch.empty(T - mix_from, H, G * dim)
    ref.head_norm_append(qkv, qw, kw, 1e-5, slots, kc, vc, H, G, dim, vdim, qn, ts, qm, mix_from)
    kg, vg = torch.zeros_like(kc, device=DEV), torch.zeros_like(vc, device=DEV)
    qng, qmg = torch.empty_like(qn, device=DEV), torch.empty_like(qm, device=DEV)
    ops.head_norm_append(qkv.to(DEV), qw.to(DEV), kw.to(DEV), 1e-5, slots.to(DEV), kg, vg, H, G,
                         dim, vdim, qng, ts.to(DEV), qmg, mix_from)
    torch.testing.assert_close(qng.cpu(), qn, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(qmg.cpu(), qm, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(kg.cpu().float(), kc.float(), **_tol(dt))
    torch.testing.assert_close(vg.cpu().float(), vc.float(), **_tol(dt))
