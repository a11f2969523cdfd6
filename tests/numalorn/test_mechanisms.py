"""Each Numalorn mechanism alone (package op on CPU tensors or the gfx950 kernel) against the
slow oracle, with inputs made so that a key, a state or a choice missed or wrongly seen shows."""
import math

import pytest
import torch

from replisense_rfq_amd import ops

from . import oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 32
D64 = torch.float64


def close(a, b, tol=2e-5):
    a, b = a.double().cpu(), b.double().cpu()
    assert float((a - b).abs().max()) <= tol * max(1.0, float(b.abs().max())), \
        float((a - b).abs().max())


def i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


@pytest.mark.parametrize("device", DEVICES)
def test_embedding_rows(device):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(50, 38, generator=g)
    ids = torch.randint(0, 50, (9,), generator=g, dtype=torch.int32)
    close(ops.embed_rows(ids.to(device), table.to(device)), table[ids.long()], 0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d", [44, 256, 1030])
def test_post_norm_residual(device, d):
    """x += m * y / rms(y) * (1 + w): the weight is stored around zero, and the norm is on the
    sublayer's output only."""
    g = torch.Generator().manual_seed(1)
    T, eps, m = 5, 1e-3, 0.3
    x, y = torch.randn(T, d, generator=g) * 4, torch.randn(T, d, generator=g) * 0.01
    w = torch.randn(d, generator=g) * 0.5
    want = x.double() + m * oracle.norm_around_zero(y.double(), w.double(), eps)
    xd = x.to(device)
    ops.post_norm_add(y.to(device), xd, w.to(device), m, eps, None)
    close(xd, want)
    if device != "cpu":                   # the bf16 model's rows come with a rounded copy
        xd, cp = x.to(device), torch.empty(T, d, dtype=torch.bfloat16, device=device)
        ops.post_norm_add(y.to(device).bfloat16(), xd, w.to(device), m, eps, cp)
        want = x.double() + m * oracle.norm_around_zero(y.bfloat16().double(), w.double(), eps)
        close(xd, want)
        close(cp, want.float().bfloat16(), 0)


@pytest.mark.parametrize("device", DEVICES)
def test_plain_and_zero_centred_norms_of_column_slices(device):
    g = torch.Generator().manual_seed(2)
    wide = torch.randn(7, 90, generator=g) * 3
    w = torch.randn(50, generator=g)
    x = wide.to(device)[:, 17:67]
    out = torch.empty(7, 50, device=device)
    close(ops.rms_norm_rows(x, w.to(device), 1e-4, out), oracle.norm_plain(wide[:, 17:67].double(), w.double(), 1e-4))
    close(ops.rms_norm_rows(x, w.to(device), 1e-4, out, 1.0),
          oracle.norm_around_zero(wide[:, 17:67].double(), w.double(), 1e-4))


# ------------------------------------------------------------------ state slots
def run_rows(cuts, slot, gen0=0, pos0=0):
    """row_state / row_back / row_fwd / positions of a sequence's portions, one launch each."""
    at, gen = pos0, gen0
    for n in cuts:
        yield at - pos0, n, ([slot * 2 + (gen & 1)] * n, list(range(n)), list(range(n - 1, -1, -1)),
                             list(range(at, at + n)))
        at += n
        gen += 1


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[50], [1] * 50, [2, 1, 3, 44], [3, 3, 1, 1, 2, 40]])
def test_token_shift_in_portions(device, cuts):
    """A sequence mixed in portions through a slot that held another sequence's row equals the
    mixes of the whole sequence; the first token sees zeros, not the slot's old contents."""
    g = torch.Generator().manual_seed(3)
    d, S, slot = 20, 3, 1
    x = torch.randn(sum(cuts), d, generator=g)
    mu = torch.rand(5, d, generator=g)
    prev = (torch.randn(2 * S, d, generator=g) * 100).to(device)
    want = torch.stack([oracle.shift_mix(x.double(), mu[s].double()) for s in range(5)])
    outs = []
    for lo, n, rows in run_rows(cuts, slot):
        out = torch.empty(5, n, d, device=device)
        ops.token_shift_mix(x[lo:lo + n].to(device), mu.to(device), prev, *(i32(r, device) for r in rows), out)
        outs.append(out.cpu())
    close(torch.cat(outs, 1), want)


@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_two_sequences_in_one_launch(device):
    g = torch.Generator().manual_seed(4)
    d = 12
    a, b = torch.randn(5, d, generator=g), torch.randn(3, d, generator=g)
    mu = torch.rand(2, d, generator=g)
    prev = torch.zeros(4, d)
    prev[0] = torch.randn(d, generator=g)              # slot 0, half 0: a's row before this run
    x = torch.cat([a, b])
    rs = [0] * 5 + [2] * 3                             # a: slot 0 half 0; b: slot 1 half 0
    rb = [0, 1, 2, 3, 4, 0, 1, 2]
    rf = [4, 3, 2, 1, 0, 2, 1, 0]
    pos = [7, 8, 9, 10, 11, 0, 1, 2]                   # a continues, b starts
    prev_d = prev.to(device)
    out = torch.empty(2, 8, d, device=device)
    ops.token_shift_mix(x.to(device), mu.to(device), prev_d, *(i32(r, device) for r in (rs, rb, rf, pos)), out)
    for s in range(2):
        wa = oracle.shift_mix(torch.cat([prev[0:1], a]).double(), mu[s].double())[1:]
        wb = oracle.shift_mix(b.double(), mu[s].double())
        close(out[s], torch.cat([wa, wb]))
    close(prev_d[2], a[-1], 0)                         # other half of slot 0
    close(prev_d[3], b[-1], 0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,N", [(2, 64), (3, 24), (1, 7), (2, 96), (32, 64)])
@pytest.mark.parametrize("cuts", [[40], [1] * 40, [2, 1, 33, 4], [17, 2, 2, 19]])
def test_wkv_recurrence_in_portions(device, H, N, cuts):
    """The recurrence in portions through a state slot with stale contents equals the scan of
    the whole sequence; the bonus u counts for the current token only; the output is
    unit-normed per head, scaled and gated."""
    g = torch.Generator().manual_seed(5)
    T, S, slot, eps = sum(cuts), 2, 1, 1e-4
    r, k, v, gate = (torch.randn(T, H * N, generator=g) for _ in range(4))
    zw = torch.randn(T, H * N, generator=g)
    w0 = torch.randn(H * N, generator=g) - 1.5
    u = torch.randn(H, N, generator=g)
    nw = torch.randn(H * N, generator=g)
    w = oracle.decay(zw.double(), w0.double())
    o, _ = oracle.wkv_scan(*(a.double().view(T, H, N) for a in (r, k, v)), w.view(T, H, N), u.double())
    want = oracle.rms_unit(o, eps).reshape(T, H * N) * nw.double() * oracle.silu(gate.double())
    state = (torch.randn(2 * S, H, N, N, generator=g) * 50).to(device)
    outs = []
    for lo, n, rows in run_rows(cuts, slot, gen0=1):
        out = torch.empty(n, H * N, device=device)
        sl = slice(lo, lo + n)
        ops.wkv_recurrence(r[sl].to(device), k[sl].to(device), v[sl].to(device), zw[sl].to(device),
                           w0.to(device), u.to(device), gate[sl].to(device), nw.to(device), eps, state,
                           *(i32(x, device) for x in rows), out)
        outs.append(out.cpu())
    close(torch.cat(outs), want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_wkv_runs_of_several_sequences_from_a_run_list(device):
    """Three runs in one launch (one continues from its slot, two start), launched from the
    list of their first rows with an empty entry in it: each as if it ran alone."""
    g = torch.Generator().manual_seed(6)
    H, N, eps = 3, 64, 1e-5
    lens, slots, first = [37, 1, 70], [2, 0, 1], [5, 0, 0]
    T = sum(lens)
    r, k, v, gate, zw = (torch.randn(T, H * N, generator=g) * 0.5 for _ in range(5))
    w0, u, nw = torch.randn(H * N, generator=g) - 1.5, torch.randn(H, N, generator=g), torch.randn(H * N, generator=g)
    state = torch.randn(6, H, N, N, generator=g)
    rs, rb, rf, pos = [], [], [], []
    for n, s_, p0 in zip(lens, slots, first):
        rs += [2 * s_] * n
        rb += list(range(n))
        rf += list(range(n - 1, -1, -1))
        pos += list(range(p0, p0 + n))
    st = state.clone().to(device)
    out = torch.empty(T, H * N, device=device)
    runs = i32([0, -1, 37, 38], device)
    ops.wkv_recurrence(*(a.to(device) for a in (r, k, v, zw)), w0.to(device), u.to(device), gate.to(device),
                       nw.to(device), eps, st, *(i32(x, device) for x in (rs, rb, rf, pos)), out, runs)
    w = oracle.decay(zw.double(), w0.double()).view(T, H, N)
    at = 0
    for n, s_, p0 in zip(lens, slots, first):
        sl = slice(at, at + n)
        S0 = state[s_].double() if p0 > 0 else None       # half 0 of the slot
        o, S1 = oracle.wkv_scan(*(a[sl].double().view(n, H, N) for a in (r, k, v)), w[sl], u.double(), S0)
        want = oracle.rms_unit(o, eps).reshape(n, H * N) * nw.double() * oracle.silu(gate[sl].double())
        close(out[sl], want, 1e-4)
        close(st[3 + s_], S1, 1e-4)                        # other half
        at += n


@pytest.mark.parametrize("device", DEVICES)
def test_wkv_state_carried_far_and_bonus_only_now(device):
    """With decay ~ 1 on one channel a key from 300 tokens back still answers a matching
    query; with u = 0 the current token's own pair does not answer at all."""
    H, N, T, eps = 1, 16, 301, 1e-6
    r, k, v = torch.zeros(T, N), torch.zeros(T, N), torch.zeros(T, N)
    k[0, 3], v[0, 5] = 2.0, 1.5
    r[300, 3] = 1.0
    k[300, 3], v[300, 9] = 1.0, 4.0                    # would answer through u only
    zw = torch.full((T, N), -30.0)                     # exp(-exp(-30)) = 1: nothing decays
    w0, u, nw, gate = torch.zeros(N), torch.zeros(H, N), torch.ones(N), torch.full((T, N), 30.0)
    state = torch.zeros(2, H, N, N, device=device)
    outs = []
    for lo, n, rows in run_rows([200, 100, 1], 0):
        out = torch.empty(n, N, device=device)
        sl = slice(lo, lo + n)
        ops.wkv_recurrence(r[sl].to(device), k[sl].to(device), v[sl].to(device), zw[sl].to(device),
                           w0.to(device), u.to(device), gate[sl].to(device), nw.to(device), eps, state,
                           *(i32(x, device) for x in rows), out)
        outs.append(out.cpu())
    last = torch.cat(outs)[300]
    # o = 2 * 1.5 on value channel 5 only -> unit rms over 16 channels = 4 there, gate ~ 30
    assert abs(float(last[5]) - 4.0 * 30.0) < 1e-2 and float(last.abs().sum() - last[5].abs()) < 1e-3


# ------------------------------------------------------------------ latent attention
def latent_case(device, H, dim, vdim, R, lens, q_lens, seed, boost=None, dtype=torch.float32):
    """Sequences with their latents in pages handed out in odd order; queries for the last
    q_len positions of each.  Returns the op inputs and the oracle's per-row outputs."""
    g = torch.Generator().manual_seed(seed)
    nblk = sum((n + BS - 1) // BS for n in lens) + 3
    order = torch.randperm(nblk - 1, generator=g).tolist()
    pool = (torch.randn(nblk, 1, BS, R, generator=g) * 9).to(device)          # stale everywhere
    uk = torch.randn(H, dim, R, generator=g) * R ** -0.5
    uv = torch.randn(H, vdim, R, generator=g) * R ** -0.5
    sink = torch.randn(H, generator=g)
    scale = 0.37
    tables, cs, qs, want = [], [], [], []
    maxb = max((n + BS - 1) // BS for n in lens)
    for n, ql in zip(lens, q_lens):
        c = torch.randn(n, R, generator=g)
        q = torch.randn(ql, H, dim, generator=g)
        if boost is not None and boost[0] < n - 1:      # one far key every last query matches
            j, hd = boost
            c[j] = 0
            c[j, 0] = 6.0
            q[-1, hd] = uk[hd][:, 0] / uk[hd][:, 0].norm() * 30.0
        blocks = [order.pop() for _ in range((n + BS - 1) // BS)]
        for p in range(n):
            pool[blocks[p // BS], 0, p % BS] = c[p].to(device)
        tables.append(blocks + [nblk - 1] * (maxb - len(blocks)))
        cs.append(c)
        qs.append(q)
        k = torch.einsum("hdr,nr->nhd", uk.double(), c.double())
        v = torch.einsum("hvr,nr->nhv", uv.double(), c.double())
        o = torch.zeros(ql, H, vdim, dtype=D64)
        for a in range(ql):
            i = n - ql + a
            for hd in range(H):
                s = (k[:i + 1, hd] @ q[a, hd].double()) * scale
                mx = torch.maximum(s.max(), sink[hd].double())
                e = torch.exp(s - mx)
                o[a, hd] = (e[:, None] * v[:i + 1, hd]).sum(0) / (e.sum() + torch.exp(sink[hd].double() - mx))
        want.append(o.reshape(ql, H * vdim))
    return pool, uk, uv, sink, scale, tables, qs, torch.cat(want)


def absorbed(q, uk, scale):
    """Queries carried into the latent space, as the model does before the attention op."""
    return (torch.einsum("thd,hdr->thr", q.float(), uk.float()) * scale).contiguous()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,dim,vdim,R", [(3, 16, 8, 24), (1, 8, 24, 40), (4, 32, 32, 64),
                                          (16, 128, 128, 512)])
def test_latent_attention_decode_rows(device, H, dim, vdim, R):
    """Rows of the decode section (1 to a few queries per sequence) over pages in odd order,
    lengths at page borders: scores and values both come from the one cached latent."""
    lens, q_lens = [1, 32, 33, 64, 97, 5], [1, 1, 2, 1, 3, 5]
    pool, uk, uv, sink, scale, tables, qs, want = latent_case(device, H, dim, vdim, R, lens, q_lens, 7)
    qa = absorbed(torch.cat(qs), uk, scale).to(device)
    starts = [sum(q_lens[:i]) for i in range(len(lens))]
    lat = torch.empty(sum(q_lens), H * R, device=device)
    ops.attn_talk_decode(qa, pool, pool, i32(tables, device), i32(starts, device), i32(q_lens, device),
                         i32(lens, device), lat, torch.zeros(H, device=device), None, sink.to(device), 1.0, 0)
    got = torch.einsum("thr,hvr->thv", lat.view(-1, H, R).cpu().double(), uv.double()).reshape(-1, H * vdim)
    close(got, want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,dim,vdim,R", [(3, 16, 8, 24), (2, 8, 24, 72), (8, 128, 128, 512)])
def test_latent_attention_prefill_rows_and_far_key(device, H, dim, vdim, R):
    """Portions of prompts behind cached tokens; one key far back (in the first page, at a page
    border) is made to dominate the last query's softmax over hundreds of others."""
    lens, q_lens = [300, 70, 33], [45, 70, 2]
    for j in (0, 31, 32, 254):
        pool, uk, uv, sink, scale, tables, qs, want = latent_case(
            device, H, dim, vdim, R, lens, q_lens, 8, boost=(j, H - 1))
        qa = absorbed(torch.cat(qs), uk, scale).to(device)
        starts = [sum(q_lens[:i]) for i in range(len(lens))]
        work = [(s, b) for s, ql in enumerate(q_lens) for b in range((ql + 31) // 32)]
        lat = torch.empty(sum(q_lens), H * R, device=device)
        ops.attn_mixq_prefill(qa, pool, pool, i32(tables, device), i32(starts, device),
                              i32(q_lens, device), i32(lens, device), i32([w[0] for w in work], device),
                              i32([w[1] for w in work], device), lat, torch.zeros(H, device=device),
                              sink.to(device), 0, 32)
        got = torch.einsum("thr,hvr->thv", lat.view(-1, H, R).cpu().double(), uv.double()).reshape(-1, H * vdim)
        close(got, want, 1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("H,R", [(3, 64), (8, 128), (5, 256), (16, 512), (32, 512)])
def test_latent_attention_on_matrix_cores(H, R):
    """bf16 pools with a latent width of the MFMA tiles: decode rows and portions of prompts
    behind cached tokens, pages in odd order, lengths at page borders, one far key that
    dominates a late query, any head count; against the softmax over the same rounded rows."""
    dev = "cuda"
    g = torch.Generator().manual_seed(13)
    lens, q_lens = [1, 32, 33, 97, 300, 70, 5, 64], [1, 1, 2, 3, 45, 70, 5, 33]
    nblk = sum((n + BS - 1) // BS for n in lens) + 2
    order = torch.randperm(nblk - 1, generator=g).tolist()
    pool = (torch.randn(nblk, 1, BS, R, generator=g) * 9).bfloat16()              # stale everywhere
    sink = torch.randn(H, generator=g)
    scale = 0.41 * R ** -0.5
    maxb = max((n + BS - 1) // BS for n in lens)
    tables, qs, want = [], [], []
    for n, ql in zip(lens, q_lens):
        c = torch.randn(n, R, generator=g).bfloat16()
        q = (torch.randn(ql, H, R, generator=g) * 3).bfloat16()
        if n > 200:                                    # key 31 answers the last query of head H-1
            c[31] = 0
            c[31, 7] = 8.0
            q[-1, H - 1] = 0
            q[-1, H - 1, 7] = 40.0 / (8.0 * scale)
        blocks = [order.pop() for _ in range((n + BS - 1) // BS)]
        for p in range(n):
            pool[blocks[p // BS], 0, p % BS] = c[p]
        tables.append(blocks + [nblk - 1] * (maxb - len(blocks)))
        qs.append(q)
        cd, o = c.double(), torch.zeros(ql, H, R, dtype=D64)
        for a in range(ql):
            i = n - ql + a
            sc = torch.einsum("hr,nr->hn", q[a].double(), cd[:i + 1]) * scale
            mx = torch.maximum(sc.max(-1).values, sink.double())
            e = torch.exp(sc - mx[:, None])
            o[a] = (e @ cd[:i + 1]) / (e.sum(-1) + torch.exp(sink.double() - mx))[:, None]
        want.append(o.reshape(ql, H * R))
    want = torch.cat(want)
    T = sum(q_lens)
    # queries as the batched product leaves them: [H, T, R], read through strides
    qh = torch.cat(qs).transpose(0, 1).contiguous().to(dev)
    starts = [sum(q_lens[:i]) for i in range(len(lens))]
    work = [(s_, b) for s_, ql in enumerate(q_lens) for b in range((ql + 31) // 32)]
    out = torch.full((T, H * R), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.attn_latent_mfma(qh.transpose(0, 1), pool.to(dev), i32(tables, dev), i32(starts, dev),
                         i32(q_lens, dev), i32(lens, dev), i32([w[0] for w in work], dev),
                         i32([w[1] for w in work], dev), out, sink.to(dev), scale)
    torch.cuda.synchronize()
    err = (out.double().cpu() - want).abs().max() / want.abs().max()
    assert float(err) < 1e-2, float(err)
    far = want[sum(q_lens[:5]) - 1].view(H, R)[H - 1]
    assert float(far[7]) > 7.5                         # the boosted key carries the row


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_weight_without_a_value(device):
    """One key with score 0 and a sink logit of ln 3: the output is a quarter of the value."""
    H, R = 2, 8
    pool = torch.zeros(2, 1, BS, R, device=device)
    pool[0, 0, 0] = torch.arange(1, R + 1, dtype=torch.float32)
    sink = torch.tensor([math.log(3.0), -1e4])
    lat = torch.empty(1, H * R, device=device)
    ops.attn_talk_decode(torch.zeros(1, H, R, device=device), pool, pool, i32([[0]], device), i32([0], device),
                         i32([1], device), i32([1], device), lat, torch.zeros(H, device=device), None,
                         sink.to(device), 1.0, 0)
    close(lat.view(H, R)[0], pool[0, 0, 0] / 4)
    close(lat.view(H, R)[1], pool[0, 0, 0])


@pytest.mark.parametrize("device", DEVICES)
def test_latent_norm_goes_to_its_page(device):
    g = torch.Generator().manual_seed(9)
    R, eps = 24, 1e-3
    wide = torch.randn(4, 40, generator=g)
    w = torch.randn(R, generator=g)
    pool = torch.zeros(3, 1, BS, R, device=device)
    slots = [2 * BS + 31, -1, 0, BS + 5]
    ops.latent_norm_append(wide.to(device)[:, 16:], w.to(device), eps, i32(slots, device), pool)
    want = oracle.norm_plain(wide[:, 16:].double(), w.double(), eps)
    flat = pool.view(-1, R)
    for t, s in enumerate(slots):
        if s >= 0:
            close(flat[s], want[t])
    assert int((flat.abs().sum(-1) > 0).sum()) == 3


# ------------------------------------------------------------------ experts
def route_case(device, z, corr, r):
    T, top = z.shape[0], r["top"]
    ids = torch.empty(T, top, dtype=torch.int32, device=device)
    wts = torch.empty(T, top, device=device)
    g = r.get("groups") or {}
    ops.moe_route_grouped(z.to(device), corr.to(device), top, g.get("count", 0), g.get("keep", 0), ids, wts)
    get = lambda k: {"router": torch.eye(z.shape[1], dtype=D64), "correction": corr.double()}[k]  # noqa: E731
    want_i, want_w = oracle.route(z.double(), get, r)
    order = torch.argsort(ids.cpu().long(), -1)
    worder = torch.argsort(want_i, -1)
    assert torch.equal(ids.cpu().long().gather(1, order), want_i.gather(1, worder))
    close(wts.cpu().gather(1, order), want_w.gather(1, worder))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("r", [
    {"experts": 10, "top": 4, "groups": {"count": 5, "keep": 3}},
    {"experts": 12, "top": 2, "groups": {"count": 3, "keep": 1}},
    {"experts": 6, "top": 3, "groups": {"count": 6, "keep": 4}},        # groups of one expert
    {"experts": 5, "top": 1}, {"experts": 7, "top": 7}])
def test_grouped_sigmoid_routing(device, r):
    g = torch.Generator().manual_seed(10)
    z = torch.randn(200, r["experts"], generator=g) * 2
    corr = torch.randn(r["experts"], generator=g) * 0.5
    route_case(device, z, corr, r)


@pytest.mark.parametrize("device", DEVICES)
def test_routing_corrections_choose_but_do_not_weigh(device):
    """Negative choice scores: an expert of a dropped group must lose against a kept one whose
    corrected score is below zero (dropped = minus infinity, not zero); the weights are the
    uncorrected scores over their sum."""
    r = {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}}
    z = torch.tensor([[-3.0, -2.0, 4.0, -9.0]])
    corr = torch.tensor([0.0, 0.0, -5.0, 3.5])         # choice: .05 .12 -4.02 3.5 -> group 0 wins
    ids = torch.empty(1, 2, dtype=torch.int32, device=device)
    wts = torch.empty(1, 2, device=device)
    ops.moe_route_grouped(z.to(device), corr.to(device), 2, 2, 1, ids, wts)
    assert sorted(ids.cpu().tolist()[0]) == [0, 1]
    corr = torch.tensor([-2.0, -2.0, -5.0, 3.6])       # group 1: 3.6 - 4.02 = -.42 > -1.83
    ops.moe_route_grouped(z.to(device), corr.to(device), 2, 2, 1, ids, wts)
    assert sorted(ids.cpu().tolist()[0]) == [2, 3]      # both negative-or-not, never group 0
    s = torch.sigmoid(z[0, 2:].double())
    close(wts.cpu()[0].sort().values, (s / s.sum()).sort().values)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d,F,E,top,shared", [(40, 24, 5, 2, True), (64, 16, 3, 3, False), (36, 70, 4, 1, True)])
def test_expert_products_and_weighted_sum(device, d, F, E, top, shared):
    g = torch.Generator().manual_seed(11)
    T = 13
    h = torch.randn(T, d, generator=g)
    W = {"router": torch.randn(E, d, generator=g), "correction": torch.randn(E, generator=g) * 0.3}
    for e in [f"e{i}." for i in range(E)] + ["shared."]:
        W[e + "gate"], W[e + "up"] = torch.randn(F, d, generator=g) * d ** -0.5, torch.randn(F, d, generator=g) * d ** -0.5
        W[e + "down"] = torch.randn(d, F, generator=g) * F ** -0.5
    f = {"router": {"experts": E, "top": top}, "shared": {"ff": F} if shared else None}
    want = oracle.moe(h.double(), lambda k: W[k].double(), f)
    ids = torch.empty(T, top, dtype=torch.int32, device=device)
    wts = torch.empty(T, top, device=device)
    hd = h.to(device)
    ops.moe_route_grouped(ops.matmul_nt(hd, W["router"].to(device)), W["correction"].to(device), top, 0, 0, ids, wts)
    w13 = torch.stack([torch.cat([W[f"e{i}.gate"], W[f"e{i}.up"]]) for i in range(E)]).to(device)
    w2 = torch.stack([W[f"e{i}.down"] for i in range(E)]).to(device)
    base = None
    if shared:
        gu = ops.matmul_nt(hd, torch.cat([W["shared.gate"], W["shared.up"]]).to(device))
        base = ops.matmul_nt(ops.silu_mul_any(gu), W["shared.down"].to(device))
    out = ops.moe_experts(hd, ids, wts, w13, w2, base, torch.empty(T, d, device=device))
    close(out, want, 1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("d,F,E,top,groups,keep,T", [(512, 512, 8, 2, 2, 1, 300), (512, 512, 8, 2, 2, 1, 40),
                                                     (1024, 1024, 16, 4, 4, 2, 700), (2048, 4096, 8, 2, 2, 1, 24)])
def test_grouped_expert_gemms_match_the_general_kernels(d, F, E, top, groups, keep, T):
    """bf16 experts whose sizes the sparse decoder's grouped GEMMs take run there behind this
    router (few rows: per-expert skinny kernels; many: expert-sorted 128-row blocks, also with
    experts that get no row); both agree with the general per-pair kernels."""
    from replisense_rfq_amd.models.moe import MoEBuffers, grouped_ok, moe_mlp

    dev = "cuda"
    g = torch.Generator().manual_seed(12)
    h = torch.randn(T, d, generator=g).bfloat16().to(dev)
    w13 = (torch.randn(E, 2 * F, d, generator=g) * d ** -0.5).bfloat16().to(dev)
    w2 = (torch.randn(E, d, F, generator=g) * F ** -0.5).bfloat16().to(dev)
    z = (torch.randn(T, E, generator=g) * 2).to(dev)
    corr = torch.randn(E, generator=g).to(dev)
    corr[E // 2:] -= 50.0                                # the upper half never gets a row
    assert grouped_ok(w13, w2)
    ids = torch.empty(T, top, dtype=torch.int32, device=dev)
    wts = torch.empty(T, top, device=dev)
    ops.moe_route_grouped(z, corr, top, groups, keep, ids, wts)
    assert int(ids.max()) < E // 2
    want = ops.moe_experts(h, ids, wts, w13, w2, None, torch.empty(T, d, device=dev))
    bufs = MoEBuffers.allocate(1 << (T - 1).bit_length(), top, E, d, F, dev, torch.bfloat16)
    got = moe_mlp(h, z.new_zeros(E, d), w13, w2, top, bufs,
                  routing=lambda w, i: ops.moe_route_grouped(z, corr, top, groups, keep, i, w))
    torch.cuda.synchronize()
    err = (got.float() - want).abs().max() / want.abs().max()
    assert float(err) < 0.03, float(err)


@pytest.mark.parametrize("device", DEVICES)
def test_logit_soft_cap(device):
    x = torch.tensor([[-100.0, -3.0, 0.0, 0.5, 29.0, 1e4]])
    got = ops.softcap(x.clone().to(device), 30.0)
    close(got, 30.0 * torch.tanh(x.double() / 30.0))
