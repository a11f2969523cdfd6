"""Each Livisun mechanism alone (package op on CPU tensors or the gfx950 kernel) against the
slow oracle, with inputs made so that a key missed or wrongly seen shows."""
import pytest
import torch

from replisense_rfq_amd import ops
from replisense_rfq_amd.models.livisun import distance_slopes

from . import oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 32


def close(a, b, tol=2e-5):
    a, b = a.double().cpu(), b.double().cpu()
    assert float((a - b).abs().max()) <= tol * max(1.0, float(b.abs().max())), \
        float((a - b).abs().max())


@pytest.mark.parametrize("device", DEVICES)
def test_scaled_embedding_with_sinusoid(device):
    g = torch.Generator().manual_seed(0)
    V, d = 50, 38
    table = torch.randn(V, d, generator=g)
    ids = torch.randint(0, V, (9,), generator=g, dtype=torch.int32)
    pos = torch.tensor([0, 1, 2, 31, 32, 33, 511, 1000, 4097], dtype=torch.int32)
    got = ops.embed_sinusoid(ids.to(device), pos.to(device), table.to(device),
                             ops.sinusoid_inv_freq(d, device), 3.0)
    want = table.double()[ids.long()] * 3.0 + oracle.sinusoid(pos.tolist(), d)
    close(got, want, 5e-4)      # fp32 angles of positions in the thousands


@pytest.mark.parametrize("device", DEVICES)
def test_sandwich_norm(device):
    g = torch.Generator().manual_seed(1)
    T, d, eps = 5, 44, 1e-3
    x, y = torch.randn(T, d, generator=g) * 4, torch.randn(T, d, generator=g) * 0.01
    wp, gn, wn = (torch.randn(d, generator=g) for _ in range(3))
    xr = x.double() + oracle.rms_unit(y.double(), eps) * wp.double() * gn.double()
    want = oracle.rms_unit(xr, eps) * wn.double()
    xd = x.to(device)
    got = ops.sandwich_norm(y.to(device), xd, wp.to(device), gn.to(device), wn.to(device), eps)
    close(xd, xr)
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 3, 4])
@pytest.mark.parametrize("cuts", [[50], [1] * 50, [2, 1, 3, 44], [3, 3, 1, 1, 2, 40]])
def test_input_convolution_in_portions(device, taps, cuts):
    """A sequence convolved in portions through a state slot that held another sequence's
    inputs equals the convolution of the whole sequence."""
    g = torch.Generator().manual_seed(2)
    d, S, slot = 20, 3, 1
    w = torch.randn(d, taps, generator=g)
    h = torch.randn(sum(cuts), d, generator=g)
    state = (torch.randn(2 * S, taps - 1, d, generator=g) * 100).to(device)   # stale contents
    want = oracle.short_conv(h.double(), w.double())
    at, gen, outs = 0, 0, []
    for q in cuts:
        mk = lambda a: torch.tensor(a, dtype=torch.int32, device=device)  # noqa: E731
        out = torch.empty(q, d, device=device)
        ops.canon_conv(h[at:at + q].to(device), w.to(device), state, mk([slot * 2 + (gen & 1)] * q),
                       mk(list(range(q))), mk(list(range(q - 1, -1, -1))),
                       mk(list(range(at, at + q))), out)
        outs.append(out.cpu())
        at, gen = at + q, gen + 1
    close(torch.cat(outs), want)


@pytest.mark.parametrize("device", DEVICES)
def test_clamped_glu(device):
    g = torch.Generator().manual_seed(3)
    gu = torch.randn(4, 2 * 30, generator=g) * 3
    got = ops.glu_clamped(gu.to(device), 0.8, 1.702)
    close(got, oracle.gelu_sigmoid_glu(gu[:, :30].double(), gu[:, 30:].double(), 0.8))


def attend(device, q_raw, k_raw, v_raw, qw, kw, talk, sink, scale, chunk, rows, seed=0):
    """The package's attention path for ONE sequence: head norms + cache append (+ query
    mixing), then the decode kernel (rows <= 32 per step) or the prefill kernel (rows 0:
    everything in one step), on pages handed out in shuffled order."""
    T, H, dim = q_raw.shape
    G, vdim = k_raw.shape[1], v_raw.shape[2]
    g = torch.Generator().manual_seed(seed)
    nb = (T + BS - 1) // BS
    pages = torch.randperm(nb + 3, generator=g)[:nb].to(torch.int32)
    kc = torch.full((nb + 4, G, BS, dim), 1e4, device=device)        # junk in unused places
    vc = torch.full((nb + 4, G, BS, vdim), 1e4, device=device)
    sl = distance_slopes(H)
    eps = 1e-5
    out = torch.empty(T, H * vdim, device=device)
    dv = lambda t: t.to(device)  # noqa: E731
    steps = [(0, T)] if rows == 0 else [(a, min(T, a + rows)) for a in range(0, T, rows)]
    for a, b in steps:
        n = b - a
        qkv = torch.cat([q_raw[a:b].reshape(n, -1), k_raw[a:b].reshape(n, -1),
                         v_raw[a:b].reshape(n, -1)], 1).to(device)
        slots = torch.tensor([int(pages[p // BS]) * BS + p % BS for p in range(a, b)],
                             dtype=torch.int32, device=device)
        qn = torch.empty(n, H, dim, device=device)
        pre = rows == 0
        qm = torch.empty(n, H, G * dim, device=device) if pre else None
        ops.head_norm_append(qkv, dv(qw), dv(kw), eps, slots, kc, vc, H, G, dim, vdim, qn,
                             dv(talk * scale), qm, 0 if pre else n)
        meta = [dv(pages[None, :].contiguous()), dv(torch.tensor([0], dtype=torch.int32)),
                dv(torch.tensor([n], dtype=torch.int32)), dv(torch.tensor([b], dtype=torch.int32))]
        if pre:
            nq = (n + 31) // 32
            ops.attn_mixq_prefill(qm, kc, vc, *meta, dv(torch.zeros(nq, dtype=torch.int32)),
                                  dv(torch.arange(nq, dtype=torch.int32)), out[a:b],
                                  dv((talk.double() @ sl.double()).float()), dv(sink), chunk)
        else:
            ops.attn_talk_decode(qn, kc, vc, *meta, out[a:b], dv(sl), dv(talk), dv(sink), scale,
                                 chunk)
    return out.cpu()


_MEMO = {}


def want_attention(q_raw, k_raw, v_raw, qw, kw, talk, sink, scale, chunk, memo=None):
    """memo: a key under which the (slow) result is kept for the same inputs of other cases."""
    if memo is not None and memo in _MEMO:
        return _MEMO[memo]
    out = _want_attention(q_raw, k_raw, v_raw, qw, kw, talk, sink, scale, chunk)
    if memo is not None:
        _MEMO[memo] = out
    return out


def _want_attention(q_raw, k_raw, v_raw, qw, kw, talk, sink, scale, chunk):
    eps = 1e-5
    q = oracle.rms_unit(q_raw.double(), eps) * qw.double()
    k = oracle.rms_unit(k_raw.double(), eps) * kw.double()
    v = oracle.rms_unit(v_raw.double(), eps)
    return oracle.attention(q, k, v, talk.double(), sink.double(), scale, chunk)


SHAPES = [(4, 2, 16, 8), (3, 1, 8, 24), (2, 2, 32, 32), (6, 3, 24, 40)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dim,vdim", SHAPES)
@pytest.mark.parametrize("rows", [0, 1, 5, 32], ids=["prefill", "decode1", "decode5", "decode32"])
@pytest.mark.parametrize("chunk", [0, 7, 32, 45])
def test_attention_random(device, H, G, dim, vdim, rows, chunk):
    g = torch.Generator().manual_seed(H * 100 + chunk)
    T = 70
    q, k, v = (torch.randn(T, n, s, generator=g) for n, s in ((H, dim), (G, dim), (G, vdim)))
    qw, kw = 1 + 0.2 * torch.randn(dim, generator=g), 1 + 0.2 * torch.randn(dim, generator=g)
    talk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
    sink = torch.randn(H, generator=g)
    got = attend(device, q, k, v, qw, kw, talk, sink, 0.3, chunk, rows)
    close(got, want_attention(q, k, v, qw, kw, talk, sink, 0.3, chunk, memo=("r", H, chunk)), 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("rows", [0, 1, 3], ids=["prefill", "decode1", "decode3"])
@pytest.mark.parametrize("chunk,T,key,query", [
    (0, 300, 3, 299),            # hundreds of tokens back
    (0, 100, 31, 99), (0, 100, 32, 99), (0, 100, 63, 64), (0, 100, 64, 64),   # page borders
    (40, 130, 80, 119),          # first key of the query's block: just inside
    (40, 130, 79, 119),          # last key of the block before: just outside
    (40, 130, 80, 80), (40, 130, 79, 80), (40, 130, 119, 120),   # a block's first query
    (33, 70, 0, 32), (33, 70, 32, 33), (33, 70, 33, 65), (33, 70, 0, 1), (33, 70, 0, 0),
])
def test_attention_one_key_stands_out(device, rows, chunk, T, key, query):
    """The chosen key points along the chosen query in every head, so it takes the whole
    softmax if it is seen (and must not be seen outside the block)."""
    g = torch.Generator().manual_seed(7)
    H, G, dim, vdim = 4, 2, 16, 8
    q, k, v = (torch.randn(T, n, s, generator=g) for n, s in ((H, dim), (G, dim), (G, vdim)))
    q[query] = q[query, 0]                          # one direction for all heads of the query
    k[key] = q[query, 0]
    ones = torch.ones(dim)
    talk = torch.eye(H) + 0.05 * torch.randn(H, H, generator=g)
    sink = torch.zeros(H)
    got = attend(device, q, k, v, ones, ones, talk, sink, 2.0, chunk, rows)
    want = want_attention(q, k, v, ones, ones, talk, sink, 2.0, chunk, memo=("s", chunk, T, key, query))
    close(got, want, 1e-4)
    seen = key <= query and (chunk == 0 or key // chunk == query // chunk)
    # the last head has the flattest distance slope: there the key wins at any distance
    vk = oracle.rms_unit(v[key, G - 1].double(), 1e-5)
    hit = float((want[query].view(H, vdim)[H - 1] - vk).abs().max()) < 1e-2
    assert hit == seen


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("rows", [0, 1])
def test_attention_sink_takes_weight(device, rows):
    """A large sink logit leaves almost no weight to the keys; without it the rows sum to one."""
    g = torch.Generator().manual_seed(8)
    H, G, dim, vdim, T = 2, 1, 8, 4, 40
    q, k = torch.randn(T, H, dim, generator=g), torch.randn(T, G, dim, generator=g)
    v = torch.ones(T, G, vdim)                      # unit-norm values: output = sum of weights
    ones = torch.ones(dim)
    sink = torch.tensor([6.0, -30.0])
    got = attend(device, q, k, v, ones, ones, torch.eye(H), sink, 0.1, 0, rows).view(T, H, vdim)
    want = want_attention(q, k, v, ones, ones, torch.eye(H), sink, 0.1, 0).view(T, H, vdim)
    close(got, want, 1e-4)
    assert float(got[:, 0].max()) < 0.3 and float((got[:, 1] - 1).abs().max()) < 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_head_mixing_moves_a_score_between_heads(device):
    """talk = a swap of two heads of different key/value groups: the output of head 0 must be
    computed from head 1's scores but head 0's values."""
    g = torch.Generator().manual_seed(9)
    H, G, dim, vdim, T = 2, 2, 8, 4, 20
    q, k, v = (torch.randn(T, n, s, generator=g) for n, s in ((H, dim), (G, dim), (G, vdim)))
    ones, swap, sink = torch.ones(dim), torch.tensor([[0.0, 1.0], [1.0, 0.0]]), torch.zeros(H)
    for rows in (0, 1):
        got = attend(device, q, k, v, ones, ones, swap, sink, 0.7, 6, rows)
        close(got, want_attention(q, k, v, ones, ones, swap, sink, 0.7, 6), 1e-4)
    plain = want_attention(q, k, v, ones, ones, torch.eye(H), sink, 0.7, 6)
    assert float((plain - got.double()).abs().max()) > 1e-2
