"""Numalorn, slowly: one function per mechanism, float64, whole sequences, no cache.

Written from the equations only; it shares no code with the package.  ``full`` maps the
checkpoint's tensor names to tensors, ``cfg`` is the dict of config.json.
"""
import math

import torch

F = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def silu(z):
    return z / (1.0 + torch.exp(-z))


def shift_mix(h, mu):
    """h_t + (h_(t-1) - h_t) mu, with zeros before the first token."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def decay(z, w0):
    """Per-channel decay in (0, 1) from the decay projection's output."""
    return torch.exp(-torch.exp(z + w0))


def wkv_scan(r, k, v, w, u, S=None):
    """Token by token per head: o_t = (S + diag(u) k_t v_t^T)^T r_t, then
    S <- diag(w_t) S + k_t v_t^T.  r, k, v, w: [T, H, N]; u: [H, N]; S: [H, N, N] (key channel,
    value channel), zeros at the start.  Returns (o [T, H, N], S)."""
    T, H, N = r.shape
    S = torch.zeros(H, N, N, dtype=F) if S is None else S.clone()
    out = torch.zeros(T, H, N, dtype=F)
    for t in range(T):
        for hd in range(H):
            kv = torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = (S[hd] + u[hd][:, None] * kv).T @ r[t, hd]
            S[hd] = w[t, hd][:, None] * S[hd] + kv
    return out, S


def wkv_mixer(h, get, m, eps):
    """RWKV-style time mixing with a data-dependent decay and a bonus for the current token."""
    T, d = h.shape
    H, N = m["heads"], m["dim"]
    xr, xk, xv, xg, xw = (shift_mix(h, get("mu." + s)) for s in "rkvgw")
    r = (xr @ get("r").T).view(T, H, N)
    k = (xk @ get("k").T).view(T, H, N)
    v = (xv @ get("v").T).view(T, H, N)
    gate = silu(xg @ get("g").T)
    w = decay(torch.tanh(xw @ get("w1").T) @ get("w2").T, get("w0")).view(T, H, N)
    out, _ = wkv_scan(r, k, v, w, get("u").view(H, N))
    out = rms_unit(out, eps).reshape(T, H * N) * get("norm") * gate
    return out @ get("o").T


def latent_of(h, get, eps):
    """The cached latent of a layer that owns a down projection."""
    return norm_plain(h @ get("dkv").T, get("dkv.norm"), eps)


def latent_attention(h, c, get, m, eps):
    """Causal attention whose keys and values are up-projections of the latent rows ``c``;
    the softmax's denominator holds exp(sink_h) once, unscaled, with no value."""
    T = h.shape[0]
    H, N, V = m["heads"], m["dim"], m["vdim"]
    cq = norm_plain(h @ get("dq").T, get("dq.norm"), eps)
    q = (cq @ get("uq").T).view(T, H, N)
    k = (c @ get("uk").T).view(T, H, N)
    v = (c @ get("uv").T).view(T, H, V)
    sink = get("sink")
    out = torch.zeros(T, H, V, dtype=F)
    for i in range(T):
        for hd in range(H):
            s = (k[:i + 1, hd] @ q[i, hd]) * m["scale"]
            mx = torch.maximum(s.max(), sink[hd])
            e = torch.exp(s - mx)
            den = e.sum() + torch.exp(sink[hd] - mx)
            out[i, hd] = (e[:, None] * v[:i + 1, hd]).sum(0) / den
    return out.reshape(T, H * V) @ get("o").T


def expert(h, get, pre):
    return (silu(h @ get(pre + "gate").T) * (h @ get(pre + "up").T)) @ get(pre + "down").T


def route(h, get, r):
    """Chosen experts and their weights for every row: sigmoid scores; the choice adds a
    correction and is limited to the best groups (a group's score = its two largest choice
    scores); the weights are the uncorrected scores over their sum."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ get("router").T)
    choice = s + get("correction")
    g = r.get("groups")
    if g:
        per = E // g["count"]
        grp = choice.view(-1, g["count"], per)
        gs = grp.topk(min(2, per), -1).values.sum(-1)
        keep = gs.topk(g["keep"], -1).indices
        allowed = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, keep, True)
        choice = torch.where(allowed[:, :, None].expand_as(grp), grp,
                             torch.full_like(grp, -math.inf)).reshape(-1, E)
    idx = choice.topk(top, -1).indices
    wt = s.gather(1, idx)
    return idx, wt / (wt.sum(-1, keepdim=True) + 1e-20)


def moe(h, get, f):
    idx, wt = route(h, get, f["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wt[t]):
            out[t] += a * expert(h[t:t + 1], get, f"e{e}.")[0]
    if f.get("shared"):
        out = out + expert(h, get, "shared.")
    return out


def forward(cfg, full, tokens, layers_out=None):
    """Logits [T, vocab] (float64) of one sequence; ``layers_out`` receives the residual
    stream after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    W = {k: v.to(F) for k, v in full.items()}
    x = W["embed"][torch.tensor(tokens)]
    latents = {}
    for i, ly in enumerate(cfg["layers"]):
        p = f"l{i}."
        mix = lambda k: W[p + "mix." + k]          # noqa: E731
        ff = lambda k: W[p + "mlp." + k]           # noqa: E731
        m = ly["mixer"]
        if ly["type"] == "wkv":
            y = wkv_mixer(x, mix, m, eps)
        elif ly["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_of(x, mix, eps)
                src = i
            y = latent_attention(x, latents[src], mix, m, eps)
        else:
            raise ValueError(ly["type"])
        x = x + mult * norm_around_zero(y, W[p + "norm1"], eps)
        if ly.get("mlp") is not None:
            x = x + mult * norm_around_zero(moe(x, ff, ly["mlp"]), W[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    y = norm_around_zero(x, W["final.norm"], eps) @ W["head"].T
    cap = cfg["logit_softcap"]
    return cap * torch.tanh(y / cap)


def greedy(cfg, full, prompt, n):
    """n tokens, each the argmax of the logits after everything before it."""
    t, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, full, t)[-1].argmax())
        out.append(nxt)
        t.append(nxt)
    return out
