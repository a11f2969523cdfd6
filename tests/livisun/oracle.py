"""Slow, plain fp64/fp32 implementation of the Livisun design, one function per mechanism.

Written from the equations, token loops and all; shares no code with the package.  Weights
come as a dict under the checkpoint's tensor names, the configuration as a plain dict with
the keys of config.json.
"""
import math

import torch

F = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_sigmoid_glu(gate, up, limit):
    """y = g * sigmoid(1.702 g) * (u + 1), g = min(gate, limit), u = clamp(up, +-limit)."""
    g = torch.minimum(gate, torch.tensor(limit, dtype=gate.dtype))
    u = torch.clamp(up, -limit, limit)
    return g / (1 + torch.exp(-1.702 * g)) * (u + 1)


def sinusoid(positions, width):
    """pe[p, 2i] = sin(p * 10000^(-2i/width)), pe[p, 2i+1] = cos(same)."""
    pe = torch.zeros(len(positions), width, dtype=F)
    for r, p in enumerate(positions):
        for i in range(0, width, 2):
            a = p * 10000.0 ** (-i / width)
            pe[r, i] = math.sin(a)
            if i + 1 < width:
                pe[r, i + 1] = math.cos(a)
    return pe


def short_conv(h, w):
    """h_t + sum_j w[:, j] * h_{t - taps + 1 + j}, zeros before the first token."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def slopes(H):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F)


def attention(q, k, v, talk, sink, scale, chunk):
    """q [T, H, dim], k [T, G, dim], v [T, G, vdim] (already normed) -> [T, H * vdim]."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    sl = slopes(H)
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for i in range(T):
        lo = (i // chunk) * chunk if chunk > 0 else 0
        js = list(range(lo, i + 1))
        raw = torch.zeros(H, len(js), dtype=F)
        dist = torch.tensor([i - j for j in js], dtype=F)
        for g in range(H):
            raw[g] = (k[lo:i + 1, g // rep] * q[i, g]).sum(-1) * scale - sl[g] * dist
        mixed = talk @ raw
        for h in range(H):
            m = max(float(mixed[h].max()), float(sink[h]))
            e = torch.exp(mixed[h] - m)
            den = e.sum() + math.exp(float(sink[h]) - m)
            out[i, h] = ((e / den)[:, None] * v[lo:i + 1, h // rep]).sum(0)
    return out.reshape(T, -1)


def forward(cfg, W, tokens, residuals=None):
    """Logits [T, vocab] (float64) of one sequence."""
    W = {k: v.to(F) for k, v in W.items()}
    T, width, eps = len(tokens), cfg["width"], cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"] + sinusoid(range(T), width)
    for li, L in enumerate(cfg["layers"]):
        p, m = f"l{li}.", L["mixer"]
        H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        h = short_conv(rms_unit(x, eps) * W[p + "norm1"], W[p + "canon1"])
        q = rms_unit((h @ W[p + "mix.q"].T).view(T, H, dim), eps) * W[p + "mix.q.norm"]
        k = rms_unit((h @ W[p + "mix.k"].T).view(T, G, dim), eps) * W[p + "mix.k.norm"]
        v = rms_unit((h @ W[p + "mix.v"].T).view(T, G, vd), eps)
        a = attention(q, k, v, W[p + "mix.talk"], W[p + "mix.sink"], m["scale"],
                      (m.get("mask") or {}).get("size", 0))
        x = x + rms_unit(a @ W[p + "mix.o"].T, eps) * W[p + "norm1b"] * W[p + "ls1"]
        if L["mlp"] is not None:
            h = short_conv(rms_unit(x, eps) * W[p + "norm2"], W[p + "canon2"])
            y = gelu_sigmoid_glu(h @ W[p + "mlp.gate"].T, h @ W[p + "mlp.up"].T, L["mlp"]["limit"])
            x = x + rms_unit(y @ W[p + "mlp.down"].T, eps) * W[p + "norm2b"] * W[p + "ls2"]
        if residuals is not None:
            residuals.append(x.clone())
    return (rms_unit(x, eps) * W["final.norm"]) @ W["head"].T


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]
