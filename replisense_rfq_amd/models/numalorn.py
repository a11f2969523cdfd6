"""Numalorn: post-norm residual layers of latent attention or wkv recurrence, each followed
by a mixture of experts with grouped sigmoid routing, on the kernels of csrc/kernels/mix_*.hip.

The residual stream x is fp32.  A sublayer reads x itself (rounded to the model's dtype for
its matrix products) and only its output is normed:

  x = embed[token]
  per layer:
    x += m * rms(mixer(x)) (1 + w1)
    x += m * rms(moe(x)) (1 + w2)            (layers with a feed-forward)
  logits = cap * tanh(head . (rms(x) (1 + w_final)) / cap)

latent attention   c_q = rms(W_dq h) w ; q = W_uq c_q ; c = rms(W_dkv h) w is the only thing
  cached (one kv_rank row per token; a layer with kv_from reads another layer's pool).  Keys
  and values are per-head up-projections of c, so both products are done in the latent
  space: q' = scale (q W_uk) per head, scores = q' . c, o' = softmax-with-sink(scores) . c,
  then o = W_uv o' per head and W_o.  The attention kernel therefore sees one shared
  key = value "head" of width kv_rank and H query heads.
wkv   five token-shift mixes h + (h' - h) mu of the layer's input (h' = the previous token's
  input: per-sequence state), r / k / v / gate projections, a decay
  w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0)), and per head the recurrence
  o_t = (S + diag(u) k_t v_t^T)^T r_t ; S <- diag(w_t) S + k_t v_t^T with S in a state slot
  (fp32); o is unit-normed per head, scaled, gated and projected.
moe   router logits and sigmoid scores in fp32; choice by score + correction inside the best
  groups; weights = chosen scores / their sum; a shared expert is added; the sum is fp32.
"""
from __future__ import annotations

import torch

from .. import ops
from ..parallel.tp import SINGLE, TPContext
from .config import LayeredConfig
from .moe import MoEBuffers, grouped_ok, moe_mlp
from .weights import init_numalorn_weights


class NumalornLM:
    stateful = True            # sequences own a state slot (wkv matrices, previous input rows)

    def __init__(self, cfg: LayeredConfig, device, tp: TPContext = SINGLE, seed: int = 0,
                 weights: dict | None = None, dtype=torch.bfloat16, moe_ep: bool = False):
        if tp.enabled:
            raise ValueError("layer-list models run at TP = 1")
        self.cfg = cfg
        self.tp = tp
        self.device = torch.device(device)
        self.dtype = dtype
        self.w = weights if weights is not None else init_numalorn_weights(cfg, self.device, dtype, seed)
        self.vocab_start = 0
        self.vocab_local = self.w["lm_head"].shape[0]
        # what the scheduler sizes the decode kernels' work lists by (column tiles of hq / hkv
        # heads per row): this model's kernels take none, one entry per row is the smallest
        self.hq = self.hkv = 1
        self.kv_k = self.kv_v = self.layer_state = None
        self.norms_folded = False
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False
        self._moe_bufs: dict = {}
        self._seq_ids = None            # work list of the decode section: sequence j, block 0
        for ly, lw in zip(cfg.layers, self.w["layers"]):
            if ly.mixer.kind == "latent_attention":
                lw["no_slope"] = torch.zeros(ly.mixer.heads, dtype=torch.float32, device=self.device)
            # experts whose sizes the framework's grouped MFMA expert GEMMs take run there
            # (the sparse decoder's alignment, GEMMs and combine, behind this model's router)
            # bf16 on the GPU with a latent width the MFMA tiles cover: both sections run the
            # MFMA latent attention; otherwise the general FMA kernels
            lw["mfma"] = bool(ly.mixer.kind == "latent_attention" and self.device.type == "cuda"
                              and dtype == torch.bfloat16 and ops.latent_mfma_ok(ly.mixer.kv_rank))
            lw["grouped"] = bool(ly.mlp is not None and self.device.type == "cuda"
                                 and dtype == torch.bfloat16 and grouped_ok(lw["w13"], lw["w2e"]))

    # engine hooks shared with the other decoders
    def fold_norms(self) -> bool:
        return False

    def tile_decode_weights(self, mode: str | None = None) -> int:
        return 0

    def attach_kv_cache(self, k_pools, v_pools, state=None, layer_state=None) -> None:
        """Latent pools [num_blocks, 1, block, kv_rank] per attention layer (shared tensors
        where a layer reads another's); layer_state[i]: "wkv" [2*slots, H, N, N] and "prev"
        [2*slots, d] fp32 for the wkv layers."""
        assert len(k_pools) == self.cfg.n_layers
        self.kv_k, self.kv_v, self.layer_state = k_pools, v_pools, layer_state

    def _decode_work(self, n: int):
        """(sequence index, query block 0) per decode-section sequence; views of two tensors
        that only grow (never inside a graph capture: the warm-up run sizes them)."""
        if self._seq_ids is None or self._seq_ids[0].numel() < n:
            size = max(1024, 2 * n)
            self._seq_ids = (torch.arange(size, dtype=torch.int32, device=self.device),
                             torch.zeros(size, dtype=torch.int32, device=self.device))
        return self._seq_ids[0][:n], self._seq_ids[1][:n]

    def _run_rows(self, m):
        """First row of every scheduled run of the step (decode section, then prefill section;
        -1 for a sequence without rows: padding of a graph step), for the recurrence's grid."""
        if self.device.type != "cuda" or not any(ly.mixer.kind == "wkv" for ly in self.cfg.layers):
            return None
        parts = []
        if m.dec_q_len is not None and m.dec_q_len.numel():
            parts.append(torch.where(m.dec_q_len > 0, m.dec_q_start, -1))
        if m.pf_q_len is not None and m.pf_q_len.numel():
            parts.append(torch.where(m.pf_q_len > 0, m.pf_q_start + m.num_decode, -1))
        if not parts:
            return None
        return (parts[0] if len(parts) == 1 else torch.cat(parts)).to(torch.int32)

    def weight_bytes(self) -> int:
        tot = sum(v.numel() * v.element_size() for v in self.w.values() if isinstance(v, torch.Tensor))
        for lw in self.w["layers"]:
            tot += sum(t.numel() * t.element_size() for t in lw.values() if isinstance(t, torch.Tensor))
        return tot

    # ------------------------------------------------------------------ mixers
    def _latent_attention(self, li, mx, lw, h, m):
        T, D = m.num_tokens, m.num_decode
        H, R, eps, dt = mx.heads, mx.kv_rank, self.cfg.rms_eps, self.dtype
        pool = self.kv_k[li]
        dn = ops.matmul_nt(h, lw["down"])                       # [T, q_rank (+ kv_rank)]
        cq = ops.rms_norm_rows(dn[:, :mx.q_rank], lw["dq_norm"], eps,
                               torch.empty((T, mx.q_rank), dtype=dt, device=h.device))
        if mx.kv_from < 0:
            ops.latent_norm_append(dn[:, mx.q_rank:], lw["dkv_norm"], eps, m.slot_mapping[:T], pool)
        q = ops.matmul_nt(cq, lw["uq"]).view(T, H, mx.dim)
        lat = torch.empty((T, H * R), dtype=dt, device=h.device)
        if lw["mfma"]:
            # queries carried into the latent space, [H, T, R] as the batched product leaves
            # them; the kernel reads them through strides and scales the scores in fp32
            qa = torch.bmm(q.transpose(0, 1), lw["uk"]).transpose(0, 1)
            if D > 0:
                ids, zeros = self._decode_work(m.dec_q_len.shape[0])
                ops.attn_latent_mfma(qa[:D], pool, m.dec_block_tables, m.dec_q_start, m.dec_q_len,
                                     m.dec_kv_len, ids, zeros, lat[:D], lw["sink"], mx.scale)
            if T > D:
                ops.attn_latent_mfma(qa[D:], pool, m.pf_block_tables, m.pf_q_start, m.pf_q_len,
                                     m.pf_kv_len, m.work_seq, m.work_qblk, lat[D:T], lw["sink"],
                                     mx.scale)
            ov = torch.bmm(lat.view(T, H, R).transpose(0, 1), lw["uv_t"])
            return ops.matmul_nt(ov.transpose(0, 1).reshape(T, H * mx.vdim), lw["o"])
        # absorbed queries, fp32 (they are score operands): [H, T, R] -> [T, H, R], scaled
        qa = torch.empty((T, H, R), dtype=torch.float32, device=h.device)
        torch.mul(ops.bmm_f32(q.transpose(0, 1), lw["uk"]).transpose(0, 1), mx.scale, out=qa)
        if D > 0:
            ops.attn_talk_decode(qa[:D], pool, pool, m.dec_block_tables, m.dec_q_start,
                                 m.dec_q_len, m.dec_kv_len, lat[:D], lw["no_slope"], None,
                                 lw["sink"], 1.0, 0)
        if T > D:
            ops.attn_mixq_prefill(qa[D:], pool, pool, m.pf_block_tables, m.pf_q_start, m.pf_q_len,
                                  m.pf_kv_len, m.work_seq, m.work_qblk, lat[D:T], lw["no_slope"],
                                  lw["sink"], 0, m.prefill_qblk)
        ov = torch.bmm(lat.view(T, H, R).transpose(0, 1), lw["uv_t"])       # [H, T, vdim]
        return ops.matmul_nt(ov.transpose(0, 1).reshape(T, H * mx.vdim), lw["o"])

    def _wkv(self, li, mx, lw, x, m, rows):
        T, dt = m.num_tokens, self.dtype
        rs, rb, rf, pos, runs = rows
        st = self.layer_state[li]
        HN = mx.heads * mx.dim
        mixes = ops.token_shift_mix(x, lw["mu"], st["prev"], rs, rb, rf, pos,
                                    torch.empty((5, T, x.shape[1]), dtype=dt, device=x.device))
        # r, k, v, gate: four plain products (one batched call over the four [d, d] weights
        # returned garbage from the vendor library at 4,096 rows of 4096-wide layers)
        rkvg = torch.empty((4, T, HN), dtype=dt, device=x.device)
        for s in range(4):
            torch.mm(mixes[s], lw["rkvg"][s].t(), out=rkvg[s])
        zw = ops.matmul_nt(torch.tanh(ops.matmul_nt(mixes[4], lw["w1"])), lw["w2"])
        y = ops.wkv_recurrence(rkvg[0], rkvg[1], rkvg[2], zw, lw["w0"], lw["u"], rkvg[3], lw["gn"],
                               self.cfg.rms_eps, st["wkv"], rs, rb, rf, pos,
                               torch.empty((T, HN), dtype=dt, device=x.device), runs)
        return ops.matmul_nt(y, lw["o"])

    def _moe_buffers(self, T: int, f, d: int) -> MoEBuffers:
        cap = 1
        while cap < T:
            cap *= 2
        key = (cap, f.top, f.experts, f.ff)
        if key not in self._moe_bufs:
            self._moe_bufs[key] = MoEBuffers.allocate(cap, f.top, f.experts, d, f.ff, self.device,
                                                      self.dtype)
        return self._moe_bufs[key]

    def _moe(self, f, lw, h):
        T, dev = h.shape[0], h.device
        z = ops.matmul_nt(h, lw["router"], out_dtype=torch.float32)
        base = None
        if f.shared_ff:
            base = ops.matmul_nt(ops.silu_mul_any(ops.matmul_nt(h, lw["shared_gu"])), lw["shared_down"])
        if lw["grouped"]:
            y = moe_mlp(h, lw["router"], lw["w13"], lw["w2e"], f.top, self._moe_buffers(T, f, h.shape[1]),
                        routing=lambda w, i: ops.moe_route_grouped(z, lw["correction"], f.top,
                                                                   f.groups, f.keep, i, w))
            return y if base is None else y.float().add_(base)
        ids = torch.empty((T, f.top), dtype=torch.int32, device=dev)
        wts = torch.empty((T, f.top), dtype=torch.float32, device=dev)
        ops.moe_route_grouped(z, lw["correction"], f.top, f.groups, f.keep, ids, wts)
        return ops.moe_experts(h, ids, wts, lw["w13"], lw["w2e"], base,
                               torch.empty((T, h.shape[1]), dtype=torch.float32, device=dev))

    # ------------------------------------------------------------------ forward
    def forward(self, m, taps: list | None = None) -> torch.Tensor:
        """Logits [rows, V] (fp32) of the step.  ``taps``: a list that receives the
        residual stream after every layer (debugging / layer-wise tests)."""
        cfg, w = self.cfg, self.w
        T, eps, mult, dt = m.num_tokens, cfg.rms_eps, cfg.residual_mult, self.dtype
        pos = m.positions[:T]
        rows = (m.extra["row_state"], m.extra["row_back"], m.extra["row_fwd"], pos,
                self._run_rows(m))
        x = ops.embed_rows(m.input_ids[:T], w["embed"])
        h = x if dt == torch.float32 else x.to(dt)
        hbuf = None if dt == torch.float32 else h
        for li, ly in enumerate(cfg.layers):
            lw, mx = w["layers"][li], ly.mixer
            if mx.kind == "latent_attention":
                y = self._latent_attention(li, mx, lw, h, m)
            else:
                y = self._wkv(li, mx, lw, x, m, rows)
            ops.post_norm_add(y, x, lw["norm1"], mult, eps, hbuf)
            if ly.mlp is not None:
                y = self._moe(ly.mlp, lw, h)
                ops.post_norm_add(y, x, lw["norm2"], mult, eps, hbuf)
            if taps is not None:
                taps.append(x.clone())
        xs = x if m.logits_idx is None else x.index_select(0, m.logits_idx.long())
        hn = ops.rms_norm_rows(xs, w["final_norm"], eps, torch.empty(xs.shape, dtype=dt, device=x.device), 1.0)
        logits = ops.matmul_nt(hn, w["lm_head"], out_dtype=torch.float32)
        if cfg.logit_softcap > 0:
            ops.softcap(logits, cfg.logit_softcap)
        return logits
