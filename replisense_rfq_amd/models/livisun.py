"""Livisun: a layer-list decoder on the gfx950 kernels of csrc/kernels/mix_*.hip.

Each layer of the list has its own attention sizes and may have no feed-forward.
The residual stream is fp32 and every norm is computed in fp32; matrix products run
in the model's dtype (bf16, or fp32 when the model is served in full precision).
A step consumes the engine's mixed token batch ``[decode / short rows | prefill
rows]`` (ForwardMeta) like the other decoders:

  embed * scale + sinusoid(position)                                   -> x (fp32)
  per layer:
    h = rms(x) w1                       (fused with the previous sublayer's update)
    h + causal conv over the last `taps` inputs of the sequence (state slot)
    q | k | v GEMM -> per-head rms norms, k and unit-norm v into the paged cache,
                      mixed queries for the prefill rows
    attention: scale q.k - slope_h (i - j), mixed over heads, block mask, sink
       decode / short rows: attn_talk_decode (mixes raw scores in LDS)
       prefill rows:        attn_mixq_prefill (queries pre-mixed, keys concatenated)
       bf16 with head sizes of the MFMA tiles: attn_mix_mfma for both sections
    o GEMM ; x += rms(y) w1b ls1 ; h = rms(x) w2          (one kernel)
    conv ; gate|up GEMM ; clamped GLU ; down GEMM ; x += rms(y) w2b ls2
  final norm on the rows that need logits -> head GEMM (fp32 logits).

Head mixing: score'_h = sum_g T[h, g] score_g is linear in the queries, so for the
prefill rows the mixing matrix (times the score scale) is applied to the normed
queries once per token: q~[h, c] = sum_{g in group c} scale T[h, g] q_g, one vector
per key/value head c.  Head h's mixed score is then the single product of
q~[h, :] with the concatenation of all G key heads, minus (T slope)_h (i - j), and
the attention kernel is an ordinary multi-query flash kernel with a wider key.
"""
from __future__ import annotations

import torch

from .. import ops
from ..parallel.tp import SINGLE, TPContext
from .config import LayeredConfig
from .weights import init_layered_weights

GLU_ALPHA = 1.702          # g * sigmoid(GLU_ALPHA * g) gate of the feed-forward
SLOPE_LOG2_SPAN = 8.0      # head h's distance slope is 2^(-SLOPE_LOG2_SPAN (h+1) / H)


def distance_slopes(heads: int) -> torch.Tensor:
    h = torch.arange(1, heads + 1, dtype=torch.float64)
    return torch.pow(2.0, -SLOPE_LOG2_SPAN * h / heads).float()


class LivisunLM:
    stateful = True            # sequences own a state slot (the convolutions' last inputs)

    def __init__(self, cfg: LayeredConfig, device, tp: TPContext = SINGLE, seed: int = 0,
                 weights: dict | None = None, dtype=torch.bfloat16, moe_ep: bool = False):
        if tp.enabled:
            raise ValueError("layer-list models run at TP = 1")
        self.cfg = cfg
        self.tp = tp
        self.device = torch.device(device)
        self.dtype = dtype
        self.w = weights if weights is not None else init_layered_weights(cfg, self.device, dtype, seed)
        self.vocab_start = 0
        self.vocab_local = self.w["lm_head"].shape[0]
        # widest layer: what the scheduler's work lists and split heuristics are sized by
        self.hq = max(ly.mixer.heads for ly in cfg.layers)
        self.hkv = max(ly.mixer.kv_heads for ly in cfg.layers)
        self.kv_k = self.kv_v = None
        self.state = None
        self.norms_folded = False
        self.inv_freq = ops.sinusoid_inv_freq(cfg.hidden, self.device)
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False
        for ly, lw in zip(cfg.layers, self.w["layers"]):
            m = ly.mixer
            slopes = distance_slopes(m.heads).to(self.device)
            lw["slopes"] = slopes
            lw["talk_scaled"] = (lw["talk"] * m.scale).contiguous()
            lw["slopes_mixed"] = (lw["talk"].double() @ slopes.double()).float().contiguous()
            # bf16 on the GPU with sizes the MFMA tiles cover: decode rows too run the
            # mixed-query kernel (one work item per sequence); otherwise attn_talk_decode
            lw["mixq_decode"] = bool(self.device.type == "cuda" and dtype == torch.bfloat16
                                     and ops.mixq_mfma_ok(m.heads, m.kv_heads, m.dim, m.vdim))
        self._seq_ids = None            # work list of the decode section: sequence j, block 0

    # engine hooks shared with DecoderLM
    def fold_norms(self) -> bool:
        return False

    def tile_decode_weights(self, mode: str | None = None) -> int:
        return 0

    def attach_kv_cache(self, k_pools, v_pools, state=None, layer_state=None) -> None:
        """Per-layer pools [num_blocks, G, block, dim | vdim]; state [L, 2, 2*slots, taps-1, d]."""
        assert len(k_pools) == self.cfg.n_layers
        self.kv_k, self.kv_v, self.state = k_pools, v_pools, state

    def _decode_work(self, n: int):
        """(sequence index, query block 0) per decode-section sequence; views of two
        tensors that only grow (never inside a graph capture: the warm-up run sizes them)."""
        if self._seq_ids is None or self._seq_ids[0].numel() < n:
            size = max(1024, 2 * n)
            self._seq_ids = (torch.arange(size, dtype=torch.int32, device=self.device),
                             torch.zeros(size, dtype=torch.int32, device=self.device))
        return self._seq_ids[0][:n], self._seq_ids[1][:n]

    def weight_bytes(self) -> int:
        tot = sum(v.numel() * v.element_size() for v in self.w.values() if isinstance(v, torch.Tensor))
        for lw in self.w["layers"]:
            tot += sum(t.numel() * t.element_size() for t in lw.values())
        return tot

    # ------------------------------------------------------------------ forward
    def forward(self, m, taps: list | None = None) -> torch.Tensor:
        """Logits [rows, V] (fp32) of the step.  ``taps``: a list that receives the
        residual stream after every layer (debugging / layer-wise tests)."""
        cfg, w = self.cfg, self.w
        T, D = m.num_tokens, m.num_decode
        eps = cfg.rms_eps
        dt, dev = self.dtype, self.device
        rs, rb, rf = m.extra["row_state"], m.extra["row_back"], m.extra["row_fwd"]
        pos = m.positions[:T]
        x = ops.embed_sinusoid(m.input_ids[:T], pos, w["embed"], self.inv_freq, cfg.embed_scale)
        h = ops.sandwich_norm(None, x, None, None, w["layers"][0]["norm1"], eps)
        hc = torch.empty((T, cfg.hidden), dtype=dt, device=dev)
        L = cfg.n_layers
        for li, ly in enumerate(cfg.layers):
            lw, mx = w["layers"][li], ly.mixer
            H, G, dim, vd = mx.heads, mx.kv_heads, mx.dim, mx.vdim
            ops.canon_conv(h, lw["canon1"], self.state[li, 0], rs, rb, rf, pos, hc)
            qkv = ops.matmul_nt(hc, lw["qkv"])
            qn = torch.empty((T, H, dim), dtype=torch.float32, device=dev)
            mfma = lw["mixq_decode"]           # queries stay unmixed: the kernel mixes them
            mix_from = T if mfma else D
            qmix = torch.empty((T - mix_from, H, G * dim), dtype=torch.float32, device=dev) \
                if T > mix_from else None
            ops.head_norm_append(qkv, lw["q_norm"], lw["k_norm"], eps, m.slot_mapping[:T],
                                 self.kv_k[li], self.kv_v[li], H, G, dim, vd, qn,
                                 lw["talk_scaled"], qmix, mix_from)
            attn = torch.empty((T, H * vd), dtype=dt, device=dev)
            if D > 0 and mfma:
                ids, zeros = self._decode_work(m.dec_q_len.shape[0])
                ops.attn_mix_mfma(qn[:D], lw["talk_scaled"], self.kv_k[li], self.kv_v[li],
                                  m.dec_block_tables, m.dec_q_start, m.dec_q_len, m.dec_kv_len,
                                  ids, zeros, attn[:D], lw["slopes_mixed"], lw["sink"], mx.chunk,
                                  grouped=True)
            elif D > 0:
                ops.attn_talk_decode(qn[:D], self.kv_k[li], self.kv_v[li], m.dec_block_tables,
                                     m.dec_q_start, m.dec_q_len, m.dec_kv_len, attn[:D],
                                     lw["slopes"], lw["talk"], lw["sink"], mx.scale, mx.chunk)
            if T > D and mfma:
                ops.attn_mix_mfma(qn[D:], lw["talk_scaled"], self.kv_k[li], self.kv_v[li],
                                  m.pf_block_tables, m.pf_q_start, m.pf_q_len, m.pf_kv_len,
                                  m.work_seq, m.work_qblk, attn[D:T], lw["slopes_mixed"],
                                  lw["sink"], mx.chunk)
            elif T > D:
                ops.attn_mixq_prefill(qmix, self.kv_k[li], self.kv_v[li], m.pf_block_tables,
                                      m.pf_q_start, m.pf_q_len, m.pf_kv_len, m.work_seq,
                                      m.work_qblk, attn[D:T], lw["slopes_mixed"], lw["sink"],
                                      mx.chunk, m.prefill_qblk)
            y = ops.matmul_nt(attn, lw["o"])
            nxt = w["layers"][li + 1]["norm1"] if li + 1 < L else w["final_norm"]
            if ly.mlp is not None:
                h = ops.sandwich_norm(y, x, lw["norm1b"], lw["ls1"], lw["norm2"], eps, out=h)
                ops.canon_conv(h, lw["canon2"], self.state[li, 1], rs, rb, rf, pos, hc)
                gu = ops.matmul_nt(hc, lw["gate_up"])
                act = ops.glu_clamped(gu, ly.mlp.limit, GLU_ALPHA)
                y = ops.matmul_nt(act, lw["down"])
                h = ops.sandwich_norm(y, x, lw["norm2b"], lw["ls2"], nxt, eps, out=h)
            else:
                h = ops.sandwich_norm(y, x, lw["norm1b"], lw["ls1"], nxt, eps, out=h)
            if taps is not None:
                taps.append(x.clone())
        hs = h if m.logits_idx is None else h.index_select(0, m.logits_idx.long())
        return ops.matmul_nt(hs.to(dt), w["lm_head"], out_dtype=torch.float32)
