"""Paged KV cache: device pools + native block manager + prefix cache.

Pools are two tensors ``[L, num_blocks, Hkv_local, 32, 128]`` (bf16), sized from a
fraction of free HBM (288 GB per MI355X: a Llama-3-8B replica gets ~100 GB of
KV = ~800K tokens, far beyond the ≤3.7K-token RFQ sequences × max batch).  The
last block is a scratch page for padded graph rows and is never handed out.
Block bookkeeping (refcounts, free list, LRU of cached prefix blocks, chained
block hashes) lives in the native engine core (csrc/runtime/engine_core.cpp over
block_manager.cpp); this class owns the device pools.
"""
from __future__ import annotations

import torch

from ..models.config import ModelConfig


class KVCache:
    def __init__(self, cfg: ModelConfig, hkv_local: int, num_blocks: int, device,
                 block_size: int = 32, dtype=torch.bfloat16, prefix_cache: bool = True):
        if block_size != 32:
            raise ValueError("the gfx950 attention kernels use 32-token pages")
        self.cfg = cfg
        self.block_size = block_size
        self.num_blocks = num_blocks
        shape = (cfg.n_layers, num_blocks, hkv_local, block_size, cfg.head_dim)
        self.k = torch.empty(shape, dtype=dtype, device=device)
        self.v = torch.empty(shape, dtype=dtype, device=device)
        if not self.k.is_cuda:
            self.k.zero_()
            self.v.zero_()
        self.scratch_block = num_blocks - 1      # blocks [0, num_blocks-1) belong to the core
        self.prefix_cache = prefix_cache
        self.core = None                         # set by the engine (block accounting)

    @staticmethod
    def bytes_per_block(cfg: ModelConfig, hkv_local: int, block_size: int = 32) -> int:
        return 2 * cfg.n_layers * hkv_local * block_size * cfg.head_dim * 2

    @classmethod
    def blocks_for_memory(cls, cfg, hkv_local, free_bytes, fraction, block_size=32) -> int:
        return max(16, int(free_bytes * fraction) // cls.bytes_per_block(cfg, hkv_local, block_size))

    def stats(self, core=None) -> dict:
        core = core if core is not None else self.core
        return {"blocks": self.num_blocks, "free": core.num_free_blocks,
                "cached": core.num_cached_blocks, "prefix_queries": core.prefix_queries,
                "prefix_hits": core.prefix_hits, "evictions": core.evictions}


class LayeredKVCache:
    """Pools of a layer-list model: one K and one V pool per layer, each with the layer's
    own head count and sizes (``[num_blocks, G, block, dim]`` / ``[..., vdim]``), all
    indexed by the same block ids, plus the state pool of the input convolutions:
    ``[L, 2 sublayers, 2 * slots, taps - 1, d]`` fp32.  A sequence owns one slot while it
    runs (native core); the pool is double buffered, a step reads half ``gen & 1`` of the
    slot and writes the other, so rows of one launch never read what the launch writes."""

    def __init__(self, cfg, num_blocks: int, device, num_slots: int, block_size: int = 32,
                 dtype=torch.bfloat16, prefix_cache: bool = False):
        self.cfg = cfg
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.num_slots = num_slots
        mk = torch.zeros if torch.device(device).type != "cuda" else torch.empty
        self.k = [mk((num_blocks, ly.mixer.kv_heads, block_size, ly.mixer.dim), dtype=dtype,
                     device=device) for ly in cfg.layers]
        self.v = [mk((num_blocks, ly.mixer.kv_heads, block_size, ly.mixer.vdim), dtype=dtype,
                     device=device) for ly in cfg.layers]
        self.state = torch.zeros((cfg.n_layers, 2, 2 * num_slots, max(0, cfg.canon_taps - 1),
                                  cfg.hidden), dtype=torch.float32, device=device)
        self.scratch_block = num_blocks - 1
        self.prefix_cache = False            # a cached page carries no convolution state
        self.core = None

    @staticmethod
    def bytes_per_block(cfg, block_size: int = 32, dtype_bytes: int = 2) -> int:
        return cfg.kv_bytes_per_token(dtype_bytes=dtype_bytes) * block_size

    stats = KVCache.stats
