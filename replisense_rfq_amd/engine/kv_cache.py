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
    """Pools of a layer-list model, all indexed by the block ids of the one block manager.

    Pools and state are held per layer RUN (``cfg.runs``: a layer that a loop runs several
    times has pages and state of its own in every pass; without a loop a run is a layer).
    Per run, by the kind of its mixer:
      attention          one K and one V pool with the layer's own head count and sizes
                         (``[num_blocks, G, block, dim]`` / ``[..., vdim]``);
      latent_attention   one pool ``[num_blocks, 1, block, kv_rank]`` of cached latents that
                         serves as keys and as values; a layer that reads another layer's
                         latent holds that layer's pool (the same tensor);
      diff_attention     K pool ``[num_blocks, G, block, 2 dim]`` (both score maps of a
                         key head side by side) and V pool ``[num_blocks, G, block, vdim]``;
      window_attention   K and V pools like ``attention``;
      rope_latent_attention   like ``latent_attention`` with rows ``[latent | rotated key
                         part]``, ``kv_rank + rot_dim`` wide;
      wkv, gla, channel_delta   no pages.
    Per-sequence state lives in slots; a sequence owns one while it runs (native core).  Every
    state pool is double buffered: a step reads half ``gen & 1`` of the slot and writes the
    other, so rows of one launch never read what the launch writes.  ``state``: the input
    convolutions' last inputs ``[L, 2 sublayers, 2 * slots, taps - 1, d]`` fp32;
    ``layer_state[i]``: name -> ``[2 * slots, ...]`` fp32 for what ``cfg.state_shapes(i)``
    lists (a wkv layer's matrices and its previous input row; a gla or channel_delta
    layer's matrices, and the convolutions' last inputs; with ``cfg.token_shift`` every
    layer's previous normed input row)."""

    def __init__(self, cfg, num_blocks: int, device, num_slots: int, block_size: int = 32,
                 dtype=torch.bfloat16, prefix_cache: bool = False):
        self.cfg = cfg
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.num_slots = num_slots
        mk = torch.zeros if torch.device(device).type != "cuda" else torch.empty
        self.k, self.v = [], []
        runs = tuple(getattr(cfg, "runs", range(cfg.n_layers)))
        for li in runs:
            m = cfg.layers[li].mixer
            if m.kind == "attention":
                self.k.append(mk((num_blocks, m.kv_heads, block_size, m.dim), dtype=dtype, device=device))
                self.v.append(mk((num_blocks, m.kv_heads, block_size, m.vdim), dtype=dtype, device=device))
            elif m.kind == "diff_attention":
                self.k.append(mk((num_blocks, m.kv_heads, block_size, 2 * m.dim), dtype=dtype, device=device))
                self.v.append(mk((num_blocks, m.kv_heads, block_size, m.vdim), dtype=dtype, device=device))
            elif m.kind == "window_attention":
                self.k.append(mk((num_blocks, m.kv_heads, block_size, m.dim), dtype=dtype, device=device))
                self.v.append(mk((num_blocks, m.kv_heads, block_size, m.vdim), dtype=dtype, device=device))
            elif m.kind in ("latent_attention", "rope_latent_attention"):
                if m.kv_from >= 0 and len(runs) != cfg.n_layers:
                    raise ValueError("a layer that reads another layer's latent cannot be looped")
                pool = self.k[m.kv_from] if m.kv_from >= 0 else \
                    mk((num_blocks, 1, block_size, m.kv_rank + m.rot_dim), dtype=dtype, device=device)
                self.k.append(pool)
                self.v.append(pool)
            else:
                self.k.append(None)
                self.v.append(None)
        self.state = torch.zeros((cfg.n_layers if cfg.canon_taps > 0 else 0, 2, 2 * num_slots,
                                  max(0, cfg.canon_taps - 1), cfg.hidden),
                                 dtype=torch.float32, device=device)
        self.layer_state = [{name: torch.zeros((2 * num_slots,) + tuple(shape), dtype=torch.float32,
                                               device=device)
                             for name, shape in cfg.state_shapes(li).items()}
                            for li in runs]
        self.scratch_block = num_blocks - 1
        self.prefix_cache = False            # a cached page carries no per-sequence state
        self.core = None

    @staticmethod
    def bytes_per_block(cfg, block_size: int = 32, dtype_bytes: int = 2) -> int:
        return cfg.kv_bytes_per_token(dtype_bytes=dtype_bytes) * block_size

    stats = KVCache.stats
