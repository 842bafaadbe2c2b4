"""Host-memory K / V tier: drop-in for spotlight/modifiers/cpu_cache.py.

Same classes and calls as the reference (KVHash :6-47, topk_and_gather :50-57,
KVCache :60-130): the codes stay on the GPU, K and V of every layer outside
``freeze`` live in host memory, ``update`` appends, ``gather`` returns the
``budget`` best rows of every (batch, kv head) on the GPU.

The reference moves the scores to the host, runs ``topk`` and ``gather`` on the
CPU and copies the selected rows back each step (:50-57, :105-113).  Here the
host buffers are PINNED and mapped into the GPU's address space: the append
kernel writes new rows into them in place, the count-select runs on the GPU on
the scores where they are, and the gather kernel reads exactly the selected
rows over the host link -- no score transfer, no CPU work, one launch each.
For repeated decoding, ``spotlight_amd.decode.LayerDecodeState(host_store=True)``
puts the LRU resident table in front of such a store, so that only rows that
were not selected recently cross the link at all.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernel as K
from .gpu_cache import KVHash as _GpuKVHash, topk_and_gather  # noqa: F401  (same function, GPU select + gather)

INIT_SEQ_LEN = 1024 * 32 + 128


class KVHash(_GpuKVHash):
    init_seq_length = INIT_SEQ_LEN


class KVCache:
    init_seq_length = INIT_SEQ_LEN

    def __init__(self, batch_size, num_kv_heads, head_dim, num_layers, dtype=torch.bfloat16, freeze=(0, 1),
                 device=None):
        self.freeze = list(freeze)
        self.num_kv_heads = num_kv_heads
        self.length = [0 for _ in range(num_layers)]
        self.max_length = self.init_seq_length
        self.num_layers = num_layers
        if device is None:
            device = ["cuda" for _ in range(num_layers)]
        self.device = device
        shape = (batch_size, self.init_seq_length, num_kv_heads, head_dim)

        def alloc(i, dev):
            if i in self.freeze:
                return torch.zeros(shape, dtype=dtype, device=dev)
            return torch.zeros(shape, dtype=dtype, pin_memory=True)

        self.key_cache: List[torch.Tensor] = [alloc(i, dev) for i, dev in enumerate(device)]
        self.val_cache: List[torch.Tensor] = [alloc(i, dev) for i, dev in enumerate(device)]

    def gather(self, layer_idx, attn, budget, max_score: Optional[int] = None):
        """attn int16 [B,n,KH] on the GPU -> (K_sel, V_sel) [B,budget,KH,d] on the GPU."""
        n = attn.shape[1]
        return topk_and_gather(attn, self.key_cache[layer_idx][:, :n], self.val_cache[layer_idx][:, :n],
                               budget, max_score)

    def update(self, layer_idx, key, val):
        start = self.length[layer_idx]
        end = start + key.shape[1]
        K.cache_append(self.key_cache[layer_idx], key, start=start)
        K.cache_append(self.val_cache[layer_idx], val, start=start)
        self.length[layer_idx] = end
        return self.key_cache[layer_idx][:, :end], self.val_cache[layer_idx][:, :end]
