"""Preallocated per-layer code / K / V buffers with append and top-k gather.

Same classes, constructor arguments, attributes and return conventions as the
reference's ``spotlight/modifiers/gpu_cache.py`` (KVHash :6-45,
topk_and_gather :48-54, KVCache :57-118): buffers are ``[B, L, KH, head_dim]``
zero-initialised tensors owned by the object, ``update`` appends at the
per-layer length and returns views ``[:, :end]``, ``gather`` returns the
``budget`` best rows of every (batch, kv head).  What differs is underneath:
the append, the top-k (count-select with lowest-index tie break, rows in
ascending token order) and the gather are HIP kernels.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernel as K

INIT_SEQ_LEN = 1024 * 2048 + 128


class KVHash:
    """Packed key codes of every layer (``head_dim`` = words per code)."""

    init_seq_length = INIT_SEQ_LEN

    def __init__(self, batch_size, num_kv_heads, head_dim, num_layers, dtype=torch.bfloat16, device=None):
        self.num_kv_heads = num_kv_heads
        self.length = [0 for _ in range(num_layers)]
        self.max_length = self.init_seq_length
        self.num_layers = num_layers
        if device is None:
            device = ["cuda" for _ in range(num_layers)]
        self.key_cache = [
            torch.zeros((batch_size, self.init_seq_length, num_kv_heads, head_dim), dtype=dtype, device=dev)
            for dev in device]

    def update(self, layer_idx, key):
        start = self.length[layer_idx]
        end = start + key.shape[1]
        K.cache_append(self.key_cache[layer_idx], key, start=start)
        self.length[layer_idx] = end
        return self.key_cache[layer_idx][:, :end]


MAX_SCORE_BOUND = 4607   # the largest score sl_topk_select covers (36 query heads of 128 bits per kv head)


def topk_and_gather(attn, keys, vals, budget, max_score: Optional[int] = None):
    """attn int16 [B,n,KH] scores, keys/vals [B,L,KH,d] -> (K_sel, V_sel) [B,budget,KH,d].

    ``max_score`` bounds the scores (G * nbits for the Hamming scorer).  Without it the widest
    range the selector covers is assumed (scores up to 4607): still exact, never a device
    round trip, but more histogram bins than a known bound needs."""
    if max_score is None:
        max_score = MAX_SCORE_BOUND
    ind = K.topk_select(attn, budget, max_score)
    return K.gather_kv(keys, vals, ind)


class KVCache:
    """K and V rows of every layer."""

    init_seq_length = INIT_SEQ_LEN

    def __init__(self, batch_size, num_kv_heads, head_dim, num_layers, dtype=torch.bfloat16, device=None,
                 **kwargs):
        self.num_kv_heads = num_kv_heads
        self.max_score = kwargs.get("max_score")   # optional bound of the scores gather() will see (G * nbits)
        self.length = [0 for _ in range(num_layers)]
        self.max_length = self.init_seq_length
        self.num_layers = num_layers
        if device is None:
            device = ["cuda" for _ in range(num_layers)]
        self.device = device
        shape = (batch_size, self.init_seq_length, num_kv_heads, head_dim)
        self.key_cache: List[torch.Tensor] = [torch.zeros(shape, dtype=dtype, device=dev) for dev in device]
        self.val_cache: List[torch.Tensor] = [torch.zeros(shape, dtype=dtype, device=dev) for dev in device]

    def gather(self, layer_idx, attn, budget, max_score: Optional[int] = None):
        n = attn.shape[1]
        return topk_and_gather(attn, self.key_cache[layer_idx][:, :n], self.val_cache[layer_idx][:, :n],
                               budget, max_score if max_score is not None else self.max_score)

    def update(self, layer_idx, key, val):
        start = self.length[layer_idx]
        end = start + key.shape[1]
        K.cache_append(self.key_cache[layer_idx], key, start=start)
        K.cache_append(self.val_cache[layer_idx], val, start=start)
        self.length[layer_idx] = end
        return self.key_cache[layer_idx][:, :end], self.val_cache[layer_idx][:, :end]
