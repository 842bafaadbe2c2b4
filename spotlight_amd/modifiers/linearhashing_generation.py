"""Training-free linear hashing on the HIP kernels: drop-in for
spotlight/modifiers/linearhashing_generation.py.  Only the hash function differs
from the MLP variant: ``x @ L`` with one Gaussian ``[1, heads, 128, 128]`` matrix
per layer (:224-231; the reference hard-codes 32 heads, here the model's head
count is used)."""
from __future__ import annotations

import types

from .spotlight_generation import (Decoder as _Decoder, LinearHashingFunction, Model, Spotlight as _Spotlight,
                                   self_attn_forward)


class Decoder(_Decoder):
    hash_kind = "linear"

    def _patch(self, attn, layer_idx):
        cfg = attn.config
        info = {"device": attn.q_proj.weight.data.device, "dtype": attn.q_proj.weight.data.dtype}
        attn.is_fix_layer = layer_idx in self.fix_layers
        attn.draft_kwargs = self.draft_kwargs
        attn.hash_fn = LinearHashingFunction(info, cfg.num_attention_heads, cfg.hidden_size // cfg.num_attention_heads)
        attn.forward = types.MethodType(self_attn_forward, attn)


class LinearHashing(_Spotlight):
    decoder_cls = Decoder


__all__ = ["Decoder", "LinearHashing", "LinearHashingFunction", "Model"]
