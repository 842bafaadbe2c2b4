"""Patched attention forward of the generation path, on the HIP kernels.

Drop-in for the reference's ``self_attn_forward`` and the objects around it
(spotlight/modifiers/spotlight_generation.py:109-226, 229-255, 298-330): same
signature ``(self, hidden_states, kv_cache) -> (attn_output, kv_cache)``, same
module attributes read (``config``, ``q_proj`` .. ``o_proj``, ``draft_kwargs``,
``is_fix_layer``, ``hash_fn``), same hash-function parameter shapes, so a
checkpoint written by the reference's ``Modifier.save_checkpoint``
(spotlight/modifier.py:74-76) loads parameter for parameter.

What differs is what happens to the cache, which callers treat as opaque
(``model_model_forward`` only threads it through, :66-75):

* keys are rotated ONCE, when they are appended, and stored post-RoPE with
  their packed 128-bit code (for a decoded token the HIP step does the rotation
  itself, inside its hash launch); the reference stores pre-RoPE keys and
  re-rotates and re-hashes the whole cache every step (:139-141, :14-17);
* K/V stay at kv-head granularity ``[B, n_cap, KH, d]``; the reference stores
  them ``repeat_kv``-expanded (:128-136);
* the decode branch (:143-215) runs as the fused HIP step instead of
  sign-matmul + topk + mask + dense SDPA;
* any batch size runs (the reference asserts B == 1, :138).

Two ways to hash keys under GQA:
  ``hash_fn_k`` present  -> one code per (token, kv head), scores summed over
                            the G query heads of the group (the kernel path the
                            reference's scorers are written for,
                            spotlight/kernel/attn_dx_u32.py:68-128);
  otherwise              -> ``per_qhead``: the cache is kept per query head
                            (K/V repeated as the reference does) and every
                            query head selects its own tokens with ``hash_fn``,
                            which is exactly the reference's PyTorch path.
"""
from __future__ import annotations

import json
import math
import time
import types
from typing import Optional

import torch

from .. import kernel as K
from ..decode import HashWeights, LayerDecodeState, any_peer_wait_failed
from ..modifier import Modifier


class MLPLayer(torch.nn.Module):
    """proj [1,H,in,out] ~ N(0,1)*0.001, bias [1,H,1,out] = 0 (spotlight_generation.py:229-240)."""

    def __init__(self, info, num_heads, in_features, out_features, silu=False, residue=True):
        super().__init__()
        self.proj = torch.nn.Parameter(torch.randn((1, num_heads, in_features, out_features), **info) * 0.001)
        self.bias = torch.nn.Parameter(torch.zeros((1, num_heads, 1, out_features), **info))
        self.silu = torch.nn.SiLU() if silu else torch.nn.Identity()
        self.resi = residue

    def forward(self, x):
        dx = self.silu(x @ self.proj + self.bias)
        return dx + x if self.resi else dx


class MLPHashingFunction(torch.nn.Module):
    """spotlight_generation.py:243-255."""

    def __init__(self, info, num_heads, num_mlp_layers, mlp_dims, mlp_residue):
        super().__init__()
        self.mlp = torch.nn.ModuleList(
            MLPLayer(info, num_heads, mlp_dims[i], mlp_dims[i + 1], i < num_mlp_layers - 1, mlp_residue)
            for i in range(num_mlp_layers))

    def forward(self, x):
        for module in self.mlp:
            x = module(x)
        return x

    def hash_weights(self) -> HashWeights:
        """The same parameters in the layout the kernels read ([H,in,out], [H,out])."""
        layers = list(self.mlp)
        if len(layers) not in (1, 2):
            raise NotImplementedError("the fused hash kernel covers one or two layers")
        w = [l.proj.data[0].contiguous() for l in layers]
        b = [l.bias.data[0, :, 0].contiguous() for l in layers]
        if len(layers) == 1:
            return HashWeights(w[0], b[0], None, None, layers[0].resi)
        return HashWeights(w[0], b[0], w[1], b[1], layers[0].resi)


class LinearHashingFunction(torch.nn.Module):
    """Gaussian projection x @ L (linearhashing_generation.py:224-231); the reference
    hard-codes 32 heads of 128, here the head count is an argument."""

    def __init__(self, info, num_heads=32, dim=128):
        super().__init__()
        self.linear = torch.nn.Parameter(torch.randn((1, num_heads, dim, dim), **info))

    def forward(self, x):
        return x @ self.linear

    def hash_weights(self) -> HashWeights:
        return HashWeights(self.linear.data[0].contiguous())


def num_remain(n: int, mask_out: float, min_remain: int) -> int:
    """spotlight_generation.py:162-164."""
    return max(min(n, min_remain), n - int(n * mask_out))


def rope_tables(positions: torch.Tensor, dim: int, theta: float, dtype) -> tuple:
    """cos / sin [len, dim] for absolute positions, the rotate_half convention
    (spotlight/modifiers/modify_llama.py:54-59 with transformers' rotary_emb)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2, device=positions.device, dtype=torch.float32) / dim))
    ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [B,t,H,d]; cos/sin [t,d]."""
    d = x.shape[-1]
    rot = torch.cat((-x[..., d // 2:], x[..., : d // 2]), dim=-1)
    return x * cos[None, :, None, :] + rot * sin[None, :, None, :]


class SpotlightKV:
    """The per-layer cache handle threaded through the model in place of the
    reference's ``(keys, vals)`` tuple.

    A sparse layer's rows live in its ``LayerDecodeState``.  A dense layer keeps a plain K/V store,
    head-major ``[B, KH, n_cap, d]`` (``keys`` / ``vals`` are ``[B, n_cap, KH, d]`` views of it), and
    a device-side copy of its length, ``pos``: in *graph mode* (``Spotlight.generate`` replaying one
    captured decode token) the forward takes every position from the device and never touches
    ``length``, which the replay loop advances on the host."""

    def __init__(self, B, QH, KH, d, n_cap, dtype, device, sparse_state: Optional[LayerDecodeState]):
        self.B, self.QH, self.KH, self.d, self.n_cap = B, QH, KH, d, n_cap
        self.state = sparse_state
        self.graph_mode = False
        if sparse_state is None:   # dense layer: plain K/V store
            self._k = torch.zeros((B, KH, n_cap, d), dtype=dtype, device=device)
            self._v = torch.zeros((B, KH, n_cap, d), dtype=dtype, device=device)
            self.keys, self.vals = self._k.permute(0, 2, 1, 3), self._v.permute(0, 2, 1, 3)
            self.pos = torch.zeros((1,), dtype=torch.int64, device=device)
            self.col = torch.arange(n_cap, device=device)
        else:
            self.keys, self.vals = sparse_state.keys, sparse_state.vals
        self.length = 0

    def append_dense(self, k, v):
        t = k.shape[1]
        if self.length + t > self.n_cap:
            raise RuntimeError(f"cache capacity {self.n_cap} exceeded")
        self._k[:, :, self.length:self.length + t] = k.permute(0, 2, 1, 3)
        self._v[:, :, self.length:self.length + t] = v.permute(0, 2, 1, 3)
        self.length += t

    def enter_graph_mode(self):
        if self.state is None:
            self.pos.fill_(self.length)
        self.graph_mode = True

    def leave_graph_mode(self):
        self.graph_mode = False

    def advance(self, tokens: int):
        """Host-side bookkeeping after ``tokens`` replays of the captured decode token (negative: rows
        taken back; on the device too, where later steps simply overwrite them)."""
        self.length += tokens
        if self.state is not None:
            self.state.host_len += tokens
            if tokens < 0:
                self.state.seq_lens.add_(tokens)
        elif tokens < 0:
            self.pos.add_(tokens)

    def dense_decode_on_device(self, q, k, v):
        """One new token of a dense layer with every position read from the device: q [B,1,QH,d],
        k / v [B,1,KH,d], q and k already rotated at ``pos``.  The row goes into the store at ``pos``,
        the attention runs over the whole capacity with the rows beyond ``pos`` masked, as two batched
        matrix products per kv-head group (no K/V expansion), and ``pos`` advances."""
        B, QH, KH, d = self.B, self.QH, self.KH, self.d
        self._k.index_copy_(2, self.pos, k.permute(0, 2, 1, 3))
        self._v.index_copy_(2, self.pos, v.permute(0, 2, 1, 3))
        sc = torch.matmul(q.reshape(B, KH, QH // KH, d), self._k.transpose(2, 3)).float() * (d ** -0.5)
        sc = sc.masked_fill((self.col > self.pos)[None, None, None, :], float("-inf"))
        o = torch.matmul(torch.softmax(sc, dim=-1).to(q.dtype), self._v)
        self.pos.add_(1)
        return o.reshape(B, 1, QH, d)


def _dense_attention(q, keys, vals):
    """q [B,t,QH,d] = the LAST t positions of keys/vals [B,n,KH,d] -> [B,t,QH,d]; torch SDPA
    with grouped heads.  Row i of the chunk sees the n - t earlier rows and rows 0..i of the
    chunk (the mask of modify_llama.py:132-143)."""
    B, t, QH, d = q.shape
    n, KH = keys.shape[1], keys.shape[2]
    G = QH // KH
    kk = keys.permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    vv = vals.permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    qq = q.permute(0, 2, 1, 3)
    if t == 1:
        o = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv)
    elif t == n:
        o = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, is_causal=True)
    else:   # a chunk behind a non-empty cache: is_causal would align the triangle top-left
        col = torch.arange(n, device=q.device)[None, :]
        row = torch.arange(n - t, n, device=q.device)[:, None]
        o = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, attn_mask=col <= row)
    return o.permute(0, 2, 1, 3)


def self_attn_forward(self, hidden_states: torch.Tensor, kv_cache=None):
    """Same contract as spotlight_generation.py:109-226."""
    cfg = self.config
    QH, hidden = cfg.num_attention_heads, cfg.hidden_size
    KH = cfg.num_key_value_heads
    d = hidden // QH
    B, t, _ = hidden_states.shape
    dtype, dev = hidden_states.dtype, hidden_states.device
    dk = self.draft_kwargs
    sparse = dk.get("enable", True) is True and not self.is_fix_layer
    per_qhead = getattr(self, "hash_fn_k", None) is None and KH != QH
    G = QH // KH

    ques = self.q_proj(hidden_states).unflatten(-1, (QH, d))
    keys = self.k_proj(hidden_states).unflatten(-1, (KH, d))
    vals = self.v_proj(hidden_states).unflatten(-1, (KH, d))

    start = 0 if kv_cache is None else kv_cache.length
    theta = float(getattr(cfg, "rope_theta", 10000.0))
    graph_mode = kv_cache is not None and kv_cache.graph_mode
    if graph_mode and t != 1:
        raise RuntimeError("graph mode covers one new token per call")
    # one new token of a sparse layer: the HIP step rotates q and the new key itself (at the
    # position it reads from the device-side length), so they are handed over un-rotated
    fused_rope = sparse and t == 1 and kv_cache is not None and kv_cache.length > 0
    if not fused_rope:
        pos = kv_cache.pos if graph_mode else torch.arange(start, start + t, device=dev)
        cos, sin = rope_tables(pos, d, theta, dtype)
        ques = apply_rope(ques, cos, sin)
        keys = apply_rope(keys, cos, sin)     # rotated once, here; stored post-RoPE
    if sparse and per_qhead:              # the reference's repeat_kv (:128-129)
        keys = keys.repeat_interleave(G, dim=2)
        vals = vals.repeat_interleave(G, dim=2)
    KHc = keys.shape[2]

    if kv_cache is None:
        n_cap = int(dk.get("max_cache_len", 0)) or (t + 1024)
        n_cap = (max(n_cap, t + 1) + 7) // 8 * 8
        state = None
        if sparse:
            hq = self.hash_fn.hash_weights()
            hk = hq if per_qhead or KH == QH else self.hash_fn_k.hash_weights()
            k_cap = num_remain(n_cap, dk["mask_out"], dk["min_remain"])
            state = LayerDecodeState(B, QH, KHc, d, n_cap, k_cap, hq, hk,
                                     dtype=dtype, device=dev, head_map="blocked", rope_theta=theta,
                                     exclusive_device=bool(dk.get("exclusive_device", True)))
            # the budget (:162-164) is evaluated on the device from the length each step reads:
            # nothing on the host changes when it grows, k_cap is only the row length of the index list
            state.set_budget(float(dk["mask_out"]), int(dk["min_remain"]))
        kv_cache = SpotlightKV(B, QH, KHc, d, n_cap, dtype, dev, state)

    if t > 1 or not sparse or kv_cache.length == 0:
        # prefill (the draft is not used there, :145) and dense layers
        if graph_mode:
            out = kv_cache.dense_decode_on_device(ques, keys, vals)
        else:
            if kv_cache.state is not None:
                # rows, values and their codes go behind what is cached (chunked prefill included)
                if kv_cache.length + t >= kv_cache.n_cap:
                    raise RuntimeError(f"cache capacity {kv_cache.n_cap} exceeded")
                kv_cache.state.load_rows(keys.contiguous(), vals.contiguous(), start=kv_cache.length)
                kv_cache.state.set_length(kv_cache.length + t)
                kv_cache.length += t
            else:
                kv_cache.append_dense(keys, vals)
            n = kv_cache.length
            out = _dense_attention(ques, kv_cache.keys[:, :n], kv_cache.vals[:, :n])
    elif graph_mode:
        # the captured decode token: inputs into the step's own buffers, grid sized for the capacity,
        # lengths and budget read from the device
        st = kv_cache.state
        st.q_in.copy_(ques[:, 0])
        st.k_in.copy_(keys[:, 0])
        st.v_in.copy_(vals[:, 0])
        st._launch(st.n_cap)
        out = st.out.unsqueeze(1)
    else:
        st = kv_cache.state
        n = kv_cache.length + 1
        out = st.step(ques[:, 0].contiguous(), keys[:, 0].contiguous(), vals[:, 0].contiguous()).unsqueeze(1)
        kv_cache.length = n
        if dk.get("bench_mark", False):
            # benchmark mode (spotlight_evaluation.py:303-316): IoU of the selected rows
            # against the true top-k of q.k, per query head, averaged over the batch
            from ..iou import selection_iou
            k = num_remain(n, dk["mask_out"], dk["min_remain"])
            self.ratios = selection_iou(st.selected()[..., :k], st.q_rot, kv_cache.keys[:, :n], k).mean(dim=0).tolist()

    attn_output = self.o_proj(out.reshape(B, t, hidden))
    return attn_output, kv_cache


def patch_attention(attn_module: torch.nn.Module, layer_idx: int, draft_kwargs: dict,
                    gqa_key_hash: bool = False) -> None:
    """What Decoder.__init__ does to every layer's attention (spotlight_generation.py:317-329):
    install draft_kwargs / is_fix_layer / hash_fn and bind the forward.  With
    ``gqa_key_hash`` a second, per-kv-head hash function ``hash_fn_k`` is created."""
    cfg = attn_module.config
    info = {"device": attn_module.q_proj.weight.data.device, "dtype": attn_module.q_proj.weight.data.dtype}
    mlp_dims = draft_kwargs.get("mlp_dims", "[128,128,128]")
    mlp_dims = json.loads(mlp_dims) if isinstance(mlp_dims, str) else list(mlp_dims)
    n_layers = draft_kwargs.get("num_mlp_layers", 2)
    residue = draft_kwargs.get("mlp_residue", True)
    attn_module.is_fix_layer = layer_idx in draft_kwargs.get("fix_layers", [])
    attn_module.draft_kwargs = draft_kwargs
    attn_module.hash_fn = MLPHashingFunction(info, cfg.num_attention_heads, n_layers, mlp_dims, residue)
    if gqa_key_hash and cfg.num_key_value_heads != cfg.num_attention_heads:
        attn_module.hash_fn_k = MLPHashingFunction(info, cfg.num_key_value_heads, n_layers, mlp_dims, residue)
    attn_module.forward = types.MethodType(self_attn_forward, attn_module)


# ---- the objects above the attention forward -----------------------------------------
# Same names, call signatures and return conventions as the reference's
# (spotlight_generation.py:24-106, 258-495); the per-layer cache handle is the
# opaque object ``self_attn_forward`` returns.

class CausalOutput:
    """What ``model_forward`` returns: the three fields of transformers'
    ``CausalLMOutputWithPast`` the reference's callers read (:57-60, :478, :487)."""

    def __init__(self, loss, logits, past_key_values):
        self.loss, self.logits, self.past_key_values = loss, logits, past_key_values


def model_forward(self, input_ids, labels=None, kv_cache=None, **kwargs):
    """spotlight_generation.py:24-60: logits of the LAST position only, as fp32."""
    hidden_states, kv_cache = self.model(input_ids=input_ids, kv_cache=kv_cache)
    logits = self.lm_head(hidden_states[..., -1:, :]).float()
    loss = None
    if labels is not None:
        shift_logits = logits[..., :-1, :].reshape(-1, self.config.vocab_size)
        shift_labels = labels[..., 1:].reshape(-1).to(shift_logits.device)
        loss = torch.nn.functional.cross_entropy(shift_logits, shift_labels)
    return CausalOutput(loss, logits, kv_cache)


def model_model_forward(self, input_ids=None, kv_cache=None):
    """spotlight_generation.py:63-79."""
    hidden_states = self.embed_tokens(input_ids)
    if kv_cache is None:
        kv_cache = [None] * len(self.layers)
    for layer_idx, decoder_layer in enumerate(self.layers):
        hidden_states, kv_cache[layer_idx] = decoder_layer(hidden_states, kv_cache[layer_idx])
    return self.norm(hidden_states), kv_cache


def layer_forward(self, hidden_states, kv_cache=None):
    """spotlight_generation.py:82-106."""
    device = self.self_attn.q_proj.weight.data.device
    if hidden_states.device != device:
        hidden_states = hidden_states.to(device)
    residual = hidden_states
    hidden_states, kv_cache = self.self_attn(self.input_layernorm(hidden_states), kv_cache)
    hidden_states = residual + hidden_states
    residual = hidden_states
    hidden_states = self.mlp(self.post_attention_layernorm(hidden_states))
    return residual + hidden_states, kv_cache


class Decoder(torch.nn.Module):
    """spotlight_generation.py:258-383 without the LoRA branch (``enable_lora`` is
    False in every generation config of the reference, and ``peft`` is not a
    dependency here)."""

    hash_kind = "mlp"

    def __init__(self, decoder, draft_kwargs):
        super().__init__()
        self.decoder = decoder
        self.enable_lora = False
        self.fix_layers = list(draft_kwargs.get("fix_layers", []))
        self.draft_kwargs = draft_kwargs
        self.model.forward = types.MethodType(model_forward, self.model)
        self.model.model.forward = types.MethodType(model_model_forward, self.model.model)
        for layer_idx, layer in enumerate(self.layers):
            layer.forward = types.MethodType(layer_forward, layer)
            self._patch(layer.self_attn, layer_idx)

    def _patch(self, attn, layer_idx):
        patch_attention(attn, layer_idx, self.draft_kwargs, gqa_key_hash=bool(self.draft_kwargs.get("gqa_key_hash", False)))

    @property
    def layers(self):
        return self.decoder.model.layers

    @property
    def model(self):
        return self.decoder

    def reset(self):
        """Nothing to drop: the caches live in the handles ``forward`` returns, not on
        the modules (the reference deletes ``k_cache`` / ``v_cache`` attributes, :282-286)."""

    def is_benchmark_mode(self):
        return self.draft_kwargs["bench_mark"]

    def enable_benchmark_mode(self):
        self.draft_kwargs["bench_mark"] = True

    def disable_benchmark_mode(self):
        self.draft_kwargs["bench_mark"] = False

    def get_ratios(self, reset=False):
        """Per layer the IoU list of the last benchmark-mode decode step, None for dense
        layers (spotlight_generation.py:344-353)."""
        ratios = []
        for layer in self.layers:
            if layer.self_attn.is_fix_layer or not hasattr(layer.self_attn, "ratios"):
                ratios.append(None)
            else:
                ratios.append(layer.self_attn.ratios)
                del layer.self_attn.ratios
        return ratios

    def _hash_modules(self, layer):
        mods = [layer.self_attn.hash_fn]
        if getattr(layer.self_attn, "hash_fn_k", None) is not None:
            mods.append(layer.self_attn.hash_fn_k)
        return mods

    def layer_ft_params(self, layer=None):
        """One layer's parameters (dense layers: none, :356-360) or, without an
        argument, the per-layer lists of every layer."""
        if layer is not None:
            lay = self.layers[layer]
            return [] if lay.self_attn.is_fix_layer else [p for m in self._hash_modules(lay) for p in m.parameters()]
        return [[p for m in self._hash_modules(lay) for p in m.parameters()] for lay in self.layers]

    def ft_params(self, layer=None):
        """Every layer's hash parameters, dense layers included (:363-369)."""
        return [p for ps in self.layer_ft_params() for p in ps]

    def forward(self, input_ids, labels=None, kv_cache=None):
        return self.decoder(input_ids=input_ids, labels=labels, kv_cache=kv_cache)


class Model(torch.nn.Module):
    """spotlight_generation.py:386-437."""

    def __init__(self, decoder: Decoder):
        super().__init__()
        self.decoder = decoder

    def ft_params(self):
        return self.decoder.ft_params()

    def reset(self):
        self.decoder.reset()

    def forward(self, input_ids, kv_cache=None, labels=None, local_rank=None, **kwargs):
        if isinstance(input_ids, list):
            input_ids = torch.tensor(input_ids, dtype=torch.int64)[None, :]
            if labels is not None:
                labels = torch.tensor(labels, dtype=torch.int64)[None, :]
        if input_ids.ndim == 3:
            input_ids = input_ids.flatten(0, 1)
        if labels is not None and labels.ndim == 3:
            labels = labels.flatten(0, 1)
        device = torch.device(local_rank) if local_rank is not None else next(iter(self.decoder.parameters())).device
        return self.decoder(input_ids.to(device), labels=labels, kv_cache=kv_cache)


class Spotlight(Modifier):
    """spotlight_generation.py:440-495: ``Spotlight(model, save_ckp, load_ckp, config)``."""

    decoder_cls = Decoder

    def __init__(self, model, save_ckp, load_ckp, config):
        torch.nn.Module.__init__(self)   # attributes below are set before Modifier.__init__ loads the checkpoint
        self.get_conf(config)
        assert isinstance(self.conf, dict)
        decoder = Model(self.decoder_cls(model, draft_kwargs=self.conf["draft_kwargs"]))
        super().__init__(decoder, save_ckp, load_ckp)

    def ft_params(self):
        return self.model.ft_params()

    def layer_ft_params(self):
        return self.model.decoder.layer_ft_params()

    def fix_layers(self):
        return self.model.decoder.fix_layers

    def reset(self):
        self.model.reset()

    def is_benchmark_mode(self):
        return self.model.decoder.is_benchmark_mode()

    def enable_benchmark_mode(self):
        return self.model.decoder.enable_benchmark_mode()

    def disable_benchmark_mode(self):
        return self.model.decoder.disable_benchmark_mode()

    @torch.no_grad()
    def generate(self, input_ids, max_new_tokens=128, eos_token_id=(2,)):
        """Greedy decoding (:470-495).  Batch 1 behaves exactly like the reference
        (stops at an eos token, which is not appended); a larger batch runs every
        row for ``max_new_tokens`` steps.

        On a GPU the decode token -- every layer, the final norm, ``lm_head`` and the argmax -- is
        captured once as a HIP graph and replayed per token (``draft_kwargs["hip_graph"]``, default
        on; off in benchmark mode, which reads the selection back every step): lengths, positions
        and the budget all live on the device, so the graph stays valid while the cache grows."""
        if input_ids.ndim == 3:
            input_ids = input_ids.flatten(0, 1)
        device = next(iter(self.model.parameters())).device
        input_ids = input_ids.to(device)
        dk = self.conf["draft_kwargs"]
        # the caches are sized by the first forward: make room for the tokens to come
        need = input_ids.shape[1] + max_new_tokens + 8
        given = dk.get("max_cache_len", None)
        if int(given or 0) < need:
            dk["max_cache_len"] = need
        # draft_kwargs["record_timing"]: leave the seconds spent in prefill, in eagerly decoded tokens, in the
        # capture and in replayed tokens in ``self.timing`` (each phase bracketed by a device synchronisation)
        rec = bool(dk.get("record_timing", False)) and device.type == "cuda"
        timing = dict(prefill_s=0.0, eager_decode_s=0.0, eager_tokens=0, capture_s=0.0, graph_decode_s=0.0, graph_tokens=0, recoveries=0)

        def clock():
            if rec:
                torch.cuda.synchronize(device)
            return time.perf_counter()

        t_mark = clock()
        try:
            output = self.model(input_ids=input_ids)
        finally:
            if given is None:
                dk.pop("max_cache_len", None)
            else:
                dk["max_cache_len"] = given
        logits, kv_cache = output.logits, output.past_key_values
        new_tok = logits[:, -1:].argmax(dim=-1)
        timing["prefill_s"] = clock() - t_mark
        new_ids = []
        single = input_ids.shape[0] == 1
        use_graph = (bool(dk.get("hip_graph", True)) and device.type == "cuda" and not dk.get("bench_mark", False)
                     and max_new_tokens > 2)
        runner = None
        unchecked = 0     # tokens decoded since the bounded waits were last looked at
        states = [c.state for c in kv_cache if c is not None and c.state is not None]
        while len(new_ids) < max_new_tokens:
            if single and new_tok.ravel().item() in eos_token_id:
                break
            new_ids.append(new_tok.clone())
            if use_graph and runner is None and len(new_ids) >= 2:
                # (the first decoded token ran eagerly: lazy initialisations are behind us)
                t_mark = clock()
                runner = _GraphedToken(self.model, kv_cache, new_tok)
                timing["capture_s"] = clock() - t_mark
            t_mark = clock() if rec and (runner is None or timing["graph_tokens"] == 0) else t_mark
            if runner is not None:
                new_tok = runner.replay(new_tok)
                timing["graph_tokens"] += 1
            else:
                output = self.model(input_ids=new_tok, kv_cache=kv_cache)
                logits, kv_cache = output.logits, output.past_key_values
                new_tok = logits[:, -1:].argmax(dim=-1)
                if rec:
                    timing["eager_decode_s"] += clock() - t_mark
                timing["eager_tokens"] += 1
            unchecked += 1
            # The head-major step's workgroups wait for each other (bounded): where the host reads the
            # device anyway (batch 1: every token; otherwise every 16 tokens and at the end) the error
            # words are looked at.  After a failure the affected tokens are taken back and decoded
            # again, eagerly, on token-major codes, whose kernels never wait.
            if states and (single or unchecked >= 16 or len(new_ids) == max_new_tokens):
                if any_peer_wait_failed(states):
                    timing["recoveries"] += 1
                    if runner is not None:    # (captured again below, over token-major codes)
                        runner.close()
                        runner = None
                    for st in states:
                        if st.error_word() is not None:
                            st.error_word().zero_()
                        st.use_token_major()
                    for c in kv_cache:
                        c.advance(-unchecked)
                    del new_ids[len(new_ids) - unchecked + 1:]
                    new_tok = new_ids[-1]
                    for _ in range(unchecked - 1):
                        new_tok = self.model(input_ids=new_tok, kv_cache=kv_cache).logits[:, -1:].argmax(dim=-1)
                        new_ids.append(new_tok)
                    new_tok = self.model(input_ids=new_tok, kv_cache=kv_cache).logits[:, -1:].argmax(dim=-1)
                unchecked = 0
        if runner is not None:
            if rec:    # the replays are timed as one stretch: nothing synchronises between them but the checks above
                timing["graph_decode_s"] = clock() - t_mark
            runner.close()
        timing["decode_s"] = timing["eager_decode_s"] + timing["graph_decode_s"]
        self.timing = timing
        self.model.reset()
        if not new_ids:
            return input_ids
        return torch.cat([input_ids] + [t.to(input_ids.dtype) for t in new_ids], dim=-1)


class _GraphedToken:
    """One decode token of the whole model as a captured HIP graph: token ids in a fixed buffer, the
    caches in graph mode (positions, lengths and budgets are read from the device), the next token
    written back into the buffer by the graph itself."""

    def __init__(self, model, kv_cache, tok):
        self.kv_cache = kv_cache
        self.tok = tok.clone()
        for c in kv_cache:
            c.enter_graph_mode()
        self.graph = torch.cuda.CUDAGraph()
        try:
            with torch.cuda.graph(self.graph):
                out = model(input_ids=self.tok, kv_cache=kv_cache)
                self.tok.copy_(out.logits[:, -1:].argmax(dim=-1))
        except Exception:
            self.close()
            raise

    def replay(self, tok):
        if tok is not self.tok:
            self.tok.copy_(tok)
        self.graph.replay()
        for c in self.kv_cache:
            c.advance(1)
        return self.tok

    def close(self):
        for c in self.kv_cache:
            c.leave_graph_mode()
