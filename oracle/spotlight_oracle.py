"""CPU restatement of Spotlight Attention's decode-time retrieval path.

TEST INFRASTRUCTURE ONLY.  This module is the checker the HIP kernels are
compared against; nothing in the shipped package imports it.  It is imported
by the test-suite, by the smoke check and by the CPU-baseline leg of the
benchmark, and by nothing else.

Every function states the reference file:line it restates (paths relative to
the reference checkout) and how it is pinned without running the reference:

  pack_sign_u32 / pack_sign_u8   closed form + numpy.packbits(bitorder='little')
                                 + the in-line recipe of pack_dx_u8.py:62-69
  hamming_score_u32 / _u8        python int.bit_count brute force, the SWAR
                                 steps of attn_dx_u32.py:118-122, and the
                                 sign-matmul identity nbits - 2*Ham
  sign_matmul_score              torch matmul of +-1 vectors (the PyTorch path)
  num_remain                     table of known (n, mask_out) -> k
  topk_stable                    argsort on the key (-score, index) brute force
                                 + set relation to torch.topk values
  gather_kv                      fancy indexing == torch.gather
  sparse_attention               textbook softmax in fp64, equivalence with the
                                 reference's masked dense form on small n
  mlp_hash / linear_hash         textbook batched matmul + SiLU in fp64
  apply_rope                     the same rotation written with complex numbers
  reference_self_attn_forward,   tests/test_oracle_composite.py: textbook RoPE as a
  decode_step_reference_form,    complex rotation, attention as fp64 loops over the
  decode_step_cached_codes       GQA groups, selection as a brute force on packed codes
  CacheModel                     slice assignment
  LruModel                       PARITY UNPINNED by the reference (there is no
                                 LRU in it): pinned only by its own sequential
                                 brute force and the invariant that attention
                                 output is identical with and without it.

Third-party behaviour left open by the reference (torch.topk tie order) is
fixed here: among equal scores the lower token index is kept.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np

try:  # torch is only needed for the float paths and the timed CPU baseline
    import torch
except Exception:  # pragma: no cover
    torch = None


# ---------------------------------------------------------------------------
# A3  sign -> packed codes
# ---------------------------------------------------------------------------

def pack_sign_u32(x: np.ndarray) -> np.ndarray:
    """bit j of word w <=> (x[..., 32*w + j] > 0), LSB first.

    Restates packbits_kernel (spotlight/kernel/packbits.cu:7-26) and
    pack_dx_u32_kernel (spotlight/kernel/pack_dx_u32.py:6-32).  The strict
    ``> 0`` maps +0, -0 and NaN to bit 0.
    """
    x = np.asarray(x)
    assert x.shape[-1] % 32 == 0, "last dimension must be divisible by 32"
    bits = (x.astype(np.float64) > 0).reshape(*x.shape[:-1], x.shape[-1] // 32, 32)
    weights = (np.uint64(1) << np.arange(32, dtype=np.uint64))
    return (bits.astype(np.uint64) * weights).sum(-1).astype(np.uint32)


def pack_sign_u8(x: np.ndarray) -> np.ndarray:
    """bit j of byte w <=> (x[..., 8*w + j] > 0).

    Restates pack_dx_u8_kernel (spotlight/kernel/pack_dx_u8.py:6-31); built
    the way that file's own self check builds its expected answer
    (pack_dx_u8.py:62-69): sum_i (x_bool[..., i] << i).
    """
    x = np.asarray(x)
    assert x.shape[-1] % 8 == 0
    xb = (x.astype(np.float64) > 0).reshape(*x.shape[:-1], x.shape[-1] // 8, 8)
    ref = np.zeros(xb.shape[:-1], dtype=np.uint8)
    for i in range(8):
        ref += (xb[..., i].astype(np.uint8) << np.uint8(i)).astype(np.uint8)
    return ref


# ---------------------------------------------------------------------------
# A4  Hamming scorer
# ---------------------------------------------------------------------------

def swar_popcount32(v: np.ndarray) -> np.ndarray:
    """The five SWAR steps of attn_dx_u32.py:118-122 on uint32 arrays."""
    v = v.astype(np.uint32)
    v = (v & np.uint32(0x55555555)) + ((v >> np.uint32(1)) & np.uint32(0x55555555))
    v = (v & np.uint32(0x33333333)) + ((v >> np.uint32(2)) & np.uint32(0x33333333))
    v = (v & np.uint32(0x0F0F0F0F)) + ((v >> np.uint32(4)) & np.uint32(0x0F0F0F0F))
    v = (v & np.uint32(0x00FF00FF)) + ((v >> np.uint32(8)) & np.uint32(0x00FF00FF))
    v = (v & np.uint32(0x0000FFFF)) + ((v >> np.uint32(16)) & np.uint32(0x0000FFFF))
    return v


def _popcount32(v: np.ndarray) -> np.ndarray:
    """Table-driven popcount, independent of the SWAR restatement above."""
    table = np.array([bin(i).count("1") for i in range(256)], dtype=np.uint16)
    b = v.astype(np.uint32).view(np.uint8).reshape(*v.shape, 4)
    return table[b].sum(-1).astype(np.int32)


def q_heads_of_kv_head(h: int, G: int, KH: int, head_map: str) -> List[int]:
    """Query heads scored against kv head ``h``.

    'interleaved' is the reference kernels' mapping, q head g*KH + h
    (attn_k4_q28.cu:38,75; attn_dx_u32.py:112).  'blocked' is repeat_kv's
    mapping, q head h*G + g (spotlight_generation.py:128).
    """
    if head_map == "interleaved":
        return [g * KH + h for g in range(G)]
    if head_map == "blocked":
        return [h * G + g for g in range(G)]
    raise ValueError(head_map)


def hamming_score_u32(q_code: np.ndarray, k_code: np.ndarray,
                      head_map: str = "interleaved") -> np.ndarray:
    """score[b, n, h] = sum_g sum_w popc(~(q[b,0,head(g,h),w] ^ k[b,n,h,w])).

    Number of MATCHING bits summed over the G query heads of kv head h.
    Restates attn_k4_q28_kernel (spotlight/kernel/attn_k4_q28.cu:14-96) and
    dx_u32_kernel (spotlight/kernel/attn_dx_u32.py:68-128).
    q_code [B,1,QH,W] uint32, k_code [B,n,KH,W] uint32 -> int16 [B,n,KH].
    """
    q_code = np.asarray(q_code, dtype=np.uint32)
    k_code = np.asarray(k_code, dtype=np.uint32)
    B, one, QH, W = q_code.shape
    Bk, n, KH, Wk = k_code.shape
    assert one == 1 and B == Bk and W == Wk and QH % KH == 0
    G = QH // KH
    out = np.zeros((B, n, KH), dtype=np.int32)
    for h in range(KH):
        for qh in q_heads_of_kv_head(h, G, KH, head_map):
            x = ~(q_code[:, 0, qh, :][:, None, :] ^ k_code[:, :, h, :])
            out[:, :, h] += _popcount32(x).sum(-1)
    return out.astype(np.int16)


def hamming_score_u8(q_code: np.ndarray, k_code: np.ndarray) -> np.ndarray:
    """Per-head (no group sum) matching-bit count on uint8 codes.

    Restates dx_u8_kernel (spotlight/kernel/attn_dx_u8.py:9-43):
    q [B,H,1,D] u8, k [B,H,n,D] u8 (head-major) -> uint8 [B,H,n].
    The uint8 accumulator wraps modulo 256 exactly as the reference's does.
    """
    q_code = np.asarray(q_code, dtype=np.uint8)
    k_code = np.asarray(k_code, dtype=np.uint8)
    B, H, one, D = q_code.shape
    assert one == 1 and k_code.shape[:2] == (B, H) and k_code.shape[3] == D
    x = ~(q_code ^ k_code)  # broadcast over n
    table = np.array([bin(i).count("1") for i in range(256)], dtype=np.uint32)
    return (table[x].sum(-1) & 0xFF).astype(np.uint8)


def sign_matmul_score(q_inner, k_inner):
    """sim = sign(q) @ sign(k)^T  (spotlight_generation.py:19-22).

    q_inner [B,H,1,nbits], k_inner [B,H,n,nbits] floats -> [B,H,1,n].
    Equals nbits - 2*Hamming whenever no pre-activation is exactly 0.
    """
    return torch.sign(q_inner) @ torch.sign(k_inner).transpose(-1, -2)


# ---------------------------------------------------------------------------
# A5  budget
# ---------------------------------------------------------------------------

def num_remain(n: int, mask_out: float, min_remain: int = 20) -> int:
    """k = max(min(n, min_remain), n - int(n * mask_out)).

    Restates spotlight_generation.py:162-164.
    """
    k = n - int(n * mask_out)
    return max(min(n, min_remain), k)


# ---------------------------------------------------------------------------
# A6  top-k with the lowest-index tie rule
# ---------------------------------------------------------------------------

def topk_stable(score: np.ndarray, k: int) -> np.ndarray:
    """Indices of the k largest scores per (b, h), ties -> lower token index.

    Restates ``attn.topk(k=budget, dim=1, sorted=False).indices``
    (spotlight/modifiers/gpu_cache.py:50) with the tie order the reference
    leaves to torch fixed to "lowest index wins".  score [B,n,KH] integer ->
    int32 [B,KH,k], each row in ASCENDING token order (the order is not
    observable downstream: gather + softmax attention are permutation
    invariant, spotlight_generation.py:200-205).
    """
    score = np.asarray(score)
    B, n, KH = score.shape
    k = min(k, n)
    out = np.empty((B, KH, k), dtype=np.int32)
    for b in range(B):
        for h in range(KH):
            s = score[b, :, h].astype(np.int64)
            order = np.argsort(-s, kind="stable")  # stable => equal scores keep index order
            out[b, h] = np.sort(order[:k])
    return out


def topk_bruteforce(score_1d: Sequence[int], k: int) -> List[int]:
    """Pure-python selection on the key (-score, index); tiny inputs only."""
    keyed = sorted(range(len(score_1d)), key=lambda i: (-int(score_1d[i]), i))
    return sorted(keyed[:k])


# ---------------------------------------------------------------------------
# A7  gather
# ---------------------------------------------------------------------------

def gather_kv(keys: np.ndarray, vals: np.ndarray, idx: np.ndarray):
    """K_sel[b,i,h,:] = K[b, idx[b,h,i], h, :]  (gpu_cache.py:48-54).

    keys/vals [B,L,KH,d]; idx [B,KH,k] -> two arrays [B,k,KH,d].
    """
    B, KH, k = idx.shape
    b = np.arange(B)[:, None, None]
    h = np.arange(KH)[None, :, None]
    ks = keys[b, idx, h]  # [B,KH,k,d]
    vs = vals[b, idx, h]
    return ks.transpose(0, 2, 1, 3), vs.transpose(0, 2, 1, 3)


# ---------------------------------------------------------------------------
# A9  attention over the selected rows
# ---------------------------------------------------------------------------

def sparse_attention(q: np.ndarray, keys: np.ndarray, vals: np.ndarray,
                     idx: np.ndarray, scale: Optional[float] = None) -> np.ndarray:
    """out[b,qh] = softmax_i(q[b,qh] . K[b,idx_i,kv(qh)] * scale) @ V[...], fp64.

    kv(qh) = qh // G as in repeat_kv (spotlight_generation.py:128).  The
    reference reaches the same value by an additive finfo.min mask and dense
    SDPA with the default 1/sqrt(d) scale (spotlight_generation.py:200-205,
    modify_llama.py:151-186); exp(finfo.min - max) underflows to 0.
    q [B,QH,d]; keys/vals [B,L,KH,d]; idx [B,KH,k] (negative = unused slot)
    -> float64 [B,QH,d].
    """
    q = np.asarray(q, dtype=np.float64)
    B, QH, d = q.shape
    KH = keys.shape[2]
    G = QH // KH
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = np.zeros((B, QH, d), dtype=np.float64)
    for b in range(B):
        for h in range(KH):
            sel = idx[b, h]
            sel = sel[sel >= 0]
            K = np.asarray(keys[b, sel, h], dtype=np.float64)
            V = np.asarray(vals[b, sel, h], dtype=np.float64)
            for g in range(G):
                qh = h * G + g
                s = K @ q[b, qh] * scale
                s -= s.max()
                p = np.exp(s)
                out[b, qh] = (p / p.sum()) @ V
    return out


def masked_dense_attention(q, keys, vals, idx):
    """The reference's literal form, in torch on CPU.

    mask = full(finfo.min); mask.scatter_(idx, 0); SDPA(q, K, V, attn_mask)
    (spotlight_generation.py:200-205, modify_llama.py:172-180; the causal
    base mask is all zero for a single query row, modify_llama.py:132-143).
    q [B,QH,d]; keys/vals [B,L,KH,d]; idx [B,KH,k] -> [B,QH,d] in q's dtype.
    """
    B, QH, d = q.shape
    L, KH = keys.shape[1], keys.shape[2]
    G = QH // KH
    K = keys.permute(0, 2, 1, 3).repeat_interleave(G, dim=1)  # repeat_kv
    V = vals.permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    mask = torch.full((B, QH, 1, L), torch.finfo(q.dtype).min, dtype=q.dtype)
    index = torch.as_tensor(idx, dtype=torch.int64).repeat_interleave(G, dim=1).unsqueeze(2)
    mask.scatter_(-1, index, 0)
    o = torch.nn.functional.scaled_dot_product_attention(
        q.unsqueeze(2), K, V, attn_mask=mask, is_causal=False)
    return o.squeeze(2)


# ---------------------------------------------------------------------------
# A1 / A2  hashing functions
# ---------------------------------------------------------------------------

def _silu(x):
    return x / (1.0 + np.exp(-x))


def mlp_hash(x: np.ndarray, weights: Sequence[Tuple[np.ndarray, np.ndarray]],
             residue: bool) -> np.ndarray:
    """Per-head MLP pre-activations in fp64.

    layer i: dx = act(x @ proj_i + bias_i), act = SiLU except for the last
    layer; x = dx + x iff residue (spotlight_generation.py:229-255).
    x [B,H,d_in]; proj_i [H,in,out]; bias_i [H,out] -> [B,H,out_last].
    """
    x = np.asarray(x, dtype=np.float64)
    L = len(weights)
    for i, (proj, bias) in enumerate(weights):
        dx = np.einsum("bhi,hio->bho", x, np.asarray(proj, dtype=np.float64))
        dx = dx + np.asarray(bias, dtype=np.float64)[None]
        if i < L - 1:
            dx = _silu(dx)
        x = dx + x if residue else dx
    return x


def linear_hash(x: np.ndarray, proj: np.ndarray) -> np.ndarray:
    """x @ L per head (linearhashing_generation.py:224-231), fp64."""
    return np.einsum("bhi,hio->bho", np.asarray(x, np.float64), np.asarray(proj, np.float64))


def mlp_hash_torch(x, weights, residue):
    """The same MLP evaluated the way the reference does: torch ops in the
    tensors' own dtype, so bf16 rounds after every matmul / add / SiLU
    (spotlight_generation.py:238-240).  x [B,H,1,in]; proj [1,H,in,out];
    bias [1,H,1,out]."""
    L = len(weights)
    for i, (proj, bias) in enumerate(weights):
        dx = x @ proj + bias
        if i < L - 1:
            dx = torch.nn.functional.silu(dx)
        x = dx + x if residue else dx
    return x


# ---------------------------------------------------------------------------
# A8  append-only cache  /  A8'  LRU resident table
# ---------------------------------------------------------------------------

class CacheModel:
    """Slice-assign append (gpu_cache.py:38-45,108-118): rows [len, len+t)."""

    def __init__(self, B, cap, KH, d, dtype):
        self.buf = np.zeros((B, cap, KH, d), dtype=dtype)
        self.length = 0

    def update(self, rows):
        t = rows.shape[1]
        self.buf[:, self.length:self.length + t] = rows
        self.length += t
        return self.buf[:, :self.length]


class LruModel:
    """Resident table of C slots for ONE (batch, kv head).  Not in the reference.

    State per slot: token id (-1 empty) and stamp (0 = never used).
    step(t, selected, new_token):
      wanted = selected U {new_token};
      a wanted token already resident is a hit, its stamp becomes t;
      the others are misses.  The M victims are the M slots, among those not
      hit, that come first in the order (stamp ascending, slot ascending);
      empty slots carry stamp 0 so they go first.  Misses in ascending token
      order are paired with victims in ascending SLOT order; the victim's old
      token is dropped and its stamp becomes t.
    Requires len(wanted) <= C.  Returns the slot of every selected token.
    """

    def __init__(self, C: int):
        self.token = [-1] * C
        self.stamp = [0] * C
        self.hits = 0
        self.misses = 0

    def step(self, t: int, selected: Sequence[int], new_token: int) -> List[int]:
        C = len(self.token)
        wanted = sorted(set(int(s) for s in selected) | {int(new_token)})
        assert len(wanted) <= C
        where = {tok: s for s, tok in enumerate(self.token) if tok >= 0}
        hit_slots = set()
        miss = []
        for tok in wanted:
            if tok in where:
                hit_slots.add(where[tok])
            else:
                miss.append(tok)
        cand = sorted((s for s in range(C) if s not in hit_slots),
                      key=lambda s: (self.stamp[s], s))
        victims = sorted(cand[:len(miss)])
        for s in hit_slots:
            self.stamp[s] = t
        for tok, s in zip(miss, victims):
            self.token[s] = tok
            self.stamp[s] = t
        self.hits += len(hit_slots)
        self.misses += len(miss)
        where = {tok: s for s, tok in enumerate(self.token) if tok >= 0}
        return [where[int(s)] for s in selected]


class LruSequentialModel:
    """Textbook one-at-a-time LRU used to pin LruModel's RESIDENT SET.

    Processes the wanted tokens one by one; a miss evicts the slot with the
    smallest stamp among slots not wanted this step (ties -> lowest slot).
    Which slot a miss lands in may differ from LruModel; the set of resident
    tokens and every stamp value must not.
    """

    def __init__(self, C: int):
        self.token = [-1] * C
        self.stamp = [0] * C

    def step(self, t, selected, new_token):
        C = len(self.token)
        wanted = sorted(set(int(s) for s in selected) | {int(new_token)})
        protected = set()
        for tok in wanted:          # hits first so they are never evicted
            if tok in self.token:
                s = self.token.index(tok)
                self.stamp[s] = t
                protected.add(s)
        for tok in wanted:
            if tok in self.token:
                continue
            s = min((x for x in range(C) if x not in protected),
                    key=lambda x: (self.stamp[x], x))
            self.token[s] = tok
            self.stamp[s] = t
            protected.add(s)


# ---------------------------------------------------------------------------
# Composite decode step (the CPU baseline that is timed beside the GPU)
# ---------------------------------------------------------------------------

def decode_step_cached_codes(q, k_codes, K, V, n, k, q_weights, residue, head_map="blocked"):
    """One decode step over precomputed key codes, torch on CPU.

    hash q (mlp_hash_torch) -> sign -> pack -> XOR/popcount against the n
    stored codes -> stable top-k -> gather -> softmax attention over k rows:
    the composition of spotlight/kernel + gpu_cache.py described by their
    layouts (attn_k4_q28.cu:118, gpu_cache.py:50-53).
    q [B,QH,d] torch; k_codes [B,cap,KH,W] uint32 numpy; K,V [B,cap,KH,d] torch.
    Returns (out [B,QH,d] float32 torch, idx [B,KH,k] int32 numpy).
    """
    B, QH, d = q.shape
    pre = mlp_hash_torch(q.unsqueeze(2), q_weights, residue).squeeze(2)  # [B,QH,nbits]
    q_code = pack_sign_u32(pre.float().numpy())[:, None]
    score = hamming_score_u32(q_code, k_codes[:, :n], head_map)
    idx = topk_stable(score, k)
    out = sparse_attention(q.float().numpy(), K[:, :n].float().numpy(),
                           V[:, :n].float().numpy(), idx)
    return torch.from_numpy(out).float(), idx


def decode_step_reference_form(q, keys_rep, vals_rep, hash_weights, residue, mask_out, min_remain=20):
    """The reference's literal decode branch (spotlight_generation.py:149-215)
    on post-RoPE inputs, torch on CPU: hash the query AND every cached key,
    sign, +-1 matmul, per-query-head topk, finfo.min mask, dense SDPA.
    q [1,QH,1,d]; keys_rep/vals_rep [1,QH,n,d] (repeat_kv'd).  Returns
    (attn [1,QH,1,d], indices [1,QH,1,k])."""
    sim = sign_matmul_score(mlp_hash_torch(q, hash_weights, residue),
                            mlp_hash_torch(keys_rep, hash_weights, residue))
    n = sim.shape[-1]
    k = num_remain(n, mask_out, min_remain)
    idx = sim.topk(k=k, dim=-1).indices
    mask = torch.full((1, q.shape[1], 1, n), torch.finfo(sim.dtype).min, dtype=sim.dtype)
    mask.scatter_(-1, idx, 0)
    out = torch.nn.functional.scaled_dot_product_attention(
        q, keys_rep, vals_rep, attn_mask=mask, is_causal=False)
    return out, idx


# ---------------------------------------------------------------------------
# The reference's patched attention forward, restated (torch, CPU)
# ---------------------------------------------------------------------------

def _rotate_half(x):
    d = x.shape[-1]
    return torch.cat((-x[..., d // 2:], x[..., : d // 2]), dim=-1)


def apply_rope(x, pos, theta=10000.0):
    """Rotary embedding of x [B,H,d] at absolute positions pos [B], in x's dtype.

    Restates apply_rotary_pos_emb (spotlight/modifiers/modify_llama.py:54-59) with the
    cos / sin table of transformers' rotary_emb (inv_freq = theta^(-2i/d), angles in
    fp32, table cast to x's dtype): x * cos + rotate_half(x) * sin."""
    d = x.shape[-1]
    inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = torch.as_tensor(pos).to(torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    cos, sin = emb.cos().to(x.dtype)[:, None, :], emb.sin().to(x.dtype)[:, None, :]
    return x * cos + _rotate_half(x) * sin


def reference_self_attn_forward(hidden_states, kv_cache, q_w, k_w, v_w, o_w, num_heads, num_kv_heads, hash_weights,
                                residue, draft_enable, mask_out, min_remain, rope_theta=10000.0):
    """spotlight_generation.py:109-226 step by step, for B == 1, on CPU.

    q_w/k_w/v_w/o_w are the Linear weights ([out, in], no bias); hash_weights the
    per-query-head [(proj [1,QH,in,out], bias [1,QH,1,out]), ...].  The cache holds
    PRE-RoPE, repeat_kv'd keys and values; every call re-rotates the whole cache
    (:139-141, modify_llama.py:68-80,103-113) and, when drafting, re-hashes it
    (:14-17).  Returns (attn_output [1,t,hidden], kv_cache, indices or None)."""
    B, t, hidden = hidden_states.shape
    assert B == 1
    d = hidden // num_heads
    G = num_heads // num_kv_heads
    is_prefill = t > 1 and kv_cache is None
    ques = (hidden_states @ q_w.T).unflatten(-1, (num_heads, d)).transpose(1, 2)
    keys = (hidden_states @ k_w.T).unflatten(-1, (num_kv_heads, d)).transpose(1, 2)
    vals = (hidden_states @ v_w.T).unflatten(-1, (num_kv_heads, d)).transpose(1, 2)
    keys = keys.repeat_interleave(G, dim=1)   # repeat_kv
    vals = vals.repeat_interleave(G, dim=1)
    if kv_cache is not None:
        keys = torch.cat([kv_cache[0], keys], dim=-2)
        vals = torch.cat([kv_cache[1], vals], dim=-2)
    kv_cache = (keys, vals)
    n = keys.shape[-2]
    inv_freq = 1.0 / (rope_theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = torch.arange(n, dtype=torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    cos, sin = emb.cos().to(ques.dtype), emb.sin().to(ques.dtype)
    rope = lambda m, p: m * cos[p][None, None] + _rotate_half(m) * sin[p][None, None]
    Q = rope(ques, torch.arange(n - t, n))
    Kr = rope(keys, torch.arange(n))
    # causal base mask (modify_llama.py:132-143)
    base = torch.full((1, 1, t, n), torch.finfo(Q.dtype).min, dtype=torch.float32)
    base[0, 0, :, -t:].triu_(diagonal=1)
    base[0, 0, :, :-t].fill_(0)
    base = base.to(Q.dtype)
    idx = None
    mask = base
    if draft_enable and not is_prefill:
        sim = sign_matmul_score(mlp_hash_torch(Q, hash_weights, residue), mlp_hash_torch(Kr, hash_weights, residue))
        k = num_remain(n, mask_out, min_remain)
        idx = sim.topk(k=k, dim=-1).indices
        m = torch.full((1, num_heads, t, n), torch.finfo(sim.dtype).min, dtype=sim.dtype)
        m.scatter_(-1, idx, 0)
        mask = torch.minimum(m, base)
    out = torch.nn.functional.scaled_dot_product_attention(Q, Kr, vals, attn_mask=mask, is_causal=False)
    out = out.transpose(1, 2).flatten(2) @ o_w.T
    return out, kv_cache, idx
