"""CPU pins of the oracle's COMPOSITE functions: the restated patched forward
(spotlight_generation.py:109-226) and the two whole-step restatements.  Each is checked
against a formulation that shares no code with it: rotary embedding as a complex rotation,
attention as explicit fp64 softmax loops over the GQA groups, selection as a brute force on
packed codes.  No GPU."""
import math

import numpy as np
import pytest
import torch

from oracle import spotlight_oracle as orc


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def _rope_complex(x, pos, theta, fp32_angles=False):
    """x [H, t, d] float64 numpy, pos [t]: pairs (i, i + d/2) rotated by pos * theta^(-2i/d).
    fp32_angles: the angle is the float32 product of float32 factors, as in transformers' table."""
    H, t, d = x.shape
    half = d // 2
    freq = theta ** (-np.arange(half, dtype=np.float64) * 2.0 / d)
    ang = np.asarray(pos, dtype=np.float64)[:, None] * freq[None, :]
    if fp32_angles:
        f32 = (1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).numpy()   # the table's definition
        ang = (np.asarray(pos, dtype=np.float32)[:, None] * f32[None, :]).astype(np.float64)
    z = x[..., :half] + 1j * x[..., half:]
    z = z * np.exp(1j * ang)[None]
    return np.concatenate([z.real, z.imag], axis=-1)


def _project(hidden, w, heads):
    """hidden [t, hidden] -> [heads, t, d] float64."""
    y = hidden.double().numpy() @ w.double().numpy().T
    t = y.shape[0]
    return y.reshape(t, heads, -1).transpose(1, 0, 2)


def _attend(Q, K, V, allowed):
    """Q [QH,t,d], K,V [KH,n,d] (one row per kv head, no expansion), allowed [QH,t,n] bool.
    kv head of q head qh is qh // G (repeat_kv).  fp64 loops."""
    QH, t, d = Q.shape
    KH = K.shape[0]
    G = QH // KH
    out = np.zeros((QH, t, d))
    for qh in range(QH):
        for i in range(t):
            sel = np.nonzero(allowed[qh, i])[0]
            s = K[qh // G, sel] @ Q[qh, i] / math.sqrt(d)
            p = np.exp(s - s.max())
            out[qh, i] = (p / p.sum()) @ V[qh // G, sel]
    return out


class _Toy:
    """A tiny attention layer with GQA and a two-layer hash per query head."""

    def __init__(self, seed, QH=4, KH=2, d=32, d_hid=64, nbits=32, theta=10000.0):
        g = _gen(seed)
        hidden = QH * d   # the reference derives head_dim as hidden_size // num_heads (:119)
        self.QH, self.KH, self.d, self.hidden, self.theta, self.nbits = QH, KH, d, hidden, theta, nbits
        r = lambda *s: torch.randn(*s, generator=g)
        self.q_w, self.k_w, self.v_w = r(QH * d, hidden) * 0.3, r(KH * d, hidden) * 0.3, r(KH * d, hidden) * 0.3
        self.o_w = r(hidden, QH * d) * 0.3
        self.hash_w = [(r(1, QH, d, d_hid) * 0.2, r(1, QH, 1, d_hid) * 0.1), (r(1, QH, d_hid, nbits) * 0.2, r(1, QH, 1, nbits) * 0.1)]
        self.g = g

    def forward_ref(self, hidden, cache, draft, mask_out=0.5, min_remain=2):
        return orc.reference_self_attn_forward(hidden, cache, self.q_w, self.k_w, self.v_w, self.o_w, self.QH, self.KH,
                                               self.hash_w, False, draft, mask_out, min_remain, rope_theta=self.theta)

    def rotated(self, hidden_all):
        """Post-RoPE Q [QH,n,d], K [KH,n,d] and V [KH,n,d] of the whole sequence, fp64."""
        n = hidden_all.shape[0]
        Q = _rope_complex(_project(hidden_all, self.q_w, self.QH), np.arange(n), self.theta)
        K = _rope_complex(_project(hidden_all, self.k_w, self.KH), np.arange(n), self.theta)
        V = _project(hidden_all, self.v_w, self.KH)
        return Q, K, V

    def out_proj(self, o):   # o [QH,t,d] -> [t, hidden]
        return o.transpose(1, 0, 2).reshape(o.shape[1], -1) @ self.o_w.double().numpy().T


def test_forward_without_draft_is_causal_attention_with_textbook_rope():
    toy = _Toy(0)
    n0, extra = 9, 3
    hid = torch.randn(1, n0 + extra + 2, toy.hidden, generator=toy.g)
    Q, K, V = toy.rotated(hid[0])
    # prefill of n0 tokens, `extra` single-token steps, then a two-token chunk on a non-empty cache
    out, cache, idx = toy.forward_ref(hid[:, :n0], None, False)
    assert idx is None
    causal = np.tril(np.ones((n0, n0), dtype=bool))[None].repeat(toy.QH, 0)
    want = toy.out_proj(_attend(Q[:, :n0], K[:, :n0], V[:, :n0], causal))
    np.testing.assert_allclose(out[0].double().numpy(), want, rtol=1e-5, atol=5e-5)
    n = n0
    for _ in range(extra):
        out, cache, idx = toy.forward_ref(hid[:, n:n + 1], cache, False)
        n += 1
        allowed = np.ones((toy.QH, 1, n), dtype=bool)
        want = toy.out_proj(_attend(Q[:, n - 1:n], K[:, :n], V[:, :n], allowed))
        np.testing.assert_allclose(out[0].double().numpy(), want, rtol=1e-5, atol=5e-5)
    out, cache, idx = toy.forward_ref(hid[:, n:n + 2], cache, False)
    allowed = np.ones((toy.QH, 2, n + 2), dtype=bool)
    allowed[:, 0, n + 1] = False   # the first row of the chunk does not see the second
    want = toy.out_proj(_attend(Q[:, n:n + 2], K[:, :n + 2], V[:, :n + 2], allowed))
    np.testing.assert_allclose(out[0].double().numpy(), want, rtol=1e-5, atol=5e-5)
    # the cache holds pre-RoPE, repeat_kv'd rows (spotlight_generation.py:128-136)
    G = toy.QH // toy.KH
    k_pre = _project(hid[0, :n + 2], toy.k_w, toy.KH)
    np.testing.assert_allclose(cache[0][0].double().numpy(), np.repeat(k_pre, G, axis=0), atol=1e-5)


@pytest.mark.parametrize("seed", [1, 3, 4, 6])   # seeds whose pre-activations all stay clear of zero (checked below)
def test_forward_with_draft_keeps_the_brute_force_top_k_and_attends_over_it(seed):
    toy = _Toy(seed)
    n0 = 40
    hid = torch.randn(1, n0 + 1, toy.hidden, generator=toy.g)
    _, cache, _ = toy.forward_ref(hid[:, :n0], None, True)   # prefill never drafts (:143-147)
    out, cache, idx = toy.forward_ref(hid[:, n0:], cache, True, mask_out=0.75, min_remain=2)
    n = n0 + 1
    k = orc.num_remain(n, 0.75, 2)
    assert idx.shape == (1, toy.QH, 1, k)
    Q, K, V = toy.rotated(hid[0])
    G = toy.QH // toy.KH
    # codes of the query and of every key, per QUERY head (keys are repeat_kv'd before hashing)
    w = [(p[0].double().numpy(), b[0, :, 0].double().numpy()) for p, b in toy.hash_w]
    q_pre = orc.mlp_hash(Q[:, n - 1][None], w, False)[0]                       # [QH,nbits]
    k_pre = np.stack([orc.mlp_hash(np.repeat(K, G, axis=0)[:, t][None], w, False)[0] for t in range(n)], 1)  # [QH,n,nbits]
    assert np.abs(q_pre).min() > 1e-4 and np.abs(k_pre).min() > 1e-4           # no sign is decided by float32 rounding
    q_code = orc.pack_sign_u32(q_pre)
    k_code = orc.pack_sign_u32(k_pre)
    allowed = np.zeros((toy.QH, 1, n), dtype=bool)
    for qh in range(toy.QH):
        match = np.array([sum(bin(int(a) ^ int(b)).count("1") for a, b in zip(q_code[qh], k_code[qh, t])) for t in range(n)])
        match = toy.nbits - match                                             # matching bits
        got = np.sort(idx[0, qh, 0].numpy())
        assert len(set(got.tolist())) == k
        # the same multiset of scores as the brute force, everything above the threshold kept
        brute = orc.topk_bruteforce(match, k)
        assert sorted(match[got].tolist()) == sorted(match[brute].tolist())
        thr = match[brute].min()
        assert set(np.nonzero(match > thr)[0].tolist()) <= set(got.tolist())
        allowed[qh, 0, got] = True
    want = toy.out_proj(_attend(Q[:, n - 1:n], K[:, :n], V[:, :n], allowed))
    np.testing.assert_allclose(out[0].double().numpy(), want, rtol=1e-5, atol=5e-5)


@pytest.mark.parametrize("seed", [0, 5])
def test_reference_form_step_and_cached_codes_step_agree_on_an_mha_toy(seed):
    """MHA, so per-query-head selection == per-kv-head selection: the literal reference step
    (re-hash every key, +-1 matmul, masked dense SDPA) and the kernel-path step (packed codes,
    XOR/popcount, stable top-k, gathered softmax) must keep the same multiset of scores, and the
    same output wherever the threshold bin is kept whole."""
    g = _gen(seed)
    H, n, d, d_hid, nbits = 3, 64, 32, 64, 32
    q = torch.randn(1, H, d, generator=g)
    K = torch.randn(1, n, H, d, generator=g)
    V = torch.randn(1, n, H, d, generator=g)
    w = [(torch.randn(1, H, d, d_hid, generator=g) * 0.2, torch.randn(1, H, 1, d_hid, generator=g) * 0.1),
         (torch.randn(1, H, d_hid, nbits, generator=g) * 0.2, torch.randn(1, H, 1, nbits, generator=g) * 0.1)]
    mask_out = 0.75
    k = orc.num_remain(n, mask_out, 2)
    keys_rep = K.permute(0, 2, 1, 3)
    vals_rep = V.permute(0, 2, 1, 3)
    out_ref, idx_ref = orc.decode_step_reference_form(q[:, :, None], keys_rep, vals_rep, w, False, mask_out, 2)
    k_pre = orc.mlp_hash_torch(keys_rep, w, False)                             # [1,H,n,nbits]
    codes = orc.pack_sign_u32(k_pre.permute(0, 2, 1, 3).numpy())               # [1,n,H,W]
    out_cc, idx_cc = orc.decode_step_cached_codes(q, codes, K, V, n, k, w, False)
    assert idx_ref.shape == (1, H, 1, k) and idx_cc.shape == (1, H, k)
    q_code = orc.pack_sign_u32(orc.mlp_hash_torch(q[:, :, None], w, False)[:, :, 0].numpy())[:, None]
    score = orc.hamming_score_u32(q_code, codes, "blocked")[0]                 # [n,H] matching bits
    for h in range(H):
        a, b = idx_ref[0, h, 0].numpy(), idx_cc[0, h]
        assert sorted(score[a, h].tolist()) == sorted(score[b, h].tolist())
        thr = score[b, h].min()
        whole = (score[:, h] == thr).sum() == (score[b, h] == thr).sum()
        if whole:   # no tie is cut: the two kept sets are the same set
            assert set(a.tolist()) == set(b.tolist())
            np.testing.assert_allclose(out_ref[0, h, 0].numpy(), out_cc[0, h].numpy(), atol=2e-5)
    # and the kernel-path step's output is attention over exactly its own rows
    want = orc.sparse_attention(q.numpy(), K.numpy(), V.numpy(), idx_cc)
    np.testing.assert_allclose(out_cc.numpy(), want, atol=1e-6)


def test_reference_form_budget_and_mask_are_the_reference_s():
    """k follows spotlight_generation.py:162-164; rows outside idx get exactly zero weight."""
    g = _gen(9)
    H, n, d = 2, 30, 16
    q = torch.randn(1, H, 1, d, generator=g)
    K = torch.randn(1, H, n, d, generator=g)
    V = torch.randn(1, H, n, d, generator=g)
    w = [(torch.randn(1, H, d, 32, generator=g), torch.zeros(1, H, 1, 32))]
    out, idx = orc.decode_step_reference_form(q, K, V, w, False, 0.9, 5)
    assert idx.shape[-1] == max(min(n, 5), n - int(n * 0.9)) == 5
    for h in range(H):
        sel = idx[0, h, 0]
        p = torch.softmax(K[0, h, sel].double() @ q[0, h, 0].double() / math.sqrt(d), dim=0)
        np.testing.assert_allclose(out[0, h, 0].numpy(), (p @ V[0, h, sel].double()).numpy(), atol=1e-5)


def test_apply_rope_is_the_complex_rotation():
    g = _gen(3)
    x = torch.randn(3, 5, 64, generator=g)
    pos = [0, 7, 31999]
    got = orc.apply_rope(x, pos, theta=5e5).double().numpy()
    for b, p in enumerate(pos):
        want = _rope_complex(x[b].double().numpy()[:, None, :], [p], 5e5, fp32_angles=True)[:, 0]
        np.testing.assert_allclose(got[b], want, atol=2e-5)
    assert torch.equal(orc.apply_rope(x, [0, 0, 0]), x)
