"""Pins the CPU oracle without running the reference.

The reference ships no golden vectors for this path (its one assert-style
check, spotlight/kernel/pack_dx_u8.py:59-71, computes the expected value
in-line on random data).  Each oracle function is therefore pinned by an
independent formulation: a library routine, a brute force on tiny inputs, the
reference's other formulation of the same quantity, or a closed form; chosen
so that a dropped term, a wrong bit order, a transposed head mapping or an
unstable tie-break fails at least one check.
"""
import math

import numpy as np
import pytest
import torch

from oracle import spotlight_oracle as orc


def rng(seed):
    return np.random.default_rng(seed)


# ---- pack ------------------------------------------------------------------------

def test_pack_u32_matches_numpy_packbits():
    x = rng(0).standard_normal((7, 3, 128)).astype(np.float32)
    want = np.packbits(x > 0, axis=-1, bitorder="little").view("<u4")
    np.testing.assert_array_equal(orc.pack_sign_u32(x), want)


def test_pack_u32_known_answers():
    x = np.full((1, 32), -1.0)
    x[0, 0] = 1.0
    assert orc.pack_sign_u32(x)[0, 0] == 1           # element 0 -> bit 0 (LSB first)
    x[0, 31] = 2.0
    assert orc.pack_sign_u32(x)[0, 0] == 0x80000001   # element 31 -> bit 31
    y = np.full((1, 64), -1.0)
    y[0, 33] = 1.0
    np.testing.assert_array_equal(orc.pack_sign_u32(y), [[0, 2]])  # element 32w+j -> word w bit j


def test_pack_strict_greater_than_zero():
    x = np.array([[0.0, -0.0, np.nan, np.inf, -np.inf, 5e-324, -5e-324, 1.0] + [0.0] * 24])
    assert orc.pack_sign_u32(x)[0, 0] == (1 << 3) | (1 << 5) | (1 << 7)


def test_pack_u8_matches_numpy_and_is_the_u32_bytes():
    x = rng(1).standard_normal((4096, 128)).astype(np.float32)
    got = orc.pack_sign_u8(x)
    np.testing.assert_array_equal(got, np.packbits(x > 0, axis=-1, bitorder="little"))
    np.testing.assert_array_equal(got.view("<u4"), orc.pack_sign_u32(x))


def test_pack_c_twin(oracle_c):
    x = rng(2).standard_normal((50, 96)).astype(np.float32)
    out = np.zeros(50 * 3, dtype=np.uint32)
    oracle_c.orc_pack_sign_f32(x.ctypes.data, out.ctypes.data, out.size)
    np.testing.assert_array_equal(out.reshape(50, 3), orc.pack_sign_u32(x))


# ---- scorer ------------------------------------------------------------------------

def _codes(r, shape):
    return r.integers(0, 2 ** 32, size=shape, dtype=np.uint64).astype(np.uint32)


def _score_bruteforce(q, k, head_map):
    B, _, QH, W = q.shape
    _, n, KH, _ = k.shape
    G = QH // KH
    out = np.zeros((B, n, KH), dtype=np.int64)
    for b in range(B):
        for t in range(n):
            for h in range(KH):
                for g in range(G):
                    qh = g * KH + h if head_map == "interleaved" else h * G + g
                    for w in range(W):
                        x = (~(int(q[b, 0, qh, w]) ^ int(k[b, t, h, w]))) & 0xFFFFFFFF
                        out[b, t, h] += bin(x).count("1")
    return out


@pytest.mark.parametrize("head_map", ["interleaved", "blocked"])
def test_score_bruteforce(head_map):
    r = rng(3)
    q, k = _codes(r, (2, 1, 12, 4)), _codes(r, (2, 9, 4, 4))
    np.testing.assert_array_equal(orc.hamming_score_u32(q, k, head_map), _score_bruteforce(q, k, head_map))


def test_head_maps_differ_and_agree_for_mha():
    r = rng(4)
    q, k = _codes(r, (1, 1, 8, 4)), _codes(r, (1, 20, 4, 4))
    assert not np.array_equal(orc.hamming_score_u32(q, k, "interleaved"), orc.hamming_score_u32(q, k, "blocked"))
    q1, k1 = _codes(r, (1, 1, 4, 4)), _codes(r, (1, 20, 4, 4))
    np.testing.assert_array_equal(orc.hamming_score_u32(q1, k1, "interleaved"),
                                  orc.hamming_score_u32(q1, k1, "blocked"))


def test_score_identities():
    r = rng(5)
    q = _codes(r, (1, 1, 28, 4))
    k_same = q.reshape(1, 7, 4, 4)[:, :1]          # kv head h = q head 0*KH + h (interleaved, g = 0)
    s = orc.hamming_score_u32(q[:, :, :4], k_same, "interleaved")
    assert (s == 128).all()
    s = orc.hamming_score_u32(q[:, :, :4], ~k_same, "interleaved")
    assert (s == 0).all()


def test_score_equals_sign_matmul_formulation():
    # the PyTorch path's formulation: sign(q).sign(k) = nbits - 2*Hamming (spotlight_generation.py:19-22)
    r = rng(6)
    qi = torch.from_numpy(r.standard_normal((1, 6, 1, 128)).astype(np.float32))
    ki = torch.from_numpy(r.standard_normal((1, 6, 40, 128)).astype(np.float32))
    sim = orc.sign_matmul_score(qi, ki)[0, :, 0].numpy()                     # [H, n]
    qc = orc.pack_sign_u32(qi[:, :, 0].numpy())[:, None]                      # [1,1,H,4]
    kc = orc.pack_sign_u32(ki.permute(0, 2, 1, 3).numpy())                    # [1,n,H,4]
    match = orc.hamming_score_u32(qc, kc, "blocked")[0].T.astype(np.int64)    # [H, n]
    np.testing.assert_array_equal(sim.astype(np.int64), 2 * match - 128)


def test_swar_popcount_steps():
    v = _codes(rng(7), (1000,))
    want = np.array([int(x).bit_count() for x in v])
    np.testing.assert_array_equal(orc.swar_popcount32(v), want)
    np.testing.assert_array_equal(orc._popcount32(v), want)


def test_score_u8_bruteforce_and_wrap():
    r = rng(8)
    q = r.integers(0, 256, (2, 3, 1, 16), dtype=np.uint8)
    k = r.integers(0, 256, (2, 3, 11, 16), dtype=np.uint8)
    got = orc.hamming_score_u8(q, k)
    for b in range(2):
        for h in range(3):
            for t in range(11):
                want = sum(bin((~(int(a) ^ int(c))) & 0xFF).count("1") for a, c in zip(q[b, h, 0], k[b, h, t]))
                assert got[b, h, t] == want
    q32 = r.integers(0, 256, (1, 1, 1, 32), dtype=np.uint8)
    assert orc.hamming_score_u8(q32, q32.reshape(1, 1, 1, 32))[0, 0, 0] == 0   # 256 wraps in uint8


def test_score_c_twin(oracle_c):
    r = rng(9)
    q, k = _codes(r, (2, 1, 20, 4)), _codes(r, (2, 33, 4, 4))
    for hm, name in ((0, "interleaved"), (1, "blocked")):
        out = np.zeros((2, 33, 4), dtype=np.int16)
        oracle_c.orc_hamming_score(q.ctypes.data, k.ctypes.data, out.ctypes.data, 2, 33, 4, 5, 4, hm)
        np.testing.assert_array_equal(out, orc.hamming_score_u32(q, k, name))


# ---- budget ----------------------------------------------------------------------

@pytest.mark.parametrize("n,mask_out,k", [
    (4096, 0.9, 410), (4096, 0.98, 82), (8192, 0.98, 164), (16384, 0.98, 328),
    (32768, 0.98, 656), (131072, 0.98, 2622), (10, 0.98, 10), (19, 0.5, 19), (100, 0.98, 20),
])
def test_num_remain(n, mask_out, k):
    assert orc.num_remain(n, mask_out) == k


# ---- top-k -------------------------------------------------------------------------

def test_topk_bruteforce_and_tie_rule():
    r = rng(10)
    s = r.integers(0, 6, (2, 40, 3)).astype(np.int16)
    got = orc.topk_stable(s, 11)
    for b in range(2):
        for h in range(3):
            assert got[b, h].tolist() == orc.topk_bruteforce(s[b, :, h], 11)
    assert orc.topk_stable(np.array([5, 7, 7, 7, 3, 7, 7], dtype=np.int16).reshape(1, 7, 1), 3)[0, 0].tolist() == [1, 2, 3]


def test_topk_invariants_and_relation_to_torch():
    r = rng(11)
    s = r.integers(200, 300, (1, 5000, 4)).astype(np.int16)
    k = 500
    idx = orc.topk_stable(s, k)
    ref_vals = torch.from_numpy(s.astype(np.int32)).topk(k, dim=1).values.numpy()
    for h in range(4):
        sel = idx[0, h]
        col = s[0, :, h]
        assert len(set(sel.tolist())) == k and (np.diff(sel) > 0).all()
        thr = col[sel].min()
        rest = np.setdiff1d(np.arange(5000), sel)
        assert col[rest].max() <= thr
        at_thr = np.flatnonzero(col == thr)
        n_thr = (col[sel] == thr).sum()
        np.testing.assert_array_equal(np.intersect1d(sel, at_thr), at_thr[:n_thr])  # lowest indices win
        np.testing.assert_array_equal(np.sort(col[sel]), np.sort(ref_vals[0, :, h]))


def test_topk_c_twin(oracle_c):
    r = rng(12)
    s = np.ascontiguousarray(r.integers(0, 64, (3, 700, 5)).astype(np.int16))
    out = np.zeros((3, 5, 123), dtype=np.int32)
    assert oracle_c.orc_topk_select(s.ctypes.data, out.ctypes.data, 3, 700, 5, 123, 512) == 0
    np.testing.assert_array_equal(out, orc.topk_stable(s, 123))


# ---- gather / attention --------------------------------------------------------------

def _attn_inputs(r, B, QH, KH, L, k):
    q = r.standard_normal((B, QH, 16)).astype(np.float32)
    K = r.standard_normal((B, L, KH, 16)).astype(np.float32)
    V = r.standard_normal((B, L, KH, 16)).astype(np.float32)
    idx = np.stack([np.stack([np.sort(r.permutation(L)[:k]) for _ in range(KH)]) for _ in range(B)]).astype(np.int32)
    return q, K, V, idx


def test_gather_matches_torch_gather_expression():
    r = rng(13)
    _, K, V, idx = _attn_inputs(r, 2, 4, 4, 30, 7)
    ks, vs = orc.gather_kv(K, V, idx)
    ind = torch.from_numpy(idx).long().permute(0, 2, 1).unsqueeze(-1).expand(-1, -1, -1, 16)   # gpu_cache.py:51
    assert torch.equal(torch.from_numpy(ks), torch.gather(torch.from_numpy(K), 1, ind))
    assert torch.equal(torch.from_numpy(vs), torch.gather(torch.from_numpy(V), 1, ind))


def test_attention_equals_reference_masked_dense_form():
    r = rng(14)
    q, K, V, idx = _attn_inputs(r, 2, 8, 4, 50, 9)
    want = orc.masked_dense_attention(torch.from_numpy(q), torch.from_numpy(K), torch.from_numpy(V), idx).numpy()
    np.testing.assert_allclose(orc.sparse_attention(q, K, V, idx), want, atol=2e-6)


def test_attention_closed_forms_and_permutation_invariance():
    r = rng(15)
    q, K, V, idx = _attn_inputs(r, 1, 4, 2, 40, 10)
    out = orc.sparse_attention(q, K, V, idx)
    perm = idx[:, :, ::-1].copy()
    np.testing.assert_allclose(orc.sparse_attention(q, K, V, perm), out, atol=1e-12)
    one = idx[:, :, :1]
    o1 = orc.sparse_attention(q, K, V, one)
    for qh in range(4):
        np.testing.assert_allclose(o1[0, qh], V[0, one[0, qh // 2, 0], qh // 2], atol=1e-12)
    Kc = np.broadcast_to(K[:, :1], K.shape)
    om = orc.sparse_attention(q, Kc, V, idx)
    for qh in range(4):
        np.testing.assert_allclose(om[0, qh], V[0, idx[0, qh // 2], qh // 2].astype(np.float64).mean(0), atol=1e-12)
    # scale is 1/sqrt(d): doubling q equals an explicit scale of 2/sqrt(d)
    np.testing.assert_allclose(orc.sparse_attention(2 * q, K, V, idx),
                               orc.sparse_attention(q, K, V, idx, scale=2 / math.sqrt(16)), atol=1e-12)


def test_attention_c_twin(oracle_c):
    r = rng(16)
    q, K, V, idx = _attn_inputs(r, 2, 6, 3, 25, 8)
    idx[0, 0, -2:] = -1
    out = np.zeros_like(q)
    oracle_c.orc_sparse_attention_f32(q.ctypes.data, K.ctypes.data, V.ctypes.data, idx.ctypes.data,
                                      out.ctypes.data, 2, 6, 3, 16, 25, 8)
    np.testing.assert_allclose(out, orc.sparse_attention(q, K, V, idx), atol=1e-6)


# ---- hashing ----------------------------------------------------------------------------

def test_mlp_hash_against_torch_modules():
    r = rng(17)
    x = r.standard_normal((2, 3, 8))
    w1, b1 = r.standard_normal((3, 8, 12)), r.standard_normal((3, 12))
    w2, b2 = r.standard_normal((3, 12, 8)), r.standard_normal((3, 8))
    got = orc.mlp_hash(x, [(w1, b1), (w2, b2)], residue=False)
    for h in range(3):
        lin1 = torch.nn.Linear(8, 12).double()
        lin2 = torch.nn.Linear(12, 8).double()
        with torch.no_grad():
            lin1.weight.copy_(torch.from_numpy(w1[h].T)); lin1.bias.copy_(torch.from_numpy(b1[h]))
            lin2.weight.copy_(torch.from_numpy(w2[h].T)); lin2.bias.copy_(torch.from_numpy(b2[h]))
            want = lin2(torch.nn.functional.silu(lin1(torch.from_numpy(x[:, h]))))
        np.testing.assert_allclose(got[:, h], want.numpy(), atol=1e-12)


def test_mlp_hash_residue_and_torch_form_agree():
    r = rng(18)
    x = r.standard_normal((2, 3, 8))
    ws = [(r.standard_normal((3, 8, 8)), r.standard_normal((3, 8))) for _ in range(2)]
    a = orc.mlp_hash(x, ws, residue=True)
    tw = [(torch.from_numpy(w)[None], torch.from_numpy(b)[None, :, None]) for w, b in ws]
    b = orc.mlp_hash_torch(torch.from_numpy(x)[:, :, None], tw, residue=True)[:, :, 0].numpy()
    np.testing.assert_allclose(a, b, atol=1e-12)
    assert not np.allclose(a, orc.mlp_hash(x, ws, residue=False))


def test_linear_hash_is_a_matmul():
    r = rng(19)
    x, L = r.standard_normal((2, 4, 8)), r.standard_normal((4, 8, 8))
    np.testing.assert_allclose(orc.linear_hash(x, L)[1, 2], x[1, 2] @ L[2], atol=1e-12)


# ---- cache / LRU ---------------------------------------------------------------------------

def test_cache_model_appends_in_order():
    c = orc.CacheModel(2, 10, 3, 4, np.float32)
    a = rng(20).standard_normal((2, 4, 3, 4)).astype(np.float32)
    b = rng(21).standard_normal((2, 1, 3, 4)).astype(np.float32)
    c.update(a)
    view = c.update(b)
    assert view.shape == (2, 5, 3, 4) and c.length == 5
    np.testing.assert_array_equal(view[:, :4], a)
    np.testing.assert_array_equal(view[:, 4:], b)
    assert not c.buf[:, 5:].any()


def test_lru_model_resident_set_equals_sequential_lru():
    # From the same state, one step of the batched model and one step of the
    # textbook one-at-a-time LRU must keep the same tokens with the same stamps;
    # only the slot a miss lands in may differ (which, through the slot-index
    # tie rule, is why the comparison restarts from a common state every step).
    r = rng(22)
    for C, n0, k in [(8, 12, 3), (6, 30, 5), (16, 40, 7)]:
        a, b = orc.LruModel(C), orc.LruSequentialModel(C)
        n = n0
        for t in range(1, 60):
            sel = np.sort(r.choice(n, size=k, replace=False))
            if t % 3 == 0:           # locality: re-use part of what is resident
                res = [x for x in a.token if x >= 0]
                sel = np.sort(np.unique(np.concatenate([sel[:k // 2], r.choice(res, size=k - k // 2)])))
            b.token, b.stamp = list(a.token), list(a.stamp)
            slots = a.step(t, sel, n)
            b.step(t, sel, n)
            assert sorted(a.token) == sorted(b.token)
            assert {tok: a.stamp[s] for s, tok in enumerate(a.token) if tok >= 0} == \
                   {tok: b.stamp[s] for s, tok in enumerate(b.token) if tok >= 0}
            assert [a.token[s] for s in slots] == [int(x) for x in sel]
            n += 1
        assert a.hits > 0 and a.misses > 0


def test_lru_model_known_trace():
    m = orc.LruModel(4)
    assert m.step(1, [0, 1], 2) == [0, 1]          # all misses fill empty slots in order
    assert m.token == [0, 1, 2, -1] and m.stamp == [1, 1, 1, 0]
    assert m.step(2, [1], 3) == [1]                # hit on 1; new token 3 takes the empty slot
    assert m.token == [0, 1, 2, 3] and m.stamp == [1, 2, 1, 2]
    m.step(3, [3, 5], 6)                           # 5 and 6 evict the two oldest: slots 0 and 2
    assert m.token == [5, 1, 6, 3] and m.stamp == [3, 2, 3, 3]
    assert (m.hits, m.misses) == (2, 6)
