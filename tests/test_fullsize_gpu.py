"""The decode step at the full benchmark shapes, checked through properties that do
not need a CPU pass over the whole cache: every property below must hold for ANY
correct implementation of the path (spotlight_generation.py:143-215 on cached codes),
and each is evaluated with plain torch on the device from the state the step left."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPES = {
    # name: B, QH, KH, n0, k, dtype, hash, lru slots
    "c1": (1, 32, 32, 4096, 410, torch.float32, "linear", 0),
    "c2": (1, 32, 8, 32768, 655, torch.bfloat16, "mlp", 0),
    "c3": (16, 32, 8, 16384, 328, torch.bfloat16, "mlp", 1024),
    "c4": (1, 40, 8, 131072, 2622, torch.bfloat16, "mlp", 0),
}


@pytest.fixture(scope="module")
def decode():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd import decode
    return decode


def _popcount_bytes():
    return torch.tensor([bin(i).count("1") for i in range(256)], dtype=torch.int32, device=DEV)


def _scores(q_codes, k_codes, KH, G):
    """q_codes [B,QH,W] int32, k_codes [B,n,KH,W] int32 -> [B,KH,n] matching bits summed
    over the G query heads of the kv head (blocked map: q head h*G+g)."""
    lut = _popcount_bytes()
    B, n = k_codes.shape[0], k_codes.shape[1]
    W = k_codes.shape[-1]
    out = torch.zeros((B, KH, n), dtype=torch.int32, device=DEV)
    qg = q_codes.reshape(B, KH, G, W)
    for g in range(G):
        x = torch.bitwise_xor(k_codes, qg[:, None, :, g, :])                  # [B,n,KH,W]
        ham = lut[x.contiguous().view(torch.uint8).long()].reshape(B, n, KH, W * 4).sum(-1)
        out += (W * 32 - ham).permute(0, 2, 1)
    return out


def _weights(decode, kind, QH, KH, dtype, cg):
    if kind == "mlp":
        hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, cg, scale=0.05)
        hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, cg, scale=0.05)
    else:
        hq = decode.HashWeights.random_linear(QH, 128, 128, dtype, DEV, cg)
        hk = hq
    return hq, hk


def check_step_properties(st, q, kn, vn, out, n):
    """What one decode step must have left behind, whatever the implementation: `st` after the
    step that appended (kn, vn) as row n - 1 and attended for q; `out` that step's output."""
    from spotlight_amd import kernel
    B, QH, KH, k, dtype, lru = st.B, st.QH, st.KH, st.current_k, st.dtype, st.lru_slots
    hq, hk = st.hash_q, st.hash_k
    G = QH // KH
    assert st.seq_lens.tolist() == [n] * B
    # the appended row is in the cache, with the code of the key hash
    assert torch.equal(st.keys[:, n - 1], kn) and torch.equal(st.vals[:, n - 1], vn)
    k_code = kernel.hash_mlp_pack(kn, hk.w1, hk.b1, hk.w2, hk.b2, hk.residue)
    codes = st.codes[:, :n].view(torch.int32)
    assert torch.equal(codes[:, n - 1], k_code.view(torch.int32))
    # selection: k distinct tokens, ascending; nothing left out scores higher than anything
    # kept; inside the threshold score the kept tokens are the lowest-numbered ones
    idx = st.selected().long()                                            # [B,KH,k]
    assert idx.shape == (B, KH, k) and int(idx.min()) >= 0 and int(idx.max()) < n
    assert bool((idx[..., 1:] > idx[..., :-1]).all())
    q_code = kernel.hash_mlp_pack(q, hq.w1, hq.b1, hq.w2, hq.b2, hq.residue).view(torch.int32)
    score = _scores(q_code, codes, KH, G)                                 # [B,KH,n]
    kept = torch.zeros((B, KH, n), dtype=torch.bool, device=DEV)
    kept.scatter_(-1, idx, True)
    thr = torch.where(kept, score, torch.full_like(score, 10 ** 6)).amin(-1, keepdim=True)
    assert bool((torch.where(kept, torch.full_like(score, -1), score).amax(-1, keepdim=True) <= thr).all())
    at_thr = score == thr
    pos = torch.arange(n, device=DEV).expand(B, KH, n)
    last_kept = torch.where(at_thr & kept, pos, torch.full_like(pos, -1)).amax(-1, keepdim=True)
    first_left = torch.where(at_thr & ~kept, pos, torch.full_like(pos, n)).amin(-1, keepdim=True)
    assert bool((last_kept < first_left).all())
    # the output is softmax attention over exactly those rows
    bi = torch.arange(B, device=DEV)[:, None, None]
    hi = torch.arange(KH, device=DEV)[None, :, None]
    ks = st.keys[bi, idx, hi].float()                                     # [B,KH,k,d]
    vs = st.vals[bi, idx, hi].float()
    qg = q.float().reshape(B, KH, G, 128)
    w = torch.softmax(torch.einsum("bhgd,bhkd->bhgk", qg, ks) / math.sqrt(128.0), dim=-1)
    want = torch.einsum("bhgk,bhkd->bhgd", w, vs).reshape(B, QH, 128)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((out.float() - want).abs().max()) <= tol
    if lru:
        # every kept token and the new one are resident, in the slot the map names
        slot = torch.gather(st.token_slot, 2, idx).long()                 # [B,KH,k]
        assert int(slot.min()) >= 0
        assert torch.equal(torch.gather(st.slot_token, 2, slot).long(), idx)
        assert torch.equal(st.k_res[bi, hi, slot].float(), ks)
        assert int(st.token_slot[:, :, n - 1].min()) >= 0


def _prefilled(decode, B, QH, KH, n0, k, dtype, kind, lru, g, cg, n_cap=None, layout="auto"):
    hq, hk = _weights(decode, kind, QH, KH, dtype, cg)
    st = decode.LayerDecodeState(B, QH, KH, 128, n_cap or (n0 + 64 + 7) // 8 * 8, k, hq, hk, dtype=dtype, device=DEV, lru_slots=lru,
                                 codes_layout=layout)
    slab = max(1, (1 << 21) // (B * KH))   # bounds the transient memory of hashing the rows
    for s0 in range(0, n0, slab):
        s1 = min(n0, s0 + slab)
        keys = torch.randn((B, s1 - s0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
        vals = torch.randn((B, s1 - s0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
        st.load_rows(keys, vals, start=s0)
    st.set_length(n0)
    return st


def _fresh(g, B, QH, KH, dtype):
    return tuple(torch.randn((B, h, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype) for h in (QH, KH, KH))


@pytest.mark.parametrize("name,layout", [(n, "auto") for n in SHAPES] + [(n, "token") for n in SHAPES])
@torch.no_grad()
def test_full_size_step_properties(decode, name, layout):
    B, QH, KH, n0, k, dtype, kind, lru = SHAPES[name]
    g = torch.Generator(device=DEV).manual_seed(7)
    st = _prefilled(decode, B, QH, KH, n0, k, dtype, kind, lru, g, torch.Generator().manual_seed(7), layout=layout)
    assert st.codes_layout == ("head" if layout == "auto" else "token")
    for step in range(2):
        q, kn, vn = _fresh(g, B, QH, KH, dtype)
        out = st.step(q, kn, vn).clone()
        check_step_properties(st, q, kn, vn, out, n0 + step + 1)


@torch.no_grad()
def test_fused_tail_large_batch_across_block_boundary(decode):
    """Headline shape at batch 32, one row short of a 4096-row block: the second step opens a
    ninth block.  The select + attend launch is 2304 workgroups, far more than the device
    holds at once, so late workgroups start after early ones have finished; every (b, kv head)
    must still agree on the row count of the step.  Eager steps and graph replays."""
    B, QH, KH, k, dtype = 32, 32, 8, 655, torch.bfloat16
    n0 = 8 * 4096 - 1
    g = torch.Generator(device=DEV).manual_seed(11)
    st = _prefilled(decode, B, QH, KH, n0, k, dtype, "mlp", 0, g, torch.Generator().manual_seed(11), layout="token")
    n = n0
    for step in range(2):
        q, kn, vn = _fresh(g, B, QH, KH, dtype)
        out = st.step(q, kn, vn).clone()
        n += 1
        check_step_properties(st, q, kn, vn, out, n)
    st.capture(8)
    for step in range(3):
        q, kn, vn = _fresh(g, B, QH, KH, dtype)
        st.q_in.copy_(q); st.k_in.copy_(kn); st.v_in.copy_(vn)
        out = st.replay().clone()
        n += 1
        check_step_properties(st, q, kn, vn, out, n)
