"""The drop-in cache classes (spotlight/modifiers/gpu_cache.py:6-118): same constructor arguments,
attributes and return conventions; update() appends and returns views, gather() is the
reference's topk + torch.gather with ties resolved to the lowest index."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def gc():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd.modifiers import gpu_cache
    return gpu_cache


def _small(cls, rows):
    return type("Small" + cls.__name__, (cls,), {"init_seq_length": rows})


def test_kvhash_update_appends_and_returns_a_view(gc):
    H = _small(gc.KVHash, 64)
    c = H(2, 4, 4, 3, dtype=torch.int32, device=[DEV] * 3)
    assert c.length == [0, 0, 0] and c.max_length == 64 and len(c.key_cache) == 3
    a = torch.randint(0, 1 << 30, (2, 10, 4, 4), dtype=torch.int32, device=DEV)
    b = torch.randint(0, 1 << 30, (2, 1, 4, 4), dtype=torch.int32, device=DEV)
    v = c.update(1, a)
    assert v.shape == (2, 10, 4, 4) and torch.equal(v, a) and c.length == [0, 10, 0]
    v = c.update(1, b)
    assert v.shape == (2, 11, 4, 4) and torch.equal(v[:, :10], a) and torch.equal(v[:, 10:], b)
    assert v.data_ptr() == c.key_cache[1].data_ptr()          # a view of the preallocated buffer (gpu_cache.py:45)
    assert int(c.key_cache[0].abs().sum()) == 0


@pytest.mark.parametrize("max_score", [None, 512])
def test_kvcache_update_and_gather_follow_the_reference(gc, max_score):
    C = _small(gc.KVCache, 600)
    B, KH, d, n, budget = 2, 4, 128, 500, 37
    g = torch.Generator().manual_seed(3)
    c = C(B, KH, d, 2, dtype=torch.bfloat16, device=[DEV, DEV], max_score=max_score)
    keys = torch.randn(B, n, KH, d, generator=g).to(torch.bfloat16).to(DEV)
    vals = torch.randn(B, n, KH, d, generator=g).to(torch.bfloat16).to(DEV)
    k_view, v_view = c.update(0, keys[:, :499], vals[:, :499])
    k_view, v_view = c.update(0, keys[:, 499:], vals[:, 499:])
    assert c.length == [n, 0] and torch.equal(k_view, keys) and torch.equal(v_view, vals)
    attn = torch.randint(200, 320, (B, n, KH), generator=g, dtype=torch.int16).to(DEV)   # many ties
    ks, vs = c.gather(0, attn, budget)
    assert ks.shape == vs.shape == (B, budget, KH, d)
    # the reference: ind = attn.topk(budget, dim=1, sorted=False).indices; gather(dim=1) (gpu_cache.py:50-53).
    # torch leaves the choice among equal scores open, so compare what is determined: the multiset of kept
    # scores, and that every kept row is a row of the cache whose score is at least the threshold
    ref = attn.long().topk(budget, dim=1).values.sort(dim=1).values                      # [B,budget,KH]
    from spotlight_amd import kernel
    ind = kernel.topk_select(attn, budget, 512).long()                                   # [B,KH,budget], ascending
    got_scores = torch.gather(attn.long().permute(0, 2, 1), 2, ind).permute(0, 2, 1).sort(dim=1).values
    assert torch.equal(got_scores, ref)
    expand = ind.permute(0, 2, 1).unsqueeze(-1).expand(-1, -1, -1, d)
    assert torch.equal(ks, torch.gather(keys, 1, expand)) and torch.equal(vs, torch.gather(vals, 1, expand))
    # ties go to the lowest index: nothing left out at the threshold score precedes a kept row of that score
    thr = ref[:, :1].permute(0, 2, 1)                                                    # [B,KH,1]
    s = attn.long().permute(0, 2, 1)
    kept = torch.zeros_like(s, dtype=torch.bool).scatter_(2, ind, True)
    pos = torch.arange(n, device=DEV).expand_as(s)
    last_kept = torch.where(kept & (s == thr), pos, torch.full_like(pos, -1)).amax(-1)
    first_left = torch.where(~kept & (s == thr), pos, torch.full_like(pos, n)).amin(-1)
    assert bool((last_kept < first_left).all())
