"""Host-memory K / V tier: pinned host store read and written in place by the kernels
(drop-in for spotlight/modifiers/cpu_cache.py:50-130, and the store behind the LRU)."""
import numpy as np
import pytest
import torch

from oracle import spotlight_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def env():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd import decode, kernel
    from spotlight_amd.modifiers import cpu_cache
    return decode, kernel, cpu_cache


def test_pageable_host_memory_is_refused(env):
    _, kernel, _ = env
    with pytest.raises(RuntimeError):
        kernel.device_ptr(torch.zeros(16))
    pinned = torch.zeros(16, pin_memory=True)
    assert kernel.device_ptr(pinned) != 0


def test_cpu_cache_update_and_gather_match_torch(env):
    """KVCache of the CPU tier: rows appended by the GPU land in host memory; gather
    returns the rows the stable top-k picks, bit for bit (cpu_cache.py:50-57,105-130)."""
    _, kernel, cc = env
    g = torch.Generator().manual_seed(0)
    B, KH, d, L = 2, 4, 128, 3
    cc.KVCache.init_seq_length = 512
    try:
        cache = cc.KVCache(B, KH, d, L, dtype=torch.bfloat16, freeze=[0])
    finally:
        cc.KVCache.init_seq_length = cc.INIT_SEQ_LEN
    assert cache.key_cache[0].is_cuda and not cache.key_cache[1].is_cuda and cache.key_cache[1].is_pinned()
    for layer in (0, 1):
        k1 = torch.randn(B, 300, KH, d, generator=g).to(torch.bfloat16)
        v1 = torch.randn(B, 300, KH, d, generator=g).to(torch.bfloat16)
        k2 = torch.randn(B, 1, KH, d, generator=g).to(torch.bfloat16)
        v2 = torch.randn(B, 1, KH, d, generator=g).to(torch.bfloat16)
        cache.update(layer, k1.to(DEV), v1.to(DEV))
        kk, vv = cache.update(layer, k2.to(DEV), v2.to(DEV))
        torch.cuda.synchronize()
        assert cache.length[layer] == 301 and kk.shape == (B, 301, KH, d)
        assert torch.equal(kk.cpu(), torch.cat([k1, k2], 1)) and torch.equal(vv.cpu(), torch.cat([v1, v2], 1))
        attn = torch.randint(0, 129, (B, 301, KH), generator=g).to(torch.int16)
        ks, vs = cache.gather(layer, attn.to(DEV), 25, max_score=128)
        assert ks.is_cuda and ks.shape == (B, 25, KH, d)
        idx = orc.topk_stable(attn.numpy(), 25)                              # [B,KH,k] ascending token order
        want_k, want_v = orc.gather_kv(kk.cpu().float().numpy(), vv.cpu().float().numpy(), idx)
        np.testing.assert_array_equal(ks.float().cpu().numpy(), want_k)
        np.testing.assert_array_equal(vs.float().cpu().numpy(), want_v)


def _state(decode, g, host, B=2, QH=32, KH=8, n0=900, n_cap=1024, k=40, lru=64, dtype=torch.bfloat16):
    hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    st = decode.LayerDecodeState(B, QH, KH, 128, n_cap, k, hq, hk, dtype=dtype, device=DEV, lru_slots=lru,
                                 host_store=host)
    keys = torch.randn(B, n0, KH, 128, generator=g).to(dtype)
    vals = torch.randn(B, n0, KH, 128, generator=g).to(dtype)
    st.prefill(keys.to(DEV), vals.to(DEV))
    return st


def test_decode_with_host_store_equals_device_store(env):
    """The same steps with the full store in pinned host memory: identical selection,
    identical output, identical resident table; the appended rows are in host memory."""
    decode, _, _ = env
    dev = _state(decode, torch.Generator().manual_seed(1), host=False)
    hst = _state(decode, torch.Generator().manual_seed(1), host=True)
    assert not hst.keys.is_cuda and hst.keys.is_pinned() and dev.keys.is_cuda
    g = torch.Generator().manual_seed(2)
    for step in range(6):
        q = torch.randn(2, 32, 128, generator=g).to(torch.bfloat16).to(DEV)
        if step % 2:
            q = prev                      # repeated query: mostly hits, nothing crosses the link
        prev = q
        kn = torch.randn(2, 8, 128, generator=g).to(torch.bfloat16)
        vn = torch.randn(2, 8, 128, generator=g).to(torch.bfloat16)
        a = dev.step(q, kn.to(DEV), vn.to(DEV)).clone()
        b = hst.step(q, kn.to(DEV), vn.to(DEV)).clone()
        torch.cuda.synchronize()
        assert torch.equal(dev.idx, hst.idx) and torch.equal(a, b), step
        assert torch.equal(dev.slot_token, hst.slot_token) and torch.equal(dev.slot_stamp, hst.slot_stamp)
        assert torch.equal(hst.keys[:, 900 + step], kn) and torch.equal(hst.vals[:, 900 + step], vn)
    assert torch.equal(dev.lru_stats, hst.lru_stats) and int(hst.lru_stats[..., 0].sum()) > 0


def test_host_store_needs_the_resident_table(env):
    decode, _, _ = env
    g = torch.Generator().manual_seed(3)
    with pytest.raises(AssertionError):
        _state(decode, g, host=True, lru=0)
