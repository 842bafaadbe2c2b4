"""Bounded soak of the cross-workgroup hand-off (partial results published with device-coherent
stores, an arrival ticket, the last workgroup merging): a few thousand graph replays at the
two benchmark shapes whose attention is cut into several runs per (b, kv head), every replay
compared with a state whose attention is ONE run per (b, kv head) -- no hand-off at all -- on
the same inputs.  Stops at the first mismatch."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REPLAYS = 2000


@pytest.fixture(scope="module")
def env():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd import _lib, decode
    return _lib, decode


def _pair(env, B, QH, KH, n0, k, lru, seed):
    """Two states over the same cache contents and the same input buffers: `multi` as the step runs by
    default, `single` with selection and attention as two launches and one attention run per head."""
    _lib, decode = env
    L = _lib.load()
    dtype = torch.bfloat16
    cg = torch.Generator().manual_seed(seed)
    hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, cg, scale=0.05)
    hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, cg, scale=0.05)
    inputs = tuple(torch.zeros((B, h, 128), dtype=dtype, device=DEV) for h in (QH, KH, KH))
    n_cap = (n0 + REPLAYS + 72) // 8 * 8
    g = torch.Generator(device=DEV).manual_seed(seed)
    # `multi` takes the layout the step picks by itself (head-major at the headline shape: scorer, selection and
    # attention in one launch, blocks swapping histograms); `single` is the three-launch step on token-major codes
    states = [decode.LayerDecodeState(B, QH, KH, 128, n_cap, k, hq, hk, dtype=dtype, device=DEV, lru_slots=lru, inputs=inputs,
                                      codes_layout=layout) for layout in ("auto", "token")]
    slab = max(1, (1 << 21) // (B * KH))
    for s0 in range(0, n0, slab):
        s1 = min(n0, s0 + slab)
        keys = torch.randn((B, s1 - s0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
        vals = torch.randn((B, s1 - s0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
        codes = hk.hash_rows(keys)
        for st in states:
            st.load_rows(keys, vals, start=s0, codes=codes)
    for st in states:
        st.set_length(n0)
    multi, single = states
    try:
        multi.capture(REPLAYS + 8)
        _lib.check(L.sl_tune(b"fuse_select_attend", 0), "sl_tune")
        _lib.check(L.sl_tune(b"attn_target_wgs", 1), "sl_tune")
        single.capture(REPLAYS + 8)
    finally:
        _lib.check(L.sl_tune(b"fuse_select_attend", 1), "sl_tune")
        _lib.check(L.sl_tune(b"attn_target_wgs", 512), "sl_tune")
    return multi, single, inputs, g


@pytest.mark.parametrize("name,B,QH,KH,n0,k,lru", [
    ("headline shape: one-launch scorer + tail, 13 blocks of 2560 rows (= attention runs) per head", 1, 32, 8, 32768, 655, 0),
    ("batch 16 with the LRU table: attention launch with deferred fetch, 4 runs per head", 16, 32, 8, 16384, 328, 1024),
])
@torch.no_grad()
def test_every_replay_matches_the_run_without_a_hand_off(env, name, B, QH, KH, n0, k, lru):
    multi, single, inputs, g = _pair(env, B, QH, KH, n0, k, lru, seed=len(name))
    for i in range(REPLAYS):
        for t in inputs:
            t.normal_(generator=g)
        a = multi.replay()
        b = single.replay()
        same_idx = torch.equal(multi.idx, single.idx)
        err = float((a.float() - b.float()).abs().max())
        assert same_idx and err <= 2e-2, f"replay {i}: idx equal {same_idx}, max-abs output difference {err}"
    assert multi.seq_lens.tolist() == single.seq_lens.tolist() == [n0 + REPLAYS] * B
    assert not multi.peer_wait_failed() and not single.peer_wait_failed()   # no bounded wait ran out in any replay
