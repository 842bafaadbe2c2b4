"""sl_topk_select_static (the entry point that allocates nothing: its scratch is a device array
inside the library) against sl_topk_select on the same scores, through the C ABI: bit-exact
index lists on two calls in a row, the second on a smaller input, so that whatever the first
call left in the shared scratch must not leak into the second."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd import _lib
    return _lib, _lib.load()


def _both(lib, score, k, max_score, seq_lens=None):
    _lib, L = lib
    B, n, KH = score.shape
    sb, sn, sh = score.stride()
    stream = torch.cuda.current_stream().cuda_stream
    lens = seq_lens.data_ptr() if seq_lens is not None else None
    want = torch.full((B, KH, k), -5, dtype=torch.int32, device=DEV)
    nbytes = L.sl_topk_workspace_bytes(B, KH, max_score, n)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=DEV)
    _lib.check(L.sl_topk_select(score.data_ptr(), sb, sn, sh, want.data_ptr(), B, n, KH, k, max_score, lens,
                                ws.data_ptr(), nbytes, stream), "sl_topk_select")
    got = torch.full((B, KH, k), -9, dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    _lib.check(L.sl_topk_select_static(score.data_ptr(), sb, sn, sh, got.data_ptr(), B, n, KH, k, max_score, lens,
                                       stream), "sl_topk_select_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return want, got


def test_static_scratch_topk_equals_workspace_topk_on_two_calls_in_a_row(lib):
    g = torch.Generator().manual_seed(5)
    # first call: 20000 tokens (several blocks, 8 histogram copies), scores of a G = 4 group
    big = torch.randint(0, 513, (2, 20000, 8), generator=g, dtype=torch.int16).to(DEV)
    want, got = _both(lib, big, 400, 512)
    assert torch.equal(want, got)
    # second call, smaller in every way, with per-sequence lengths and heavy ties
    small = torch.randint(60, 70, (3, 777, 4), generator=g, dtype=torch.int16).to(DEV)
    lens = torch.tensor([777, 5, 300], dtype=torch.int32, device=DEV)
    want, got = _both(lib, small, 33, 128, lens)
    assert torch.equal(want, got)
    assert int(got[1, :, 5:].max()) == -1 and int(got[1, :, :5].min()) >= 0   # 5 tokens only: tail is -1
    # and the first input again: the same answer as before
    want2, got2 = _both(lib, big, 400, 512)
    assert torch.equal(want2, got2)


def test_static_scratch_topk_rejects_what_does_not_fit(lib):
    _lib, L = lib
    B, n, KH, max_score = 64, 70000, 8, 1024   # needs far more than the built-in 8 MiB
    assert L.sl_topk_workspace_bytes(B, KH, max_score, n) > (8 << 20)
    score = torch.zeros((1,), dtype=torch.int16, device=DEV)
    idx = torch.zeros((1,), dtype=torch.int32, device=DEV)
    rc = L.sl_topk_select_static(score.data_ptr(), n * KH, KH, 1, idx.data_ptr(), B, n, KH, 10, max_score, None,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == -7 and b"scratch" in L.sl_strerror(rc)
