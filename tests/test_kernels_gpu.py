"""Parity of every HIP kernel, through the C ABI, against the CPU oracle.

Integer results (codes, scores, selected indices, slot maps) must be bit
exact; attention outputs must be within 1e-5 (fp32) / 2e-2 (bf16, fp16)
max-abs of the fp64 oracle.
"""
import numpy as np
import pytest
import torch

from oracle import spotlight_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd import kernel
    return kernel


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def _rand_codes(g, shape):
    x = torch.randint(0, 2 ** 32, shape, generator=g, dtype=torch.int64)
    return x.numpy().astype(np.uint32)


def _u32(arr):
    return torch.from_numpy(np.ascontiguousarray(arr)).to(DEV)


# ---- (a) pack -------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 32), (3, 5, 128), (4096, 128), (7, 1, 8, 256)])
def test_pack_u32(K, dtype, shape):
    x = torch.randn(shape, generator=_gen(1)).to(dtype)
    got = K.pack_cuda_func(x.to(DEV)).cpu().numpy()
    want = orc.pack_sign_u32(x.float().numpy())
    assert got.dtype == np.uint32 and got.shape == want.shape
    np.testing.assert_array_equal(got, want)


def test_pack_edge_values(K):
    vals = [0.0, -0.0, float("nan"), float("inf"), -float("inf"), 1e-45, -1e-45, 1e-30, -1e-30, 1.0, -1.0]
    x = torch.tensor((vals * 6)[:64], dtype=torch.float32).reshape(1, 64)
    got = K.pack_cuda_func(x.to(DEV)).cpu().numpy()
    np.testing.assert_array_equal(got, orc.pack_sign_u32(x.numpy()))
    xb = x.to(torch.bfloat16)
    got = K.pack_cuda_func(xb.to(DEV)).cpu().numpy()
    np.testing.assert_array_equal(got, orc.pack_sign_u32(xb.float().numpy()))


def test_pack_rejects_bad_last_dim(K):
    with pytest.raises(RuntimeError):
        K.pack_cuda_func(torch.zeros(4, 48, device=DEV))


@pytest.mark.parametrize("shape", [(4096, 128), (5, 8), (3, 7, 24)])
def test_pack_u8(K, shape):
    # the reference's own self check: pack_dx_u8.py:59-71
    x = torch.randn(shape, generator=_gen(2))
    got = K.pack_dx_u8_func(x.to(DEV)).cpu().numpy()
    np.testing.assert_array_equal(got, orc.pack_sign_u8(x.numpy()))


def test_pack_noncontiguous_input(K):
    x = torch.randn(64, 16, generator=_gen(3)).t()  # [16, 64] strided
    got = K.pack_cuda_func(x.to(DEV)).cpu().numpy()
    np.testing.assert_array_equal(got, orc.pack_sign_u32(x.contiguous().numpy()))


# ---- (b) scorer ------------------------------------------------------------------

SCORE_CASES = [
    # B, n, KH, G, W
    (1, 64, 4, 7, 4),      # the one shape the reference's CUDA kernel ships (attn_k4_q28.cu)
    (2, 65, 4, 7, 4),      # tail: n % 64 != 0 (attn_k4_q28.cu:53,71)
    (1, 1000, 8, 4, 4),    # Llama-3-8B
    (1, 333, 8, 5, 4),     # Qwen2.5-14B
    (1, 515, 32, 1, 4),    # MHA
    (2, 100, 2, 3, 4),     # generic G path
    (1, 257, 8, 4, 2),     # 64-bit codes
    (1, 130, 8, 2, 8),     # 256-bit codes, generic G
    (3, 77, 16, 2, 1),     # 32-bit codes
    (1, 1, 8, 4, 4),
]


@pytest.mark.parametrize("B,n,KH,G,W", SCORE_CASES)
@pytest.mark.parametrize("head_map", ["interleaved", "blocked"])
def test_hamming_score(K, B, n, KH, G, W, head_map):
    g = _gen(B * 1000 + n)
    q = _rand_codes(g, (B, 1, KH * G, W))
    k = _rand_codes(g, (B, n, KH, W))
    got = K.hamming_score(_u32(q), _u32(k), head_map).cpu().numpy()
    want = orc.hamming_score_u32(q, k, head_map)
    assert got.dtype == np.int16
    np.testing.assert_array_equal(got, want)


def test_hamming_identities(K):
    g = _gen(5)
    q = _rand_codes(g, (1, 1, 8, 4))
    k = np.concatenate([q.reshape(1, 1, 8, 4), ~q.reshape(1, 1, 8, 4)], axis=1)  # k = q, then ~q
    got = K.attn_cuda_func(_u32(q), _u32(k)).cpu().numpy()
    assert (got[0, 0] == 128).all() and (got[0, 1] == 0).all()


def test_reference_named_entry_points(K):
    g = _gen(6)
    q = _rand_codes(g, (2, 1, 28, 4))
    k = _rand_codes(g, (2, 300, 4, 4))
    want = orc.hamming_score_u32(q, k, "interleaved")
    for fn in (K.attn_cuda_func, K.attn_triton_func, K.attn_dx_u32_func):
        np.testing.assert_array_equal(fn(_u32(q), _u32(k)).cpu().numpy(), want)
    with pytest.raises(RuntimeError):
        K.attn_cuda_func(_u32(q).view(2, 28, 1, 4).expand(2, 28, 2, 4).contiguous(), _u32(k))  # QN != 1


def test_hamming_seq_lens(K):
    g = _gen(7)
    q = _rand_codes(g, (3, 1, 32, 4))
    k = _rand_codes(g, (3, 500, 8, 4))
    lens = torch.tensor([500, 17, 256], dtype=torch.int32)
    got = K.hamming_score(_u32(q), _u32(k), "blocked", lens.to(DEV)).cpu().numpy()
    want = orc.hamming_score_u32(q, k, "blocked")
    for b, l in enumerate(lens.tolist()):
        np.testing.assert_array_equal(got[b, :l], want[b, :l])
        assert (got[b, l:] == 0).all()   # untouched rows keep the zero fill


@pytest.mark.parametrize("D", [4, 8, 16, 32])
def test_hamming_u8(K, D):
    g = _gen(8)
    q = torch.randint(0, 256, (2, 5, 1, D), generator=g, dtype=torch.uint8)
    k = torch.randint(0, 256, (2, 5, 301, D), generator=g, dtype=torch.uint8)
    if D == 32:
        k[0, 0, 0] = q[0, 0, 0]   # 256 matching bits wrap to 0, as the reference's uint8 does
    got = K.attn_dx_u8_func(q.to(DEV), k.to(DEV)).cpu().numpy()
    np.testing.assert_array_equal(got, orc.hamming_score_u8(q.numpy(), k.numpy()))


# ---- (c) top-k ---------------------------------------------------------------------

def _scores(g, B, n, KH, lo, hi):
    return torch.randint(lo, hi + 1, (B, n, KH), generator=g, dtype=torch.int16)


@pytest.mark.parametrize("B,n,KH,k,lo,hi,max_score", [
    (1, 4096, 8, 410, 200, 312, 512),       # massive ties, like real code scores
    (2, 1000, 4, 100, 0, 896, 896),
    (1, 32768, 8, 655, 216, 296, 512),      # headline shape: one pass of the selector
    (1, 40000, 2, 800, 250, 262, 512),      # more than one selector pass
    (1, 100, 8, 100, 0, 5, 128),            # k == n
    (1, 50, 3, 64, 0, 128, 128),            # k > n  -> -1 tail
    (3, 777, 5, 1, 0, 640, 640),            # k == 1
    (1, 9000, 1, 4500, 7, 7, 16),           # all scores equal: pure tie-break
    (1, 20, 8, 20, 0, 4096, 4096),
])
def test_topk_select(K, B, n, KH, k, lo, hi, max_score):
    s = _scores(_gen(n + k), B, n, KH, lo, hi)
    got = K.topk_select(s.to(DEV), k, max_score).cpu().numpy()
    want = orc.topk_stable(s.numpy(), k)
    kk = want.shape[2]
    np.testing.assert_array_equal(got[:, :, :kk], want)
    assert (got[:, :, kk:] == -1).all()
    # run twice: the selector is deterministic and leaves its workspace clean
    again = K.topk_select(s.to(DEV), k, max_score).cpu().numpy()
    np.testing.assert_array_equal(again, got)


def test_topk_select_head_major_and_seq_lens(K):
    g = _gen(11)
    s = _scores(g, 2, 5000, 8, 230, 290)
    lens = torch.tensor([5000, 1234], dtype=torch.int32)
    sh = s.permute(0, 2, 1).contiguous()  # [B, KH, n]
    got = K.topk_select(sh.to(DEV), 99, 512, lens.to(DEV), layout="bhn").cpu().numpy()
    for b, l in enumerate(lens.tolist()):
        want = orc.topk_stable(s[b:b + 1, :l].numpy(), 99)
        np.testing.assert_array_equal(got[b:b + 1], want)


def test_topk_relation_to_torch_topk(K):
    # torch.topk may pick other indices among ties; the multiset of kept scores must agree
    s = _scores(_gen(12), 2, 3000, 4, 240, 272)
    idx = K.topk_select(s.to(DEV), 300, 512).cpu().long()
    kept = torch.gather(s.permute(0, 2, 1), 2, idx).sort(dim=2).values
    ref = s.permute(0, 2, 1).to(torch.int32).topk(300, dim=2).values.sort(dim=2).values
    assert torch.equal(kept.to(torch.int32), ref)


# ---- gather ------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gather_kv(K, dtype):
    g = _gen(13)
    B, L, KH, d, k = 2, 300, 4, 128, 37
    keys = torch.randn(B, L, KH, d, generator=g).to(dtype)
    vals = torch.randn(B, L, KH, d, generator=g).to(dtype)
    idx = torch.stack([torch.stack([torch.randperm(L, generator=g)[:k].sort().values for _ in range(KH)])
                       for _ in range(B)]).to(torch.int32)
    ks, vs = K.gather_kv(keys.to(DEV), vals.to(DEV), idx.to(DEV))
    wk, wv = orc.gather_kv(keys.float().numpy(), vals.float().numpy(), idx.numpy())
    np.testing.assert_array_equal(ks.float().cpu().numpy(), wk)
    np.testing.assert_array_equal(vs.float().cpu().numpy(), wv)
    # same thing as the reference's expression (gpu_cache.py:50-53)
    ind = idx.long().permute(0, 2, 1).unsqueeze(-1).expand(-1, -1, -1, d)
    assert torch.equal(ks.cpu(), torch.gather(keys, 1, ind))


# ---- (e) attention ---------------------------------------------------------------------

ATTN_CASES = [
    # B, QH, KH, L, k
    (1, 32, 8, 2048, 655),
    (1, 32, 32, 600, 410),
    (2, 40, 8, 3000, 100),
    (1, 28, 4, 500, 17),
    (1, 8, 8, 64, 1),
    (3, 16, 8, 200, 33),
    (16, 32, 8, 700, 328),
    (1, 10, 2, 6000, 2622),     # long runs: the 8-wave flavour, 5 query heads per kv head
    (1, 4, 4, 3000, 2500),
]


def _attn_inputs(g, B, QH, KH, L, k, dtype):
    q = torch.randn(B, QH, 128, generator=g).to(dtype)
    keys = torch.randn(B, L, KH, 128, generator=g).to(dtype)
    vals = torch.randn(B, L, KH, 128, generator=g).to(dtype)
    idx = torch.stack([torch.stack([torch.randperm(L, generator=g)[:k].sort().values for _ in range(KH)])
                       for _ in range(B)]).to(torch.int32)
    return q, keys, vals, idx


@pytest.mark.parametrize("B,QH,KH,L,k", ATTN_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_sparse_attention(K, B, QH, KH, L, k, dtype):
    q, keys, vals, idx = _attn_inputs(_gen(L + k), B, QH, KH, L, k, dtype)
    got = K.sparse_gqa_attn(q.to(DEV), keys.to(DEV), vals.to(DEV), idx.to(DEV)).float().cpu().numpy()
    want = orc.sparse_attention(q.float().numpy(), keys.float().numpy(), vals.float().numpy(), idx.numpy())
    assert np.abs(got - want).max() <= TOL[dtype]


@pytest.mark.parametrize("B,QH,KH,L,k", ATTN_CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sparse_attention_matrix_core_flavour(K, B, QH, KH, L, k, dtype):
    """The same attention with the q.K products on the matrix cores (sl_tune "attn_mfma")."""
    from spotlight_amd import _lib
    L_ = _lib.load()
    q, keys, vals, idx = _attn_inputs(_gen(L + k), B, QH, KH, L, k, dtype)
    if k > 1:
        idx[:, :, k // 2] = -1                  # a skipped row in the middle
    _lib.check(L_.sl_tune(b"attn_mfma", 1), "sl_tune")
    try:
        got = K.sparse_gqa_attn(q.to(DEV), keys.to(DEV), vals.to(DEV), idx.to(DEV)).float().cpu().numpy()
    finally:
        _lib.check(L_.sl_tune(b"attn_mfma", 0), "sl_tune")
    want = orc.sparse_attention(q.float().numpy(), keys.float().numpy(), vals.float().numpy(), idx.numpy())
    assert np.abs(got - want).max() <= TOL[dtype]


def test_sparse_attention_skips_negative_rows_and_head_major(K):
    q, keys, vals, idx = _attn_inputs(_gen(21), 2, 32, 8, 400, 50, torch.float32)
    idx[:, :, 40:] = -1
    kh = keys.permute(0, 2, 1, 3).contiguous()
    vh = vals.permute(0, 2, 1, 3).contiguous()
    got = K.sparse_gqa_attn(q.to(DEV), kh.to(DEV), vh.to(DEV), idx.to(DEV), layout="bhnd").cpu().numpy()
    want = orc.sparse_attention(q.numpy(), keys.numpy(), vals.numpy(), idx.numpy())
    assert np.abs(got - want).max() <= 1e-5


def test_sparse_attention_closed_forms(K):
    g = _gen(22)
    q, keys, vals, idx = _attn_inputs(g, 1, 8, 8, 100, 20, torch.float32)
    # k = 1: the output is the selected V row
    one = idx[:, :, :1].contiguous()
    got = K.sparse_gqa_attn(q.to(DEV), keys.to(DEV), vals.to(DEV), one.to(DEV)).cpu()
    want = torch.stack([vals[0, one[0, h, 0], h] for h in range(8)])[None]
    assert (got - want).abs().max() <= 1e-6
    # identical keys: the output is the mean of the selected V rows
    keys[:] = keys[:, :1]
    got = K.sparse_gqa_attn(q.to(DEV), keys.to(DEV), vals.to(DEV), idx.to(DEV)).cpu()
    want = torch.stack([vals[0, idx[0, h].long(), h].mean(0) for h in range(8)])[None]
    assert (got - want).abs().max() <= 1e-5


def test_sparse_attention_equals_reference_masked_form(K):
    # the reference's literal expression: finfo.min mask + dense SDPA
    q, keys, vals, idx = _attn_inputs(_gen(23), 1, 8, 4, 96, 12, torch.float32)
    got = K.sparse_gqa_attn(q.to(DEV), keys.to(DEV), vals.to(DEV), idx.to(DEV)).cpu()
    want = orc.masked_dense_attention(q, keys, vals, idx.numpy())
    assert (got - want).abs().max() <= 1e-5


# ---- (a) fused hash ----------------------------------------------------------------------

def _hash_weights(g, H, dims, dtype, scale):
    ws = []
    for i in range(len(dims) - 1):
        w = (torch.randn(H, dims[i], dims[i + 1], generator=g) * scale).to(dtype)
        b = (torch.randn(H, dims[i + 1], generator=g) * scale).to(dtype)
        ws.append((w, b))
    return ws


def _flip_report(got_codes, pre64, margin):
    """Bits may differ from the fp64 oracle only where |pre-activation| < margin."""
    want = orc.pack_sign_u32(pre64)
    diff = np.bitwise_xor(got_codes, want)
    bits = ((diff[..., None] >> np.arange(32, dtype=np.uint32)) & 1).reshape(pre64.shape).astype(bool)
    assert (np.abs(pre64[bits]) < margin).all(), f"{bits.sum()} flips, worst |pre|={np.abs(pre64[bits]).max()}"
    return int(bits.sum())


@pytest.mark.parametrize("B,H,d_hid", [(1, 32, 256), (16, 8, 256), (3, 5, 128), (1, 40, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hash_mlp_two_layers(K, B, H, d_hid, dtype):
    g = _gen(B + H + d_hid)
    x = torch.randn(B, H, 128, generator=g).to(dtype)
    # reference init is randn * 0.001 (spotlight_generation.py:232); a larger scale exercises SiLU
    (w1, b1), (w2, b2) = _hash_weights(g, H, [128, d_hid, 128], dtype, 0.05)
    got = K.hash_mlp_pack(x.to(DEV), w1.to(DEV), b1.to(DEV), w2.to(DEV), b2.to(DEV)).cpu().numpy()
    pre = orc.mlp_hash(x.float().numpy(), [(w1.float().numpy(), b1.float().numpy()),
                                           (w2.float().numpy(), b2.float().numpy())], residue=False)
    margin = 1e-5 if dtype == torch.float32 else 2e-2
    flips = _flip_report(got, pre, margin)
    assert flips <= 0.02 * pre.size
    if dtype == torch.bfloat16:
        # against the reference's own torch expression, rounding where torch rounds
        ref = orc.mlp_hash_torch(x.unsqueeze(2), [(w1[None], b1[None, :, None]), (w2[None], b2[None, :, None])],
                                 residue=False).squeeze(2)
        want = orc.pack_sign_u32(ref.float().numpy())
        diff = np.unpackbits(np.bitwise_xor(got, want).view(np.uint8)).sum()
        assert diff <= 0.005 * pre.size


@pytest.mark.parametrize("B,H", [(1, 32), (4, 8)])
def test_hash_mlp_shipped_flavour_bf16_residue_and_biases(K, B, H):
    """The hash function the reference ships (config/llama3-8b-spotlight-generation.json: mlp_dims
    [128,128,128], two layers; mlp_residue defaults to True, spotlight_generation.py:307) in the model's
    dtype, bf16, with non-zero biases as a trained checkpoint has them: the kernel rounds to bf16 after
    the matmul, the bias add, SiLU and the residual add of BOTH layers (spotlight_generation.py:229-255).
    Against the fp64 oracle a bit may differ only where the pre-activation is within 2e-2 of zero;
    against the reference's own bf16 torch expression at most 0.5 % of the bits differ."""
    g = _gen(700 + B + H)
    dtype = torch.bfloat16
    x = torch.randn(B, H, 128, generator=g).to(dtype)
    (w1, b1), (w2, b2) = _hash_weights(g, H, [128, 128, 128], dtype, 0.08)
    got = K.hash_mlp_pack(x.to(DEV), w1.to(DEV), b1.to(DEV), w2.to(DEV), b2.to(DEV), residue=True).cpu().numpy()
    pre = orc.mlp_hash(x.float().numpy(), [(w1.float().numpy(), b1.float().numpy()),
                                           (w2.float().numpy(), b2.float().numpy())], residue=True)
    flips = _flip_report(got, pre, 2e-2)
    assert flips <= 0.02 * pre.size
    ref = orc.mlp_hash_torch(x.unsqueeze(2), [(w1[None], b1[None, :, None]), (w2[None], b2[None, :, None])],
                             residue=True).squeeze(2)
    want = orc.pack_sign_u32(ref.float().numpy())
    diff = np.unpackbits(np.bitwise_xor(got, want).view(np.uint8)).sum()
    assert diff <= 0.005 * pre.size, (int(diff), pre.size)
    # the many-rows kernel (prompt keys) gives the same bits as the decode-step kernel
    rows = K.hash_rows_pack(x[:, None].to(DEV), w1.to(DEV), b1.to(DEV), w2.to(DEV), b2.to(DEV), True).cpu().numpy()
    np.testing.assert_array_equal(rows[:, 0], got)


@pytest.mark.parametrize("dims,dtype", [([128, 256, 128], torch.bfloat16), ([128, 128, 128], torch.float16), ([128, 512, 128], torch.bfloat16),
                                        ([128, 128], torch.float32)])
def test_hash_codes_do_not_depend_on_the_rows_a_workgroup_takes(K, dims, dtype):
    """A workgroup of the hash launch takes 1 to 8 batch rows through the projections together; the
    codes of a row must be the same bits whichever grouping ran, ragged last group included, and equal
    the many-rows kernel's."""
    from spotlight_amd import _lib
    L = _lib.load()
    g = _gen(77)
    B, H = 13, 6
    x = torch.randn(B, H, 128, generator=g).to(dtype).to(DEV)
    layers = _hash_weights(g, H, dims, dtype, 0.08)
    args = [t.to(DEV) for pair in layers for t in pair]
    if len(layers) == 1:
        args = [args[0], args[1], None, None]
    want = None
    try:
        for rows in (1, 2, 3, 4, 6, 8):
            if rows == 8 and dims[1] == 512:
                continue   # no such flavour: its tables exceed the LDS
            _lib.check(L.sl_tune(b"hash_rows", rows), "sl_tune")
            got = K.hash_mlp_pack(x, args[0], args[1], args[2], args[3], residue=False).cpu().numpy()
            if want is None:
                want = got
            np.testing.assert_array_equal(got, want, err_msg=f"{rows} rows per workgroup")
    finally:
        _lib.check(L.sl_tune(b"hash_rows", 0), "sl_tune")
    if len(layers) == 2:
        many = K.hash_rows_pack(x[:, None], args[0], args[1], args[2], args[3], False).cpu().numpy()
        np.testing.assert_array_equal(many[:, 0], want)


def test_hash_mlp_residue_and_no_bias(K):
    g = _gen(31)
    x = torch.randn(2, 8, 128, generator=g)
    (w1, b1), (w2, b2) = _hash_weights(g, 8, [128, 128, 128], torch.float32, 0.05)
    got = K.hash_mlp_pack(x.to(DEV), w1.to(DEV), None, w2.to(DEV), None, residue=True).cpu().numpy()
    z = [np.zeros((8, 128))] * 2
    pre = orc.mlp_hash(x.numpy(), [(w1.numpy(), z[0]), (w2.numpy(), z[1])], residue=True)
    _flip_report(got, pre, 1e-4)


@pytest.mark.parametrize("B", [1, 5])
def test_hash_linear(K, B):
    # training-free linear hashing: x @ L with L ~ N(0,1) per head (linearhashing_generation.py:224-231)
    g = _gen(32)
    x = torch.randn(B, 32, 128, generator=g)
    L = torch.randn(32, 128, 128, generator=g)
    got = K.hash_mlp_pack(x.to(DEV), L.to(DEV), None).cpu().numpy()
    pre = orc.linear_hash(x.numpy(), L.numpy())
    assert _flip_report(got, pre, 1e-4) <= 4


# ---- (d) append ----------------------------------------------------------------------------

def test_cache_append(K):
    g = _gen(41)
    dst = torch.zeros(3, 50, 8, 128, dtype=torch.bfloat16, device=DEV)
    a = torch.randn(3, 7, 8, 128, generator=g).to(torch.bfloat16)
    K.cache_append(dst, a.to(DEV), start=0)
    b = torch.randn(3, 1, 8, 128, generator=g).to(torch.bfloat16)
    lens = torch.tensor([7, 9, 30], dtype=torch.int32, device=DEV)
    K.cache_append(dst, b.to(DEV), start=0, seq_lens=lens)
    out = dst.cpu()
    assert torch.equal(out[:, :7], a)
    for bi, l in enumerate([7, 9, 30]):
        assert torch.equal(out[bi, l], b[bi, 0])
    assert int((out.float().abs().sum(dim=(2, 3)) > 0).sum()) == 3 * 7 + 3   # nothing else was written
