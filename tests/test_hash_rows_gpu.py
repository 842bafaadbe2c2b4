"""The many-rows hash kernel (codes of the keys a prompt leaves in the cache): bit-identical to
the decode step's hash, whichever of the two a vector goes through, and within the stated
margin of the fp64 oracle.  The reference hashes keys and query with one function
(spotlight_generation.py:14-17,229-255), so a key's code cannot depend on how it arrived."""
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
    return decode, kernel


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def _weights(g, H, dims, dtype, scale, bias=True):
    ws = []
    for i in range(len(dims) - 1):
        w = (torch.randn(H, dims[i], dims[i + 1], generator=g) * scale).to(dtype).to(DEV)
        b = (torch.randn(H, dims[i + 1], generator=g) * 0.1).to(dtype).to(DEV) if bias else None
        ws += [w, b]
    return ws


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("d_hid", [64, 128, 256, 512])
def test_two_layer_rows_equal_the_decode_hash_bit_for_bit(env, dtype, d_hid):
    decode, K = env
    g = _gen(d_hid)
    B, n, H = 2, 1030, 3                      # not a multiple of the row tile
    x = torch.randn(B, n, H, 128, generator=g).to(dtype).to(DEV)
    w1, b1, w2, b2 = _weights(g, H, [128, d_hid, 128], dtype, 0.05)
    got = K.hash_rows_pack(x, w1, b1, w2, b2)
    want = K.hash_mlp_pack(x.reshape(B * n, H, 128), w1, b1, w2, b2).reshape(B, n, H, 4)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    # and against the fp64 oracle: bits may differ only where the pre-activation is within the margin of zero
    pre = orc.mlp_hash(x.reshape(B * n, H, 128).float().cpu().numpy(),
                       [(w1.float().cpu().numpy(), b1.float().cpu().numpy()), (w2.float().cpu().numpy(), b2.float().cpu().numpy())], False)
    bits = np.unpackbits(got.reshape(B * n, H, 4).cpu().numpy().view(np.uint8), bitorder="little").reshape(B * n, H, 128)
    wrong = bits != (pre > 0)
    margin = 1e-5 if dtype == torch.float32 else 2e-2
    assert not (wrong & (np.abs(pre) > margin)).any()


@pytest.mark.parametrize("kind", ["linear", "residue", "nobias", "linear64"])
def test_other_flavours_equal_the_decode_hash(env, kind):
    decode, K = env
    g = _gen(7)
    H = 5
    x = torch.randn(1, 777, H, 128, generator=g).to(DEV)
    if kind == "linear":      # one layer, nbits = 128 (linearhashing_generation.py:224-231)
        args = (torch.randn(H, 128, 128, generator=g).to(DEV), None, None, None, False)
    elif kind == "linear64":
        args = (torch.randn(H, 128, 64, generator=g).to(DEV), None, None, None, False)
    elif kind == "residue":   # mlp_residue = True needs equal widths (spotlight_generation.py:240)
        args = (*_weights(g, H, [128, 128, 128], torch.float32, 0.05), True)
    else:
        w1, _, w2, _ = _weights(g, H, [128, 256, 128], torch.float32, 0.05, bias=False)
        args = (w1, None, w2, None, False)
    got = K.hash_rows_pack(x, *args)
    want = K.hash_mlp_pack(x[0], *args)
    assert torch.equal(got[0].view(torch.int32), want.view(torch.int32))


def test_codes_do_not_depend_on_how_a_key_arrived(env):
    """4096 keys hashed with the prompt == the same keys fed one by one through decode steps."""
    decode, K = env
    dtype = torch.bfloat16
    g = _gen(11)
    QH, KH, n = 8, 2, 4096
    hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    keys = torch.randn(1, n, KH, 128, generator=g).to(dtype).to(DEV)
    vals = torch.randn(1, n, KH, 128, generator=g).to(dtype).to(DEV)
    by_prompt = decode.LayerDecodeState(1, QH, KH, 128, n + 8, 4, hq, hk, dtype=dtype, device=DEV)
    by_prompt.prefill(keys, vals)
    by_step = decode.LayerDecodeState(1, QH, KH, 128, n + 8, 4, hq, hk, dtype=dtype, device=DEV)
    q = torch.randn(1, QH, 128, generator=g).to(dtype).to(DEV)
    for t in range(n):
        by_step.step(q, keys[:, t], vals[:, t])
    torch.cuda.synchronize()
    assert by_step.seq_lens.tolist() == [n]
    assert torch.equal(by_step.keys[:, :n], by_prompt.keys[:, :n])
    assert torch.equal(by_step.codes[:, :n].view(torch.int32), by_prompt.codes[:, :n].view(torch.int32))


def test_rows_written_into_a_strided_destination(env):
    decode, K = env
    g = _gen(12)
    H = 4
    w1, b1, w2, b2 = _weights(g, H, [128, 256, 128], torch.bfloat16, 0.05)
    cache = torch.zeros(3, 64, H, 4, dtype=torch.int32, device=DEV).view(torch.uint32)
    x = torch.randn(3, 20, H, 128, generator=g).to(torch.bfloat16).to(DEV)
    K.hash_rows_pack(x, w1, b1, w2, b2, out=cache[:, 10:30])
    want = K.hash_rows_pack(x, w1, b1, w2, b2)
    c = cache.view(torch.int32)
    assert torch.equal(c[:, 10:30], want.view(torch.int32))
    assert int(c[:, :10].abs().sum()) == 0 and int(c[:, 30:].abs().sum()) == 0
