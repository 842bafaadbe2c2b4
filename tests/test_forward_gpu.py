"""The patched attention forward (drop-in for spotlight_generation.py:109-226)
against a CPU restatement of the reference's own forward on the same weights."""
import types

import numpy as np
import pytest
import torch

from oracle import spotlight_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def gen():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd.modifiers import spotlight_generation
    return spotlight_generation


class TinyAttention(torch.nn.Module):
    def __init__(self, QH, KH, d, g):
        super().__init__()
        hidden = QH * d
        self.config = types.SimpleNamespace(num_attention_heads=QH, hidden_size=hidden, num_key_value_heads=KH,
                                            rope_theta=10000.0)
        mk = lambda o, i: torch.nn.Parameter(torch.randn(o, i, generator=g) / i ** 0.5)
        self.q_proj = torch.nn.Linear(hidden, hidden, bias=False)
        self.k_proj = torch.nn.Linear(hidden, KH * d, bias=False)
        self.v_proj = torch.nn.Linear(hidden, KH * d, bias=False)
        self.o_proj = torch.nn.Linear(hidden, hidden, bias=False)
        for lin in (self.q_proj, self.k_proj, self.v_proj, self.o_proj):
            lin.weight = mk(*lin.weight.shape)


def _setup(gen, QH, KH, draft_kwargs, seed, fix=False):
    g = torch.Generator()
    g.manual_seed(seed)
    attn = TinyAttention(QH, KH, 128, g).to(DEV)
    dk = dict(draft_kwargs)
    dk["fix_layers"] = [0] if fix else []
    gen.patch_attention(attn, 0, dk)
    with torch.no_grad():   # non-trivial hash weights (the reference's init gives pre-activations ~1e-3)
        for layer in attn.hash_fn.mlp:
            layer.proj.copy_(torch.randn(layer.proj.shape, generator=g) * 0.08)
            layer.bias.copy_(torch.randn(layer.bias.shape, generator=g) * 0.05)
    return attn, g


def _ref_args(attn):
    c = attn.config
    hw = [(l.proj.data.cpu(), l.bias.data.cpu()) for l in attn.hash_fn.mlp]
    return dict(q_w=attn.q_proj.weight.data.cpu(), k_w=attn.k_proj.weight.data.cpu(),
                v_w=attn.v_proj.weight.data.cpu(), o_w=attn.o_proj.weight.data.cpu(),
                num_heads=c.num_attention_heads, num_kv_heads=c.num_key_value_heads, hash_weights=hw,
                residue=attn.hash_fn.mlp[0].resi, draft_enable=attn.draft_kwargs["enable"] and not attn.is_fix_layer,
                mask_out=attn.draft_kwargs["mask_out"], min_remain=attn.draft_kwargs["min_remain"])


DK = {"enable": True, "mask_out": 0.9, "min_remain": 8, "num_mlp_layers": 2, "mlp_dims": "[128,128,128]",
      "max_cache_len": 256}


@pytest.mark.parametrize("QH,KH,fix", [(4, 4, False), (4, 2, False), (4, 2, True)])
@torch.no_grad()
def test_prefill_and_keep_everything_match_the_reference(gen, QH, KH, fix):
    """With the budget covering every token the draft cannot change the result:
    prefill and decode must equal the reference's forward to fp32 round-off."""
    dk = dict(DK, min_remain=10 ** 6)
    attn, g = _setup(gen, QH, KH, dk, 1, fix)
    ra = _ref_args(attn)
    x = torch.randn(1, 40, QH * 128, generator=g)
    out, cache = attn(x.to(DEV), None)
    ref_out, ref_cache, _ = orc.reference_self_attn_forward(x, None, **ra)
    assert (out.cpu() - ref_out).abs().max() < 2e-4
    for _ in range(3):
        x = torch.randn(1, 1, QH * 128, generator=g)
        out, cache = attn(x.to(DEV), cache)
        ref_out, ref_cache, _ = orc.reference_self_attn_forward(x, ref_cache, **ra)
        assert (out.cpu() - ref_out).abs().max() < 2e-4
    assert cache.length == 43


@pytest.mark.parametrize("QH,KH", [(4, 4), (4, 2)])
@torch.no_grad()
def test_pruned_decode_matches_the_reference_selection(gen, QH, KH):
    """per-query-head mode (no hash_fn_k) is the reference's PyTorch path: the scores
    kept must be the ones torch.topk keeps (indices may differ inside a tie), and the
    output must equal softmax attention over OUR kept set."""
    attn, g = _setup(gen, QH, KH, DK, 2)
    ra = _ref_args(attn)
    x = torch.randn(1, 120, QH * 128, generator=g)
    _, cache = attn(x.to(DEV), None)
    _, ref_cache, _ = orc.reference_self_attn_forward(x, None, **ra)
    for step in range(3):
        x = torch.randn(1, 1, QH * 128, generator=g)
        out, cache = attn(x.to(DEV), cache)
        ref_out, ref_cache, ref_idx = orc.reference_self_attn_forward(x, ref_cache, **ra)
        n = cache.length
        k = orc.num_remain(n, DK["mask_out"], DK["min_remain"])
        st = cache.state
        # the budget is evaluated on the device: an index row is as long as the budget at capacity and
        # holds -1 beyond this step's budget
        full = st.selected().cpu().long()                              # [1, QH, k_cap] (cache kept per query head)
        assert ref_idx.shape[-1] == k and (full[..., :k] >= 0).all() and (full[..., k:] == -1).all()
        ours = full[..., :k]
        # reference scores per query head, recomputed from its cache
        keys_r, vals_r = ref_cache
        hid = x
        d = 128
        sim = _ref_scores(hid, keys_r, ra)
        kept_ours = torch.gather(sim[0, :, 0], 1, ours[0]).sort(dim=1).values
        kept_ref = torch.gather(sim[0, :, 0], 1, ref_idx[0, :, 0]).sort(dim=1).values
        assert torch.equal(kept_ours, kept_ref), step
        strict = sim[0, :, 0] > kept_ref[:, :1]                        # strictly above the threshold: in both sets
        for qh in range(QH):
            must = set(torch.nonzero(strict[qh]).flatten().tolist())
            assert must <= set(ours[0, qh].tolist()) and must <= set(ref_idx[0, qh, 0].tolist())
        # output equals attention over our kept set
        want = orc.sparse_attention(_rope_q(hid, ra, n), _rope_k(keys_r, n).permute(0, 2, 1, 3).numpy(),
                                    vals_r.permute(0, 2, 1, 3).numpy(), ours.numpy().astype(np.int32))
        want = torch.from_numpy(want).float().reshape(1, 1, -1) @ ra["o_w"].T
        assert (out.cpu() - want).abs().max() < 2e-4
        if torch.equal(ours.sort(dim=-1).values, ref_idx[:, :, 0].sort(dim=-1).values):
            assert (out.cpu() - ref_out).abs().max() < 2e-4          # same set -> same output as the reference


def _rope(m, pos):
    d = m.shape[-1]
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = pos.to(torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    rot = torch.cat((-m[..., d // 2:], m[..., : d // 2]), dim=-1)
    return m * emb.cos()[None, None] + rot * emb.sin()[None, None]


def _rope_k(keys_r, n):
    return _rope(keys_r, torch.arange(n))


def _rope_q(hid, ra, n):
    q = (hid @ ra["q_w"].T).unflatten(-1, (ra["num_heads"], 128)).transpose(1, 2)
    return _rope(q, torch.arange(n - 1, n))[:, :, 0].numpy()


def _ref_scores(hid, keys_r, ra):
    n = keys_r.shape[-2]
    q = (hid @ ra["q_w"].T).unflatten(-1, (ra["num_heads"], 128)).transpose(1, 2)
    Q = _rope(q, torch.arange(n - 1, n))
    Kr = _rope_k(keys_r, n)
    return orc.sign_matmul_score(orc.mlp_hash_torch(Q, ra["hash_weights"], ra["residue"]),
                                 orc.mlp_hash_torch(Kr, ra["hash_weights"], ra["residue"]))


@torch.no_grad()
def test_gqa_key_hash_mode_runs_batched(gen):
    """hash_fn_k present: codes per kv head, any batch size, bf16."""
    g = torch.Generator()
    g.manual_seed(3)
    attn = TinyAttention(8, 2, 128, g).to(DEV).to(torch.bfloat16)
    gen.patch_attention(attn, 2, dict(DK, fix_layers=[0, 1]), gqa_key_hash=True)
    x = torch.randn(3, 64, 8 * 128, generator=g).to(torch.bfloat16)
    out, cache = attn(x.to(DEV), None)
    assert out.shape == (3, 64, 1024) and cache.state.KH == 2
    for _ in range(2):
        x = torch.randn(3, 1, 8 * 128, generator=g).to(torch.bfloat16)
        out, cache = attn(x.to(DEV), cache)
    n = cache.length
    assert n == 66 and cache.state.seq_lens.cpu().tolist() == [66] * 3
    k = orc.num_remain(n, 0.9, 8)
    idx = cache.state.selected().cpu().numpy()
    assert (idx[..., k:] == -1).all()          # beyond the budget the device evaluated for n rows
    idx = idx[..., :k]
    assert idx.shape == (3, 2, k) and (np.diff(idx, axis=-1) > 0).all() and idx.max() < n and idx.min() >= 0
    assert torch.isfinite(out.float()).all()
