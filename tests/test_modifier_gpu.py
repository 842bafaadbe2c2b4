"""The modifier layer (drop-in for spotlight/modifiers/spotlight_generation.py:258-495,
spotlight/modifier.py:21-88, spotlight/modifiers/__init__.py): a tiny Llama-shaped
model goes through ``get_modifier`` -> ``Spotlight(model, save_ckp, load_ckp, config)``
-> ``generate`` and is checked against a CPU loop built on the oracle's restatement
of the reference's attention forward."""
import copy
import types

import pytest
import torch

from oracle import spotlight_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128


class RMSNorm(torch.nn.Module):
    def __init__(self, hidden):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.ones(hidden))

    def forward(self, x):
        return self.weight * x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)


class TinyAttention(torch.nn.Module):
    def __init__(self, cfg):
        super().__init__()
        self.config = cfg
        h, kv = cfg.hidden_size, cfg.num_key_value_heads * D
        self.q_proj = torch.nn.Linear(h, h, bias=False)
        self.k_proj = torch.nn.Linear(h, kv, bias=False)
        self.v_proj = torch.nn.Linear(h, kv, bias=False)
        self.o_proj = torch.nn.Linear(h, h, bias=False)


class TinyLayer(torch.nn.Module):
    def __init__(self, cfg):
        super().__init__()
        self.self_attn = TinyAttention(cfg)
        self.input_layernorm = RMSNorm(cfg.hidden_size)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size)
        self.mlp = torch.nn.Sequential(torch.nn.Linear(cfg.hidden_size, 256, bias=False), torch.nn.SiLU(),
                                       torch.nn.Linear(256, cfg.hidden_size, bias=False))


class TinyInner(torch.nn.Module):
    def __init__(self, cfg, n_layers):
        super().__init__()
        self.embed_tokens = torch.nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = torch.nn.ModuleList([TinyLayer(cfg) for _ in range(n_layers)])
        self.norm = RMSNorm(cfg.hidden_size)


class TinyLM(torch.nn.Module):
    def __init__(self, QH, KH, n_layers, vocab=97, seed=0):
        super().__init__()
        torch.manual_seed(seed)
        self.config = types.SimpleNamespace(num_attention_heads=QH, hidden_size=QH * D, num_key_value_heads=KH,
                                            rope_theta=10000.0, vocab_size=vocab)
        self.model = TinyInner(self.config, n_layers)
        self.lm_head = torch.nn.Linear(QH * D, vocab, bias=False)


@pytest.fixture(scope="module")
def mods():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd.modifiers import get_modifier
    return get_modifier


CONF = {"draft_kwargs": {"enable": True, "fix_layers": [0], "mask_out": 0.9, "bench_mark": False, "min_remain": 8,
                         "num_mlp_layers": 2, "mlp_dims": "[128,128,128]", "max_cache_len": 256}}


def _wrap(mods, method, base, conf, load_ckp=None, save_ckp=None, seed=5):
    _, cls = mods(method)
    m = cls(base.to(DEV), save_ckp, load_ckp, copy.deepcopy(conf))
    if load_ckp is None:   # non-trivial hash weights (the reference's init gives pre-activations ~1e-3)
        g = torch.Generator()
        g.manual_seed(seed)
        with torch.no_grad():
            for p in m.ft_params():
                p.copy_((torch.randn(p.shape, generator=g) * 0.08).to(p.device))
    return m.eval()


def _ref_generate(base_cpu, hash_params, conf, ids, steps):
    """Greedy loop of spotlight_generation.py:470-495 over the reference attention
    forward (oracle), fp32 on the CPU.  Returns tokens and per-step last logits."""
    dk = conf["draft_kwargs"]
    cfg = base_cpu.config
    caches = [None] * len(base_cpu.model.layers)

    def forward(tok):
        x = base_cpu.model.embed_tokens(tok)
        for i, lay in enumerate(base_cpu.model.layers):
            a = lay.self_attn
            out, caches[i], _ = orc.reference_self_attn_forward(
                lay.input_layernorm(x), caches[i], q_w=a.q_proj.weight, k_w=a.k_proj.weight, v_w=a.v_proj.weight,
                o_w=a.o_proj.weight, num_heads=cfg.num_attention_heads, num_kv_heads=cfg.num_key_value_heads,
                hash_weights=hash_params[i], residue=dk.get("mlp_residue", True),
                draft_enable=dk["enable"] and i not in dk["fix_layers"], mask_out=dk["mask_out"],
                min_remain=dk["min_remain"])
            x = x + out
            x = x + lay.mlp(lay.post_attention_layernorm(x))
        return base_cpu.lm_head(base_cpu.model.norm(x)[..., -1:, :]).float()

    logits = [forward(ids)]
    toks = []
    for _ in range(steps):
        nxt = logits[-1][:, -1:].argmax(dim=-1)
        toks.append(nxt)
        logits.append(forward(nxt))
    return torch.cat(toks, dim=-1), logits


def _hash_params_cpu(m):
    out = []
    for ps in m.layer_ft_params():
        ps = [p.detach().cpu() for p in ps]
        out.append([(ps[j], ps[j + 1]) for j in range(0, len(ps), 2)])
    return out


@pytest.mark.parametrize("QH,KH", [(2, 2), (4, 2)])
@torch.no_grad()
def test_generate_matches_reference_loop_when_nothing_is_pruned(mods, QH, KH):
    """Budget >= context: the draft cannot change anything, so tokens and logits must
    equal the reference's loop (dense layer 0, sparse layers 1-2)."""
    conf = copy.deepcopy(CONF)
    conf["draft_kwargs"]["min_remain"] = 10 ** 6
    base = TinyLM(QH, KH, 3)
    base_cpu = copy.deepcopy(base)
    m = _wrap(mods, "spotlight-generation", base, conf)
    ids = torch.randint(0, 97, (1, 37), generator=torch.Generator().manual_seed(1))
    want_toks, want_logits = _ref_generate(base_cpu, _hash_params_cpu(m), conf, ids, 6)
    got = m.generate(ids, max_new_tokens=6, eos_token_id=[-1])
    assert got.shape == (1, 43) and torch.equal(got[:, :37].cpu(), ids)
    assert torch.equal(got[:, 37:].cpu(), want_toks)
    out = m(input_ids=ids)
    assert out.logits.shape == (1, 1, 97) and out.logits.dtype == torch.float32 and out.loss is None
    assert (out.logits.cpu() - want_logits[0]).abs().max() < 2e-3
    assert len(out.past_key_values) == 3 and out.past_key_values[0].state is None     # layer 0 is dense
    assert out.past_key_values[1].state is not None


@torch.no_grad()
def test_pruned_generate_runs_the_sparse_step_and_matches_manual_loop(mods):
    base = TinyLM(4, 2, 3, seed=2)
    m = _wrap(mods, "spotlight-generation", base, CONF)
    ids = torch.randint(0, 97, (1, 120), generator=torch.Generator().manual_seed(3))
    got = m.generate(ids, max_new_tokens=5, eos_token_id=[-1])
    # the same loop by hand through the public forward
    out = m(input_ids=ids.to(DEV))
    toks = []
    for step in range(5):
        nxt = out.logits[:, -1:].argmax(dim=-1)
        toks.append(nxt)
        out = m(input_ids=nxt, kv_cache=out.past_key_values)
        st = out.past_key_values[1].state
        n = 120 + step + 1
        k = orc.num_remain(n, 0.9, 8)
        idx = st.selected()
        assert out.past_key_values[1].length == n and (idx[..., k:] == -1).all()   # the device's budget for n rows
        assert int(idx[..., :k].max()) < n and int(idx[..., :k].min()) >= 0
    assert torch.equal(got[:, 120:], torch.cat(toks, dim=-1))


@torch.no_grad()
def test_eos_stops_generation_like_the_reference(mods):
    base = TinyLM(2, 2, 2, seed=4)
    m = _wrap(mods, "spotlight-generation", base, CONF)
    ids = torch.randint(0, 97, (1, 20), generator=torch.Generator().manual_seed(5))
    free = m.generate(ids, max_new_tokens=4, eos_token_id=[-1])
    stop_at = int(free[0, 22])                      # third generated token becomes "eos"
    first = free[0, 20:].tolist().index(stop_at)
    got = m.generate(ids, max_new_tokens=4, eos_token_id=[stop_at])
    assert got.shape[1] == 20 + first and torch.equal(got, free[:, :20 + first])   # eos itself is not appended


@torch.no_grad()
def test_checkpoint_round_trip_and_training_layout(mods, tmp_path):
    from spotlight_amd.modifier import read_checkpoint, write_checkpoint
    base = TinyLM(4, 2, 3, seed=6)
    base2 = copy.deepcopy(base)
    base3 = copy.deepcopy(base)
    m = _wrap(mods, "spotlight-generation", base, CONF)
    path = str(tmp_path / "hash.pth")
    m.save_checkpoint(path)
    ck = read_checkpoint(path)
    assert len(ck) == 3 * 4 and ck[0].shape == (1, 4, 128, 128) and ck[1].shape == (1, 4, 1, 128)
    ids = torch.randint(0, 97, (1, 100), generator=torch.Generator().manual_seed(7))
    want = m.generate(ids, max_new_tokens=4, eos_token_id=[-1])
    m2 = _wrap(mods, "spotlight-generation", base2, CONF, load_ckp=path)
    for a, b in zip(m.ft_params(), m2.ft_params()):
        assert torch.equal(a, b)
    assert torch.equal(m2.generate(ids, max_new_tokens=4, eos_token_id=[-1]), want)
    # the training modifier's list leaves the dense layer out (spotlight_train.py:412-419)
    train_path = str(tmp_path / "train.pth")
    write_checkpoint(ck[4:], train_path)
    m3 = _wrap(mods, "spotlight-generation", base3, CONF, load_ckp=train_path)
    for a, b in zip(m.ft_params()[4:], m3.ft_params()[4:]):
        assert torch.equal(a, b)
    assert torch.equal(m3.generate(ids, max_new_tokens=4, eos_token_id=[-1]), want)   # layer 0 never hashes
    bad = str(tmp_path / "bad.pth")
    write_checkpoint(ck[:5], bad)
    with pytest.raises(ValueError):
        m3.load_checkpoint(bad)


@torch.no_grad()
def test_linear_hashing_modifier(mods):
    conf = {"draft_kwargs": {"enable": True, "fix_layers": [0], "mask_out": 0.9, "bench_mark": False,
                             "min_remain": 8, "max_cache_len": 256}}
    base = TinyLM(2, 2, 2, seed=8)
    _, cls = mods("linearhashing-generation")
    m = cls(base.to(DEV), None, None, conf).eval()
    assert [tuple(p.shape) for p in m.ft_params()] == [(1, 2, 128, 128)] * 2
    ids = torch.randint(0, 97, (1, 90), generator=torch.Generator().manual_seed(9))
    got = m.generate(ids, max_new_tokens=3, eos_token_id=[-1])
    assert got.shape == (1, 93)
    out = m(input_ids=ids.to(DEV))
    out = m(input_ids=got[:, 90:91], kv_cache=out.past_key_values)
    sel = out.past_key_values[1].state.selected()
    k = orc.num_remain(91, 0.9, 8)
    assert (sel[..., :k] >= 0).all() and (sel[..., k:] == -1).all()
    with pytest.raises(NotImplementedError):
        mods("upperbound-generation")


@torch.no_grad()
def test_benchmark_mode_reports_iou_per_layer_and_head(mods):
    conf = copy.deepcopy(CONF)
    conf["draft_kwargs"]["bench_mark"] = True
    base = TinyLM(4, 2, 3, seed=10)
    m = _wrap(mods, "spotlight-generation", base, conf)
    assert m.is_benchmark_mode()
    ids = torch.randint(0, 97, (1, 150), generator=torch.Generator().manual_seed(11))
    out = m(input_ids=ids.to(DEV))
    out = m(input_ids=ids[:, :1].to(DEV), kv_cache=out.past_key_values)
    ratios = m.model.decoder.get_ratios(reset=True)
    assert ratios[0] is None and len(ratios[1]) == 4 and len(ratios[2]) == 4
    assert all(0.0 <= r <= 1.0 for row in ratios[1:] for r in row)
    assert m.model.decoder.get_ratios() == [None, None, None]         # consumed
    # a budget that covers the whole context selects what the true scores select
    conf["draft_kwargs"]["min_remain"] = 10 ** 6
    m2 = _wrap(mods, "spotlight-generation", TinyLM(4, 2, 3, seed=10), conf)
    out = m2(input_ids=ids.to(DEV))
    m2(input_ids=ids[:, :1].to(DEV), kv_cache=out.past_key_values)
    assert all(r == 1.0 for row in m2.model.decoder.get_ratios()[1:] for r in row)
    m2.disable_benchmark_mode()
    assert not m2.is_benchmark_mode()


@torch.no_grad()
def test_chunked_prefill_equals_one_shot_prefill(mods):
    """A prompt fed in two chunks (the second behind a non-empty cache) must leave the same cache
    -- rows and codes -- as the prompt fed at once, in dense and in sparse layers, and decode the
    same tokens afterwards.  The reference's forward treats a chunk the same way
    (spotlight_generation.py:131-136: concatenate, mask by position)."""
    base = TinyLM(4, 2, 3, seed=12)
    m = _wrap(mods, "spotlight-generation", base, CONF)
    ids = torch.randint(0, 97, (1, 90), generator=torch.Generator().manual_seed(13)).to(DEV)
    whole = m(input_ids=ids)
    part = m(input_ids=ids[:, :60])
    part = m(input_ids=ids[:, 60:], kv_cache=part.past_key_values)
    assert (whole.logits - part.logits).abs().max() < 2e-3
    for a, b in zip(whole.past_key_values, part.past_key_values):
        assert a.length == b.length == 90
        assert (a.keys[:, :90].float() - b.keys[:, :90].float()).abs().max() < 1e-4
        if a.state is not None:
            same = (a.state.codes[:, :90].view(torch.int32) == b.state.codes[:, :90].view(torch.int32)).float().mean()
            assert float(same) > 0.999       # a code word may differ where a pre-activation is ~0
            assert a.state.seq_lens.tolist() == b.state.seq_lens.tolist() == [90]
    for _ in range(3):
        nxt = whole.logits[:, -1:].argmax(dim=-1)
        assert torch.equal(nxt, part.logits[:, -1:].argmax(dim=-1))
        whole = m(input_ids=nxt, kv_cache=whole.past_key_values)
        part = m(input_ids=nxt, kv_cache=part.past_key_values)
        assert (whole.logits - part.logits).abs().max() < 2e-3


@pytest.mark.parametrize("B,gqa", [(1, False), (3, True)])
@torch.no_grad()
def test_generate_replaying_its_captured_token_equals_eager_generate(mods, B, gqa):
    """generate() decodes its first token eagerly and replays one captured HIP graph for the rest
    (positions, lengths and the budget are read from the device).  With the graph switched off
    (draft_kwargs["hip_graph"] = False) every token runs eagerly: both must emit the same tokens, over
    a stretch in which the budget changes several times, for batch 1 and for a batch with the
    per-kv-head key hash."""
    conf = copy.deepcopy(CONF)
    conf["draft_kwargs"].update(max_cache_len=0, gqa_key_hash=gqa)
    eager_conf = copy.deepcopy(conf)
    eager_conf["draft_kwargs"]["hip_graph"] = False
    base = TinyLM(4, 2, 3, seed=11)
    base2 = copy.deepcopy(base)
    m = _wrap(mods, "spotlight-generation", base, conf, seed=12)
    e = _wrap(mods, "spotlight-generation", base2, eager_conf, seed=12)
    ids = torch.randint(0, 97, (B, 150), generator=torch.Generator().manual_seed(13))
    got = m.generate(ids, max_new_tokens=40, eos_token_id=[-1])
    want = e.generate(ids, max_new_tokens=40, eos_token_id=[-1])
    assert got.shape == (B, 190) and torch.equal(got, want)
    assert m.timing["graph_tokens"] == 39 and e.timing["graph_tokens"] == 0
    assert {orc.num_remain(n, 0.9, 8) for n in range(151, 191)} >= {16, 17, 18, 19}   # the budget moved under the graph


@torch.no_grad()
def test_generate_recovers_when_a_bounded_wait_runs_out(mods):
    """A prompt long enough for two blocks of rows per head, so that the one-launch step exchanges
    histograms; every such exchange is made to fail from the host (a peer that does not exist, a short
    poll limit).  generate() sees the error word at its per-token read of the device, moves every layer
    to token-major codes, takes the token back and decodes it again: the output must equal an
    undisturbed run's."""
    from spotlight_amd import _lib
    L = _lib.load()
    conf = copy.deepcopy(CONF)
    conf["draft_kwargs"].update(max_cache_len=0)
    base = TinyLM(4, 2, 3, seed=21)
    base2 = copy.deepcopy(base)
    m = _wrap(mods, "spotlight-generation", base, conf, seed=22)
    m2 = _wrap(mods, "spotlight-generation", base2, conf, seed=22)
    ids = torch.randint(0, 97, (1, 700), generator=torch.Generator().manual_seed(23))
    want = m.generate(ids, max_new_tokens=6, eos_token_id=[-1])
    _lib.check(L.sl_tune(b"fused_spin_limit", 64), "sl_tune")
    _lib.check(L.sl_tune(b"fused_phantom_peer", 1), "sl_tune")
    try:
        got = m2.generate(ids, max_new_tokens=6, eos_token_id=[-1])
    finally:
        _lib.check(L.sl_tune(b"fused_spin_limit", 0), "sl_tune")
        _lib.check(L.sl_tune(b"fused_phantom_peer", 0), "sl_tune")
    assert torch.equal(got, want)
    # one failure (the first decoded token), one recovery; the graph captured afterwards runs on token-major codes
    assert m2.timing["recoveries"] == 1 and m.timing["recoveries"] == 0
