"""Parity of the fused decode step (hash -> score -> top-k -> (LRU) -> attention)
and of the LRU resident table against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import spotlight_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


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


def _make_state(decode, g, B, QH, KH, n0, n_cap, k, dtype, kind="mlp", lru=0, scale=0.05, head_map="blocked",
                codes_layout="auto"):
    if kind == "mlp":
        hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, g, scale=scale)
        hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, g, scale=scale)
    else:
        hq = decode.HashWeights.random_linear(QH, 128, 128, dtype, DEV, g)
        hk = hq if KH == QH else decode.HashWeights.random_linear(KH, 128, 128, dtype, DEV, g)
    st = decode.LayerDecodeState(B, QH, KH, 128, n_cap, k, hq, hk, dtype=dtype, device=DEV,
                                 head_map=head_map, lru_slots=lru, codes_layout=codes_layout)
    keys = torch.randn(B, n0, KH, 128, generator=g).to(dtype)
    vals = torch.randn(B, n0, KH, 128, generator=g).to(dtype)
    st.prefill(keys.to(DEV), vals.to(DEV))
    return st


def _check_step(kernel, st, q, k_new, v_new, out, n_before, dtype):
    """Everything the step produced, checked against the oracle on the codes the GPU holds."""
    B, QH, KH = st.B, st.QH, st.KH
    n = n_before + 1
    hq = st.hash_q
    q_code = kernel.hash_mlp_pack(q.to(DEV), hq.w1, hq.b1, hq.w2, hq.b2, hq.residue).cpu().numpy()[:, None]
    codes = st.codes[:, :n].cpu().numpy()
    keys = st.keys[:, :n].float().cpu().numpy()
    vals = st.vals[:, :n].float().cpu().numpy()
    # appended row
    np.testing.assert_array_equal(keys[:, n - 1], k_new.float().numpy())
    np.testing.assert_array_equal(vals[:, n - 1], v_new.float().numpy())
    hk = st.hash_k
    k_code = kernel.hash_mlp_pack(k_new.to(DEV), hk.w1, hk.b1, hk.w2, hk.b2, hk.residue).cpu().numpy()
    np.testing.assert_array_equal(codes[:, n - 1], k_code)
    assert st.seq_lens.cpu().tolist() == [n] * B
    # selection: bit exact
    score = orc.hamming_score_u32(q_code, codes, st.head_map)
    want_idx = orc.topk_stable(score, st.k)
    got_idx = st.idx.cpu().numpy()
    kk = want_idx.shape[2]
    np.testing.assert_array_equal(got_idx[:, :, :kk], want_idx)
    assert (got_idx[:, :, kk:] == -1).all()
    # attention
    want = orc.sparse_attention(q.float().numpy(), keys, vals, want_idx)
    err = np.abs(out.float().cpu().numpy() - want).max()
    assert err <= TOL[dtype], err
    assert not st.peer_wait_failed()


DECODE_CASES = [
    # B, QH, KH, n0, k, dtype, kind
    (1, 32, 8, 1000, 20, torch.bfloat16, "mlp"),
    (1, 32, 8, 2047, 41, torch.float32, "mlp"),
    (2, 40, 8, 777, 16, torch.bfloat16, "mlp"),
    (1, 32, 32, 512, 52, torch.float32, "linear"),     # Llama-2 shape, training-free hash (config 1 style)
    (3, 28, 4, 300, 30, torch.float16, "mlp"),
    (1, 8, 8, 5, 20, torch.float32, "mlp"),            # fewer tokens than k
]


@pytest.mark.parametrize("layout", ["auto", "token"])
@pytest.mark.parametrize("B,QH,KH,n0,k,dtype,kind", DECODE_CASES)
def test_decode_step_matches_oracle(env, B, QH, KH, n0, k, dtype, kind, layout):
    decode, kernel = env
    g = _gen(n0 + k)
    st = _make_state(decode, g, B, QH, KH, n0, 2048 + 64, k, dtype, kind, codes_layout=layout)
    for step in range(3):
        q = torch.randn(B, QH, 128, generator=g).to(dtype)
        k_new = torch.randn(B, KH, 128, generator=g).to(dtype)
        v_new = torch.randn(B, KH, 128, generator=g).to(dtype)
        out = st.step(q.to(DEV), k_new.to(DEV), v_new.to(DEV))
        _check_step(kernel, st, q, k_new, v_new, out, n0 + step, dtype)


def test_decode_step_interleaved_head_map(env):
    decode, kernel = env
    g = _gen(77)
    st = _make_state(decode, g, 1, 28, 4, 400, 512, 25, torch.bfloat16, head_map="interleaved")
    q = torch.randn(1, 28, 128, generator=g).to(torch.bfloat16)
    kn = torch.randn(1, 4, 128, generator=g).to(torch.bfloat16)
    vn = torch.randn(1, 4, 128, generator=g).to(torch.bfloat16)
    out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV))
    _check_step(kernel, st, q, kn, vn, out, 400, torch.bfloat16)


def test_decode_ragged_batch(env):
    """Sequences of different lengths in one batch (lengths live on the device)."""
    decode, kernel = env
    g = _gen(78)
    B, QH, KH, k = 3, 32, 8, 24
    st = _make_state(decode, g, B, QH, KH, 600, 1024, k, torch.float32)
    lens = [600, 77, 333]
    st.seq_lens.copy_(torch.tensor(lens, dtype=torch.int32))
    q = torch.randn(B, QH, 128, generator=g)
    kn = torch.randn(B, KH, 128, generator=g)
    vn = torch.randn(B, KH, 128, generator=g)
    out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).cpu().numpy()
    hq = st.hash_q
    q_code = kernel.hash_mlp_pack(q.to(DEV), hq.w1, hq.b1, hq.w2, hq.b2).cpu().numpy()[:, None]
    assert st.seq_lens.cpu().tolist() == [l + 1 for l in lens]
    for b, l in enumerate(lens):
        n = l + 1
        codes = st.codes[b:b + 1, :n].cpu().numpy()
        score = orc.hamming_score_u32(q_code[b:b + 1], codes, "blocked")
        want_idx = orc.topk_stable(score, k)
        np.testing.assert_array_equal(st.idx[b:b + 1].cpu().numpy(), want_idx)
        want = orc.sparse_attention(q[b:b + 1].numpy(), st.keys[b:b + 1, :n].cpu().numpy(),
                                    st.vals[b:b + 1, :n].cpu().numpy(), want_idx)
        assert np.abs(out[b:b + 1] - want).max() <= 1e-5


@pytest.mark.parametrize("lru,layout", [(0, "auto"), (0, "token"), (64, "token"), (64, "head")])
def test_decode_graph_replay_equals_eager(env, lru, layout):
    """A captured step replayed while the cache grows gives what eager steps give
    (also with the LRU table, whose misses the attention launch fetches)."""
    decode, kernel = env
    dtype = torch.bfloat16
    states = [_make_state(decode, _gen(90), 2, 32, 8, 500, 640, 30, dtype, lru=lru, codes_layout=layout) for _ in range(2)]
    eager, graphed = states
    graphed.capture(steps_ahead=8)
    g = _gen(91)
    for step in range(6):
        q = torch.randn(2, 32, 128, generator=g).to(dtype).to(DEV)
        kn = torch.randn(2, 8, 128, generator=g).to(dtype).to(DEV)
        vn = torch.randn(2, 8, 128, generator=g).to(dtype).to(DEV)
        a = eager.step(q, kn, vn).clone()
        graphed.q_in.copy_(q); graphed.k_in.copy_(kn); graphed.v_in.copy_(vn)
        b = graphed.replay().clone()
        torch.cuda.synchronize()
        assert torch.equal(eager.idx, graphed.idx), step
        assert torch.equal(a, b), step
        assert torch.equal(eager.seq_lens, graphed.seq_lens)
        if lru:
            assert torch.equal(eager.slot_token, graphed.slot_token) and torch.equal(eager.k_res, graphed.k_res)
            assert torch.equal(eager.v_res, graphed.v_res)
    with pytest.raises(RuntimeError):
        for _ in range(5):
            graphed.replay()


def test_decode_is_deterministic(env):
    decode, kernel = env
    outs = []
    for _ in range(2):
        g = _gen(95)
        st = _make_state(decode, g, 1, 32, 8, 3000, 3072, 60, torch.bfloat16)
        q = torch.randn(1, 32, 128, generator=g).to(torch.bfloat16)
        kn = torch.randn(1, 8, 128, generator=g).to(torch.bfloat16)
        vn = torch.randn(1, 8, 128, generator=g).to(torch.bfloat16)
        outs.append((st.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).clone(), st.idx.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


# ---- LRU ---------------------------------------------------------------------------------

def _lru_call(kernel, lib, L, idx, new_tok, st, ss, ts, keys, vals, kres, vres, stamp):
    B, KH, k = idx.shape
    C = st.shape[2]
    slots = torch.full((B, KH, k), -7, dtype=torch.int32, device=DEV)
    stats = torch.zeros((B, KH, 2), dtype=torch.int32, device=DEV)
    rc = L.sl_lru_update(idx.data_ptr(), new_tok.data_ptr(), st.data_ptr(), ss.data_ptr(), ts.data_ptr(),
                         keys.data_ptr(), vals.data_ptr(), kres.data_ptr(), vres.data_ptr(), slots.data_ptr(),
                         stats.data_ptr(), kernel._DTYPES[keys.dtype], B, KH, keys.shape[3], k, C, ts.shape[2],
                         keys.stride(0), stamp, None, torch.cuda.current_stream().cuda_stream)
    lib.check(rc, "sl_lru_update")
    return slots, stats


# `scale` spreads the stamps: with 1 every age stays small (the victims' threshold comes from the age
# histogram), with 700 the oldest slots are older than the histogram resolves (the select on the stamp runs)
@pytest.mark.parametrize("scale", [1, 700])
@pytest.mark.parametrize("C,k,n0,steps", [(8, 3, 12, 40), (64, 20, 100, 30), (1024, 328, 2000, 6), (4096, 1000, 5000, 3)])
def test_lru_matches_bruteforce_model(env, C, k, n0, steps, scale):
    decode, kernel = env
    from spotlight_amd import _lib as lib
    L = lib.load()
    r = np.random.default_rng(C + k)
    B, KH, d = 2, 3, 128
    cap = n0 + steps + 1
    keys = torch.randn(B, cap, KH, d, generator=_gen(1)).to(torch.bfloat16).to(DEV)
    vals = torch.randn(B, cap, KH, d, generator=_gen(2)).to(torch.bfloat16).to(DEV)
    st = torch.full((B, KH, C), -1, dtype=torch.int32, device=DEV)
    ss = torch.zeros((B, KH, C), dtype=torch.int32, device=DEV)
    ts = torch.full((B, KH, cap), -1, dtype=torch.int32, device=DEV)
    kres = torch.zeros((B, KH, C, d), dtype=torch.bfloat16, device=DEV)
    vres = torch.zeros_like(kres)
    models = [[orc.LruModel(C) for _ in range(KH)] for _ in range(B)]
    n = n0
    for step in range(1, steps + 1):
        t = step * scale
        idx = np.zeros((B, KH, k), dtype=np.int32)
        for b in range(B):
            for h in range(KH):
                sel = r.choice(n, size=k, replace=False)
                res = [x for x in models[b][h].token if x >= 0]
                if res and step % 2 == 0:      # re-use resident tokens so that hits occur
                    take = min(len(res), k // 2)
                    sel = np.unique(np.concatenate([r.choice(res, size=take, replace=False), sel]))[:k]
                    while len(sel) < k:
                        sel = np.unique(np.concatenate([sel, r.choice(n, size=k)]))[:k]
                idx[b, h] = np.sort(sel)
        new_tok = torch.full((B,), n, dtype=torch.int32, device=DEV)
        slots, stats = _lru_call(kernel, lib, L, torch.from_numpy(idx).to(DEV), new_tok, st, ss, ts, keys, vals,
                                 kres, vres, t)
        slots = slots.cpu().numpy()
        st_h, ss_h, ts_h = st.cpu().numpy(), ss.cpu().numpy(), ts.cpu().numpy()
        stats = stats.cpu().numpy()
        for b in range(B):
            for h in range(KH):
                m = models[b][h]
                h0, m0 = m.hits, m.misses
                want_slots = m.step(t, idx[b, h], n)
                assert st_h[b, h].tolist() == m.token, (t, b, h)
                assert ss_h[b, h].tolist() == m.stamp, (t, b, h)
                assert slots[b, h].tolist() == want_slots
                assert stats[b, h].tolist() == [m.hits - h0, m.misses - m0]
                inv = np.full(cap, -1, dtype=np.int32)
                for s, tok in enumerate(m.token):
                    if tok >= 0:
                        inv[tok] = s
                np.testing.assert_array_equal(ts_h[b, h], inv)
        # resident rows hold the rows of the tokens they claim to hold
        tok = st.long().clamp(min=0)
        want_k = torch.gather(keys.permute(0, 2, 1, 3), 2, tok.unsqueeze(-1).expand(-1, -1, -1, d))
        want_v = torch.gather(vals.permute(0, 2, 1, 3), 2, tok.unsqueeze(-1).expand(-1, -1, -1, d))
        live = (st >= 0).unsqueeze(-1)
        assert torch.equal(torch.where(live, kres, 0), torch.where(live, want_k, 0))
        assert torch.equal(torch.where(live, vres, 0), torch.where(live, want_v, 0))
        n += 1


@pytest.mark.parametrize("fuse,layout", [(0, "token"), (1, "token"), (0, "head"), (1, "head")])
def test_decode_with_lru_gives_identical_attention(env, fuse, layout):
    """The LRU layer changes where rows are read from, never the result.  With the
    two-launch tail (fuse=0) both states run the same attention kernel on the same rows
    in the same order and must agree bit for bit; with the fused tail the plain state
    sums its runs by token block instead of by rank, so agreement is to rounding."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    dtype = torch.bfloat16
    _lib.check(L.sl_tune(b"fuse_select_attend", fuse), "sl_tune")
    try:
        plain = _make_state(decode, _gen(60), 2, 32, 8, 900, 1024, 40, dtype, codes_layout="token")
        lru = _make_state(decode, _gen(60), 2, 32, 8, 900, 1024, 40, dtype, lru=64, codes_layout=layout)
        models = [[orc.LruModel(64) for _ in range(8)] for _ in range(2)]
        g = _gen(61)
        for step in range(1, 9):
            q = torch.randn(2, 32, 128, generator=g).to(dtype).to(DEV)
            if step % 2 == 0:
                q = prev_q          # repeat the query: the second time most selected rows are hits
            prev_q = q
            kn = torch.randn(2, 8, 128, generator=g).to(dtype).to(DEV)
            vn = torch.randn(2, 8, 128, generator=g).to(dtype).to(DEV)
            a = plain.step(q, kn, vn).clone()
            b = lru.step(q, kn, vn).clone()
            assert torch.equal(plain.idx, lru.idx)
            if fuse:
                assert (a.float() - b.float()).abs().max() <= 2e-2, step
            else:
                assert torch.equal(a, b), step
            idx = lru.idx.cpu().numpy()
            toks, stamps = lru.slot_token.cpu().numpy(), lru.slot_stamp.cpu().numpy()
            for bb in range(2):
                for h in range(8):
                    m = models[bb][h]
                    m.step(step, idx[bb, h], 900 + step - 1)
                    assert toks[bb, h].tolist() == m.token and stamps[bb, h].tolist() == m.stamp
        stats = lru.lru_stats.cpu().numpy()
        assert stats[..., 0].sum() > 0 and stats[..., 1].sum() > 0
        assert stats.sum() == sum(m.hits + m.misses for row in models for m in row)
    finally:
        _lib.check(L.sl_tune(b"fuse_select_attend", 1), "sl_tune")


@pytest.mark.parametrize("n0,k,C,rows", [(700, 30, 64, 0), (9000, 150, 1024, 3072), (9000, 150, 2048, 0), (20000, 300, 512, 4096),
                                         (9000, 150, 4096, 0), (3000, 63, 64, 0), (5000, 2047, 2048, 0)])
def test_table_update_inside_the_selection_launch_equals_the_launch_of_its_own(env, n0, k, C, rows):
    """Over head-major codes the block of a (b, kv head) that finishes last runs the head's table update
    at the end of the scorer + selection launch (tables of up to 2048 slots; larger ones keep the launch
    of their own).  Both forms must leave identical tables, slot lists, statistics, resident rows and
    outputs, step after step, with one block per head and with several, with hits and with misses."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    dtype = torch.bfloat16
    B, QH, KH = 3, 16, 4
    n_cap = (n0 + 32 + 7) // 8 * 8
    try:
        _lib.check(L.sl_tune(b"fused_rows", rows), "sl_tune")
        inside, own = (_make_state(decode, _gen(70), B, QH, KH, n0, n_cap, k, dtype, lru=C, codes_layout="head") for _ in range(2))
        g = _gen(71)
        for step in range(6):
            q = torch.randn(B, QH, 128, generator=g).to(dtype).to(DEV)
            if step % 2 == 1:
                q = prev_q          # the same query again: most selected rows are hits
            prev_q = q
            kn = torch.randn(B, KH, 128, generator=g).to(dtype).to(DEV)
            vn = torch.randn(B, KH, 128, generator=g).to(dtype).to(DEV)
            _lib.check(L.sl_tune(b"fused_lru", 1), "sl_tune")
            a = inside.step(q, kn, vn).clone()
            _lib.check(L.sl_tune(b"fused_lru", 0), "sl_tune")
            b = own.step(q, kn, vn).clone()
            assert not inside.peer_wait_failed() and not own.peer_wait_failed()
            for name in ("idx", "slots_out", "slot_token", "slot_stamp", "token_slot", "lru_stats", "k_res", "v_res"):
                assert torch.equal(getattr(inside, name), getattr(own, name)), (step, name)
            assert torch.equal(a, b), step
        stats = inside.lru_stats.cpu().numpy()
        assert stats[..., 0].sum() > 0 and stats[..., 1].sum() > 0
    finally:
        _lib.check(L.sl_tune(b"fused_lru", 1), "sl_tune")
        _lib.check(L.sl_tune(b"fused_rows", 0), "sl_tune")


@pytest.mark.parametrize("B,QH,KH,n0,k,dtype,kind", DECODE_CASES[:4])
def test_decode_step_two_launch_tail_matches_oracle(env, B, QH, KH, n0, k, dtype, kind):
    """The same step with selection and attention kept as two launches."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    _lib.check(L.sl_tune(b"fuse_select_attend", 0), "sl_tune")
    try:
        g = _gen(n0 + k + 1)
        st = _make_state(decode, g, B, QH, KH, n0, 2048 + 64, k, dtype, kind, codes_layout="token")
        for step in range(2):
            q = torch.randn(B, QH, 128, generator=g).to(dtype)
            k_new = torch.randn(B, KH, 128, generator=g).to(dtype)
            v_new = torch.randn(B, KH, 128, generator=g).to(dtype)
            out = st.step(q.to(DEV), k_new.to(DEV), v_new.to(DEV))
            _check_step(kernel, st, q, k_new, v_new, out, n0 + step, dtype)
    finally:
        _lib.check(L.sl_tune(b"fuse_select_attend", 1), "sl_tune")


def test_decode_many_blocks_and_long_cache(env):
    """More than one 4096-token block per (b, kv head) in the fused tail (4 and 8
    histogram copies); 8192-token
    spans with 16 and with 32 histogram copies (single-launch selection); and the
    two-launch selector once the copies wrap around (beyond 256k tokens)."""
    decode, kernel = env
    for n0, k, layout in ((9000, 180, "token"), (9000, 180, "head"), (20000, 100, "token"), (20000, 100, "head"),
                          (40000, 200, "head"), (60000, 300, "head"), (70000, 300, "auto"), (140000, 500, "auto"), (270000, 64, "auto")):
        g = _gen(n0)
        st = _make_state(decode, g, 1, 8, 2, n0, (n0 + 64 + 7) // 8 * 8, k, torch.bfloat16, codes_layout=layout)
        assert st.codes_layout == ("token" if n0 > 262144 else layout if layout != "auto" else "head")
        for step in range(2):
            q = torch.randn(1, 8, 128, generator=g).to(torch.bfloat16)
            kn = torch.randn(1, 2, 128, generator=g).to(torch.bfloat16)
            vn = torch.randn(1, 2, 128, generator=g).to(torch.bfloat16)
            out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV))
            _check_step(kernel, st, q, kn, vn, out, n0 + step, torch.bfloat16)


@pytest.mark.parametrize("rows,lru", [(4096, 0), (8192, 0), (4096, 512), (8192, 512), (1024, 0), (2048, 0)])
def test_head_major_blocks_of_every_size(env, rows, lru):
    """Head-major codes with several blocks per (b, kv head), in every block size, without and with
    the LRU table (where the launch ends at the selection and lowers its own flags): every step
    equals the oracle and the state with token-major codes, over a block boundary."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    dtype = torch.bfloat16
    B, QH, KH, k = 2, 8, 2, 150
    n0 = 2 * rows - 3          # the third step starts a new block
    n_cap = (n0 + 64 + 7) // 8 * 8
    _lib.check(L.sl_tune(b"fused_rows", rows), "sl_tune")
    try:
        head = _make_state(decode, _gen(80), B, QH, KH, n0, n_cap, k, dtype, lru=lru, codes_layout="head")
        token = _make_state(decode, _gen(80), B, QH, KH, n0, n_cap, k, dtype, lru=lru, codes_layout="token")
        g = _gen(81)
        for step in range(6):
            q = torch.randn(B, QH, 128, generator=g).to(dtype)
            kn = torch.randn(B, KH, 128, generator=g).to(dtype)
            vn = torch.randn(B, KH, 128, generator=g).to(dtype)
            out = head.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).clone()
            ref = token.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).clone()
            assert not head.peer_wait_failed()
            assert torch.equal(head.idx, token.idx), step
            assert torch.equal(head.seq_lens, token.seq_lens)
            if lru:   # same attention launch on the same rows
                assert torch.equal(out, ref), step
                assert torch.equal(head.slot_token, token.slot_token) and torch.equal(head.slot_stamp, token.slot_stamp)
            else:
                assert (out.float() - ref.float()).abs().max() <= 2e-2, step
            if step in (0, 3):
                _check_step(kernel, head, q, kn, vn, out, n0 + step, dtype)
    finally:
        _lib.check(L.sl_tune(b"fused_rows", 0), "sl_tune")


@pytest.mark.parametrize("rows,lru", [(4096, 0), (8192, 0), (4096, 256), (8192, 256), (1024, 0), (2048, 0)])
def test_head_major_ragged_batch_with_different_block_counts(env, rows, lru):
    """One batch whose sequences have 1, 2 and 3 blocks of rows (and one that ends exactly on a block
    boundary, so the step opens a new block): every (b, kv head) swaps histograms among ITS blocks
    only, blocks beyond a sequence's length drop out, and each sequence matches the oracle."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    dtype = torch.bfloat16
    B, QH, KH, k = 4, 8, 2, 120
    lens = [rows // 2, rows, 2 * rows + 5, 3 * rows - 1]
    n_cap = (3 * rows + 64 + 7) // 8 * 8
    _lib.check(L.sl_tune(b"fused_rows", rows), "sl_tune")
    try:
        g = _gen(88)
        st = _make_state(decode, g, B, QH, KH, 3 * rows, n_cap, k, dtype, lru=lru, codes_layout="head")
        st.seq_lens.copy_(torch.tensor(lens, dtype=torch.int32))
        for step in range(2):
            q = torch.randn(B, QH, 128, generator=g).to(dtype)
            kn = torch.randn(B, KH, 128, generator=g).to(dtype)
            vn = torch.randn(B, KH, 128, generator=g).to(dtype)
            out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).float().cpu().numpy()
            assert not st.peer_wait_failed()
            hq = st.hash_q
            q_code = kernel.hash_mlp_pack(q.to(DEV), hq.w1, hq.b1, hq.w2, hq.b2).cpu().numpy()[:, None]
            assert st.seq_lens.cpu().tolist() == [l + step + 1 for l in lens]
            for b, l in enumerate(lens):
                n = l + step + 1
                codes = st.codes[b:b + 1, :n].cpu().numpy()
                want_idx = orc.topk_stable(orc.hamming_score_u32(q_code[b:b + 1], codes, "blocked"), k)
                np.testing.assert_array_equal(st.idx[b:b + 1].cpu().numpy(), want_idx)
                want = orc.sparse_attention(q[b:b + 1].float().numpy(), st.keys[b:b + 1, :n].float().cpu().numpy(),
                                            st.vals[b:b + 1, :n].float().cpu().numpy(), want_idx)
                assert np.abs(out[b:b + 1] - want).max() <= 2e-2, (step, b)
    finally:
        _lib.check(L.sl_tune(b"fused_rows", 0), "sl_tune")


def test_head_major_equals_token_major_on_random_shapes(env):
    """Both code layouts are the same function of the same inputs: 200 seeded shapes (batch, heads, group
    size, rows around the block boundaries, k, LRU table or not, dtype, block size), three steps each;
    indices and lengths must be identical, outputs equal to rounding, and no wait may have run out."""
    import random
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    rnd = random.Random(2024)
    try:
        for case in range(200):
            KH = rnd.choice([1, 2, 4, 8]); G = rnd.choice([1, 2, 4]); QH = KH * G
            B = rnd.choice([1, 1, 2, 3, 5])
            n0 = rnd.choice([1, 5, 63, 100, 1000, 4095, 4096, 4097, 8191, 8192, 8193, 12000, 12287, 12288, 16384, 20000])
            k = rnd.choice([1, 7, 64, 100, 300, 600])
            lru = rnd.choice([0, 0, 1024])
            dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
            rows = rnd.choice([0, 4096, 8192, 1024, 2048])
            if rows in (1024, 2048) and (lru or n0 + 3 > 16 * rows):   # the small blocks: attention in the launch, <= 16 blocks
                rows = 0
            n_cap = (n0 + 16 + 7) // 8 * 8
            cg = torch.Generator().manual_seed(case)
            g = torch.Generator(device=DEV).manual_seed(case)
            hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, cg)
            hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, cg)
            kk = torch.randn((B, n0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
            vv = torch.randn((B, n0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
            head, token = (decode.LayerDecodeState(B, QH, KH, 128, n_cap, k, hq, hk, dtype=dtype, device=DEV, lru_slots=lru,
                                                   codes_layout=layout) for layout in ("head", "token"))
            head.prefill(kk, vv)
            token.prefill(kk, vv)
            _lib.check(L.sl_tune(b"fused_rows", rows), "sl_tune")
            what = (case, B, QH, KH, n0, k, lru, dtype, rows)
            for step in range(3):
                q, kn, vn = (torch.randn((B, h, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype) for h in (QH, KH, KH))
                a = head.step(q, kn, vn).float().clone()
                b = token.step(q, kn, vn).float().clone()
                assert torch.equal(head.idx, token.idx), (what, step)
                assert torch.equal(head.seq_lens, token.seq_lens), (what, step)
                assert not head.peer_wait_failed(), (what, step)
                assert (a - b).abs().max().item() <= TOL[dtype], (what, step)
    finally:
        _lib.check(L.sl_tune(b"fused_rows", 0), "sl_tune")


@pytest.mark.parametrize("lru", [0, 256])
def test_bounded_wait_gives_up_reports_and_drains(env, lru):
    """The blocks of a head wait for each other's flags at most a fixed number of polls.  Forced
    from the host -- every head also waits for a block that does not exist, with a short limit --
    each workgroup gives up, the launch still finishes, the error word says so, and after the
    workspace is cleared the state steps normally again."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    dtype = torch.bfloat16
    B, QH, KH, n0, k = 1, 8, 2, 9000, 100
    st = _make_state(decode, _gen(85), B, QH, KH, n0, (n0 + 64 + 7) // 8 * 8, k, dtype, lru=lru, codes_layout="head")
    g = _gen(86)
    fresh = lambda: tuple(torch.randn(B, h, 128, generator=g).to(dtype) for h in (QH, KH, KH))
    q, kn, vn = fresh()
    out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).clone()
    _check_step(kernel, st, q, kn, vn, out, n0, dtype)
    _lib.check(L.sl_tune(b"fused_spin_limit", 64), "sl_tune")
    _lib.check(L.sl_tune(b"fused_phantom_peer", 1), "sl_tune")
    try:
        q, kn, vn = fresh()
        st.step(q.to(DEV), kn.to(DEV), vn.to(DEV))
        torch.cuda.synchronize()          # the launch drained
        assert st.peer_wait_failed()
        assert st.seq_lens.cpu().tolist() == [n0 + 2] * B
    finally:
        _lib.check(L.sl_tune(b"fused_spin_limit", 0), "sl_tune")
        _lib.check(L.sl_tune(b"fused_phantom_peer", 0), "sl_tune")
    st.reset_workspace()
    assert not st.peer_wait_failed()
    q, kn, vn = fresh()
    out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).clone()
    _check_step(kernel, st, q, kn, vn, out, n0 + 2, dtype)


def _random_cases(count, seed):
    import random
    rnd = random.Random(seed)
    cases = []
    for _ in range(count):
        KH = rnd.choice([1, 2, 4, 8, 16])
        G = rnd.choice([1, 2, 3, 4, 5, 8])
        while KH * G > 64:
            G = rnd.choice([1, 2, 4])
        B = rnd.choice([1, 2, 3, 5])
        n0 = rnd.choice([1, 7, 63, 64, 65, 255, 256, 257, 1000, 2047, 4095, 4096, 4097, 8191, 8200])
        k = rnd.choice([1, 2, 17, 64, 100, 333, 600])
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        kind = rnd.choice(["mlp", "mlp", "linear"])
        if kind == "linear" and G != 1:
            kind = "mlp"               # the linear hash of the reference is per head, no grouped variant
        cases.append((B, KH * G, KH, n0, k, dtype, kind))
    return cases


@pytest.mark.parametrize("layout", ["auto", "token"])
@pytest.mark.parametrize("B,QH,KH,n0,k,dtype,kind", _random_cases(24, 2024))
def test_decode_step_random_shapes(env, B, QH, KH, n0, k, dtype, kind, layout):
    """Seeded sweep over head counts, group sizes, batch sizes, cache lengths around the
    block / tile / span boundaries, budgets above and below the cache length."""
    decode, kernel = env
    g = _gen(QH * 131 + n0 + k)
    st = _make_state(decode, g, B, QH, KH, n0, (n0 + 16 + 7) // 8 * 8, k, dtype, kind, codes_layout=layout)
    for step in range(2):
        q = torch.randn(B, QH, 128, generator=g).to(dtype)
        k_new = torch.randn(B, KH, 128, generator=g).to(dtype)
        v_new = torch.randn(B, KH, 128, generator=g).to(dtype)
        out = st.step(q.to(DEV), k_new.to(DEV), v_new.to(DEV))
        _check_step(kernel, st, q, k_new, v_new, out, n0 + step, dtype)


@pytest.mark.parametrize("layout", ["token", "head"])
def test_budget_changes_on_a_live_lru_state(env, layout):
    """k lowered and raised between steps on one workspace, with the LRU table on and more than
    one attention run per (b, kv head): the arrival tickets must stay where they are (and zero)
    whatever k is, so every step still matches the oracle and the state without a table."""
    decode, kernel = env
    dtype = torch.bfloat16
    B, QH, KH, n0, k_max = 2, 32, 8, 900, 100
    plain = _make_state(decode, _gen(70), B, QH, KH, n0, 1024, k_max, dtype)
    lru = _make_state(decode, _gen(70), B, QH, KH, n0, 1024, k_max, dtype, lru=128, codes_layout=layout)
    g = _gen(71)
    n = n0
    for step, k in enumerate([100, 37, 100, 64, 12, 100, 99]):
        plain.set_k(k)
        lru.set_k(k)
        q = torch.randn(B, QH, 128, generator=g).to(dtype)
        kn = torch.randn(B, KH, 128, generator=g).to(dtype)
        vn = torch.randn(B, KH, 128, generator=g).to(dtype)
        a = plain.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).clone()
        b = lru.step(q.to(DEV), kn.to(DEV), vn.to(DEV)).clone()
        n += 1
        hq = lru.hash_q
        q_code = kernel.hash_mlp_pack(q.to(DEV), hq.w1, hq.b1, hq.w2, hq.b2, hq.residue).cpu().numpy()[:, None]
        score = orc.hamming_score_u32(q_code, lru.codes[:, :n].cpu().numpy(), "blocked")
        want_idx = orc.topk_stable(score, k)
        np.testing.assert_array_equal(lru.selected().cpu().numpy(), want_idx)
        np.testing.assert_array_equal(plain.selected().cpu().numpy(), want_idx)
        want = orc.sparse_attention(q.float().numpy(), lru.keys[:, :n].float().cpu().numpy(),
                                    lru.vals[:, :n].float().cpu().numpy(), want_idx)
        assert np.abs(b.float().cpu().numpy() - want).max() <= TOL[dtype], (step, k)
        assert np.abs(a.float().cpu().numpy() - want).max() <= TOL[dtype], (step, k)
        # every kept row is resident where the table says
        slot = torch.gather(lru.token_slot, 2, lru.selected().long()).long()
        assert int(slot.min()) >= 0
        assert torch.equal(torch.gather(lru.slot_token, 2, slot), lru.selected())


@pytest.mark.parametrize("dtype,lru", [(torch.float32, 0), (torch.bfloat16, 0), (torch.float16, 0), (torch.bfloat16, 64)])
def test_decode_step_rotates_new_query_and_key(env, dtype, lru):
    """Rotary embedding inside the step (modify_llama.py:54-80): q and k_new go in un-rotated, the
    step rotates both at position seq_lens[b], hashes and attends with the rotated vectors and
    stores the rotated key.  Rotated values against the oracle's apply_rope; everything
    downstream against the oracle on the values the GPU holds."""
    decode, kernel = env
    theta = 5e5
    B, QH, KH, n0, k = 2, 32, 8, 700, 40
    g = _gen(123)
    hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    st = decode.LayerDecodeState(B, QH, KH, 128, 1024, k, hq, hk, dtype=dtype, device=DEV, lru_slots=lru, rope_theta=theta)
    st.prefill(torch.randn(B, n0, KH, 128, generator=g).to(dtype).to(DEV), torch.randn(B, n0, KH, 128, generator=g).to(dtype).to(DEV))
    tol = TOL[dtype]
    for step in range(3):
        q = torch.randn(B, QH, 128, generator=g).to(dtype)
        kn = torch.randn(B, KH, 128, generator=g).to(dtype)
        vn = torch.randn(B, KH, 128, generator=g).to(dtype)
        out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV))
        n = n0 + step + 1
        pos = [n - 1] * B
        q_rot, k_row = st.q_rot.cpu(), st.keys[:, n - 1].cpu()
        assert (q_rot.float() - orc.apply_rope(q, pos, theta).float()).abs().max() <= tol
        assert (k_row.float() - orc.apply_rope(kn, pos, theta).float()).abs().max() <= tol
        _check_step(kernel, st, q_rot, k_row, vn, out, n - 1, dtype)


def test_rotation_uses_each_sequence_s_own_position(env):
    decode, kernel = env
    dtype, theta = torch.bfloat16, 10000.0
    B, QH, KH = 5, 8, 2
    g = _gen(124)
    hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, g, scale=0.05)
    st = decode.LayerDecodeState(B, QH, KH, 128, 40000, 16, hq, hk, dtype=dtype, device=DEV, rope_theta=theta)
    st.prefill(torch.randn(B, 64, KH, 128, generator=g).to(dtype).to(DEV), torch.randn(B, 64, KH, 128, generator=g).to(dtype).to(DEV))
    lens = [64, 0, 5, 39990, 8191]
    st.seq_lens.copy_(torch.tensor(lens, dtype=torch.int32))
    st.host_len = max(lens)
    q = torch.randn(B, QH, 128, generator=g).to(dtype)
    kn = torch.randn(B, KH, 128, generator=g).to(dtype)
    vn = torch.randn(B, KH, 128, generator=g).to(dtype)
    st.step(q.to(DEV), kn.to(DEV), vn.to(DEV))
    assert (st.q_rot.cpu().float() - orc.apply_rope(q, lens, theta).float()).abs().max() <= 2e-2
    k_rows = torch.stack([st.keys[b, l].cpu() for b, l in enumerate(lens)])
    assert (k_rows.float() - orc.apply_rope(kn, lens, theta).float()).abs().max() <= 2e-2
    assert torch.equal(st.q_rot[1].cpu(), q[1])            # position 0: the identity
    assert st.seq_lens.tolist() == [l + 1 for l in lens]


@pytest.mark.parametrize("layout", ["head", "token"])
def test_budget_rule_on_the_device_survives_graph_replay_across_a_change_of_k(env, layout):
    """The budget max(min(n, min_remain), n - int(n * mask_out)) (spotlight_generation.py:162-164) is
    evaluated on the device from the length each step reads, so ONE captured graph keeps matching the
    oracle while k changes (here: 0.9 of the rows dropped, k grows every few tokens), in a ragged batch
    whose sequences have different lengths and therefore different budgets."""
    decode, kernel = env
    dtype = torch.bfloat16
    B, QH, KH, n0 = 2, 8, 2, 1195
    mask_out, min_remain = 0.9, 20
    n_cap = 1280
    k_cap = orc.num_remain(n_cap, mask_out, min_remain)
    st = _make_state(decode, _gen(310), B, QH, KH, n0, n_cap, k_cap, dtype, codes_layout=layout)
    st.seq_lens.copy_(torch.tensor([n0, n0 - 333], dtype=torch.int32))      # second sequence is shorter
    st.set_budget(mask_out, min_remain)
    g = _gen(311)
    st.capture(steps_ahead=40)
    ks = set()
    for step in range(30):
        q, kn, vn = (torch.randn(B, h, 128, generator=g).to(dtype) for h in (QH, KH, KH))
        st.q_in.copy_(q.to(DEV)); st.k_in.copy_(kn.to(DEV)); st.v_in.copy_(vn.to(DEV))
        out = st.replay().float().cpu().numpy()
        idx = st.selected().cpu().numpy()
        assert idx.shape == (B, KH, k_cap)
        q_code = kernel.hash_mlp_pack(q.to(DEV), st.hash_q.w1, st.hash_q.b1, st.hash_q.w2, st.hash_q.b2).cpu().numpy()[:, None]
        for b, n in enumerate([n0 + step + 1, n0 - 333 + step + 1]):
            k = orc.num_remain(n, mask_out, min_remain)
            ks.add(k)
            score = orc.hamming_score_u32(q_code[b:b + 1], st.codes[b:b + 1, :n].cpu().numpy(), "blocked")
            want = orc.topk_stable(score, k)
            np.testing.assert_array_equal(idx[b:b + 1, :, :k], want, err_msg=f"step {step} sequence {b} k {k}")
            assert (idx[b, :, k:] == -1).all()
            ref = orc.sparse_attention(q[b:b + 1].float().numpy(), st.keys[b:b + 1, :n].float().cpu().numpy(),
                                       st.vals[b:b + 1, :n].float().cpu().numpy(), want)
            assert np.abs(out[b:b + 1] - ref).max() <= TOL[dtype], (step, b)
    assert len(ks) >= 6          # the budget did change under the one graph, several times
    assert st.seq_lens.cpu().tolist() == [n0 + 30, n0 - 333 + 30]


def test_budget_rule_matches_python_for_awkward_products(env):
    """int(n * mask_out) truncates a double-precision product; the device must land on the same side
    of every integer boundary as Python does (mask_out values whose products sit just below / above
    an integer), and below min_remain rows everything is kept."""
    decode, kernel = env
    dtype = torch.float32
    B, QH, KH = 1, 2, 2
    for mask_out, min_remain in [(0.98, 20), (0.7, 5), (0.1, 3), (0.29, 1), (0.57, 0), (1.0, 4), (0.0, 2)]:
        n_cap = 256
        k_cap = n_cap
        st = _make_state(decode, _gen(int(mask_out * 100) + 3), B, QH, KH, 1, n_cap, k_cap, dtype, codes_layout="token")
        st.set_budget(mask_out, min_remain)
        g = _gen(5)
        for step in range(120):
            q, kn, vn = (torch.randn(B, h, 128, generator=g).to(dtype) for h in (QH, KH, KH))
            st.step(q.to(DEV), kn.to(DEV), vn.to(DEV))
            n = 2 + step
            k = orc.num_remain(n, mask_out, min_remain)
            kept = (st.idx[0, 0] >= 0).sum().item()
            assert kept == min(k, n), (mask_out, min_remain, n, kept, k)


@pytest.mark.parametrize("lru", [0, 256])
def test_a_bounded_wait_that_ran_out_is_raised_and_the_state_falls_back_to_token_major(env, lru):
    """What the product path does with the error word: check_peer_wait() (called by selected() and by
    Spotlight.generate where they read the device anyway) raises PeerWaitError, clears the word and
    re-lays the codes token-major, whose kernels never wait; lengths, rows, LRU table and budget are
    kept and the next steps are right.  The failure is forced from the host (a peer that does not
    exist, a short poll limit): every kernel still finishes normally."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    dtype = torch.bfloat16
    B, QH, KH, n0, k = 1, 8, 2, 9000, 100
    st = _make_state(decode, _gen(185), B, QH, KH, n0, (n0 + 64 + 7) // 8 * 8, k, dtype, lru=lru, codes_layout="head")
    g = _gen(186)
    fresh = lambda: tuple(torch.randn(B, h, 128, generator=g).to(dtype) for h in (QH, KH, KH))
    q, kn, vn = fresh()
    st.step(q.to(DEV), kn.to(DEV), vn.to(DEV), check=True)       # healthy: no raise
    _lib.check(L.sl_tune(b"fused_spin_limit", 64), "sl_tune")
    _lib.check(L.sl_tune(b"fused_phantom_peer", 1), "sl_tune")
    try:
        q, kn, vn = fresh()
        with pytest.raises(decode.PeerWaitError):
            st.step(q.to(DEV), kn.to(DEV), vn.to(DEV), check=True)
    finally:
        _lib.check(L.sl_tune(b"fused_spin_limit", 0), "sl_tune")
        _lib.check(L.sl_tune(b"fused_phantom_peer", 0), "sl_tune")
    assert st.codes_layout == "token" and not st.peer_wait_failed()
    assert st.seq_lens.cpu().tolist() == [n0 + 2] * B               # the failed step did append its row
    for step in range(2):
        q, kn, vn = fresh()
        out = st.step(q.to(DEV), kn.to(DEV), vn.to(DEV), check=True).clone()
        if lru == 0:
            _check_step(kernel, st, q, kn, vn, out, n0 + 2 + step, dtype)
        else:
            assert st.seq_lens.cpu().tolist() == [n0 + 3 + step] * B
            idx = st.selected().cpu().numpy()
            q_code = kernel.hash_mlp_pack(q.to(DEV), st.hash_q.w1, st.hash_q.b1, st.hash_q.w2, st.hash_q.b2).cpu().numpy()[:, None]
            n = n0 + 3 + step
            want = orc.topk_stable(orc.hamming_score_u32(q_code, st.codes[:, :n].cpu().numpy(), "blocked"), k)
            np.testing.assert_array_equal(idx, want)
    # selected() is the other place that looks: a word set behind its back is raised there
    st2 = _make_state(decode, _gen(187), B, QH, KH, n0, (n0 + 64 + 7) // 8 * 8, k, dtype, lru=lru, codes_layout="head")
    st2.error_word().fill_(1)
    with pytest.raises(decode.PeerWaitError):
        st2.selected()
    assert st2.codes_layout == "token"


def test_head_major_grids_larger_than_the_device_run_in_rounds(env):
    """Batches whose grid the device cannot hold at once (hundreds of (b, kv head) pairs times several
    blocks) still run the one-launch step: the blocks of a head are numbered consecutively in start
    order, so a head never waits for a workgroup that cannot start.  Indices must equal the
    token-major step's, outputs agree to rounding, and no bounded wait may run out."""
    decode, kernel = env
    from spotlight_amd import _lib
    L = _lib.load()
    dtype = torch.bfloat16
    try:
        for case, (B, KH, G, n0, k, rows, lru) in enumerate([(64, 8, 4, 1500, 30, 512, 0), (48, 8, 1, 3000, 64, 1024, 0),
                                                             (32, 8, 4, 2500, 50, 0, 0), (64, 4, 2, 5000, 100, 1024, 0),
                                                             (64, 8, 4, 7000, 60, 3072, 128), (40, 8, 5, 2000, 40, 512, 0),
                                                             (64, 8, 4, 9000, 60, 0, 128), (24, 8, 4, 24000, 100, 0, 0)]):
            QH = KH * G
            n_cap = (n0 + 16 + 7) // 8 * 8
            cg = torch.Generator().manual_seed(900 + case)
            g = torch.Generator(device=DEV).manual_seed(900 + case)
            hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, DEV, cg)
            hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, DEV, cg)
            kk = torch.randn((B, n0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
            vv = torch.randn((B, n0, KH, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype)
            head, token = (decode.LayerDecodeState(B, QH, KH, 128, n_cap, k, hq, hk, dtype=dtype, device=DEV, lru_slots=lru,
                                                   codes_layout=layout) for layout in ("head", "token"))
            head.prefill(kk, vv)
            token.prefill(kk, vv)
            _lib.check(L.sl_tune(b"fused_rows", rows), "sl_tune")
            for step in range(2):
                q, kn, vn = (torch.randn((B, h, 128), generator=g, device=DEV, dtype=torch.float32).to(dtype) for h in (QH, KH, KH))
                a = head.step(q, kn, vn).float().clone()
                b = token.step(q, kn, vn).float().clone()
                assert not head.peer_wait_failed(), (case, step)
                assert torch.equal(head.idx, token.idx), (case, step)
                assert (a - b).abs().max().item() <= TOL[dtype], (case, step)
    finally:
        _lib.check(L.sl_tune(b"fused_rows", 0), "sl_tune")


def test_seeded_inputs_end_to_end_against_the_oracle_s_own_codes(env):
    """ONE seeded input through both pipelines from the raw vectors on: the oracle hashes the query and
    every key itself (fp64 pre-activations -> sign -> pack), scores, selects and attends; the GPU does
    the same from the same vectors (prompt keys through the many-rows hash, the decoded token through
    the step).  Where no pre-activation lies within the margin of zero -- asserted for these seeds, so
    the comparison is not vacuous -- the codes, and with them the kept indices, must be identical; else
    the count is reported and the comparison falls back to the codes the GPU holds."""
    decode, kernel = env
    dtype, margin = torch.float32, 1e-4
    B, QH, KH, n0, k = 2, 4, 2, 300, 40
    g = _gen(300)

    def mk(H):
        w = [torch.randn(H, 128, 256, generator=g) * 0.5, torch.randn(H, 256, 128, generator=g) * 0.5]
        b = [torch.randn(H, 256, generator=g) * 0.5, torch.randn(H, 128, generator=g) * 0.5]
        return w, b
    (wq, bq), (wk, bk) = mk(QH), mk(KH)
    keys_all = torch.randn(B, n0 + 1, KH, 128, generator=g)
    q = torch.randn(B, QH, 128, generator=g)
    vals_all = torch.randn(B, n0 + 1, KH, 128, generator=g)
    as_np = lambda w, b: [(w[0].numpy(), b[0].numpy()), (w[1].numpy(), b[1].numpy())]
    pre_k = orc.mlp_hash(keys_all.reshape(B * (n0 + 1), KH, 128).numpy(), as_np(wk, bk), False)
    pre_q = orc.mlp_hash(q.numpy(), as_np(wq, bq), False)
    inside = int((np.abs(pre_k) < margin).sum() + (np.abs(pre_q) < margin).sum())
    codes_o = orc.pack_sign_u32(pre_k).reshape(B, n0 + 1, KH, 4)
    hq = decode.HashWeights(wq[0].to(DEV), bq[0].to(DEV), wq[1].to(DEV), bq[1].to(DEV))
    hk = decode.HashWeights(wk[0].to(DEV), bk[0].to(DEV), wk[1].to(DEV), bk[1].to(DEV))
    for layout in ("head", "token"):
        st = decode.LayerDecodeState(B, QH, KH, 128, 320, k, hq, hk, dtype=dtype, device=DEV, codes_layout=layout)
        st.prefill(keys_all[:, :n0].to(DEV), vals_all[:, :n0].to(DEV))
        out = st.step(q.to(DEV), keys_all[:, n0].to(DEV), vals_all[:, n0].to(DEV)).float().cpu().numpy()
        n = n0 + 1
        got_codes = st.codes[:, :n].cpu().numpy()
        score = orc.hamming_score_u32(orc.pack_sign_u32(pre_q)[:, None], codes_o, "blocked")
        want_idx = orc.topk_stable(score, k)
        want = orc.sparse_attention(q.numpy(), keys_all.numpy(), vals_all.numpy(), want_idx)
        if inside == 0:
            np.testing.assert_array_equal(got_codes, codes_o)
            np.testing.assert_array_equal(st.idx.cpu().numpy(), want_idx)
            assert np.abs(out - want).max() <= 1e-5
        else:   # pragma: no cover - not reached with these seeds
            print(f"{inside} pre-activations within {margin} of zero: comparing on the GPU's codes")
            _check_step(kernel, st, q, keys_all[:, n0], vals_all[:, n0], torch.from_numpy(out), n0, dtype)
    assert inside == 0, "pick another seed: the strict comparison did not run"
