"""The end-to-end decode workload (random-init Llama-3-8B dims, batch 4, 32768-token prompt,
dense first layer, sparse layers on the HIP step) on a few layers: a token decoded eagerly and
the same token decoded by replaying the captured HIP graph must agree, and every sparse layer's
step must satisfy the properties any correct implementation has (tests/test_fullsize_gpu.py).
Stands for the loop of spotlight_generation.py:470-495 at the shape the benchmark times."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from spotlight_amd.workloads import E2EModel
    m = E2EModel(L=4, B=4, n0=32768, k=655, fix_layers=(0,), seed=3)
    m.prefill()
    return m


def _layer_checks(m, n):
    from test_fullsize_gpu import check_step_properties
    for st in m.sparse:
        # what the step was given is un-rotated; what it hashed, stored and attended with is rotated
        k_row = st.keys[:, n - 1].clone()
        check_step_properties(st, st.q_rot, k_row, st.v_in, st.out, n)


def _rope_ref(m, x, pos):
    return m.rope(x[:, None], torch.tensor([pos], device=x.device))[:, 0]


@torch.no_grad()
def test_eager_token_equals_graph_token_and_every_sparse_layer_is_consistent(model):
    m = model
    n0 = m.n0
    tok0 = m.tok.clone()
    # token 1 eagerly
    m.step_body()
    torch.cuda.synchronize()
    _layer_checks(m, n0 + 1)
    for st in m.sparse:   # the rotation the step did is the model's own rotary embedding at position n0
        assert (st.q_rot.float() - _rope_ref(m, st.q_in, n0).float()).abs().max() <= 2e-2
        assert (st.keys[:, n0].float() - _rope_ref(m, st.k_in, n0).float()).abs().max() <= 2e-2
    eager = dict(tok=m.tok.clone(), out=[st.out.clone() for st in m.sparse], idx=[st.idx.clone() for st in m.sparse],
                 rows=[st.keys[:, n0].clone() for st in m.sparse])
    # the same token again, as a graph replay
    m.rewind(1, tok0)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        m.step_body()        # (capture runs nothing: positions and lengths are still rewound)
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(m.tok, eager["tok"])
    for st, out, idx, row in zip(m.sparse, eager["out"], eager["idx"], eager["rows"]):
        assert torch.equal(st.idx, idx)
        assert torch.equal(st.keys[:, n0], row)
        assert (st.out.float() - out.float()).abs().max() <= 2e-2
    _layer_checks(m, n0 + 1)
    # two more tokens by replay: lengths and positions advance on the device
    for i in range(2):
        g.replay()
        torch.cuda.synchronize()
        _layer_checks(m, n0 + 2 + i)
    assert int(m.pos) == n0 + 3
