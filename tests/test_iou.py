"""IoU of selected rows against the true top-k (spotlight_evaluation.py:303-316), host only."""
import torch

from spotlight_amd.iou import ratio_table, selection_iou


def test_iou_matches_set_arithmetic():
    g = torch.Generator().manual_seed(0)
    B, QH, KH, n, d, k = 2, 4, 2, 50, 16, 7
    q = torch.randn(B, QH, d, generator=g)
    keys = torch.randn(B, n, KH, d, generator=g)
    sel = torch.stack([torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(KH)]) for _ in range(B)]).int()
    sel[1, 0, -2:] = -1                                   # unused slots
    got = selection_iou(sel, q, keys, k)
    assert got.shape == (B, QH)
    for b in range(B):
        for qh in range(QH):
            h = qh // (QH // KH)
            true = set((keys[b, :, h] @ q[b, qh]).topk(k).indices.tolist())
            draft = set(t for t in sel[b, h].tolist() if t >= 0)
            assert abs(float(got[b, qh]) - len(true & draft) / len(true | draft)) < 1e-6


def test_iou_is_one_when_the_true_top_k_is_selected_and_zero_when_disjoint():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(1, 2, 8, generator=g)
    keys = torch.randn(1, 30, 2, 8, generator=g)
    order = torch.stack([(keys[0, :, h] @ q[0, h]).argsort(descending=True) for h in range(2)])
    assert torch.allclose(selection_iou(order[None, :, :5].int(), q, keys, 5), torch.ones(1, 2))
    assert torch.equal(selection_iou(order[None, :, -5:].int(), q, keys, 5), torch.zeros(1, 2))


def test_ratio_table_layout():
    text = ratio_table([None, [0.5, 1.0], [0.25, 0.75]])
    lines = text.splitlines()
    assert lines[0].split() == ["#", "0", "#", "1", "avg"] or "avg" in lines[0]
    assert lines[1].split() == ["1:", "50", "100", "75"]
    assert lines[2].split() == ["2:", "25", "75", "50"]
    assert lines[3].split() == ["37", "87", "62"]
