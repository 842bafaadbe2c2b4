"""Quality of the retrieval: intersection-over-union of the rows the hash codes
select against the rows the true attention scores would select.

The reference computes it in benchmark mode for the last query position, per
query head, as ``|draft ∩ true| / |draft ∪ true|`` with ``true`` the top-k of the
RoPE'd ``q·kᵀ`` (spotlight/modifiers/spotlight_evaluation.py:303-316) and prints a
layer × head table of percentages (test_iou/test.py:30-58)."""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch


def selection_iou(selected: torch.Tensor, query: torch.Tensor, keys: torch.Tensor, k: int) -> torch.Tensor:
    """selected int [B, KH, k'] (negative = unused) rows chosen per kv head;
    query [B, QH, d] and keys [B, n, KH, d], both post-RoPE.  Returns [B, QH]
    float32: for every query head the IoU between its kv head's selected set and
    the k rows with the largest q·k of that query head."""
    B, QH, d = query.shape
    n, KH = keys.shape[1], keys.shape[2]
    G = QH // KH
    qg = query.reshape(B, KH, G, d).float()
    true = torch.einsum("bhgd,bnhd->bhgn", qg, keys.float())            # [B, KH, G, n]
    k = min(k, n)
    true_idx = true.topk(k=k, dim=-1).indices
    true_mask = torch.zeros((B, KH, G, n), dtype=torch.bool, device=query.device)
    true_mask.scatter_(-1, true_idx, True)
    sel = selected.long()
    valid = sel >= 0
    draft_mask = torch.zeros((B, KH, n + 1), dtype=torch.bool, device=query.device)
    draft_mask.scatter_(-1, torch.where(valid, sel, torch.full_like(sel, n)), True)
    draft_mask = draft_mask[..., :n][:, :, None, :]
    inter = (true_mask & draft_mask).sum(-1).float()
    union = (true_mask | draft_mask).sum(-1).float()
    return (inter / union.clamp_min(1.0)).reshape(B, QH)


def ratio_table(ratios: Sequence[Optional[Sequence[float]]]) -> str:
    """Layer × head table of IoU percentages with per-layer and per-head means, the
    layout test_iou/test.py:30-58 prints (without the colours).  ``ratios[i]`` is
    None for a dense layer."""
    num_heads = max([len(r) if r is not None else 0 for r in ratios] + [0])
    lines = ["      " + " ".join(f"#{h:>4d}" for h in range(num_heads)) + "  avg"]
    cols: List[List[int]] = [[] for _ in range(num_heads + 1)]
    for idx, row in enumerate(ratios):
        if row is None:
            continue
        vals = [int(r * 100) for r in row]
        mean = int(sum(row) / len(row) * 100)
        for h, v in enumerate(vals):
            cols[h].append(v)
        cols[-1].append(mean)
        lines.append(f"{idx:>4d}: " + " ".join(f"{v:>5d}" for v in vals) + f" {mean:>5d}")
    if cols[-1]:
        lines.append("      " + " ".join(f"{sum(c) // len(c):>5d}" if c else "    -" for c in cols))
    return "\n".join(lines)
