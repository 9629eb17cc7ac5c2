"""
Attention-score fidelity metrics of the reference's validation script
(turboquant/validate_v3.py:87 for the scores, :93-125 for the metrics).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def attention_scores(queries: torch.Tensor, keys: torch.Tensor) -> torch.Tensor:
    """q . k for one query per head: queries [B,H,1,D], keys [B,H,S,D] -> scores [B,H,S] in float32
    (validate_v3.py:87)."""
    return torch.matmul(queries.float(), keys.float().transpose(-2, -1)).squeeze(-2)


def compute_metrics(real_scores: torch.Tensor, tq_scores: torch.Tensor, H: int) -> dict:
    """Cosine similarity of the score vectors, top-1 agreement and "true top-1 within the
    compressed top-5", per head of batch element 0, averaged over heads (validate_v3.py:93-125).
    The per-head work runs as three batched device operations instead of a Python loop with a
    host synchronisation per head; the results are the reference's."""
    rs = real_scores[0, :H]
    ts = tq_scores[0, :H]
    cosine_sims = F.cosine_similarity(rs, ts, dim=-1).tolist()
    real_top1 = rs.argmax(dim=-1)
    top1_matches = int((real_top1 == ts.argmax(dim=-1)).sum().item())
    k = min(5, ts.shape[-1])
    tq_top5 = ts.topk(k, dim=-1).indices
    top5_matches = int((tq_top5 == real_top1.unsqueeze(-1)).any(dim=-1).sum().item())
    n_checks = H
    return {
        "cosine_sim": sum(cosine_sims) / len(cosine_sims),
        "top1_pct": 100 * top1_matches / n_checks,
        "top5_pct": 100 * top5_matches / n_checks,
        "top1_matches": top1_matches,
        "top5_matches": top5_matches,
        "n_checks": n_checks,
    }
