"""ORACLE (test infrastructure, never on the product path): distance measures between two sets of embeddings.

The reference's own tests compare embeddings by cosine similarity per output tensor
(python/tests/task_executors/eric/utils.py:144-163); the build's bar adds the largest error relative to the
largest reference magnitude.  Both are global figures, so this also reports the worst single row (token).
"""

from __future__ import annotations

import torch


def distances(got: torch.Tensor, ref: torch.Tensor) -> dict:
    """got, ref: [rows, hidden].  All reductions in float64 (an fp32 reduction over millions of elements can print a
    cosine above 1).

    cosine            of the two tensors flattened
    max_rel_err       max |got - ref| / max |ref|  (the bar's error measure)
    min_row_cosine    the worst row's cosine
    max_row_rel_l2    the worst row's ||got - ref|| / ||ref||
    """
    g, r = got.detach().double().cpu(), ref.detach().double().cpu()
    if g.shape != r.shape or g.dim() != 2:
        raise ValueError(f"shapes {tuple(g.shape)} and {tuple(r.shape)}: two [rows, hidden] tensors expected")
    d = g - r
    rn = r.norm(dim=1).clamp_min(1e-300)
    gn = g.norm(dim=1).clamp_min(1e-300)
    row_cos = (g * r).sum(dim=1) / (gn * rn)
    return {
        "cosine": min(1.0, ((g * r).sum() / (g.norm() * r.norm())).item()),
        "max_rel_err": (d.abs().max() / r.abs().max()).item(),
        "min_row_cosine": row_cos.min().item(),
        "max_row_rel_l2": (d.norm(dim=1) / rn).max().item(),
    }
