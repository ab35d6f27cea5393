"""Expert dispatch shared by the mixture-of-experts feed-forwards.

Two routes from (token, expert) assignments to per-expert GEMMs, both
parameterised on the activation between the two projections so that a
gated (SwiGLU) and an ungated (relu^2) expert use the same machinery:

* experts_padded: sync-free scatter into a [E, C, h] buffer and two
  batched GEMMs — decode-sized batches, where streaming every expert's
  weights bounds the step and padding rows are free.
* experts_sorted: sort assignments by expert and run one contiguous GEMM
  pair per non-empty expert — prompt-sized batches, where the padded
  route's E/K-fold FLOP overhead would dominate (one host sync for the
  per-expert counts).
"""
from __future__ import annotations

from typing import Callable

import torch


def flat_tokens(T: int, K: int, device) -> torch.Tensor:
    return (torch.arange(T, device=device).unsqueeze(1)
            .expand(T, K).reshape(-1))


def experts_padded(x: torch.Tensor, weights: torch.Tensor,
                   dst: torch.Tensor, up_t: torch.Tensor,
                   down_t: torch.Tensor, capacity: int,
                   act: Callable[[torch.Tensor], torch.Tensor]
                   ) -> torch.Tensor:
    """x [T, h]; weights [T, K] (x.dtype or fp32); dst [T*K] int64 rows
    of the padded buffer (expert * capacity + rank); up_t [E, h, f_in],
    down_t [E, f, h]; act maps [E*C, f_in] -> [E*C, f]."""
    T, h = x.shape
    E = up_t.shape[0]
    K = weights.shape[1]
    tok = flat_tokens(T, K, x.device)
    buf = x.new_zeros((E * capacity, h))
    buf.index_copy_(0, dst, x[tok])
    mid = torch.bmm(buf.view(E, capacity, h), up_t)
    a = act(mid.view(E * capacity, -1))
    y = torch.bmm(a.view(E, capacity, -1), down_t).view(E * capacity, h)
    ys = y.index_select(0, dst)
    out = torch.zeros((T, h), dtype=torch.float32, device=x.device)
    out.index_add_(0, tok, ys.float() * weights.reshape(-1, 1).float())
    return out.to(x.dtype)


def experts_sorted(x: torch.Tensor, weights: torch.Tensor,
                   topk_idx: torch.Tensor, up_t: torch.Tensor,
                   down_t: torch.Tensor,
                   act: Callable[[torch.Tensor], torch.Tensor]
                   ) -> torch.Tensor:
    """Same interface as experts_padded with topk_idx [T, K] instead of
    padded rows; per-expert contiguous GEMMs."""
    T, h = x.shape
    E = up_t.shape[0]
    K = weights.shape[1]
    flat_e = topk_idx.reshape(-1).long()
    tok = flat_tokens(T, K, x.device)
    order = torch.argsort(flat_e, stable=True)
    sorted_tok = tok[order]
    counts = torch.bincount(flat_e, minlength=E).tolist()
    flat_w = weights.reshape(-1).float()[order]
    out = torch.zeros((T, h), dtype=torch.float32, device=x.device)
    start = 0
    for e, cnt in enumerate(counts):
        if cnt == 0:
            continue
        rows = sorted_tok[start:start + cnt]
        xe = x.index_select(0, rows)
        ye = act(xe @ up_t[e]) @ down_t[e]
        out.index_add_(0, rows,
                       ye.float() * flat_w[start:start + cnt, None])
        start += cnt
    return out.to(x.dtype)


def padded_rows(topk_idx: torch.Tensor, num_experts: int, capacity: int
                ) -> torch.Tensor:
    """Sync-free padded-buffer rows from expert ids [T, K]: row =
    expert * capacity + (rank of this assignment among the expert's)."""
    flat_e = topk_idx.reshape(-1).long()
    oh = torch.nn.functional.one_hot(flat_e, num_experts)
    rank = (torch.cumsum(oh, 0) - oh).mul(oh).sum(-1)
    return flat_e * capacity + rank
