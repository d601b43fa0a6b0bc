"""Expert paths of routed feed-forwards, shared by the layered models.

A routed layer picks its path by batch size.  Small batches (every decode step, captured in
hipGraphs) run ALL experts as one GEMM over the stacked up-projections, scale the activations by
the routing weights (0 for experts not chosen) and sum the chosen experts inside one GEMM over
the side-by-side down-projections: every expert's weights are streamed regardless, there is no
sort and no host round trip.  Prompt-sized batches sort the (token, choice) pairs by expert (one
host read of the counts) and run each expert's rows through its own GEMMs.
"""
from __future__ import annotations

from typing import Callable

import torch

from ..ops import stream as sops

# batches up to this many rows take the all-experts GEMM pair
MOE_DENSE_ROWS = 256


def routed_sorted(h2: torch.Tensor, ids: torch.Tensor, w: torch.Tensor, experts: int,
                  outputs: int, expert_fn: Callable[[int, torch.Tensor], torch.Tensor]
                  ) -> torch.Tensor:
    """The routed feed-forward of h2 [T, d] by expert-sorted rows, as fp32 [T, d].  ids / w
    [T, top]: chosen outputs and their weights; outputs >= experts are identity outputs (they
    return their input and run no expert).  expert_fn(e, rows) is expert e applied to its rows
    [c, d] -> [c, d]."""
    T, d = h2.shape
    top = ids.shape[1]
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)                 # sorted pair -> flat (t, k)
    counts = torch.bincount(flat, minlength=outputs)[:experts].tolist()
    inv = torch.empty(T * top, dtype=torch.int32, device=h2.device)
    inv[order] = torch.arange(T * top, dtype=torch.int32, device=h2.device)
    n_real = sum(counts)
    xs = h2.index_select(0, order[:n_real] // top)
    ys = torch.empty(max(1, n_real), d, dtype=h2.dtype, device=h2.device)
    a = 0
    for e, c in enumerate(counts):
        if c:
            ys[a:a + c] = expert_fn(e, xs[a:a + c])
            a += c
    out = torch.empty(T, d, dtype=torch.float32, device=h2.device)
    sops.moe_combine(out, ys, inv.view(T, top), ids, w, h2, experts)
    return out
