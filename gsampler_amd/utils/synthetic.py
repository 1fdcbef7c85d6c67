"""Seeded synthetic graphs in CSC form (int64 indptr / indices), built with
torch so the same code runs on the CPU (tests) and on the GPU (benchmark).

The generators follow the workload definitions used for measurement:
R-MAT for the small 2-layer case and Chung-Lu power-law graphs (expected degree
of node i proportional to (i+1)^(-1/(gamma-1))) for the large ones.  Parallel
edges are kept, as a sampled multigraph would have them.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch


def _generator(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def coo_to_csc(row: torch.Tensor, col: torch.Tensor, num_nodes: int,
               sort_rows: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """(indptr[num_nodes + 1], indices[E]); rows inside a column are sorted
    when sort_rows is set (what node2vec's connectivity test needs)."""
    if row.is_cuda and not sort_rows:
        from .. import capi  # the library's own edge-list ingest (stable sort by column)
        indptr, indices, _ = capi.coo_to_csc(row, col, num_nodes)
        return indptr, indices
    if sort_rows:
        order = torch.argsort(col * num_nodes + row)
    else:
        order = torch.argsort(col, stable=True)
    indices = row[order].contiguous()
    counts = torch.bincount(col, minlength=num_nodes)
    indptr = torch.zeros(num_nodes + 1, dtype=torch.int64, device=row.device)
    torch.cumsum(counts, 0, out=indptr[1:])
    return indptr, indices


def rmat_csc(num_nodes: int, num_edges: int, a: float = 0.57, b: float = 0.19,
             c: float = 0.19, seed: int = 1, device="cpu",
             sort_rows: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """R-MAT edge list over 2^ceil(log2 num_nodes) ids, truncated to ids below
    num_nodes, first num_edges survivors kept."""
    scale = max(1, (num_nodes - 1).bit_length())
    g = _generator(seed, device)
    rows, cols, have = [], [], 0
    while have < num_edges:
        n = int((num_edges - have) * 1.5) + 1024
        row = torch.zeros(n, dtype=torch.int64, device=device)
        col = torch.zeros(n, dtype=torch.int64, device=device)
        for _ in range(scale):
            r = torch.rand(n, generator=g, device=device)
            row_bit = r >= (a + b)
            col_bit = ((r >= a) & (r < a + b)) | (r >= a + b + c)
            row = row * 2 + row_bit.to(torch.int64)
            col = col * 2 + col_bit.to(torch.int64)
        keep = (row < num_nodes) & (col < num_nodes)
        rows.append(row[keep])
        cols.append(col[keep])
        have += int(keep.sum().item())
    row = torch.cat(rows)[:num_edges]
    col = torch.cat(cols)[:num_edges]
    return coo_to_csc(row, col, num_nodes, sort_rows)


def chung_lu_csc(num_nodes: int, num_edges: int, exponent: float = 2.1,
                 seed: int = 1, device="cpu", sort_rows: bool = False,
                 chunk: int = 1 << 26) -> Tuple[torch.Tensor, torch.Tensor]:
    """Chung-Lu power-law multigraph: both endpoints of every edge are drawn
    independently with probability proportional to w_i = (i+1)^(-1/(exponent-1))."""
    g = _generator(seed, device)
    w = torch.arange(1, num_nodes + 1, dtype=torch.float64, device=device)
    w = w.pow(-1.0 / (exponent - 1.0))
    cdf = torch.cumsum(w, 0)
    cdf = cdf / cdf[-1]
    rows, cols = [], []
    for start in range(0, num_edges, chunk):
        n = min(chunk, num_edges - start)
        for dst in (rows, cols):
            u = torch.rand(n, generator=g, device=device, dtype=torch.float64)
            dst.append(torch.searchsorted(cdf, u).clamp_(max=num_nodes - 1))
    row, col = torch.cat(rows), torch.cat(cols)
    del rows, cols
    return coo_to_csc(row, col, num_nodes, sort_rows)


def batched_seeds(num_nodes: int, num_batches: int, batch_size: int,
                  seed: int = 1, device="cpu") -> Tuple[torch.Tensor, torch.Tensor]:
    """num_batches x batch_size seed nodes, distinct inside every batch, drawn
    uniformly; returns (seeds[B * batch_size], seeds_ptr[B + 1])."""
    g = _generator(seed, device)
    out = []
    for _ in range(num_batches):
        if batch_size * 4 <= num_nodes:
            # rejection-free for sparse draws: oversample, keep first distinct
            cand = torch.randint(0, num_nodes, (batch_size * 2,), generator=g,
                                 device=device)
            uniq, inv = torch.unique(cand, return_inverse=True)
            first = torch.full((uniq.numel(),), cand.numel(), dtype=torch.int64,
                               device=device)
            first.scatter_reduce_(0, inv, torch.arange(cand.numel(), device=device),
                                  reduce="amin")
            keep = torch.sort(first).values[:batch_size]
            pick = cand[keep]
            if pick.numel() < batch_size:
                pick = torch.randperm(num_nodes, generator=g, device=device)[:batch_size]
        else:
            pick = torch.randperm(num_nodes, generator=g, device=device)[:batch_size]
        out.append(pick)
    seeds = torch.cat(out).to(torch.int64)
    ptr = torch.arange(num_batches + 1, dtype=torch.int64, device=device) * batch_size
    return seeds, ptr
