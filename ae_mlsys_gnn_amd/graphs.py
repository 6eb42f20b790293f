"""Synthetic graph builders for tests and benchmarks (uniform random, R-MAT power law, kNN
point clouds) and the host/device glue that turns an edge list into the CSR-by-destination
arrays the operators take.  Everything is seeded; torch ops only, so the same code runs on the
CPU (small cases) and on the GPU (the 115 M-edge benchmark graph).

Convention (reference script/train/train_gatconv_our.py:82-95): row = destination, col_ind =
source, self-loops removed and then added once per node, duplicate edges merged."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class Graph:
    n: int
    row_ptr: torch.Tensor            # int32 [n+1]   CSR by destination
    col_ind: torch.Tensor            # int32 [E]     source node of each CSR position
    col_ptr: Optional[torch.Tensor] = None   # int32 [n+1]   CSC (by source)
    row_ind: Optional[torch.Tensor] = None   # int32 [E]     destination node of each CSC position
    permute: Optional[torch.Tensor] = None   # int32 [E]     CSR position of each CSC position

    @property
    def n_edges(self) -> int:
        return int(self.col_ind.numel())

    def to(self, device):
        mv = lambda t: None if t is None else t.to(device)
        return Graph(self.n, mv(self.row_ptr), mv(self.col_ind), mv(self.col_ptr), mv(self.row_ind), mv(self.permute))


def validate_graph(g: "Graph", what: str = "graph") -> None:
    """Raises ValueError unless the arrays describe a graph the gather kernels can walk: integer index
    arrays, pointer arrays that start at 0, never decrease and end at E, every node id in [0, n) and every
    permute entry in [0, E).  Plain torch reductions (host or device), to be called BEFORE any operator
    sees arrays that came from a file or another untrusted source: the kernels index feature rows with
    these ids unchecked."""
    int_types = (torch.int8, torch.int16, torch.int32, torch.int64, torch.uint8)
    e = int(g.col_ind.numel())
    for name, ptr_arr, idx in (("row_ptr/col_ind", g.row_ptr, g.col_ind), ("col_ptr/row_ind", g.col_ptr, g.row_ind)):
        if ptr_arr is None and idx is None:
            continue
        if ptr_arr is None or idx is None:
            raise ValueError("%s: %s must be given together" % (what, name))
        if ptr_arr.dtype not in int_types or idx.dtype not in int_types:
            raise ValueError("%s: %s must be integer arrays, got %s / %s" % (what, name, ptr_arr.dtype, idx.dtype))
        if ptr_arr.dim() != 1 or idx.dim() != 1 or ptr_arr.numel() != g.n + 1 or idx.numel() != e:
            raise ValueError("%s: %s have %d / %d entries, expected %d / %d" % (what, name, ptr_arr.numel(), idx.numel(), g.n + 1, e))
        p = ptr_arr.to(torch.int64)
        if int(p[0]) != 0 or int(p[-1]) != e or (g.n > 0 and bool((p[1:] < p[:-1]).any())):
            raise ValueError("%s: %s: the pointer array must start at 0, never decrease and end at E=%d" % (what, name, e))
        if e and (int(idx.min()) < 0 or int(idx.max()) >= g.n):
            raise ValueError("%s: %s: node ids must lie in [0, %d), found [%d, %d]" % (what, name, g.n, int(idx.min()), int(idx.max())))
    if g.permute is not None:
        if g.permute.dtype not in int_types or g.permute.numel() != e:
            raise ValueError("%s: permute must be an integer array of %d entries" % (what, e))
        if e and (int(g.permute.min()) < 0 or int(g.permute.max()) >= e):
            raise ValueError("%s: permute entries must lie in [0, %d)" % (what, e))


def csr_from_keys(keys: torch.Tensor, n: int) -> Graph:
    """keys = dst * n + src, sorted and unique (int64)."""
    dst = torch.div(keys, n, rounding_mode="floor")
    src = keys - dst * n
    deg = torch.bincount(dst, minlength=n)
    row_ptr = torch.zeros(n + 1, dtype=torch.int64, device=keys.device)
    row_ptr[1:] = torch.cumsum(deg, 0)
    return Graph(n, row_ptr.to(torch.int32), src.to(torch.int32))


def with_self_loops(keys: torch.Tensor, n: int) -> torch.Tensor:
    ar = torch.arange(n, dtype=torch.int64, device=keys.device)
    return torch.unique(torch.cat([keys, ar * n + ar]))


def uniform_graph(n: int, n_edges: int, seed: int = 0, device="cpu", self_loops: bool = True) -> Graph:
    """n_edges directed edges with uniform endpoints, merged, self-loops normalised (config C1)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    src = torch.randint(0, n, (n_edges,), generator=g, dtype=torch.int64)
    dst = torch.randint(0, n, (n_edges,), generator=g, dtype=torch.int64)
    keep = src != dst
    keys = torch.unique(dst[keep] * n + src[keep]).to(device)
    if self_loops:
        keys = with_self_loops(keys, n)
    return csr_from_keys(keys, n)


def _rmat_batch(count: int, scale: int, a: float, b: float, c: float, gen: torch.Generator, device):
    """One batch of R-MAT endpoints: per level pick a quadrant with probabilities (a,b,c,d);
    a/b keep the row (destination) bit 0, a/c keep the column (source) bit 0."""
    dst = torch.zeros(count, dtype=torch.int64, device=device)
    src = torch.zeros(count, dtype=torch.int64, device=device)
    for _ in range(scale):
        r = torch.rand(count, generator=gen, device=device)
        row_bit = (r >= a + b).to(torch.int64)
        col_bit = (((r >= a) & (r < a + b)) | (r >= a + b + c)).to(torch.int64)
        dst = dst * 2 + row_bit
        src = src * 2 + col_bit
    return dst, src


def rmat_graph(n: int, n_edges: int, seed: int = 0, a: float = 0.57, b: float = 0.19, c: float = 0.19,
               device="cpu", self_loops: bool = True, batch: int = 1 << 26, permute_labels: bool = False) -> Graph:
    """R-MAT power-law graph with n nodes (endpoints >= n rejected) and n_edges unique directed
    non-loop edges (fewer only if the generator saturates), plus one self-loop per node.
    permute_labels: relabel the nodes by a seeded random permutation, as the Graph500 generator does.  The raw recursion
    puts the hubs at ids that are sums of a few powers of two (0, 1, 2, 4, ...), so the rows of a feature matrix that are
    gathered most often sit at addresses with few bits set; on a graph whose features exceed the caches that alone costs
    7-18 % of a gather pass (they fall on few memory channels), and no dataset labels its nodes that way."""
    scale = max(1, math.ceil(math.log2(max(n, 2))))
    gen = torch.Generator(device=device).manual_seed(seed)
    keys = torch.empty(0, dtype=torch.int64, device=device)
    for _ in range(64):
        need = n_edges - keys.numel()
        if need <= 0:
            break
        cnt = int(min(batch, max(1 << 16, need * 2)))
        dst, src = _rmat_batch(cnt, scale, a, b, c, gen, device)
        ok = (dst < n) & (src < n) & (dst != src)
        keys = torch.unique(torch.cat([keys, dst[ok] * n + src[ok]]))
    if keys.numel() > n_edges:
        # drop a seeded random subset of the surplus (keeps the degree distribution)
        sel = torch.randperm(keys.numel(), generator=gen, device=device)[:n_edges]
        keys = torch.sort(keys[sel]).values
    if permute_labels:
        relabel = torch.randperm(n, generator=gen, device=device)
        keys = torch.sort(relabel[keys // n] * n + relabel[keys % n]).values
    if self_loops:
        keys = with_self_loops(keys, n)
    return csr_from_keys(keys, n)


def knn_graph(points: torch.Tensor, k: int) -> torch.Tensor:
    """points [B, P, D] -> src_ind int32 [B*P*k]: for every point the k nearest points of its own
    cloud (itself included), as global node ids, grouped by destination (DGL KNNGraph layout used
    by script/train/train_edgeconv_our.py:51-55)."""
    bsz, npts, _ = points.shape
    d = torch.cdist(points, points)                                   # [B,P,P]
    idx = torch.topk(d, k, dim=-1, largest=False).indices             # [B,P,k]
    off = (torch.arange(bsz, device=points.device) * npts).view(bsz, 1, 1)
    return (idx + off).reshape(-1).to(torch.int32)


def add_csc_torch(g: Graph) -> Graph:
    """CSC arrays by a stable sort with torch (host or device); the library's own csr2csc is the
    production path, this is input plumbing for tests."""
    col = g.col_ind.to(torch.int64)
    perm = torch.sort(col, stable=True).indices
    deg = (g.row_ptr[1:] - g.row_ptr[:-1]).to(torch.int64)
    rows = torch.repeat_interleave(torch.arange(g.n, device=col.device), deg)
    cnt = torch.bincount(col, minlength=g.n)
    col_ptr = torch.zeros(g.n + 1, dtype=torch.int64, device=col.device)
    col_ptr[1:] = torch.cumsum(cnt, 0)
    g.col_ptr = col_ptr.to(torch.int32)
    g.row_ind = rows[perm].to(torch.int32)
    g.permute = perm.to(torch.int32)
    return g
