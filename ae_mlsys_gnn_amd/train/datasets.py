"""Data for the training drivers.

Node-classification graphs (the datasets of the reference's script/train/train_gatconv_our.py:71-81
and train_gmmconv_our.py:97-104) come from local files when they are there and are generated at
the published shape otherwise; nothing is ever downloaded.

Accepted files under --data-root:
  <name>.npz                     keys src, dst (directed edges src -> dst), feat [N,D], label [N],
                                 train_mask, val_mask, test_mask [N] bool
  reddit/reddit_data.npz +       the layout of DGL's Reddit download: feature, label, node_types
  reddit/reddit_graph.npz        (1 train, 2 validation, 3 test) and a scipy-saved adjacency
Point clouds (train_edgeconv_our.py:86-137): <file>.npz with data [M,P,3] float32 and label [M]; an
HDF5 file with train/data and train/label is read when h5py is importable.

Graph arrays are built on the device by the library itself: self-loops removed and added once per
node (train_gatconv_our.py:84-85), COO -> CSR by destination, CSR -> CSC with the permutation."""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .. import graphs
from ..operators import csr2csc as csc_op

# nodes, directed edges before self-loops, input features, classes
SHAPES = {
    "cora": (2708, 10556, 1433, 7),
    "citeseer": (3327, 9228, 3703, 6),
    "pubmed": (19717, 88651, 500, 3),
    "reddit": (232965, 114615892, 602, 41),
    "ogbn-arxiv": (169343, 2315598, 128, 40),
    "ogbn-products": (2449029, 61859140, 100, 47),
}


@dataclass
class NodeData:
    name: str
    source: str                       # "file:<path>" or "synthetic"
    graph: graphs.Graph               # device arrays incl. CSC and permute
    feat: torch.Tensor                # [N, D] float32
    label: torch.Tensor               # [N] int64
    train_mask: torch.Tensor
    val_mask: torch.Tensor
    test_mask: torch.Tensor
    n_classes: int


def graph_from_edges(src, dst, n, device, self_loops=True, dedupe=False) -> graphs.Graph:
    """Directed edges src -> dst (any integer tensors) -> CSR by destination + CSC + permute, all on
    `device` through fgnn_coo2csr / fgnn_csr2csc.  Duplicate edges stay independent edges unless
    `dedupe`; with `self_loops` every node ends up with exactly one."""
    src, dst = torch.as_tensor(src), torch.as_tensor(dst)
    # checked in the file's own integer type, before the cast to int32 could wrap an id into range and
    # before any kernel indexes a feature row with it
    for name, t in (("src", src), ("dst", dst)):
        if t.dtype.is_floating_point or t.dtype == torch.bool or t.dim() != 1:
            raise ValueError("graph_from_edges: %s must be a 1-D integer array, got %s %s" % (name, t.dtype, tuple(t.shape)))
        if t.numel() and (int(t.min()) < 0 or int(t.max()) >= n):
            raise ValueError("graph_from_edges: %s ids must lie in [0, %d), found [%d, %d]" % (name, n, int(t.min()), int(t.max())))
    if src.numel() != dst.numel():
        raise ValueError("graph_from_edges: %d sources for %d destinations" % (src.numel(), dst.numel()))
    if not 0 <= n <= 2147483647 or src.numel() + (n if self_loops else 0) > 2147483647:
        raise ValueError("graph_from_edges: node or edge count exceeds int32")
    src = src.to(device=device, dtype=torch.int32)
    dst = dst.to(device=device, dtype=torch.int32)
    if self_loops:
        keep = src != dst
        ar = torch.arange(n, dtype=torch.int32, device=device)
        src, dst = torch.cat([src[keep], ar]), torch.cat([dst[keep], ar])
    row_ptr, col_ind = csc_op.coo2csr(dst.contiguous(), src.contiguous(), n, dedupe=dedupe)
    col_ind = col_ind.contiguous()
    col_ptr, row_ind, permute = csc_op.csr2csc(row_ptr, col_ind)
    return graphs.Graph(n, row_ptr, col_ind, col_ptr, row_ind, permute)


def save_graph(path, g: graphs.Graph):
    """On-disk cache of the preprocessed arrays (plain .npz, no pickles)."""
    np.savez(path, n=np.int64(g.n), **{k: getattr(g, k).cpu().numpy() for k in ("row_ptr", "col_ind", "col_ptr", "row_ind", "permute")})


def load_graph(path, device) -> graphs.Graph:
    with np.load(path, allow_pickle=False) as z:
        host = {k: torch.from_numpy(z[k]) for k in ("row_ptr", "col_ind", "col_ptr", "row_ind", "permute")}
        n = int(z["n"])
    # a cache file is untrusted input: every id is range-checked on the host before anything reaches the device
    graphs.validate_graph(graphs.Graph(n, **host), what=str(path))
    return graphs.Graph(n, **{k: v.to(device=device, dtype=torch.int32) for k, v in host.items()})


def _masks_from_types(node_types):
    t = torch.from_numpy(np.asarray(node_types))
    return t == 1, t == 2, t == 3


def _read_node_files(name, root):
    """Returns (src, dst, feat, label, train, val, test, path) from local files, or None."""
    if not root:
        return None
    own = os.path.join(root, name + ".npz")
    if os.path.exists(own):
        with np.load(own, allow_pickle=False) as z:
            return (torch.from_numpy(z["src"]), torch.from_numpy(z["dst"]), torch.from_numpy(z["feat"]).float(),
                    torch.from_numpy(z["label"]).long(), torch.from_numpy(z["train_mask"]).bool(),
                    torch.from_numpy(z["val_mask"]).bool(), torch.from_numpy(z["test_mask"]).bool(), own)
    if name == "reddit":
        d, gfile = os.path.join(root, "reddit", "reddit_data.npz"), os.path.join(root, "reddit", "reddit_graph.npz")
        if os.path.exists(d) and os.path.exists(gfile):
            import scipy.sparse as sp
            adj = sp.load_npz(gfile).tocoo()                      # refuses pickled content by default
            with np.load(d, allow_pickle=False) as z:
                tr, va, te = _masks_from_types(z["node_types"])
                return (torch.from_numpy(adj.row.astype(np.int64)), torch.from_numpy(adj.col.astype(np.int64)),
                        torch.from_numpy(z["feature"]).float(), torch.from_numpy(z["label"]).long(), tr, va, te, d)
    return None


def load_node_dataset(name, device, root=None, seed=0, scale=1.0, cache_dir=None) -> NodeData:
    """The named dataset from local files under `root`, else an R-MAT graph with the dataset's node,
    edge, feature and class counts (times `scale`, for quick runs), N(0,1) features, uniform labels
    and a 66/10/24 split.  With `cache_dir` the preprocessed graph arrays are kept on disk."""
    if name not in SHAPES:
        raise ValueError("Unknown dataset: {}".format(name))
    files = _read_node_files(name, root)
    cache = os.path.join(cache_dir, "%s_%s_%g.graph.npz" % (name, "file" if files else "synthetic%d" % seed, scale)) if cache_dir else None
    if files is not None:
        src, dst, feat, label, tr, va, te, path = files
        n = feat.shape[0]
        g = load_graph(cache, device) if cache and os.path.exists(cache) else graph_from_edges(src, dst, n, device)
        source, n_classes = "file:" + path, int(label.max()) + 1
    else:
        n0, e0, d, n_classes = SHAPES[name]
        n, e = max(8, int(n0 * scale)), max(8, int(e0 * scale))
        if cache and os.path.exists(cache):
            g = load_graph(cache, device)
        else:
            r = graphs.rmat_graph(n, e, seed=seed, device=device, self_loops=False)
            deg = (r.row_ptr[1:] - r.row_ptr[:-1]).long()
            dst = torch.repeat_interleave(torch.arange(n, device=device), deg)
            g = graph_from_edges(r.col_ind, dst, n, device)
            del r, dst
        gen = torch.Generator(device="cpu").manual_seed(seed + 1)
        feat = torch.randn(n, d, generator=gen)
        label = torch.randint(0, n_classes, (n,), generator=gen)
        u = torch.rand(n, generator=gen)
        tr, va, te = u < 0.66, (u >= 0.66) & (u < 0.76), u >= 0.76
        source = "synthetic"
    if cache and not os.path.exists(cache):
        os.makedirs(cache_dir, exist_ok=True)
        save_graph(cache, g)
    return NodeData(name, source, g, feat.to(device), label.to(device), tr.to(device), va.to(device), te.to(device), n_classes)


def degree_pseudo(g: graphs.Graph) -> torch.Tensor:
    """MoNet's pseudo-coordinates per CSR position: (1/sqrt(deg(source)), 1/sqrt(deg(destination)))
    with in-degrees, as train_gmmconv_our.py:112-114 builds them."""
    deg = (g.row_ptr[1:] - g.row_ptr[:-1]).float()
    inv = torch.rsqrt(deg.clamp(min=1))
    dst = torch.repeat_interleave(torch.arange(g.n, device=deg.device), deg.long())
    return torch.stack([inv[g.col_ind.long()], inv[dst]], dim=1).contiguous()


@dataclass
class CloudData:
    source: str
    data: torch.Tensor                # [M, P, 3] float32 on the device
    label: torch.Tensor               # [M] int64
    n_classes: int


def load_point_clouds(device, path: Optional[str] = None, n_clouds=9840, n_points=1024, n_classes=40, seed=0) -> CloudData:
    """ModelNet40-shaped training clouds: from `path` (.npz, or .h5 with h5py) truncated to n_points
    per cloud as train_edgeconv_our.py:128 does, else uniform random points in [-1, 1]^3."""
    if path:
        if path.endswith(".npz"):
            with np.load(path, allow_pickle=False) as z:
                data, label = z["data"], z["label"]
        else:
            try:
                import h5py
            except ImportError as exc:
                raise RuntimeError("reading %s needs h5py, which is not installed; convert it to .npz (data, label)" % path) from exc
            with h5py.File(path, "r") as f:
                data, label = f["train/data"][:], f["train/label"][:]
        data = torch.from_numpy(np.asarray(data, dtype=np.float32))[:, :n_points].contiguous()
        label = torch.from_numpy(np.asarray(label)).long().view(-1)
        return CloudData("file:" + path, data.to(device), label.to(device), int(label.max()) + 1)
    gen = torch.Generator(device="cpu").manual_seed(seed)
    data = torch.rand(n_clouds, n_points, 3, generator=gen) * 2 - 1
    label = torch.randint(0, n_classes, (n_clouds,), generator=gen)
    return CloudData("synthetic", data.to(device), label.to(device), n_classes)
