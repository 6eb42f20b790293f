"""k-nearest-neighbour graph builder for batched point clouds (the graph fused EdgeConv consumes).
The reference calls DGL's KNNGraph for this (script/train/train_edgeconv_our.py:51-55)."""
from __future__ import annotations

import torch

from .._lib import FgnnError, as_f32, check, lib, ptr, require_cuda, stream_ptr


def knn_graph(points, k):
    """points [B, P, D] (or [B*P, D] with n_clouds given by the first form only) -> src_ind int32
    [B*P*k]: for every point the k nearest points of its own cloud, itself included, nearest first,
    as global node ids grouped by destination."""
    require_cuda(points)
    points = as_f32(points)
    if points.dim() != 3:
        raise FgnnError("knn_graph expects points of shape [clouds, points, dims], got %s" % (tuple(points.shape),))
    b, p, d = points.shape
    out = torch.empty(b * p * int(k), dtype=torch.int32, device=points.device)
    with torch.cuda.device(points.device):
        check(lib().fgnn_knn_graph(b, p, d, int(k), ptr(points), ptr(out), stream_ptr()), "fgnn_knn_graph")
    return out
