"""CSR -> CSC transpose: the reference's operators/csr2csc.py surface, on the library's own
stable GPU transpose instead of cuSPARSE."""
from __future__ import annotations

import torch

from .._lib import as_i32, check, lib, ptr, require_cuda, stream_ptr, workspace


def csr2csc(rowptr, colind, n_cols=None):
    """Returns (col_ptr, row_ind, permute) int32; permute[q] = CSR position of CSC entry q."""
    require_cuda(rowptr, colind)
    rowptr, colind = as_i32(rowptr), as_i32(colind)
    n = rowptr.numel() - 1
    nc = n if n_cols is None else int(n_cols)
    e = colind.numel()
    dev = colind.device
    col_ptr = torch.empty(nc + 1, dtype=torch.int32, device=dev)
    row_ind = torch.empty(e, dtype=torch.int32, device=dev)
    permute = torch.empty(e, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        ws, wsb = workspace(lib().fgnn_csr2csc_workspace_bytes(n, nc, e), dev)
        check(lib().fgnn_csr2csc(n, nc, e, ptr(rowptr), ptr(colind), ptr(col_ptr), ptr(row_ind), ptr(permute), ptr(ws), wsb,
                                 stream_ptr()), "fgnn_csr2csc")
    return col_ptr, row_ind, permute


def sparsetrans(rowptr, colind, numlist):
    """operators/csr2csc.py:14-16: the values of `numlist` (CSR order) in CSC order."""
    _, _, permute = csr2csc(rowptr, colind)
    return numlist[permute.long()]


def coo2csr(dst, src, n_rows, n_cols=None, dedupe=True, return_edge_pos=False):
    """Edge list -> (row_ptr, col_ind[, edge_pos]) int32 on the device: CSR by destination, sources
    ascending inside a row, duplicate edges merged when `dedupe`.  edge_pos[e] is the CSR position of
    input edge e.  The scipy call of the reference's drivers, done on the GPU."""
    require_cuda(dst, src)
    dst, src = as_i32(dst), as_i32(src)
    e = dst.numel()
    nc = n_rows if n_cols is None else int(n_cols)
    dev = dst.device
    row_ptr = torch.empty(n_rows + 1, dtype=torch.int32, device=dev)
    col_ind = torch.empty(e, dtype=torch.int32, device=dev)
    n_out = torch.zeros(1, dtype=torch.int64, device=dev)
    edge_pos = torch.empty(e, dtype=torch.int32, device=dev) if return_edge_pos else None
    with torch.cuda.device(dev):
        ws, wsb = workspace(lib().fgnn_coo2csr_workspace_bytes(n_rows, nc, e), dev)
        check(lib().fgnn_coo2csr(n_rows, nc, e, ptr(dst), ptr(src), int(bool(dedupe)), ptr(row_ptr), ptr(col_ind), ptr(n_out),
                                 ptr(edge_pos), ptr(ws), wsb, stream_ptr()), "fgnn_coo2csr")
    col_ind = col_ind[: int(n_out.item())]
    return (row_ptr, col_ind, edge_pos) if return_edge_pos else (row_ptr, col_ind)
