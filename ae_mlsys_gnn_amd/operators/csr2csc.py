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
