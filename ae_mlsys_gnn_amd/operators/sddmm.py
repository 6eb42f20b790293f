"""Single-head SDDMM entry points of the reference's native `sddmm` module
(src/sddmm/sddmm.cpp:12-50): per-edge dot products of two node-feature matrices, for a CSR matrix
or an edge list."""
from __future__ import annotations

import torch

from .._lib import as_f32, as_i32, check, lib, ptr, require_cuda, stream_ptr
from .mhspmm import mhsddmm


def csr_sddmm(rowptr, colind, D1, D2):
    """out[p] = <D1[row(p),:], D2[colind[p],:]> for every CSR position p; D1, D2 are [N, F]."""
    return mhsddmm(rowptr, colind, D1.unsqueeze(1), D2.unsqueeze(1)).squeeze(1)


def coo_sddmm(rowind, colind, D1, D2):
    """out[e] = <D1[rowind[e],:], D2[colind[e],:]> for an edge list; D1, D2 are [N, F] (or [N, H, F],
    then out is [E, H])."""
    require_cuda(rowind, colind, D1, D2)
    rowind, colind, D1, D2 = as_i32(rowind), as_i32(colind), as_f32(D1), as_f32(D2)
    heads = D1.dim() == 3
    a = D1 if heads else D1.unsqueeze(1)
    b = D2 if heads else D2.unsqueeze(1)
    e, (_, h, f) = rowind.numel(), a.shape
    out = torch.empty(e, h, dtype=torch.float32, device=a.device)
    with torch.cuda.device(a.device):
        check(lib().fgnn_sddmm_coo(e, a.shape[0], b.shape[0], h, f, ptr(rowind), ptr(colind), ptr(a), ptr(b), ptr(out), stream_ptr()),
              "fgnn_sddmm_coo")
    return out if heads else out.squeeze(1)
