"""Single-head SpMM: the reference's operators/spmm.py surface (its own native sources are
missing from the reference tree; the semantics follow the Python of operators/spmm.py:25-66)."""
from __future__ import annotations

import torch

from .._lib import FgnnError
from .csr2csc import csr2csc
from .mhspmm import mhsddmm, mhspmm


def csrspmm(rowptr, colind, x, csr_data, sym=False, actnn=False):
    if actnn:
        raise FgnnError("csrspmm(actnn=True) needs the third-party actnn package, which this build does not provide")
    return SPMMFunction.apply(rowptr, colind, x, csr_data, sym)


class SPMMFunction(torch.autograd.Function):
    """out[i,:] = sum_p w[p] * x[colind[p],:] (w = 1 when csr_data is None).  Backward over the
    transpose (the matrix itself when sym), edge-weight gradient by SDDMM when requested."""

    @staticmethod
    def forward(ctx, rowptr, colind, feat, edge_weight_csr=None, sym=False):
        att = None if edge_weight_csr is None else edge_weight_csr.reshape(-1, 1)
        out = mhspmm(rowptr, colind, att, feat.unsqueeze(1)).squeeze(1)
        ctx.save_for_backward(rowptr, colind, feat, edge_weight_csr)
        ctx.sym = sym
        return out

    @staticmethod
    def backward(ctx, grad_out):
        rowptr, colind, feat, edge_weight_csr = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        att = None if edge_weight_csr is None else edge_weight_csr.reshape(-1, 1)
        if ctx.sym:
            grad_feat = mhspmm(rowptr, colind, att, grad_out.unsqueeze(1)).squeeze(1)
        else:
            colptr, rowind, permute = csr2csc(rowptr, colind)
            grad_feat = mhspmm(colptr, rowind, att, grad_out.unsqueeze(1), pos_map=permute).squeeze(1)
        grad_edge_weight = None
        if edge_weight_csr is not None and ctx.needs_input_grad[3]:
            grad_edge_weight = mhsddmm(rowptr, colind, grad_out.unsqueeze(1), feat.unsqueeze(1)).reshape(edge_weight_csr.shape)
        return None, None, grad_feat, grad_edge_weight, None
