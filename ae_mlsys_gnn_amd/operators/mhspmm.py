"""Multi-head SpMM / SDDMM / permuted gather: the reference's operators/mhspmm.py surface."""
from __future__ import annotations

import torch

from .._lib import FgnnError, as_f32, as_i32, check, lib, ptr, require_cuda, schedule_for, stream_ptr, workspace, xcd_buckets_enabled


def mhspmm(ptr_arr, idx, attention, feat, pos_map=None, own_order=False):
    """mhspmm.mhspmm(rowptr, colind, attention, feat) (src/spmm/mhspmm.cc): out[i,h,:] = sum_p att[p,h]*feat[idx[p],h,:].
    own_order: attention (or pos_map, when given) is indexed by the entry order of the work list of (ptr_arr, idx)
    (_lib.own_order_view), not by the caller's positions."""
    require_cuda(ptr_arr, idx, feat)
    ptr_arr, idx, feat = as_i32(ptr_arr), as_i32(idx), as_f32(feat)
    attention = None if attention is None else as_f32(attention)
    if pos_map is not None:
        require_cuda(pos_map)
        pos_map = as_i32(pos_map)
        if pos_map.numel() != idx.numel():
            raise FgnnError("mhspmm: pos_map has %d entries, expected %d" % (pos_map.numel(), idx.numel()))
    n, h, f = feat.shape
    e = idx.numel()
    if attention is not None and attention.shape != (e, h):
        raise FgnnError("mhspmm: attention is %s, expected (%d, %d)" % (tuple(attention.shape), e, h))
    out = torch.empty((ptr_arr.numel() - 1, h, f), dtype=torch.float32, device=feat.device)
    sched = schedule_for(ptr_arr, idx_tensor=idx, n_cols=n, own_order=own_order)          # the ids index the rows of feat
    with torch.cuda.device(feat.device):
        # unweighted: only the partial results of split rows (the same figure as the GMMConv forward's)
        need = (lib().fgnn_mhspmm_workspace_bytes if attention is not None else lib().fgnn_gmm_forward_workspace_bytes)(sched.handle, h, f)
        ws, wsb = workspace(need, feat.device)
        check(lib().fgnn_mhspmm(ptr_arr.numel() - 1, e, h, f, ptr(ptr_arr), ptr(idx), ptr(pos_map), ptr(attention), ptr(feat),
                                ptr(out), sched.handle, ptr(ws), wsb, stream_ptr()), "fgnn_mhspmm")
    return out


def mhsddmm(rowptr, colind, grad, feat, own_order=False):
    """mhsddmm.mhsddmm (src/sddmm/mhsddmm.cc): out[p,h] = <grad[row(p),h,:], feat[colind[p],h,:]>.
    own_order: the result is written in the entry order of the work list of (rowptr, colind) (_lib.own_order_view)."""
    require_cuda(rowptr, colind, grad, feat)
    rowptr, colind, grad, feat = as_i32(rowptr), as_i32(colind), as_f32(grad), as_f32(feat)
    n, h, f = feat.shape
    e = colind.numel()
    out = torch.empty((e, h), dtype=torch.float32, device=feat.device)
    # a skewed graph is walked under its XCD-aware work list (each XCD then gathers from one eighth of the feature
    # rows); otherwise the kernel cuts the entry array into equal chunks itself and needs no list
    sched = schedule_for(rowptr, idx_tensor=colind, n_cols=n, own_order=own_order) if e and xcd_buckets_enabled(rowptr, e) else None
    with torch.cuda.device(feat.device):
        if sched is not None:
            check(lib().fgnn_mhsddmm_scheduled(rowptr.numel() - 1, e, h, f, ptr(rowptr), ptr(colind), ptr(grad), ptr(feat), ptr(out),
                                               sched.handle, stream_ptr()), "fgnn_mhsddmm_scheduled")
        else:
            check(lib().fgnn_mhsddmm(rowptr.numel() - 1, e, h, f, ptr(rowptr), ptr(colind), ptr(grad), ptr(feat), ptr(out), stream_ptr()),
                  "fgnn_mhsddmm")
    return out


def mhtranspose(permute, attention):
    """mhtranspose.mhtranspose (src/csr2csc/mhtranspose.cc): out[q,:] = attention[permute[q],:]."""
    require_cuda(permute, attention)
    permute, attention = as_i32(permute), as_f32(attention)
    e = permute.numel()
    w = attention.numel() // max(e, 1) if e else (attention.shape[1] if attention.dim() > 1 else 1)
    out = torch.empty_like(attention)
    with torch.cuda.device(attention.device):
        check(lib().fgnn_gather_rows(e, max(w, 1), ptr(permute), ptr(attention), ptr(out), stream_ptr()), "fgnn_gather_rows")
    return out


def csrmhspmm(rowptr, colind, colptr, rowind, permute, feat, attention):
    return MHSPMMFunction.apply(rowptr, colind, colptr, rowind, permute, feat, attention)


class MHSPMMFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, permute, feat, attention):
        out = mhspmm(rowptr, colind, attention, feat)
        ctx.save_for_backward(rowptr, colind, colptr, rowind, permute, feat, attention)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        rowptr, colind, colptr, rowind, permute, feat, attention = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        # the CSC pass reads attention[permute[q]] directly instead of materialising the transpose
        grad_feat = mhspmm(colptr, rowind, attention, grad_out, pos_map=as_i32(permute))
        grad_edge_weight = mhsddmm(rowptr, colind, grad_out, feat)
        return None, None, None, None, None, grad_feat, grad_edge_weight
