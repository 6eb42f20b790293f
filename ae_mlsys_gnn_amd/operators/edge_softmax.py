"""Edge softmax: the reference's operators/edge_softmax.py surface."""
from __future__ import annotations

import torch

from .._lib import as_f32, as_i32, check, lib, ptr, require_cuda, stream_ptr


class edge_softmax_native:
    @staticmethod
    def edge_softmax(rowptr, h):
        require_cuda(rowptr, h)
        rowptr, h = as_i32(rowptr), as_f32(h)
        hh = h.view(h.shape[0], -1)
        out = torch.empty_like(hh)
        with torch.cuda.device(h.device):
            check(lib().fgnn_edge_softmax(rowptr.numel() - 1, hh.shape[0], hh.shape[1], ptr(rowptr), ptr(hh), ptr(out), stream_ptr()),
                  "fgnn_edge_softmax")
        return out.view_as(h)

    @staticmethod
    def edge_softmax_backward(rowptr, out, grad_out):
        require_cuda(rowptr, out, grad_out)
        rowptr, out, grad_out = as_i32(rowptr), as_f32(out), as_f32(grad_out)
        oo = out.view(out.shape[0], -1)
        gin = torch.empty_like(oo)
        with torch.cuda.device(out.device):
            check(lib().fgnn_edge_softmax_backward(rowptr.numel() - 1, oo.shape[0], oo.shape[1], ptr(rowptr), ptr(oo),
                                                   ptr(grad_out.view_as(oo)), ptr(gin), stream_ptr()), "fgnn_edge_softmax_backward")
        return gin.view_as(out)


def csr_edge_softmax(rowptr, h):
    return EdgeSoftmaxFunction.apply(rowptr, h)


class EdgeSoftmaxFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, h):
        out = edge_softmax_native.edge_softmax(rowptr, h)
        ctx.save_for_backward(rowptr, out)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        rowptr, out = ctx.saved_tensors
        return None, edge_softmax_native.edge_softmax_backward(rowptr, out, grad_out.contiguous())
