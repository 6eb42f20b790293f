"""Fused EdgeConv operator: the reference's operators/fused_edgeconv.py surface on libfgnn_hip.so."""
from __future__ import annotations

import torch

from .._lib import FgnnError, as_f32, as_i32, check, lib, ptr, require_cuda, stream_ptr, workspace


class edgeconv_native:
    """fused_edgeconv.edgeconv_forward / edgeconv_backward (src/fused_edgeconv/fused_edgeconv.cpp:12-51)."""

    @staticmethod
    def edgeconv_forward(k, src_ind, h_src, h_dst, out_slope=None):
        """out_slope: LeakyReLU slope applied to the maxima on the way out (None: the reference's operator)."""
        require_cuda(src_ind, h_src, h_dst)
        src_ind, h_src, h_dst = as_i32(src_ind), as_f32(h_src), as_f32(h_dst)
        n, f = h_dst.shape
        if h_src.shape[1] != f or src_ind.numel() != n * int(k):
            raise FgnnError("edgeconv: src_ind has %d entries, expected N*k = %d*%d; feature widths %d vs %d" % (
                src_ind.numel(), n, int(k), h_src.shape[1], f))
        out = torch.empty_like(h_dst)
        max_idx = torch.empty((n, f), dtype=torch.int32, device=h_dst.device)
        with torch.cuda.device(h_dst.device):
            if out_slope is None:
                check(lib().fgnn_edgeconv_forward(n, h_src.shape[0], f, int(k), ptr(src_ind), ptr(h_src), ptr(h_dst), ptr(out),
                                                  ptr(max_idx), stream_ptr()), "fgnn_edgeconv_forward")
            else:
                check(lib().fgnn_edgeconv_forward_lrelu(n, h_src.shape[0], f, int(k), ptr(src_ind), ptr(h_src), ptr(h_dst), float(out_slope),
                                                        ptr(out), ptr(max_idx), stream_ptr()), "fgnn_edgeconv_forward_lrelu")
        return out, max_idx

    @staticmethod
    def edgeconv_backward_lrelu(grad_out, max_idx, out, out_slope, n_src=None, block=None):
        """Backward of edgeconv_forward(out_slope=...): (grad_src, grad_dst), the LeakyReLU mask replayed from `out`."""
        require_cuda(grad_out, max_idx, out)
        grad_out, max_idx, out = as_f32(grad_out), as_i32(max_idx), as_f32(out)
        n, f = grad_out.shape
        if tuple(out.shape) != (n, f) or tuple(max_idx.shape) != (n, f):
            raise FgnnError("edgeconv_backward_lrelu: out %s / argmax %s do not match grad_out %s" % (tuple(out.shape), tuple(max_idx.shape), (n, f)))
        n_src = n if n_src is None else n_src
        grad_src = torch.empty((n_src, f), dtype=torch.float32, device=grad_out.device)
        grad_dst = torch.empty_like(grad_out)
        with torch.cuda.device(grad_out.device):
            ws, wsb = workspace(lib().fgnn_edgeconv_backward_blocked_workspace_bytes(n, f), grad_out.device) if block else (None, 0)
            check(lib().fgnn_edgeconv_backward_lrelu(n, n_src, f, int(block or 0), ptr(max_idx), ptr(out), float(out_slope), ptr(grad_out),
                                                     ptr(grad_src), ptr(grad_dst), ptr(ws), wsb, stream_ptr()), "fgnn_edgeconv_backward_lrelu")
        return grad_src, grad_dst

    @staticmethod
    def edgeconv_backward(grad_out, max_idx, n_src=None, block=None):
        """block: points per cloud when the graph is a kNN graph of equally sized point clouds (a hint:
        neighbours outside a node's own block are still handled, just more slowly)."""
        require_cuda(grad_out, max_idx)
        grad_out, max_idx = as_f32(grad_out), as_i32(max_idx)
        n, f = grad_out.shape
        n_src = n if n_src is None else n_src
        grad_src = torch.empty((n_src, f), dtype=torch.float32, device=grad_out.device)
        with torch.cuda.device(grad_out.device):
            if block:
                ws, wsb = workspace(lib().fgnn_edgeconv_backward_blocked_workspace_bytes(n, f), grad_out.device)
                check(lib().fgnn_edgeconv_backward_blocked(n, n_src, f, int(block), ptr(max_idx), ptr(grad_out), ptr(grad_src), ptr(ws), wsb,
                                                           stream_ptr()), "fgnn_edgeconv_backward_blocked")
            else:
                check(lib().fgnn_edgeconv_backward(n, n_src, f, ptr(max_idx), ptr(grad_out), ptr(grad_src), stream_ptr()),
                      "fgnn_edgeconv_backward")
        return grad_src


def fused_edgeconv_op(k, src_ind, h_src, h_dst, block=None, negative_slope_out=None):
    """block (optional, not in the reference): points per cloud of a batched kNN graph; lets the backward
    accumulate per cloud in LDS instead of scattering with global atomics.
    negative_slope_out (optional, not in the reference): fuse the LeakyReLU that follows the operator in the
    reference's DGCNN stack (script/train/train_edgeconv_our.py:56) into both passes; must be positive."""
    return FusedEdgeConvFunction.apply(k, src_ind, h_src, h_dst, block, negative_slope_out)


class FusedEdgeConvFunction(torch.autograd.Function):
    """out[i,f] = h_dst[i,f] + max_j h_src[j,f] over the k neighbours of i; the argmax (int32 source
    node id, first maximum wins) is kept for the backward (operators/fused_edgeconv.py:18-29)."""

    @staticmethod
    def forward(ctx, k, src_ind, h_src, h_dst, block=None, negative_slope_out=None):
        ctx.n_src = h_src.shape[0]
        ctx.block = block
        ctx.slope = negative_slope_out
        if negative_slope_out is None:
            out_feat, max_idx = edgeconv_native.edgeconv_forward(k, src_ind, h_src, h_dst)
            ctx.save_for_backward(max_idx)
        else:
            out_feat, max_idx = edgeconv_native.edgeconv_forward(k, src_ind, h_src, h_dst, out_slope=negative_slope_out)
            ctx.save_for_backward(max_idx, out_feat)
        return out_feat

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = grad_out.contiguous()
        if ctx.slope is None:
            max_idx = ctx.saved_tensors[0]
            grad_src = edgeconv_native.edgeconv_backward(grad_out, max_idx, ctx.n_src, ctx.block)
            return None, None, grad_src, grad_out, None, None
        max_idx, out_feat = ctx.saved_tensors
        grad_src, grad_dst = edgeconv_native.edgeconv_backward_lrelu(grad_out, max_idx, out_feat, ctx.slope, ctx.n_src, ctx.block)
        return None, None, grad_src, grad_dst, None, None
