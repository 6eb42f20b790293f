"""Softmax cross-entropy of the training drivers as one fused pass each way (fgnn_cross_entropy_forward / _backward)."""
from __future__ import annotations

import torch

from .._lib import FgnnError, check, lib, ptr, require_cuda, stream_ptr


class CrossEntropyRows(torch.autograd.Function):
    """row_loss[i] = logsumexp(logits[i, :C]) - logits[i, labels[i]] for a float32 [N, >= C] array whose rows may be
    views of a wider (padded) array: it is read in place, and the gradient comes back in the logits' full width with
    zeros in the columns beyond C."""

    @staticmethod
    def forward(ctx, logits, labels, n_classes):
        require_cuda(logits, labels)
        if logits.dtype != torch.float32 or logits.dim() != 2 or (logits.shape[1] > 1 and logits.stride(1) != 1):
            raise FgnnError("cross entropy: logits must be a float32 [N, C] array with contiguous rows, got %s %s strides %s" % (
                logits.dtype, tuple(logits.shape), logits.stride()))
        if labels.dtype != torch.int64 or labels.shape != (logits.shape[0],):
            raise FgnnError("cross entropy: labels must be int64 [N], got %s %s" % (labels.dtype, tuple(labels.shape)))
        labels = labels.contiguous()
        n, width = logits.shape
        c = width if n_classes is None else int(n_classes)
        if not 1 <= c <= width:
            raise FgnnError("cross entropy: %d classes in rows of %d logits" % (c, width))
        ld = logits.stride(0) if n > 1 else max(width, 1)
        if ld < width:
            raise FgnnError("cross entropy: overlapping logits rows (stride %d < %d)" % (ld, width))
        lse = torch.empty(n, dtype=torch.float32, device=logits.device)
        row_loss = torch.empty(n, dtype=torch.float32, device=logits.device)
        with torch.cuda.device(logits.device):
            check(lib().fgnn_cross_entropy_forward(n, c, ld, ptr(logits), ptr(labels), ptr(lse), ptr(row_loss), stream_ptr()),
                  "fgnn_cross_entropy_forward")
        ctx.save_for_backward(logits, labels, lse)
        ctx.c, ctx.ld = c, ld
        return row_loss

    @staticmethod
    def backward(ctx, grad_rows):
        logits, labels, lse = ctx.saved_tensors
        n, width = logits.shape
        grad = torch.empty((n, width), dtype=torch.float32, device=logits.device)
        up = grad_rows.contiguous()
        with torch.cuda.device(logits.device):
            check(lib().fgnn_cross_entropy_backward(n, ctx.c, ctx.ld, width, ptr(logits), ptr(labels), ptr(lse), ptr(up), ptr(grad),
                                                    stream_ptr()), "fgnn_cross_entropy_backward")
        return grad, None, None


def cross_entropy_rows(logits, labels, n_classes=None):
    return CrossEntropyRows.apply(logits, labels, n_classes)
