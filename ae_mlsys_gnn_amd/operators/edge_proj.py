"""Per-edge Linear(2, D) + Tanh of the MoNet drivers (script/train/train_gmmconv_our.py:46-57, the
`pseudo_proj` of every layer), as one fused pass over the edges each way."""
from __future__ import annotations

import torch

from .._lib import as_f32, check, lib, ptr, require_cuda, stream_ptr, workspace

MAX_OUT = 4


class EdgeLinearTanhFunction(torch.autograd.Function):
    """y = tanh(x @ W.T + b) for x [E, 2], W [D, 2], b [D], D <= 4.  The coordinates x are data: the
    backward returns the gradients of W and b only (summed over the edges in a fixed order)."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        require_cuda(x, weight, bias)
        x, w, b = as_f32(x), as_f32(weight), as_f32(bias)
        e, d = x.shape[0], w.shape[0]
        y = torch.empty((e, d), dtype=torch.float32, device=x.device)
        with torch.cuda.device(x.device):
            check(lib().fgnn_edge_linear_tanh(e, d, ptr(x), ptr(w), ptr(b), ptr(y), stream_ptr()), "fgnn_edge_linear_tanh")
        ctx.save_for_backward(x, y)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, y = ctx.saved_tensors
        e, d = y.shape
        g = as_f32(grad_y)
        grad_w = torch.empty((d, 2), dtype=torch.float32, device=x.device)
        grad_b = torch.empty((d,), dtype=torch.float32, device=x.device)
        ws, ws_bytes = workspace(lib().fgnn_edge_linear_tanh_backward_workspace_bytes(e, d), x.device)
        with torch.cuda.device(x.device):
            check(lib().fgnn_edge_linear_tanh_backward(e, d, ptr(x), ptr(y), ptr(g), ptr(grad_w), ptr(grad_b), ptr(ws), ws_bytes, stream_ptr()),
                  "fgnn_edge_linear_tanh_backward")
        return None, grad_w, grad_b


def edge_linear_tanh(x, weight, bias):
    """tanh(x @ weight.T + bias) over the edges; x [E, 2] (not differentiated), weight [D, 2], bias [D], D <= 4."""
    if x.dim() != 2 or x.shape[1] != 2 or weight.shape[0] > MAX_OUT:
        raise ValueError("edge_linear_tanh: x must be [E, 2] and weight [D, 2] with D <= %d" % MAX_OUT)
    return EdgeLinearTanhFunction.apply(x, weight, bias)
