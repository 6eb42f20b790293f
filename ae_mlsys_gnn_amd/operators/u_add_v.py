"""u_add_v: the reference's operators/u_add_v.py surface."""
from __future__ import annotations

import torch

from .._lib import as_f32, as_i32, check, colsum_plan_for, lib, ptr, require_cuda, stream_ptr, workspace


class u_add_v_native:
    @staticmethod
    def u_add_v_forward(row_ptr, col_ind, row_val, col_val):
        require_cuda(row_ptr, col_ind, row_val, col_val)
        row_ptr, col_ind, row_val, col_val = as_i32(row_ptr), as_i32(col_ind), as_f32(row_val), as_f32(col_val)
        n = row_ptr.numel() - 1
        w = row_val.numel() // max(n, 1)
        e = col_ind.numel()
        out = torch.empty((e,) + tuple(row_val.shape[1:]), dtype=torch.float32, device=row_val.device)
        with torch.cuda.device(row_val.device):
            check(lib().fgnn_u_add_v(n, e, w, ptr(row_ptr), ptr(col_ind), ptr(row_val), ptr(col_val), ptr(out), stream_ptr()), "fgnn_u_add_v")
        return out

    @staticmethod
    def u_add_v_backward(row_ptr, col_ind, grad_out, atomics=False):
        """grad_row, grad_col of u_add_v (u_add_v.u_add_v_backward of the reference).  The column sums run under a cached
        tile-ordered plan of (row_ptr, col_ind) without atomics, bit-reproducible; atomics=True (and rows wider than the
        plan supports) selects the reference's float-atomic scatter instead."""
        require_cuda(row_ptr, col_ind, grad_out)
        row_ptr, col_ind, grad_out = as_i32(row_ptr), as_i32(col_ind), as_f32(grad_out)
        n = row_ptr.numel() - 1
        e = col_ind.numel()
        w = grad_out.numel() // max(e, 1)
        shape = (n,) + tuple(grad_out.shape[1:])
        grad_row = torch.empty(shape, dtype=torch.float32, device=grad_out.device)
        grad_col = torch.empty(shape, dtype=torch.float32, device=grad_out.device)
        planned = not atomics and e > 0 and (w <= 64 or (w % 4 == 0 and w <= 256))
        with torch.cuda.device(grad_out.device):
            if planned:
                plan = colsum_plan_for(row_ptr, col_ind, n, w)
                ws, wsb = workspace(lib().fgnn_colsum_workspace_bytes(plan.handle, w), grad_out.device)
                check(lib().fgnn_u_add_v_backward_planned(n, e, w, ptr(row_ptr), ptr(col_ind), ptr(grad_out), ptr(grad_row), ptr(grad_col),
                                                          plan.handle, ptr(ws), wsb, stream_ptr()), "fgnn_u_add_v_backward_planned")
            else:
                check(lib().fgnn_u_add_v_backward(n, e, w, ptr(row_ptr), ptr(col_ind), ptr(grad_out), ptr(grad_row), ptr(grad_col), stream_ptr()),
                      "fgnn_u_add_v_backward")
        return grad_row, grad_col


def u_add_v_op(row_ptr, col_ind, row_val, col_val):
    return u_add_v_Function.apply(row_ptr, col_ind, row_val, col_val)


class u_add_v_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, row_ptr, col_ind, row_val, col_val):
        result = u_add_v_native.u_add_v_forward(row_ptr, col_ind, row_val, col_val)
        ctx.save_for_backward(row_ptr, col_ind)
        return result

    @staticmethod
    def backward(ctx, grad_out):
        row_ptr, col_ind = ctx.saved_tensors
        grad_row, grad_col = u_add_v_native.u_add_v_backward(row_ptr, col_ind, grad_out.contiguous())
        return None, None, grad_row, grad_col
