"""Fused GAT operators: the reference's operators/fused_gat.py surface on libfgnn_hip.so.

``fused_gat_op`` / ``FusedGATFunction_SM``        recompute variant (operators/fused_gat.py:30-31,52-71)
``fused_gat_stash_op`` / ``FusedGATFunction_stash``  stash variant  (operators/fused_gat.py:33-34,73-86)
``fused_gat_fusescatter`` / ``FusedGATFunction``  fuse-scatter variant (operators/fused_gat.py:27-28,36-50)

The recompute and stash variants share one forward kernel and one backward kernel; the stash variant additionally
writes / reads the per-edge ``[E,H]`` softmax tensor.  What the recompute variant keeps for the backward is
node-sized only: ``out``, ``out2`` ([N,H,F]) and three ``[N,H]`` arrays.  The fuse-scatter variant is the reference's
unfused-SpMM data flow (scatter kernel -> [E,H] -> SpMM), kept for the ablation it stands for.
"""
from __future__ import annotations

import torch

from .. import _lib
from .._lib import as_f32, as_i32, check, colsum_plan_for, lib, ptr, require_cuda, schedule_for, stream_ptr, workspace


class gat_native:
    """Native entry points with the argument order of the reference's pybind modules
    (fused_gat_SM.gat_forward / gat_backward, src/fused_gat/fused_gat_SM.cpp:14-124)."""

    @staticmethod
    def gat_forward(attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat, *, need_aux=True, stash=False,
                    stash_lrelu=True, use_schedule=True):
        require_cuda(attn_row, attn_col, row_ptr, col_ind, in_feat)
        attn_row, attn_col, in_feat = as_f32(attn_row), as_f32(attn_col), as_f32(in_feat)
        row_ptr, col_ind = as_i32(row_ptr), as_i32(col_ind)
        if in_feat.dim() != 3:
            raise _lib.FgnnError("in_feat must be [N,H,F], got %s" % (tuple(in_feat.shape),))
        n, h, f = in_feat.shape
        e = col_ind.numel()
        if attn_row.shape != (n, h) or attn_col.shape != (n, h) or row_ptr.numel() != n + 1:
            raise _lib.FgnnError("shape mismatch: attn_row %s attn_col %s row_ptr %s for N=%d H=%d" % (
                tuple(attn_row.shape), tuple(attn_col.shape), tuple(row_ptr.shape), n, h))
        dev = in_feat.device
        out = torch.empty_like(in_feat)
        edge_max = torch.empty((n, h), dtype=torch.float32, device=dev)
        edge_sum = torch.empty((n, h), dtype=torch.float32, device=dev)
        out2 = torch.empty_like(in_feat) if need_aux else None
        cc = torch.empty((n, h), dtype=torch.float32, device=dev) if need_aux else None
        e_lrelu = torch.empty((e, h), dtype=torch.float32, device=dev) if (stash and stash_lrelu) else None
        e_soft = torch.empty((e, h), dtype=torch.float32, device=dev) if stash else None
        sched = schedule_for(row_ptr, idx_tensor=col_ind, need_positions=False, n_cols=n) if use_schedule else None
        sh = sched.handle if sched is not None else None
        with torch.cuda.device(dev):
            ws, wsb = workspace(lib().fgnn_gat_forward_workspace_bytes(sh, h, f), dev)
            check(lib().fgnn_gat_forward(n, e, h, f, ptr(attn_row), ptr(attn_col), ptr(row_ptr), ptr(col_ind),
                                         float(negative_slope), ptr(in_feat), ptr(out), ptr(edge_max), ptr(edge_sum),
                                         ptr(out2), ptr(cc), ptr(e_lrelu), ptr(e_soft), sh, ptr(ws), wsb, stream_ptr()),
                  "fgnn_gat_forward")
        return out, edge_max, edge_sum, out2, cc, e_lrelu, e_soft

    @staticmethod
    def gat_backward(negative_slope, row_ptr, col_ind, col_ptr, row_ind, edge_max, edge_sum, in_feat, attn_row, attn_col,
                     grad, *, out_feat=None, out2=None, cc=None, permute=None, e_lrelu=None, e_soft=None, e_soft_order="csr",
                     use_schedule=True):
        """e_soft: stashed attention [E,H].  e_soft_order="csr": the CSR-ordered stash of gat_forward(stash=True), read
        through `permute` (required); e_soft_order="own": the stash of gat_stash_own_order (entry order of this pass,
        signed), streamed.  The two layouts are not interchangeable and nothing in the data tells them apart."""
        if e_soft_order not in ("csr", "own"):
            raise _lib.FgnnError("gat_backward: e_soft_order must be 'csr' or 'own', got %r" % (e_soft_order,))
        own = e_soft is not None and e_soft_order == "own"
        if e_soft is not None and not own and permute is None:
            raise _lib.FgnnError("gat_backward: stashed attention needs permute (pass e_soft_order='own' for a stash written by "
                                 "gat_stash_own_order)")
        require_cuda(grad, in_feat, col_ptr, row_ind, attn_row, attn_col, edge_max, edge_sum, row_ptr, col_ind, out_feat, out2, cc,
                     permute, e_soft)
        # the kernels take raw pointers: every tensor is made contiguous and checked here, so a strided view
        # (or a tensor of another shape) can neither give wrong gradients nor be read past its storage
        grad, in_feat, attn_row, attn_col = as_f32(grad), as_f32(in_feat), as_f32(attn_row), as_f32(attn_col)
        edge_max, edge_sum = as_f32(edge_max), as_f32(edge_sum)
        if in_feat.dim() != 3:
            raise _lib.FgnnError("in_feat must be [N,H,F], got %s" % (tuple(in_feat.shape),))
        n, h, f = in_feat.shape
        e = row_ind.numel()
        dev = in_feat.device
        col_ptr, row_ind = as_i32(col_ptr), as_i32(row_ind)
        row_ptr = None if row_ptr is None else as_i32(row_ptr)
        col_ind = None if col_ind is None else as_i32(col_ind)
        out_feat, out2, cc = (None if t is None else as_f32(t) for t in (out_feat, out2, cc))
        permute = None if permute is None else as_i32(permute)
        e_soft = None if e_soft is None else as_f32(e_soft)
        for name, t, shape in (("grad", grad, (n, h, f)), ("attn_row", attn_row, (n, h)), ("attn_col", attn_col, (n, h)),
                               ("edge_max", edge_max, (n, h)), ("edge_sum", edge_sum, (n, h)), ("out_feat", out_feat, (n, h, f)),
                               ("out2", out2, (n, h, f)), ("cc", cc, (n, h)), ("e_soft", e_soft, (e, h))):
            if t is not None and tuple(t.shape) != shape:
                raise _lib.FgnnError("gat_backward: %s has shape %s, expected %s" % (name, tuple(t.shape), shape))
        for name, t, numel in (("col_ptr", col_ptr, n + 1), ("row_ptr", row_ptr, n + 1), ("col_ind", col_ind, e), ("permute", permute, e)):
            if t is not None and t.numel() != numel:
                raise _lib.FgnnError("gat_backward: %s has %d elements, expected %d" % (name, t.numel(), numel))
        grad_feat = torch.empty_like(in_feat)
        grad_attn_row = torch.empty((n, h), dtype=torch.float32, device=dev)
        grad_attn_col = torch.empty((n, h), dtype=torch.float32, device=dev)
        recompute = out_feat is None or out2 is None or cc is None
        sched_csc = schedule_for(col_ptr, idx_tensor=row_ind, need_positions=e_soft is not None and not own, n_cols=n) if use_schedule else None
        sched_csr = schedule_for(row_ptr, idx_tensor=col_ind, need_positions=False, n_cols=n) if (use_schedule and recompute) else None
        hc = sched_csc.handle if sched_csc is not None else None
        hr = sched_csr.handle if sched_csr is not None else None
        with torch.cuda.device(dev):
            ws, wsb = workspace(lib().fgnn_gat_backward_workspace_bytes(n, h, f, hc, hr, int(recompute) | (2 if e_soft is not None else 0)), dev)
            saved = (None if recompute else ptr(out_feat), None if recompute else ptr(out2), None if recompute else ptr(cc))
            if own:
                check(lib().fgnn_gat_backward_own_order(n, e, h, f, float(negative_slope), ptr(row_ptr), ptr(col_ind), ptr(col_ptr),
                                                        ptr(row_ind), ptr(e_soft), ptr(edge_max), ptr(edge_sum), ptr(in_feat),
                                                        ptr(attn_row), ptr(attn_col), *saved, ptr(grad), ptr(grad_feat),
                                                        ptr(grad_attn_row), ptr(grad_attn_col), hc, hr, ptr(ws), wsb, stream_ptr()),
                      "fgnn_gat_backward_own_order")
            else:
                check(lib().fgnn_gat_backward(n, e, h, f, float(negative_slope), ptr(row_ptr), ptr(col_ind), ptr(col_ptr),
                                              ptr(row_ind), ptr(permute), ptr(e_lrelu), ptr(e_soft), ptr(edge_max),
                                              ptr(edge_sum), ptr(in_feat), ptr(attn_row), ptr(attn_col), *saved, ptr(grad),
                                              ptr(grad_feat), ptr(grad_attn_row), ptr(grad_attn_col), hc, hr, ptr(ws), wsb, stream_ptr()),
                      "fgnn_gat_backward")
        return grad_feat, grad_attn_row, grad_attn_col


    @staticmethod
    def gat_stash_own_order(negative_slope, col_ptr, row_ind, edge_max, edge_sum, attn_row, attn_col, use_schedule=True):
        """The attention weights [E,H] in the entry order of the backward pass over (col_ptr, row_ind): what
        gat_backward(..., e_soft=<this>, permute=None) streams instead of gathering a CSR-ordered stash."""
        require_cuda(col_ptr, row_ind, edge_max, edge_sum, attn_row, attn_col)
        col_ptr, row_ind = as_i32(col_ptr), as_i32(row_ind)
        edge_max, edge_sum, attn_row, attn_col = as_f32(edge_max), as_f32(edge_sum), as_f32(attn_row), as_f32(attn_col)
        n, h = attn_row.shape
        e = row_ind.numel()
        if col_ptr.numel() != n + 1 or any(tuple(t.shape) != (n, h) for t in (attn_col, edge_max, edge_sum)):
            raise _lib.FgnnError("gat_stash_own_order: shape mismatch for N=%d H=%d" % (n, h))
        out = torch.empty((e, h), dtype=torch.float32, device=attn_row.device)
        sched = schedule_for(col_ptr, idx_tensor=row_ind, need_positions=False, n_cols=n) if use_schedule else None
        with torch.cuda.device(attn_row.device):
            check(lib().fgnn_gat_stash_own_order(n, e, h, float(negative_slope), ptr(col_ptr), ptr(row_ind), ptr(attn_row), ptr(attn_col),
                                                 ptr(edge_max), ptr(edge_sum), ptr(out), sched.handle if sched is not None else None,
                                                 stream_ptr()), "fgnn_gat_stash_own_order")
        return out


    @staticmethod
    def gat_scatter(attn_row, attn_col, row_ptr, col_ind, negative_slope, want_lrelu=False):
        """fused_scatter_kernel of the reference's fuse-scatter variant (src/fused_gat/fused_gat.cu:235-300): (e_lrelu or None,
        e_softmax [E,H]) in one pass over the rows."""
        require_cuda(attn_row, attn_col, row_ptr, col_ind)
        attn_row, attn_col, row_ptr, col_ind = as_f32(attn_row), as_f32(attn_col), as_i32(row_ptr), as_i32(col_ind)
        n, h = attn_row.shape
        e = col_ind.numel()
        if attn_col.shape != (n, h) or row_ptr.numel() != n + 1:
            raise _lib.FgnnError("gat_scatter: shape mismatch for N=%d H=%d" % (n, h))
        e_soft = torch.empty((e, h), dtype=torch.float32, device=attn_row.device)
        e_lrelu = torch.empty((e, h), dtype=torch.float32, device=attn_row.device) if want_lrelu else None
        with torch.cuda.device(attn_row.device):
            check(lib().fgnn_gat_scatter(n, e, h, ptr(row_ptr), ptr(col_ind), ptr(attn_row), ptr(attn_col), float(negative_slope),
                                         ptr(e_lrelu), ptr(e_soft), stream_ptr()), "fgnn_gat_scatter")
        return e_lrelu, e_soft

    @staticmethod
    def gat_gather_row(negative_slope, row_ptr, col_ind, attn_row, attn_col, e_soft, grad_edge, e_lrelu=None, inplace=False):
        """fused_gather_row (src/fused_gat/fused_gat.cu:502-556): (gradient of the pre-activations [E,H], grad_attn_row [N,H])."""
        require_cuda(row_ptr, col_ind, attn_row, attn_col, e_soft, grad_edge, e_lrelu)
        row_ptr, col_ind = as_i32(row_ptr), as_i32(col_ind)
        attn_row, attn_col, e_soft, grad_edge = as_f32(attn_row), as_f32(attn_col), as_f32(e_soft), as_f32(grad_edge)
        e_lrelu = None if e_lrelu is None else as_f32(e_lrelu)
        n, h = attn_row.shape
        e = col_ind.numel()
        if e_soft.shape != (e, h) or grad_edge.shape != (e, h) or (e_lrelu is not None and e_lrelu.shape != (e, h)) or row_ptr.numel() != n + 1:
            raise _lib.FgnnError("gat_gather_row: shape mismatch for N=%d E=%d H=%d" % (n, e, h))
        out = grad_edge if inplace else torch.empty_like(grad_edge)
        gar = torch.empty((n, h), dtype=torch.float32, device=attn_row.device)
        with torch.cuda.device(attn_row.device):
            check(lib().fgnn_gat_gather_row(n, e, h, ptr(row_ptr), ptr(col_ind), ptr(attn_row), ptr(attn_col), ptr(e_lrelu),
                                            float(negative_slope), ptr(e_soft), ptr(grad_edge), ptr(out), ptr(gar), stream_ptr()),
                  "fgnn_gat_gather_row")
        return out, gar


def fused_gat_fusescatter(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute):
    return FusedGATFunction.apply(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute)


def fused_gat_op(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, save_memory=True):
    return FusedGATFunction_SM.apply(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat)


def fused_gat_stash_op(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute):
    return FusedGATFunction_stash.apply(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute)


def _needs_grad(ctx):
    return any(ctx.needs_input_grad)


def _contig(t):
    return t if t.is_contiguous() else t.contiguous()


class FusedGATFunction_SM(torch.autograd.Function):
    """Recompute ("save memory") variant: nothing edge-sized is kept between forward and backward."""

    @staticmethod
    def forward(ctx, attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat):
        need = _needs_grad(ctx)
        # contiguous copies of strided views are made once, here, and these are what the backward gets
        attn_row, attn_col, in_feat = _contig(attn_row), _contig(attn_col), _contig(in_feat)
        row_ptr, col_ind, col_ptr, row_ind = _contig(row_ptr), _contig(col_ind), _contig(col_ptr), _contig(row_ind)
        out, edge_max, edge_sum, out2, cc, _, _ = gat_native.gat_forward(
            attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat, need_aux=need)
        if need:
            ctx.save_for_backward(row_ptr, col_ind, col_ptr, row_ind, edge_max, edge_sum, in_feat, attn_row, attn_col,
                                  out, out2, cc)
        ctx.negative_slope = negative_slope
        return out

    @staticmethod
    def backward(ctx, grad_out):
        row_ptr, col_ind, col_ptr, row_ind, edge_max, edge_sum, in_feat, attn_row, attn_col, out, out2, cc = ctx.saved_tensors
        grad_feat, grad_attn_row, grad_attn_col = gat_native.gat_backward(
            ctx.negative_slope, row_ptr, col_ind, col_ptr, row_ind, edge_max, edge_sum, in_feat, attn_row, attn_col,
            grad_out.contiguous(), out_feat=out, out2=out2, cc=cc)
        return grad_attn_row, grad_attn_col, None, None, None, None, None, grad_feat


class FusedGATFunction_stash(torch.autograd.Function):
    """Stash variant: the forward also writes the edge softmax [E,H] and the backward reads it instead
    of recomputing.  (The reference stashes the edge LeakyReLU values too, fused_gat_stash.cu:420-442;
    the backward here takes the one thing it needs from them, the sign of the pre-activation, from
    attn_row + attn_col, so they are not written: half the stash.)  The stash is kept in the entry order
    of the backward pass, so that pass streams it; the CSR-ordered stash of the reference's signature
    (gat_forward(stash=True) + gat_backward(permute=...)) stays available through gat_native."""

    @staticmethod
    def forward(ctx, attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute):
        need = _needs_grad(ctx)
        attn_row, attn_col, in_feat = _contig(attn_row), _contig(attn_col), _contig(in_feat)
        row_ptr, col_ind, col_ptr, row_ind, permute = _contig(row_ptr), _contig(col_ind), _contig(col_ptr), _contig(row_ind), _contig(permute)
        out, edge_max, edge_sum, out2, cc, _, _ = gat_native.gat_forward(
            attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat, need_aux=need)
        if need:       # inference / no_grad: no stash pass, no [E,H] tensor, no CSC work list
            # the stash is this function's own tensor: it is written in the order in which the backward walks the edges
            e_soft = gat_native.gat_stash_own_order(negative_slope, col_ptr, row_ind, edge_max, edge_sum, attn_row, attn_col)
            ctx.save_for_backward(row_ptr, col_ind, col_ptr, row_ind, permute, e_soft, in_feat, attn_row, attn_col,
                                  edge_max, edge_sum, out, out2, cc)
        ctx.negative_slope = negative_slope
        return out

    @staticmethod
    def backward(ctx, grad_out):
        (row_ptr, col_ind, col_ptr, row_ind, permute, e_soft, in_feat, attn_row, attn_col,
         edge_max, edge_sum, out, out2, cc) = ctx.saved_tensors
        grad_feat, grad_attn_row, grad_attn_col = gat_native.gat_backward(
            ctx.negative_slope, row_ptr, col_ind, col_ptr, row_ind, edge_max, edge_sum, in_feat, attn_row, attn_col,
            grad_out.contiguous(), out_feat=out, out2=out2, cc=cc, e_soft=e_soft, e_soft_order="own")
        return grad_attn_row, grad_attn_col, None, None, None, None, None, grad_feat, None


class FusedGATFunction(torch.autograd.Function):
    """Fuse-scatter variant with the reference's own data flow (operators/fused_gat.py:36-50; src/fused_gat/fused_gat.cu):
    forward = one scatter kernel (scores, LeakyReLU, row softmax -> e_softmax [E,H]) + multi-head SpMM; backward = the
    permuted SpMM over the CSC arrays (grad_feat), the SDDMM (gradient of the weights), one gather-row kernel (softmax and
    LeakyReLU backward + row sums = grad_attn_row, in place) and the column sums (grad_attn_col).  Kept between the passes:
    e_softmax only; the reference also keeps the LeakyReLU values, whose sign this backward forms again from the scores."""

    @staticmethod
    def forward(ctx, attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute):
        from .mhspmm import mhspmm
        attn_row, attn_col, in_feat = _contig(attn_row), _contig(attn_col), _contig(in_feat)
        row_ptr, col_ind, col_ptr, row_ind, permute = _contig(row_ptr), _contig(col_ind), _contig(col_ptr), _contig(row_ind), _contig(permute)
        # e_softmax and the edge gradients live in the entry order of the work lists: rows keep their places, the entries
        # of a row are regrouped by source bucket when the list is XCD-aware, so every pass below streams them
        idx_own, perm_own = _lib.own_order_view(row_ptr, col_ind, col_ptr, row_ind, as_i32(permute))
        _, e_soft = gat_native.gat_scatter(attn_row, attn_col, row_ptr, idx_own, negative_slope)
        out = mhspmm(row_ptr, col_ind, e_soft, in_feat, own_order=True)
        if _needs_grad(ctx):
            ctx.save_for_backward(row_ptr, col_ind, col_ptr, row_ind, idx_own, perm_own, e_soft, in_feat, attn_row, attn_col)
        ctx.negative_slope = negative_slope
        return out

    @staticmethod
    def backward(ctx, grad_out):
        from .mhspmm import mhsddmm, mhspmm
        row_ptr, col_ind, col_ptr, row_ind, idx_own, perm_own, e_soft, in_feat, attn_row, attn_col = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_feat = mhspmm(col_ptr, row_ind, e_soft, grad_out, pos_map=perm_own, own_order=True)
        grad_edge = mhsddmm(row_ptr, col_ind, grad_out, in_feat, own_order=True)
        grad_edge, grad_attn_row = gat_native.gat_gather_row(ctx.negative_slope, row_ptr, idx_own, attn_row, attn_col, e_soft, grad_edge, inplace=True)
        n, h = attn_row.shape
        grad_attn_col = colsum_plan_for(row_ptr, idx_own, n, h).colsum(grad_edge)
        return grad_attn_row, grad_attn_col, None, None, None, None, None, grad_feat, None


def fused_gat_fusescatter_pipeline(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute):
    """The fuse-scatter ablation of the reference: FusedGATFunction above (its own kernels in its own order)."""
    return FusedGATFunction.apply(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute)


def fused_gat_operator_pipeline(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, negative_slope, in_feat, permute):
    """The same layer composed from this package's stand-alone operators, each with its own autograd function: u_add_v ->
    LeakyReLU -> edge softmax ([E,H] materialised three times) -> multi-head SpMM; the backward runs the permuted SpMM
    over the CSC arrays, the SDDMM, the softmax backward and the row / column sums of u_add_v.  Same results as the fused
    operators; what an unfused layer costs on this part."""
    from .edge_softmax import csr_edge_softmax
    from .mhspmm import csrmhspmm
    from .u_add_v import u_add_v_op
    e = torch.nn.functional.leaky_relu(u_add_v_op(row_ptr, col_ind, attn_row, attn_col), negative_slope)
    return csrmhspmm(row_ptr, col_ind, col_ptr, row_ind, permute, in_feat, csr_edge_softmax(row_ptr, e))
