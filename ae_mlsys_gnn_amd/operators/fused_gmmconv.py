"""Fused GMMConv (MoNet) operators: the reference's operators/fused_gmmconv.py surface on
libfgnn_hip.so.  The backward is one pass over the CSC arrays (the reference runs mhsddmm,
mhtranspose, a CSC gmmconv and GaussianBp: operators/fused_gmmconv.py:51-58) and implements the
closed-form Gaussian derivatives."""
from __future__ import annotations

import torch

from .._lib import FgnnError, as_f32, as_i32, check, edge_positions, lib, ptr, require_cuda, schedule_for, stream_ptr, workspace


def _plain_list_for_summed_backward(n, e):
    """The summed backward gathers narrow rows ([N,F]); below an average degree of 64 it measured faster
    on the plain work list than on the XCD-aware one."""
    return e < 64 * n


class gmm_native:
    """gmmconv.gmmconv / gmmconvstash / Gaussian / GaussianBp (src/fused_gmmconv/gmmconv.cc:36-94)."""

    @staticmethod
    def gmmconv(rowptr, colind, node_feat, pseudo, mu, sigma, *, pos_map=None, want_gauss=False, sum_kernels=False, own_order=False,
                bias=None, residual=None):
        """bias [F] / residual [N,F] (with sum_kernels only): added to the summed output inside the operator's store."""
        require_cuda(rowptr, colind, node_feat, pseudo, mu, sigma, bias, residual)
        rowptr, colind = as_i32(rowptr), as_i32(colind)
        node_feat, pseudo, mu, sigma = as_f32(node_feat), as_f32(pseudo), as_f32(mu), as_f32(sigma)
        if node_feat.dim() != 3:
            raise FgnnError("node_feat must be [N,K,F], got %s" % (tuple(node_feat.shape),))
        n, k, f = node_feat.shape
        e = colind.numel()
        dim = mu.shape[1]
        if mu.shape != (k, dim) or sigma.shape != (k, dim) or pseudo.shape != (e, dim) or rowptr.numel() != n + 1:
            raise FgnnError("gmmconv: shape mismatch mu %s sigma %s pseudo %s for K=%d E=%d" % (
                tuple(mu.shape), tuple(sigma.shape), tuple(pseudo.shape), k, e))
        out = torch.empty((n, f), dtype=torch.float32, device=node_feat.device) if sum_kernels else torch.empty_like(node_feat)
        gauss = torch.empty((e, k), dtype=torch.float32, device=node_feat.device) if want_gauss else None
        # own_order: pseudo (and gauss) are indexed by the schedule's entry order, pseudo_caller[edge_positions(rowptr, colind)]
        sched = schedule_for(rowptr, idx_tensor=colind, own_order=own_order, n_cols=n)
        epilogue = bias is not None or residual is not None
        if epilogue:
            if not sum_kernels:
                raise FgnnError("gmmconv: bias / residual are added to the sum over the kernels (sum_kernels=True)")
            bias = None if bias is None else as_f32(bias)
            residual = None if residual is None else as_f32(residual)
            if (bias is not None and tuple(bias.shape) != (f,)) or (residual is not None and tuple(residual.shape) != (n, f)):
                raise FgnnError("gmmconv: bias must be [%d] and residual [%d, %d]" % (f, n, f))
        with torch.cuda.device(node_feat.device):
            ws, wsb = workspace(lib().fgnn_gmm_forward_workspace_bytes(sched.handle, k, f), node_feat.device)
            if epilogue:
                check(lib().fgnn_gmm_forward_epilogue(n, e, k, dim, f, ptr(rowptr), ptr(colind), ptr(pos_map), ptr(node_feat), ptr(pseudo),
                                                      ptr(mu), ptr(sigma), ptr(bias), ptr(residual), ptr(out), ptr(gauss), sched.handle,
                                                      ptr(ws), wsb, stream_ptr()), "fgnn_gmm_forward_epilogue")
            else:
                check(lib().fgnn_gmm_forward(n, e, k, dim, f, ptr(rowptr), ptr(colind), ptr(pos_map), ptr(node_feat), ptr(pseudo),
                                             ptr(mu), ptr(sigma), ptr(out), ptr(gauss), int(sum_kernels), sched.handle, ptr(ws), wsb, stream_ptr()),
                      "fgnn_gmm_forward")
        return (out, gauss) if want_gauss else out

    @staticmethod
    def gmmconv_backward(colptr, rowind, permute, node_feat, pseudo, mu, sigma, grad_out, sum_kernels=False, own_order=False):
        require_cuda(colptr, rowind, permute, node_feat, pseudo, mu, sigma, grad_out)
        colptr, rowind = as_i32(colptr), as_i32(rowind)
        permute = None if permute is None else as_i32(permute)      # None: pseudo / grad_pseudo in CSC order
        # raw pointers go to the kernels: contiguous copies of strided views, and every shape checked
        grad_out, node_feat, pseudo, mu, sigma = as_f32(grad_out), as_f32(node_feat), as_f32(pseudo), as_f32(mu), as_f32(sigma)
        if node_feat.dim() != 3 or mu.dim() != 2:
            raise FgnnError("gmmconv_backward: node_feat must be [N,K,F] and mu [K,dim], got %s and %s" % (tuple(node_feat.shape), tuple(mu.shape)))
        n, k, f = node_feat.shape
        e = rowind.numel()
        dim = mu.shape[1]
        dev = node_feat.device
        want_go = (n, f) if sum_kernels else (n, k, f)
        if (mu.shape != (k, dim) or sigma.shape != (k, dim) or pseudo.shape != (e, dim) or colptr.numel() != n + 1
                or tuple(grad_out.shape) != want_go or (permute is not None and permute.numel() != e)):
            raise FgnnError("gmmconv_backward: shape mismatch mu %s sigma %s pseudo %s grad_out %s col_ptr %d for N=%d K=%d F=%d E=%d" % (
                tuple(mu.shape), tuple(sigma.shape), tuple(pseudo.shape), tuple(grad_out.shape), colptr.numel(), n, k, f, e))
        grad_feat = torch.empty_like(node_feat)
        grad_pseudo = torch.empty((e, dim), dtype=torch.float32, device=dev)
        grad_mu = torch.empty_like(mu)
        grad_sigma = torch.empty_like(sigma)
        # own_order: pseudo, grad_pseudo (and permute) are indexed by the schedule's entry order (gmm_edge_positions(colptr, rowind, True))
        sched = schedule_for(colptr, idx_tensor=None if (sum_kernels and _plain_list_for_summed_backward(n, e)) else rowind, own_order=own_order, n_cols=n)
        with torch.cuda.device(dev):
            ws, wsb = workspace(lib().fgnn_gmm_backward_workspace_bytes(sched.handle, k, dim, f), dev)
            check(lib().fgnn_gmm_backward(n, e, k, dim, f, ptr(colptr), ptr(rowind), ptr(permute), ptr(node_feat), ptr(pseudo),
                                          ptr(mu), ptr(sigma), ptr(grad_out), int(sum_kernels), ptr(grad_feat), ptr(grad_pseudo), ptr(grad_mu),
                                          ptr(grad_sigma), sched.handle, ptr(ws), wsb, stream_ptr()), "fgnn_gmm_backward")
        return grad_feat, grad_pseudo, grad_mu, grad_sigma

    @staticmethod
    def shared_supported(k, f):
        """Shapes the shared-feature (aggregate first) entry points take: the [N,f] rows as 128-bit slabs over
        at most a wave, the K accumulators in registers."""
        return f % 4 == 0 and 0 < f <= 256 and 0 < k <= 4

    @staticmethod
    def gmmconv_shared(rowptr, colind, feat, pseudo, mu, sigma, *, pos_map=None, own_order=False):
        """out[i,k,:] = sum_p w[p,k] * feat[colind[p],:] for one [N,F] feature matrix shared by the K mixture
        kernels (the reference's gmmconv with node_feat[:,k,:] == feat for every k).  Returns [N,K,F]."""
        require_cuda(rowptr, colind, feat, pseudo, mu, sigma)
        rowptr, colind = as_i32(rowptr), as_i32(colind)
        feat, pseudo, mu, sigma = as_f32(feat), as_f32(pseudo), as_f32(mu), as_f32(sigma)
        if feat.dim() != 2:
            raise FgnnError("feat must be [N,F], got %s" % (tuple(feat.shape),))
        n, f = feat.shape
        k, dim = mu.shape
        e = colind.numel()
        if sigma.shape != (k, dim) or pseudo.shape != (e, dim) or rowptr.numel() != n + 1:
            raise FgnnError("gmmconv_shared: shape mismatch mu %s sigma %s pseudo %s for E=%d" % (
                tuple(mu.shape), tuple(sigma.shape), tuple(pseudo.shape), e))
        out = torch.empty((n, k, f), dtype=torch.float32, device=feat.device)
        sched = schedule_for(rowptr, idx_tensor=colind, own_order=own_order, n_cols=n)
        with torch.cuda.device(feat.device):
            ws, wsb = workspace(lib().fgnn_gmm_forward_workspace_bytes(sched.handle, k, f), feat.device)
            check(lib().fgnn_gmm_forward(n, e, k, dim, f, ptr(rowptr), ptr(colind), ptr(pos_map), ptr(feat), ptr(pseudo),
                                         ptr(mu), ptr(sigma), ptr(out), None, 2, sched.handle, ptr(ws), wsb, stream_ptr()),
                  "fgnn_gmm_forward (shared features)")
        return out

    @staticmethod
    def gmmconv_shared_backward(colptr, rowind, permute, feat, pseudo, mu, sigma, grad_out, own_order=False):
        """Backward of gmmconv_shared for grad_out [N,K,F]: (grad_feat [N,F], grad_pseudo, grad_mu, grad_sigma)."""
        require_cuda(colptr, rowind, permute, feat, pseudo, mu, sigma, grad_out)
        colptr, rowind = as_i32(colptr), as_i32(rowind)
        permute = None if permute is None else as_i32(permute)
        grad_out, feat, pseudo, mu, sigma = as_f32(grad_out), as_f32(feat), as_f32(pseudo), as_f32(mu), as_f32(sigma)
        if feat.dim() != 2 or mu.dim() != 2:
            raise FgnnError("gmmconv_shared_backward: feat must be [N,F] and mu [K,dim], got %s and %s" % (tuple(feat.shape), tuple(mu.shape)))
        n, f = feat.shape
        k, dim = mu.shape
        e = rowind.numel()
        dev = feat.device
        if grad_out.shape != (n, k, f):
            raise FgnnError("gmmconv_shared_backward: grad_out is %s, expected (%d, %d, %d)" % (tuple(grad_out.shape), n, k, f))
        if sigma.shape != (k, dim) or pseudo.shape != (e, dim) or colptr.numel() != n + 1 or (permute is not None and permute.numel() != e):
            raise FgnnError("gmmconv_shared_backward: shape mismatch sigma %s pseudo %s col_ptr %d for N=%d K=%d E=%d" % (
                tuple(sigma.shape), tuple(pseudo.shape), colptr.numel(), n, k, e))
        parts = torch.empty((n, k, f), dtype=torch.float32, device=dev)      # kernel k's share of grad_feat
        grad_pseudo = torch.empty((e, dim), dtype=torch.float32, device=dev)
        grad_mu = torch.empty_like(mu)
        grad_sigma = torch.empty_like(sigma)
        # same work list as the summed backward, so that one CSC-side copy of own-order edge data serves both kinds of layer
        sched = schedule_for(colptr, idx_tensor=None if _plain_list_for_summed_backward(n, e) else rowind, own_order=own_order, n_cols=n)
        with torch.cuda.device(dev):
            ws, wsb = workspace(lib().fgnn_gmm_backward_workspace_bytes(sched.handle, k, dim, f), dev)
            check(lib().fgnn_gmm_backward(n, e, k, dim, f, ptr(colptr), ptr(rowind), ptr(permute), ptr(feat), ptr(pseudo),
                                          ptr(mu), ptr(sigma), ptr(grad_out), 2, ptr(parts), ptr(grad_pseudo), ptr(grad_mu),
                                          ptr(grad_sigma), sched.handle, ptr(ws), wsb, stream_ptr()), "fgnn_gmm_backward (shared features)")
        return parts.sum(1), grad_pseudo, grad_mu, grad_sigma

    @staticmethod
    def Gaussian(pseudo, mu, sigma):
        require_cuda(pseudo, mu, sigma)
        pseudo, mu, sigma = as_f32(pseudo), as_f32(mu), as_f32(sigma)
        e, dim = pseudo.shape
        k = mu.shape[0]
        out = torch.empty((e, k), dtype=torch.float32, device=pseudo.device)
        with torch.cuda.device(pseudo.device):
            check(lib().fgnn_gaussian(e, k, dim, ptr(pseudo), ptr(mu), ptr(sigma), ptr(out), stream_ptr()), "fgnn_gaussian")
        return out

    @staticmethod
    def GaussianBp(pseudo, mu, sigma, grad_out):
        require_cuda(pseudo, mu, sigma, grad_out)
        pseudo, mu, sigma, grad_out = as_f32(pseudo), as_f32(mu), as_f32(sigma), as_f32(grad_out)
        e, dim = pseudo.shape
        k = mu.shape[0]
        gp = torch.empty_like(pseudo)
        gm = torch.empty_like(mu)
        gs = torch.empty_like(sigma)
        with torch.cuda.device(pseudo.device):
            ws, wsb = workspace(lib().fgnn_gaussian_backward_workspace_bytes(e, k, dim), pseudo.device)
            check(lib().fgnn_gaussian_backward(e, k, dim, ptr(pseudo), ptr(mu), ptr(sigma), ptr(grad_out), ptr(gp), ptr(gm),
                                               ptr(gs), ptr(ws), wsb, stream_ptr()), "fgnn_gaussian_backward")
        return gp, gm, gs


def _epilogue_grads(ctx, grad_out, first):
    """Gradients of the optional (bias, residual) inputs at positions first, first + 1 of a Function's inputs."""
    from ..layers.dense import column_sum
    gb = column_sum(grad_out) if (ctx.has_bias and ctx.needs_input_grad[first]) else None
    gr = grad_out if (ctx.has_res and ctx.needs_input_grad[first + 1]) else None
    return gb, gr


def GmmConvFuse(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma):
    return GmmFuseFunction.apply(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma)


class GmmFuseFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma):
        out = gmm_native.gmmconv(rowptr, colind, node_feat, pseudo, mu, sigma)      # [N, K, F]
        ctx.save_for_backward(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma = ctx.saved_tensors
        grad_feat, grad_pseudo, grad_mu, grad_sigma = gmm_native.gmmconv_backward(
            colptr, rowind, permute, node_feat, pseudo, mu, sigma, grad_out.contiguous())
        return None, None, None, None, None, grad_feat, grad_pseudo, grad_mu, grad_sigma


def GmmConvFuseSum(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma, bias=None, residual=None):
    """GmmConvFuse(...).sum(1) as one operator: the sum over the K mixture kernels is fused into the
    forward's store and the backward gathers [N,F] gradient rows.  Returns [N,F].
    bias [F], residual [N,F] (optional): the rest of the layer's forward (layers/gmmconv_layer.py:69-75), added in
    the same store."""
    return GmmFuseSumFunction.apply(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma, bias, residual)


def GmmConvFuseSumTwoOrders(rowptr, colind, colptr, rowind, node_feat, pseudo_csr, pseudo_csc, mu, sigma, own_order=False, bias=None,
                            residual=None):
    """GmmConvFuseSum for a caller that has the pseudo-coordinates in both edge orders
    (pseudo_csc == pseudo_csr[permute], e.g. the same elementwise projection applied to constant
    edge data stored both ways).  The forward reads pseudo_csr, the backward reads pseudo_csc and
    returns its gradient in CSC order: no per-edge gather or scatter through permute.  pseudo_csr
    gets no gradient; the caller's parameters receive theirs through pseudo_csc (None: forward only).
    own_order: the two tensors are in the entry order of the operators' own schedules,
    pseudo_csr[gmm_edge_positions(rowptr, colind)] and pseudo_csc[gmm_edge_positions(colptr, rowind, True)]:
    every pass then streams its per-edge data."""
    if pseudo_csc is None:
        return gmm_native.gmmconv(rowptr, colind, node_feat, pseudo_csr, mu, sigma, sum_kernels=True, own_order=own_order, bias=bias,
                                  residual=residual)
    return GmmFuseSumTwoOrdersFunction.apply(rowptr, colind, colptr, rowind, node_feat, pseudo_csr, pseudo_csc, mu, sigma, own_order, bias, residual)


def GmmConvStashSumTwoOrders(rowptr, colind, colptr, rowind, node_feat, pseudo_csr, pseudo_csc, mu, sigma, own_order=False, bias=None,
                             residual=None):
    """The stash variant with the pseudo-coordinates in both edge orders: as GmmConvFuseSumTwoOrders, and the
    forward also writes the Gaussian weights [E,K] (in the order of pseudo_csr) and keeps them until the
    backward, the memory cost of the reference's stash variant (operators/fused_gmmconv.py:100-118).  The
    backward is the same single pass: recomputing a weight is cheaper than reading it back through a
    transposition."""
    return GmmStashSumTwoOrdersFunction.apply(rowptr, colind, colptr, rowind, node_feat, pseudo_csr, pseudo_csc, mu, sigma, own_order, bias, residual)


class GmmStashSumTwoOrdersFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, node_feat, pseudo_csr, pseudo_csc, mu, sigma, own_order, bias=None, residual=None):
        out, gauss = gmm_native.gmmconv(rowptr, colind, node_feat, pseudo_csr, mu, sigma, want_gauss=True, sum_kernels=True,
                                        own_order=own_order, bias=bias, residual=residual)
        ctx.save_for_backward(colptr, rowind, node_feat, pseudo_csc, mu, sigma, gauss)
        ctx.own_order = own_order
        ctx.has_bias, ctx.has_res = bias is not None, residual is not None
        return out

    @staticmethod
    def backward(ctx, grad_out):
        colptr, rowind, node_feat, pseudo_csc, mu, sigma, _gauss = ctx.saved_tensors
        grad_feat, grad_pseudo_csc, grad_mu, grad_sigma = gmm_native.gmmconv_backward(
            colptr, rowind, None, node_feat, pseudo_csc, mu, sigma, grad_out.contiguous(), sum_kernels=True, own_order=ctx.own_order)
        return (None, None, None, None, grad_feat, None, grad_pseudo_csc, grad_mu, grad_sigma, None) + _epilogue_grads(ctx, grad_out.contiguous(), 10)


def gmm_edge_positions(ptr_arr, idx, summed_backward=False):
    """int32 [E] (or None = identity): caller's position of every entry in the order in which the GMMConv
    operators walk (ptr_arr, idx) when called with own_order=True.  summed_backward: for the (col_ptr,
    row_ind) arrays of the layers' backward passes (GmmConvFuseSumTwoOrders, GmmAggregateTwoOrders), which
    keep the caller's order on graphs of low average degree."""
    require_cuda(ptr_arr, idx)
    ptr_arr, idx = as_i32(ptr_arr), as_i32(idx)
    if summed_backward and _plain_list_for_summed_backward(ptr_arr.numel() - 1, idx.numel()):
        schedule_for(ptr_arr)
        return None
    return edge_positions(ptr_arr, idx)


class GmmFuseSumTwoOrdersFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, node_feat, pseudo_csr, pseudo_csc, mu, sigma, own_order, bias=None, residual=None):
        out = gmm_native.gmmconv(rowptr, colind, node_feat, pseudo_csr, mu, sigma, sum_kernels=True, own_order=own_order, bias=bias,
                                 residual=residual)      # [N, F]
        ctx.save_for_backward(colptr, rowind, node_feat, pseudo_csc, mu, sigma)
        ctx.own_order = own_order
        ctx.has_bias, ctx.has_res = bias is not None, residual is not None
        return out

    @staticmethod
    def backward(ctx, grad_out):
        colptr, rowind, node_feat, pseudo_csc, mu, sigma = ctx.saved_tensors
        grad_feat, grad_pseudo_csc, grad_mu, grad_sigma = gmm_native.gmmconv_backward(
            colptr, rowind, None, node_feat, pseudo_csc, mu, sigma, grad_out.contiguous(), sum_kernels=True, own_order=ctx.own_order)
        return (None, None, None, None, grad_feat, None, grad_pseudo_csc, grad_mu, grad_sigma, None) + _epilogue_grads(ctx, grad_out.contiguous(), 10)


def GmmAggregate(rowptr, colind, colptr, rowind, permute, feat, pseudo, mu, sigma):
    """Aggregate first: agg[i,k,:] = sum_p w[p,k] * feat[colind[p],:] for feat [N,F] -> [N,K,F].  A GMMConv
    layer whose input is narrower than K x its output multiplies by the fc weights afterwards
    (sum_k agg[:,k,:] @ W_k equals the reference's sum over k of the aggregated fc(feat)[:,k,:]), so an
    edge gathers F floats instead of K x out."""
    return GmmAggregateFunction.apply(rowptr, colind, colptr, rowind, permute, feat, pseudo, mu, sigma)


class GmmAggregateFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, permute, feat, pseudo, mu, sigma):
        out = gmm_native.gmmconv_shared(rowptr, colind, feat, pseudo, mu, sigma)
        ctx.save_for_backward(colptr, rowind, permute, feat, pseudo, mu, sigma)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        colptr, rowind, permute, feat, pseudo, mu, sigma = ctx.saved_tensors
        grad_feat, grad_pseudo, grad_mu, grad_sigma = gmm_native.gmmconv_shared_backward(
            colptr, rowind, permute, feat, pseudo, mu, sigma, grad_out.contiguous())
        return None, None, None, None, None, grad_feat, grad_pseudo, grad_mu, grad_sigma


def GmmAggregateTwoOrders(rowptr, colind, colptr, rowind, feat, pseudo_csr, pseudo_csc, mu, sigma, own_order=False):
    """GmmAggregate for a caller that has the pseudo-coordinates in both edge orders (see
    GmmConvFuseSumTwoOrders; pseudo_csc None: forward only)."""
    if pseudo_csc is None:
        return gmm_native.gmmconv_shared(rowptr, colind, feat, pseudo_csr, mu, sigma, own_order=own_order)
    return GmmAggregateTwoOrdersFunction.apply(rowptr, colind, colptr, rowind, feat, pseudo_csr, pseudo_csc, mu, sigma, own_order)


class GmmAggregateTwoOrdersFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, feat, pseudo_csr, pseudo_csc, mu, sigma, own_order):
        out = gmm_native.gmmconv_shared(rowptr, colind, feat, pseudo_csr, mu, sigma, own_order=own_order)
        ctx.save_for_backward(colptr, rowind, feat, pseudo_csc, mu, sigma)
        ctx.own_order = own_order
        return out

    @staticmethod
    def backward(ctx, grad_out):
        colptr, rowind, feat, pseudo_csc, mu, sigma = ctx.saved_tensors
        grad_feat, grad_pseudo_csc, grad_mu, grad_sigma = gmm_native.gmmconv_shared_backward(
            colptr, rowind, None, feat, pseudo_csc, mu, sigma, grad_out.contiguous(), own_order=ctx.own_order)
        return None, None, None, None, grad_feat, None, grad_pseudo_csc, grad_mu, grad_sigma, None


class GmmFuseSumFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma, bias=None, residual=None):
        out = gmm_native.gmmconv(rowptr, colind, node_feat, pseudo, mu, sigma, sum_kernels=True, bias=bias, residual=residual)      # [N, F]
        ctx.save_for_backward(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma)
        ctx.has_bias, ctx.has_res = bias is not None, residual is not None
        return out

    @staticmethod
    def backward(ctx, grad_out):
        rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma = ctx.saved_tensors
        grad_feat, grad_pseudo, grad_mu, grad_sigma = gmm_native.gmmconv_backward(
            colptr, rowind, permute, node_feat, pseudo, mu, sigma, grad_out.contiguous(), sum_kernels=True)
        return (None, None, None, None, None, grad_feat, grad_pseudo, grad_mu, grad_sigma) + _epilogue_grads(ctx, grad_out.contiguous(), 9)


def GmmConvFuseEb(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma):
    return GmmFuseEbFunction.apply(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma)


class GmmFuseEbFunction(GmmFuseFunction):
    """The reference's edge-balanced variant (operators/fused_gmmconv.py:61-79).  Load balance is
    handled by the degree-binned schedule here, so it is the same computation."""


def GaussianCp(pseudo, mu, sigma):
    return GaussianFunction.apply(pseudo, mu, sigma)


class GaussianFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, pseudo, mu, sigma):
        out = gmm_native.Gaussian(pseudo, mu, sigma)
        ctx.save_for_backward(pseudo, mu, sigma)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        pseudo, mu, sigma = ctx.saved_tensors
        return gmm_native.GaussianBp(pseudo, mu, sigma, grad_out.contiguous())


def GmmConvStash(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma):
    return GmmStashFunction.apply(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma)


class GmmStashFunction(torch.autograd.Function):
    """Stash variant (operators/fused_gmmconv.py:100-118): the forward also writes the Gaussian
    weights [E,K].  The backward uses the same single CSC pass as GmmFuseFunction (recomputing
    the weights is cheaper than reading them back through `permute`)."""

    @staticmethod
    def forward(ctx, rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, sigma):
        out, gauss = gmm_native.gmmconv(rowptr, colind, node_feat, pseudo, mu, sigma, want_gauss=True)
        ctx.save_for_backward(rowptr, colind, colptr, rowind, permute, gauss, node_feat, pseudo, mu, sigma)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        rowptr, colind, colptr, rowind, permute, gauss, node_feat, pseudo, mu, sigma = ctx.saved_tensors
        grad_feat, grad_pseudo, grad_mu, grad_sigma = gmm_native.gmmconv_backward(
            colptr, rowind, permute, node_feat, pseudo, mu, sigma, grad_out.contiguous())
        return None, None, None, None, None, grad_feat, grad_pseudo, grad_mu, grad_sigma
