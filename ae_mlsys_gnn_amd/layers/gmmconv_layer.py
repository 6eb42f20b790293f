"""GMMConv (MoNet) layers on the fused operators (interface of the reference's
layers/gmmconv_layer.py:17-76 and :221-282)."""
from __future__ import annotations

import torch as th
from torch import nn
from torch.nn import init

from ..operators.fused_gmmconv import (GmmAggregate, GmmAggregateTwoOrders, GmmConvFuseSum, GmmConvFuseSumTwoOrders, GmmConvStash,
                                        GmmConvStashSumTwoOrders, gmm_native)
from .dense import add_bias, tall_linear


class _GMMBase(nn.Module):
    _op = None          # callable(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, mu, inv_sigma) -> [N, F]

    def __init__(self, in_feats, out_feats, dim, n_kernels, aggregator_type="sum", residual=False, bias=True,
                 allow_zero_in_degree=False):
        super().__init__()
        if aggregator_type != "sum":
            raise KeyError("Aggregator type {} not recognized.".format(aggregator_type))
        self._out_feats = out_feats
        self._dim = dim
        self._n_kernels = n_kernels
        self._allow_zero_in_degree = allow_zero_in_degree
        self.mu = nn.Parameter(th.empty(n_kernels, dim))
        self.inv_sigma = nn.Parameter(th.empty(n_kernels, dim))
        self.fc = nn.Linear(in_feats, n_kernels * out_feats, bias=False)
        if residual:
            self.res_fc = nn.Linear(in_feats, out_feats, bias=False) if in_feats != out_feats else nn.Identity()
        else:
            self.register_buffer("res_fc", None)
        if bias:
            self.bias = nn.Parameter(th.empty(out_feats))
        else:
            self.register_buffer("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        # layers/gmmconv_layer.py:55-62: Xavier-normal fc, mu ~ N(0, 0.1), inv_sigma = 1, bias = 0
        gain = init.calculate_gain("relu")
        init.xavier_normal_(self.fc.weight, gain=gain)
        if isinstance(self.res_fc, nn.Linear):
            init.xavier_normal_(self.res_fc.weight, gain=gain)
        init.normal_(self.mu.data, 0, 0.1)
        init.constant_(self.inv_sigma.data, 1)
        if self.bias is not None:
            init.zeros_(self.bias.data)

    def set_allow_zero_in_degree(self, set_value):
        self._allow_zero_in_degree = set_value

    def forward(self, rowptr, colind, colptr, rowind, permute, feat, pseudo, pseudo_csc=None, own_order=False):
        """pseudo_csc: the same pseudo-coordinates in CSC order, pseudo[permute], built by
        the caller from its own CSC-ordered edge data.  The backward then works in CSC order throughout
        and the gradient of the pseudo-coordinates flows through pseudo_csc instead of pseudo.
        own_order: pseudo and pseudo_csc are in the entry order of the operators' schedules
        (operators.fused_gmmconv.gmm_edge_positions); without pseudo_csc the layer is forward-only."""
        if self._aggregate_first(feat):
            return self._finish(self._forward_aggregate_first(rowptr, colind, colptr, rowind, permute, feat, pseudo, pseudo_csc, own_order), feat)
        node_feat = tall_linear(feat, self.fc.weight).view(-1, self._n_kernels, self._out_feats)    # = self.fc(feat)
        pad = (-self._out_feats) % 4
        if pad:         # zero columns up to a multiple of 4: the operator then takes its 128-bit row layout
            node_feat = th.nn.functional.pad(node_feat, (0, pad))
        # residual and bias (layers/gmmconv_layer.py:69-75 of the reference) go into the operator's store when the
        # width needs no padding; otherwise they are added afterwards
        fuse_tail = pad == 0 and (self.bias is not None or self.res_fc is not None)
        tail = lambda: {"bias": self.bias, "residual": None if self.res_fc is None else self.res_fc(feat)} if fuse_tail else {}
        if pseudo_csc is not None or own_order:
            if own_order and pseudo_csc is None and th.is_grad_enabled() and (node_feat.requires_grad or pseudo.requires_grad):
                raise ValueError("own_order without pseudo_csc is forward-only")
            two_orders = GmmConvFuseSumTwoOrders if (type(self)._op is GmmConvFuseSum or pseudo_csc is None) else GmmConvStashSumTwoOrders
            rst = two_orders(rowptr, colind, colptr, rowind, node_feat, pseudo.detach(), pseudo_csc, self.mu, self.inv_sigma,
                             own_order=own_order, **tail())
        elif type(self)._op is GmmConvFuseSum:
            rst = GmmConvFuseSum(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, self.mu, self.inv_sigma, **tail())
        else:
            rst = type(self)._op(rowptr, colind, colptr, rowind, permute, node_feat, pseudo, self.mu, self.inv_sigma)
            fuse_tail = False
        if fuse_tail:
            return rst
        if pad:
            rst = rst[..., :self._out_feats]
        return self._finish(rst, feat)

    def _finish(self, rst, feat):
        if self.res_fc is not None:
            rst = rst + self.res_fc(feat)
        if self.bias is not None:
            rst = add_bias(rst, self.bias)
        return rst

    def _aggregate_first(self, feat):
        """Whether the layer aggregates its input before the fc (recomputing layer only): when the input is
        narrower than the K x out floats an edge would gather otherwise, and the operator takes the shape."""
        k, fin = self._n_kernels, feat.shape[1]
        return (type(self)._op is GmmConvFuseSum and feat.dim() == 2 and fin < k * self._out_feats
                and gmm_native.shared_supported(k, fin))

    def _forward_aggregate_first(self, rowptr, colind, colptr, rowind, permute, feat, pseudo, pseudo_csc, own_order):
        """sum_k (sum_p w[p,k] feat[col(p),:]) @ W_k: the reference's sum over k of the aggregated fc(feat)[:,k,:]
        (layers/gmmconv_layer.py:67-69) with the two linear steps exchanged."""
        k, fin, fout = self._n_kernels, feat.shape[1], self._out_feats
        feat = feat.contiguous()
        if pseudo_csc is not None or own_order:
            if own_order and pseudo_csc is None and th.is_grad_enabled() and (feat.requires_grad or pseudo.requires_grad):
                raise ValueError("own_order without pseudo_csc is forward-only")
            agg = GmmAggregateTwoOrders(rowptr, colind, colptr, rowind, feat, pseudo.detach(), pseudo_csc, self.mu, self.inv_sigma,
                                        own_order=own_order)
        else:
            agg = GmmAggregate(rowptr, colind, colptr, rowind, permute, feat, pseudo, self.mu, self.inv_sigma)
        w = self.fc.weight.view(k, fout, fin).permute(1, 0, 2).reshape(fout, k * fin)       # [out, K*in]: rst = agg.view(N, K*in) @ w^T
        return tall_linear(agg.view(-1, k * fin), w)


class GMMConv(_GMMBase):
    """The `.sum(1)` over the mixture kernels of the reference layer (layers/gmmconv_layer.py:69) is
    fused into the operator."""
    _op = staticmethod(GmmConvFuseSum)


def _stash_sum(*args):
    return GmmConvStash(*args).sum(1)


class GMMConv_stash(_GMMBase):
    _op = staticmethod(_stash_sum)
