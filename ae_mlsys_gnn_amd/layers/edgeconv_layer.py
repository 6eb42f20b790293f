"""EdgeConv layer on the fused operator (interface of the reference's layers/edgeconv_layer.py:6-43)."""
from __future__ import annotations

import torch
from torch import nn

from ..operators.fused_edgeconv import fused_edgeconv_op
from .dense import tall_linear


class EdgeConv(nn.Module):
    """out_i = max_j (theta(x_j) + phi(x_i) - theta(x_i)) over the k neighbours j of i, i.e. the
    operator-reorganised form of max_j (theta(x_j - x_i) + phi(x_i)) with bias-free theta, phi."""

    def __init__(self, in_feat, out_feat, batch_norm=False, allow_zero_in_degree=False):
        super().__init__()
        self.batch_norm = batch_norm
        self._allow_zero_in_degree = allow_zero_in_degree
        self.theta = nn.Linear(in_feat, out_feat, bias=False)
        self.phi = nn.Linear(in_feat, out_feat, bias=False)
        if batch_norm:
            self.bn = nn.BatchNorm1d(out_feat)

    def set_allow_zero_in_degree(self, set_value):
        self._allow_zero_in_degree = set_value

    def forward(self, k, src_ind, feat, block=None, negative_slope_out=None):
        """block: points per cloud when src_ind is a kNN graph of equally sized clouds (see fused_edgeconv_op).
        negative_slope_out: apply LeakyReLU with this slope to the result inside the operator (the activation that
        follows every EdgeConv of the reference's DGCNN, script/train/train_edgeconv_our.py:56)."""
        # theta and phi read the same rows: one product with the stacked weights (its weight gradient
        # reduced over the points in chunks), split afterwards
        out_feat = self.theta.out_features
        h = tall_linear(feat, torch.cat([self.theta.weight, self.phi.weight], 0))
        h_theta, h_phi = h[:, :out_feat], h[:, out_feat:]
        h_src = h_theta.contiguous()
        h_dst = h_phi - h_theta
        return fused_edgeconv_op(k, src_ind, h_src, h_dst, block, negative_slope_out)
