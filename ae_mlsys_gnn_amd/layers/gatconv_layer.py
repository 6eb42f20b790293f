"""GAT layers on the fused operators (interface of the reference's layers/gatconv_layer.py:10-158).

Orientation: the graph is CSR by destination; ``attn_l`` scores the destination (row) side and
``attn_r`` the source (column) side (layers/gatconv_layer.py:52-55), the mirror image of DGL's
GATConv where ``attn_l`` belongs to the source."""
from __future__ import annotations

import torch
from torch import nn

from ..operators.fused_gat import fused_gat_fusescatter, fused_gat_op, fused_gat_stash_op


class _GATBase(nn.Module):
    def __init__(self, in_feats, out_feats, num_heads, negative_slope=0.2):
        super().__init__()
        self.in_feats = in_feats
        self.out_feats = out_feats
        self.num_heads = num_heads
        self.negative_slope = negative_slope
        self.W = nn.Parameter(torch.empty(in_feats, out_feats * num_heads))
        self.attn_l = nn.Parameter(torch.empty(1, num_heads, out_feats))
        self.attn_r = nn.Parameter(torch.empty(1, num_heads, out_feats))
        self.reset_parameters()

    def reset_parameters(self):
        # Xavier-normal with the ReLU gain on all three parameters (layers/gatconv_layer.py:30-45)
        gain = nn.init.calculate_gain("relu")
        for p in (self.W, self.attn_l, self.attn_r):
            nn.init.xavier_normal_(p, gain=gain)

    def _project(self, feat):
        """h = feat @ W and the two attention scores (attn_l * h).sum(-1), (attn_r * h).sum(-1)
        (layers/gatconv_layer.py:50-53 of the reference).  The scores are formed as
        feat @ ((W * attn).sum(-1)): the same sums taken in another order, as one thin GEMM over
        `feat` instead of two strided reductions over the [N,H,F] projection."""
        hh, ff = self.num_heads, self.out_feats
        h = torch.matmul(feat, self.W).view(-1, hh, ff)
        wv = self.W.view(self.in_feats, hh, ff)
        w_score = torch.cat([(wv * self.attn_l).sum(-1), (wv * self.attn_r).sum(-1)], dim=1)      # [in, 2H]
        score = torch.matmul(feat, w_score)
        return h, score[:, :hh].contiguous(), score[:, hh:].contiguous()


class GATConv(_GATBase):
    """Recompute variant: nothing edge-sized survives the forward."""

    def forward(self, row_ptr, col_ind, col_ptr, row_ind, feat, save_memory=True):
        h, attn_row, attn_col = self._project(feat)
        return fused_gat_op(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, self.negative_slope, h, save_memory)


class GATConv_stash(_GATBase):
    """Stash variant: per-edge LeakyReLU / softmax values [E,H] are kept for the backward."""

    def forward(self, row_ptr, col_ind, col_ptr, row_ind, feat, permute):
        h, attn_row, attn_col = self._project(feat)
        return fused_gat_stash_op(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, self.negative_slope, h, permute)


class GATConv_fusescatter(_GATBase):
    def forward(self, row_ptr, col_ind, col_ptr, row_ind, feat, permute):
        h, attn_row, attn_col = self._project(feat)
        return fused_gat_fusescatter(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, self.negative_slope, h, permute)
