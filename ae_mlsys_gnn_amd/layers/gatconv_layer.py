"""GAT layers on the fused operators (interface of the reference's layers/gatconv_layer.py:10-158).

Orientation: the graph is CSR by destination; ``attn_l`` scores the destination (row) side and
``attn_r`` the source (column) side (layers/gatconv_layer.py:52-55), the mirror image of DGL's
GATConv where ``attn_l`` belongs to the source."""
from __future__ import annotations

import torch
from torch import nn

from ..operators.fused_gat import fused_gat_fusescatter, fused_gat_op, fused_gat_stash_op
from .dense import reduce_over_rows


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
        (layers/gatconv_layer.py:50-53 of the reference).  When out_feats is not a multiple of 4
        (output layers: one head x number of classes) h gets zero columns up to the next multiple,
        so that the operator takes its 128-bit row layout; `_crop` drops them again."""
        return _ProjectScores.apply(feat, self.W, self.attn_l, self.attn_r, (-self.out_feats) % 4)

    def _crop(self, out, keep_padding=False):
        """keep_padding: hand the operator's zero-padded [N, H, out_feats rounded up to 4] array on as it is (a consumer
        that takes the number of valid columns, such as the drivers' fused cross-entropy, then needs neither the
        cropped view nor the zero-filled copy its gradient would go through)."""
        return out if keep_padding or out.shape[-1] == self.out_feats else out[..., :self.out_feats]


class _ProjectScores(torch.autograd.Function):
    """The dense part of the layer.  The scores are formed as feat @ ((W * attn).sum(-1)): the same
    sums taken in another order, as one thin GEMM over `feat` instead of two strided reductions over
    the [N,H,F] projection.  The backward stacks the gradients of the projection and of the scores
    into one [N, H*F + 2H] operand when the input gradient is wanted, so that it is one GEMM and `feat` is
    reduced over the nodes once; a first layer reduces the two parts separately instead of copying the wide one."""

    @staticmethod
    def forward(ctx, feat, W, attn_l, attn_r, pad):
        _, hh, ff = attn_l.shape
        wv = W.view(W.shape[0], hh, ff)
        w_score = torch.cat([(wv * attn_l).sum(-1), (wv * attn_r).sum(-1)], dim=1)       # [in, 2H]
        w_proj = W if pad == 0 else torch.cat([wv, wv.new_zeros(W.shape[0], hh, pad)], dim=2).reshape(W.shape[0], -1)
        h = torch.matmul(feat, w_proj)
        score = torch.matmul(feat, w_score)
        ctx.save_for_backward(feat, W, attn_l, attn_r, torch.cat([w_proj, w_score], dim=1))
        ctx.pad = pad
        return h.view(-1, hh, ff + pad), score[:, :hh].contiguous(), score[:, hh:].contiguous()

    @staticmethod
    def backward(ctx, dh, drow, dcol):
        feat, W, attn_l, attn_r, w_all = ctx.saved_tensors
        _, hh, ff = attn_l.shape
        n, hfp = feat.shape[0], hh * (ff + ctx.pad)
        zeros = lambda cols: feat.new_zeros(n, cols)
        if ctx.needs_input_grad[0] or dh is None:
            g = torch.cat([zeros(hfp) if dh is None else dh.reshape(n, hfp), zeros(hh) if drow is None else drow,
                           zeros(hh) if dcol is None else dcol], dim=1)                    # [N, H*Fp + 2H]
            dfeat = torch.matmul(g, w_all.t()) if ctx.needs_input_grad[0] else None
            dw_ext = reduce_over_rows(feat, g)                                          # [in, H*Fp + 2H]
        else:
            # first layer (no input gradient): nothing needs the stacked operand, so the wide gradient is not copied;
            # two reductions over feat (2.45 M x 100 -> 256 + 16 columns: 1.2 + 0.3 ms against 1.3 ms of copy + 1.7 ms)
            dfeat = None
            gs = torch.cat([zeros(hh) if drow is None else drow, zeros(hh) if dcol is None else dcol], dim=1)
            dw_ext = torch.cat([reduce_over_rows(feat, dh.reshape(n, hfp)), reduce_over_rows(feat, gs)], dim=1)
        dwl, dwr = dw_ext[:, hfp:hfp + hh].unsqueeze(-1), dw_ext[:, hfp + hh:].unsqueeze(-1)   # [in, H, 1]
        wv = W.view(W.shape[0], hh, ff)
        dW = dw_ext[:, :hfp].view(W.shape[0], hh, ff + ctx.pad)[:, :, :ff] + dwl * attn_l + dwr * attn_r
        return dfeat, dW.reshape(W.shape), (wv * dwl).sum(0, keepdim=True), (wv * dwr).sum(0, keepdim=True), None


class GATConv(_GATBase):
    """Recompute variant: nothing edge-sized survives the forward."""

    def forward(self, row_ptr, col_ind, col_ptr, row_ind, feat, save_memory=True, keep_padding=False):
        h, attn_row, attn_col = self._project(feat)
        return self._crop(fused_gat_op(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, self.negative_slope, h, save_memory), keep_padding)


class GATConv_stash(_GATBase):
    """Stash variant: per-edge LeakyReLU / softmax values [E,H] are kept for the backward."""

    def forward(self, row_ptr, col_ind, col_ptr, row_ind, feat, permute, keep_padding=False):
        h, attn_row, attn_col = self._project(feat)
        return self._crop(fused_gat_stash_op(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, self.negative_slope, h, permute), keep_padding)


class GATConv_fusescatter(_GATBase):
    def forward(self, row_ptr, col_ind, col_ptr, row_ind, feat, permute, keep_padding=False):
        h, attn_row, attn_col = self._project(feat)
        return self._crop(fused_gat_fusescatter(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, self.negative_slope, h, permute), keep_padding)
