"""MoNet (GMMConv) node-classification training on the fused GMMConv operators.

Command line, model and protocol of the reference's script/train/train_gmmconv_our.py and
train_gmmconv_stash.py: `n-layers` + 2 GMMConv layers, each with its own Linear(2, pseudo-dim) + Tanh
projection of the degree pseudo-coordinates, dropout between layers; cross-entropy on the training
nodes, Adam; 5 warm-up steps, then `n-epochs` timed steps (each followed by a validation pass, as in
the reference); row "train_monet_<variant>,dataset=..,k=..,d=..,latency=..s,memory=..MB".

    python -m ae_mlsys_gnn_amd.train.train_gmmconv --dataset reddit --n-kernels 2 --pseudo-dim 1
"""
from __future__ import annotations

import argparse

import torch
from torch import nn

from ..layers import GMMConv, GMMConv_stash
from ..operators import edge_proj
from ..operators.fused_gmmconv import gmm_edge_positions
from . import common, datasets

VARIANTS = {"our": GMMConv, "stash": GMMConv_stash}


class PseudoProj(nn.Linear):
    """Linear(2, dim) + Tanh over the per-edge pseudo-coordinates (train_gmmconv_our.py:46-57), same
    parameters as nn.Linear.  Up to 4 output columns run as one fused pass over the edges each way
    (operators.edge_proj; the coordinates are data, only the parameters get gradients).  Wider
    projections are written as two broadcast multiplies: the weight gradient is then a column reduction
    over the edges rather than a 2 x dim GEMM with a reduction length of E, which GEMM libraries run
    on a single workgroup."""

    def forward(self, pseudo):
        if self.out_features <= edge_proj.MAX_OUT and pseudo.is_cuda and not pseudo.requires_grad:
            return edge_proj.edge_linear_tanh(pseudo, self.weight, self.bias)
        out = pseudo[:, 0:1] * self.weight[:, 0] + pseudo[:, 1:2] * self.weight[:, 1]
        return torch.tanh(out + self.bias)


class MoNet(nn.Module):
    def __init__(self, conv, in_feats, n_hidden, out_feats, n_layers, dim, n_kernels, dropout):
        super().__init__()
        sizes = [in_feats] + [n_hidden] * (n_layers + 1) + [out_feats]
        self.layers = nn.ModuleList(conv(sizes[i], sizes[i + 1], dim, n_kernels) for i in range(len(sizes) - 1))
        self.pseudo_proj = nn.ModuleList(PseudoProj(2, dim) for _ in self.layers)
        self.dropout = nn.Dropout(dropout)

    def forward(self, g, feat, pseudo, pseudo_csc=None, own_order=False):
        """pseudo: raw per-edge coordinates [E, 2] in CSR order; pseudo_csc: the same rows in CSC order
        (pseudo[permute]).  With both, each layer projects both copies (the projection is elementwise per
        edge, so the results are each other's permutation) and the layer's backward runs in CSC order.
        own_order: both copies are in the entry order of the operators' schedules instead (`schedule_order_copies`)."""
        h = feat
        for i, (layer, proj) in enumerate(zip(self.layers, self.pseudo_proj)):
            if i:
                h = self.dropout(h)
            if pseudo_csc is not None and torch.is_grad_enabled():
                with torch.no_grad():
                    ps = proj(pseudo)
                h = layer(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, h, ps, pseudo_csc=proj(pseudo_csc), own_order=own_order)
            else:
                h = layer(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, h, proj(pseudo), own_order=own_order)
        return h


def schedule_order_copies(g, pseudo):
    """The raw coordinates in the entry order of the forward (CSR) and backward (CSC) schedules of the
    GMMConv operators.  The coordinates are constant and their projection is elementwise, so the whole
    per-edge pipeline (projection, Gaussian weights, their gradients) can run in those orders and every
    pass streams its per-edge data instead of reaching it through a position map."""
    pos_r = gmm_edge_positions(g.row_ptr, g.col_ind)
    pos_c = gmm_edge_positions(g.col_ptr, g.row_ind, summed_backward=True)
    fwd = pseudo if pos_r is None else pseudo[pos_r.long()].contiguous()
    to_csc = g.permute.long() if pos_c is None else g.permute[pos_c.long()].long()
    return fwd, pseudo[to_csc].contiguous()


def build_parser():
    p = argparse.ArgumentParser(description="MoNet")
    p.add_argument("--dataset", type=str, default="cora")
    p.add_argument("--dropout", type=float, default=0.5)
    p.add_argument("--gpu", type=int, default=0)
    p.add_argument("--lr", type=float, default=1e-2)
    p.add_argument("--n-epochs", type=int, default=2, help="number of timed training steps")
    p.add_argument("--n-hidden", type=int, default=16)
    p.add_argument("--n-layers", type=int, default=0, help="number of extra hidden layers")
    p.add_argument("--pseudo-dim", type=int, default=2)
    p.add_argument("--n-kernels", type=int, default=3)
    p.add_argument("--weight-decay", type=float, default=5e-4)
    p.add_argument("--output", type=str, default="figure7.csv")
    p.add_argument("--variant", choices=sorted(VARIANTS), default="our")
    p.add_argument("--csc-pseudo", type=int, default=2, help="2: keep the edge coordinates in the entry order of the forward and the backward "
                   "schedule, so every pass streams its per-edge data; 1: in CSR and CSC order (no per-edge transposition in "
                   "the backward); 0: one copy, as the reference")
    p.add_argument("--data-root", type=str, default=None)
    p.add_argument("--cache-dir", type=str, default=None)
    p.add_argument("--scale", type=float, default=1.0)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--hip-graph", action="store_true", help="capture the training step into a HIP graph and replay it (pays off on small graphs)")
    return p


def main(argv=None):
    args = build_parser().parse_args(argv)
    dev = torch.device("cuda", args.gpu)
    torch.cuda.set_device(dev)
    data = datasets.load_node_dataset(args.dataset, dev, root=args.data_root, seed=args.seed, scale=args.scale, cache_dir=args.cache_dir)
    g = data.graph
    print("----Data statistics------ (%s)\n  #Nodes %d\n  #Edges %d\n  #Classes %d\n  #Train samples %d\n  #Val samples %d\n  #Test samples %d"
          % (data.source, g.n, g.n_edges, data.n_classes, int(data.train_mask.sum()), int(data.val_mask.sum()), int(data.test_mask.sum())))
    pseudo = datasets.degree_pseudo(g)
    own_order = args.csc_pseudo == 2
    if own_order:
        pseudo, pseudo_csc = schedule_order_copies(g, pseudo)
    else:
        pseudo_csc = pseudo[g.permute.long()].contiguous() if args.csc_pseudo else None
    torch.manual_seed(args.seed)
    model = MoNet(VARIANTS[args.variant], data.feat.shape[1], args.n_hidden, data.n_classes, args.n_layers, args.pseudo_dim, args.n_kernels,
                  args.dropout).to(dev)
    opt = torch.optim.Adam(model.parameters(), lr=args.lr, weight_decay=args.weight_decay, capturable=args.hip_graph)
    train_rows = common.MaskedRows(data.train_mask, data.label)

    def evaluate(mask):
        model.eval()
        with torch.no_grad():
            return common.accuracy(model(g, data.feat, pseudo, own_order=own_order)[mask], data.label[mask])      # no gradients: one copy is enough

    def train_step():
        model.train()
        loss = common.masked_cross_entropy(model(g, data.feat, pseudo, pseudo_csc, own_order=own_order), train_rows)      # the mean over logits[train_mask]
        opt.zero_grad(set_to_none=False)
        loss.backward()
        opt.step()
        return loss.detach()

    def epoch():
        loss = train_step()
        evaluate(data.val_mask)
        return loss

    first = float(train_step())
    if args.hip_graph:
        train_step = common.capture_step(train_step, dev)
    for _ in range(args.warmup):
        train_step()
    sec, mem, loss = common.timed_steps(epoch, 0, args.n_epochs, dev)
    acc = evaluate(data.test_mask)
    print("loss {:.4f} -> {:.4f}".format(first, float(loss)))
    print("one epoch time: {:.4f} s".format(sec))
    print("Test Accuracy {:.4f}".format(acc))
    common.append_row(args.output, "train_monet_{},dataset={},k={},d={},latency={}s,memory={:.1f}MB".format(
        args.variant, args.dataset, args.n_kernels, args.pseudo_dim, sec, mem))
    return {"latency_s": sec, "memory_MB": mem, "first_loss": first, "last_loss": float(loss), "test_acc": acc, "source": data.source,
            "nodes": g.n, "edges": g.n_edges}


if __name__ == "__main__":
    main()
