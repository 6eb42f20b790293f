"""GAT node-classification training on the fused GAT operators.

Command line, model and protocol of the reference's script/train/train_gatconv_our.py (recompute
variant), train_gatconv_stash.py (stash) and the fuse-scatter layer: `num-layers` hidden GATConv
layers with `num-heads` heads, flattened, plus an output GATConv averaged over `num-out-heads`;
cross-entropy on the training nodes, Adam; 10 warm-up steps, then `epochs` timed steps; one row
"train_GAT_<variant>,dataset=..,head=..,f=..,latency=..s,memory=..MB" appended to --output.

    python -m ae_mlsys_gnn_amd.train.train_gatconv --dataset reddit --num-heads 4 --num-hidden 64
"""
from __future__ import annotations

import argparse

import torch
from torch import nn

from ..layers import GATConv, GATConv_fusescatter, GATConv_stash
from . import common, datasets

VARIANTS = {"our": GATConv, "stash": GATConv_stash, "fusescatter": GATConv_fusescatter}


class GAT(nn.Module):
    def __init__(self, conv, num_layers, in_dim, num_hidden, num_classes, heads, negative_slope):
        super().__init__()
        dims = [in_dim] + [num_hidden * heads[l] for l in range(num_layers)]
        self.hidden = nn.ModuleList(conv(dims[l], num_hidden, heads[l], negative_slope) for l in range(num_layers))
        self.out = conv(dims[-1], num_classes, heads[-1], negative_slope)

    def forward(self, g, x, extra, keep_padding=False):
        """keep_padding: the logits keep the output layer's zero columns up to a multiple of four ([N, >= classes]); the
        loss is told the number of classes instead of reading a cropped view."""
        for layer in self.hidden:
            x = layer(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, x, extra).flatten(1)
        return common.head_mean(self.out(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, x, extra, keep_padding=keep_padding))


def build_parser():
    p = argparse.ArgumentParser(description="GAT")
    p.add_argument("--dataset", type=str, default="cora")
    p.add_argument("--gpu", type=int, default=0, help="which GPU to use")
    p.add_argument("--epochs", type=int, default=10, help="number of timed training steps")
    p.add_argument("--num-heads", type=int, default=1, help="number of hidden attention heads")
    p.add_argument("--num-out-heads", type=int, default=1, help="number of output attention heads")
    p.add_argument("--num-layers", type=int, default=1, help="number of hidden layers")
    p.add_argument("--num-hidden", type=int, default=8, help="number of hidden units")
    p.add_argument("--lr", type=float, default=0.005)
    p.add_argument("--weight-decay", type=float, default=5e-4)
    p.add_argument("--negative-slope", type=float, default=0.2)
    p.add_argument("--output", type=str, default="figure7.csv")
    p.add_argument("--variant", choices=sorted(VARIANTS), default="our", help="our = recompute in backward, stash / fusescatter = keep per-edge tensors")
    p.add_argument("--data-root", type=str, default=None, help="directory with dataset files; synthetic data of the dataset's shape when absent")
    p.add_argument("--cache-dir", type=str, default=None, help="keep the preprocessed graph arrays here")
    p.add_argument("--scale", type=float, default=1.0, help="shrink a synthetic dataset (nodes and edges) by this factor")
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--hip-graph", action="store_true", help="capture the training step into a HIP graph and replay it (pays off on small graphs)")
    return p


def main(argv=None):
    args = build_parser().parse_args(argv)
    dev = torch.device("cuda", args.gpu)
    torch.cuda.set_device(dev)
    data = datasets.load_node_dataset(args.dataset, dev, root=args.data_root, seed=args.seed, scale=args.scale, cache_dir=args.cache_dir)
    g = data.graph
    print("----Data statistics------ (%s)\n  #Nodes %d\n  #Edges %d\n  #Classes %d\n  #Train samples %d\n  #Val samples %d\n  #Test samples %d\n  #Input features %d"
          % (data.source, g.n, g.n_edges, data.n_classes, int(data.train_mask.sum()), int(data.val_mask.sum()), int(data.test_mask.sum()),
             data.feat.shape[1]))
    torch.manual_seed(args.seed)
    heads = [args.num_heads] * args.num_layers + [args.num_out_heads]
    model = GAT(VARIANTS[args.variant], args.num_layers, data.feat.shape[1], args.num_hidden, data.n_classes, heads, args.negative_slope).to(dev)
    extra = True if args.variant == "our" else g.permute
    opt = torch.optim.Adam(model.parameters(), lr=args.lr, weight_decay=args.weight_decay, capturable=args.hip_graph)
    train_rows = common.MaskedRows(data.train_mask, data.label)

    def step():
        model.train()
        logits = model(g, data.feat, extra, keep_padding=True)
        loss = common.masked_cross_entropy(logits, train_rows, data.n_classes)      # the mean over logits[train_mask]
        opt.zero_grad(set_to_none=False)
        loss.backward()
        opt.step()
        return loss.detach()

    first = float(step())
    if args.hip_graph:
        step = common.capture_step(step, dev)
    sec, mem, loss = common.timed_steps(step, args.warmup, args.epochs, dev)
    model.eval()
    with torch.no_grad():
        acc = common.accuracy(model(g, data.feat, extra)[data.test_mask], data.label[data.test_mask])
    print("loss {:.4f} -> {:.4f}".format(first, float(loss)))
    print("Test Accuracy {:.4f}".format(acc))
    print("train time:", sec)
    common.append_row(args.output, "train_GAT_{},dataset={},head={},f={},latency={}s,memory={:.1f}MB".format(
        args.variant, args.dataset, args.num_heads, args.num_hidden, sec, mem))
    return {"latency_s": sec, "memory_MB": mem, "first_loss": first, "last_loss": float(loss), "test_acc": acc, "source": data.source,
            "nodes": g.n, "edges": g.n_edges}


if __name__ == "__main__":
    main()
