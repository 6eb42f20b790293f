"""Single-layer forward latency and memory: the three fused rows of the reference's figure 9
(script/inference/gatconv_our_forward.py, edgeconv_our_forward.py, gmmconv_our_forward.py; driver
script/figure9.sh).  Five untimed calls, then `epochs` timed calls between two synchronisations;
rows "gat_with_fusion,latency=..s,memory=..MB" etc. appended to --output.

    python -m ae_mlsys_gnn_amd.train.forward_latency gat --dataset reddit --in_feats 64 --out_feats 64 --num-heads 4
    python -m ae_mlsys_gnn_amd.train.forward_latency edgeconv --batch-size 64 --k 40
    python -m ae_mlsys_gnn_amd.train.forward_latency monet --dataset reddit --in-feat 16 --out-feat 16 --n-kernels 2 --pseudo-dim 1
"""
from __future__ import annotations

import argparse

import torch

from ..layers import EdgeConv, GATConv, GMMConv
from ..operators.knn import knn_graph
from . import common, datasets


def build_parser():
    p = argparse.ArgumentParser(description="single-layer forward latency")
    sub = p.add_subparsers(dest="layer", required=True)
    g = sub.add_parser("gat")
    g.add_argument("--in_feats", type=int, default=16)
    g.add_argument("--out_feats", type=int, default=6)
    g.add_argument("--num-heads", type=int, default=1)
    g.add_argument("--epochs", type=int, default=400)
    e = sub.add_parser("edgeconv")
    e.add_argument("--batch-size", type=int, default=64)
    e.add_argument("--k", type=int, default=40)
    e.add_argument("--out-feat", type=int, default=64)
    e.add_argument("--epochs", type=int, default=200)
    m = sub.add_parser("monet")
    m.add_argument("--in-feat", type=int, default=16)
    m.add_argument("--out-feat", type=int, default=16)
    m.add_argument("--pseudo-dim", type=int, default=2)
    m.add_argument("--n-kernels", type=int, default=3)
    m.add_argument("--n-epochs", dest="epochs", type=int, default=200)
    for s in (g, e, m):
        s.add_argument("--gpu", type=int, default=0)
        s.add_argument("--output", type=str, default="figure9.csv")
        s.add_argument("--seed", type=int, default=0)
    for s in (g, m):
        s.add_argument("--dataset", type=str, default="cora")
        s.add_argument("--data-root", type=str, default=None)
        s.add_argument("--cache-dir", type=str, default=None)
        s.add_argument("--scale", type=float, default=1.0)
    return p


def main(argv=None):
    args = build_parser().parse_args(argv)
    dev = torch.device("cuda", args.gpu)
    torch.cuda.set_device(dev)
    torch.manual_seed(args.seed)
    if args.layer == "edgeconv":
        pts = torch.randn(args.batch_size, 1024, 3, device=dev)
        src = knn_graph(pts, args.k)
        model = EdgeConv(3, args.out_feat).to(dev)
        x = pts.reshape(-1, 3)
        call, row = (lambda: model(args.k, src, x)), "edgeconv_with_fusion"
    else:
        data = datasets.load_node_dataset(args.dataset, dev, root=args.data_root, seed=args.seed, scale=args.scale, cache_dir=args.cache_dir)
        g = data.graph
        del data
        if args.layer == "gat":
            model = GATConv(args.in_feats, args.out_feats, args.num_heads).to(dev)
            x = torch.rand(g.n, args.in_feats, device=dev)
            call, row = (lambda: model(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, x, True)), "gat_with_fusion"
        else:
            model = GMMConv(args.in_feat, args.out_feat, args.pseudo_dim, args.n_kernels).to(dev)
            x = torch.rand(g.n, args.in_feat, device=dev)
            pseudo = torch.rand(g.n_edges, args.pseudo_dim, device=dev)
            call, row = (lambda: model(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, x, pseudo)), "monet_with_fusion"
    with torch.no_grad():
        sec, mem, _ = common.timed_steps(call, 5, args.epochs, dev)
    print("%s forward time:" % args.layer, sec)
    common.append_row(args.output, "{},latency={}s,memory={:.1f}MB".format(row, sec, mem))
    return {"latency_s": sec, "memory_MB": mem}


if __name__ == "__main__":
    main()
