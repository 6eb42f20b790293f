"""DGCNN point-cloud classification training on the fused EdgeConv operator.

Model and protocol of the reference's script/train/train_edgeconv_our.py: four EdgeConv layers
(64, 64, 128, 256) on a kNN graph rebuilt from each layer's input, LeakyReLU(0.2) after each,
concatenation, Linear to 512, max + mean pooling over the cloud, two Linear/BatchNorm/LeakyReLU/
Dropout blocks, Linear to the classes; smoothed cross-entropy (eps 0.2), SGD(0.1, momentum 0.9,
weight decay 1e-4) with cosine annealing; random scale/shift augmentation and point shuffling per
sample.  The kNN graph comes from the library's own builder (--knn fgnn) or torch cdist + topk.
Row: "train_edgeconv_our,dataset=modelnet40,k=..,batch=..,latency=..s,memory=..MB", latency per
training iteration.

    python -m ae_mlsys_gnn_amd.train.train_edgeconv --k 20 --batch-size 32
"""
from __future__ import annotations

import argparse

import torch
import torch.nn.functional as F
from torch import nn

from .. import graphs
from ..layers import EdgeConv
from ..layers.dense import tall_linear
from ..operators.knn import knn_graph
from . import common, datasets


class Model(nn.Module):
    def __init__(self, k, feature_dims, emb_dims, output_classes, input_dims=3, dropout_prob=0.5, knn="fgnn"):
        super().__init__()
        self.k = k
        self.knn = knn_graph if knn == "fgnn" else graphs.knn_graph
        dims = [input_dims] + list(feature_dims)
        self.conv = nn.ModuleList(EdgeConv(dims[i], dims[i + 1]) for i in range(len(feature_dims)))
        self.proj = nn.Linear(sum(feature_dims), emb_dims[0])
        ins = [emb_dims[0] * 2] + list(emb_dims[1:-1])          # * 2: max- and mean-pooling concatenated
        self.embs = nn.ModuleList(nn.Linear(i, o) for i, o in zip(ins, emb_dims[1:]))
        self.bn_embs = nn.ModuleList(nn.BatchNorm1d(o) for o in emb_dims[1:])
        self.dropouts = nn.ModuleList(nn.Dropout(dropout_prob) for _ in emb_dims[1:])
        self.proj_output = nn.Linear(emb_dims[-1], output_classes)

    def forward(self, x):
        b, p, _ = x.shape
        h, hs = x, []
        for conv in self.conv:
            src = self.knn(h.detach(), self.k)
            h = conv(self.k, src, h.reshape(b * p, -1), block=p, negative_slope_out=0.2).view(b, p, -1)     # LeakyReLU(0.2) fused in
            hs.append(h)
        h = tall_linear(torch.cat(hs, 2).view(b * p, -1), self.proj.weight, self.proj.bias).view(b, p, -1)
        h = torch.cat([h.max(1).values, h.mean(1)], 1)
        for emb, bn, drop in zip(self.embs, self.bn_embs, self.dropouts):
            h = drop(F.leaky_relu(bn(emb(h)), 0.2))
        return self.proj_output(h)


def compute_loss(logits, y, eps=0.2):
    """Cross-entropy against the true class at weight 1-eps and every other class at eps/(C-1)."""
    c = logits.shape[1]
    lp = F.log_softmax(logits, 1)
    true = lp.gather(1, y.view(-1, 1)).squeeze(1)
    return -((1 - eps) * true + eps / (c - 1) * (lp.sum(1) - true)).mean()


def augment(x, gen):
    """Per-cloud random anisotropic scale in [2/3, 3/2] and shift in [-0.2, 0.2], points shuffled."""
    b, p, _ = x.shape
    scale = torch.rand(b, 1, 3, device=x.device, generator=gen) * (3 / 2 - 2 / 3) + 2 / 3
    shift = torch.rand(b, 1, 3, device=x.device, generator=gen) * 0.4 - 0.2
    order = torch.rand(b, p, device=x.device, generator=gen).argsort(1)
    return torch.gather(x * scale + shift, 1, order.unsqueeze(2).expand(b, p, 3))


def build_parser():
    p = argparse.ArgumentParser(description="DGCNN")
    p.add_argument("--dataset-path", type=str, default="", help=".npz (data, label) or .h5 with train/data, train/label; synthetic clouds when empty")
    p.add_argument("--num-epochs", type=int, default=10)
    p.add_argument("--batch-size", type=int, default=64)
    p.add_argument("--k", type=int, default=40)
    p.add_argument("--output", type=str, default="figure7.csv")
    p.add_argument("--gpu", type=int, default=0)
    p.add_argument("--num-clouds", type=int, default=9840, help="synthetic training set size (one fifth is held out, as in the reference)")
    p.add_argument("--num-points", type=int, default=1024)
    p.add_argument("--iters-per-epoch", type=int, default=0, help="0 = one pass over the training clouds")
    p.add_argument("--warmup-epochs", type=int, default=3)
    p.add_argument("--knn", choices=["fgnn", "torch"], default="fgnn")
    p.add_argument("--seed", type=int, default=0)
    return p


def main(argv=None):
    args = build_parser().parse_args(argv)
    print(args)
    dev = torch.device("cuda", args.gpu)
    torch.cuda.set_device(dev)
    clouds = datasets.load_point_clouds(dev, args.dataset_path or None, args.num_clouds, args.num_points, seed=args.seed)
    n_train = clouds.data.shape[0] - clouds.data.shape[0] // 5
    iters = args.iters_per_epoch or max(1, n_train // args.batch_size)
    torch.manual_seed(args.seed)
    model = Model(args.k, [64, 64, 128, 256], [512, 512, 256], clouds.n_classes, knn=args.knn).to(dev)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=1e-4)
    sched = torch.optim.lr_scheduler.CosineAnnealingLR(opt, max(1, args.num_epochs), eta_min=0.001)
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    losses, accs = [], []

    def epoch():
        model.train()
        order = torch.randperm(n_train, device=dev, generator=gen)
        total, correct = torch.zeros((), device=dev), torch.zeros((), device=dev)
        for it in range(iters):
            idx = order[(it * args.batch_size) % max(1, n_train - args.batch_size + 1):][:args.batch_size]
            x, y = augment(clouds.data[idx], gen), clouds.label[idx]
            opt.zero_grad()
            logits = model(x)
            loss = compute_loss(logits, y)
            loss.backward()
            opt.step()
            total += loss.detach()
            correct += (logits.argmax(1) == y).float().mean()
        sched.step()
        losses.append(float(total) / iters)
        accs.append(float(correct) / iters)
        return losses[-1]

    sec, mem, _ = common.timed_steps(epoch, args.warmup_epochs, args.num_epochs, dev)
    per_iter = sec / iters
    print("mean loss per epoch:", ["%.4f" % l for l in losses])
    print("training accuracy per epoch:", ["%.3f" % a for a in accs])
    print("train time:", per_iter)
    common.append_row(args.output, "train_edgeconv_our,dataset=modelnet40,k={},batch={},latency={}s,memory={:.1f}MB".format(
        args.k, args.batch_size, per_iter, mem))
    return {"latency_s": per_iter, "memory_MB": mem, "losses": losses, "train_acc": accs, "source": clouds.source, "iters_per_epoch": iters}


if __name__ == "__main__":
    main()
