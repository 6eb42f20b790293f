"""The end-to-end sweeps of the reference's script/train/end_2_end.py (figure 7) and figure10.sh
(recompute against stash) on this build's drivers, in one process, one configuration after the
other.  Data comes from --data-root when the files are there, else synthetic graphs and clouds of
the datasets' shapes.  Prints every row next to the figure the reference's authors recorded for it
on their hardware (example_data/figure7.csv, figure10.csv: RTX 3090), which is context rather than
a like-for-like comparison.

    python -m ae_mlsys_gnn_amd.train.end_2_end --sets gat monet edgeconv --output figure7.csv
"""
from __future__ import annotations

import argparse
import gc

import torch

from . import forward_latency, train_edgeconv, train_gatconv, train_gmmconv

# (seconds, MB) the reference's example_data holds for its fused ("our") rows; figure10 for stash
PUBLISHED = {
    ("gat", "cora", "our"): (0.004127, 1410), ("gat", "pubmed", "our"): (0.004253, 1470), ("gat", "citeseer", "our"): (0.004212, 1436),
    ("gat", "reddit", "our"): (0.2914, 4128),
    ("gat4x64", "reddit", "our"): (0.5762, 5688), ("gat4x64", "reddit", "stash"): (0.5532, 10692),
    ("monet", "reddit", "our"): (0.7364, 7202), ("monet", "reddit", "stash"): (0.7447, 9396),
    ("edgeconv", (20, 32), "our"): (0.0947, 2376), ("edgeconv", (20, 64), "our"): (0.1774, 2762),
    ("edgeconv", (40, 32), "our"): (0.1036, 2376), ("edgeconv", (40, 64), "our"): (0.1883, 2762),
    # figure9.csv: single-layer forward
    ("forward", "gat 64->4x64", "our"): (0.1021, 2774), ("forward", "edgeconv b=64 k=40", "our"): (0.004418, 1470),
    ("forward", "monet 16->16 K=2 d=1", "our"): (0.02439, 3212),
}


def _free():
    gc.collect()
    from .. import _lib
    _lib.clear_schedule_cache()
    torch.cuda.empty_cache()


def main(argv=None):
    p = argparse.ArgumentParser(description="end-to-end sweeps")
    p.add_argument("--sets", nargs="+", default=["gat", "monet", "edgeconv", "stash", "forward"], choices=["gat", "monet", "edgeconv", "stash", "forward"])
    p.add_argument("--datasets", nargs="+", default=["cora", "pubmed", "citeseer", "reddit"])
    p.add_argument("--epochs", type=int, default=20)
    p.add_argument("--edgeconv-iters", type=int, default=20, help="training iterations per timed epoch of the DGCNN runs")
    p.add_argument("--output", type=str, default="")
    p.add_argument("--data-root", type=str, default=None)
    p.add_argument("--scale", type=float, default=1.0)
    args = p.parse_args(argv)
    common = ["--output", args.output, "--scale", str(args.scale)] + (["--data-root", args.data_root] if args.data_root else [])
    rows = []

    def record(kind, key, variant, r):
        pub = PUBLISHED.get((kind, key, variant))
        rows.append((kind, key, variant, r["latency_s"], r["memory_MB"], pub))
        _free()

    if "gat" in args.sets:                      # end_2_end.py:7-11: 1 head x 128
        for ds in args.datasets:
            record("gat", ds, "our", train_gatconv.main(["--dataset", ds, "--num-heads", "1", "--num-hidden", "128", "--epochs", str(args.epochs)] + common))
    if "monet" in args.sets:                    # end_2_end.py:20-24
        dims = {"cora": (3, 2), "pubmed": (3, 3), "citeseer": (3, 3), "reddit": (2, 1)}
        for ds in args.datasets:
            k, d = dims.get(ds, (3, 2))
            record("monet", ds, "our", train_gmmconv.main(["--dataset", ds, "--n-epochs", str(args.epochs), "--n-hidden", "16", "--n-kernels", str(k),
                                                           "--pseudo-dim", str(d)] + common))
    if "edgeconv" in args.sets:                 # end_2_end.py:14-17
        for k in (20, 40):
            for batch in (32, 64):
                record("edgeconv", (k, batch), "our", train_edgeconv.main(["--k", str(k), "--batch-size", str(batch), "--num-epochs", "2", "--warmup-epochs", "1",
                                                                           "--iters-per-epoch", str(args.edgeconv_iters), "--num-clouds", "2048",
                                                                           "--output", args.output]))
    if "stash" in args.sets and "reddit" in args.datasets:      # figure10.sh: 4 heads x 64, K=2 / dim 1
        for variant in ("our", "stash"):
            record("gat4x64", "reddit", variant, train_gatconv.main(["--dataset", "reddit", "--num-heads", "4", "--num-hidden", "64", "--epochs", str(args.epochs),
                                                                     "--variant", variant] + common))
            record("monet", "reddit", variant, train_gmmconv.main(["--dataset", "reddit", "--n-epochs", str(args.epochs), "--n-hidden", "16", "--n-kernels", "2",
                                                                   "--pseudo-dim", "1", "--variant", variant] + common))
    if "forward" in args.sets:                  # figure9.sh
        fwd = ["--output", args.output, "--epochs", str(max(20, args.epochs))]
        ds = ["--dataset", "reddit", "--scale", str(args.scale)] + (["--data-root", args.data_root] if args.data_root else [])
        record("forward", "gat 64->4x64", "our", forward_latency.main(["gat", "--in_feats", "64", "--out_feats", "64", "--num-heads", "4"] + ds + fwd))
        record("forward", "edgeconv b=64 k=40", "our", forward_latency.main(["edgeconv", "--batch-size", "64", "--k", "40"] + fwd))
        record("forward", "monet 16->16 K=2 d=1", "our", forward_latency.main(["monet", "--in-feat", "16", "--out-feat", "16", "--n-kernels", "2", "--pseudo-dim", "1"]
                                                                             + ds + ["--output", args.output, "--n-epochs", str(max(20, args.epochs))]))
    print("\n| run | config | variant | s/step | peak MB | recorded by the reference (RTX 3090) |")
    print("|---|---|---|---|---|---|")
    for kind, key, variant, sec, mem, pub in rows:
        print("| %s | %s | %s | %.5f | %.0f | %s |" % (kind, key, variant, sec, mem, "%.4f s, %d MB" % pub if pub else "-"))
    return rows


if __name__ == "__main__":
    main()
