"""Shared pieces of the training drivers: the timing protocol of the reference's scripts (untimed
warm-up steps, then N steps between two device synchronisations, script/train/train_gatconv_our.py:
158-200), peak-memory accounting and the result row appended to the output CSV."""
from __future__ import annotations

import time

import torch


def head_mean(t):
    """Mean over the heads of [N, H, C] (the reference's `.mean(1)` on the output layer); with one head it is
    the same values without a pass over the tensor."""
    return t.squeeze(1) if t.shape[1] == 1 else t.mean(1)


def accuracy(logits, labels):
    if labels.numel() == 0:
        return float("nan")
    return float((logits.argmax(dim=1) == labels).float().mean())


def cross_entropy(logits, labels, n_classes=None):
    """Mean cross-entropy, the value of torch.nn.CrossEntropyLoss()(logits[:, :n_classes], labels).  float32 logits on
    the GPU go through the library's fused row pass (one kernel each way; `logits` may be a zero-padded [N, >= n_classes]
    array, whose gradient then comes back in the same width); anything else is written as logsumexp minus the true-class
    logit: with millions of rows torch's nll_loss kernels reduce on very few workgroups (9 ms of a 70 ms step at 2.4 M
    nodes), a gather does not."""
    if logits.is_cuda and logits.dtype == torch.float32 and logits.dim() == 2 and labels.dtype == torch.int64 and logits.shape[0] > 0:
        from ..operators.loss import cross_entropy_rows
        if logits.shape[1] > 1 and logits.stride(1) != 1:
            logits = logits.contiguous()
        return cross_entropy_rows(logits, labels, n_classes).mean()
    if n_classes is not None:
        logits = logits[:, :n_classes]
    return (torch.logsumexp(logits, dim=1) - logits.gather(1, labels.unsqueeze(1)).squeeze(1)).mean()


class MaskedRows:
    """The rows a loss is taken over (script/train/train_gatconv_our.py:167: loss_fcn(logits[train_mask],
    labels[train_mask])) as a weight per row (1 on the selected rows, 0 elsewhere) and their count.  masked_cross_entropy then
    needs no gathered copy of the selected logits rows and no scatter of their gradient back into a zero-filled
    array (at 2.4 M nodes x 47 classes those two index kernels were 0.9 ms of a 15 ms step); the labels of the other
    rows are replaced by class 0 so that a placeholder outside [0, C) cannot turn into 0 x NaN."""

    def __init__(self, mask, labels):
        mask = mask.bool()
        count = int(mask.sum())
        self.count = count
        self.weight = mask.to(torch.float32)
        self.labels = torch.where(mask, labels, torch.zeros_like(labels)).contiguous()


def masked_cross_entropy(logits, rows: MaskedRows, n_classes=None):
    """Mean cross-entropy over the rows selected by `rows`: the value and gradient of
    cross_entropy(logits[mask], labels[mask], n_classes), computed from the per-row losses of ALL rows weighted by
    rows.weight and divided by rows.count (fused row pass on the GPU; the unselected rows get a zero gradient)."""
    if logits.is_cuda and logits.dtype == torch.float32 and logits.dim() == 2 and logits.shape[0] > 0:
        from ..operators.loss import cross_entropy_rows
        if logits.shape[1] > 1 and logits.stride(1) != 1:
            logits = logits.contiguous()
        return torch.dot(cross_entropy_rows(logits, rows.labels, n_classes), rows.weight) / max(rows.count, 1)
    if n_classes is not None:
        logits = logits[:, :n_classes]
    per_row = torch.logsumexp(logits, dim=1) - logits.gather(1, rows.labels.unsqueeze(1)).squeeze(1)
    return (per_row * rows.weight.to(per_row.dtype)).sum() / max(rows.count, 1)


def timed_steps(step, warmup, steps, device):
    """Runs `step` warmup + steps times; returns (seconds per timed step, peak MB of HBM allocated by
    torch on `device` over all of them, value returned by the last step)."""
    torch.cuda.reset_peak_memory_stats(device)
    last = None
    for _ in range(warmup):
        last = step()
    torch.cuda.synchronize(device)
    t0 = time.time()
    for _ in range(steps):
        last = step()
    torch.cuda.synchronize(device)
    sec = (time.time() - t0) / max(1, steps)
    return sec, torch.cuda.max_memory_allocated(device) / 2**20, last


def capture_step(step, device, warmup=3):
    """Captures `step` (forward, loss, backward, optimizer step; it must return the loss tensor) into
    a HIP graph after `warmup` eager calls on a side stream, and returns a callable that replays it
    and hands back the graph's loss tensor.  For small graphs a training step is a few dozen short
    kernels and launch-bound; the replay submits them as one unit.  The library's operators enqueue
    kernels only (buffers are cleared with fill kernels, never memset nodes, and nothing
    synchronises once the schedules exist), so they can be captured; the optimizer must be built
    with capturable=True."""
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        for _ in range(warmup):
            step()
    torch.cuda.current_stream(device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loss = step()

    def replay():
        graph.replay()
        return loss
    replay.graph = graph
    return replay


def append_row(path, row):
    print(row)
    if path:
        with open(path, "a") as f:
            print(row, file=f)
