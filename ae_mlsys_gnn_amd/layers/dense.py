"""Dense helpers shared by the layers: linear maps over very many rows (one per node or point).

The weight gradient of such a map, x^T @ g, reduces over the rows.  As one GEMM that reduction
lands on the few workgroups the small output has tiles for (117 us for 32,768 rows, 64 x 64; 4.6 ms
for 2.4 M rows, 100 x 272); cut into chunks of rows it is a batched matmul over all of them plus a
small sum (26 us and 1.5 ms)."""
from __future__ import annotations

import torch


def reduce_over_rows(x, g):
    """x^T @ g for tall x [N, a], g [N, b]."""
    n = x.shape[0]
    chunks = min(256, n // 2048)
    if chunks < 2:
        return torch.matmul(x.t(), g)
    rows = n // chunks
    body = chunks * rows
    out = torch.bmm(x[:body].view(chunks, rows, -1).transpose(1, 2), g[:body].view(chunks, rows, -1)).sum(0)
    if body < n:
        out = out + torch.matmul(x[body:].t(), g[body:])
    return out


def column_sum(g):
    """g.sum(0) for tall g [N, c].  torch's reduction over the rows falls off a cliff when c is not a
    multiple of 4 (19 ms for 2.4 M x 47, 1.2 ms for 233 k x 41, against 40 us and 14 us for 16
    columns): the rows are cut into chunks that are summed side by side, then the chunk sums are added
    (0.15 ms and 0.04 ms).  Narrow, aligned, moderately sized inputs keep the single reduction."""
    n, c = g.shape
    chunks = min(256, n // 2048)
    if chunks < 2 or (c % 4 == 0 and n * c < (1 << 25)):
        return g.sum(0)
    rows = n // chunks
    body = chunks * rows
    out = g[:body].view(chunks, rows, c).sum(1).sum(0)
    return out + g[body:].sum(0) if body < n else out


class _AddBias(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bias):
        return x + bias

    @staticmethod
    def backward(ctx, g):
        return g, (column_sum(g.contiguous()) if ctx.needs_input_grad[1] else None)


def add_bias(x, bias):
    """x + bias for x [N, c], bias [c]; the bias gradient is taken by `column_sum`."""
    return _AddBias.apply(x, bias)


class _TallLinear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        y = torch.matmul(x, weight.t())
        return y if bias is None else y.add_(bias)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        g = g.contiguous()
        gx = torch.matmul(g, weight) if ctx.needs_input_grad[0] else None
        gw = reduce_over_rows(g, x) if ctx.needs_input_grad[1] else None
        gb = column_sum(g) if (ctx.has_bias and ctx.needs_input_grad[2]) else None
        return gx, gw, gb


def tall_linear(x, weight, bias=None):
    """torch.nn.functional.linear for x [N, in] with N large; same values, the weight gradient
    is reduced over the rows in chunks."""
    return _TallLinear.apply(x.contiguous(), weight, bias)
