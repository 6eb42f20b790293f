"""Shared helpers of the test suite: seeded inputs and the parity bar."""
import numpy as np
import torch

from ae_mlsys_gnn_amd import graphs

# fp32 parity bar of the fused operators against the float64 oracle
RTOL = 1e-4
ATOL = 1e-5


def assert_close(got, ref, what, rtol=RTOL, atol=ATOL):
    got = got.detach().cpu().double()
    ref = ref.detach().cpu().double()
    assert got.shape == ref.shape, "%s: shape %s vs %s" % (what, tuple(got.shape), tuple(ref.shape))
    err = (got - ref).abs()
    tol = atol + rtol * ref.abs()
    bad = err > tol
    if bad.any():
        i = int(torch.argmax(err - tol))
        raise AssertionError("%s: %d/%d outside rtol=%g atol=%g; worst |err|=%.3e at flat %d (got %.7g ref %.7g)" % (
            what, int(bad.sum()), bad.numel(), rtol, atol, float(err.flatten()[i]), i,
            float(got.flatten()[i]), float(ref.flatten()[i])))


# Outputs that are sums of terms of either sign (the score / parameter gradients: up to E summands that
# largely cancel) cannot be held to a bar relative to the RESULT: fp32 rounding scales with the sum of
# the absolute summands S.  Their bar is  rtol*|ref| + max(atol, C_SUM * 2^-24 * S)  with S from the
# oracle (gat_abs_sums / gmm_abs_sums: elementary products of the inputs, no cancellation inside).
# C_SUM stands for the roundings a summand carries at unit roundoff 2^-24 apart from its exponent (exp2, the
# 1/sum normalisation, the weight product, the dot product feeding it, the accumulation).  A weight
# exp(v) inherits the ABSOLUTE rounding of v as a relative error, so operators with an exponential add
# a quarter of that per unit of max|v| (c_exp).  The constant is set from measurement, not from a worst-case
# count: every comparison records how much of its allowance it used (PARITY_LOG below); with C_SUM = 2.5 the
# largest share over the whole suite is 0.39 (a stored-weight SpMM over rows of 1024+ floats) and 0.36 at the
# benchmark sizes (grad_attn_col of the 1 x 47 output layer on the 64 M-edge graph), and the full-size tests assert
# that no element uses more than half (MAX_RATIO).  With the constants of a worst-case count (16, and 4 per unit)
# no element used more than a tenth of its allowance.  Not tuned per test.
EPS32 = 2.0 ** -24
C_SUM = 2.5
MAX_RATIO = 0.5


def c_exp(max_abs_exponent):
    return C_SUM * (1.0 + 0.25 * float(max_abs_exponent))


# Every assert_close_sum call leaves a record here: how much of the derived allowance the comparison needed.
# conftest.py writes the list to a JSON file at the end of a session when FGNN_PARITY_LOG names one.
PARITY_LOG = []


def assert_close_sum(got, ref, s_abs, what, rtol=RTOL, atol=ATOL, c=C_SUM, extra=None, where="cpu", max_ratio=None):
    """extra: an additional absolute allowance per element (e.g. what a LeakyReLU' jump at a pre-activation of
    zero can change), zero wherever it does not apply.  where: the device the comparison runs on (arrays of
    10^9 elements stay on the GPU).
    Returns (and logs) how much of the allowance was used: `frac_beyond_plain` = the share of elements whose
    error exceeds the plain bar rtol*|ref| + atol, `worst_ratio` = max over those elements of
    err / (c * 2^-24 * S) (0 when there are none).  max_ratio: an upper limit asserted on worst_ratio, so a
    constant c with an order of magnitude to spare cannot hide a loss of accuracy."""
    got = got.detach().to(where).double()
    ref = ref.detach().to(where).double()
    s_abs = torch.as_tensor(s_abs).detach().to(where).double()
    assert got.shape == ref.shape, "%s: shape %s vs %s" % (what, tuple(got.shape), tuple(ref.shape))
    s_abs = s_abs.expand_as(ref)
    err = (got - ref).abs()
    allow = c * EPS32 * s_abs
    tol = rtol * ref.abs() + torch.clamp(allow, min=atol)
    ex = None
    if extra is not None:
        ex = torch.as_tensor(extra).detach().to(where).double().expand_as(ref)
        tol = tol + ex
    bad = err > tol
    if bad.any():
        i = int(torch.argmax(err - tol))
        raise AssertionError("%s: %d/%d outside rtol=%g + max(%g, %g*2^-24*S); worst |err|=%.3e at flat %d (got %.7g ref %.7g S %.4g)" % (
            what, int(bad.sum()), bad.numel(), rtol, atol, c, float(err.flatten()[i]), i,
            float(got.flatten()[i]), float(ref.flatten()[i]), float(s_abs.flatten()[i])))
    beyond = err > rtol * ref.abs() + atol
    if ex is not None:
        beyond &= ex == 0                      # elements under the explicit jump allowance are not rounding cases
    n_beyond = int(beyond.sum())
    worst = float((err[beyond] / allow[beyond]).max()) if n_beyond else 0.0
    rec = {"what": what, "elements": int(ref.numel()), "beyond_plain": n_beyond, "frac_beyond_plain": n_beyond / max(1, ref.numel()),
           "worst_ratio": worst, "c": float(c)}
    PARITY_LOG.append(rec)
    if n_beyond:
        print("[parity] %s: %d of %d elements (%.3g) beyond rtol=%g atol=%g; worst err / (c 2^-24 S) = %.3f (c = %.1f)" % (
            what, n_beyond, ref.numel(), rec["frac_beyond_plain"], rtol, atol, worst, c), flush=True)
    if max_ratio is not None:
        assert worst <= max_ratio, "%s: an element used %.3f of the derived allowance (limit %.2f)" % (what, worst, max_ratio)
    return rec


def gat_inputs(g, h, f, seed=0, attn_scale=1.0, dtype=torch.float64):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(g.n, h, f, generator=gen, dtype=dtype)
    ar = torch.randn(g.n, h, generator=gen, dtype=dtype) * attn_scale
    ac = torch.randn(g.n, h, generator=gen, dtype=dtype) * attn_scale
    go = torch.randn(g.n, h, f, generator=gen, dtype=dtype)
    return x, ar, ac, go


def custom_graph(row_lists, n=None):
    """Graph from per-destination source lists."""
    n = len(row_lists) if n is None else n
    rp = [0]
    ci = []
    for r in row_lists:
        ci.extend(r)
        rp.append(len(ci))
    while len(rp) < n + 1:
        rp.append(len(ci))
    return graphs.Graph(n, torch.tensor(rp, dtype=torch.int32), torch.tensor(ci, dtype=torch.int32))


def degree_edge_graph(n=700, seed=0):
    """Rows with degrees 0, 1, 31..33, 63..65, 511..513 and one hub; sources uniform random."""
    gen = np.random.default_rng(seed)
    degs = [0, 1, 2, 7, 8, 9, 31, 32, 33, 63, 64, 65, 127, 128, 129, 511, 512, 513, 0, 3000]
    rows = []
    for i in range(n):
        d = degs[i] if i < len(degs) else int(gen.integers(0, 12))
        rows.append(list(gen.integers(0, n, size=d)))
    return custom_graph(rows, n)
