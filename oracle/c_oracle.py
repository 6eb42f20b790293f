"""ctypes loader for the plain-C oracle (oracle/fgnn_oracle.c).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libfgnn_oracle.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "fgnn_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i32(a):
    return np.ascontiguousarray(np.asarray(a), dtype=np.int32)


def _f64(a):
    return np.ascontiguousarray(np.asarray(a), dtype=np.float64)


def gat_forward(row_ptr, col_ind, attn_row, attn_col, slope, in_feat):
    rp, ci = _i32(row_ptr), _i32(col_ind)
    ar, ac, x = _f64(attn_row), _f64(attn_col), _f64(in_feat)
    n, h, f = x.shape
    out = np.empty_like(x)
    mx = np.empty((n, h)); sm = np.empty((n, h))
    lib().fgo_gat_forward(n, h, f, _p(rp), _p(ci), _p(ar), _p(ac), ctypes.c_double(slope), _p(x), _p(out), _p(mx), _p(sm))
    return out, mx, sm


def gat_backward(row_ptr, col_ind, attn_row, attn_col, slope, in_feat, grad_out):
    rp, ci = _i32(row_ptr), _i32(col_ind)
    ar, ac, x, g = _f64(attn_row), _f64(attn_col), _f64(in_feat), _f64(grad_out)
    n, h, f = x.shape
    gx = np.empty_like(x); gar = np.empty((n, h)); gac = np.empty((n, h))
    lib().fgo_gat_backward(n, h, f, _p(rp), _p(ci), _p(ar), _p(ac), ctypes.c_double(slope), _p(x), _p(g), _p(gx), _p(gar), _p(gac))
    return gx, gar, gac


def edgeconv_forward(k, src_ind, h_src, h_dst):
    si = _i32(src_ind)
    hs = np.ascontiguousarray(h_src, dtype=np.float32); hd = np.ascontiguousarray(h_dst, dtype=np.float32)
    n, f = hd.shape
    out = np.empty((n, f), np.float32); arg = np.empty((n, f), np.int32)
    lib().fgo_edgeconv_forward(n, f, k, _p(si), _p(hs), _p(hd), _p(out), _p(arg))
    return out, arg


def edgeconv_backward(argmax, grad_out, n_src):
    am = _i32(argmax); g = _f64(grad_out)
    n, f = g.shape
    gs = np.empty((n_src, f))
    lib().fgo_edgeconv_backward(n, n_src, f, _p(am), _p(g), _p(gs))
    return gs


def gmm_forward(row_ptr, col_ind, node_feat, pseudo, mu, inv_sigma):
    rp, ci = _i32(row_ptr), _i32(col_ind)
    x, ps, m, sg = _f64(node_feat), _f64(pseudo), _f64(mu), _f64(inv_sigma)
    n, kk, f = x.shape
    out = np.empty_like(x)
    lib().fgo_gmm_forward(n, kk, ps.shape[1], f, _p(rp), _p(ci), _p(x), _p(ps), _p(m), _p(sg), _p(out))
    return out


def gmm_backward(row_ptr, col_ind, node_feat, pseudo, mu, inv_sigma, grad_out):
    rp, ci = _i32(row_ptr), _i32(col_ind)
    x, ps, m, sg, g = _f64(node_feat), _f64(pseudo), _f64(mu), _f64(inv_sigma), _f64(grad_out)
    n, kk, f = x.shape
    gx = np.empty_like(x); gp = np.empty_like(ps); gm = np.empty_like(m); gs = np.empty_like(sg)
    lib().fgo_gmm_backward(n, kk, ps.shape[1], f, _p(rp), _p(ci), _p(x), _p(ps), _p(m), _p(sg), _p(g), _p(gx), _p(gp), _p(gm), _p(gs))
    return gx, gp, gm, gs


def csr2csc(row_ptr, col_ind, n_cols=None):
    rp, ci = _i32(row_ptr), _i32(col_ind)
    n = rp.shape[0] - 1
    nc = n if n_cols is None else n_cols
    cp = np.empty(nc + 1, np.int32); ri = np.empty(ci.shape[0], np.int32); pm = np.empty(ci.shape[0], np.int32)
    lib().fgo_csr2csc(n, nc, _p(rp), _p(ci), _p(cp), _p(ri), _p(pm))
    return cp, ri, pm
