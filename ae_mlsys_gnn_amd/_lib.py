"""ctypes binding of libfgnn_hip.so (the C ABI declared in include/fgnn.h).

There is no CPU fallback: every operator of this package runs the HIP kernels or raises."""
from __future__ import annotations

import collections
import ctypes
import functools
import os
import threading
from ctypes import c_float, c_int, c_int64, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfgnn_hip.so")

_lib = None


class FgnnError(RuntimeError):
    pass


_SIGNATURES = {
    "fgnn_version": (c_int, []),
    "fgnn_last_error": (ctypes.c_char_p, []),
    "fgnn_schedule_create": (c_int, [c_void_p, c_int, c_int, c_void_p, ctypes.POINTER(c_void_p)]),
    "fgnn_schedule_create_bucketed": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, ctypes.POINTER(c_void_p)]),
    "fgnn_schedule_take_positions": (c_int, [c_void_p, c_void_p, c_void_p]),
    "fgnn_schedule_destroy": (None, [c_void_p]),
    "fgnn_schedule_num_items": (c_int, [c_void_p]),
    "fgnn_schedule_num_buckets": (c_int, [c_void_p]),
    "fgnn_xcd_mapping_for": (c_int, [ctypes.c_char_p, c_int]),
    "fgnn_schedule_num_partials": (c_int, [c_void_p]),
    "fgnn_schedule_num_edges": (c_int64, [c_void_p]),
    "fgnn_schedule_device_bytes": (c_size_t, [c_void_p]),
    "fgnn_schedule_num_splits": (c_int, [c_void_p]),
    "fgnn_schedule_num_wave_slots": (c_int, [c_void_p]),
    "fgnn_schedule_export": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "fgnn_validate_graph": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int64, c_void_p]),
    "fgnn_row_length_stats": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "fgnn_gat_forward_workspace_bytes": (c_size_t, [c_void_p, c_int, c_int]),
    "fgnn_gat_forward": (c_int, [c_int, c_int64, c_int, c_int] + [c_void_p] * 4 + [c_float] + [c_void_p] * 8
                         + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_gat_backward_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_void_p, c_void_p, c_int]),
    "fgnn_gat_backward": (c_int, [c_int, c_int64, c_int, c_int, c_float] + [c_void_p] * 19
                          + [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_gat_backward_own_order": (c_int, [c_int, c_int64, c_int, c_int, c_float] + [c_void_p] * 17
                                    + [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_gat_scatter": (c_int, [c_int, c_int64, c_int] + [c_void_p] * 4 + [c_float] + [c_void_p] * 2 + [c_void_p]),
    "fgnn_gat_gather_row": (c_int, [c_int, c_int64, c_int] + [c_void_p] * 5 + [c_float] + [c_void_p] * 4 + [c_void_p]),
    "fgnn_gat_stash_own_order": (c_int, [c_int, c_int64, c_int, c_float] + [c_void_p] * 7 + [c_void_p, c_void_p]),
    "fgnn_edgeconv_forward": (c_int, [c_int, c_int, c_int, c_int] + [c_void_p] * 5 + [c_void_p]),
    "fgnn_edgeconv_backward": (c_int, [c_int, c_int, c_int] + [c_void_p] * 3 + [c_void_p]),
    "fgnn_edgeconv_forward_lrelu": (c_int, [c_int, c_int, c_int, c_int] + [c_void_p] * 3 + [c_float] + [c_void_p] * 2 + [c_void_p]),
    "fgnn_edgeconv_backward_lrelu": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float] + [c_void_p] * 3
                                     + [c_void_p, c_size_t, c_void_p]),
    "fgnn_edgeconv_backward_blocked_workspace_bytes": (c_size_t, [c_int, c_int]),
    "fgnn_edgeconv_backward_blocked": (c_int, [c_int, c_int, c_int, c_int] + [c_void_p] * 4 + [c_size_t, c_void_p]),
    "fgnn_edgeconv_backward_blocked_static_max_elems": (c_size_t, []),
    "fgnn_edgeconv_backward_blocked_static": (c_int, [c_int, c_int, c_int, c_int] + [c_void_p] * 3 + [c_void_p]),
    "fgnn_knn_graph": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "fgnn_gmm_forward_workspace_bytes": (c_size_t, [c_void_p, c_int, c_int]),
    "fgnn_gmm_forward": (c_int, [c_int, c_int64, c_int, c_int, c_int] + [c_void_p] * 9 + [c_int]
                         + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_gmm_forward_epilogue": (c_int, [c_int, c_int64, c_int, c_int, c_int] + [c_void_p] * 11 + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_gmm_backward_workspace_bytes": (c_size_t, [c_void_p, c_int, c_int, c_int]),
    "fgnn_gmm_backward": (c_int, [c_int, c_int64, c_int, c_int, c_int] + [c_void_p] * 8 + [c_int] + [c_void_p] * 4
                          + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_gaussian": (c_int, [c_int64, c_int, c_int] + [c_void_p] * 4 + [c_void_p]),
    "fgnn_gaussian_backward_workspace_bytes": (c_size_t, [c_int64, c_int, c_int]),
    "fgnn_gaussian_backward": (c_int, [c_int64, c_int, c_int] + [c_void_p] * 7 + [c_void_p, c_size_t, c_void_p]),
    "fgnn_mhspmm_workspace_bytes": (c_size_t, [c_void_p, c_int, c_int]),
    "fgnn_mhspmm": (c_int, [c_int, c_int64, c_int, c_int] + [c_void_p] * 6 + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_mhsddmm": (c_int, [c_int, c_int64, c_int, c_int] + [c_void_p] * 5 + [c_void_p]),
    "fgnn_mhsddmm_scheduled": (c_int, [c_int, c_int64, c_int, c_int] + [c_void_p] * 5 + [c_void_p, c_void_p]),
    "fgnn_sddmm_coo": (c_int, [c_int64, c_int, c_int, c_int, c_int] + [c_void_p] * 5 + [c_void_p]),
    "fgnn_gather_rows": (c_int, [c_int64, c_int] + [c_void_p] * 3 + [c_void_p]),
    "fgnn_edge_softmax": (c_int, [c_int, c_int64, c_int] + [c_void_p] * 3 + [c_void_p]),
    "fgnn_edge_softmax_backward": (c_int, [c_int, c_int64, c_int] + [c_void_p] * 4 + [c_void_p]),
    "fgnn_u_add_v": (c_int, [c_int, c_int64, c_int] + [c_void_p] * 5 + [c_void_p]),
    "fgnn_u_add_v_backward": (c_int, [c_int, c_int64, c_int] + [c_void_p] * 5 + [c_void_p]),
    "fgnn_colsum_plan_create": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_int, c_int, c_void_p, ctypes.POINTER(c_void_p)]),
    "fgnn_colsum_plan_destroy": (None, [c_void_p]),
    "fgnn_colsum_plan_device_bytes": (c_size_t, [c_void_p]),
    "fgnn_colsum_plan_columns_per_range": (c_int, [c_void_p]),
    "fgnn_colsum_plan_num_tasks": (c_int, [c_void_p]),
    "fgnn_colsum_plan_matches": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64]),
    "fgnn_colsum_workspace_bytes": (c_size_t, [c_void_p, c_int]),
    "fgnn_edge_colsum": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_edge_rowsum": (c_int, [c_int, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "fgnn_u_add_v_backward_planned": (c_int, [c_int, c_int64, c_int] + [c_void_p] * 5 + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "fgnn_edge_linear_tanh": (c_int, [c_int64, c_int] + [c_void_p] * 4 + [c_void_p]),
    "fgnn_edge_linear_tanh_backward_workspace_bytes": (c_size_t, [c_int64, c_int]),
    "fgnn_edge_linear_tanh_backward": (c_int, [c_int64, c_int] + [c_void_p] * 5 + [c_void_p, c_size_t, c_void_p]),
    "fgnn_cross_entropy_forward": (c_int, [c_int64, c_int, c_int64] + [c_void_p] * 4 + [c_void_p]),
    "fgnn_cross_entropy_backward": (c_int, [c_int64, c_int, c_int64, c_int64] + [c_void_p] * 5 + [c_void_p]),
    "fgnn_coo2csr_workspace_bytes": (c_size_t, [c_int, c_int, c_int64]),
    "fgnn_coo2csr": (c_int, [c_int, c_int, c_int64, c_void_p, c_void_p, c_int] + [c_void_p] * 4 + [c_void_p, c_size_t, c_void_p]),
    "fgnn_csr2csc_workspace_bytes": (c_size_t, [c_int, c_int, c_int64]),
    "fgnn_csr2csc": (c_int, [c_int, c_int, c_int64] + [c_void_p] * 5 + [c_void_p, c_size_t, c_void_p]),
}


def exported_symbols():
    """Names the C ABI must export (kept in step with include/fgnn.h)."""
    return sorted(_SIGNATURES)


def lib():
    """The loaded library; raises when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FgnnError(
                "libfgnn_hip.so is missing at %s; build it with "
                "`python -m ae_mlsys_gnn_amd.build` (needs hipcc)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = lib().fgnn_last_error().decode("utf-8", "replace")
        raise FgnnError("%s failed (code %d): %s" % (what, rc, msg))


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    if t is None:
        return None
    return c_void_p(t.data_ptr())


def stream_ptr():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise FgnnError("fgnn operators run on the GPU only (got a %s tensor); there is no CPU path" % t.device)


def as_f32(t):
    if t.dtype != torch.float32:
        raise FgnnError("expected float32, got %s" % t.dtype)
    return t.contiguous()


def as_i32(t):
    if t.dtype != torch.int32:
        raise FgnnError("expected int32 indices, got %s" % t.dtype)
    return t.contiguous()


class Schedule:
    """Degree-binned work list of one pointer array (row_ptr or col_ptr).  With `idx_tensor` it is
    the XCD-aware form: long rows are cut by source bucket and each XCD gets one bucket."""

    def __init__(self, ptr_tensor, seg_len=0, idx_tensor=None, min_deg=0, with_positions=True, n_cols=None):
        require_cuda(ptr_tensor)
        self.ptr_tensor = as_i32(ptr_tensor)      # keeps the device memory alive
        self.idx_tensor = None if idx_tensor is None else as_i32(idx_tensor)
        self.n_rows = self.ptr_tensor.numel() - 1
        handle = c_void_p()
        with torch.cuda.device(self.ptr_tensor.device):
            if self.idx_tensor is not None and os.environ.get("FGNN_VALIDATE", "0") not in ("0", ""):
                # opt-in: range-check the graph once, when its work list is built, before any gather kernel runs.  The ids
                # index another array than the pointer array's rows (mhspmm / csrspmm: the gathered matrix), so the bound is
                # the caller's n_cols; without one only the pointer array and the sign of the ids can be checked
                bound = int(n_cols) if n_cols is not None else 2147483647
                check(lib().fgnn_validate_graph(ptr(self.ptr_tensor), ptr(self.idx_tensor), self.n_rows, bound,
                                                self.idx_tensor.numel(), stream_ptr()), "fgnn_validate_graph")
            if self.idx_tensor is None:
                check(lib().fgnn_schedule_create(ptr(self.ptr_tensor), self.n_rows, int(seg_len), stream_ptr(),
                                                 ctypes.byref(handle)), "fgnn_schedule_create")
            else:
                check(lib().fgnn_schedule_create_bucketed(ptr(self.ptr_tensor), ptr(self.idx_tensor), self.n_rows, int(seg_len),
                                                          int(min_deg), int(bool(with_positions)), stream_ptr(), ctypes.byref(handle)),
                      "fgnn_schedule_create_bucketed")
        self.handle = handle
        self.n_items = lib().fgnn_schedule_num_items(handle)
        self.n_buckets = lib().fgnn_schedule_num_buckets(handle)     # 0: plain list (also when the device lacks the XCD mapping)
        self.n_partials = lib().fgnn_schedule_num_partials(handle)
        self.n_wave_slots = lib().fgnn_schedule_num_wave_slots(handle)   # items from this slot on have at most 64 entries
        self.n_edges = lib().fgnn_schedule_num_edges(handle)
        self.own_order = False

    def export(self):
        """(items int32 [n_items, 4], splits int32 [n_split, 4]) on the device: the work list itself."""
        dev = self.ptr_tensor.device
        n_split = lib().fgnn_schedule_num_splits(self.handle)
        items = torch.empty((self.n_items, 4), dtype=torch.int32, device=dev)
        splits = torch.empty((n_split, 4), dtype=torch.int32, device=dev)
        with torch.cuda.device(dev):
            check(lib().fgnn_schedule_export(self.handle, ptr(items), ptr(splits), stream_ptr()), "fgnn_schedule_export")
        return items, splits

    def device_bytes(self):
        """Device memory the schedule holds outside torch's allocator."""
        return int(lib().fgnn_schedule_device_bytes(self.handle))

    def take_positions(self):
        """int32 [E]: caller's edge position of every entry in the schedule's own order.  The schedule gives
        up its copy; operators called with it afterwards take per-edge tensors in that order."""
        out = torch.empty(self.n_edges, dtype=torch.int32, device=self.ptr_tensor.device)
        with torch.cuda.device(self.ptr_tensor.device):
            check(lib().fgnn_schedule_take_positions(self.handle, ptr(out), stream_ptr()), "fgnn_schedule_take_positions")
        self.own_order = True
        return out

    def __del__(self):
        h = getattr(self, "handle", None)
        if h is not None and _lib is not None:
            _lib.fgnn_schedule_destroy(h)
            self.handle = None


_sched_cache: "collections.OrderedDict" = collections.OrderedDict()
_SCHED_CACHE_MAX = 32
# The caches below are read and filled by the thread that runs the forward pass and by autograd's backward
# thread: one re-entrant lock serialises every look-up-then-insert sequence (and the builds inside them).
_cache_lock = threading.RLock()


def _locked(fn):
    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        with _cache_lock:
            return fn(*args, **kwargs)
    return wrapper


def default_seg_len() -> int:
    return int(os.environ.get("FGNN_SEG_LEN", "0"))


_bucket_rule_cache: "collections.OrderedDict" = collections.OrderedDict()
BUCKET_ROW_LEN = 64          # rows longer than this are the ones an XCD-aware schedule cuts by source bucket
BUCKET_MIN_SHARE = 0.25      # ...and they must hold at least this share of the entries
BUCKET_MIN_SKEW = 4          # longest row / mean row length


@_locked
def xcd_buckets_enabled(ptr_tensor, idx_numel=None) -> bool:
    """Whether operators get the XCD-aware schedule for this pointer array (FGNN_XCD_BUCKETS=0/1
    overrides).  It pays off on skewed graphs, where the rows longer than 64 entries hold a good part
    of the work: cutting them by source bucket keeps each XCD's L2 on one eighth of the gathered rows
    and shortens the longest work item.  It costs time on graphs without hubs (every row of a
    uniform degree-100 graph would become eight short segments with nothing to reuse between them),
    so the rule asks for both: rows longer than 64 hold a quarter of the entries, and the longest row
    is at least 4x the mean.  The two numbers come from one reduction kernel, once per array, and are cached.
    idx_numel: the number of entries when the caller has it (saves reading ptr[-1] back)."""
    env = os.environ.get("FGNN_XCD_BUCKETS")
    if env is not None:
        return env not in ("0", "")
    n_rows = ptr_tensor.numel() - 1
    if n_rows <= 0:
        return False
    key = (ptr_tensor.data_ptr(), ptr_tensor.numel(), ptr_tensor.device.index, ptr_tensor._version)
    hit = _bucket_rule_cache.get(key)
    if hit is None:
        stats = (ctypes.c_int64 * 2)()
        with torch.cuda.device(ptr_tensor.device):
            check(lib().fgnn_row_length_stats(ptr(ptr_tensor), n_rows, BUCKET_ROW_LEN, ctypes.cast(stats, c_void_p), stream_ptr()),
                  "fgnn_row_length_stats")
        n_long, longest = int(stats[0]), int(stats[1])
        n_edges = int(idx_numel) if idx_numel is not None else int(ptr_tensor[-1])
        hit = (n_edges > 0 and n_long >= BUCKET_MIN_SHARE * n_edges and longest * n_rows >= BUCKET_MIN_SKEW * n_edges,
               ptr_tensor)         # the entry holds the tensor: its address cannot be reused while the entry lives
        _bucket_rule_cache[key] = hit
        while len(_bucket_rule_cache) > 4 * _SCHED_CACHE_MAX:
            _bucket_rule_cache.popitem(last=False)
    return hit[0]


@_locked
def schedule_for(ptr_tensor, seg_len=None, idx_tensor=None, need_positions=True, own_order=False, n_cols=None) -> Schedule:
    """Cached schedule of a pointer array.  The cache entry holds the tensors, so their device
    addresses cannot be reused while the entry lives; in-place edits bump `_version`.
    idx_tensor: the index array, for operators that may use an XCD-aware schedule.
    need_positions: whether the operator has per-edge tensors (an XCD-aware schedule then also keeps
    the caller's position of every entry, 4*E bytes more); a schedule with positions serves both.
    n_cols: rows of the array the ids index, for the opt-in FGNN_VALIDATE check (None: only ids >= 0 is checked).
    own_order: a schedule of its own (never shared with the other kinds) whose position map was taken
    out (`edge_positions`): operators called with it take per-edge tensors in the schedule's order."""
    if seg_len is None:
        seg_len = default_seg_len()
    if idx_tensor is not None and not xcd_buckets_enabled(ptr_tensor, idx_tensor.numel()):
        idx_tensor = None
    min_deg = int(os.environ.get("FGNN_BUCKET_MIN_DEG", "0"))

    def key(pos):
        return (ptr_tensor.data_ptr(), ptr_tensor.numel(), ptr_tensor.device.index, ptr_tensor._version, int(seg_len),
                None if idx_tensor is None else (idx_tensor.data_ptr(), idx_tensor._version, min_deg, pos))
    if own_order:
        k = key("own")
        s = _sched_cache.get(k)
        if s is None:
            raise FgnnError("no own-order schedule for these arrays: call edge_positions(ptr, idx) first and pass per-edge "
                            "tensors permuted by its result")
        _sched_cache.move_to_end(k)
        return s
    k = key(True)
    s = _sched_cache.get(k)
    if s is None and not need_positions and idx_tensor is not None:
        k = key(False)
        s = _sched_cache.get(k)
    if s is None:
        s = Schedule(ptr_tensor, seg_len, idx_tensor, min_deg, with_positions=need_positions, n_cols=n_cols)
        _sched_cache[k] = s
        while len(_sched_cache) > _SCHED_CACHE_MAX:
            _sched_cache.popitem(last=False)
    else:
        _sched_cache.move_to_end(k)
    return s


@_locked
def edge_positions(ptr_tensor, idx_tensor, seg_len=None):
    """Builds (once) the own-order schedule of (ptr, idx) and returns int32 [E]: the caller's position of
    every entry in that schedule's order, or None when the order is the caller's (plain schedule).
    Per-edge tensors passed to operators with own_order=True must be t[edge_positions]."""
    if seg_len is None:
        seg_len = default_seg_len()
    bucketed = xcd_buckets_enabled(ptr_tensor)
    min_deg = int(os.environ.get("FGNN_BUCKET_MIN_DEG", "0"))
    k = (ptr_tensor.data_ptr(), ptr_tensor.numel(), ptr_tensor.device.index, ptr_tensor._version, int(seg_len),
         (idx_tensor.data_ptr(), idx_tensor._version, min_deg, "own") if bucketed else None)
    if not bucketed:
        schedule_for(ptr_tensor, seg_len)          # the plain schedule serves both orders
        return None
    s = Schedule(ptr_tensor, seg_len, idx_tensor, min_deg, with_positions=True)
    pos = s.take_positions()
    if k in _sched_cache:                   # asked again: the map is a function of the arrays, the cached schedule stays
        _sched_cache.move_to_end(k)
        return pos
    _sched_cache[k] = s
    while len(_sched_cache) > _SCHED_CACHE_MAX:
        _sched_cache.popitem(last=False)
    return pos


class ColsumPlan:
    """Tile-ordered entry list of one (row_ptr, col_ind) pair for atomic-free column sums of per-edge arrays
    (fgnn_colsum_plan_create).  Built for rows of `width` floats; serves every narrower array."""

    def __init__(self, ptr_tensor, idx_tensor, n_cols, width, lds_bytes=0, task_len=0):
        require_cuda(ptr_tensor, idx_tensor)
        self.ptr_tensor = as_i32(ptr_tensor)      # keep the device memory alive
        self.idx_tensor = as_i32(idx_tensor)
        self.n_rows = self.ptr_tensor.numel() - 1
        self.n_cols = int(n_cols)
        self.width = int(width)
        handle = c_void_p()
        with torch.cuda.device(self.ptr_tensor.device):
            check(lib().fgnn_colsum_plan_create(ptr(self.ptr_tensor), ptr(self.idx_tensor), self.n_rows, self.n_cols, self.idx_tensor.numel(),
                                                self.width, int(lds_bytes), int(task_len), stream_ptr(), ctypes.byref(handle)),
                  "fgnn_colsum_plan_create")
        self.handle = handle
        self.columns_per_range = lib().fgnn_colsum_plan_columns_per_range(handle)
        self.n_tasks = lib().fgnn_colsum_plan_num_tasks(handle)

    def device_bytes(self):
        return int(lib().fgnn_colsum_plan_device_bytes(self.handle))

    def colsum(self, g):
        """[n_cols, ...] column sums of the per-edge array g [E, ...] (CSR position order)."""
        require_cuda(g)
        g = as_f32(g)
        e = self.idx_tensor.numel()
        if g.shape[0] != e:
            raise FgnnError("colsum: the array has %d rows, the plan %d entries" % (g.shape[0], e))
        w = g.numel() // max(e, 1) if e else int(torch.tensor(g.shape[1:]).prod()) if g.dim() > 1 else 1
        out = torch.empty((self.n_cols,) + tuple(g.shape[1:]), dtype=torch.float32, device=g.device)
        with torch.cuda.device(g.device):
            ws, wsb = workspace(lib().fgnn_colsum_workspace_bytes(self.handle, w), g.device)
            check(lib().fgnn_edge_colsum(self.handle, w, ptr(g), ptr(out), ptr(ws), wsb, stream_ptr()), "fgnn_edge_colsum")
        return out

    def __del__(self):
        h = getattr(self, "handle", None)
        if h is not None and _lib is not None:
            _lib.fgnn_colsum_plan_destroy(h)
            self.handle = None


_colsum_cache: "collections.OrderedDict" = collections.OrderedDict()
_COLSUM_CACHE_MAX = 8


def colsum_plan_for(ptr_tensor, idx_tensor, n_cols, width) -> ColsumPlan:
    """Cached plan of (row_ptr, col_ind); a cached plan built for wider rows is reused.  The entry holds the
    tensors, so their addresses cannot be reused while it lives; in-place edits bump `_version`."""
    key = (ptr_tensor.data_ptr(), ptr_tensor.numel(), ptr_tensor._version, idx_tensor.data_ptr(), idx_tensor.numel(), idx_tensor._version,
           ptr_tensor.device.index, int(n_cols))
    with _cache_lock:
        p = _colsum_cache.get(key)
        if p is None or p.width < width:
            p = ColsumPlan(ptr_tensor, idx_tensor, n_cols, width)
            _colsum_cache[key] = p
        _colsum_cache.move_to_end(key)
        while len(_colsum_cache) > _COLSUM_CACHE_MAX:
            _colsum_cache.popitem(last=False)
        return p


def schedule_device_bytes() -> int:
    """Device memory held by all cached schedules and column-sum plans: the library allocates it itself, so
    torch's max_memory_allocated does not see it and peak-memory reports add it."""
    with _cache_lock:
        return sum(s.device_bytes() for s in _sched_cache.values()) + sum(p.device_bytes() for p in _colsum_cache.values())


_own_view_cache: "collections.OrderedDict" = collections.OrderedDict()
_OWN_VIEW_CACHE_MAX = 4


def _gather_i32(src, index):
    """src[index] for int32 device vectors, by the library's row-gather kernel (the words move as they are)."""
    out = torch.empty_like(index)
    if index.numel():
        with torch.cuda.device(src.device):
            check(lib().fgnn_gather_rows(index.numel(), 1, ptr(index), ptr(src), ptr(out), stream_ptr()), "fgnn_gather_rows")
    return out


def own_order_view(row_ptr, col_ind, col_ptr, row_ind, permute):
    """(col_ind_own, permute_own) for pipelines that keep their per-edge tensors in the ENTRY ORDER of the work lists:
    col_ind_own is col_ind in the order the CSR-side list walks the entries (an XCD-aware list regroups the entries of a row
    by source bucket, so (row_ptr, col_ind_own) is a CSR of the same graph), and permute_own[q] is the position in that
    order of the entry that the CSC-side list walks q-th.  Operators called with own_order=True then read and write [E,H]
    tensors as contiguous runs; with plain lists on both sides the caller's arrays come back.  Built once per set of
    arrays and cached with the two own-order schedules (the cache holds the tensors)."""
    key = tuple((t.data_ptr(), t.numel(), t._version) for t in (row_ptr, col_ind, col_ptr, row_ind, permute)) + (
        row_ptr.device.index, default_seg_len(), os.environ.get("FGNN_BUCKET_MIN_DEG", "0"), os.environ.get("FGNN_XCD_BUCKETS"))
    with _cache_lock:
        hit = _own_view_cache.get(key)
        if hit is not None:
            _own_view_cache.move_to_end(key)
            return hit[0], hit[1]
    pos_r = edge_positions(row_ptr, col_ind)
    pos_c = edge_positions(col_ptr, row_ind)
    perm = permute if pos_c is None else _gather_i32(permute, pos_c)
    if pos_r is None:
        idx_own, perm_own = col_ind, perm
    else:
        idx_own = _gather_i32(col_ind, pos_r)
        e = pos_r.numel()
        iota = torch.arange(e, dtype=torch.int32, device=pos_r.device)
        inv = torch.empty_like(pos_r)
        inv.scatter_(0, pos_r.long(), iota)
        if not torch.equal(_gather_i32(inv, pos_r), iota):
            raise FgnnError("own_order_view: the position map of the work list is not a permutation")
        perm_own = _gather_i32(inv, perm)
        del inv, iota
    with _cache_lock:
        _own_view_cache[key] = (idx_own, perm_own, (row_ptr, col_ind, col_ptr, row_ind, permute))
        while len(_own_view_cache) > _OWN_VIEW_CACHE_MAX:
            _own_view_cache.popitem(last=False)
    return idx_own, perm_own


def clear_schedule_cache():
    with _cache_lock:
        _sched_cache.clear()
        _bucket_rule_cache.clear()
        _colsum_cache.clear()
        _own_view_cache.clear()


def workspace(nbytes: int, device):
    """A float-aligned scratch tensor of at least nbytes (None when nothing is needed)."""
    if nbytes <= 0:
        return None, 0
    t = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)
    return t, t.numel() * 4
