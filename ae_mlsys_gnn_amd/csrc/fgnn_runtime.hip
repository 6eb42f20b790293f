// Error reporting, version and row schedules of libfgnn_hip.so.
#include <algorithm>
#include <cstdarg>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>
#include "fgnn_common.h"

static thread_local char g_err[512] = "";

void fgnn_set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char *fgnn_last_error(void) { return g_err; }
extern "C" int fgnn_version(void) { return 100; }

// Per row: stable partition of the row's index entries by source bucket.  One wave per row; pass 1
// counts the buckets (ballots), pass 2 places every entry at its bucket's running offset.  Writes
// the permuted index array, the original position of every entry and the per-(row, bucket) counts.
__global__ __launch_bounds__(FGNN_TPB) void bucket_partition_kernel(int n_rows, const int *__restrict__ ptr, const int *__restrict__ idx,
                                                                    int *__restrict__ bidx, int *__restrict__ bpos, int *__restrict__ bcnt)
{
    int row = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (row >= n_rows) return;
    const int lane = fg_lane();
    const int pb = fg_uni(ptr[row]), pe = fg_uni(ptr[row + 1]);
    int cnt[FGNN_NUM_XCD];
#pragma unroll
    for (int b = 0; b < FGNN_NUM_XCD; ++b) cnt[b] = 0;
    for (int c = pb; c < pe; c += 64) {
        int q = c + lane;
        bool ok = q < pe;
        int bk = ok ? fgnn_bucket_of(idx[q]) : -1;
#pragma unroll
        for (int b = 0; b < FGNN_NUM_XCD; ++b) cnt[b] += __popcll(__builtin_amdgcn_ballot_w64(bk == b));
    }
    int off[FGNN_NUM_XCD];
    int run = pb;
#pragma unroll
    for (int b = 0; b < FGNN_NUM_XCD; ++b) { off[b] = run; run += cnt[b]; }
    if (lane < FGNN_NUM_XCD) {
        int v = 0;
#pragma unroll
        for (int b = 0; b < FGNN_NUM_XCD; ++b) v = (lane == b) ? cnt[b] : v;
        bcnt[(size_t)row * FGNN_NUM_XCD + lane] = v;
    }
    const unsigned long long lt = (1ull << lane) - 1ull;
    for (int c = pb; c < pe; c += 64) {
        int q = c + lane;
        bool ok = q < pe;
        int id = ok ? idx[q] : 0;
        int bk = ok ? fgnn_bucket_of(id) : -1;
        int dst = 0;
#pragma unroll
        for (int b = 0; b < FGNN_NUM_XCD; ++b) {
            unsigned long long m = __builtin_amdgcn_ballot_w64(bk == b);
            if (bk == b) dst = off[b] + __popcll(m & lt);
            off[b] += __popcll(m);
        }
        if (ok) { bidx[dst] = id; if (bpos) bpos[dst] = q; }
    }
}

static void split_range(std::vector<fgnn_item> &out, int row, int b, int e, int seg_len, int &n_part, int &nseg_total)
{
    int len = e - b;
    int nseg = (len + seg_len - 1) / seg_len;
    int step = (((len + nseg - 1) / nseg) + 63) & ~63;
    for (int s = b; s < e; s += step) {
        out.push_back({row, s, std::min(e, s + step), n_part++});
        ++nseg_total;
    }
}

// Stable sort of work items by length, longest first.  Lengths are bounded by the segment length
// (or the row-length cap of whole rows), so a counting sort does it in one pass.
static void sort_longest_first(std::vector<fgnn_item> &v, size_t first = 0)
{
    if (v.size() - first < 2) return;
    int max_len = 0;
    for (size_t i = first; i < v.size(); ++i) max_len = std::max(max_len, v[i].end - v[i].begin);
    std::vector<size_t> start((size_t)max_len + 2, 0);
    for (size_t i = first; i < v.size(); ++i) ++start[(size_t)(max_len - (v[i].end - v[i].begin)) + 1];
    for (size_t l = 1; l < start.size(); ++l) start[l] += start[l - 1];
    std::vector<fgnn_item> sorted(v.size() - first);
    for (size_t i = first; i < v.size(); ++i) sorted[start[(size_t)(max_len - (v[i].end - v[i].begin))]++] = v[i];
    std::copy(sorted.begin(), sorted.end(), v.begin() + first);
}

// k + 1 for the last slot k (counted per source bucket in an XCD-aware list) that holds an item of more than `limit` entries
__global__ __launch_bounds__(256) void sched_long_prefix_kernel(int n_items, const fgnn_item *__restrict__ items, int bucketed, int limit,
                                                                int *__restrict__ out)
{
    const int i = (int)(blockIdx.x * 256 + threadIdx.x);
    if (i >= n_items) return;
    const fgnn_item it = items[i];
    if (it.row < 0 || it.end - it.begin <= limit) return;
    const int k = bucketed ? (i / (FGNN_NUM_XCD * FGNN_WPB)) * FGNN_WPB + i % FGNN_WPB : i;
    atomicMax(out, k + 1);
}

// Sets s->n_wave_slots from the finished item array (one more read-back of one int).
static int schedule_mark_long_prefix(fgnn_schedule *s, hipStream_t st)
{
    s->n_wave_slots = 0;
    if (s->n_items == 0) return 0;
    int *dev = nullptr, last = 0;
    FGNN_HIP(hipMalloc((void **)&dev, sizeof(int)));
    hipError_t err = hipMemcpyAsync(dev, &last, sizeof(int), hipMemcpyHostToDevice, st);
    if (err == hipSuccess) {
        hipLaunchKernelGGL(sched_long_prefix_kernel, dim3((unsigned)((s->n_items + 255) / 256)), dim3(256), 0, st, s->n_items, s->items_dev,
                           s->n_buckets > 0 ? 1 : 0, FGNN_GROUP_ITEM_MAX, dev);
        err = hipGetLastError();
    }
    if (err == hipSuccess) err = hipMemcpyAsync(&last, dev, sizeof(int), hipMemcpyDeviceToHost, st);
    if (err == hipSuccess) err = hipStreamSynchronize(st);
    (void)hipFree(dev);
    if (err != hipSuccess) { fgnn_set_error("schedule: %s", hipGetErrorString(err)); return (int)err; }
    const int64_t per = s->n_buckets > 0 ? FGNN_NUM_XCD : 1;
    const int64_t slots = ((int64_t)last + 63) / 64 * 64 * per;
    s->n_wave_slots = (int)std::min<int64_t>(slots, s->n_items);
    return 0;
}

static int upload_schedule(fgnn_schedule *s, const std::vector<fgnn_item> &items, const std::vector<fgnn_split> &splits, hipStream_t st)
{
    hipError_t err = hipSuccess;
    if (!items.empty()) {
        err = hipMalloc((void **)&s->items_dev, items.size() * sizeof(fgnn_item));
        if (err == hipSuccess) err = hipMemcpyAsync(s->items_dev, items.data(), items.size() * sizeof(fgnn_item), hipMemcpyHostToDevice, st);
    }
    if (err == hipSuccess && !splits.empty()) {
        err = hipMalloc((void **)&s->split_dev, splits.size() * sizeof(fgnn_split));
        if (err == hipSuccess) err = hipMemcpyAsync(s->split_dev, splits.data(), splits.size() * sizeof(fgnn_split), hipMemcpyHostToDevice, st);
    }
    if (err == hipSuccess) err = hipStreamSynchronize(st);   // the host vectors die at return
    if (err != hipSuccess) {
        fgnn_set_error("schedule upload: %s", hipGetErrorString(err));
        return (int)err;
    }
    return schedule_mark_long_prefix(s, st);
}

static int read_ptr(const int32_t *ptr_dev, int n_rows, hipStream_t st, std::vector<int32_t> &ptr)
{
    ptr.resize((size_t)n_rows + 1);
    FGNN_HIP(hipMemcpyAsync(ptr.data(), ptr_dev, sizeof(int32_t) * ((size_t)n_rows + 1), hipMemcpyDeviceToHost, st));
    FGNN_HIP(hipStreamSynchronize(st));
    FGNN_REQUIRE(ptr[0] == 0, FGNN_ERR_SHAPE, "schedule: ptr[0]=%d, expected 0", ptr[0]);
    for (int i = 0; i < n_rows; ++i)
        FGNN_REQUIRE(ptr[i + 1] >= ptr[i], FGNN_ERR_SHAPE, "schedule: ptr decreases at row %d", i);
    return 0;
}

static fgnn_schedule *new_schedule(const int32_t *ptr_dev, int n_rows, int64_t n_edges, int seg_len)
{
    fgnn_schedule *s = new fgnn_schedule();
    s->n_rows = n_rows; s->n_edges = n_edges; s->seg_len = seg_len;
    s->n_items = s->n_partials = s->n_split = 0;
    s->items_dev = nullptr; s->split_dev = nullptr; s->ptr_dev = ptr_dev;
    s->n_buckets = 0; s->idx_src_dev = nullptr; s->bidx_dev = nullptr; s->bpos_dev = nullptr; s->own_order = 0; s->n_wave_slots = 0;
    (void)hipGetDevice(&s->device);
    return s;
}

// The work list built on the host from a read-back of the pointer array: the first implementation, kept as the
// cross-check of the device builder below (FGNN_SCHEDULE_BUILDER=host selects it).
static int schedule_create_host(const int32_t *ptr_dev, int n_rows, int seg_len, void *stream, fgnn_schedule_t **out)
{
    hipStream_t st = (hipStream_t)stream;
    std::vector<int32_t> ptr;
    int rc = read_ptr(ptr_dev, n_rows, st, ptr);
    if (rc) return rc;

    std::vector<fgnn_item> items;
    std::vector<fgnn_split> splits;
    items.reserve((size_t)n_rows + 1024);
    int n_part = 0;
    // segments of long rows first (they are the largest items), then whole rows, longest first
    for (int i = 0; i < n_rows; ++i) {
        int deg = ptr[i + 1] - ptr[i];
        if (deg <= seg_len) continue;
        int first = n_part, nseg = 0;
        split_range(items, i, ptr[i], ptr[i + 1], seg_len, n_part, nseg);
        splits.push_back({i, first, nseg, 0});
    }
    size_t first_whole = items.size();
    for (int i = 0; i < n_rows; ++i) {
        int deg = ptr[i + 1] - ptr[i];
        if (deg <= seg_len) items.push_back({i, ptr[i], ptr[i + 1], -1});
    }
    sort_longest_first(items, first_whole);

    fgnn_schedule *s = new_schedule(ptr_dev, n_rows, n_rows ? ptr[n_rows] : 0, seg_len);
    s->n_items = (int)items.size();
    s->n_partials = n_part;
    s->n_split = (int)splits.size();
    rc = upload_schedule(s, items, splits, st);
    if (rc) { fgnn_schedule_destroy(s); return rc; }
    *out = s;
    return 0;
}

// XCD-aware schedule.  Rows with more than `min_deg` entries are cut by SOURCE BUCKET (8 buckets,
// fgnn_bucket_of): the library keeps a copy of the index array with every row's entries grouped by
// bucket, and lays the work items out so that workgroup w only gets segments of bucket w % 8.  Each
// XCD's L2 then sees one eighth of the gathered rows, which is what lets the hot ones stay resident.
// Shorter rows stay whole and are dealt round-robin.  Segments are partial results merged by row.
static int schedule_create_bucketed_host(const int32_t *ptr_dev, const int32_t *idx_dev, int n_rows, int seg_len, int min_deg,
                                         int with_positions, void *stream, fgnn_schedule_t **out)
{
    hipStream_t st = (hipStream_t)stream;
    std::vector<int32_t> ptr;
    int rc = read_ptr(ptr_dev, n_rows, st, ptr);
    if (rc) return rc;
    const int64_t n_edges = n_rows ? ptr[n_rows] : 0;
    FGNN_REQUIRE(idx_dev || n_edges == 0, FGNN_ERR_NULL, "fgnn_schedule_create_bucketed: idx is NULL");

    fgnn_schedule *s = new_schedule(ptr_dev, n_rows, n_edges, seg_len);
    s->n_buckets = FGNN_NUM_XCD;
    s->idx_src_dev = idx_dev;
    std::vector<int32_t> bcnt((size_t)n_rows * FGNN_NUM_XCD);
    if (n_rows > 0) {
        int32_t *bcnt_dev = nullptr;
        hipError_t err = hipMalloc((void **)&bcnt_dev, bcnt.size() * sizeof(int32_t));
        if (err == hipSuccess && n_edges > 0) err = hipMalloc((void **)&s->bidx_dev, (size_t)n_edges * sizeof(int32_t));
        if (err == hipSuccess && n_edges > 0 && with_positions) err = hipMalloc((void **)&s->bpos_dev, (size_t)n_edges * sizeof(int32_t));
        if (err == hipSuccess) {
            hipLaunchKernelGGL(bucket_partition_kernel, dim3((unsigned)((n_rows + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, st,
                               n_rows, ptr_dev, idx_dev, s->bidx_dev, s->bpos_dev, bcnt_dev);
            err = hipGetLastError();
        }
        if (err == hipSuccess) err = hipMemcpyAsync(bcnt.data(), bcnt_dev, bcnt.size() * sizeof(int32_t), hipMemcpyDeviceToHost, st);
        if (err == hipSuccess) err = hipStreamSynchronize(st);
        if (bcnt_dev) (void)hipFree(bcnt_dev);
        if (err != hipSuccess) {
            fgnn_set_error("fgnn_schedule_create_bucketed: %s", hipGetErrorString(err));
            fgnn_schedule_destroy(s);
            return (int)err;
        }
    }

    std::vector<fgnn_item> lists[FGNN_NUM_XCD];
    std::vector<fgnn_split> splits;
    int n_part = 0;
    for (int i = 0; i < n_rows; ++i) {
        int deg = ptr[i + 1] - ptr[i];
        if (deg <= min_deg) continue;
        int first = n_part, nseg = 0, b0 = ptr[i];
        for (int b = 0; b < FGNN_NUM_XCD; ++b) {
            int c = bcnt[(size_t)i * FGNN_NUM_XCD + b];
            if (c > 0) split_range(lists[b], i, b0, b0 + c, seg_len, n_part, nseg);
            b0 += c;
        }
        splits.push_back({i, first, nseg, 0});
    }
    for (int b = 0; b < FGNN_NUM_XCD; ++b) sort_longest_first(lists[b]);
    // whole (short) rows, longest first, dealt round-robin; they run after the bucketed segments, so
    // their gathers from arbitrary buckets do not disturb the per-XCD working sets
    std::vector<fgnn_item> tails[FGNN_NUM_XCD];
    {
        std::vector<fgnn_item> whole;
        for (int i = 0; i < n_rows; ++i) {
            int deg = ptr[i + 1] - ptr[i];
            if (deg <= min_deg) whole.push_back({i, ptr[i], ptr[i + 1], -1});
        }
        sort_longest_first(whole);
        for (size_t w = 0; w < whole.size(); ++w) tails[w % FGNN_NUM_XCD].push_back(whole[w]);
    }
    std::vector<fgnn_item> items;
    for (const std::vector<fgnn_item> *part : {lists, tails}) {
        size_t longest = 0;
        for (int b = 0; b < FGNN_NUM_XCD; ++b) longest = std::max(longest, part[b].size());
        size_t groups = (longest + FGNN_WPB - 1) / FGNN_WPB, base = items.size();
        items.resize(base + groups * FGNN_NUM_XCD * FGNN_WPB, fgnn_item{-1, 0, 0, -1});
        for (int b = 0; b < FGNN_NUM_XCD; ++b)
            for (size_t k = 0; k < part[b].size(); ++k)
                items[base + ((k / FGNN_WPB) * FGNN_NUM_XCD + b) * FGNN_WPB + (k % FGNN_WPB)] = part[b][k];   // workgroup = group*8 + bucket
    }

    s->n_items = (int)items.size();
    s->n_partials = n_part;
    s->n_split = (int)splits.size();
    rc = upload_schedule(s, items, splits, st);
    if (rc) { fgnn_schedule_destroy(s); return rc; }
    *out = s;
    return 0;
}

// ------------------------------------------------------------------------------------------------
// The same work lists built on the device.  Per row: how many segments it is cut into (count kernel), two scans
// (first partial slot of every split row, rank of every split row), ONE read-back of a dozen counters for the
// allocation sizes, then the segments and the whole rows are emitted in the host builder's generation order,
// stably sorted longest first with the library's radix sort (per source bucket for an XCD-aware list) and placed.
// Item for item the result equals the host builder's.
struct SchedCounts { int err, n_part, n_split, e_total; int cntb[FGNN_NUM_XCD]; };

// Pieces a range of `len` entries is cut into, as split_range does it; step = length of all but the last.
static __host__ __device__ inline int sched_pieces(int len, int seg_len, int &step)
{
    const int nseg = (len + seg_len - 1) / seg_len;
    step = (((len + nseg - 1) / nseg) + 63) & ~63;
    return (len + step - 1) / step;
}

__global__ __launch_bounds__(256) void sched_count_kernel(int n_rows, const int *__restrict__ ptr, const int *__restrict__ bcnt, int cut, int seg_len,
                                                          int *__restrict__ segs, int *__restrict__ longf, SchedCounts *__restrict__ c)
{
    __shared__ int cb[FGNN_NUM_XCD];
    if (threadIdx.x < FGNN_NUM_XCD) cb[threadIdx.x] = 0;
    __syncthreads();
    const int row = (int)(blockIdx.x * 256 + threadIdx.x);
    if (row < n_rows) {
        const int pb = ptr[row], pe = ptr[row + 1];
        const int deg = pe - pb;
        int err = (row == 0 && pb != 0) ? 1 : 0;
        if (deg < 0) err |= 2;
        if (row == n_rows - 1) c->e_total = pe;
        if (err) atomicOr(&c->err, err);
        const bool lng = deg > cut;
        int nseg = 0, step;
        if (lng) {
            if (bcnt) {
#pragma unroll
                for (int b = 0; b < FGNN_NUM_XCD; ++b) {
                    const int cnt = bcnt[(size_t)row * FGNN_NUM_XCD + b];
                    if (cnt > 0) { const int pc = sched_pieces(cnt, seg_len, step); nseg += pc; atomicAdd(&cb[b], pc); }
                }
            } else {
                nseg = sched_pieces(deg, seg_len, step);
            }
        }
        segs[row] = nseg;
        longf[row] = lng ? 1 : 0;
    }
    __syncthreads();
    if (bcnt && threadIdx.x < FGNN_NUM_XCD && cb[threadIdx.x]) atomicAdd(&c->cntb[threadIdx.x], cb[threadIdx.x]);
}

// Segments of the split rows into gen[slot] (slot order = rows ascending, buckets ascending, pieces ascending), with
// the sort key of an XCD-aware list (bucket major, longest first); the split table; the whole rows into (wkey, wrow).
__global__ __launch_bounds__(256) void sched_emit_kernel(int n_rows, const int *__restrict__ ptr, const int *__restrict__ bcnt, int cut, int seg_len,
                                                         const int *__restrict__ segs, const int *__restrict__ seg_incl,
                                                         const int *__restrict__ long_incl, fgnn_item *__restrict__ gen, int *__restrict__ key,
                                                         fgnn_split *__restrict__ splits, int *__restrict__ wkey, int *__restrict__ wrow)
{
    const int row = (int)(blockIdx.x * 256 + threadIdx.x);
    if (row >= n_rows) return;
    const int pb = ptr[row], deg = ptr[row + 1] - pb;
    if (deg > cut) {
        int slot = seg_incl[row] - segs[row];
        splits[long_incl[row] - 1] = fgnn_split{row, slot, segs[row], 0};
        int b0 = pb;
        const int nb = bcnt ? FGNN_NUM_XCD : 1;
        for (int b = 0; b < nb; ++b) {
            const int cnt = bcnt ? bcnt[(size_t)row * FGNN_NUM_XCD + b] : deg;
            if (cnt > 0) {
                int step;
                (void)sched_pieces(cnt, seg_len, step);
                for (int sb = b0; sb < b0 + cnt; sb += step) {
                    const int se = min(b0 + cnt, sb + step);
                    gen[slot] = fgnn_item{row, sb, se, slot};
                    if (key) key[slot] = b * (seg_len + 1) + (seg_len - (se - sb));
                    ++slot;
                }
            }
            b0 += cnt;
        }
    } else {
        const int w = row - long_incl[row];
        wkey[w] = cut - deg;
        wrow[w] = row;
    }
}

struct SchedBucketStart { int v[FGNN_NUM_XCD]; };
// XCD-aware list: sorted segment p of bucket b, k-th of its bucket, goes to workgroup (k / WPB) * 8 + b, wave k % WPB.
__global__ __launch_bounds__(256) void sched_place_segments_kernel(int n_part, const int *__restrict__ sorted_slot, const int *__restrict__ sorted_key,
                                                                   int seg_len, SchedBucketStart bs, const fgnn_item *__restrict__ gen,
                                                                   fgnn_item *__restrict__ items)
{
    const int p = (int)(blockIdx.x * 256 + threadIdx.x);
    if (p >= n_part) return;
    const int b = sorted_key[p] / (seg_len + 1);
    const int k = p - bs.v[b];
    items[((size_t)(k / FGNN_WPB) * FGNN_NUM_XCD + b) * FGNN_WPB + (k % FGNN_WPB)] = gen[sorted_slot[p]];
}
// Whole rows, longest first: rank w goes to slot base + w (plain list) or is dealt round-robin over the eight buckets.
__global__ __launch_bounds__(256) void sched_place_whole_kernel(int n_whole, const int *__restrict__ sorted_row, const int *__restrict__ ptr,
                                                                int bucketed, size_t base, fgnn_item *__restrict__ items)
{
    const int w = (int)(blockIdx.x * 256 + threadIdx.x);
    if (w >= n_whole) return;
    const int row = sorted_row[w];
    size_t dest = base + (size_t)w;
    if (bucketed) {
        const int b = w % FGNN_NUM_XCD, k = w / FGNN_NUM_XCD;
        dest = base + ((size_t)(k / FGNN_WPB) * FGNN_NUM_XCD + b) * FGNN_WPB + (k % FGNN_WPB);
    }
    items[dest] = fgnn_item{row, ptr[row], ptr[row + 1], -1};
}
__global__ __launch_bounds__(256) void sched_fill_padding_kernel(size_t n, fgnn_item *__restrict__ items)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) items[i] = fgnn_item{-1, 0, 0, -1};
}

#define SCHED_HIP(call)                                                                 \
    do {                                                                                \
        hipError_t e__ = (call);                                                        \
        if (e__ != hipSuccess && rc == 0) {                                             \
            fgnn_set_error("schedule: %s failed: %s", #call, hipGetErrorString(e__));   \
            rc = (int)e__;                                                              \
        }                                                                               \
    } while (0)

// bcnt_dev: per (row, bucket) entry counts of an XCD-aware list (NULL: plain list); cut: rows longer than this are split.
static int schedule_build_device(fgnn_schedule *s, const int32_t *ptr_dev, const int *bcnt_dev, int n_rows, int cut, int seg_len, hipStream_t st)
{
    if (n_rows == 0) return 0;
    const bool bucketed = bcnt_dev != nullptr;
    int rc = 0;
    char *tmp1 = nullptr, *tmp2 = nullptr;
    const size_t rb = fgnn_align256((size_t)n_rows * sizeof(int));
    const size_t scan_b = fgnn_scan_workspace(n_rows);
    SCHED_HIP(hipMalloc((void **)&tmp1, 4 * rb + scan_b + 512));
    if (rc) return rc;
    int *segs = (int *)tmp1, *longf = (int *)(tmp1 + rb), *seg_incl = (int *)(tmp1 + 2 * rb), *long_incl = (int *)(tmp1 + 3 * rb);
    int *scan_ws = (int *)(tmp1 + 4 * rb);
    SchedCounts *cnt_dev = (SchedCounts *)(tmp1 + 4 * rb + scan_b);          // 48 bytes, then two scan totals
    int *tot = (int *)(cnt_dev + 1);
    SchedCounts cnt;
    memset(&cnt, 0, sizeof(cnt));
    SCHED_HIP(hipMemcpyAsync(cnt_dev, &cnt, sizeof(cnt), hipMemcpyHostToDevice, st));
    const unsigned gr = (unsigned)((n_rows + 255) / 256);
    if (!rc) {
        hipLaunchKernelGGL(sched_count_kernel, dim3(gr), dim3(256), 0, st, n_rows, ptr_dev, bcnt_dev, cut, seg_len, segs, longf, cnt_dev);
        rc = fgnn_launch_status("sched_count_kernel");
    }
    if (!rc) rc = fgnn_inclusive_scan_i32(segs, n_rows, seg_incl, scan_ws, tot, st);
    if (!rc) rc = fgnn_inclusive_scan_i32(longf, n_rows, long_incl, scan_ws, tot + 1, st);
    int totals[2] = {0, 0};
    SCHED_HIP(hipMemcpyAsync(&cnt, cnt_dev, sizeof(cnt), hipMemcpyDeviceToHost, st));
    SCHED_HIP(hipMemcpyAsync(totals, tot, sizeof(totals), hipMemcpyDeviceToHost, st));
    SCHED_HIP(hipStreamSynchronize(st));                                     // the one read-back: a dozen counters
    if (!rc && cnt.err) {
        fgnn_set_error("schedule: %s", (cnt.err & 1) ? "ptr[0] != 0" : "ptr decreases");
        rc = FGNN_ERR_SHAPE;
    }
    if (rc) { (void)hipFree(tmp1); return rc; }
    const int n_part = totals[0], n_split = totals[1], n_whole = n_rows - n_split;
    s->n_edges = cnt.e_total;
    s->n_partials = n_part;
    s->n_split = n_split;
    size_t base2 = (size_t)n_part;
    SchedBucketStart bs;
    if (bucketed) {
        int longest = 0, run = 0;
        for (int b = 0; b < FGNN_NUM_XCD; ++b) { bs.v[b] = run; run += cnt.cntb[b]; longest = std::max(longest, cnt.cntb[b]); }
        base2 = (size_t)((longest + FGNN_WPB - 1) / FGNN_WPB) * FGNN_NUM_XCD * FGNN_WPB;
        const int longest_tail = (n_whole + FGNN_NUM_XCD - 1) / FGNN_NUM_XCD;
        s->n_items = (int)(base2 + (size_t)((longest_tail + FGNN_WPB - 1) / FGNN_WPB) * FGNN_NUM_XCD * FGNN_WPB);
    } else {
        for (int b = 0; b < FGNN_NUM_XCD; ++b) bs.v[b] = 0;
        s->n_items = n_part + n_whole;
    }
    // second stage: sized by the counters
    const size_t pb = fgnn_align256((size_t)std::max(n_part, 1) * sizeof(int)), wb = fgnn_align256((size_t)std::max(n_whole, 1) * sizeof(int));
    const size_t gen_b = fgnn_align256((size_t)std::max(n_part, 1) * sizeof(fgnn_item));
    const size_t sort_b = fgnn_align256(fgnn_rs_sort_workspace(std::max(std::max(n_part, n_whole), 1)));
    SCHED_HIP(hipMalloc((void **)&tmp2, gen_b + 2 * pb + 3 * wb + sort_b));
    if (!rc && s->n_items > 0) SCHED_HIP(hipMalloc((void **)&s->items_dev, (size_t)s->n_items * sizeof(fgnn_item)));
    if (!rc && n_split > 0) SCHED_HIP(hipMalloc((void **)&s->split_dev, (size_t)n_split * sizeof(fgnn_split)));
    if (!rc) {
        fgnn_item *gen = (fgnn_item *)tmp2;
        int *key = (int *)(tmp2 + gen_b), *pay = (int *)(tmp2 + gen_b + pb);
        int *wkey = (int *)(tmp2 + gen_b + 2 * pb), *wrow = wkey + wb / sizeof(int), *wsorted = wrow + wb / sizeof(int);
        void *sort_ws = tmp2 + gen_b + 2 * pb + 3 * wb;
        // a plain list keeps its segments in generation order: they go straight into the item array
        hipLaunchKernelGGL(sched_emit_kernel, dim3(gr), dim3(256), 0, st, n_rows, ptr_dev, bcnt_dev, cut, seg_len, segs, seg_incl, long_incl,
                           bucketed ? gen : s->items_dev, bucketed ? key : nullptr, s->split_dev, wkey, wrow);
        rc = fgnn_launch_status("sched_emit_kernel");
        if (!rc && bucketed) {
            hipLaunchKernelGGL(sched_fill_padding_kernel, dim3((unsigned)((s->n_items + 255) / 256)), dim3(256), 0, st, (size_t)s->n_items, s->items_dev);
            rc = fgnn_launch_status("sched_fill_padding_kernel");
            if (!rc && n_part > 0) {
                const int *sorted_key = nullptr;
                rc = fgnn_rs_sort_pairs(key, nullptr, n_part, fgnn_rs_key_bits(FGNN_NUM_XCD * (seg_len + 1)), pay, &sorted_key, sort_ws, st);
                if (!rc) {
                    hipLaunchKernelGGL(sched_place_segments_kernel, dim3((unsigned)((n_part + 255) / 256)), dim3(256), 0, st, n_part, pay, sorted_key,
                                       seg_len, bs, gen, s->items_dev);
                    rc = fgnn_launch_status("sched_place_segments_kernel");
                }
            }
        }
        if (!rc && n_whole > 0) {
            const int *sorted_key = nullptr;
            rc = fgnn_rs_sort_pairs(wkey, wrow, n_whole, fgnn_rs_key_bits(cut + 1), wsorted, &sorted_key, sort_ws, st);
            if (!rc) {
                hipLaunchKernelGGL(sched_place_whole_kernel, dim3((unsigned)((n_whole + 255) / 256)), dim3(256), 0, st, n_whole, wsorted, ptr_dev,
                                   bucketed ? 1 : 0, base2, s->items_dev);
                rc = fgnn_launch_status("sched_place_whole_kernel");
            }
        }
    }
    SCHED_HIP(hipStreamSynchronize(st));          // the temporaries are freed below
    if (tmp2) (void)hipFree(tmp2);
    (void)hipFree(tmp1);
    if (!rc) rc = schedule_mark_long_prefix(s, st);
    return rc;
}

// out[0] |= 1: ptr[0] != 0; 2: ptr decreases somewhere; out[1] = ptr[n_rows]
__global__ __launch_bounds__(256) void sched_check_ptr_kernel(int n_rows, const int *__restrict__ ptr, int *__restrict__ out)
{
    int bad = 0;
    for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < n_rows; i += (int)(gridDim.x * 256)) {
        if (i == 0 && ptr[0] != 0) bad |= 1;
        if (ptr[i + 1] < ptr[i]) bad |= 2;
        if (i == n_rows - 1) out[1] = ptr[n_rows];
    }
    if (bad) atomicOr(out, bad);
}

static bool schedule_builder_is_host()
{
    const char *v = getenv("FGNN_SCHEDULE_BUILDER");
    return v && strcmp(v, "host") == 0;
}

extern "C" int fgnn_schedule_create(const int32_t *ptr_dev, int n_rows, int seg_len, void *stream, fgnn_schedule_t **out)
{
    FGNN_REQUIRE(ptr_dev && out, FGNN_ERR_NULL, "fgnn_schedule_create: NULL argument");
    FGNN_REQUIRE(n_rows >= 0, FGNN_ERR_SHAPE, "fgnn_schedule_create: n_rows=%d", n_rows);
    if (seg_len <= 0) seg_len = 2048;
    seg_len = (seg_len + 63) & ~63;
    if (schedule_builder_is_host()) return schedule_create_host(ptr_dev, n_rows, seg_len, stream, out);
    fgnn_schedule *s = new_schedule(ptr_dev, n_rows, 0, seg_len);
    int rc = schedule_build_device(s, ptr_dev, nullptr, n_rows, seg_len, seg_len, (hipStream_t)stream);
    if (rc) { fgnn_schedule_destroy(s); return rc; }
    *out = s;
    return 0;
}

// The XCD-aware list rests on one property of the part: workgroup w of a dispatch runs on XCD w % 8.  That holds for a
// gfx950 device that shows all of its 256 compute units (eight XCDs of 32, SPX mode); a partition of the part (fewer
// compute units per device) or another part spreads workgroups differently, and the bucketed list would then cost its
// extra segments and its index copy for nothing.  Returns the number of XCDs the mapping is known for, 0 otherwise.
extern "C" int fgnn_xcd_mapping_for(const char *gcn_arch, int compute_units)
{
    if (!gcn_arch) return 0;
    const bool gfx950 = strncmp(gcn_arch, "gfx950", 6) == 0 && (gcn_arch[6] == '\0' || gcn_arch[6] == ':');
    return gfx950 && compute_units == 32 * FGNN_NUM_XCD ? FGNN_NUM_XCD : 0;
}

// 1: the current device has the workgroup-to-XCD mapping the bucketed lists assume; 0: it has not (or cannot be asked)
int fgnn_current_device_has_xcd_mapping()
{
    static std::mutex mu;
    static int known[64];          // per device: 0 = not asked yet, 1 = no, 2 = yes
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    std::lock_guard<std::mutex> lock(mu);
    if (known[dev] == 0) {
        hipDeviceProp_t prop;
        known[dev] = (hipGetDeviceProperties(&prop, dev) == hipSuccess && fgnn_xcd_mapping_for(prop.gcnArchName, prop.multiProcessorCount) > 0) ? 2 : 1;
    }
    return known[dev] == 2;
}

extern "C" int fgnn_schedule_create_bucketed(const int32_t *ptr_dev, const int32_t *idx_dev, int n_rows, int seg_len, int min_deg,
                                             int with_positions, void *stream, fgnn_schedule_t **out)
{
    FGNN_REQUIRE(ptr_dev && out, FGNN_ERR_NULL, "fgnn_schedule_create_bucketed: NULL argument");
    FGNN_REQUIRE(n_rows >= 0, FGNN_ERR_SHAPE, "fgnn_schedule_create_bucketed: n_rows=%d", n_rows);
    // on a device without the assumed workgroup-to-XCD mapping the plain list is built instead (fgnn_schedule_num_buckets
    // of the result is then 0); FGNN_XCD_MAPPING=0 / 1 in the environment overrides the check
    const char *force = getenv("FGNN_XCD_MAPPING");
    if (force ? (strcmp(force, "0") == 0) : !fgnn_current_device_has_xcd_mapping())
        return fgnn_schedule_create(ptr_dev, n_rows, seg_len, stream, out);
    if (seg_len <= 0) seg_len = 2048;
    seg_len = (seg_len + 63) & ~63;
    if (min_deg <= 0) min_deg = 64;
    if (schedule_builder_is_host()) return schedule_create_bucketed_host(ptr_dev, idx_dev, n_rows, seg_len, min_deg, with_positions, stream, out);
    hipStream_t st = (hipStream_t)stream;
    // the pointer array is checked before the partition kernel walks the index array with it; the same 8-byte
    // read-back brings the edge count, which sizes the bucket-ordered copies
    int32_t e32 = 0;
    if (n_rows > 0) {
        int *chk_dev = nullptr, chk[2] = {0, 0};
        FGNN_HIP(hipMalloc((void **)&chk_dev, sizeof(chk)));
        hipError_t err = hipMemcpyAsync(chk_dev, chk, sizeof(chk), hipMemcpyHostToDevice, st);
        if (err == hipSuccess) {
            hipLaunchKernelGGL(sched_check_ptr_kernel, dim3((unsigned)std::min((n_rows + 255) / 256, 4096)), dim3(256), 0, st, n_rows, ptr_dev, chk_dev);
            err = hipGetLastError();
        }
        if (err == hipSuccess) err = hipMemcpyAsync(chk, chk_dev, sizeof(chk), hipMemcpyDeviceToHost, st);
        if (err == hipSuccess) err = hipStreamSynchronize(st);
        (void)hipFree(chk_dev);
        if (err != hipSuccess) { fgnn_set_error("fgnn_schedule_create_bucketed: %s", hipGetErrorString(err)); return (int)err; }
        FGNN_REQUIRE(chk[0] == 0, FGNN_ERR_SHAPE, "schedule: %s", (chk[0] & 1) ? "ptr[0] != 0" : "ptr decreases");
        e32 = chk[1];
    }
    FGNN_REQUIRE(e32 >= 0, FGNN_ERR_SHAPE, "schedule: ptr[n_rows]=%d", e32);
    FGNN_REQUIRE(idx_dev || e32 == 0, FGNN_ERR_NULL, "fgnn_schedule_create_bucketed: idx is NULL");
    fgnn_schedule *s = new_schedule(ptr_dev, n_rows, e32, seg_len);
    s->n_buckets = FGNN_NUM_XCD;
    s->idx_src_dev = idx_dev;
    int rc = 0;
    int32_t *bcnt_dev = nullptr;
    if (n_rows > 0) {
        SCHED_HIP(hipMalloc((void **)&bcnt_dev, (size_t)n_rows * FGNN_NUM_XCD * sizeof(int32_t)));
        if (!rc && e32 > 0) SCHED_HIP(hipMalloc((void **)&s->bidx_dev, (size_t)e32 * sizeof(int32_t)));
        if (!rc && e32 > 0 && with_positions) SCHED_HIP(hipMalloc((void **)&s->bpos_dev, (size_t)e32 * sizeof(int32_t)));
        if (!rc) {
            hipLaunchKernelGGL(bucket_partition_kernel, dim3((unsigned)((n_rows + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, st,
                               n_rows, ptr_dev, idx_dev, s->bidx_dev, s->bpos_dev, bcnt_dev);
            rc = fgnn_launch_status("bucket_partition_kernel");
        }
        if (!rc) rc = schedule_build_device(s, ptr_dev, bcnt_dev, n_rows, min_deg, seg_len, st);
        if (bcnt_dev) (void)hipFree(bcnt_dev);
    }
    if (rc) { fgnn_schedule_destroy(s); return rc; }
    *out = s;
    return 0;
}

// Copies the work items (4 ints each: row, begin, end, slot) and the split table (4 ints each: row, first slot,
// segments, 0) to caller memory on the device; either pointer may be NULL.
extern "C" int fgnn_schedule_export(const fgnn_schedule_t *s, int32_t *items_out, int32_t *splits_out, void *stream)
{
    FGNN_REQUIRE(s, FGNN_ERR_NULL, "fgnn_schedule_export: NULL schedule");
    hipStream_t st = (hipStream_t)stream;
    if (items_out && s->n_items > 0)
        FGNN_HIP(hipMemcpyAsync(items_out, s->items_dev, (size_t)s->n_items * sizeof(fgnn_item), hipMemcpyDeviceToDevice, st));
    if (splits_out && s->n_split > 0)
        FGNN_HIP(hipMemcpyAsync(splits_out, s->split_dev, (size_t)s->n_split * sizeof(fgnn_split), hipMemcpyDeviceToDevice, st));
    return 0;
}
extern "C" int fgnn_schedule_num_splits(const fgnn_schedule_t *s) { return s ? s->n_split : 0; }
extern "C" int fgnn_schedule_num_wave_slots(const fgnn_schedule_t *s) { return s ? s->n_wave_slots : 0; }

__global__ __launch_bounds__(256) void iota_i32_kernel(int64_t n, int *__restrict__ out)
{
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = (int)i;
}

// Hands the map (schedule entry order -> caller's edge position) to the caller and drops the
// schedule's own copy.  From then on operators index per-edge tensors (and `permute`) by the
// schedule's entry order: an XCD then reads and writes the per-edge data of its segments as
// contiguous runs instead of scattered elements of lines that all eight XCDs touch.
extern "C" int fgnn_schedule_take_positions(fgnn_schedule_t *s, int32_t *pos_out_dev, void *stream)
{
    FGNN_REQUIRE(s, FGNN_ERR_NULL, "fgnn_schedule_take_positions: NULL schedule");
    FGNN_REQUIRE(pos_out_dev || s->n_edges == 0, FGNN_ERR_NULL, "fgnn_schedule_take_positions: NULL output");
    FGNN_REQUIRE(!s->own_order, FGNN_ERR_SCHEDULE, "fgnn_schedule_take_positions: the positions of this schedule were taken before");
    FGNN_REQUIRE(fgnn_sched_has_pos(s), FGNN_ERR_SCHEDULE, "fgnn_schedule_take_positions: the schedule was built without edge positions");
    hipStream_t st = (hipStream_t)stream;
    if (s->n_edges > 0) {
        if (s->n_buckets > 0) {
            FGNN_HIP(hipMemcpyAsync(pos_out_dev, s->bpos_dev, (size_t)s->n_edges * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
        } else {        // plain schedules walk the caller's arrays: identity
            hipLaunchKernelGGL(iota_i32_kernel, dim3((unsigned)((s->n_edges + 255) / 256)), dim3(256), 0, st, s->n_edges, pos_out_dev);
            int rc = fgnn_launch_status("iota_i32_kernel");
            if (rc) return rc;
        }
        FGNN_HIP(hipStreamSynchronize(st));      // the copy must be done before the source is freed
    }
    if (s->bpos_dev) { (void)hipFree(s->bpos_dev); s->bpos_dev = nullptr; }
    s->own_order = 1;
    return 0;
}

extern "C" void fgnn_schedule_destroy(fgnn_schedule_t *s)
{
    if (!s) return;
    if (s->items_dev) (void)hipFree(s->items_dev);
    if (s->split_dev) (void)hipFree(s->split_dev);
    if (s->bidx_dev) (void)hipFree(s->bidx_dev);
    if (s->bpos_dev) (void)hipFree(s->bpos_dev);
    delete s;
}

extern "C" size_t fgnn_schedule_device_bytes(const fgnn_schedule_t *s)
{
    if (!s) return 0;
    size_t b = (size_t)s->n_items * sizeof(fgnn_item) + (size_t)s->n_split * sizeof(fgnn_split);
    if (s->bidx_dev) b += (size_t)s->n_edges * sizeof(int32_t);
    if (s->bpos_dev) b += (size_t)s->n_edges * sizeof(int32_t);
    return b;
}

// flags[0] |= 1: ptr[0] != 0; 2: ptr decreases; 4: ptr[n_rows] != E; 8: an index outside [0, n_cols)
__global__ __launch_bounds__(256) void validate_graph_kernel(const int *__restrict__ ptr, const int *__restrict__ idx, int n_rows, int n_cols,
                                                             int64_t E, int *__restrict__ flags)
{
    int bad = 0;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i <= n_rows; i += stride) {
        const int v = ptr[i];
        if (i == 0 && v != 0) bad |= 1;
        if (i < n_rows && ptr[i + 1] < v) bad |= 2;
        if (i == n_rows && (int64_t)v != E) bad |= 4;
    }
    for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < E; q += stride) {
        const int j = idx[q];
        if (j < 0 || j >= n_cols) bad |= 8;
    }
    if (bad) atomicOr(flags, bad);
}

extern "C" int fgnn_validate_graph(const int32_t *ptr_dev, const int32_t *idx_dev, int n_rows, int n_cols, int64_t E, void *stream)
{
    FGNN_REQUIRE(ptr_dev && (idx_dev || E == 0), FGNN_ERR_NULL, "fgnn_validate_graph: NULL argument");
    FGNN_REQUIRE(n_rows >= 0 && n_cols >= 0 && E >= 0 && E <= 2147483647LL, FGNN_ERR_SHAPE, "fgnn_validate_graph: bad sizes n_rows=%d n_cols=%d E=%lld",
                 n_rows, n_cols, (long long)E);
    hipStream_t st = (hipStream_t)stream;
    int *flags_dev = nullptr;
    int flags = 0;
    FGNN_HIP(hipMalloc((void **)&flags_dev, sizeof(int)));
    hipError_t err = hipMemcpyAsync(flags_dev, &flags, sizeof(int), hipMemcpyHostToDevice, st);
    if (err == hipSuccess) {
        const int64_t work = std::max<int64_t>(E, (int64_t)n_rows + 1);
        const unsigned grid = (unsigned)std::min<int64_t>((work + 255) / 256, 8192);
        hipLaunchKernelGGL(validate_graph_kernel, dim3(grid), dim3(256), 0, st, ptr_dev, idx_dev, n_rows, n_cols, E, flags_dev);
        err = hipGetLastError();
    }
    if (err == hipSuccess) err = hipMemcpyAsync(&flags, flags_dev, sizeof(int), hipMemcpyDeviceToHost, st);
    if (err == hipSuccess) err = hipStreamSynchronize(st);
    (void)hipFree(flags_dev);
    if (err != hipSuccess) {
        fgnn_set_error("fgnn_validate_graph: %s", hipGetErrorString(err));
        return (int)err;
    }
    FGNN_REQUIRE(flags == 0, FGNN_ERR_SHAPE, "fgnn_validate_graph: malformed graph:%s%s%s%s", (flags & 1) ? " ptr[0] != 0;" : "",
                 (flags & 2) ? " ptr decreases;" : "", (flags & 4) ? " ptr[n_rows] != E;" : "", (flags & 8) ? " an index lies outside [0, n_cols);" : "");
    return 0;
}

// stats[0] += entries of the rows longer than long_len, stats[1] = max row length (both as unsigned 64-bit)
__global__ __launch_bounds__(256) void row_length_stats_kernel(const int *__restrict__ ptr, int n_rows, int long_len,
                                                               unsigned long long *__restrict__ stats)
{
    __shared__ unsigned long long sh_sum[4];
    __shared__ int sh_max[4];
    unsigned long long sum = 0;
    int longest = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_rows; i += (int64_t)gridDim.x * 256) {
        const int d = ptr[i + 1] - ptr[i];
        if (d > long_len) sum += (unsigned long long)d;
        longest = max(longest, d);
    }
    for (int off = 32; off > 0; off >>= 1) {
        sum += __shfl_down(sum, off);
        longest = max(longest, __shfl_down(longest, off));
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sh_sum[wave] = sum; sh_max[wave] = longest; }
    __syncthreads();
    if (threadIdx.x == 0) {
        sum = (sh_sum[0] + sh_sum[1]) + (sh_sum[2] + sh_sum[3]);
        longest = max(max(sh_max[0], sh_max[1]), max(sh_max[2], sh_max[3]));
        if (sum) atomicAdd(stats, sum);
        if (longest > 0) atomicMax(stats + 1, (unsigned long long)longest);
    }
}

extern "C" int fgnn_row_length_stats(const int32_t *ptr_dev, int n_rows, int long_len, int64_t *stats_host, void *stream)
{
    FGNN_REQUIRE(ptr_dev && stats_host, FGNN_ERR_NULL, "fgnn_row_length_stats: NULL argument");
    FGNN_REQUIRE(n_rows >= 0 && long_len >= 0, FGNN_ERR_SHAPE, "fgnn_row_length_stats: bad sizes n_rows=%d long_len=%d", n_rows, long_len);
    stats_host[0] = stats_host[1] = 0;
    if (n_rows == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    unsigned long long *dev = nullptr, host[2] = {0, 0};
    FGNN_HIP(hipMalloc((void **)&dev, sizeof(host)));
    hipError_t err = hipMemcpyAsync(dev, host, sizeof(host), hipMemcpyHostToDevice, st);
    if (err == hipSuccess) {
        const unsigned grid = (unsigned)std::min<int64_t>(((int64_t)n_rows + 255) / 256, 2048);
        hipLaunchKernelGGL(row_length_stats_kernel, dim3(grid), dim3(256), 0, st, ptr_dev, n_rows, long_len, dev);
        err = hipGetLastError();
    }
    if (err == hipSuccess) err = hipMemcpyAsync(host, dev, sizeof(host), hipMemcpyDeviceToHost, st);
    if (err == hipSuccess) err = hipStreamSynchronize(st);
    (void)hipFree(dev);
    if (err != hipSuccess) {
        fgnn_set_error("fgnn_row_length_stats: %s", hipGetErrorString(err));
        return (int)err;
    }
    stats_host[0] = (int64_t)host[0];
    stats_host[1] = (int64_t)host[1];
    return 0;
}

extern "C" int fgnn_schedule_num_items(const fgnn_schedule_t *s) { return s ? s->n_items : 0; }
extern "C" int fgnn_schedule_num_buckets(const fgnn_schedule_t *s) { return s ? s->n_buckets : 0; }
extern "C" int fgnn_schedule_num_partials(const fgnn_schedule_t *s) { return s ? s->n_partials : 0; }
extern "C" int64_t fgnn_schedule_num_edges(const fgnn_schedule_t *s) { return s ? s->n_edges : 0; }
