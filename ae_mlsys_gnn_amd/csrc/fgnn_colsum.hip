// Column sums of a per-edge array: out[j,:] = sum over the CSR positions p with col_ind[p] == j of g[p,:]
// (the grad_col half of u_add_v's backward, src/u_add_v/u_add_v.cu:43-90 of the reference, and the
// gather_col step of its fuse-scatter GAT backward, src/fused_gat/fused_gat.cu:558-586), without
// global atomics and bit-reproducible.
//
// g arrives in CSR order, the sums run over columns: read in CSC order every 32-byte entry would pull a
// whole 128-byte line.  The plan cuts the COLUMNS into ranges of C = 2^k and lists the entries of each
// range in CSR order ("tile order").  Inside a row the columns ascend, so the entries of (row, range)
// are one contiguous run of g: a range's task streams runs instead of single entries (on a 115 M-entry
// power-law graph with C = 256 the lines it touches hold 1.7 x the bytes it needs), and C columns x W
// floats of accumulators fit the LDS share of ONE wave.  A task is a span of a range's list; one wave
// walks it from front to back: an instruction takes a batch of entries, equal columns inside the batch
// are first combined in registers (the plan keeps every aligned group of 64 entries sorted by column,
// so they sit in neighbouring lanes and a segmented scan does it), then one lane per distinct column
// adds into the wave's private LDS accumulators with a plain read-add-write.  No atomics anywhere
// (ds_add_f32 on colliding addresses took four times as long as the whole memory traffic), and every
// sum is formed in an order fixed by the plan.  Ranges cut into several tasks are summed over their
// partial results in task order by a second small kernel.
#include <algorithm>
#include <vector>
#include "fgnn_common.h"

struct fgnn_colsum_plan {
    int n_rows, n_cols;
    int64_t n_edges;
    int log_c;               // columns per range = 1 << log_c
    int n_ranges;
    int n_tasks, n_slots, n_merge;
    const int32_t *ptr_dev, *idx_dev;
    int32_t *tpos_dev;       // [E] CSR position of every entry in tile order
    uint16_t *lcol_dev;      // [E] its column minus the first column of its range
    fgnn_item *tasks_dev;    // {range, begin, end, partial slot or -1}
    fgnn_split *merge_dev;   // {range, first slot, tasks, 0} of every range cut into several tasks
    int device;
};

#define CS_MAX_LDS 65536     // accumulator bytes of one wave at most

__global__ __launch_bounds__(256) void cs_key_kernel(int64_t E, int n_cols, int log_c, const int *__restrict__ idx, int *__restrict__ key,
                                                     int *__restrict__ bad)
{
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= E) return;
    const int j = idx[p];
    const bool ok = j >= 0 && j < n_cols;
    if (!ok) atomicOr(bad, 1);
    key[p] = ok ? (j >> log_c) : 0;
}

// range_ptr[r] = first tile-order position of range r (r = 0 .. n_ranges), from the sorted range ids
__global__ __launch_bounds__(256) void cs_range_ptr_kernel(int64_t E, int n_ranges, const int *__restrict__ skey, int *__restrict__ range_ptr)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t > E) return;
    const int prev = t == 0 ? -1 : skey[t - 1];
    const int cur = t == E ? n_ranges : skey[t];
    for (int r = prev + 1; r <= cur; ++r) range_ptr[r] = (int)t;
}

__global__ __launch_bounds__(256) void cs_lcol_kernel(int64_t E, int log_c, const int *__restrict__ tpos, const int *__restrict__ idx,
                                                      uint16_t *__restrict__ lcol)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= E) return;
    lcol[t] = (uint16_t)(idx[tpos[t]] & ((1 << log_c) - 1));
}

// Sorts every aligned group of 64 entries of a task by column (equal columns keep their order), in place: one wave per
// task, the rank of an entry is the number of smaller keys among the group's 64 (column * 64 + lane: all different).
__global__ __launch_bounds__(64) void cs_group_sort_kernel(const fgnn_item *__restrict__ tasks, int *__restrict__ tpos, uint16_t *__restrict__ lcol)
{
    const fgnn_item tk = tasks[blockIdx.x];
    const int tb = fg_uni(tk.begin), te = fg_uni(tk.end);
    const int lane = fg_lane();
    for (int t0 = tb; t0 < te; t0 += 64) {
        const int t = t0 + lane;
        const bool ok = t < te;
        const int p = ok ? tpos[t] : 0;
        const int lc = ok ? (int)lcol[t] : 0;
        const int key = ok ? lc * 64 + lane : 0x7fffffff;
        int rank = 0;
        for (int j = 0; j < 64; ++j) rank += __builtin_amdgcn_readlane(key, j) < key ? 1 : 0;
        if (ok) { tpos[t0 + rank] = p; lcol[t0 + rank] = (uint16_t)lc; }
    }
}

extern "C" void fgnn_colsum_plan_destroy(fgnn_colsum_plan_t *p)
{
    if (!p) return;
    if (p->tpos_dev) (void)hipFree(p->tpos_dev);
    if (p->lcol_dev) (void)hipFree(p->lcol_dev);
    if (p->tasks_dev) (void)hipFree(p->tasks_dev);
    if (p->merge_dev) (void)hipFree(p->merge_dev);
    delete p;
}

#define CS_HIP(call)                                                                           \
    do {                                                                                       \
        hipError_t e__ = (call);                                                               \
        if (e__ != hipSuccess && rc == 0) {                                                    \
            fgnn_set_error("fgnn_colsum_plan_create: %s failed: %s", #call, hipGetErrorString(e__)); \
            rc = (int)e__;                                                                     \
        }                                                                                      \
    } while (0)

extern "C" int fgnn_colsum_plan_create(const int32_t *row_ptr, const int32_t *col_ind, int n_rows, int n_cols, int64_t E, int W,
                                       int lds_bytes, int task_len, void *stream, fgnn_colsum_plan_t **out)
{
    FGNN_REQUIRE(out && row_ptr && (col_ind || E == 0), FGNN_ERR_NULL, "fgnn_colsum_plan_create: NULL argument");
    FGNN_REQUIRE(n_rows >= 0 && n_cols >= 0 && E >= 0 && W >= 1, FGNN_ERR_SHAPE, "fgnn_colsum_plan_create: bad sizes");
    FGNN_REQUIRE(E <= 2147483647LL - 4096, FGNN_ERR_LIMIT, "fgnn_colsum_plan_create: E=%lld exceeds int32 positions", (long long)E);
    FGNN_REQUIRE(E == 0 || n_cols > 0, FGNN_ERR_SHAPE, "fgnn_colsum_plan_create: edges without columns");
    if (lds_bytes <= 0) lds_bytes = 8192;
    FGNN_REQUIRE(lds_bytes >= 1024 && lds_bytes <= CS_MAX_LDS, FGNN_ERR_LIMIT, "fgnn_colsum_plan_create: lds_bytes=%d outside [1024, %d]", lds_bytes, CS_MAX_LDS);
    // columns per range: the largest power of two whose accumulators (padded to groups of four floats) fit
    const int wpad = (W + 3) & ~3;
    FGNN_REQUIRE((int64_t)wpad * 4 * 4 <= lds_bytes, FGNN_ERR_LIMIT, "fgnn_colsum_plan_create: W=%d too wide for %d bytes of accumulators", W, lds_bytes);
    int log_c = 0;
    while (log_c < 16 && ((int64_t)2 << log_c) * wpad * 4 <= lds_bytes) ++log_c;
    hipStream_t st = (hipStream_t)stream;
    fgnn_colsum_plan *p = new fgnn_colsum_plan();
    p->n_rows = n_rows; p->n_cols = n_cols; p->n_edges = E; p->log_c = log_c;
    p->n_ranges = (int)(((int64_t)n_cols + (1 << log_c) - 1) >> log_c);
    p->n_tasks = p->n_slots = p->n_merge = 0;
    p->ptr_dev = row_ptr; p->idx_dev = col_ind;
    p->tpos_dev = nullptr; p->lcol_dev = nullptr; p->tasks_dev = nullptr; p->merge_dev = nullptr;
    (void)hipGetDevice(&p->device);
    if (task_len <= 0) task_len = (int)std::min<int64_t>(32768, std::max<int64_t>(2048, ((E / 4096) + 255) & ~(int64_t)255));
    int rc = 0;
    std::vector<int> range_ptr((size_t)p->n_ranges + 1, 0);
    if (E > 0) {
        char *tmp = nullptr;
        const size_t eb = fgnn_align256((size_t)E * sizeof(int)), rb = fgnn_align256(((size_t)p->n_ranges + 1) * sizeof(int));
        const size_t sort_b = fgnn_align256(fgnn_rs_sort_workspace(E));
        CS_HIP(hipMalloc((void **)&tmp, eb + rb + 256 + sort_b));
        CS_HIP(hipMalloc((void **)&p->tpos_dev, (size_t)E * sizeof(int32_t)));
        CS_HIP(hipMalloc((void **)&p->lcol_dev, (size_t)E * sizeof(uint16_t)));
        if (!rc) {
            int *key = (int *)tmp, *rptr = (int *)(tmp + eb), *bad = (int *)(tmp + eb + rb);
            void *sort_ws = tmp + eb + rb + 256;
            const unsigned ge = (unsigned)((E + 255) / 256);
            int zero = 0, bad_host = 0;
            CS_HIP(hipMemcpyAsync(bad, &zero, sizeof(int), hipMemcpyHostToDevice, st));
            if (!rc) {
                hipLaunchKernelGGL(cs_key_kernel, dim3(ge), dim3(256), 0, st, E, n_cols, log_c, col_ind, key, bad);
                rc = fgnn_launch_status("cs_key_kernel");
            }
            const int *skey = nullptr;
            if (!rc) rc = fgnn_rs_sort_pairs(key, nullptr, E, fgnn_rs_key_bits(std::max(p->n_ranges, 2)), p->tpos_dev, &skey, sort_ws, st);
            if (!rc) {
                hipLaunchKernelGGL(cs_range_ptr_kernel, dim3((unsigned)((E + 256) / 256)), dim3(256), 0, st, E, p->n_ranges, skey, rptr);
                rc = fgnn_launch_status("cs_range_ptr_kernel");
            }
            if (!rc) {
                hipLaunchKernelGGL(cs_lcol_kernel, dim3(ge), dim3(256), 0, st, E, log_c, p->tpos_dev, col_ind, p->lcol_dev);
                rc = fgnn_launch_status("cs_lcol_kernel");
            }
            CS_HIP(hipMemcpyAsync(range_ptr.data(), rptr, range_ptr.size() * sizeof(int), hipMemcpyDeviceToHost, st));
            CS_HIP(hipMemcpyAsync(&bad_host, bad, sizeof(int), hipMemcpyDeviceToHost, st));
            CS_HIP(hipStreamSynchronize(st));
            if (!rc && bad_host) {
                fgnn_set_error("fgnn_colsum_plan_create: an index lies outside [0, n_cols)");
                rc = FGNN_ERR_SHAPE;
            }
        }
        if (tmp) (void)hipFree(tmp);
    }
    if (rc) { fgnn_colsum_plan_destroy(p); return rc; }
    // tasks: every range gets at least one (an empty range still has its columns zero-filled), long ranges are cut
    std::vector<fgnn_item> tasks;
    std::vector<fgnn_split> merges;
    int n_slots = 0;
    for (int r = 0; r < p->n_ranges; ++r) {
        const int b = range_ptr[r], e = range_ptr[r + 1];
        const int len = e - b;
        if (len <= task_len) { tasks.push_back({r, b, e, -1}); continue; }
        const int nseg = (len + task_len - 1) / task_len;
        const int step = (((len + nseg - 1) / nseg) + 63) & ~63;
        const int first = n_slots;
        for (int s = b; s < e; s += step) tasks.push_back({r, s, std::min(e, s + step), n_slots++});
        merges.push_back({r, first, n_slots - first, 0});
    }
    std::stable_sort(tasks.begin(), tasks.end(), [](const fgnn_item &a, const fgnn_item &b) { return a.end - a.begin > b.end - b.begin; });
    p->n_tasks = (int)tasks.size(); p->n_slots = n_slots; p->n_merge = (int)merges.size();
    if (!tasks.empty()) {
        CS_HIP(hipMalloc((void **)&p->tasks_dev, tasks.size() * sizeof(fgnn_item)));
        CS_HIP(hipMemcpyAsync(p->tasks_dev, tasks.data(), tasks.size() * sizeof(fgnn_item), hipMemcpyHostToDevice, st));
    }
    if (!merges.empty()) {
        CS_HIP(hipMalloc((void **)&p->merge_dev, merges.size() * sizeof(fgnn_split)));
        CS_HIP(hipMemcpyAsync(p->merge_dev, merges.data(), merges.size() * sizeof(fgnn_split), hipMemcpyHostToDevice, st));
    }
    if (!rc && E > 0) {
        hipLaunchKernelGGL(cs_group_sort_kernel, dim3((unsigned)p->n_tasks), dim3(64), 0, st, p->tasks_dev, p->tpos_dev, p->lcol_dev);
        rc = fgnn_launch_status("cs_group_sort_kernel");
    }
    CS_HIP(hipStreamSynchronize(st));            // the host vectors die at return
    if (rc) { fgnn_colsum_plan_destroy(p); return rc; }
    *out = p;
    return 0;
}

extern "C" size_t fgnn_colsum_plan_device_bytes(const fgnn_colsum_plan_t *p)
{
    if (!p) return 0;
    return (size_t)p->n_edges * (sizeof(int32_t) + sizeof(uint16_t)) + (size_t)p->n_tasks * sizeof(fgnn_item) + (size_t)p->n_merge * sizeof(fgnn_split);
}
extern "C" int fgnn_colsum_plan_matches(const fgnn_colsum_plan_t *p, const int32_t *row_ptr, const int32_t *col_ind, int n_rows, int n_cols, int64_t E)
{
    return p && p->ptr_dev == row_ptr && p->idx_dev == col_ind && p->n_rows == n_rows && p->n_cols == n_cols && p->n_edges == E;
}
extern "C" int fgnn_colsum_plan_columns_per_range(const fgnn_colsum_plan_t *p) { return p ? 1 << p->log_c : 0; }
extern "C" int fgnn_colsum_plan_num_tasks(const fgnn_colsum_plan_t *p) { return p ? p->n_tasks : 0; }

// floats of one partial result: the accumulators of a range, W padded to a multiple of four
static inline size_t cs_partial_floats(const fgnn_colsum_plan *p, int W) { return ((size_t)1 << p->log_c) * (size_t)((W + 3) & ~3); }

extern "C" size_t fgnn_colsum_workspace_bytes(const fgnn_colsum_plan_t *p, int W)
{
    if (!p || W < 1) return 0;
    return fgnn_align256((size_t)p->n_slots * cs_partial_floats(p, W) * sizeof(float));
}

// One wave per task.  VEC = 4: an entry is G groups of four floats (W = 4G, 16-byte aligned arrays), lane (e, c) of an
// instruction owns group c of entry e, `per` entries per instruction (the largest power of two <= 64 / G: batches then
// never straddle the sorted groups of 64); VEC = 1: G = W single floats.  The accumulators are kept component-major
// (acc[k][column * G + c]) so that the lanes of an instruction fall into consecutive banks.
template <int VEC, int CS_U>
__global__ __launch_bounds__(64) void colsum_kernel(const fgnn_item *__restrict__ tasks, int log_c, int n_cols, int G, int per,
                                                    const int *__restrict__ tpos, const uint16_t *__restrict__ lcol,
                                                    const float *__restrict__ g, float *__restrict__ out, float *__restrict__ partials,
                                                    size_t partial_floats)
{
    extern __shared__ float acc[];
    const fgnn_item tk = tasks[blockIdx.x];
    const int range = fg_uni(tk.row), tb = fg_uni(tk.begin), te = fg_uni(tk.end), slot = fg_uni(tk.slot);
    const int lane = fg_lane();
    const int CG = G << log_c;                        // accumulator groups
    for (int i = lane; i < CG * VEC; i += 64) acc[i] = 0.f;
    fg_wave_lds_sync();
    const int e = lane / G, c = lane - e * G;
    const bool act = e < per;
    // The positions of trip i + 1 are fetched while the entries of trip i are in flight: a trip then costs one
    // memory latency instead of two (position, then entry), which is what bounds a wave that streams alone.
    int pp[CS_U], lc[CS_U];
    auto fetch_pos = [&](int t0) {
#pragma unroll
        for (int u = 0; u < CS_U; ++u) {
            const int t = t0 + u * per + e;
            const int tt = (act && t < te) ? t : tb;
            pp[u] = tpos[tt];
            lc[u] = (int)lcol[tt];
        }
    };
    if (tb < te) fetch_pos(tb);
    for (int t0 = tb; t0 < te; t0 += per * CS_U) {
        fg_vec<VEC> v[CS_U];
        int col[CS_U];
#pragma unroll
        for (int u = 0; u < CS_U; ++u) {
            v[u].load(g + ((size_t)pp[u] * G + c) * VEC);
            col[u] = (act && t0 + u * per + e < te) ? lc[u] : -1 - e;       // entries past the end: a column of their own
        }
        fetch_pos(t0 + per * CS_U);                   // past the end it re-reads the task's first entry
#pragma unroll
        for (int u = 0; u < CS_U; ++u) {
            if (col[u] < 0) v[u].zero();
            // Segmented inclusive scan over the entries of the batch (equal columns are neighbours).  Step d is needed only
            // if some entry equals the one d places before it, which (sorted columns) implies the same for every smaller
            // step: most batches hold no repeated column and leave after one exchange.
            bool last = true;
            for (int d = 1; d < per; d <<= 1) {
                const int src = (lane - d * G) & 63;
                const int col_src = __shfl(col[u], src);          // every lane takes part in the exchange
                const bool take = e >= d && col_src == col[u];
                if (__builtin_amdgcn_ballot_w64(take) == 0ull) break;
                if constexpr (VEC == 4) {
                    const float x = __shfl(v[u].v.x, src), y = __shfl(v[u].v.y, src), z = __shfl(v[u].v.z, src), w = __shfl(v[u].v.w, src);
                    if (take) { v[u].v.x += x; v[u].v.y += y; v[u].v.z += z; v[u].v.w += w; }
                } else {
                    const float x = __shfl(v[u].v, src);
                    if (take) v[u].v += x;
                }
                if (d == 1) {                                     // some column repeats: only its last entry stores
                    const int col_next = __shfl(col[u], (lane + G) & 63);
                    last = e == per - 1 || col_next != col[u];
                }
            }
            if (col[u] >= 0 && last) {                // one lane per distinct column and group: plain read-add-write
                float *a = acc + col[u] * G + c;
                if constexpr (VEC == 4) { a[0] += v[u].v.x; a[CG] += v[u].v.y; a[2 * CG] += v[u].v.z; a[3 * CG] += v[u].v.w; }
                else a[0] += v[u].v;
            }
        }
    }
    fg_wave_lds_sync();
    // groups of this range that exist: the last range may hold fewer than C columns
    const int c0 = range << log_c;
    const int n_here = slot >= 0 ? CG : min(1 << log_c, n_cols - c0) * G;
    float *dst = slot >= 0 ? partials + (size_t)slot * partial_floats : out + (size_t)c0 * G * VEC;
    for (int i = lane; i < n_here; i += 64) {
        fg_vec<VEC> r;
        if constexpr (VEC == 4) r.v = make_float4(acc[i], acc[i + CG], acc[i + 2 * CG], acc[i + 3 * CG]);
        else r.v = acc[i];
        r.store(dst + (size_t)i * VEC);
    }
}

// out[columns of a cut range] = its partial results added in task order
template <int VEC>
__global__ __launch_bounds__(256) void colsum_merge_kernel(const fgnn_split *__restrict__ merges, int log_c, int n_cols, int G,
                                                           const float *__restrict__ partials, size_t partial_floats, float *__restrict__ out)
{
    const fgnn_split m = merges[blockIdx.x];
    const int c0 = m.row << log_c;
    const int n_here = min(1 << log_c, n_cols - c0) * G;
    const int i = (int)(blockIdx.y * 256 + threadIdx.x);
    if (i >= n_here) return;
    fg_vec<VEC> s;
    s.load(partials + (size_t)m.first_slot * partial_floats + (size_t)i * VEC);
    for (int k = 1; k < m.nseg; ++k) {
        fg_vec<VEC> t;
        t.load(partials + (size_t)(m.first_slot + k) * partial_floats + (size_t)i * VEC);
        s.add(t);
    }
    s.store(out + ((size_t)c0 * G + i) * VEC);
}

extern "C" int fgnn_edge_colsum(const fgnn_colsum_plan_t *p, int W, const float *g, float *out, void *workspace, size_t workspace_bytes,
                                void *stream)
{
    FGNN_REQUIRE(p, FGNN_ERR_NULL, "fgnn_edge_colsum: NULL plan");
    FGNN_REQUIRE(W >= 1, FGNN_ERR_SHAPE, "fgnn_edge_colsum: W=%d", W);
    FGNN_REQUIRE((out || p->n_cols == 0) && (g || p->n_edges == 0), FGNN_ERR_NULL, "fgnn_edge_colsum: NULL argument");
    if (p->n_cols == 0) return 0;
    const bool vec4 = W % 4 == 0 && fgnn_aligned16(g) && fgnn_aligned16(out) && fgnn_aligned16(workspace);
    const int G = vec4 ? W / 4 : W, VEC = vec4 ? 4 : 1;
    FGNN_REQUIRE(G <= 64, FGNN_ERR_LIMIT, "fgnn_edge_colsum: W=%d unsupported (at most 64 floats, or 256 in multiples of four on 16-byte aligned arrays)", W);
    const size_t lds = ((size_t)G << p->log_c) * VEC * sizeof(float);
    FGNN_REQUIRE(lds <= CS_MAX_LDS, FGNN_ERR_LIMIT, "fgnn_edge_colsum: the plan was built for narrower entries (W=%d needs %zu bytes of accumulators)", W, lds);
    const size_t pf = cs_partial_floats(p, W);
    const size_t need = fgnn_colsum_workspace_bytes(p, W);
    FGNN_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), FGNN_ERR_WORKSPACE, "fgnn_edge_colsum: workspace %zu < %zu bytes", workspace_bytes, need);
    hipStream_t st = (hipStream_t)stream;
    float *part = (float *)workspace;
    int per = 1;
    while (per * 2 * G <= 64) per *= 2;
    if (vec4)
        hipLaunchKernelGGL((colsum_kernel<4, 8>), dim3((unsigned)p->n_tasks), dim3(64), lds, st, p->tasks_dev, p->log_c, p->n_cols, G, per, p->tpos_dev,
                           p->lcol_dev, g, out, part, pf);
    else
        hipLaunchKernelGGL((colsum_kernel<1, 8>), dim3((unsigned)p->n_tasks), dim3(64), lds, st, p->tasks_dev, p->log_c, p->n_cols, G, per, p->tpos_dev,
                           p->lcol_dev, g, out, part, pf);
    int rc = fgnn_launch_status("colsum_kernel");
    if (rc || p->n_merge == 0) return rc;
    const dim3 grid((unsigned)p->n_merge, (unsigned)((((size_t)G << p->log_c) + 255) / 256));
    if (vec4)
        hipLaunchKernelGGL(colsum_merge_kernel<4>, grid, dim3(256), 0, st, p->merge_dev, p->log_c, p->n_cols, G, part, pf, out);
    else
        hipLaunchKernelGGL(colsum_merge_kernel<1>, grid, dim3(256), 0, st, p->merge_dev, p->log_c, p->n_cols, G, part, pf, out);
    return fgnn_launch_status("colsum_merge_kernel");
}
