// Weighted gather-and-sum kernels that share the row engine of the fused GAT kernels:
//   multi-head SpMM with stored edge weights (mhspmm / spmm of the reference),
//   GMMConv forward (Gaussian mixture weights computed on the fly, src/fused_gmmconv/gmmconv.cu:48-80),
//   GMMConv backward in one pass over the CSC arrays, and the standalone Gaussian kernels.
#include <algorithm>
#include "fgnn_common.h"

struct SpmmP {
    const fgnn_item *items; int n_items;
    const int *ptr; const int *idx; const int *pos;      // pos: caller's edge position of entry q of idx (NULL = q)
    const int *pos_map;
    const float *feat; float *out; float *part;
    int N, H, F, HF;
    int sum_h;      // != 0: out is [N,F], the sum over the H heads (GMMConv's .sum(1) fused into the store)
    const float *bias; const float *res;     // with sum_h: out[i,:] += bias[:] (+ res[i,:]) in the same store (either may be NULL)
    int own_order;  // != 0: per-edge arrays are indexed by the work list's own entry positions (pos is not applied)
    int ld, ldo;    // floats between consecutive rows of feat / of out when they are views of wider arrays (0: HF)
    int scr_floats; // LDS floats per wave behind the staged weights (the sum over heads in the store): set by spmm_launch
};
__host__ __device__ static inline int spmm_pw(int HF) { return (HF + 3) & ~3; }

// Gaussian mixture weight of one edge for kernel k: exp(-0.5 sum_d ((ps[d]-mu[k,d])*isg[k,d])^2).  The
// first GMM_PV pseudo-coordinates of the edge are fetched once, up front and together (pv); fetched
// inside the k / d loops every one of them would be a separate round trip to memory.
#define GMM_PV 4
__device__ __forceinline__ void gmm_load_pseudo(const float *ps, int dim, float (&pv)[GMM_PV])
{
#pragma unroll
    for (int d = 0; d < GMM_PV; ++d) pv[d] = d < dim ? ps[d] : 0.f;
}
__device__ __forceinline__ float gmm_weight(const float (&pv)[GMM_PV], const float *ps, const float *mu_k, const float *isg_k, int dim)
{
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < GMM_PV; ++d) {
        if (d < dim) { float t = (pv[d] - mu_k[d]) * isg_k[d]; acc = fmaf(t, t, acc); }
    }
    for (int d = GMM_PV; d < dim; ++d) { float t = (ps[d] - mu_k[d]) * isg_k[d]; acc = fmaf(t, t, acc); }
    return __expf(-0.5f * acc);
}

// Final store of an accumulated row: either the [H,F] row itself or, with sum_h, its sum over heads.
// scr: wave-private LDS of HF floats (only touched with sum_h).
template <int VEC, int R, bool FULL>
__device__ __forceinline__ void spmm_store_row(const SpmmP &p, int row, const fg_lanemap<VEC, R> &lm, fg_vec<VEC> (&T)[R], float *scr)
{
    if (!p.sum_h) {
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (FULL || lm.ok[r]) T[r].store_nt(p.out + (size_t)row * p.ldo + lm.eoff[r]);
        return;
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
        if (FULL || lm.ok[r]) T[r].store(scr + lm.eoff[r]);
    fg_wave_lds_sync();
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if ((FULL || lm.ok[r]) && lm.eoff[r] < p.F) {
            fg_vec<VEC> acc; acc.zero();
            for (int h = 0; h < p.H; ++h) { fg_vec<VEC> t; t.load(scr + h * p.F + lm.eoff[r]); acc.add(t); }
            // the layer's epilogue (layers/gmmconv_layer.py:69-75 of the reference): residual, then bias
            if (p.res) { fg_vec<VEC> t; t.load(p.res + (size_t)row * p.F + lm.eoff[r]); acc.add(t); }
            if (p.bias) { fg_vec<VEC> t; t.load(p.bias + lm.eoff[r]); acc.add(t); }
            acc.store(p.out + (size_t)row * p.F + lm.eoff[r]);
        }
    }
    fg_wave_lds_sync();
}

// Weight sources.  fill() runs with lanes-as-edges: lane t writes wl[h*64 + t] for every head.
struct WAtt {
    const float *att;   // [E,H] or NULL (all ones)
    int ld;             // floats between consecutive entries of att (H, or more when att is a view of a wider array)
    bool vec4;          // H % 4 == 0, ld % 4 == 0 and att 16-byte aligned: an entry's weights load as 128-bit words
    __device__ __forceinline__ void prepare(float *, int, int) const {}
    __device__ __forceinline__ void fill(float *wl, const float *, int lane, size_t pos, bool ok, int H) const
    {
        if (att && vec4) {
            // one 128-bit load per four heads instead of four strided 32-bit ones: the entry positions of a chunk are
            // scattered wherever the work list reorders a row, and each instruction costs a pass of the address unit
            const float4 *src = reinterpret_cast<const float4 *>(att + pos * ld);
            for (int h = 0; h < H; h += 4) {
                const float4 v = ok ? src[h >> 2] : make_float4(0.f, 0.f, 0.f, 0.f);
                wl[h * 64 + lane] = v.x; wl[(h + 1) * 64 + lane] = v.y; wl[(h + 2) * 64 + lane] = v.z; wl[(h + 3) * 64 + lane] = v.w;
            }
            return;
        }
        for (int h = 0; h < H; ++h) wl[h * 64 + lane] = ok ? (att ? att[pos * ld + h] : 1.f) : 0.f;
    }
};
struct WGauss {
    const float *pseudo; const float *mu; const float *isg; float *gauss_out; int dim;
    // stage mu / inv_sigma [K,dim] into workgroup LDS
    __device__ __forceinline__ void prepare(float *shared, int tid, int K) const
    {
        for (int i = tid; i < K * dim; i += FGNN_TPB) { shared[i] = mu[i]; shared[K * dim + i] = isg[i]; }
    }
    __device__ __forceinline__ void fill(float *wl, const float *shared, int lane, size_t pos, bool ok, int K) const
    {
        const float *ps = pseudo + pos * dim;
        float pv[GMM_PV];
        gmm_load_pseudo(ps, dim, pv);
        for (int k = 0; k < K; ++k) {
            float w = gmm_weight(pv, ps, shared + k * dim, shared + K * dim + k * dim, dim);
            wl[k * 64 + lane] = ok ? w : 0.f;
            if (gauss_out && ok) gauss_out[pos * K + k] = w;
        }
    }
};

template <int VEC, int R, bool FULL, class WF>
__global__ __launch_bounds__(FGNN_TPB) void spmm_kernel(SpmmP p, WF wf, int shared_floats)
{
    extern __shared__ float lds[];
    float *shared = lds + FGNN_WPB * (p.H * 64 + p.scr_floats);
    if (shared_floats > 0) {
        wf.prepare(shared, (int)threadIdx.x, p.H);
        __syncthreads();
    }
    int row, b, e, slot;
    if (!fg_get_item(p.items, p.n_items, p.ptr, row, b, e, slot)) return;
    const int lane = fg_lane();
    float *wl = lds + fg_wave() * (p.H * 64 + p.scr_floats);
    float *scr = wl + p.H * 64;
    fg_lanemap<VEC, R> lm;
    lm.init(lane, p.HF, p.F);
    fg_vec<VEC> T[R];
#pragma unroll
    for (int r = 0; r < R; ++r) T[r].zero();
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        bool ok = q < e;
        int cnt = min(64, e - c);
        int qq = ok ? q : c;
        int id = p.idx[qq];
        int orig = p.pos ? p.pos[qq] : qq;
        size_t pos = p.pos_map ? (size_t)p.pos_map[orig] : (size_t)orig;
        wf.fill(wl, shared, lane, pos, ok, p.H);
        fg_wave_lds_sync();
        fg_accum_chunk<VEC, R, FULL>(p.feat, p.ld, id, cnt, wl, lm, T);
        fg_wave_lds_sync();
    }
    if (slot < 0) {
        spmm_store_row<VEC, R, FULL>(p, row, lm, T, scr);
    } else {
        float *dst = p.part + (size_t)slot * spmm_pw(p.HF);
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (FULL || lm.ok[r]) T[r].store_nt(dst + lm.eoff[r]);
    }
}

// The same gather with STORED per-edge weights handled in a pair layout (that of the fused GAT forward): lane
// (u << hp_shift) | h owns (entry u of a batch of U, head h) and alone loads that weight, one 32-bit load per lane and batch
// issued a batch ahead of its use; the feature lanes take the weight of (their entry, their head) with ds_bpermute.  No
// staging of a chunk's weights in LDS and none of its two wave-wide waits per 64 entries.  Needs U << hp_shift <= 64 lanes and
// no sum over heads in the store.
template <int VEC, int R, bool FULL>
__global__ __launch_bounds__(FGNN_TPB) void spmm_pair_kernel(SpmmP p, const float *__restrict__ att, int att_ld, int hp_shift)
{
    int row, b, e, slot;
    if (!fg_get_item(p.items, p.n_items, p.ptr, row, b, e, slot)) return;
    const int lane = fg_lane();
    fg_lanemap<VEC, R> lm;
    lm.init(lane, p.HF, p.F);
    fg_vec<VEC> T[R];
    uint32_t boff[R];
#pragma unroll
    for (int r = 0; r < R; ++r) { T[r].zero(); boff[r] = (uint32_t)((FULL || lm.ok[r]) ? lm.eoff[r] : 0) * 4u; }
    constexpr int U = (R >= 8) ? 1 : 8 / R;          // feature rows in flight per wave
    const int pu = lane >> hp_shift, ph = lane & ((1 << hp_shift) - 1);
    const bool pok = ph < p.H && pu < U;
    const uint32_t row_bytes = (uint32_t)p.ld * 4u;
    for (int c = b; c < e; c += 64) {
        const int q = c + lane, cnt = min(64, e - c), qq = q < e ? q : c;      // lanes past the end repeat a valid entry
        const int idv = p.idx[qq];
        const int orig = p.pos ? p.pos[qq] : qq;
        const int posv = p.pos_map ? p.pos_map[orig] : orig;
        // weight of the lane's pair in the batch that starts at entry t (0 for a slot without an entry); the lane
        // exchange stays outside divergent code
        auto fetch = [&](int t) {
            const int pp = __builtin_amdgcn_ds_bpermute(((t + pu) & 63) << 2, posv);
            float a = 0.f;
            if (pok && t + pu < cnt) a = att[(size_t)(unsigned)pp * att_ld + ph];
            return a;
        };
        float av = fetch(0);
        for (int t = 0; t < cnt; t += U) {
            float an = 0.f;
            if (t + U < cnt) an = fetch(t + U);                                  // wave-uniform
            fg_vec<VEC> ld[U][R];
            uint32_t bo[R];
#pragma unroll
            for (int r = 0; r < R; ++r) bo[r] = fg_pin(boff[r]);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint64_t j = (uint64_t)(uint32_t)__builtin_amdgcn_readlane(idv, (t + u) & 63);      // past the chunk: a valid row, weight 0
                const fg_gptr base = fg_uniform_ptr((const char *)p.feat + j * row_bytes);
#pragma unroll
                for (int r = 0; r < R; ++r) ld[u][r].load_off(base, bo[r]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float a = __int_as_float(__builtin_amdgcn_ds_bpermute(((u << hp_shift) + lm.hd[r]) << 2, __float_as_int(av)));
                    T[r].fma(a, ld[u][r]);
                }
            }
            av = an;
        }
    }
    if (slot < 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (FULL || lm.ok[r]) T[r].store_nt(p.out + (size_t)row * p.ldo + lm.eoff[r]);
    } else {
        float *dst = p.part + (size_t)slot * spmm_pw(p.HF);
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (FULL || lm.ok[r]) T[r].store_nt(dst + lm.eoff[r]);
    }
}

// Rows narrower than a wave take the packed lane layout (fg_packmap): G entries of the row per load
// instruction, one partial sum per lane group, a butterfly over the groups at the end.
template <int G, class WF>
__device__ __forceinline__ void spmm_packed_item(const SpmmP &p, const WF &wf, const float *shared, float *wl, float *scr, int n_head)
{
    int row, b, e, slot;
    if (!fg_get_item(p.items, n_head, p.ptr, row, b, e, slot)) return;
    const int lane = fg_lane();
    fg_packmap<G> pm;
    pm.init(lane, p.HF, p.F);
    fg_vec<4> T;
    T.zero();
    constexpr int U = 8;
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        bool ok = q < e;
        int cnt = min(64, e - c);
        int qq = ok ? q : c;
        int id = p.idx[qq];
        int orig = p.pos ? p.pos[qq] : qq;
        size_t pos = p.pos_map ? (size_t)p.pos_map[orig] : (size_t)orig;
        wf.fill(wl, shared, lane, pos, ok, p.H);
        fg_wave_lds_sync();
        for (int t = 0; t < cnt; t += U * G) {
            fg_vec<4> ld[U];
            float w[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + pm.grp;
                const bool live = ei < cnt && pm.ok;
                const int rid = __builtin_amdgcn_ds_bpermute((ei & 63) << 2, id);
                w[u] = live ? wl[pm.hd * 64 + ei] : 0.f;
                if (live) ld[u].load(p.feat + (size_t)rid * (size_t)p.ld + pm.eoff); else ld[u].zero();
            }
#pragma unroll
            for (int u = 0; u < U; ++u) T.fma(w[u], ld[u]);
        }
        fg_wave_lds_sync();
    }
    fg_pack_reduce<G>(T, lane);
    fg_lanemap<4, 1> lm;
    lm.eoff[0] = pm.eoff; lm.hd[0] = pm.hd; lm.ok[0] = pm.ok && pm.grp == 0;
    fg_vec<4> Ts[1] = {T};
    if (slot < 0) {
        spmm_store_row<4, 1, false>(p, row, lm, Ts, scr);
    } else if (lm.ok[0]) {
        T.store_nt(p.part + (size_t)slot * spmm_pw(p.HF) + pm.eoff);
    }
}

// The same with the lane groups on DIFFERENT work items (fg_group_slot): group g walks its own item 64/G entries at a time
// (its lanes stage the weights of those entries), four gathered rows of the group in flight, and stores its own row; nothing
// is combined at the end.  For lists of short items: with a wave per item, a dozen entries fill a fraction of the 8*G load
// slots of a batch.  scr: 256 floats per wave (a row per group) when the store sums over the heads.
template <int G, class WF>
__device__ __forceinline__ void spmm_packed_group_items(const SpmmP &p, const WF &wf, const float *shared, float *wl, float *scr, int bucketed,
                                                        int first, int w)
{
    constexpr int LPR = 64 / G, U = 4;
    const int lane = fg_lane();
    fg_packmap<G> pm;
    pm.init(lane, p.HF, p.F);
    const int sl = lane & (LPR - 1), gbase = lane - sl;
    const int it = fg_group_slot(G, pm.grp, bucketed, first, w);
    int row = -1, b = 0, e = 0, slot = -1;
    if (it < p.n_items) {
        if (p.items) { const fgnn_item q = p.items[it]; row = q.row; b = q.begin; e = q.end; slot = q.slot; }
        else { row = it; b = p.ptr[it]; e = p.ptr[it + 1]; }
    }
    if (row < 0) { b = 0; e = 0; }                      // padding item or past the list: nothing to walk or store
    if (__builtin_amdgcn_ballot_w64(row >= 0) == 0ull) return;
    fg_vec<4> T;
    T.zero();
    for (int c = b; __builtin_amdgcn_ballot_w64(c < e) != 0ull; c += LPR) {
        const bool ok = c + sl < e;
        const int cnt = min(LPR, e - c);                // <= 0: this group is done
        int id = 0;
        size_t pos = 0;                                 // idle lanes and finished groups name entry 0 (there is one: some group has entries)
        if (c < e) {
            const int qq = ok ? c + sl : c;
            id = p.idx[qq];
            const int orig = p.pos ? p.pos[qq] : qq;
            pos = p.pos_map ? (size_t)p.pos_map[orig] : (size_t)orig;
        }
        wf.fill(wl, shared, lane, pos, ok, p.H);
        fg_wave_lds_sync();
        for (int t = 0; __builtin_amdgcn_ballot_w64(t < cnt) != 0ull; t += U) {
            fg_vec<4> ld[U];
            float wv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u, src = gbase + (ei & (LPR - 1));
                const bool live = ei < cnt && pm.ok;
                const int rid = __builtin_amdgcn_ds_bpermute(src << 2, id);
                wv[u] = live ? wl[pm.hd * 64 + src] : 0.f;
                if (live) ld[u].load(p.feat + (size_t)rid * (size_t)p.ld + pm.eoff); else ld[u].zero();
            }
#pragma unroll
            for (int u = 0; u < U; ++u) T.fma(wv[u], ld[u]);
        }
        fg_wave_lds_sync();
    }
    const bool mine = pm.ok && row >= 0;
    if (slot >= 0) {
        if (mine) T.store_nt(p.part + (size_t)slot * spmm_pw(p.HF) + pm.eoff);
    } else if (!p.sum_h) {
        if (mine) T.store_nt(p.out + (size_t)row * p.ldo + pm.eoff);
    }
    if (p.sum_h) {                                      // as spmm_store_row, a row of scratch per group
        float *sg = scr + pm.grp * (LPR * 4);
        if (pm.ok) T.store(sg + pm.eoff);
        fg_wave_lds_sync();
        if (mine && slot < 0 && pm.eoff < p.F) {
            fg_vec<4> acc; acc.zero();
            for (int h = 0; h < p.H; ++h) { fg_vec<4> t; t.load(sg + h * p.F + pm.eoff); acc.add(t); }
            if (p.res) { fg_vec<4> t; t.load(p.res + (size_t)row * p.F + pm.eoff); acc.add(t); }
            if (p.bias) { fg_vec<4> t; t.load(p.bias + pm.eoff); acc.add(t); }
            acc.store(p.out + (size_t)row * p.F + pm.eoff);
        }
        fg_wave_lds_sync();
    }
}

template <int G, class WF>
__global__ __launch_bounds__(FGNN_TPB) void spmm_packed_kernel(SpmmP p, WF wf, int shared_floats)
{
    extern __shared__ float lds[];
    float *shared = lds + FGNN_WPB * (p.H * 64 + p.scr_floats);
    if (shared_floats > 0) {
        wf.prepare(shared, (int)threadIdx.x, p.H);
        __syncthreads();
    }
    float *wl = lds + fg_wave() * (p.H * 64 + p.scr_floats);
    spmm_packed_item<G, WF>(p, wf, shared, wl, wl + p.H * 64, p.n_items);
}
// One launch for a list with a long head: the first head_blocks workgroups put a wave on each of the `first` leading items,
// the others give every lane group an item of the rest, so the long items run beside the short ones.
template <int G, class WF>
__global__ __launch_bounds__(FGNN_TPB) void spmm_packed_mixed_kernel(SpmmP p, WF wf, int shared_floats, int bucketed, int first, unsigned head_blocks)
{
    extern __shared__ float lds[];
    float *shared = lds + FGNN_WPB * (p.H * 64 + p.scr_floats);
    if (shared_floats > 0) {
        wf.prepare(shared, (int)threadIdx.x, p.H);
        __syncthreads();
    }
    float *wl = lds + fg_wave() * (p.H * 64 + p.scr_floats);
    if (blockIdx.x < head_blocks) spmm_packed_item<G, WF>(p, wf, shared, wl, wl + p.H * 64, first);
    else spmm_packed_group_items<G, WF>(p, wf, shared, wl, wl + p.H * 64, bucketed, first, (int)(blockIdx.x - head_blocks));
}

template <int VEC, int R>
__global__ __launch_bounds__(FGNN_TPB) void spmm_merge_kernel(SpmmP p, const fgnn_split *split, int n_split)
{
    extern __shared__ float lds[];
    int w = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (w >= n_split) return;
    fgnn_split sp = split[w];
    const int row = fg_uni(sp.row), first = fg_uni(sp.first_slot), nseg = fg_uni(sp.nseg);
    fg_lanemap<VEC, R> lm;
    lm.init(fg_lane(), p.HF, p.F);
    const int pw = spmm_pw(p.HF);
    fg_vec<VEC> T[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        T[r].zero();
        if (!lm.ok[r]) continue;
        for (int g = 0; g < nseg; ++g) { fg_vec<VEC> t; t.load(p.part + (size_t)(first + g) * pw + lm.eoff[r]); T[r].add(t); }
    }
    spmm_store_row<VEC, R, false>(p, row, lm, T, lds + fg_wave() * pw);
}


static int spmm_checks(const char *fn, int N, int64_t E, int H, int F, const fgnn_schedule_t *sched, const int32_t *ptr, const int32_t *idx)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1 && F >= 1, FGNN_ERR_SHAPE, "%s: bad sizes N=%d E=%lld H=%d F=%d", fn, N, (long long)E, H, F);
    FGNN_REQUIRE(E <= 2147483647LL, FGNN_ERR_LIMIT, "%s: E=%lld exceeds int32 positions", fn, (long long)E);
    FGNN_REQUIRE(H <= 64 && F <= 1024, FGNN_ERR_LIMIT, "%s: H=%d, F=%d unsupported (at most 64 heads of at most 1024 floats)", fn, H, F);
    if (sched) {
        FGNN_REQUIRE(sched->ptr_dev == ptr && sched->n_rows == N && sched->n_edges == E, FGNN_ERR_SCHEDULE,
                     "%s: schedule was built for another pointer array", fn);
        FGNN_REQUIRE(sched->n_buckets == 0 || sched->idx_src_dev == idx, FGNN_ERR_SCHEDULE,
                     "%s: XCD-aware schedule was built from another index array", fn);
        FGNN_REQUIRE(fgnn_sched_has_pos(sched), FGNN_ERR_SCHEDULE, "%s: the schedule was built without edge positions", fn);
    }
    return 0;
}

// pair_att != NULL: stored weights [*, pair_ld] that the pair-layout kernel reads itself where its lane budget allows
template <class WF>
static int spmm_launch(const char *name, SpmmP p, WF wf, int shared_floats, const fgnn_schedule_t *sched, bool aligned,
                       void *workspace, size_t workspace_bytes, hipStream_t st, const float *pair_att = nullptr, int pair_ld = 0)
{
    fgnn_rowcfg cfg;
    FGNN_REQUIRE(fgnn_pick_rowcfg(p.HF, p.F, aligned && fgnn_aligned16(workspace), &cfg), FGNN_ERR_LIMIT, "%s: unsupported row width %d", name, p.HF);
    p.items = sched ? sched->items_dev : nullptr;
    p.n_items = sched ? sched->n_items : p.N;
    p.idx = fgnn_sched_idx(sched, p.idx);
    p.pos = p.own_order ? nullptr : fgnn_sched_pos(sched);
    p.part = (float *)workspace;
    if (p.ld == 0) p.ld = p.HF;
    if (p.ldo == 0) p.ldo = p.HF;
    if (sched && sched->n_partials > 0) {
        size_t need = (size_t)sched->n_partials * spmm_pw(p.HF) * sizeof(float);
        FGNN_REQUIRE(workspace && workspace_bytes >= need, FGNN_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", name, workspace_bytes, need);
    }
    if (p.n_items == 0) return 0;
    const unsigned grid = (unsigned)((p.n_items + FGNN_WPB - 1) / FGNN_WPB);
    const int pack = fgnn_pick_pack(cfg.vec, p.HF);
    // rows of at most 64 floats on graphs of short rows: the items behind the long head of the list go `pack` to a wave
    // (spmm_packed_group_items; MoNet's 2 x 16 forward at 2.4 M nodes x 26 entries per row: 2.18 -> 0.94 ms)
    const int first = (pack >= 4 && sched && sched->n_edges < 256 * (int64_t)sched->n_rows) ? sched->n_wave_slots : p.n_items;
    const int bucketed = sched && sched->n_buckets > 0;
    const unsigned head_blocks = (unsigned)((first + FGNN_WPB - 1) / FGNN_WPB);
    const unsigned grid_mixed = head_blocks + fgnn_group_item_grid(p.n_items - first, pack, bucketed);
    p.scr_floats = p.sum_h ? (first < p.n_items ? 256 : spmm_pw(p.HF)) : 0;
    const size_t shm = ((size_t)FGNN_WPB * (p.H * 64 + p.scr_floats) + shared_floats) * sizeof(float);
    const size_t shm_merge = p.sum_h ? (size_t)FGNN_WPB * spmm_pw(p.HF) * sizeof(float) : 0;
    FGNN_REQUIRE(shm <= 64 * 1024, FGNN_ERR_LIMIT, "%s: H=%d needs %zu bytes of LDS per workgroup (limit 64 KiB)", name, p.H, shm);
    return fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
        if (pack == 8 && first < p.n_items) hipLaunchKernelGGL((spmm_packed_mixed_kernel<8, WF>), dim3(grid_mixed), dim3(FGNN_TPB), shm, st, p, wf, shared_floats, bucketed, first, head_blocks);
        else if (pack == 4 && first < p.n_items) hipLaunchKernelGGL((spmm_packed_mixed_kernel<4, WF>), dim3(grid_mixed), dim3(FGNN_TPB), shm, st, p, wf, shared_floats, bucketed, first, head_blocks);
        else if (pack == 8) hipLaunchKernelGGL((spmm_packed_kernel<8, WF>), dim3(grid), dim3(FGNN_TPB), shm, st, p, wf, shared_floats);
        else if (pack == 4) hipLaunchKernelGGL((spmm_packed_kernel<4, WF>), dim3(grid), dim3(FGNN_TPB), shm, st, p, wf, shared_floats);
        else if (pack == 2) hipLaunchKernelGGL((spmm_packed_kernel<2, WF>), dim3(grid), dim3(FGNN_TPB), shm, st, p, wf, shared_floats);
        else {
            constexpr int U = (R >= 8) ? 1 : 8 / R;
            int hp_shift = 0;
            while ((1 << hp_shift) < p.H) ++hp_shift;
            if (pair_att && !p.sum_h && (U << hp_shift) <= 64)
                hipLaunchKernelGGL((spmm_pair_kernel<VEC, R, FULL>), dim3(grid), dim3(FGNN_TPB), 0, st, p, pair_att, pair_ld, hp_shift);
            else
                hipLaunchKernelGGL((spmm_kernel<VEC, R, FULL, WF>), dim3(grid), dim3(FGNN_TPB), shm, st, p, wf, shared_floats);
        }
        int rc = fgnn_launch_status(name);
        if (rc) return rc;
        if (sched && sched->n_split > 0) {
            unsigned g2 = (unsigned)((sched->n_split + FGNN_WPB - 1) / FGNN_WPB);
            hipLaunchKernelGGL((spmm_merge_kernel<VEC, R>), dim3(g2), dim3(FGNN_TPB), shm_merge, st, p, sched->split_dev, sched->n_split);
            return fgnn_launch_status("spmm_merge_kernel");
        }
        return 0;
    });
}

static size_t spmm_partial_bytes(const fgnn_schedule_t *sched, int H, int F)
{
    return sched ? (((size_t)sched->n_partials * spmm_pw(H * F) * sizeof(float) + 255) & ~(size_t)255) : 0;
}

// The per-edge weights of an XCD-aware list sit at scattered positions (a row's entries are regrouped by source bucket).
// With H % 4 == 0 a lane fetches the H weights of its entry as H / 4 128-bit words straight from there (115 M edges, 8 heads:
// 8.1 ms, against 8.3 ms with the weights first copied into list order and 11.1 ms with eight 32-bit loads per lane; loads
// marked nontemporal: 8.9 ms, the four entries of a 128-byte line are wanted by neighbouring lanes); other head counts
// above two take the copy, whose gather pass then streams the weights.
static inline bool spmm_att_wants_copy(int H) { return H % 4 != 0 && H > 2; }

extern "C" size_t fgnn_mhspmm_workspace_bytes(const fgnn_schedule_t *sched, int H, int F)
{
    // partial results of the split rows, and for an XCD-aware work list room for the weights in the list's entry order
    // where they cannot be read as 128-bit words
    size_t own = (sched && sched->n_buckets > 0 && sched->bpos_dev && spmm_att_wants_copy(H)) ? (size_t)sched->n_edges * H * sizeof(float) : 0;
    return spmm_partial_bytes(sched, H, F) + own;
}

// own[q, :] = att[map(pos[q]), :]: the per-edge weights copied into the entry order of an XCD-aware work list, so that the
// gather pass streams them.  Read through `pos` inside that pass, the eight source buckets of a row are eight workgroups on
// eight XCDs that each pull every 128-byte line of the row's weights for a quarter of its bytes (measured at 115 M edges,
// 8 heads: 70.6 GB moved, 35 GB of it weights, 11.2 ms; the bare gather moves 39 GB in 5.6 ms).  Here a workgroup takes a
// run of ATT_RUN consecutive entries and workgroup w the run (w mod 8) * runs_per_xcd + w / 8: an XCD works through one
// contiguous eighth of the list, so the bucket runs of a row follow each other on the same L2 and its lines are fetched once.
#define ATT_RUN 2048
template <int VEC>
__global__ __launch_bounds__(256) void att_own_order_kernel(int64_t E, int H, int64_t runs_per_xcd, const int *__restrict__ pos,
                                                            const int *__restrict__ pos_map, const float *__restrict__ att,
                                                            float *__restrict__ own)
{
    const int64_t run = (int64_t)(blockIdx.x % FGNN_NUM_XCD) * runs_per_xcd + blockIdx.x / FGNN_NUM_XCD;
    const int64_t q0 = run * ATT_RUN;
    if (blockIdx.x / FGNN_NUM_XCD >= runs_per_xcd || q0 >= E) return;
    const unsigned uh = (unsigned)H / VEC;                              // groups of VEC floats per entry
    const unsigned n = (unsigned)(min(q0 + ATT_RUN, E) - q0) * uh;      // groups of this run (< 2^17)
    for (unsigned k = threadIdx.x; k < n; k += 256) {
        const unsigned dq = k / uh, g = k - dq * uh;
        int o = pos[q0 + dq];
        if (pos_map) o = pos_map[o];
        fg_vec<VEC> v;
        v.load(att + ((size_t)(unsigned)o * uh + g) * VEC);
        v.store_nt(own + ((size_t)(q0 + dq) * uh + g) * VEC);
    }
}

extern "C" int fgnn_mhspmm(int N, int64_t E, int H, int F, const int32_t *ptr, const int32_t *idx, const int32_t *pos_map,
                           const float *att, const float *feat, float *out, const fgnn_schedule_t *sched, void *workspace,
                           size_t workspace_bytes, void *stream)
{
    int rc = spmm_checks("fgnn_mhspmm", N, E, H, F, sched, ptr, idx);
    if (rc) return rc;
    FGNN_REQUIRE(ptr && (idx || E == 0) && feat && out, FGNN_ERR_NULL, "fgnn_mhspmm: NULL argument");
    const float *att_use = att;
    int own_order = 0;
    hipStream_t st = (hipStream_t)stream;
    const size_t part_bytes = spmm_partial_bytes(sched, H, F), own_bytes = (size_t)E * H * sizeof(float);
    if (att && E > 0 && spmm_att_wants_copy(H) && sched && sched->n_buckets > 0 && sched->bpos_dev && workspace && workspace_bytes >= part_bytes + own_bytes) {
        float *own = (float *)((char *)workspace + part_bytes);
        const int64_t runs = (E + ATT_RUN - 1) / ATT_RUN, runs_per_xcd = (runs + FGNN_NUM_XCD - 1) / FGNN_NUM_XCD;
        const dim3 grid((unsigned)(runs_per_xcd * FGNN_NUM_XCD));
        if (H % 4 == 0 && fgnn_aligned16(att) && fgnn_aligned16(own))
            hipLaunchKernelGGL(att_own_order_kernel<4>, grid, dim3(256), 0, st, E, H, runs_per_xcd, sched->bpos_dev, pos_map, att, own);
        else
            hipLaunchKernelGGL(att_own_order_kernel<1>, grid, dim3(256), 0, st, E, H, runs_per_xcd, sched->bpos_dev, pos_map, att, own);
        rc = fgnn_launch_status("att_own_order_kernel");
        if (rc) return rc;
        att_use = own;
        pos_map = nullptr;
        own_order = 1;              // the weights are indexed by the list's own entry positions
    }
    // Rows of more than 1024 floats (the reference serves any number of heads of up to 1024 floats each,
    // src/fused_gat/fused_gat_SM.cu:518-522) go in passes over groups of heads: heads are independent, a pass
    // works on a view of `hg` heads of the wide arrays (same row strides, shifted base).
    const int hmax = (int64_t)H * F <= 1024 ? H : std::max(1, 1024 / F);
    for (int h0 = 0; h0 < H; h0 += hmax) {
        const int hg = std::min(hmax, H - h0);
        SpmmP p{};
        p.ptr = ptr; p.idx = idx; p.pos_map = pos_map; p.feat = feat + (size_t)h0 * F; p.out = out + (size_t)h0 * F;
        p.N = N; p.H = hg; p.F = F; p.HF = hg * F; p.ld = p.ldo = H * F; p.own_order = own_order;
        WAtt wf{att_use ? att_use + h0 : nullptr, H, att_use && H % 4 == 0 && hg % 4 == 0 && h0 % 4 == 0 && fgnn_aligned16(att_use)};
        rc = spmm_launch("fgnn_mhspmm", p, wf, 0, sched, fgnn_aligned16(feat) && fgnn_aligned16(out) && (hmax == H || F % 4 == 0), workspace,
                         workspace_bytes, st, wf.att, H);
        if (rc) return rc;
    }
    return 0;
}

extern "C" size_t fgnn_gmm_forward_workspace_bytes(const fgnn_schedule_t *sched, int K, int F)
{
    return spmm_partial_bytes(sched, K, F);
}

static int gmm_forward_shared(int N, int K, int dim, int F, const int32_t *ptr, const int32_t *idx, const int32_t *pos_map, const float *feat,
                              const float *pseudo, const float *mu, const float *isg, float *out, const fgnn_schedule_t *sched,
                              void *workspace, size_t workspace_bytes, hipStream_t st);

extern "C" int fgnn_gmm_forward(int N, int64_t E, int K, int dim, int F, const int32_t *ptr, const int32_t *idx,
                                const int32_t *pos_map, const float *node_feat, const float *pseudo, const float *mu,
                                const float *inv_sigma, float *out, float *gauss_out, int sum_kernels,
                                const fgnn_schedule_t *sched, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = spmm_checks("fgnn_gmm_forward", N, E, K, F, sched, ptr, idx);
    if (rc) return rc;
    FGNN_REQUIRE((int64_t)K * F <= 1024, FGNN_ERR_LIMIT, "fgnn_gmm_forward: K*F=%lld > 1024 unsupported", (long long)K * F);
    FGNN_REQUIRE(dim >= 1 && dim <= 64 && K * dim <= 1024, FGNN_ERR_LIMIT, "fgnn_gmm_forward: dim=%d K*dim=%d unsupported", dim, K * dim);
    FGNN_REQUIRE(ptr && (idx || E == 0) && node_feat && (pseudo || E == 0) && mu && inv_sigma && out, FGNN_ERR_NULL, "fgnn_gmm_forward: NULL argument");
    FGNN_REQUIRE(sum_kernels >= 0 && sum_kernels <= 2, FGNN_ERR_SHAPE, "fgnn_gmm_forward: sum_kernels=%d (0, 1 or 2)", sum_kernels);
    if (sum_kernels == 2) {
        FGNN_REQUIRE(!gauss_out, FGNN_ERR_SHAPE, "fgnn_gmm_forward: gauss_out is not available with shared node features");
        return gmm_forward_shared(N, K, dim, F, ptr, idx, pos_map, node_feat, pseudo, mu, inv_sigma, out, sched, workspace, workspace_bytes,
                                  (hipStream_t)stream);
    }
    SpmmP p{};
    p.ptr = ptr; p.idx = idx; p.pos_map = pos_map; p.feat = node_feat; p.out = out; p.N = N; p.H = K; p.F = F; p.HF = K * F;
    p.sum_h = sum_kernels;
    WGauss wf{pseudo, mu, inv_sigma, gauss_out, dim};
    return spmm_launch("fgnn_gmm_forward", p, wf, 2 * K * dim, sched, fgnn_aligned16(node_feat) && fgnn_aligned16(out), workspace,
                       workspace_bytes, (hipStream_t)stream);
}

// fgnn_gmm_forward with sum_kernels == 1 and the rest of the layer's forward in the store: out[i,:] = sum_k sum_p ... +
// residual[i,:] + bias[:].
extern "C" int fgnn_gmm_forward_epilogue(int N, int64_t E, int K, int dim, int F, const int32_t *ptr, const int32_t *idx,
                                         const int32_t *pos_map, const float *node_feat, const float *pseudo, const float *mu,
                                         const float *inv_sigma, const float *bias, const float *residual, float *out, float *gauss_out,
                                         const fgnn_schedule_t *sched, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = spmm_checks("fgnn_gmm_forward_epilogue", N, E, K, F, sched, ptr, idx);
    if (rc) return rc;
    FGNN_REQUIRE((int64_t)K * F <= 1024, FGNN_ERR_LIMIT, "fgnn_gmm_forward_epilogue: K*F=%lld > 1024 unsupported", (long long)K * F);
    FGNN_REQUIRE(dim >= 1 && dim <= 64 && K * dim <= 1024, FGNN_ERR_LIMIT, "fgnn_gmm_forward_epilogue: dim=%d K*dim=%d unsupported", dim, K * dim);
    FGNN_REQUIRE(ptr && (idx || E == 0) && node_feat && (pseudo || E == 0) && mu && inv_sigma && out, FGNN_ERR_NULL,
                 "fgnn_gmm_forward_epilogue: NULL argument");
    SpmmP p{};
    p.ptr = ptr; p.idx = idx; p.pos_map = pos_map; p.feat = node_feat; p.out = out; p.N = N; p.H = K; p.F = F; p.HF = K * F;
    p.sum_h = 1; p.bias = bias; p.res = residual;
    WGauss wf{pseudo, mu, inv_sigma, gauss_out, dim};
    const bool aligned = fgnn_aligned16(node_feat) && fgnn_aligned16(out) && (!bias || fgnn_aligned16(bias)) && (!residual || fgnn_aligned16(residual));
    return spmm_launch("fgnn_gmm_forward_epilogue", p, wf, 2 * K * dim, sched, aligned, workspace, workspace_bytes, (hipStream_t)stream);
}

// ------------------------------------------------------------------------------- GMM backward
struct GmmBwdP {
    const fgnn_item *items; int n_items;
    const int *ptr; const int *idx; const int *pos; const int *permute;
    const float *x; const float *g; const float *pseudo; const float *mu; const float *isg;
    float *gfeat; float *gww; float *part;      // gww: [E,K] in CSR position order, gw * w per edge and kernel
    int N, K, dim, F, HF;
    int g_stride;   // floats per grad_out row: HF, or F when grad_out is the gradient of the sum over kernels
    int x_stride;   // floats per node_feat row: HF, or F when all mixture kernels share one [N,F] feature matrix
    int lphp;       // > 0: head-aligned lane map with this many lanes per mixture kernel
};

// One pass over CSC column j (x[j] stays in registers): per in-edge gather grad_out[i], accumulate
// w * grad_out[i] into grad_feat[j] and form gw = <grad_out[i,k,:], x[j,k,:]> per mixture kernel
// (DPP butterflies inside head groups).  gw*w is written once per edge at its CSR position; the
// Gaussian derivatives are finished by gauss_grad_kernel below.
template <int VEC, int R, bool FULL, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void gmm_bwd_kernel(GmmBwdP p)
{
    extern __shared__ float lds[];
    const int K = p.K, dim = p.dim, KD = K * dim;
    const int per_wave = K * 64 + 64 * R;
    float *shared = lds + FGNN_WPB * per_wave;          // mu | inv_sigma
    for (int i = (int)threadIdx.x; i < KD; i += FGNN_TPB) { shared[i] = p.mu[i]; shared[KD + i] = p.isg[i]; }
    __syncthreads();
    int col, b, e, slot;
    if (!fg_get_item(p.items, p.n_items, p.ptr, col, b, e, slot)) return;
    const int lane = fg_lane();
    float *wl = lds + fg_wave() * per_wave;
    float *scr = wl + K * 64;
    fg_lanemap<VEC, R> lm;
    if (p.lphp) lm.init_padded(lane, p.K, p.F, p.lphp); else lm.init(lane, p.HF, p.F);
    fg_vec<VEC> T[R], xr[R];
    int goff[R];        // float offset of the lane's slab inside a grad_out row
#pragma unroll
    for (int r = 0; r < R; ++r) {
        T[r].zero();
        if (FULL || lm.ok[r]) xr[r].load(p.x + (size_t)col * p.x_stride + (p.x_stride == p.HF ? lm.eoff[r] : lm.eoff[r] % p.F)); else xr[r].zero();
        goff[r] = (p.g_stride == p.HF) ? lm.eoff[r] : lm.eoff[r] % p.F;
    }
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        bool ok = q < e;
        int cnt = min(64, e - c);
        int qq = ok ? q : c;
        int id = p.idx[qq];
        int posv = p.pos ? p.pos[qq] : qq;
        if (p.permute) posv = p.permute[posv];      // NULL: pseudo and gww are in this pass's own (CSC) order
        // the first rows are requested before the weights are formed: the pseudo-coordinate fetch
        // (itself behind the permute fetch) then overlaps with the row fetches
        constexpr int UG = (R >= 8) ? 1 : 8 / R;
        fg_vec<VEC> ld[UG][R];
        auto request = [&](int t) {
#pragma unroll
            for (int u = 0; u < UG; ++u) {
                int rid = __builtin_amdgcn_readlane(id, (t + u) & 63);
                const float *base = p.g + (size_t)rid * p.g_stride;
#pragma unroll
                for (int r = 0; r < R; ++r) { if (FULL || lm.ok[r]) ld[u][r].load(base + goff[r]); else ld[u][r].zero(); }
            }
        };
        request(0);
        const float *ps = p.pseudo + (size_t)(unsigned)posv * dim;
        float pv[GMM_PV];
        gmm_load_pseudo(ps, dim, pv);
        for (int k = 0; k < K; ++k) wl[k * 64 + lane] = ok ? gmm_weight(pv, ps, shared + k * dim, shared + KD + k * dim, dim) : 0.f;
        fg_wave_lds_sync();
        for (int t = 0; t < cnt; t += UG) {
            if (t > 0) request(t);
#pragma unroll
            for (int u = 0; u < UG; ++u) {
                if (t + u >= cnt) break;
                float *gdst = p.gww + (size_t)(unsigned)__builtin_amdgcn_readlane(posv, t + u) * K;
                float dpart[R], w[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    w[r] = wl[lm.hd[r] * 64 + t + u];
                    T[r].fma(w[r], ld[u][r]);
                    dpart[r] = ld[u][r].dot(xr[r]);
                }
                if constexpr (LPH > 0) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        float sum = fg_group_sum<LPH>(dpart[r]);
                        if ((FULL || lm.ok[r]) && lm.eoff[r] % p.F == 0) __builtin_nontemporal_store(sum * w[r], gdst + lm.hd[r]);
                    }
                } else {
                    float sum = K <= FGNN_FEW_HEADS ? fg_head_reduce_few<VEC, R>(dpart, lm, lane, K)
                                                    : fg_head_reduce<VEC, R>(scr, dpart, lm, lane, K, p.F);
                    if (lane < K) __builtin_nontemporal_store(sum * wl[lane * 64 + t + u], gdst + lane);
                }
            }
        }
        fg_wave_lds_sync();
    }
    float *dst = slot < 0 ? p.gfeat + (size_t)col * p.HF : p.part + (size_t)slot * spmm_pw(p.HF);
#pragma unroll
    for (int r = 0; r < R; ++r)
        if (FULL || lm.ok[r]) T[r].store_nt(dst + lm.eoff[r]);
}

// The same pass for rows narrower than a wave, G column entries per load instruction (see
// spmm_packed_kernel).  Needs F/4 lanes per mixture kernel to be a power of two (LPH > 0).
template <int G, int LPH>
__device__ __forceinline__ void gmm_bwd_packed_item(const GmmBwdP &p, int n_head, float *lds)
{
    const int K = p.K, dim = p.dim, KD = K * dim;
    const int per_wave = K * 64 + 64;
    float *shared = lds + FGNN_WPB * per_wave;          // mu | inv_sigma
    for (int i = (int)threadIdx.x; i < KD; i += FGNN_TPB) { shared[i] = p.mu[i]; shared[KD + i] = p.isg[i]; }
    __syncthreads();
    int col, b, e, slot;
    if (!fg_get_item(p.items, n_head, p.ptr, col, b, e, slot)) return;
    const int lane = fg_lane();
    float *wl = lds + fg_wave() * per_wave;
    fg_packmap<G> pm;
    if (p.lphp) pm.init_padded(lane, p.K, p.F, p.lphp); else pm.init(lane, p.HF, p.F);
    fg_vec<4> T, xr;
    T.zero();
    if (pm.ok) xr.load(p.x + (size_t)col * p.x_stride + (p.x_stride == p.HF ? pm.eoff : pm.eoff % p.F)); else xr.zero();
    const int goff = (p.g_stride == p.HF) ? pm.eoff : pm.eoff % p.F;
    const bool writer = pm.ok && pm.eoff % p.F == 0;
    constexpr int U = 8;
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        bool ok = q < e;
        int cnt = min(64, e - c);
        int qq = ok ? q : c;
        int id = p.idx[qq];
        int posv = p.pos ? p.pos[qq] : qq;
        if (p.permute) posv = p.permute[posv];      // NULL: pseudo and gww are in this pass's own (CSC) order
        const float *ps = p.pseudo + (size_t)(unsigned)posv * dim;
        float pv[GMM_PV];
        gmm_load_pseudo(ps, dim, pv);
        for (int k = 0; k < K; ++k) wl[k * 64 + lane] = ok ? gmm_weight(pv, ps, shared + k * dim, shared + KD + k * dim, dim) : 0.f;
        fg_wave_lds_sync();
        for (int t = 0; t < cnt; t += U * G) {
            fg_vec<4> ld[U];
            int pv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + pm.grp;
                const bool live = ei < cnt && pm.ok;
                const int rid = __builtin_amdgcn_ds_bpermute((ei & 63) << 2, id);
                pv[u] = __builtin_amdgcn_ds_bpermute((ei & 63) << 2, posv);
                if (live) ld[u].load(p.g + (size_t)rid * p.g_stride + goff); else ld[u].zero();
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + pm.grp;
                const bool live = ei < cnt && pm.ok;
                const float w = live ? wl[pm.hd * 64 + ei] : 0.f;
                T.fma(w, ld[u]);
                const float sum = fg_group_sum<LPH>(ld[u].dot(xr));
                if (live && writer) __builtin_nontemporal_store(sum * w, p.gww + (size_t)(unsigned)pv[u] * K + pm.hd);
            }
        }
        fg_wave_lds_sync();
    }
    fg_pack_reduce<G>(T, lane);
    float *dst = slot < 0 ? p.gfeat + (size_t)col * p.HF : p.part + (size_t)slot * spmm_pw(p.HF);
    if (pm.ok && pm.grp == 0) T.store_nt(dst + pm.eoff);
}

// The same with the lane groups on different work items (see spmm_packed_group_items).
template <int G, int LPH>
__device__ __forceinline__ void gmm_bwd_packed_group_items(const GmmBwdP &p, int bucketed, int first, int w, float *lds)
{
    constexpr int LPR = 64 / G, U = 4;
    const int K = p.K, dim = p.dim, KD = K * dim;
    const int per_wave = K * 64 + 64;
    float *shared = lds + FGNN_WPB * per_wave;          // mu | inv_sigma
    for (int i = (int)threadIdx.x; i < KD; i += FGNN_TPB) { shared[i] = p.mu[i]; shared[KD + i] = p.isg[i]; }
    __syncthreads();
    const int lane = fg_lane();
    float *wl = lds + fg_wave() * per_wave;
    fg_packmap<G> pm;
    if (p.lphp) pm.init_padded(lane, p.K, p.F, p.lphp); else pm.init(lane, p.HF, p.F);
    const int sl = lane & (LPR - 1), gbase = lane - sl;
    const int it = fg_group_slot(G, pm.grp, bucketed, first, w);
    int col = -1, b = 0, e = 0, slot = -1;
    if (it < p.n_items) {
        if (p.items) { const fgnn_item q = p.items[it]; col = q.row; b = q.begin; e = q.end; slot = q.slot; }
        else { col = it; b = p.ptr[it]; e = p.ptr[it + 1]; }
    }
    if (col < 0) { b = 0; e = 0; }                      // padding item or past the list: nothing to walk or store
    if (__builtin_amdgcn_ballot_w64(col >= 0) == 0ull) return;
    const bool mine = pm.ok && col >= 0;
    fg_vec<4> T, xr;
    T.zero();
    if (mine) xr.load(p.x + (size_t)col * p.x_stride + (p.x_stride == p.HF ? pm.eoff : pm.eoff % p.F)); else xr.zero();
    const int goff = (p.g_stride == p.HF) ? pm.eoff : pm.eoff % p.F;
    const bool writer = pm.ok && pm.eoff % p.F == 0;
    for (int c = b; __builtin_amdgcn_ballot_w64(c < e) != 0ull; c += LPR) {
        const bool ok = c + sl < e;
        const int cnt = min(LPR, e - c);                // <= 0: this group is done
        int id = 0, posv = 0;
        if (c < e) {
            const int qq = ok ? c + sl : c;             // idle lanes repeat a valid entry
            id = p.idx[qq];
            posv = p.pos ? p.pos[qq] : qq;
            if (p.permute) posv = p.permute[posv];
        }
        if (ok) {
            const float *ps = p.pseudo + (size_t)(unsigned)posv * dim;
            float pv[GMM_PV];
            gmm_load_pseudo(ps, dim, pv);
            for (int k = 0; k < K; ++k) wl[k * 64 + lane] = gmm_weight(pv, ps, shared + k * dim, shared + KD + k * dim, dim);
        } else {
            for (int k = 0; k < K; ++k) wl[k * 64 + lane] = 0.f;
        }
        fg_wave_lds_sync();
        for (int t = 0; __builtin_amdgcn_ballot_w64(t < cnt) != 0ull; t += U) {
            fg_vec<4> ld[U];
            int pe[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u, src = gbase + (ei & (LPR - 1));
                const bool live = ei < cnt && pm.ok;
                const int rid = __builtin_amdgcn_ds_bpermute(src << 2, id);
                pe[u] = __builtin_amdgcn_ds_bpermute(src << 2, posv);
                if (live) ld[u].load(p.g + (size_t)rid * p.g_stride + goff); else ld[u].zero();
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u;
                const bool live = ei < cnt && pm.ok;
                const float wv = live ? wl[pm.hd * 64 + gbase + (ei & (LPR - 1))] : 0.f;
                T.fma(wv, ld[u]);
                const float sum = fg_group_sum<LPH>(ld[u].dot(xr));
                if (live && writer) __builtin_nontemporal_store(sum * wv, p.gww + (size_t)(unsigned)pe[u] * K + pm.hd);
            }
        }
        fg_wave_lds_sync();
    }
    if (!mine) return;
    float *dst = slot < 0 ? p.gfeat + (size_t)col * p.HF : p.part + (size_t)slot * spmm_pw(p.HF);
    T.store_nt(dst + pm.eoff);
}

template <int G, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void gmm_bwd_packed_kernel(GmmBwdP p)
{
    extern __shared__ float lds[];
    gmm_bwd_packed_item<G, LPH>(p, p.n_items, lds);
}
template <int G, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void gmm_bwd_packed_mixed_kernel(GmmBwdP p, int bucketed, int first, unsigned head_blocks)
{
    extern __shared__ float lds[];
    if (blockIdx.x < head_blocks) gmm_bwd_packed_item<G, LPH>(p, first, lds);
    else gmm_bwd_packed_group_items<G, LPH>(p, bucketed, first, (int)(blockIdx.x - head_blocks), lds);
}

// The column pass when grad_out is the gradient of the SUM over the mixture kernels ([N, F], the
// GMMConv layers): the gathered row is the same for every kernel, so the lanes spread over F only
// (LPF = lanes per row, a power of two >= F/4) and keep the K accumulators and the K slices of x[col]
// in registers.  One load instruction then fetches 64/LPF different rows, every lane of it is used,
// and a row is read once instead of once per mixture kernel.  K <= GMM_SUMK_MAX, F % 4 == 0, F <= 256.
// With GWW == false the same loop is the forward of a layer whose K mixture kernels share one [N,F]
// feature matrix (aggregate first, transform afterwards): out[i,k,:] = sum_p w[p,k] * g[idx[p],:], nothing
// per edge is written and x is not read.
#define GMM_SUMK_MAX 4
template <int LPF, bool GWW>
__device__ __forceinline__ void gmm_bwd_sum_item(const GmmBwdP &p, int n_head, float *lds)
{
    constexpr int G = 64 / LPF;         // rows per load instruction
    constexpr int U = G > 8 ? 64 / G : 8;       // load instructions in flight; U * G divides 64
    const int K = p.K, dim = p.dim, KD = K * dim, F = p.F;
    const int per_wave = K * 64;
    float *shared = lds + FGNN_WPB * per_wave;          // mu | inv_sigma
    for (int i = (int)threadIdx.x; i < KD; i += FGNN_TPB) { shared[i] = p.mu[i]; shared[KD + i] = p.isg[i]; }
    __syncthreads();
    int col, b, e, slot;
    if (!fg_get_item(p.items, n_head, p.ptr, col, b, e, slot)) return;
    const int lane = fg_lane();
    float *wl = lds + fg_wave() * per_wave;
    const int grp = lane / LPF, sub = lane % LPF;
    const bool fok = sub * 4 < F;
    const int foff = fok ? sub * 4 : 0;
    fg_vec<4> T[GMM_SUMK_MAX], xr[GMM_SUMK_MAX];
#pragma unroll
    for (int k = 0; k < GMM_SUMK_MAX; ++k) {
        T[k].zero();
        if (GWW && k < K && fok) xr[k].load(p.x + (size_t)col * p.HF + k * F + foff); else xr[k].zero();
    }
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        bool ok = q < e;
        int cnt = min(64, e - c);
        int qq = ok ? q : c;
        int id = p.idx[qq];
        int posv = p.pos ? p.pos[qq] : qq;
        if (p.permute) posv = p.permute[posv];      // NULL: pseudo and gww are in this pass's own (CSC) order
        const float *ps = p.pseudo + (size_t)(unsigned)posv * dim;
        float pv[GMM_PV];
        gmm_load_pseudo(ps, dim, pv);
        for (int k = 0; k < K; ++k) wl[k * 64 + lane] = ok ? gmm_weight(pv, ps, shared + k * dim, shared + KD + k * dim, dim) : 0.f;
        fg_wave_lds_sync();
        for (int t = 0; t < cnt; t += U * G) {
            fg_vec<4> ld[U];
            int pe[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + grp;                     // < 64: U*G divides 64
                const int rid = __builtin_amdgcn_ds_bpermute(ei << 2, id);
                pe[u] = __builtin_amdgcn_ds_bpermute(ei << 2, posv);
                if (ei < cnt && fok) ld[u].load(p.g + (size_t)rid * F + foff); else ld[u].zero();
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + grp;
                float *gdst = p.gww + (size_t)(unsigned)pe[u] * K;
                float mine = 0.f;                                   // lane `sub` of a row keeps the value of kernel `sub`
#pragma unroll
                for (int k = 0; k < GMM_SUMK_MAX; ++k) {
                    if (k < K) {
                        const float w = wl[k * 64 + ei];            // 0 past the end of the chunk
                        T[k].fma(w, ld[u]);
                        if constexpr (GWW) {
                            const float sum = fg_group_sum<LPF>(ld[u].dot(xr[k]));
                            if constexpr (LPF >= GMM_SUMK_MAX) mine = sub == k ? sum * w : mine;
                            else if (ei < cnt && sub == 0) __builtin_nontemporal_store(sum * w, gdst + k);
                        }
                    }
                }
                // the K values of an edge leave with one store instruction, K adjacent lanes writing K adjacent floats
                if constexpr (GWW && LPF >= GMM_SUMK_MAX) { if (ei < cnt && sub < K) __builtin_nontemporal_store(mine, gdst + sub); }
            }
        }
        fg_wave_lds_sync();
    }
    float *dst = slot < 0 ? p.gfeat + (size_t)col * p.HF : p.part + (size_t)slot * spmm_pw(p.HF);
#pragma unroll
    for (int k = 0; k < GMM_SUMK_MAX; ++k) {
        if (k < K) {
            fg_pack_reduce<G>(T[k], lane);
            if (fok && grp == 0) T[k].store_nt(dst + k * F + foff);
        }
    }
}

// The same pass with the lane groups on different work items (fg_group_slot): group g walks its own item LPF entries at a
// time (its LPF lanes compute the weights of LPF entries), min(4, LPF) gathered rows of the group in flight, and writes its
// own result; no butterfly over the groups.
template <int LPF, bool GWW>
__device__ __forceinline__ void gmm_bwd_sum_group_items(const GmmBwdP &p, int bucketed, int first, int w, float *lds)
{
    constexpr int G = 64 / LPF;
    constexpr int U = LPF < 4 ? LPF : 4;
    const int K = p.K, dim = p.dim, KD = K * dim, F = p.F;
    const int per_wave = K * 64;
    float *shared = lds + FGNN_WPB * per_wave;          // mu | inv_sigma
    for (int i = (int)threadIdx.x; i < KD; i += FGNN_TPB) { shared[i] = p.mu[i]; shared[KD + i] = p.isg[i]; }
    __syncthreads();
    const int lane = fg_lane();
    const int grp = lane / LPF, sub = lane % LPF, gbase = lane - sub;
    const int it = fg_group_slot(G, grp, bucketed, first, w);
    int col = -1, b = 0, e = 0, slot = -1;
    if (it < p.n_items) {
        if (p.items) { const fgnn_item q = p.items[it]; col = q.row; b = q.begin; e = q.end; slot = q.slot; }
        else { col = it; b = p.ptr[it]; e = p.ptr[it + 1]; }
    }
    if (col < 0) { b = 0; e = 0; }                      // padding item or past the list: nothing to walk or store
    if (__builtin_amdgcn_ballot_w64(col >= 0) == 0ull) return;
    float *wl = lds + fg_wave() * per_wave;
    const bool fok = sub * 4 < F;
    const int foff = fok ? sub * 4 : 0;
    fg_vec<4> T[GMM_SUMK_MAX], xr[GMM_SUMK_MAX];
#pragma unroll
    for (int k = 0; k < GMM_SUMK_MAX; ++k) {
        T[k].zero();
        if (GWW && k < K && fok && col >= 0) xr[k].load(p.x + (size_t)col * p.HF + k * F + foff); else xr[k].zero();
    }
    for (int c = b; __builtin_amdgcn_ballot_w64(c < e) != 0ull; c += LPF) {
        const bool ok = c + sub < e;
        const int cnt = min(LPF, e - c);                // <= 0: this group is done
        int id = 0, posv = 0;
        if (c < e) {
            const int qq = ok ? c + sub : c;            // idle lanes repeat a valid entry
            id = p.idx[qq];
            posv = p.pos ? p.pos[qq] : qq;
            if (p.permute) posv = p.permute[posv];
        }
        if (ok) {
            const float *ps = p.pseudo + (size_t)(unsigned)posv * dim;
            float pv[GMM_PV];
            gmm_load_pseudo(ps, dim, pv);
            for (int k = 0; k < K; ++k) wl[k * 64 + lane] = gmm_weight(pv, ps, shared + k * dim, shared + KD + k * dim, dim);
        } else {
            for (int k = 0; k < K; ++k) wl[k * 64 + lane] = 0.f;
        }
        fg_wave_lds_sync();
        for (int t = 0; __builtin_amdgcn_ballot_w64(t < cnt) != 0ull; t += U) {
            fg_vec<4> ld[U];
            int pe[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u, src = (gbase + (ei & (LPF - 1))) << 2;
                const int rid = __builtin_amdgcn_ds_bpermute(src, id);
                pe[u] = __builtin_amdgcn_ds_bpermute(src, posv);
                if (ei < cnt && fok) ld[u].load(p.g + (size_t)rid * F + foff); else ld[u].zero();
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u;
                const bool live = ei < cnt;
                float *gdst = p.gww + (size_t)(unsigned)pe[u] * K;
                float mine = 0.f;                                   // lane `sub` of a row keeps the value of kernel `sub`
#pragma unroll
                for (int k = 0; k < GMM_SUMK_MAX; ++k) {
                    if (k < K) {
                        const float w = live ? wl[k * 64 + gbase + (ei & (LPF - 1))] : 0.f;
                        T[k].fma(w, ld[u]);
                        if constexpr (GWW) {
                            const float sum = fg_group_sum<LPF>(ld[u].dot(xr[k]));
                            if constexpr (LPF >= GMM_SUMK_MAX) mine = sub == k ? sum * w : mine;
                            else if (live && sub == 0) __builtin_nontemporal_store(sum * w, gdst + k);
                        }
                    }
                }
                if constexpr (GWW && LPF >= GMM_SUMK_MAX) { if (live && sub < K) __builtin_nontemporal_store(mine, gdst + sub); }
            }
        }
        fg_wave_lds_sync();
    }
    if (col < 0 || !fok) return;
    float *dst = slot < 0 ? p.gfeat + (size_t)col * p.HF : p.part + (size_t)slot * spmm_pw(p.HF);
#pragma unroll
    for (int k = 0; k < GMM_SUMK_MAX; ++k)
        if (k < K) T[k].store_nt(dst + k * F + foff);
}

template <int LPF, bool GWW = true>
__global__ __launch_bounds__(FGNN_TPB) void gmm_bwd_sum_kernel(GmmBwdP p)
{
    extern __shared__ float lds[];
    gmm_bwd_sum_item<LPF, GWW>(p, p.n_items, lds);
}
// One launch for a list with a long head: the first head_blocks workgroups put a wave on each of the `first` leading items,
// the others give every lane group an item of the rest; the long items then run beside the short ones.
template <int LPF, bool GWW = true>
__global__ __launch_bounds__(FGNN_TPB) void gmm_bwd_sum_mixed_kernel(GmmBwdP p, int bucketed, int first, unsigned head_blocks)
{
    extern __shared__ float lds[];
    if (blockIdx.x < head_blocks) gmm_bwd_sum_item<LPF, GWW>(p, first, lds);
    else gmm_bwd_sum_group_items<LPF, GWW>(p, bucketed, first, (int)(blockIdx.x - head_blocks), lds);
}

// Where the lane-group part of a launch starts (-1: a wave per item throughout).  Groups of at most 16 lanes (F <= 64) on
// graphs under 256 entries per row; measured with K = 3 on R-MAT graphs of 14-26 entries per row, column pass / shared-feature
// forward: F = 64 0.329 -> 0.316 / 0.167 -> 0.124 ms at 169 k nodes, 1.35 -> 1.05 / 0.71 -> 0.61 ms at 500 k nodes;
// K = 2, F = 16 0.211 -> 0.174 / 0.132 -> 0.082 ms at 169 k nodes, 5.9 -> 4.6 / 2.3 -> 1.7 ms at 2.4 M nodes; F = 128 (two
// groups of 32 lanes) 9.7 -> 10.1 ms at 2.4 M nodes: not taken.
static inline int gmm_group_items_first(const fgnn_schedule_t *sched, int lpf)
{
    if (!sched || lpf > 16 || sched->n_edges >= 256 * (int64_t)sched->n_rows) return -1;
    return sched->n_wave_slots;
}

template <bool GWW>
static void gmm_sum_launch(int lpf, unsigned grid, size_t shm, hipStream_t st, const GmmBwdP &p, int first = -1, int bucketed = 0)
{
    // first >= 0: the items from slot `first` on are short and go 64/lpf to a wave (gmm_bwd_sum_group_items)
    if (first >= 0 && first < p.n_items && lpf <= 32) {
        const unsigned hb = (unsigned)((first + FGNN_WPB - 1) / FGNN_WPB);
        const unsigned g2 = hb + fgnn_group_item_grid(p.n_items - first, 64 / lpf, bucketed != 0);
        switch (lpf) {
        case 1: hipLaunchKernelGGL((gmm_bwd_sum_mixed_kernel<1, GWW>), dim3(g2), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); break;
        case 2: hipLaunchKernelGGL((gmm_bwd_sum_mixed_kernel<2, GWW>), dim3(g2), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); break;
        case 4: hipLaunchKernelGGL((gmm_bwd_sum_mixed_kernel<4, GWW>), dim3(g2), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); break;
        case 8: hipLaunchKernelGGL((gmm_bwd_sum_mixed_kernel<8, GWW>), dim3(g2), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); break;
        case 16: hipLaunchKernelGGL((gmm_bwd_sum_mixed_kernel<16, GWW>), dim3(g2), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); break;
        default: hipLaunchKernelGGL((gmm_bwd_sum_mixed_kernel<32, GWW>), dim3(g2), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); break;
        }
        return;
    }
    switch (lpf) {
    case 1: hipLaunchKernelGGL((gmm_bwd_sum_kernel<1, GWW>), dim3(grid), dim3(FGNN_TPB), shm, st, p); break;
    case 2: hipLaunchKernelGGL((gmm_bwd_sum_kernel<2, GWW>), dim3(grid), dim3(FGNN_TPB), shm, st, p); break;
    case 4: hipLaunchKernelGGL((gmm_bwd_sum_kernel<4, GWW>), dim3(grid), dim3(FGNN_TPB), shm, st, p); break;
    case 8: hipLaunchKernelGGL((gmm_bwd_sum_kernel<8, GWW>), dim3(grid), dim3(FGNN_TPB), shm, st, p); break;
    case 16: hipLaunchKernelGGL((gmm_bwd_sum_kernel<16, GWW>), dim3(grid), dim3(FGNN_TPB), shm, st, p); break;
    case 32: hipLaunchKernelGGL((gmm_bwd_sum_kernel<32, GWW>), dim3(grid), dim3(FGNN_TPB), shm, st, p); break;
    default: hipLaunchKernelGGL((gmm_bwd_sum_kernel<64, GWW>), dim3(grid), dim3(FGNN_TPB), shm, st, p); break;
    }
}

// Forward with one [N,F] feature matrix shared by the K mixture kernels: out[i,k,:] = sum_p w[p,k] * feat[idx[p],:].
static int gmm_forward_shared(int N, int K, int dim, int F, const int32_t *ptr, const int32_t *idx, const int32_t *pos_map, const float *feat,
                              const float *pseudo, const float *mu, const float *isg, float *out, const fgnn_schedule_t *sched,
                              void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const int HF = K * F, KD = K * dim;
    FGNN_REQUIRE(F % 4 == 0 && F <= 256 && K <= GMM_SUMK_MAX && fgnn_aligned16(feat) && fgnn_aligned16(out), FGNN_ERR_LIMIT,
                 "fgnn_gmm_forward: shared node features need F %% 4 == 0, F <= 256, K <= %d and 16-byte aligned tensors (F=%d, K=%d)",
                 GMM_SUMK_MAX, F, K);
    if (sched && sched->n_partials > 0) {
        size_t need = (size_t)sched->n_partials * spmm_pw(HF) * sizeof(float);
        FGNN_REQUIRE(workspace && workspace_bytes >= need && fgnn_aligned16(workspace), FGNN_ERR_WORKSPACE,
                     "fgnn_gmm_forward: workspace %zu < %zu bytes (or unaligned)", workspace_bytes, need);
    }
    GmmBwdP p{};
    p.items = sched ? sched->items_dev : nullptr; p.n_items = sched ? sched->n_items : N;
    if (p.n_items == 0) return 0;
    p.ptr = ptr; p.idx = fgnn_sched_idx(sched, idx); p.pos = fgnn_sched_pos(sched); p.permute = pos_map;
    p.g = feat; p.pseudo = pseudo; p.mu = mu; p.isg = isg; p.gfeat = out; p.part = (float *)workspace;
    p.N = N; p.K = K; p.dim = dim; p.F = F; p.HF = HF; p.g_stride = F; p.x_stride = HF;
    int lpf = 1;
    while (lpf * 4 < F) lpf *= 2;
    const size_t shm = ((size_t)FGNN_WPB * K * 64 + 2 * KD) * sizeof(float);
    FGNN_REQUIRE(shm <= 64 * 1024, FGNN_ERR_LIMIT, "fgnn_gmm_forward: K=%d, dim=%d need %zu bytes of LDS per workgroup (limit 64 KiB)", K, dim, shm);
    const unsigned grid = (unsigned)((p.n_items + FGNN_WPB - 1) / FGNN_WPB);
    gmm_sum_launch<false>(lpf, grid, shm, st, p, gmm_group_items_first(sched, lpf), sched && sched->n_buckets > 0);
    int rc = fgnn_launch_status("gmm_bwd_sum_kernel (forward, shared features)");
    if (rc) return rc;
    if (sched && sched->n_split > 0) {
        fgnn_rowcfg cfg;
        FGNN_REQUIRE(fgnn_pick_rowcfg(HF, F, true, &cfg), FGNN_ERR_LIMIT, "fgnn_gmm_forward: unsupported row width %d", HF);
        SpmmP mp{};
        mp.part = p.part; mp.out = out; mp.N = N; mp.H = K; mp.F = F; mp.HF = HF; mp.ld = mp.ldo = HF;
        unsigned g2 = (unsigned)((sched->n_split + FGNN_WPB - 1) / FGNN_WPB);
        rc = fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
            hipLaunchKernelGGL((spmm_merge_kernel<VEC, R>), dim3(g2), dim3(FGNN_TPB), 0, st, mp, sched->split_dev, sched->n_split);
            return fgnn_launch_status("spmm_merge_kernel");
        });
    }
    return rc;
}

// Closed-form derivatives of w[p,k] = exp(-0.5 sum_d ((pseudo[p,d]-mu[k,d])*isg[k,d])^2), one edge per
// thread.  src[p,k] is either dL/dw (premultiplied == 0: the weight is recomputed here) or dL/dw * w.
//   d/dpseudo[p,d] = -sum_k gww*diff*isg^2,  d/dmu[k,d] = sum_p gww*diff*isg^2,  d/disg[k,d] = -sum_p gww*diff^2*isg
// The mu / isg sums are reduced per workgroup in a fixed order into red[block, 2*K*dim].
__global__ __launch_bounds__(256) void gauss_grad_kernel(int64_t E, int K, int dim, const float *__restrict__ pseudo,
                                                         const float *__restrict__ mu, const float *__restrict__ isg,
                                                         const float *__restrict__ src, int premultiplied,
                                                         float *__restrict__ gp, float *__restrict__ red)
{
    extern __shared__ float lds[];
    const int KD = K * dim;
    float *shared = lds;                 // mu | isg
    float *wsum = lds + 2 * KD;          // [4 waves][2*KD]
    for (int i = (int)threadIdx.x; i < KD; i += 256) { shared[i] = mu[i]; shared[KD + i] = isg[i]; }
    __syncthreads();
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool ok = e < E;
    const int64_t ee = ok ? e : 0;
    const int lane = fg_lane(), wave = fg_wave();
    for (int k = 0; k < K; ++k) {
        float gww = ok ? src[ee * K + k] : 0.f;
        if (!premultiplied) {
            float acc = 0.f;
            for (int d = 0; d < dim; ++d) {
                float t = (pseudo[ee * dim + d] - shared[k * dim + d]) * shared[KD + k * dim + d];
                acc = fmaf(t, t, acc);
            }
            gww *= __expf(-0.5f * acc);
        }
        for (int d = 0; d < dim; ++d) {
            float diff = pseudo[ee * dim + d] - shared[k * dim + d];
            float sg = shared[KD + k * dim + d];
            float a = gww * diff * sg;
            float sm = fg_wave_sum(a * sg);
            float ss = fg_wave_sum(-a * diff);
            if (lane == 0) { wsum[wave * 2 * KD + k * dim + d] = sm; wsum[wave * 2 * KD + KD + k * dim + d] = ss; }
        }
    }
    if (ok) {
        for (int d = 0; d < dim; ++d) {
            float acc = 0.f, psd = pseudo[ee * dim + d];
            for (int k = 0; k < K; ++k) {
                float gww = src[ee * K + k];
                if (!premultiplied) {
                    float a2 = 0.f;
                    for (int dd = 0; dd < dim; ++dd) {
                        float t = (pseudo[ee * dim + dd] - shared[k * dim + dd]) * shared[KD + k * dim + dd];
                        a2 = fmaf(t, t, a2);
                    }
                    gww *= __expf(-0.5f * a2);
                }
                float sg = shared[KD + k * dim + d];
                acc = fmaf(-gww * (psd - shared[k * dim + d]), sg * sg, acc);
            }
            gp[e * dim + d] = acc;
        }
    }
    __syncthreads();
    for (int i = (int)threadIdx.x; i < 2 * KD; i += 256)
        red[(size_t)blockIdx.x * 2 * KD + i] = (wsum[i] + wsum[2 * KD + i]) + (wsum[4 * KD + i] + wsum[6 * KD + i]);
}

// The same derivatives for small mixtures (K <= 4, dim <= 3: the MoNet models), K and dim known at
// compile time: mu and inv_sigma live in registers, a thread handles GG_EPT edges 256 apart and keeps
// its partial mu / isg sums in registers, so the wave reductions run once per GG_EPT * 64 edges.
#define GG_EPT 4
template <int K, int DIM>
__global__ __launch_bounds__(256) void gauss_grad_small_kernel(int64_t E, const float *__restrict__ pseudo, const float *__restrict__ mu,
                                                               const float *__restrict__ isg, const float *__restrict__ src,
                                                               int premultiplied, float *__restrict__ gp, float *__restrict__ red)
{
    constexpr int KD = K * DIM;
    __shared__ float wsum[4][2 * KD];
    float m[KD], s[KD], amu[KD], asg[KD];
#pragma unroll
    for (int i = 0; i < KD; ++i) { m[i] = mu[i]; s[i] = isg[i]; amu[i] = 0.f; asg[i] = 0.f; }
    const int64_t base = (int64_t)blockIdx.x * (256 * GG_EPT) + threadIdx.x;
#pragma unroll
    for (int t = 0; t < GG_EPT; ++t) {
        const int64_t e = base + t * 256;
        if (e < E) {
            float p[DIM], g[K], gpd[DIM];
#pragma unroll
            for (int d = 0; d < DIM; ++d) { p[d] = pseudo[e * DIM + d]; gpd[d] = 0.f; }
#pragma unroll
            for (int k = 0; k < K; ++k) g[k] = src[e * K + k];
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float diff[DIM], acc = 0.f;
#pragma unroll
                for (int d = 0; d < DIM; ++d) {
                    diff[d] = p[d] - m[k * DIM + d];
                    const float u = diff[d] * s[k * DIM + d];
                    acc = fmaf(u, u, acc);
                }
                float gww = g[k];
                if (!premultiplied) gww *= __expf(-0.5f * acc);
#pragma unroll
                for (int d = 0; d < DIM; ++d) {
                    const float sg = s[k * DIM + d];
                    const float a = gww * diff[d] * sg;
                    amu[k * DIM + d] += a * sg;
                    asg[k * DIM + d] -= a * diff[d];
                    gpd[d] = fmaf(-gww * diff[d], sg * sg, gpd[d]);
                }
            }
#pragma unroll
            for (int d = 0; d < DIM; ++d) gp[e * DIM + d] = gpd[d];
        }
    }
    const int lane = fg_lane(), wave = fg_wave();
#pragma unroll
    for (int i = 0; i < KD; ++i) {
        const float sm = fg_wave_sum(amu[i]), ss = fg_wave_sum(asg[i]);
        if (lane == 0) { wsum[wave][i] = sm; wsum[wave][KD + i] = ss; }
    }
    __syncthreads();
    for (int i = (int)threadIdx.x; i < 2 * KD; i += 256)
        red[(size_t)blockIdx.x * 2 * KD + i] = (wsum[0][i] + wsum[1][i]) + (wsum[2][i] + wsum[3][i]);
}

template <int K>
static bool gauss_grad_small_launch(int dim, int nblk, hipStream_t st, int64_t E, const float *pseudo, const float *mu, const float *isg,
                                    const float *src, int premultiplied, float *gp, float *red)
{
    switch (dim) {
    case 1: hipLaunchKernelGGL((gauss_grad_small_kernel<K, 1>), dim3(nblk), dim3(256), 0, st, E, pseudo, mu, isg, src, premultiplied, gp, red); return true;
    case 2: hipLaunchKernelGGL((gauss_grad_small_kernel<K, 2>), dim3(nblk), dim3(256), 0, st, E, pseudo, mu, isg, src, premultiplied, gp, red); return true;
    case 3: hipLaunchKernelGGL((gauss_grad_small_kernel<K, 3>), dim3(nblk), dim3(256), 0, st, E, pseudo, mu, isg, src, premultiplied, gp, red); return true;
    default: return false;
    }
}

// Column sums of red[rows, width] in two deterministic levels.
__global__ __launch_bounds__(256) void colsum_level1(const float *red, int rows, int width, float *tmp /*[gridDim.x, width]*/)
{
    __shared__ float sh[256];
    int chunk = (rows + gridDim.x - 1) / gridDim.x;
    int r0 = blockIdx.x * chunk, r1 = min(rows, r0 + chunk);
    for (int c = 0; c < width; ++c) {
        float acc = 0.f;
        for (int r = r0 + (int)threadIdx.x; r < r1; r += 256) acc += red[(size_t)r * width + c];
        sh[threadIdx.x] = acc;
        __syncthreads();
        for (int s = 128; s > 0; s >>= 1) {
            if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
            __syncthreads();
        }
        if (threadIdx.x == 0) tmp[(size_t)blockIdx.x * width + c] = sh[0];
        __syncthreads();
    }
}
__global__ __launch_bounds__(64) void colsum_level2(const float *tmp, int nblk, int KD, float *gmu, float *gsig)
{
    for (int c = (int)threadIdx.x; c < 2 * KD; c += 64) {
        float acc = 0.f;
        for (int b = 0; b < nblk; ++b) acc += tmp[(size_t)b * 2 * KD + c];
        if (c < KD) gmu[c] = acc; else gsig[c - KD] = acc;
    }
}

static const int kColsumBlocks = 64;

// gauss_grad_kernel + column sums on `st`; ws must hold gauss_grad_workspace(E, K, dim) bytes.
static size_t gauss_grad_workspace(int64_t E, int K, int dim)
{
    size_t nblk = (size_t)((E + 255) / 256);
    return fgnn_align256(nblk * 2 * K * dim * sizeof(float)) + fgnn_align256((size_t)kColsumBlocks * 2 * K * dim * sizeof(float));
}
static int gauss_grad_launch(int64_t E, int K, int dim, const float *pseudo, const float *mu, const float *isg, const float *src,
                             int premultiplied, float *gp, float *gmu, float *gsig, void *ws, hipStream_t st)
{
    const int KD = K * dim;
    if (E == 0) {
        int rc = fgnn_fill_f32(gmu, KD, 0.f, st);
        return rc ? rc : fgnn_fill_f32(gsig, KD, 0.f, st);
    }
    int nblk = (int)((E + 255) / 256);
    float *red = (float *)ws;
    float *tmp = (float *)((char *)ws + fgnn_align256((size_t)nblk * 2 * KD * sizeof(float)));     // layout sized for one edge per thread
    const int nblk_small = (int)((E + 256 * GG_EPT - 1) / (256 * GG_EPT));
    bool small = false;
    switch (K) {
    case 1: small = gauss_grad_small_launch<1>(dim, nblk_small, st, E, pseudo, mu, isg, src, premultiplied, gp, red); break;
    case 2: small = gauss_grad_small_launch<2>(dim, nblk_small, st, E, pseudo, mu, isg, src, premultiplied, gp, red); break;
    case 3: small = gauss_grad_small_launch<3>(dim, nblk_small, st, E, pseudo, mu, isg, src, premultiplied, gp, red); break;
    case 4: small = gauss_grad_small_launch<4>(dim, nblk_small, st, E, pseudo, mu, isg, src, premultiplied, gp, red); break;
    default: break;
    }
    if (small) {
        nblk = nblk_small;
    } else {
        size_t shm = (size_t)(2 * KD + 4 * 2 * KD) * sizeof(float);
        hipLaunchKernelGGL(gauss_grad_kernel, dim3(nblk), dim3(256), shm, st, E, K, dim, pseudo, mu, isg, src, premultiplied, gp, red);
    }
    int rc = fgnn_launch_status("gauss_grad_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(colsum_level1, dim3(kColsumBlocks), dim3(256), 0, st, red, nblk, 2 * KD, tmp);
    rc = fgnn_launch_status("colsum_level1");
    if (rc) return rc;
    hipLaunchKernelGGL(colsum_level2, dim3(1), dim3(64), 0, st, tmp, kColsumBlocks, KD, gmu, gsig);
    return fgnn_launch_status("colsum_level2");
}

extern "C" size_t fgnn_gmm_backward_workspace_bytes(const fgnn_schedule_t *sched_csc, int K, int dim, int F)
{
    // partials | gw*w [E,K] | reduction scratch
    if (!sched_csc) return 0;
    size_t b = fgnn_align256((size_t)sched_csc->n_partials * spmm_pw(K * F) * sizeof(float));
    b += fgnn_align256((size_t)sched_csc->n_edges * K * sizeof(float));
    b += gauss_grad_workspace(sched_csc->n_edges, K, dim);
    return b;
}

extern "C" int fgnn_gmm_backward(int N, int64_t E, int K, int dim, int F, const int32_t *col_ptr, const int32_t *row_ind,
                                 const int32_t *permute, const float *node_feat, const float *pseudo, const float *mu,
                                 const float *inv_sigma, const float *grad_out, int sum_kernels, float *grad_feat, float *grad_pseudo,
                                 float *grad_mu, float *grad_sigma, const fgnn_schedule_t *sched_csc, void *workspace,
                                 size_t workspace_bytes, void *stream)
{
    int rc = spmm_checks("fgnn_gmm_backward", N, E, K, F, sched_csc, col_ptr, row_ind);
    if (rc) return rc;
    FGNN_REQUIRE((int64_t)K * F <= 1024, FGNN_ERR_LIMIT, "fgnn_gmm_backward: K*F=%lld > 1024 unsupported", (long long)K * F);
    FGNN_REQUIRE(dim >= 1 && dim <= 64 && K * dim <= 1024, FGNN_ERR_LIMIT, "fgnn_gmm_backward: dim=%d K*dim=%d unsupported", dim, K * dim);
    FGNN_REQUIRE(col_ptr && (row_ind || E == 0) && node_feat && (pseudo || E == 0) && mu && inv_sigma &&
                     grad_out && grad_feat && (grad_pseudo || E == 0) && grad_mu && grad_sigma,
                 FGNN_ERR_NULL, "fgnn_gmm_backward: NULL argument");
    FGNN_REQUIRE(sched_csc, FGNN_ERR_SCHEDULE, "fgnn_gmm_backward: a schedule of col_ptr is required");
    FGNN_REQUIRE(sum_kernels >= 0 && sum_kernels <= 2, FGNN_ERR_SHAPE, "fgnn_gmm_backward: sum_kernels=%d (0, 1 or 2)", sum_kernels);
    size_t need = fgnn_gmm_backward_workspace_bytes(sched_csc, K, dim, F);
    FGNN_REQUIRE(workspace && workspace_bytes >= need && fgnn_aligned16(workspace), FGNN_ERR_WORKSPACE,
                 "fgnn_gmm_backward: workspace %zu < %zu bytes (or unaligned)", workspace_bytes, need);
    hipStream_t st = (hipStream_t)stream;
    const int HF = K * F, KD = K * dim;
    char *w = (char *)workspace;
    float *part = (float *)w; w += fgnn_align256((size_t)sched_csc->n_partials * spmm_pw(HF) * sizeof(float));
    float *gww = (float *)w; w += fgnn_align256((size_t)E * K * sizeof(float));
    void *gws = w;
    if (sched_csc->n_items > 0) {
        bool aligned = fgnn_aligned16(node_feat) && fgnn_aligned16(grad_out) && fgnn_aligned16(grad_feat);
        fgnn_rowcfg cfg;
        FGNN_REQUIRE(fgnn_pick_rowcfg(HF, F, aligned, &cfg), FGNN_ERR_LIMIT, "fgnn_gmm_backward: unsupported row width %d", HF);
        GmmBwdP p{};
        p.items = sched_csc->items_dev; p.n_items = sched_csc->n_items; p.ptr = col_ptr; p.idx = fgnn_sched_idx(sched_csc, row_ind);
        p.pos = fgnn_sched_pos(sched_csc); p.permute = permute;
        p.x = node_feat; p.g = grad_out; p.pseudo = pseudo; p.mu = mu; p.isg = inv_sigma; p.gfeat = grad_feat; p.gww = gww;
        p.part = part; p.N = N; p.K = K; p.dim = dim; p.F = F; p.HF = HF;
        p.g_stride = sum_kernels == 1 ? F : HF;
        p.x_stride = sum_kernels == 2 ? F : HF;
        // widths like 44 or 48 (quarter not a power of two): head-aligned lane map, so the per-edge dot
        // products still reduce with DPP and narrow rows still pack
        p.lphp = fgnn_pad_lph(cfg.vec, K, F);
        int lanes_hf = HF;          // floats the lane map spans
        if (p.lphp) {
            lanes_hf = K * p.lphp * 4;
            cfg.r = lanes_hf <= 256 ? 1 : lanes_hf <= 512 ? 2 : 4;
            cfg.full = false;
        }
        const int lph = p.lphp ? p.lphp : fgnn_pick_lph(cfg.vec, F);
        const unsigned grid = (unsigned)((p.n_items + FGNN_WPB - 1) / FGNN_WPB);
        const bool sumk = sum_kernels == 1 && cfg.vec == 4 && F % 4 == 0 && F <= 256 && K <= GMM_SUMK_MAX;
        rc = sumk ? 0 : 1;
        if (sumk) {
            // lanes over F only, the K mixture kernels in registers (see gmm_bwd_sum_kernel)
            int lpf = 1;
            while (lpf * 4 < F) lpf *= 2;
            const size_t shm = ((size_t)FGNN_WPB * K * 64 + 2 * KD) * sizeof(float);
            FGNN_REQUIRE(shm <= 64 * 1024, FGNN_ERR_LIMIT, "fgnn_gmm_backward: K=%d, dim=%d need %zu bytes of LDS per workgroup (limit 64 KiB)", K, dim, shm);
            p.lphp = 0;
            gmm_sum_launch<true>(lpf, grid, shm, st, p, gmm_group_items_first(sched_csc, lpf), sched_csc->n_buckets > 0);
            rc = fgnn_launch_status("gmm_bwd_sum_kernel");
            if (rc) return rc;
            if (sched_csc->n_split > 0) {
                SpmmP mp{};
                mp.part = part; mp.out = grad_feat; mp.N = N; mp.H = K; mp.F = F; mp.HF = HF; mp.ld = mp.ldo = HF;
                unsigned g2 = (unsigned)((sched_csc->n_split + FGNN_WPB - 1) / FGNN_WPB);
                rc = fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
                    hipLaunchKernelGGL((spmm_merge_kernel<VEC, R>), dim3(g2), dim3(FGNN_TPB), 0, st, mp, sched_csc->split_dev, sched_csc->n_split);
                    return fgnn_launch_status("spmm_merge_kernel");
                });
                if (rc) return rc;
            }
        }
        if (!sumk) rc = fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
            size_t shm = ((size_t)FGNN_WPB * (K * 64 + 64 * R) + 2 * KD) * sizeof(float);
            FGNN_REQUIRE(shm <= 64 * 1024, FGNN_ERR_LIMIT, "fgnn_gmm_backward: K=%d, dim=%d need %zu bytes of LDS per workgroup (limit 64 KiB)", K, dim, shm);
            const int pack = lph > 0 ? fgnn_pick_pack(cfg.vec, lanes_hf) : 1;
            int rc2 = fgnn_dispatch_lph(VEC == 4 ? lph : 0, [&]<int LPH>() -> int {
                if constexpr (VEC == 4 && R == 1 && LPH > 0 && LPH <= 32) {
                    // a mixture kernel's LPH lanes must fit inside one group of 64/pack lanes
                    // graphs of short rows: the items behind the long head of the list go `pack` to a wave (gmm_bwd_packed_group_items;
                    // [N,2,16] rows at 2.4 M nodes x 26 entries per column: 2.59 -> 1.50 ms)
                    const int first = (pack >= 4 && sched_csc->n_edges < 256 * (int64_t)sched_csc->n_rows) ? sched_csc->n_wave_slots : p.n_items;
                    const int bucketed = sched_csc->n_buckets > 0;
                    const unsigned hb = (unsigned)((first + FGNN_WPB - 1) / FGNN_WPB);
                    const unsigned gm = hb + fgnn_group_item_grid(p.n_items - first, pack, bucketed);
                    if (pack == 8 && LPH <= 8 && first < p.n_items) { hipLaunchKernelGGL((gmm_bwd_packed_mixed_kernel<8, (LPH <= 8 ? LPH : 1)>), dim3(gm), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); return fgnn_launch_status("gmm_bwd_packed_mixed_kernel"); }
                    if (pack == 4 && LPH <= 16 && first < p.n_items) { hipLaunchKernelGGL((gmm_bwd_packed_mixed_kernel<4, (LPH <= 16 ? LPH : 1)>), dim3(gm), dim3(FGNN_TPB), shm, st, p, bucketed, first, hb); return fgnn_launch_status("gmm_bwd_packed_mixed_kernel"); }
                    if (pack == 8 && LPH <= 8) { hipLaunchKernelGGL((gmm_bwd_packed_kernel<8, (LPH <= 8 ? LPH : 1)>), dim3(grid), dim3(FGNN_TPB), shm, st, p); return fgnn_launch_status("gmm_bwd_packed_kernel"); }
                    if (pack == 4 && LPH <= 16) { hipLaunchKernelGGL((gmm_bwd_packed_kernel<4, (LPH <= 16 ? LPH : 1)>), dim3(grid), dim3(FGNN_TPB), shm, st, p); return fgnn_launch_status("gmm_bwd_packed_kernel"); }
                    if (pack == 2 && LPH <= 32) { hipLaunchKernelGGL((gmm_bwd_packed_kernel<2, LPH>), dim3(grid), dim3(FGNN_TPB), shm, st, p); return fgnn_launch_status("gmm_bwd_packed_kernel"); }
                }
                hipLaunchKernelGGL((gmm_bwd_kernel<VEC, R, FULL, (VEC == 4 ? LPH : 0)>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                return fgnn_launch_status("gmm_bwd_kernel");
            });
            if (rc2) return rc2;
            if (sched_csc->n_split > 0) {
                SpmmP mp{};
                mp.part = part; mp.out = grad_feat; mp.N = N; mp.H = K; mp.F = F; mp.HF = HF; mp.ld = mp.ldo = HF;
                unsigned g2 = (unsigned)((sched_csc->n_split + FGNN_WPB - 1) / FGNN_WPB);
                hipLaunchKernelGGL((spmm_merge_kernel<VEC, R>), dim3(g2), dim3(FGNN_TPB), 0, st, mp, sched_csc->split_dev, sched_csc->n_split);
                return fgnn_launch_status("spmm_merge_kernel");
            }
            return 0;
        });
        if (rc) return rc;
    }
    return gauss_grad_launch(E, K, dim, pseudo, mu, inv_sigma, gww, 1, grad_pseudo, grad_mu, grad_sigma, gws, st);
}

// ------------------------------------------------------------------------------- standalone Gaussian
__global__ __launch_bounds__(256) void gaussian_kernel(int64_t E, int K, int dim, const float *pseudo, const float *mu,
                                                       const float *isg, float *out)
{
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= E * K) return;
    int64_t e = tid / K;
    int k = (int)(tid - e * K);
    float acc = 0.f;
    for (int d = 0; d < dim; ++d) {
        float t = (pseudo[e * dim + d] - mu[k * dim + d]) * isg[k * dim + d];
        acc = fmaf(t, t, acc);
    }
    out[tid] = __expf(-0.5f * acc);
}

extern "C" int fgnn_gaussian(int64_t E, int K, int dim, const float *pseudo, const float *mu, const float *inv_sigma,
                             float *out, void *stream)
{
    FGNN_REQUIRE(E >= 0 && K >= 1 && dim >= 1, FGNN_ERR_SHAPE, "fgnn_gaussian: bad sizes");
    FGNN_REQUIRE((pseudo || E == 0) && mu && inv_sigma && (out || E == 0), FGNN_ERR_NULL, "fgnn_gaussian: NULL argument");
    if (E == 0) return 0;
    int64_t total = E * K;
    hipLaunchKernelGGL(gaussian_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, E, K, dim, pseudo, mu, inv_sigma, out);
    return fgnn_launch_status("gaussian_kernel");
}

extern "C" size_t fgnn_gaussian_backward_workspace_bytes(int64_t E, int K, int dim) { return gauss_grad_workspace(E, K, dim); }

extern "C" int fgnn_gaussian_backward(int64_t E, int K, int dim, const float *pseudo, const float *mu, const float *inv_sigma,
                                      const float *grad_w, float *grad_pseudo, float *grad_mu, float *grad_sigma,
                                      void *workspace, size_t workspace_bytes, void *stream)
{
    FGNN_REQUIRE(E >= 0 && K >= 1 && dim >= 1 && K * dim <= 1024, FGNN_ERR_SHAPE, "fgnn_gaussian_backward: bad sizes");
    FGNN_REQUIRE((pseudo || E == 0) && mu && inv_sigma && (grad_w || E == 0) && (grad_pseudo || E == 0) && grad_mu && grad_sigma,
                 FGNN_ERR_NULL, "fgnn_gaussian_backward: NULL argument");
    size_t need = gauss_grad_workspace(E, K, dim);
    FGNN_REQUIRE(E == 0 || (workspace && workspace_bytes >= need), FGNN_ERR_WORKSPACE, "fgnn_gaussian_backward: workspace %zu < %zu bytes",
                 workspace_bytes, need);
    return gauss_grad_launch(E, K, dim, pseudo, mu, inv_sigma, grad_w, 0, grad_pseudo, grad_mu, grad_sigma, workspace, (hipStream_t)stream);
}
