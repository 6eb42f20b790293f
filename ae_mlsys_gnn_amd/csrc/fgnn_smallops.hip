// The small per-edge operators of the reference's operators/ package: multi-head SDDMM,
// permuted row gather (mhtranspose), edge softmax and u_add_v, each with its backward.
// None of them takes a work list, so each balances its own load: the element-wise ones cut the
// [E, W] array into fixed chunks and find the rows of a chunk by bisection of row_ptr, the row
// reductions give short rows to single waves and long rows to whole workgroups.
#include <algorithm>
#include "fgnn_common.h"

// largest r in [lo, hi] with ptr[r] <= q
__device__ __forceinline__ int so_row_of(const int *__restrict__ ptr, int lo, int hi, int q)
{
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (ptr[mid] <= q) lo = mid; else hi = mid - 1;
    }
    return lo;
}

// out[p,h] = <a[row,h,:], b[col_ind[p],h,:]> (src/sddmm/mhsddmm.cu:5-81 of the reference, which
// finds the row of each edge by binary search).  The entries [pb, pe) of one row, 64 at a time, four gathered
// b-rows in flight; pos (NULL = identity) maps an entry to the position its result is stored at.
template <int VEC, int R, bool FULL, int LPH>
__device__ __forceinline__ void sddmm_row_piece(int row, int pb, int pe, int H, int F, int ld, int ldo, const fg_lanemap<VEC, R> &lm, int lane, float *scr,
                                                const int *__restrict__ idx, const int *__restrict__ pos, const float *__restrict__ a,
                                                const float *__restrict__ b, float *__restrict__ out)
{
    fg_vec<VEC> ar[R];
#pragma unroll
    for (int r = 0; r < R; ++r) { if (FULL || lm.ok[r]) ar[r].load(a + (size_t)row * ld + lm.eoff[r]); else ar[r].zero(); }
    if constexpr (R == 1 && LPH >= 4) {
        // Head h owns the LPH lanes from h * LPH on and fg_group_sum leaves a head's dot product in all of them, so lane
        // h * LPH + u simply keeps the result of entry u of a batch of EB; one lane exchange then brings (entry u, head h) to
        // lane u * H + h and ONE store instruction writes the batch (EB runs of H floats, one contiguous run where the
        // positions are consecutive) instead of one instruction of H active lanes per entry: on a 115 M-entry graph with 8
        // heads the per-entry stores held the address unit as long as the gathered rows did.
        constexpr int EB = LPH < 8 ? LPH : 8;
        const int sub = lane & (LPH - 1);
        const int ou = lane / H, oh = lane - ou * H;              // the (entry, head) this lane stores
        const bool olive = ou < EB;
        const int osrc = (oh * LPH + ou) << 2;
        for (int c = pb; c < pe; c += 64) {
            const int q = c + lane;
            const int cnt = min(64, pe - c);
            const int qq = q < pe ? q : c;
            const int id = idx[qq];
            const int pv = pos ? pos[qq] : qq;
            for (int t = 0; t < cnt; t += EB) {
                float keep = 0.f;
                constexpr int UL = EB < 4 ? EB : 4;                   // gathered rows in flight (eight: same time, 12 % more L2 misses)
#pragma unroll
                for (int t4 = 0; t4 < EB; t4 += UL) {
                    fg_vec<VEC> lb[UL];
#pragma unroll
                    for (int u = 0; u < UL; ++u) {
                        const int j = __builtin_amdgcn_readlane(id, (t + t4 + u) & 63);      // past the chunk: a valid row, result not stored
                        if (FULL || lm.ok[0]) lb[u].load(b + (size_t)j * ld + lm.eoff[0]); else lb[u].zero();
                    }
#pragma unroll
                    for (int u = 0; u < UL; ++u) {
                        const float sum = fg_group_sum<LPH>(lb[u].dot(ar[0]));
                        keep = sub == t4 + u ? sum : keep;
                    }
                }
                const float v = __int_as_float(__builtin_amdgcn_ds_bpermute(osrc, __float_as_int(keep)));
                const int po = __builtin_amdgcn_ds_bpermute(((t + ou) & 63) << 2, pv);
                if (olive && t + ou < cnt) __builtin_nontemporal_store(v, out + (size_t)(unsigned)po * ldo + oh);
            }
        }
        return;
    }
    for (int c = pb; c < pe; c += 64) {
        const int q = c + lane;
        const int cnt = min(64, pe - c);
        const int qq = q < pe ? q : c;
        const int id = idx[qq];
        const int pv = pos ? pos[qq] : qq;
        for (int t = 0; t < cnt; t += 4) {
            fg_vec<VEC> lb[4][R];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int j = __builtin_amdgcn_readlane(id, (t + u) & 63);
#pragma unroll
                for (int r = 0; r < R; ++r) { if (FULL || lm.ok[r]) lb[u][r].load(b + (size_t)j * ld + lm.eoff[r]); else lb[u][r].zero(); }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (t + u >= cnt) break;
                float d[R];
#pragma unroll
                for (int r = 0; r < R; ++r) d[r] = lb[u][r].dot(ar[r]);
                const size_t o = (size_t)(unsigned)__builtin_amdgcn_readlane(pv, (t + u) & 63) * ldo;
                if constexpr (LPH > 0) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        float s = fg_group_sum<LPH>(d[r]);
                        if ((FULL || lm.ok[r]) && lm.eoff[r] % F == 0) __builtin_nontemporal_store(s, out + o + lm.hd[r]);
                    }
                } else {
                    float s = H <= FGNN_FEW_HEADS ? fg_head_reduce_few<VEC, R>(d, lm, lane, H) : fg_head_reduce<VEC, R>(scr, d, lm, lane, H, F);
                    if (lane < H) __builtin_nontemporal_store(s, out + o + lane);
                }
            }
        }
    }
}

// Without a work list: one wave per SDDMM_CHUNK consecutive CSR positions, the row of the first one by
// bisection, the following rows by walking row_ptr, so a hub row is shared by as many waves as it has chunks
// and the a-row is loaded once per (wave, row).
#define SDDMM_CHUNK 256
template <int VEC, int R, bool FULL, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void mhsddmm_kernel(int N, int64_t E, int H, int F, int HF, int ld, int ldo, int lphp, const int *ptr, const int *idx,
                                                           const float *a, const float *b, float *out)
{
    extern __shared__ float lds[];
    const int64_t c0 = ((int64_t)blockIdx.x * FGNN_WPB + fg_wave()) * SDDMM_CHUNK;
    if (c0 >= E) return;
    const int c1 = fg_uni((int)min(c0 + SDDMM_CHUNK, E));
    const int lane = fg_lane();
    float *scr = lds + fg_wave() * (64 * R);
    fg_lanemap<VEC, R> lm;
    if (lphp) lm.init_padded(lane, H, F, lphp); else lm.init(lane, HF, F);      // lphp: head-aligned lanes for DPP sums
    int row = fg_uni(so_row_of(ptr, 0, N - 1, (int)c0));     // ptr[row] <= c0 < ptr[row + 1]
    int pb = fg_uni((int)c0);
    while (pb < c1 && row < N) {                             // ptr[N] = E >= c1 keeps row < N on a consistent graph
        const int pe = min(fg_uni(ptr[row + 1]), c1);
        if (pe > pb) sddmm_row_piece<VEC, R, FULL, LPH>(row, pb, pe, H, F, ld, ldo, lm, lane, scr, idx, nullptr, a, b, out);
        pb = pe;
        ++row;
    }
}

// Under a work list (one wave per item; an XCD-aware list keeps each XCD on one eighth of the gathered b-rows):
// the entries are walked in the list's order and every result goes to its caller's position.
template <int VEC, int R, bool FULL, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void mhsddmm_items_kernel(const fgnn_item *items, int n_items, int H, int F, int HF, int ld, int ldo, int lphp, const int *ptr,
                                                                 const int *idx, const int *pos, const float *a, const float *b, float *out)
{
    extern __shared__ float lds[];
    int row, pb, pe, slot;
    if (!fg_get_item(items, n_items, ptr, row, pb, pe, slot)) return;
    const int lane = fg_lane();
    float *scr = lds + fg_wave() * (64 * R);
    fg_lanemap<VEC, R> lm;
    if (lphp) lm.init_padded(lane, H, F, lphp); else lm.init(lane, HF, F);
    sddmm_row_piece<VEC, R, FULL, LPH>(row, pb, pe, H, F, ld, ldo, lm, lane, scr, idx, pos, a, b, out);
}

// The same for rows narrower than a wave (at most 128 floats in the 128-bit layout): the wave is cut into G lane groups
// (fg_packmap) that take G different entries of the row with the same load instruction, eight instructions in flight; a head's
// dot product is summed inside its LPH lanes and its first lane stores it.  With one entry per instruction a row of 48 floats
// kept 12 lanes busy (64 M entries of 1 x 48: 3.5 ms).
template <int G, int LPH>
__device__ __forceinline__ void sddmm_row_piece_packed(int row, int pb, int pe, int H, int F, int HF, int ld, int ldo, int lphp, int lane,
                                                       const int *__restrict__ idx, const int *__restrict__ pos, const float *__restrict__ a,
                                                       const float *__restrict__ b, float *__restrict__ out)
{
    constexpr int U = 8;
    fg_packmap<G> pm;
    if (lphp) pm.init_padded(lane, H, F, lphp); else pm.init(lane, HF, F);
    fg_vec<4> ar;
    if (pm.ok) ar.load(a + (size_t)row * ld + pm.eoff); else ar.zero();
    const bool writer = pm.ok && pm.eoff % F == 0;
    for (int c = pb; c < pe; c += 64) {
        const int q = c + lane;
        const int cnt = min(64, pe - c);
        const int qq = q < pe ? q : c;
        const int id = idx[qq];
        const int pv = pos ? pos[qq] : qq;
        for (int t = 0; t < cnt; t += U * G) {
            fg_vec<4> lb[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + pm.grp;
                const size_t j = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((ei & 63) << 2, id);
                if (ei < cnt && pm.ok) lb[u].load(b + j * ld + pm.eoff); else lb[u].zero();
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + pm.grp;
                const float sum = fg_group_sum<LPH>(lb[u].dot(ar));
                const size_t po = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((ei & 63) << 2, pv);
                if (writer && ei < cnt) __builtin_nontemporal_store(sum, out + po * ldo + pm.hd);
            }
        }
    }
}

template <int G, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void mhsddmm_packed_kernel(int N, int64_t E, int H, int F, int HF, int ld, int ldo, int lphp, const int *ptr, const int *idx,
                                                                  const float *a, const float *b, float *out)
{
    const int64_t c0 = ((int64_t)blockIdx.x * FGNN_WPB + fg_wave()) * SDDMM_CHUNK;
    if (c0 >= E) return;
    const int c1 = fg_uni((int)min(c0 + SDDMM_CHUNK, E));
    const int lane = fg_lane();
    int row = fg_uni(so_row_of(ptr, 0, N - 1, (int)c0));     // ptr[row] <= c0 < ptr[row + 1]
    int pb = fg_uni((int)c0);
    while (pb < c1 && row < N) {
        const int pe = min(fg_uni(ptr[row + 1]), c1);
        if (pe > pb) sddmm_row_piece_packed<G, LPH>(row, pb, pe, H, F, HF, ld, ldo, lphp, lane, idx, nullptr, a, b, out);
        pb = pe;
        ++row;
    }
}

template <int G, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void mhsddmm_packed_items_kernel(const fgnn_item *items, int n_items, int H, int F, int HF, int ld, int ldo, int lphp,
                                                                        const int *ptr, const int *idx, const int *pos, const float *a, const float *b,
                                                                        float *out)
{
    int row, pb, pe, slot;
    if (!fg_get_item(items, n_items, ptr, row, pb, pe, slot)) return;
    sddmm_row_piece_packed<G, LPH>(row, pb, pe, H, F, HF, ld, ldo, lphp, fg_lane(), idx, pos, a, b, out);
}

static int mhsddmm_run(const char *fn, int N, int64_t E, int H, int F, const int32_t *row_ptr, const int32_t *col_ind, const float *a,
                       const float *b, float *out, const fgnn_schedule_t *sched, hipStream_t st)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1 && F >= 1, FGNN_ERR_SHAPE, "%s: bad sizes", fn);
    FGNN_REQUIRE(H <= 64 && F <= 1024, FGNN_ERR_LIMIT, "%s: H=%d F=%d unsupported (at most 64 heads of at most 1024 floats)", fn, H, F);
    FGNN_REQUIRE(row_ptr && (col_ind || E == 0) && a && b && (out || E == 0), FGNN_ERR_NULL, "%s: NULL argument", fn);
    FGNN_REQUIRE(E <= 2147483647LL, FGNN_ERR_LIMIT, "%s: E=%lld exceeds the 32-bit row_ptr", fn, (long long)E);
    if (sched) {
        FGNN_REQUIRE(sched->ptr_dev == row_ptr && sched->n_rows == N && sched->n_edges == E, FGNN_ERR_SCHEDULE,
                     "%s: schedule was built for another pointer array", fn);
        FGNN_REQUIRE(sched->n_buckets == 0 || sched->idx_src_dev == col_ind, FGNN_ERR_SCHEDULE,
                     "%s: XCD-aware schedule was built from another index array", fn);
        // a list whose position map was handed to the caller (fgnn_schedule_take_positions) stores in its own entry order
        FGNN_REQUIRE(fgnn_sched_has_pos(sched), FGNN_ERR_SCHEDULE,
                     "%s: the schedule must carry its edge positions (results are stored at the caller's positions)", fn);
    }
    if (N == 0 || E == 0) return 0;
    const int64_t waves = sched ? sched->n_items : (E + SDDMM_CHUNK - 1) / SDDMM_CHUNK;
    if (waves == 0) return 0;
    const unsigned grid = (unsigned)((waves + FGNN_WPB - 1) / FGNN_WPB);
    // rows of more than 1024 floats: passes over groups of heads on views of the wide arrays (heads are independent)
    const int hmax = (int64_t)H * F <= 1024 ? H : std::max(1, 1024 / F);
    for (int h0 = 0; h0 < H; h0 += hmax) {
        const int hg = std::min(hmax, H - h0), HF = hg * F, ld = H * F;
        const float *ag = a + (size_t)h0 * F, *bg = b + (size_t)h0 * F;
        float *og = out + h0;
        fgnn_rowcfg cfg;
        FGNN_REQUIRE(fgnn_pick_rowcfg(HF, F, fgnn_aligned16(a) && fgnn_aligned16(b), &cfg), FGNN_ERR_LIMIT, "%s: unsupported row width %d", fn, HF);
        const int lphp = fgnn_pad_lph(cfg.vec, hg, F);
        if (lphp) { int w = hg * lphp * 4; cfg.r = w <= 256 ? 1 : w <= 512 ? 2 : 4; cfg.full = false; }
        const int lph = lphp ? lphp : fgnn_pick_lph(cfg.vec, F);
        // rows narrower than a wave: `pack` entries per load instruction (a head's lanes must fit inside a group of 64 / pack)
        const int pack = lph > 0 ? fgnn_pick_pack(cfg.vec, lphp ? hg * lphp * 4 : HF) : 1;
        int rc = fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
            return fgnn_dispatch_lph(VEC == 4 ? lph : 0, [&]<int LPH>() -> int {
                const size_t shm = (size_t)FGNN_WPB * 64 * R * sizeof(float);
                if constexpr (VEC == 4 && R == 1 && LPH > 0 && LPH <= 32) {
                    auto packed = [&]<int G>() -> int {
                        constexpr int L = LPH <= 64 / G ? LPH : 1;          // never launched with L != LPH
                        if (sched)
                            hipLaunchKernelGGL((mhsddmm_packed_items_kernel<G, L>), dim3(grid), dim3(FGNN_TPB), 0, st, sched->items_dev, sched->n_items, hg, F,
                                               HF, ld, H, lphp, row_ptr, fgnn_sched_idx(sched, col_ind), fgnn_sched_pos(sched), ag, bg, og);
                        else
                            hipLaunchKernelGGL((mhsddmm_packed_kernel<G, L>), dim3(grid), dim3(FGNN_TPB), 0, st, N, E, hg, F, HF, ld, H, lphp, row_ptr, col_ind,
                                               ag, bg, og);
                        return fgnn_launch_status("mhsddmm_packed_kernel");
                    };
                    if (pack == 8 && LPH <= 8) return packed.template operator()<8>();
                    if (pack == 4 && LPH <= 16) return packed.template operator()<4>();
                    if (pack == 2 && LPH <= 32) return packed.template operator()<2>();
                }
                if (sched)
                    hipLaunchKernelGGL((mhsddmm_items_kernel<VEC, R, FULL, (VEC == 4 ? LPH : 0)>), dim3(grid), dim3(FGNN_TPB), shm, st, sched->items_dev,
                                       sched->n_items, hg, F, HF, ld, H, lphp, row_ptr, fgnn_sched_idx(sched, col_ind), fgnn_sched_pos(sched), ag, bg, og);
                else
                    hipLaunchKernelGGL((mhsddmm_kernel<VEC, R, FULL, (VEC == 4 ? LPH : 0)>), dim3(grid), dim3(FGNN_TPB), shm, st, N, E, hg, F, HF, ld, H, lphp,
                                       row_ptr, col_ind, ag, bg, og);
                return fgnn_launch_status("mhsddmm_kernel");
            });
        });
        if (rc) return rc;
    }
    return 0;
}

extern "C" int fgnn_mhsddmm(int N, int64_t E, int H, int F, const int32_t *row_ptr, const int32_t *col_ind, const float *a,
                            const float *b, float *out, void *stream)
{
    return mhsddmm_run("fgnn_mhsddmm", N, E, H, F, row_ptr, col_ind, a, b, out, nullptr, (hipStream_t)stream);
}

extern "C" int fgnn_mhsddmm_scheduled(int N, int64_t E, int H, int F, const int32_t *row_ptr, const int32_t *col_ind, const float *a,
                                      const float *b, float *out, const fgnn_schedule_t *sched, void *stream)
{
    return mhsddmm_run("fgnn_mhsddmm_scheduled", N, E, H, F, row_ptr, col_ind, a, b, out, sched, (hipStream_t)stream);
}

// out[e,h] = <a[row_ind[e],h,:], b[col_ind[e],h,:]> for an edge list (sddmm.coo_sddmm of the
// reference, src/sddmm/sddmm.cpp:12-27, with H heads).  One wave per 64 edges; both rows of an edge
// are fetched by base-plus-lane-offset loads, four edges in flight.
template <int VEC, int R, bool FULL, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void sddmm_coo_kernel(int64_t E, int H, int F, int HF, int lphp, const int *rows, const int *cols,
                                                             const float *a, const float *b, float *out)
{
    extern __shared__ float lds[];
    const int64_t c = ((int64_t)blockIdx.x * FGNN_WPB + fg_wave()) * 64;
    if (c >= E) return;
    const int lane = fg_lane();
    float *scr = lds + fg_wave() * (64 * R);
    fg_lanemap<VEC, R> lm;
    if (lphp) lm.init_padded(lane, H, F, lphp); else lm.init(lane, HF, F);      // lphp: head-aligned lanes for DPP sums
    const int cnt = (int)min((int64_t)64, E - c);
    const int64_t q = c + (lane < cnt ? lane : 0);
    const int ri = rows[q], ci = cols[q];
    for (int t = 0; t < cnt; t += 4) {
        fg_vec<VEC> la[4][R], lb[4][R];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int i = __builtin_amdgcn_readlane(ri, (t + u) & 63), j = __builtin_amdgcn_readlane(ci, (t + u) & 63);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (FULL || lm.ok[r]) { la[u][r].load(a + (size_t)i * HF + lm.eoff[r]); lb[u][r].load(b + (size_t)j * HF + lm.eoff[r]); }
                else { la[u][r].zero(); lb[u][r].zero(); }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (t + u >= cnt) break;
            float d[R];
#pragma unroll
            for (int r = 0; r < R; ++r) d[r] = la[u][r].dot(lb[u][r]);
            size_t o = (size_t)(c + t + u) * H;
            if constexpr (LPH > 0) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    float s = fg_group_sum<LPH>(d[r]);
                    if ((FULL || lm.ok[r]) && lm.eoff[r] % F == 0) out[o + lm.hd[r]] = s;
                }
            } else {
                float s = H <= FGNN_FEW_HEADS ? fg_head_reduce_few<VEC, R>(d, lm, lane, H) : fg_head_reduce<VEC, R>(scr, d, lm, lane, H, F);
                if (lane < H) out[o + lane] = s;
            }
        }
    }
}

extern "C" int fgnn_sddmm_coo(int64_t E, int n_rows, int n_cols, int H, int F, const int32_t *row_ind, const int32_t *col_ind,
                              const float *a, const float *b, float *out, void *stream)
{
    FGNN_REQUIRE(E >= 0 && n_rows >= 0 && n_cols >= 0 && H >= 1 && F >= 1, FGNN_ERR_SHAPE, "fgnn_sddmm_coo: bad sizes");
    FGNN_REQUIRE(H <= 64 && (int64_t)H * F <= 1024, FGNN_ERR_LIMIT, "fgnn_sddmm_coo: H=%d H*F=%lld unsupported", H, (long long)H * F);
    FGNN_REQUIRE(E == 0 || (row_ind && col_ind && a && b && out), FGNN_ERR_NULL, "fgnn_sddmm_coo: NULL argument");
    FGNN_REQUIRE(E == 0 || (n_rows > 0 && n_cols > 0), FGNN_ERR_SHAPE, "fgnn_sddmm_coo: edges without nodes");
    if (E == 0) return 0;
    const int HF = H * F;
    fgnn_rowcfg cfg;
    FGNN_REQUIRE(fgnn_pick_rowcfg(HF, F, fgnn_aligned16(a) && fgnn_aligned16(b), &cfg), FGNN_ERR_LIMIT, "fgnn_sddmm_coo: unsupported row width %d", HF);
    const int lphp = fgnn_pad_lph(cfg.vec, H, F);
    if (lphp) { int w = H * lphp * 4; cfg.r = w <= 256 ? 1 : w <= 512 ? 2 : 4; cfg.full = false; }
    const int lph = lphp ? lphp : fgnn_pick_lph(cfg.vec, F);
    const int64_t waves = (E + 63) / 64;
    const unsigned grid = (unsigned)((waves + FGNN_WPB - 1) / FGNN_WPB);
    hipStream_t st = (hipStream_t)stream;
    return fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
        return fgnn_dispatch_lph(VEC == 4 ? lph : 0, [&]<int LPH>() -> int {
            hipLaunchKernelGGL((sddmm_coo_kernel<VEC, R, FULL, (VEC == 4 ? LPH : 0)>), dim3(grid), dim3(FGNN_TPB),
                               (size_t)FGNN_WPB * 64 * R * sizeof(float), st, E, H, F, HF, lphp, row_ind, col_ind, a, b, out);
            return fgnn_launch_status("sddmm_coo_kernel");
        });
    });
}

// out[q,:] = in[permute[q],:]  (src/csr2csc/mhtranspose.cu:6-47).  A row is G groups of VEC floats (VEC = 4: W % 4 == 0
// and 16-byte aligned arrays, 128-bit lanes); a wave takes RW consecutive output rows = at most 64 * GR_U groups, lane j of
// a trip owns group j of that span.  Its row inside the span is j / G by a multiply and a shift (inv = ceil(2^20 / G), exact
// for j * G < 2^20; spans of one row pass inv = 0), so there is no division per element, and the GR_U loads of a lane are
// all issued before the first store.  With per_xcd > 0 the workgroups of one XCD (blockIdx.x % FGNN_NUM_XCD) take one contiguous
// eighth of the output between them, in launch order: a 128-byte line of `in` holds several short rows, and when permute
// is the map of a transposition, rows that are neighbours in `in` are wanted by nearby outputs (the neighbouring columns of
// one matrix row) - close in time on ONE XCD's L2 instead of spread round-robin over eight that share nothing.
#define GR_U 8
template <int VEC>
__global__ __launch_bounds__(FGNN_TPB) void gather_rows_kernel(int64_t E, int G, int RW, unsigned inv, unsigned per_xcd, const int *__restrict__ permute,
                                                               const float *__restrict__ in, float *__restrict__ out)
{
    const unsigned chunk = per_xcd ? (blockIdx.x % FGNN_NUM_XCD) * per_xcd + blockIdx.x / FGNN_NUM_XCD : blockIdx.x;
    const int64_t q0 = ((int64_t)chunk * FGNN_WPB + fg_wave()) * RW;
    if (q0 >= E) return;
    const int rows = (int)min((int64_t)RW, E - q0);
    const int64_t n = (int64_t)rows * G;                 // groups of this wave: <= 64 * GR_U unless RW == 1
    const int lane = fg_lane();
    float *dst = out + (size_t)q0 * G * VEC;
    for (int64_t j0 = 0; j0 < n; j0 += 64 * GR_U) {
        fg_vec<VEC> v[GR_U];
        int src[GR_U];
        unsigned c[GR_U];
#pragma unroll
        for (int u = 0; u < GR_U; ++u) {
            const int64_t j = j0 + 64 * u + lane;
            const unsigned jj = j < n ? (unsigned)(j & 0x7fffffff) : 0u;       // RW > 1: j < 512
            const unsigned ql = inv ? (jj * inv) >> 20 : 0u;
            c[u] = inv ? jj - ql * (unsigned)G : 0u;
            src[u] = permute[q0 + ql];
        }
#pragma unroll
        for (int u = 0; u < GR_U; ++u) {
            const int64_t j = j0 + 64 * u + lane;
            const size_t col = inv ? (size_t)c[u] : (size_t)(j < n ? j : 0);
            v[u].load(in + ((size_t)src[u] * G + col) * VEC);
        }
#pragma unroll
        for (int u = 0; u < GR_U; ++u) {
            const int64_t j = j0 + 64 * u + lane;
            if (j < n) v[u].store_nt(dst + (size_t)j * VEC);
        }
    }
}

extern "C" int fgnn_gather_rows(int64_t E, int W, const int32_t *permute, const float *in, float *out, void *stream)
{
    FGNN_REQUIRE(E >= 0 && W >= 1, FGNN_ERR_SHAPE, "fgnn_gather_rows: bad sizes");
    FGNN_REQUIRE(E == 0 || (permute && in && out), FGNN_ERR_NULL, "fgnn_gather_rows: NULL argument");
    if (E == 0) return 0;
    const bool vec4 = W % 4 == 0 && fgnn_aligned16(in) && fgnn_aligned16(out);
    const int G = vec4 ? W / 4 : W;
    const int RW = G >= 64 * GR_U ? 1 : (64 * GR_U) / G;          // whole rows per wave
    const unsigned inv = RW > 1 ? (unsigned)(((1u << 20) + (unsigned)G - 1u) / (unsigned)G) : 0u;
    const int64_t waves = (E + RW - 1) / RW;
    const int64_t blocks = (waves + FGNN_WPB - 1) / FGNN_WPB;
    FGNN_REQUIRE(blocks <= 2147483647LL - FGNN_NUM_XCD, FGNN_ERR_LIMIT, "fgnn_gather_rows: too many rows");
    // rows shorter than a cache line, enough workgroups to matter, and a device whose workgroups go round the XCDs in turn
    const unsigned per_xcd = (G * (vec4 ? 16 : 4) < 128 && blocks >= 64 * FGNN_NUM_XCD && fgnn_current_device_has_xcd_mapping())
                                 ? (unsigned)((blocks + FGNN_NUM_XCD - 1) / FGNN_NUM_XCD) : 0u;
    const unsigned grid = per_xcd ? per_xcd * FGNN_NUM_XCD : (unsigned)blocks;
    if (vec4)
        hipLaunchKernelGGL(gather_rows_kernel<4>, dim3(grid), dim3(FGNN_TPB), 0, (hipStream_t)stream, E, G, RW, inv, per_xcd, permute, in, out);
    else
        hipLaunchKernelGGL(gather_rows_kernel<1>, dim3(grid), dim3(FGNN_TPB), 0, (hipStream_t)stream, E, G, RW, inv, per_xcd, permute, in, out);
    return fgnn_launch_status("gather_rows_kernel");
}

// ------------------------------------------------------------------- row reductions over [E, W] arrays, W <= 64
// A row's entries are one contiguous run of (pe - pb) * W floats.  Lanes t < S0 = (64 / W) * W of a
// wave take part and stride by a multiple of W, so lane t only ever sees column t % W and every
// load is a contiguous run of S0 floats.  Rows of up to SO_LONG_ELEMS floats are taken by one wave
// each, longer ones by a whole workgroup each: a 100 k-entry hub row is then a few hundred trips of a
// workgroup instead of tens of thousands of trips of one wave.  Both kinds run in ONE launch: its first
// workgroups each look at SO_CAND candidate rows (the first wave reads their lengths, a ballot names the
// long ones, the workgroup takes those one after the other), the workgroups behind them give one short
// row to each of their waves and fill the machine while the last long rows finish.  (On a 233 k-row
// power-law graph 31 k rows are long and hold 83 % of the entries; a workgroup per row would start
// 233 k workgroups of which seven in eight leave at once.)
#define SO_LONG_ELEMS 8192
#define SO_CAND 16            // candidate rows per workgroup of a long-row launch
// Registers a row-reduction kernel spends on a row: CACHE groups of VEC floats per lane kept over both phases by a wave on a short
// row, CLONG by the workgroup on a long row, STREAM loads in flight per lane in the part of a row that is streamed.  The numbers
// set the kernel's register count and with it the waves resident per SIMD: rows that mostly fit one trip of a wave want a small
// footprint (each row is a chain of dependent memory round trips, and only the rows in flight hide it), rows of thousands of
// values want the cache (what is not cached is read twice).  A launch picks between a configuration for dense rows and one for
// sparse rows by the mean row length.  Measured (softmax / backward / scatter / gather-row, ms; [cache, long cache, stream]):
//   114.8 M entries in 233 k rows, 8 heads:  [8,16,8] 1.79 / 2.49 / 3.60 / 4.07   [4,8,4] 1.85 / 2.70 / 2.56 / 3.56   [2,4,4] 1.97 / 2.89 / 2.67 / 3.74
//   64.3 M entries in 2.45 M rows, 8 heads:  [8,16,8] 3.13 / 3.61 / 6.92 / 7.34   [4,8,4] 2.50 / 2.41 / 3.58 / 4.07   [2,4,4] 2.01 / 2.00 / 3.55 / 3.53
// L: lanes a short row gets (64: a wave per row; 32, 16, 8: a wave takes 64 / L rows side by side, each in its own group of L
// lanes - where the mean row fills a fraction of a wave's trip, the per-row chain of dependent loads is shared by 2-8 rows).
template <int CACHE_, int CLONG_, int STREAM_, int L_ = 64> struct so_cfg { static constexpr int CACHE = CACHE_, CLONG = CLONG_, STREAM = STREAM_, L = L_; };
#define SO_DENSE_ROW_FLOATS 1024          // mean floats per row from which a launch takes its dense-row configuration
static inline bool so_dense_rows(int N, int64_t elems) { return elems >= (int64_t)SO_DENSE_ROW_FLOATS * N; }
// Lanes a short row gets in the sparse configuration, from the mean row length in groups of VEC floats.  Rows of a power-law graph
// scatter widely about their mean, so a group is sized generously: 32 lanes down to a mean of 12 groups.  Measured on 64.3 M
// entries in 2.45 M rows (softmax / backward / scatter / gather-row, ms; lanes 64 | 32 | 16 | 8):
//   8 heads (mean 53 groups of four floats): 1.97 / 1.92 / 3.00 / 3.60 | 1.58 / 1.83 / 2.74 / 3.17 | 1.47 / 1.97 / 3.14 / 3.56 | 1.67 / 2.40 / 4.24 / 4.72
//   1 head (mean 26 floats):                  1.05 / 1.09 / 1.67 / 1.46 | 0.71 / 0.89 / 1.51 / 1.29 | 0.65 / 0.99 / 1.82 / 1.49 | 0.76 / 1.34 / 2.71 / 2.10
static inline int so_pick_lanes(int N, int64_t elems, int vec, int W)
{
    const int64_t mean_groups = elems / vec / std::max(N, 1);
    int L = mean_groups > 64 ? 64 : mean_groups > 12 ? 32 : mean_groups > 6 ? 16 : 8;
    while (L < W) L *= 2;                                   // a group holds at least one entry
    return L;
}
// launch.operator()<VEC, CFG>() with VEC = 4 or 1 and CFG = the `dense` type of the calling scope or so_cfg<SP_CACHE, SP_CLONG,
// SP_STREAM, lanes> from its constants
#define SO_LAUNCH_CFG(launch, vec4, ...) do { if (vec4) launch.template operator()<4, __VA_ARGS__>(); else launch.template operator()<1, __VA_ARGS__>(); } while (0)
#define SO_LAUNCH_BY_ROWS(launch, vec4, is_dense, lanes)                                              \
    do {                                                                                              \
        if (is_dense) SO_LAUNCH_CFG(launch, vec4, dense);                                             \
        else if ((lanes) == 32) SO_LAUNCH_CFG(launch, vec4, so_cfg<SP_CACHE, SP_CLONG, SP_STREAM, 32>); \
        else if ((lanes) == 16) SO_LAUNCH_CFG(launch, vec4, so_cfg<SP_CACHE, SP_CLONG, SP_STREAM, 16>); \
        else if ((lanes) == 8) SO_LAUNCH_CFG(launch, vec4, so_cfg<SP_CACHE, SP_CLONG, SP_STREAM, 8>);   \
        else SO_LAUNCH_CFG(launch, vec4, so_cfg<SP_CACHE, SP_CLONG, SP_STREAM, 64>);                    \
    } while (0)

// Threads of the workgroups of a row-reduction launch and the grid: n_long workgroups for the long-row candidates, then one
// short row per wave.  More, smaller workgroups keep more long rows in flight per compute unit (a workgroup works through
// its rows one after the other, each a chain of dependent memory round trips); larger ones hold more of a row in registers.
// Measured on a 115 M-entry power-law graph, 8 heads (128 / 256 / 512 threads): softmax 1.93 / 1.78 / 1.84 ms, its backward
// 3.29 / 2.77 / 2.48, the scatter kernel 3.93 / 3.60 / 4.43, gather-row 4.03 / 4.06 / 4.83, row sums 1.08 / 0.79 / 0.66.
static inline unsigned so_grid(int N, int64_t elems, int tpb, unsigned *n_long, int lanes_per_row = 64)
{
    *n_long = elems > SO_LONG_ELEMS ? (unsigned)((N + SO_CAND - 1) / SO_CAND) : 0u;      // otherwise no row can be long
    const int rows_per_block = (tpb / 64) * (64 / lanes_per_row);
    return *n_long + (unsigned)((N + rows_per_block - 1) / rows_per_block);
}

struct so_max { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct so_add { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };

template <int VEC> struct so_grp { float c[VEC]; };

// Combines, per component, the values of the lanes t, t + W, t + 2W, ... < S0 (any count, by suffix doubling) and
// of the workgroup's NW waves in a fixed order; every lane gets the result of its column.  W * VEC <= 64.
template <int NW, int VEC, class Op>      // NW: waves that share the row (1: a single wave, no LDS step)
__device__ __forceinline__ so_grp<VEC> so_column_reduce(so_grp<VEC> v, int lane, int W, int S0, float (*sh)[64], Op op)
{
    for (int off = W; off < S0; off <<= 1) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            const float o = __shfl(v.c[c], (lane + off) & 63);
            if (lane + off < S0) v.c[c] = op(v.c[c], o);
        }
    }
    const int col = lane % W;
#pragma unroll
    for (int c = 0; c < VEC; ++c) v.c[c] = __shfl(v.c[c], col);
    if constexpr (NW > 1) {
        const int w = fg_wave();
        if (lane < W) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) sh[w][c * W + lane] = v.c[c];
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            float r = sh[0][c * W + col];
            for (int i = 1; i < NW; ++i) r = op(r, sh[i][c * W + col]);
            v.c[c] = r;
        }
        __syncthreads();
    }
    return v;
}

// The same combination inside aligned groups of L lanes (L a power of two, W <= L): group-relative lane sl = lane % L, the lanes
// sl, sl + W, ... < S0 = (L / W) * W of a group are combined and every lane of the group gets the result of its column.
template <int VEC, int L, class Op>
__device__ __forceinline__ so_grp<VEC> so_group_reduce(so_grp<VEC> v, int lane, int W, int S0, Op op)
{
    const int sl = lane & (L - 1);
    for (int off = W; off < S0; off <<= 1) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            const float o = __shfl(v.c[c], (lane + off) & 63);          // used only where sl + off < S0 <= L: the same group
            if (sl + off < S0) v.c[c] = op(v.c[c], o);
        }
    }
    const int src = lane - sl + sl % W;
#pragma unroll
    for (int c = 0; c < VEC; ++c) v.c[c] = __shfl(v.c[c], src);
    return v;
}

// Work unit u (a wave of the short launch, a candidate of the long launch) takes row (u * p) mod N with p a prime
// above 2^31: a bijection of [0, N) that scatters neighbouring rows.  Workgroups go to the eight XCDs round-robin, and on a
// power-law graph generated by recursive quadrants a row's length follows the low bits of its number (the
// rows = 0 mod 8 of an R-MAT graph hold 44 % of the entries): in row order one XCD would get most of the work.
__device__ __forceinline__ int so_scattered_row(unsigned u, int N) { return (int)(((unsigned long long)u * 2654435761ull) % (unsigned)N); }

// Short launch: the row of this wave, false when it is empty or belongs to the long launch.  W counts the groups of VEC
// floats per entry, n the groups of the row.
template <int VEC>
__device__ __forceinline__ bool so_take_short_row(unsigned u, int N, int W, const int *ptr, int &row, int &pb, int64_t &n)
{
    if (u >= (unsigned)N) return false;
    row = fg_uni(so_scattered_row(u, N));
    pb = fg_uni(ptr[row]);
    n = (int64_t)(fg_uni(ptr[row + 1]) - pb) * W;
    return n * VEC <= SO_LONG_ELEMS;
}
// Short launch with groups of L < 64 lanes: group g of work unit u takes row (u * 64 / L + g) scattered as above; n = 0 marks a group
// without a row of its own (past the end, empty, or a long row).  False when no group of the wave has one.
template <int VEC, int L>
__device__ __forceinline__ bool so_take_short_rows(unsigned u, int N, int W, const int *ptr, int &row, int &pb, int64_t &n, bool &mine)
{
    const unsigned v = u * (64 / L) + (unsigned)fg_lane() / L;
    mine = v < (unsigned)N;
    row = mine ? so_scattered_row(v, N) : 0;
    pb = mine ? ptr[row] : 0;
    n = mine ? (int64_t)(ptr[row + 1] - pb) * W : 0;
    if (n * VEC > SO_LONG_ELEMS) { n = 0; mine = false; }          // the long launch has it
    return __builtin_amdgcn_ballot_w64(mine) != 0ull;
}
// Long launch: bit l of the result is set when candidate blockIdx.x * SO_CAND + l is a long row (uniform over the workgroup).
template <int VEC>
__device__ __forceinline__ unsigned long long so_long_candidates(int N, int W, const int *ptr, unsigned long long *sh_mask)
{
    if (fg_wave() == 0) {
        const unsigned u = blockIdx.x * SO_CAND + (unsigned)fg_lane();
        bool lng = false;
        if (fg_lane() < SO_CAND && u < (unsigned)N) {
            const int r = so_scattered_row(u, N);
            lng = (int64_t)(ptr[r + 1] - ptr[r]) * W * VEC > SO_LONG_ELEMS;
        }
        const unsigned long long m = __builtin_amdgcn_ballot_w64(lng);
        if (fg_lane() == 0) *sh_mask = m;
    }
    __syncthreads();
    const unsigned long long m = *sh_mask;
    return ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(m >> 32)) << 32) | (unsigned)__builtin_amdgcn_readfirstlane((int)m);
}

template <int VEC> __device__ __forceinline__ so_grp<VEC> so_load(const float *p)
{
    so_grp<VEC> r;
    if constexpr (VEC == 4) { const float4 t = *reinterpret_cast<const float4 *>(p); r.c[0] = t.x; r.c[1] = t.y; r.c[2] = t.z; r.c[3] = t.w; }
    else r.c[0] = *p;
    return r;
}
template <int VEC> __device__ __forceinline__ void so_store(float *p, const so_grp<VEC> &r)
{
    if constexpr (VEC == 4) *reinterpret_cast<float4 *>(p) = make_float4(r.c[0], r.c[1], r.c[2], r.c[3]);
    else *p = r.c[0];
}
template <int VEC> __device__ __forceinline__ so_grp<VEC> so_fill(float x)
{
    so_grp<VEC> r;
#pragma unroll
    for (int c = 0; c < VEC; ++c) r.c[c] = x;
    return r;
}

// Per-row, per-head softmax over [E,H] (src/edge_softmax/edge_softmax.cu:7-61) and its backward
// s*(g - sum_row s*g) (:63-98).  VEC = 4 (H % 4 == 0, 16-byte aligned arrays): a lane owns four consecutive
// heads of an entry.  One row: the first CACHE groups of a lane stay in registers over both phases; what a longer
// row has beyond them is folded into a running (maximum, sum) pair while it streams by (one read instead of a
// maximum pass and a sum pass) and read once more for the result.
// Where a row's values come from.  load(k, first): group k of the row (lane t only ever asks for groups with k % W == t % W);
// first = false on the second read of a group that did not fit the registers.
template <int VEC> struct so_from_array {
    const float *p;         // the row's first value
    __device__ __forceinline__ so_grp<VEC> load(int64_t k, bool) const { return so_load<VEC>(p + k * VEC); }
};
// lrelu(attn_row[row, h] + attn_col[col_ind[entry], h]): the scores of the fuse-scatter GAT forward, formed on the fly
// (src/fused_gat/fused_gat.cu:235-300 reads them back from the edge_relu array it has just written).
template <int VEC> struct so_from_scores {
    const int *idx;         // col_ind of the row's first entry
    const float *ac;        // attn_col
    float *elrelu;          // where the row's LeakyReLU values go (NULL: nowhere)
    so_grp<VEC> ar;         // attn_row[row, this lane's heads]
    int W, col;             // groups per entry, this lane's group
    float slope;
    __device__ __forceinline__ so_grp<VEC> load(int64_t k, bool first) const
    {
        const unsigned e = (unsigned)k / (unsigned)W;                  // k is relative to the row: fits 32 bits
        so_grp<VEC> v = so_load<VEC>(ac + ((size_t)idx[e] * W + col) * VEC);
#pragma unroll
        for (int c = 0; c < VEC; ++c) { const float x = v.c[c] + ar.c[c]; v.c[c] = x > 0.f ? x : x * slope; }
        if (first && elrelu) so_store<VEC>(elrelu + k * VEC, v);
        return v;
    }
};

template <int NW, int VEC, int CACHE, int STREAM, class Src, int L = 64>          // L < 64 (NW == 1): n, src and dst are per group of L lanes
__device__ __forceinline__ void so_softmax_row(int W, int64_t n, const Src &src, float *dst, float (*sh)[64])
{
    static_assert(L == 64 || NW == 1, "lane groups only where one wave has the row");
    const int lane = fg_lane(), sl = lane & (L - 1), S0 = (L / W) * W;
    const int64_t first = (NW > 1 ? fg_wave() * S0 : 0) + sl, step = (int64_t)S0 * NW;
    const bool act = sl < S0;
    auto reduce = [&](so_grp<VEC> v, auto op) {
        if constexpr (L < 64) return so_group_reduce<VEC, L>(v, lane, W, S0, op);
        else return so_column_reduce<NW, VEC>(v, lane, W, S0, sh, op);
    };
    so_grp<VEC> v[CACHE], m = so_fill<VEC>(-INFINITY), s = so_fill<VEC>(0.f);
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int64_t k = first + i * step;
        v[i] = (act && k < n) ? src.load(k, true) : so_fill<VEC>(-INFINITY);
    }
#pragma unroll
    for (int i = 0; i < CACHE; ++i)
#pragma unroll
        for (int c = 0; c < VEC; ++c) m.c[c] = fmaxf(m.c[c], v[i].c[c]);
    const int64_t rest = first + CACHE * step;
    // a lane that gets here has CACHE valid groups, so its m is finite and m - max(m, t) is never inf - inf.
    // STREAM loads are issued before the first is used: a row that one workgroup streams alone is bound by the
    // bytes it keeps in flight.
    if (act) {
        for (int64_t k0 = rest; k0 < n; k0 += STREAM * step) {
            so_grp<VEC> t[STREAM];
#pragma unroll
            for (int j = 0; j < STREAM; ++j) t[j] = k0 + j * step < n ? src.load(k0 + j * step, true) : so_fill<VEC>(-INFINITY);
            so_grp<VEC> mn = m;
#pragma unroll
            for (int j = 0; j < STREAM; ++j)
#pragma unroll
                for (int c = 0; c < VEC; ++c) mn.c[c] = fmaxf(mn.c[c], t[j].c[c]);
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                float acc = s.c[c] * __expf(m.c[c] - mn.c[c]);
#pragma unroll
                for (int j = 0; j < STREAM; ++j) acc += __expf(t[j].c[c] - mn.c[c]);       // exp(-inf) = 0 past the row
                s.c[c] = acc;
                m.c[c] = mn.c[c];
            }
        }
    }
    const so_grp<VEC> mall = reduce(m, so_max());
#pragma unroll
    for (int c = 0; c < VEC; ++c) s.c[c] = s.c[c] > 0.f ? s.c[c] * __expf(m.c[c] - mall.c[c]) : 0.f;      // the streamed part, rebased
#pragma unroll
    for (int i = 0; i < CACHE; ++i)
#pragma unroll
        for (int c = 0; c < VEC; ++c) { v[i].c[c] = __expf(v[i].c[c] - mall.c[c]); s.c[c] += v[i].c[c]; }      // exp(-inf) = 0 past the row
    so_grp<VEC> inv = reduce(s, so_add());
#pragma unroll
    for (int c = 0; c < VEC; ++c) inv.c[c] = 1.f / inv.c[c];
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int64_t k = first + i * step;
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[i].c[c] *= inv.c[c];
        if (act && k < n) so_store<VEC>(dst + k * VEC, v[i]);
    }
    if (act) {
        for (int64_t k0 = rest; k0 < n; k0 += STREAM * step) {
            so_grp<VEC> t[STREAM];
#pragma unroll
            for (int j = 0; j < STREAM; ++j) t[j] = k0 + j * step < n ? src.load(k0 + j * step, false) : so_fill<VEC>(0.f);
#pragma unroll
            for (int j = 0; j < STREAM; ++j) {
#pragma unroll
                for (int c = 0; c < VEC; ++c) t[j].c[c] = __expf(t[j].c[c] - mall.c[c]) * inv.c[c];
                if (k0 + j * step < n) so_store<VEC>(dst + (k0 + j * step) * VEC, t[j]);
            }
        }
    }
}

// One launch for both kinds of row: the first n_long_blocks workgroups take the long rows among their SO_CAND candidates
// (they start first, so the longest rows are not left for the end), the workgroups after them give one short row to each
// of their eight waves.
template <int VEC, int TPB, class CFG>
__global__ __launch_bounds__(TPB) void edge_softmax_kernel(int N, int W, unsigned n_long_blocks, const int *__restrict__ ptr,
                                                                   const float *__restrict__ in, float *__restrict__ out)
{
    __shared__ float sh[TPB / 64][64];
    __shared__ unsigned long long sh_mask;
    if (blockIdx.x < n_long_blocks) {
        for (unsigned long long m = so_long_candidates<VEC>(N, W, ptr, &sh_mask); m; m &= m - 1) {
            const int row = so_scattered_row(blockIdx.x * SO_CAND + (unsigned)__builtin_ctzll(m), N);
            const int pb = fg_uni(ptr[row]);
            so_softmax_row<TPB / 64, VEC, CFG::CLONG, CFG::STREAM>(W, (int64_t)(fg_uni(ptr[row + 1]) - pb) * W, so_from_array<VEC>{in + (size_t)pb * W * VEC},
                                                     out + (size_t)pb * W * VEC, sh);
        }
        return;
    }
    int row, pb;
    int64_t n;
    const unsigned u = (unsigned)fg_uni((int)((blockIdx.x - n_long_blocks) * (TPB / 64)) + fg_wave());
    if constexpr (CFG::L < 64) {
        bool mine;
        if (!so_take_short_rows<VEC, CFG::L>(u, N, W, ptr, row, pb, n, mine)) return;
        so_softmax_row<1, VEC, CFG::CACHE, CFG::STREAM, so_from_array<VEC>, CFG::L>(W, n, so_from_array<VEC>{in + (size_t)pb * W * VEC},
                                                                                     out + (size_t)pb * W * VEC, nullptr);
        return;
    }
    if (!so_take_short_row<VEC>(u, N, W, ptr, row, pb, n) || n == 0) return;
    so_softmax_row<1, VEC, CFG::CACHE, CFG::STREAM>(W, n, so_from_array<VEC>{in + (size_t)pb * W * VEC}, out + (size_t)pb * W * VEC, nullptr);
}

// The fuse-scatter GAT forward (fused_scatter_kernel, src/fused_gat/fused_gat.cu:235-300): scores, LeakyReLU and the row softmax in
// one pass that writes e_softmax [E,H] (and e_lrelu when asked for).
template <int VEC, int TPB, class CFG>
__global__ __launch_bounds__(TPB) void gat_scatter_kernel(int N, int W, unsigned n_long_blocks, const int *__restrict__ ptr,
                                                                  const int *__restrict__ idx, const float *__restrict__ ar,
                                                                  const float *__restrict__ ac, float slope, float *__restrict__ elrelu,
                                                                  float *__restrict__ esoft)
{
    __shared__ float sh[TPB / 64][64];
    __shared__ unsigned long long sh_mask;
    auto source = [&](int row, int pb, int col) {
        so_from_scores<VEC> src;
        src.idx = idx + pb; src.ac = ac; src.elrelu = elrelu ? elrelu + (size_t)pb * W * VEC : nullptr;
        src.ar = so_load<VEC>(ar + ((size_t)row * W + col) * VEC);
        src.W = W; src.col = col; src.slope = slope;
        return src;
    };
    const int col = fg_lane() % W;
    if (blockIdx.x < n_long_blocks) {
        for (unsigned long long m = so_long_candidates<VEC>(N, W, ptr, &sh_mask); m; m &= m - 1) {
            const int row = so_scattered_row(blockIdx.x * SO_CAND + (unsigned)__builtin_ctzll(m), N);
            const int pb = fg_uni(ptr[row]);
            so_softmax_row<TPB / 64, VEC, CFG::CLONG, CFG::STREAM>(W, (int64_t)(fg_uni(ptr[row + 1]) - pb) * W, source(row, pb, col), esoft + (size_t)pb * W * VEC, sh);
        }
        return;
    }
    int row, pb;
    int64_t n;
    const unsigned u = (unsigned)fg_uni((int)((blockIdx.x - n_long_blocks) * (TPB / 64)) + fg_wave());
    if constexpr (CFG::L < 64) {
        bool mine;
        if (!so_take_short_rows<VEC, CFG::L>(u, N, W, ptr, row, pb, n, mine)) return;
        so_softmax_row<1, VEC, CFG::CACHE, CFG::STREAM, so_from_scores<VEC>, CFG::L>(W, n, source(row, pb, (fg_lane() & (CFG::L - 1)) % W),
                                                                                      esoft + (size_t)pb * W * VEC, nullptr);
        return;
    }
    if (!so_take_short_row<VEC>(u, N, W, ptr, row, pb, n) || n == 0) return;
    so_softmax_row<1, VEC, CFG::CACHE, CFG::STREAM>(W, n, source(row, pb, col), esoft + (size_t)pb * W * VEC, nullptr);
}

// The factor LeakyReLU' puts on an entry's gradient, for the fused gather_row pass of the fuse-scatter GAT backward
// (src/fused_gat/fused_gat.cu:502-556): none (plain softmax backward), from the stashed LeakyReLU values, or from the
// sign of attn_row + attn_col formed again (no [E,H] array is read for it).
template <int VEC> struct so_sign_none {
    static constexpr bool active = false;
    __device__ __forceinline__ so_grp<VEC> factor(int64_t) const { return so_fill<VEC>(1.f); }
};
template <int VEC> struct so_sign_array {
    static constexpr bool active = true;
    const float *elrelu; float slope;          // the row's first LeakyReLU value
    __device__ __forceinline__ so_grp<VEC> factor(int64_t k) const
    {
        so_grp<VEC> v = so_load<VEC>(elrelu + k * VEC);
#pragma unroll
        for (int c = 0; c < VEC; ++c) v.c[c] = v.c[c] > 0.f ? 1.f : slope;      // a pre-activation of exactly 0 takes the slope, as torch's LeakyReLU does
        return v;
    }
};
template <int VEC> struct so_sign_scores {
    static constexpr bool active = true;
    const int *idx; const float *ac; so_grp<VEC> ar; int W, col; float slope;
    __device__ __forceinline__ so_grp<VEC> factor(int64_t k) const
    {
        const unsigned e = (unsigned)k / (unsigned)W;
        so_grp<VEC> v = so_load<VEC>(ac + ((size_t)idx[e] * W + col) * VEC);
#pragma unroll
        for (int c = 0; c < VEC; ++c) v.c[c] = v.c[c] + ar.c[c] > 0.f ? 1.f : slope;
        return v;
    }
};

// gin = factor * sm * (g - sum_row sm * g); with an active Sign also rowsum[lane's heads] = sum_row gin (the grad_attn_row of
// the fuse-scatter backward).  gin may be g itself: every value is read before it is overwritten, by the same lane.
template <int NW, int VEC, int CACHE, int STREAM, class Sign, int L = 64>         // L < 64 (NW == 1): pb, n, sign and rowsum are per group of L lanes
__device__ __forceinline__ void so_softmax_bwd_row(int W, int pb, int64_t n, const float *__restrict__ sm, const float *g,
                                                   float *gin, const Sign &sign, float *rowsum, float (*sh)[64])
{
    static_assert(L == 64 || NW == 1, "lane groups only where one wave has the row");
    const int lane = fg_lane(), sl = lane & (L - 1), S0 = (L / W) * W;
    const int64_t first = (NW > 1 ? fg_wave() * S0 : 0) + sl, step = (int64_t)S0 * NW;
    const bool act = sl < S0;
    auto reduce = [&](so_grp<VEC> v, auto op) {
        if constexpr (L < 64) return so_group_reduce<VEC, L>(v, lane, W, S0, op);
        else return so_column_reduce<NW, VEC>(v, lane, W, S0, sh, op);
    };
    const size_t base = (size_t)pb * W * VEC;
    so_grp<VEC> sv[CACHE], gv[CACHE], acc = so_fill<VEC>(0.f);
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int64_t k = first + i * step;
        const bool ok = act && k < n;
        sv[i] = ok ? so_load<VEC>(sm + base + k * VEC) : so_fill<VEC>(0.f);
        gv[i] = ok ? so_load<VEC>(g + base + k * VEC) : so_fill<VEC>(0.f);
    }
#pragma unroll
    for (int i = 0; i < CACHE; ++i)
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc.c[c] = fmaf(sv[i].c[c], gv[i].c[c], acc.c[c]);
    const int64_t rest = first + CACHE * step;
    if (act) {
        for (int64_t k0 = rest; k0 < n; k0 += STREAM * step) {
            so_grp<VEC> a[STREAM], b[STREAM];
#pragma unroll
            for (int j = 0; j < STREAM; ++j) {
                const bool ok = k0 + j * step < n;
                a[j] = ok ? so_load<VEC>(sm + base + (k0 + j * step) * VEC) : so_fill<VEC>(0.f);
                b[j] = ok ? so_load<VEC>(g + base + (k0 + j * step) * VEC) : so_fill<VEC>(0.f);
            }
#pragma unroll
            for (int j = 0; j < STREAM; ++j)
#pragma unroll
                for (int c = 0; c < VEC; ++c) acc.c[c] = fmaf(a[j].c[c], b[j].c[c], acc.c[c]);
        }
    }
    acc = reduce(acc, so_add());
    so_grp<VEC> rs = so_fill<VEC>(0.f);
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int64_t k = first + i * step;
        const bool ok = act && k < n;
#pragma unroll
        for (int c = 0; c < VEC; ++c) sv[i].c[c] *= gv[i].c[c] - acc.c[c];
        if constexpr (Sign::active) {
            if (ok) {
                const so_grp<VEC> f = sign.factor(k);
#pragma unroll
                for (int c = 0; c < VEC; ++c) { sv[i].c[c] *= f.c[c]; rs.c[c] += sv[i].c[c]; }
            }
        }
        if (ok) so_store<VEC>(gin + base + k * VEC, sv[i]);
    }
    if (act) {
        for (int64_t k0 = rest; k0 < n; k0 += STREAM * step) {
            so_grp<VEC> a[STREAM], b[STREAM];
#pragma unroll
            for (int j = 0; j < STREAM; ++j) {
                const bool ok = k0 + j * step < n;
                a[j] = ok ? so_load<VEC>(sm + base + (k0 + j * step) * VEC) : so_fill<VEC>(0.f);
                b[j] = ok ? so_load<VEC>(g + base + (k0 + j * step) * VEC) : so_fill<VEC>(0.f);
            }
#pragma unroll
            for (int j = 0; j < STREAM; ++j) {
                const bool ok = k0 + j * step < n;
#pragma unroll
                for (int c = 0; c < VEC; ++c) a[j].c[c] *= b[j].c[c] - acc.c[c];
                if constexpr (Sign::active) {
                    if (ok) {
                        const so_grp<VEC> f = sign.factor(k0 + j * step);
#pragma unroll
                        for (int c = 0; c < VEC; ++c) { a[j].c[c] *= f.c[c]; rs.c[c] += a[j].c[c]; }
                    }
                }
                if (ok) so_store<VEC>(gin + base + (k0 + j * step) * VEC, a[j]);
            }
        }
    }
    if constexpr (Sign::active) {
        rs = reduce(rs, so_add());
        if (sl < W && rowsum && (NW == 1 || fg_wave() == 0)) so_store<VEC>(rowsum + (size_t)sl * VEC, rs);      // rowsum == NULL: a group without a row
    }
}

template <int VEC, int TPB, class CFG>
__global__ __launch_bounds__(TPB) void edge_softmax_bwd_kernel(int N, int W, unsigned n_long_blocks, const int *__restrict__ ptr,
                                                                       const float *__restrict__ sm, const float *__restrict__ g,
                                                                       float *__restrict__ gin)
{
    __shared__ float sh[TPB / 64][64];
    __shared__ unsigned long long sh_mask;
    if (blockIdx.x < n_long_blocks) {
        for (unsigned long long m = so_long_candidates<VEC>(N, W, ptr, &sh_mask); m; m &= m - 1) {
            const int row = so_scattered_row(blockIdx.x * SO_CAND + (unsigned)__builtin_ctzll(m), N);
            const int pb = fg_uni(ptr[row]);
            so_softmax_bwd_row<TPB / 64, VEC, CFG::CACHE, CFG::STREAM>(W, pb, (int64_t)(fg_uni(ptr[row + 1]) - pb) * W, sm, g, gin, so_sign_none<VEC>{}, nullptr, sh);
        }
        return;
    }
    int row, pb;
    int64_t n;
    const unsigned u = (unsigned)fg_uni((int)((blockIdx.x - n_long_blocks) * (TPB / 64)) + fg_wave());
    if constexpr (CFG::L < 64) {
        bool mine;
        if (!so_take_short_rows<VEC, CFG::L>(u, N, W, ptr, row, pb, n, mine)) return;
        so_softmax_bwd_row<1, VEC, CFG::CACHE, CFG::STREAM, so_sign_none<VEC>, CFG::L>(W, pb, n, sm, g, gin, so_sign_none<VEC>{}, nullptr, nullptr);
        return;
    }
    if (!so_take_short_row<VEC>(u, N, W, ptr, row, pb, n) || n == 0) return;
    so_softmax_bwd_row<1, VEC, CFG::CACHE, CFG::STREAM>(W, pb, n, sm, g, gin, so_sign_none<VEC>{}, nullptr, nullptr);
}

// fused_gather_row of the fuse-scatter GAT backward (src/fused_gat/fused_gat.cu:502-556): softmax backward, LeakyReLU backward
// and the row sums (grad_attn_row) in one pass; gout may be g (in place).  Rows without entries get a zero row sum.
template <int VEC, bool FROM_ARRAY, int TPB, class CFG>
__global__ __launch_bounds__(TPB) void gat_gather_row_kernel(int N, int W, unsigned n_long_blocks, const int *__restrict__ ptr,
                                                                     const int *__restrict__ idx, const float *__restrict__ ar,
                                                                     const float *__restrict__ ac, const float *__restrict__ elrelu, float slope,
                                                                     const float *__restrict__ sm, const float *g, float *gout,
                                                                     float *__restrict__ gar)
{
    __shared__ float sh[TPB / 64][64];
    __shared__ unsigned long long sh_mask;
    // L: lanes per row (64 except on the packed short path); mine: the lane group has a row whose sums it stores
    auto run = [&]<int NW, int L>(int row, int pb, int64_t n, bool mine, float (*shp)[64]) {
        float *rowsum = mine ? gar + (size_t)row * W * VEC : nullptr;
        const int col = (fg_lane() & (L - 1)) % W;
        if constexpr (FROM_ARRAY) {
            so_softmax_bwd_row<NW, VEC, CFG::CACHE, CFG::STREAM, so_sign_array<VEC>, L>(W, pb, n, sm, g, gout, so_sign_array<VEC>{elrelu + (size_t)pb * W * VEC, slope},
                                                                                      rowsum, shp);
        } else {
            so_sign_scores<VEC> sg;
            sg.idx = idx + pb; sg.ac = ac; sg.ar = so_load<VEC>(ar + ((size_t)row * W + col) * VEC); sg.W = W; sg.col = col; sg.slope = slope;
            so_softmax_bwd_row<NW, VEC, CFG::CACHE, CFG::STREAM, so_sign_scores<VEC>, L>(W, pb, n, sm, g, gout, sg, rowsum, shp);
        }
    };
    if (blockIdx.x < n_long_blocks) {
        for (unsigned long long m = so_long_candidates<VEC>(N, W, ptr, &sh_mask); m; m &= m - 1) {
            const int row = so_scattered_row(blockIdx.x * SO_CAND + (unsigned)__builtin_ctzll(m), N);
            const int pb = fg_uni(ptr[row]);
            run.template operator()<TPB / 64, 64>(row, pb, (int64_t)(fg_uni(ptr[row + 1]) - pb) * W, true, sh);
        }
        return;
    }
    int row, pb;
    int64_t n;
    const unsigned u = (unsigned)fg_uni((int)((blockIdx.x - n_long_blocks) * (TPB / 64)) + fg_wave());
    if constexpr (CFG::L < 64) {
        bool mine;
        if (!so_take_short_rows<VEC, CFG::L>(u, N, W, ptr, row, pb, n, mine)) return;
        run.template operator()<1, CFG::L>(row, pb, n, mine, nullptr);
        return;
    }
    if (!so_take_short_row<VEC>(u, N, W, ptr, row, pb, n)) return;
    run.template operator()<1, 64>(row, pb, n, true, nullptr);             // an empty row stores its zero sums
}

// More than 64 heads: one wave per row, one head at a time.
__global__ __launch_bounds__(FGNN_TPB) void edge_softmax_wide_kernel(int N, int H, const int *ptr, const float *in, float *out)
{
    int row = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (row >= N) return;
    const int lane = fg_lane();
    const int pb = fg_uni(ptr[row]), pe = fg_uni(ptr[row + 1]);
    for (int h = 0; h < H; ++h) {
        float m = -INFINITY;
        for (int q = pb + lane; q < pe; q += 64) m = fmaxf(m, in[(size_t)q * H + h]);
        m = fg_wave_max(m);
        float s = 0.f;
        for (int q = pb + lane; q < pe; q += 64) s += __expf(in[(size_t)q * H + h] - m);
        s = fg_wave_sum(s);
        float inv = 1.f / s;
        for (int q = pb + lane; q < pe; q += 64) out[(size_t)q * H + h] = __expf(in[(size_t)q * H + h] - m) * inv;
    }
}

__global__ __launch_bounds__(FGNN_TPB) void edge_softmax_bwd_wide_kernel(int N, int H, const int *ptr, const float *sm, const float *g, float *gin)
{
    int row = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (row >= N) return;
    const int lane = fg_lane();
    const int pb = fg_uni(ptr[row]), pe = fg_uni(ptr[row + 1]);
    for (int h = 0; h < H; ++h) {
        float acc = 0.f;
        for (int q = pb + lane; q < pe; q += 64) acc += sm[(size_t)q * H + h] * g[(size_t)q * H + h];
        acc = fg_wave_sum(acc);
        for (int q = pb + lane; q < pe; q += 64) {
            size_t o = (size_t)q * H + h;
            gin[o] = sm[o] * (g[o] - acc);
        }
    }
}

extern "C" int fgnn_edge_softmax(int N, int64_t E, int H, const int32_t *row_ptr, const float *in, float *out, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1, FGNN_ERR_SHAPE, "fgnn_edge_softmax: bad sizes");
    FGNN_REQUIRE(row_ptr && (E == 0 || (in && out)), FGNN_ERR_NULL, "fgnn_edge_softmax: NULL argument");
    if (N == 0 || E == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    const unsigned waves = (unsigned)((N + FGNN_WPB - 1) / FGNN_WPB);
    if (H > 64) {
        hipLaunchKernelGGL(edge_softmax_wide_kernel, dim3(waves), dim3(FGNN_TPB), 0, st, N, H, row_ptr, in, out);
        return fgnn_launch_status("edge_softmax_wide_kernel");
    }
    constexpr int TPB = 256;
    const bool vec4 = H % 4 == 0 && fgnn_aligned16(in) && fgnn_aligned16(out);
    auto launch = [&]<int VEC, class CFG>() {
        unsigned n_long;
        const unsigned grid = so_grid(N, E * H, TPB, &n_long, CFG::L);
        hipLaunchKernelGGL((edge_softmax_kernel<VEC, TPB, CFG>), dim3(grid), dim3(TPB), 0, st, N, H / VEC, n_long, row_ptr, in, out);
    };
    using dense = so_cfg<8, 16, 8>;
    constexpr int SP_CACHE = 2, SP_CLONG = 4, SP_STREAM = 4;
    SO_LAUNCH_BY_ROWS(launch, vec4, so_dense_rows(N, E * H), so_pick_lanes(N, E * H, vec4 ? 4 : 1, vec4 ? H / 4 : H));
    return fgnn_launch_status("edge_softmax_kernel");
}

extern "C" int fgnn_edge_softmax_backward(int N, int64_t E, int H, const int32_t *row_ptr, const float *sm, const float *grad_out,
                                          float *grad_in, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1, FGNN_ERR_SHAPE, "fgnn_edge_softmax_backward: bad sizes");
    FGNN_REQUIRE(row_ptr && (E == 0 || (sm && grad_out && grad_in)), FGNN_ERR_NULL, "fgnn_edge_softmax_backward: NULL argument");
    if (N == 0 || E == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    const unsigned waves = (unsigned)((N + FGNN_WPB - 1) / FGNN_WPB);
    if (H > 64) {
        hipLaunchKernelGGL(edge_softmax_bwd_wide_kernel, dim3(waves), dim3(FGNN_TPB), 0, st, N, H, row_ptr, sm, grad_out, grad_in);
        return fgnn_launch_status("edge_softmax_bwd_wide_kernel");
    }
    constexpr int TPB = 512;
    const bool vec4 = H % 4 == 0 && fgnn_aligned16(sm) && fgnn_aligned16(grad_out) && fgnn_aligned16(grad_in);
    auto launch = [&]<int VEC, class CFG>() {
        unsigned n_long;
        const unsigned grid = so_grid(N, E * H, TPB, &n_long, CFG::L);
        hipLaunchKernelGGL((edge_softmax_bwd_kernel<VEC, TPB, CFG>), dim3(grid), dim3(TPB), 0, st, N, H / VEC, n_long, row_ptr, sm, grad_out, grad_in);
    };
    using dense = so_cfg<8, 8, 4>;           // the backward keeps two arrays: CACHE groups of each, STREAM loads of each in flight
    constexpr int SP_CACHE = 2, SP_CLONG = 2, SP_STREAM = 2;
    SO_LAUNCH_BY_ROWS(launch, vec4, so_dense_rows(N, E * H), so_pick_lanes(N, E * H, vec4 ? 4 : 1, vec4 ? H / 4 : H));
    return fgnn_launch_status("edge_softmax_bwd_kernel");
}

// Forward half of the reference's fuse-scatter GAT (fused_gat.gat_forward minus its SpMM, src/fused_gat/fused_gat.cu:235-300,
// 365-386): e_softmax[p,h] = softmax over row(p) of lrelu(attn_row[row(p),h] + attn_col[col_ind[p],h]); e_lrelu (optional)
// gets the LeakyReLU values.  H <= 64.
extern "C" int fgnn_gat_scatter(int N, int64_t E, int H, const int32_t *row_ptr, const int32_t *col_ind, const float *attn_row,
                                const float *attn_col, float negative_slope, float *e_lrelu, float *e_softmax, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1, FGNN_ERR_SHAPE, "fgnn_gat_scatter: bad sizes");
    FGNN_REQUIRE(H <= 64, FGNN_ERR_LIMIT, "fgnn_gat_scatter: H=%d > 64 heads unsupported", H);
    FGNN_REQUIRE(E <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_gat_scatter: E=%lld exceeds int32 positions", (long long)E);
    if (N == 0 || E == 0) return 0;
    FGNN_REQUIRE(row_ptr && col_ind && attn_row && attn_col && e_softmax, FGNN_ERR_NULL, "fgnn_gat_scatter: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    constexpr int TPB = 256;
    const bool vec4 = H % 4 == 0 && fgnn_aligned16(attn_row) && fgnn_aligned16(attn_col) && fgnn_aligned16(e_softmax) && fgnn_aligned16(e_lrelu);
    auto launch = [&]<int VEC, class CFG>() {
        unsigned n_long;
        const unsigned grid = so_grid(N, E * H, TPB, &n_long, CFG::L);
        hipLaunchKernelGGL((gat_scatter_kernel<VEC, TPB, CFG>), dim3(grid), dim3(TPB), 0, st, N, H / VEC, n_long, row_ptr, col_ind, attn_row, attn_col,
                           negative_slope, e_lrelu, e_softmax);
    };
    using dense = so_cfg<4, 8, 4>;           // every load is an index and a gathered row: fewer in flight, more waves resident
    constexpr int SP_CACHE = 2, SP_CLONG = 4, SP_STREAM = 4;
    SO_LAUNCH_BY_ROWS(launch, vec4, so_dense_rows(N, E * H), so_pick_lanes(N, E * H, vec4 ? 4 : 1, vec4 ? H / 4 : H));
    return fgnn_launch_status("gat_scatter_kernel");
}

// fused_gather_row of the same variant's backward (src/fused_gat/fused_gat.cu:502-556): grad_edge_out = lrelu'(e) * e_softmax *
// (grad_edge - sum_row e_softmax * grad_edge), grad_attn_row = its row sums.  The sign of the pre-activation comes from e_lrelu
// when it is given, else from attn_row + attn_col formed again (col_ind, attn_row, attn_col required).  grad_edge_out may be
// grad_edge.
extern "C" int fgnn_gat_gather_row(int N, int64_t E, int H, const int32_t *row_ptr, const int32_t *col_ind, const float *attn_row,
                                   const float *attn_col, const float *e_lrelu, float negative_slope, const float *e_softmax,
                                   const float *grad_edge, float *grad_edge_out, float *grad_attn_row, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1, FGNN_ERR_SHAPE, "fgnn_gat_gather_row: bad sizes");
    FGNN_REQUIRE(H <= 64, FGNN_ERR_LIMIT, "fgnn_gat_gather_row: H=%d > 64 heads unsupported", H);
    FGNN_REQUIRE(E <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_gat_gather_row: E=%lld exceeds int32 positions", (long long)E);
    if (N == 0) return 0;
    FGNN_REQUIRE(row_ptr && grad_attn_row && (E == 0 || (e_softmax && grad_edge && grad_edge_out)), FGNN_ERR_NULL, "fgnn_gat_gather_row: NULL argument");
    FGNN_REQUIRE(E == 0 || e_lrelu || (col_ind && attn_row && attn_col), FGNN_ERR_NULL,
                 "fgnn_gat_gather_row: without e_lrelu the scores are formed again from col_ind, attn_row and attn_col");
    hipStream_t st = (hipStream_t)stream;
    constexpr int TPB = 256;
    const bool vec4 = H % 4 == 0 && fgnn_aligned16(e_softmax) && fgnn_aligned16(grad_edge) && fgnn_aligned16(grad_edge_out) && fgnn_aligned16(grad_attn_row) &&
                      fgnn_aligned16(e_lrelu) && fgnn_aligned16(attn_row) && fgnn_aligned16(attn_col);
    auto launch = [&]<int VEC, class CFG>() {
        unsigned n_long;
        const unsigned grid = so_grid(N, E * H, TPB, &n_long, CFG::L);
        auto go = [&]<bool FROM_ARRAY>() {
            hipLaunchKernelGGL((gat_gather_row_kernel<VEC, FROM_ARRAY, TPB, CFG>), dim3(grid), dim3(TPB), 0, st, N, H / VEC, n_long, row_ptr, col_ind,
                               attn_row, attn_col, e_lrelu, negative_slope, e_softmax, grad_edge, grad_edge_out, grad_attn_row);
        };
        if (e_lrelu) go.template operator()<true>(); else go.template operator()<false>();
    };
    using dense = so_cfg<8, 8, 2>;
    constexpr int SP_CACHE = 4, SP_CLONG = 4, SP_STREAM = 1;
    SO_LAUNCH_BY_ROWS(launch, vec4, so_dense_rows(N, E * H), so_pick_lanes(N, E * H, vec4 ? 4 : 1, vec4 ? H / 4 : H));
    return fgnn_launch_status("gat_gather_row_kernel");
}

// out[p,w] = row_val[row(p),w] + col_val[col_ind[p],w]  (src/u_add_v/u_add_v.cu:4-26).  W <= 64: one thread per
// element of out, a wave takes 2048 consecutive ones; the row of an edge is found by bisection of row_ptr, first
// for the wave's first and last edge (wave-uniform), then per lane inside that usually one- or two-row window.
#define UAV_CHUNKS 32           // 64-element chunks per wave
#define UAV_UJ 8                // chunks in flight; divides UAV_CHUNKS
// VEC = 4: an element is four consecutive columns (W % 4 == 0, 16-byte aligned arrays), W counts such groups.
template <int VEC>
__global__ __launch_bounds__(FGNN_TPB) void u_add_v_kernel(int N, int64_t E, int W, const int *__restrict__ ptr, const int *__restrict__ idx,
                                                           const float *__restrict__ rv, const float *__restrict__ cv, float *__restrict__ out)
{
    const int64_t total = E * W;
    const int64_t k0 = ((int64_t)blockIdx.x * FGNN_WPB + fg_wave()) * (64 * UAV_CHUNKS);
    if (k0 >= total) return;
    const int64_t k1 = min(k0 + 64 * UAV_CHUNKS, total);
    const int lane = fg_lane();
    const unsigned uw = (unsigned)W;
    const unsigned inv_w = (65536u + uw - 1u) / uw;          // ceil(2^16 / W)
    int qbase = fg_uni((int)(k0 / W));                       // edge of the wave's first element
    unsigned rem = (unsigned)fg_uni((int)(k0 - (int64_t)qbase * W));
    const int qlast = fg_uni((int)((k1 - 1) / W));
    int rlo = fg_uni(so_row_of(ptr, 0, N - 1, qbase));
    const int rhi = fg_uni(so_row_of(ptr, rlo, N - 1, qlast));
    constexpr int UJ = UAV_UJ;
    for (int64_t kk = k0; kk < k1; kk += 64 * UJ) {
        int q[UJ], w[UJ], lo[UJ], hi[UJ];
#pragma unroll
        for (int j = 0; j < UJ; ++j) {
            const unsigned x = rem + (unsigned)(64 * j + lane);           // < W + 64 * UJ <= 320
            const unsigned dq = (x * inv_w) >> 16;                          // = x / W for x < 1024 (W <= 64)
            w[j] = (int)(x - dq * uw);
            q[j] = min(qbase + (int)dq, qlast);
            lo[j] = rlo; hi[j] = rhi;
        }
        for (int span = rhi - rlo; span > 0; span >>= 1) {   // wave-uniform trip count: ceil(log2(window))
#pragma unroll
            for (int j = 0; j < UJ; ++j) {
                const int mid = (lo[j] + hi[j] + 1) >> 1;    // lo == hi: mid == lo, nothing changes
                if (lo[j] < hi[j]) { if (ptr[mid] <= q[j]) lo[j] = mid; else hi[j] = mid - 1; }
            }
        }
        int src[UJ];
#pragma unroll
        for (int j = 0; j < UJ; ++j) src[j] = idx[q[j]];
#pragma unroll
        for (int j = 0; j < UJ; ++j) {
            const int64_t k = kk + 64 * j + lane;
            if (k < k1) {
                fg_vec<VEC> a, b;
                a.load(rv + ((size_t)lo[j] * W + w[j]) * VEC);
                b.load(cv + ((size_t)src[j] * W + w[j]) * VEC);
                a.add(b);
                a.store_nt(out + (size_t)k * VEC);
            }
        }
        rem += 64u * UJ;
        const unsigned adv = rem / uw;
        qbase += (int)adv;
        rem -= adv * uw;
        rlo = __builtin_amdgcn_readlane(lo[UJ - 1], 63);     // rows only grow along the chunks
    }
}

// More than 64 columns: one wave per row.
__global__ __launch_bounds__(FGNN_TPB) void u_add_v_wide_kernel(int N, int W, const int *ptr, const int *idx, const float *rv, const float *cv, float *out)
{
    int row = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (row >= N) return;
    const int lane = fg_lane();
    const int64_t lo = (int64_t)fg_uni(ptr[row]) * W, hi = (int64_t)fg_uni(ptr[row + 1]) * W;
    for (int64_t k = lo + lane; k < hi; k += 64) {
        int64_t p = k / W;
        int w = (int)(k - p * W);
        out[k] = rv[(size_t)row * W + w] + cv[(size_t)idx[p] * W + w];
    }
}

// grad_row[i,w] = sum over the row's edges (fixed order) and, with COLS, grad_col[j,w] += g[p,w] with float atomics
// into a zero-filled buffer as the reference does it (src/u_add_v/u_add_v.cu:43-90, which adds into uninitialised
// memory); without COLS the column sums are left to the tile-ordered pass of fgnn_edge_colsum.  One pass over grad_out,
// rows shared out as in the softmax kernels.
template <int NW, int VEC, bool COLS, int L = 64>        // L < 64 (NW == 1): row, pb, pe per group of L lanes; row < 0: a group without a row
__device__ __forceinline__ void so_rowsum_row(int W, int row, int pb, int pe, const int *__restrict__ idx, const float *__restrict__ g,
                                              float *__restrict__ grow, float *__restrict__ gcol, float (*sh)[64])
{
    static_assert(L == 64 || NW == 1, "lane groups only where one wave has the row");
    const int lane = fg_lane(), sl = lane & (L - 1), S0 = (L / W) * W, w = sl % W;
    const int per = S0 / W;                                        // entries per trip of the wave (of the lane group)
    constexpr int nw = NW;
    const bool act = sl < S0;
    so_grp<VEC> acc = so_fill<VEC>(0.f);
    if (act) {
#pragma unroll 8
        for (int q = pb + (NW > 1 ? fg_wave() * per : 0) + sl / W; q < pe; q += per * nw) {
            const so_grp<VEC> v = so_load<VEC>(g + ((size_t)q * W + w) * VEC);
#pragma unroll
            for (int c = 0; c < VEC; ++c) acc.c[c] += v.c[c];
            if constexpr (COLS) {
                float *dst = gcol + ((size_t)idx[q] * W + w) * VEC;
#pragma unroll
                for (int c = 0; c < VEC; ++c) unsafeAtomicAdd(dst + c, v.c[c]);
            }
        }
    }
    if constexpr (L < 64) acc = so_group_reduce<VEC, L>(acc, lane, W, S0, so_add());
    else acc = so_column_reduce<NW, VEC>(acc, lane, W, S0, sh, so_add());
    if (sl < W && row >= 0 && (NW == 1 || fg_wave() == 0)) so_store<VEC>(grow + ((size_t)row * W + sl) * VEC, acc);
}

template <int VEC, bool COLS, int TPB, int L = 64>
__global__ __launch_bounds__(TPB) void edge_rowsum_kernel(int N, int W, unsigned n_long_blocks, const int *__restrict__ ptr,
                                                                  const int *__restrict__ idx, const float *__restrict__ g, float *__restrict__ grow,
                                                                  float *__restrict__ gcol)
{
    __shared__ float sh[TPB / 64][64];
    __shared__ unsigned long long sh_mask;
    if (blockIdx.x < n_long_blocks) {
        for (unsigned long long m = so_long_candidates<VEC>(N, W, ptr, &sh_mask); m; m &= m - 1) {
            const int row = so_scattered_row(blockIdx.x * SO_CAND + (unsigned)__builtin_ctzll(m), N);
            so_rowsum_row<TPB / 64, VEC, COLS>(W, row, fg_uni(ptr[row]), fg_uni(ptr[row + 1]), idx, g, grow, gcol, sh);
        }
        return;
    }
    int row, pb;
    int64_t n;
    const unsigned u = (unsigned)fg_uni((int)((blockIdx.x - n_long_blocks) * (TPB / 64)) + fg_wave());
    if constexpr (L < 64) {
        bool mine;
        if (!so_take_short_rows<VEC, L>(u, N, W, ptr, row, pb, n, mine)) return;
        so_rowsum_row<1, VEC, COLS, L>(W, mine ? row : -1, pb, pb + (int)(n / W), idx, g, grow, gcol, nullptr);
        return;
    }
    if (!so_take_short_row<VEC>(u, N, W, ptr, row, pb, n)) return;      // empty rows stay here: they store zeros
    so_rowsum_row<1, VEC, COLS>(W, row, pb, fg_uni(ptr[row + 1]), idx, g, grow, gcol, nullptr);
}

__global__ __launch_bounds__(FGNN_TPB) void u_add_v_bwd_wide_kernel(int N, int W, const int *ptr, const int *idx, const float *g, float *grow, float *gcol)
{
    int row = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (row >= N) return;
    const int lane = fg_lane();
    const int pb = fg_uni(ptr[row]), pe = fg_uni(ptr[row + 1]);
    for (int w = 0; w < W; ++w) {
        float acc = 0.f;
        for (int q = pb + lane; q < pe; q += 64) {
            float v = g[(size_t)q * W + w];
            acc += v;
            unsafeAtomicAdd(gcol + (size_t)idx[q] * W + w, v);
        }
        acc = fg_wave_sum(acc);
        if (lane == 0) grow[(size_t)row * W + w] = acc;
    }
}

extern "C" int fgnn_u_add_v(int N, int64_t E, int W, const int32_t *row_ptr, const int32_t *col_ind, const float *row_val,
                            const float *col_val, float *out, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && W >= 1, FGNN_ERR_SHAPE, "fgnn_u_add_v: bad sizes");
    FGNN_REQUIRE(row_ptr && row_val && col_val && (E == 0 || (col_ind && out)), FGNN_ERR_NULL, "fgnn_u_add_v: NULL argument");
    if (N == 0 || E == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    if (W > 64) {
        hipLaunchKernelGGL(u_add_v_wide_kernel, dim3((unsigned)((N + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, st, N, W, row_ptr, col_ind,
                           row_val, col_val, out);
        return fgnn_launch_status("u_add_v_wide_kernel");
    }
    FGNN_REQUIRE(E <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_u_add_v: E=%lld exceeds the 32-bit row_ptr", (long long)E);
    const int64_t per_block = (int64_t)FGNN_WPB * 64 * UAV_CHUNKS;
    if (W % 4 == 0 && fgnn_aligned16(row_val) && fgnn_aligned16(col_val) && fgnn_aligned16(out)) {
        const int64_t blocks = (E * (W / 4) + per_block - 1) / per_block;
        hipLaunchKernelGGL(u_add_v_kernel<4>, dim3((unsigned)blocks), dim3(FGNN_TPB), 0, st, N, E, W / 4, row_ptr, col_ind, row_val, col_val, out);
    } else {
        const int64_t blocks = (E * W + per_block - 1) / per_block;
        hipLaunchKernelGGL(u_add_v_kernel<1>, dim3((unsigned)blocks), dim3(FGNN_TPB), 0, st, N, E, W, row_ptr, col_ind, row_val, col_val, out);
    }
    return fgnn_launch_status("u_add_v_kernel");
}

extern "C" int fgnn_u_add_v_backward(int N, int64_t E, int W, const int32_t *row_ptr, const int32_t *col_ind, const float *grad_out,
                                     float *grad_row, float *grad_col, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && W >= 1, FGNN_ERR_SHAPE, "fgnn_u_add_v_backward: bad sizes");
    FGNN_REQUIRE(row_ptr && grad_row && grad_col && (E == 0 || (col_ind && grad_out)), FGNN_ERR_NULL, "fgnn_u_add_v_backward: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    int rc = fgnn_fill_f32(grad_col, (size_t)N * W, 0.f, st);
    if (rc || N == 0) return rc;
    const unsigned waves = (unsigned)((N + FGNN_WPB - 1) / FGNN_WPB);
    if (W > 64) {
        hipLaunchKernelGGL(u_add_v_bwd_wide_kernel, dim3(waves), dim3(FGNN_TPB), 0, st, N, W, row_ptr, col_ind, grad_out, grad_row, grad_col);
        return fgnn_launch_status("u_add_v_bwd_wide_kernel");
    }
    // one float per lane: the atomics of a wave instruction then fall into the fewest cache lines (with four per lane
    // the pass took three times as long on a 115 M-entry graph)
    unsigned n_long;
    const unsigned grid = so_grid(N, E * W, 512, &n_long);
    hipLaunchKernelGGL((edge_rowsum_kernel<1, true, 512>), dim3(grid), dim3(512), 0, st, N, W, n_long, row_ptr, col_ind, grad_out, grad_row, grad_col);
    return fgnn_launch_status("edge_rowsum_kernel");
}

// More than 64 columns: one wave per row, lanes over the columns.
__global__ __launch_bounds__(FGNN_TPB) void edge_rowsum_wide_kernel(int N, int W, const int *__restrict__ ptr, const float *__restrict__ g,
                                                                    float *__restrict__ out)
{
    const int row = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (row >= N) return;
    const int pb = fg_uni(ptr[row]), pe = fg_uni(ptr[row + 1]);
    for (int w = fg_lane(); w < W; w += 64) {
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;       // four interleaved partial sums: four loads in flight, a quarter of the rounding growth
        int q = pb;
        for (; q + 4 <= pe; q += 4) {
            a0 += g[(size_t)q * W + w]; a1 += g[(size_t)(q + 1) * W + w]; a2 += g[(size_t)(q + 2) * W + w]; a3 += g[(size_t)(q + 3) * W + w];
        }
        for (; q < pe; ++q) a0 += g[(size_t)q * W + w];
        out[(size_t)row * W + w] = (a0 + a1) + (a2 + a3);
    }
}

// out[i,:] = sum of g[p,:] over the CSR positions p of row i, in a fixed order.
extern "C" int fgnn_edge_rowsum(int N, int64_t E, int W, const int32_t *row_ptr, const float *g, float *out, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && W >= 1, FGNN_ERR_SHAPE, "fgnn_edge_rowsum: bad sizes");
    FGNN_REQUIRE((row_ptr && out) || N == 0, FGNN_ERR_NULL, "fgnn_edge_rowsum: NULL argument");
    FGNN_REQUIRE(g || E == 0, FGNN_ERR_NULL, "fgnn_edge_rowsum: NULL argument");
    if (N == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    const unsigned waves = (unsigned)((N + FGNN_WPB - 1) / FGNN_WPB);
    if (W > 64) {
        hipLaunchKernelGGL(edge_rowsum_wide_kernel, dim3(waves), dim3(FGNN_TPB), 0, st, N, W, row_ptr, g, out);
        return fgnn_launch_status("edge_rowsum_wide_kernel");
    }
    const bool vec4 = W % 4 == 0 && fgnn_aligned16(g) && fgnn_aligned16(out);
    unsigned n_long;
    constexpr int TPB = 512;
    // sparse rows share waves, as in the softmax kernels
    const int lanes = so_dense_rows(N, E * W) ? 64 : so_pick_lanes(N, E * W, vec4 ? 4 : 1, vec4 ? W / 4 : W);
    auto launch = [&]<int VEC, int L>() {
        const unsigned grid = so_grid(N, E * W, TPB, &n_long, L);
        hipLaunchKernelGGL((edge_rowsum_kernel<VEC, false, TPB, L>), dim3(grid), dim3(TPB), 0, st, N, W / VEC, n_long, row_ptr, nullptr, g, out, nullptr);
    };
#define RS_L(LL) do { if (vec4) launch.template operator()<4, LL>(); else launch.template operator()<1, LL>(); } while (0)
    if (lanes == 32) RS_L(32); else if (lanes == 16) RS_L(16); else if (lanes == 8) RS_L(8); else RS_L(64);
#undef RS_L
    return fgnn_launch_status("edge_rowsum_kernel");
}

// u_add_v's backward without atomics: the row sums by the pass above, the column sums by the tile-ordered pass of
// fgnn_edge_colsum under a plan of (row_ptr, col_ind).  Both are summed in a fixed order.
extern "C" int fgnn_u_add_v_backward_planned(int N, int64_t E, int W, const int32_t *row_ptr, const int32_t *col_ind, const float *grad_out,
                                             float *grad_row, float *grad_col, const fgnn_colsum_plan_t *plan, void *workspace,
                                             size_t workspace_bytes, void *stream)
{
    FGNN_REQUIRE(plan, FGNN_ERR_NULL, "fgnn_u_add_v_backward_planned: NULL plan");
    FGNN_REQUIRE(fgnn_colsum_plan_matches(plan, row_ptr, col_ind, N, N, E), FGNN_ERR_SCHEDULE,
                 "fgnn_u_add_v_backward_planned: the plan was built for other arrays");
    int rc = fgnn_edge_rowsum(N, E, W, row_ptr, grad_out, grad_row, stream);
    if (rc) return rc;
    return fgnn_edge_colsum(plan, W, grad_out, grad_col, workspace, workspace_bytes, stream);
}

// ------------------------------------------------------------------------------- per-edge Linear(2, D) + tanh
// The pseudo-coordinate projection of the MoNet drivers (script/train/train_gmmconv_our.py:46-57:
// nn.Sequential(nn.Linear(2, dim), nn.Tanh()) applied to the [E, 2] edge coordinates), as one pass
// over the edges each way instead of a chain of elementwise kernels; its weight gradient is a
// reduction over all E edges, done here with per-thread partial sums, a fixed-order workgroup
// reduction and a fixed-order sum over the workgroups (deterministic).
#define ELT_BLOCKS 1024
template <int D>
__global__ __launch_bounds__(256) void edge_linear_tanh_kernel(int64_t E, const float2 *__restrict__ x, const float *__restrict__ W,
                                                               const float *__restrict__ b, float *__restrict__ y)
{
    float w0[D], w1[D], bb[D];
#pragma unroll
    for (int o = 0; o < D; ++o) { w0[o] = W[2 * o]; w1[o] = W[2 * o + 1]; bb[o] = b[o]; }
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < E; e += (int64_t)gridDim.x * 256) {
        const float2 v = x[e];
#pragma unroll
        for (int o = 0; o < D; ++o) y[e * D + o] = tanhf(fmaf(v.y, w1[o], fmaf(v.x, w0[o], bb[o])));
    }
}

// part[block][3*D]: per output o the partial sums of gt*x0, gt*x1, gt with gt = g * (1 - y^2).
template <int D>
__global__ __launch_bounds__(256) void edge_linear_tanh_bwd_kernel(int64_t E, const float2 *__restrict__ x, const float *__restrict__ y,
                                                                   const float *__restrict__ g, float *__restrict__ part)
{
    __shared__ float sh[4][3 * D];
    float acc[3 * D];
#pragma unroll
    for (int i = 0; i < 3 * D; ++i) acc[i] = 0.f;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < E; e += (int64_t)gridDim.x * 256) {
        const float2 v = x[e];
#pragma unroll
        for (int o = 0; o < D; ++o) {
            const float yy = y[e * D + o];
            const float gt = g[e * D + o] * (1.f - yy * yy);
            acc[3 * o] = fmaf(gt, v.x, acc[3 * o]);
            acc[3 * o + 1] = fmaf(gt, v.y, acc[3 * o + 1]);
            acc[3 * o + 2] += gt;
        }
    }
    const int lane = fg_lane(), wave = fg_wave();
#pragma unroll
    for (int i = 0; i < 3 * D; ++i) {
        float s = fg_wave_sum(acc[i]);
        if (lane == 0) sh[wave][i] = s;
    }
    __syncthreads();
    if ((int)threadIdx.x < 3 * D)
        part[(size_t)blockIdx.x * 3 * D + threadIdx.x] = (sh[0][threadIdx.x] + sh[1][threadIdx.x]) + (sh[2][threadIdx.x] + sh[3][threadIdx.x]);
}

__global__ __launch_bounds__(64) void edge_linear_tanh_finish_kernel(int nblk, int D, const float *__restrict__ part, float *__restrict__ gW,
                                                                     float *__restrict__ gb)
{
    const int i = (int)threadIdx.x;
    if (i >= 3 * D) return;
    float s = 0.f;
    for (int k = 0; k < nblk; ++k) s += part[(size_t)k * 3 * D + i];
    const int o = i / 3, c = i - 3 * o;
    if (c < 2) gW[2 * o + c] = s; else gb[o] = s;
}

static int elt_blocks(int64_t E) { return (int)std::min<int64_t>(ELT_BLOCKS, (E + 255) / 256); }

extern "C" int fgnn_edge_linear_tanh(int64_t E, int D, const float *x, const float *W, const float *b, float *y, void *stream)
{
    FGNN_REQUIRE(E >= 0, FGNN_ERR_SHAPE, "fgnn_edge_linear_tanh: E=%lld", (long long)E);
    FGNN_REQUIRE(D >= 1 && D <= 4, FGNN_ERR_LIMIT, "fgnn_edge_linear_tanh: %d output columns unsupported (1..4)", D);
    if (E == 0) return 0;
    FGNN_REQUIRE(x && W && b && y, FGNN_ERR_NULL, "fgnn_edge_linear_tanh: NULL argument");
    FGNN_REQUIRE((((uintptr_t)x) & 7u) == 0, FGNN_ERR_ALIGN, "fgnn_edge_linear_tanh: x not 8-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)std::min<int64_t>(8192, (E + 255) / 256));
    switch (D) {
    case 1: hipLaunchKernelGGL(edge_linear_tanh_kernel<1>, grid, dim3(256), 0, st, E, (const float2 *)x, W, b, y); break;
    case 2: hipLaunchKernelGGL(edge_linear_tanh_kernel<2>, grid, dim3(256), 0, st, E, (const float2 *)x, W, b, y); break;
    case 3: hipLaunchKernelGGL(edge_linear_tanh_kernel<3>, grid, dim3(256), 0, st, E, (const float2 *)x, W, b, y); break;
    default: hipLaunchKernelGGL(edge_linear_tanh_kernel<4>, grid, dim3(256), 0, st, E, (const float2 *)x, W, b, y); break;
    }
    return fgnn_launch_status("edge_linear_tanh_kernel");
}

extern "C" size_t fgnn_edge_linear_tanh_backward_workspace_bytes(int64_t E, int D)
{
    return (size_t)elt_blocks(E) * 3 * (size_t)(D > 0 ? D : 1) * sizeof(float);
}

extern "C" int fgnn_edge_linear_tanh_backward(int64_t E, int D, const float *x, const float *y, const float *grad_y, float *grad_W,
                                              float *grad_b, void *workspace, size_t workspace_bytes, void *stream)
{
    FGNN_REQUIRE(E >= 0, FGNN_ERR_SHAPE, "fgnn_edge_linear_tanh_backward: E=%lld", (long long)E);
    FGNN_REQUIRE(D >= 1 && D <= 4, FGNN_ERR_LIMIT, "fgnn_edge_linear_tanh_backward: %d output columns unsupported (1..4)", D);
    FGNN_REQUIRE(grad_W && grad_b, FGNN_ERR_NULL, "fgnn_edge_linear_tanh_backward: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    if (E == 0) {
        int rc = fgnn_fill_f32(grad_W, 2 * (size_t)D, 0.f, st);
        return rc ? rc : fgnn_fill_f32(grad_b, (size_t)D, 0.f, st);
    }
    FGNN_REQUIRE(x && y && grad_y, FGNN_ERR_NULL, "fgnn_edge_linear_tanh_backward: NULL argument");
    FGNN_REQUIRE((((uintptr_t)x) & 7u) == 0, FGNN_ERR_ALIGN, "fgnn_edge_linear_tanh_backward: x not 8-byte aligned");
    const size_t need = fgnn_edge_linear_tanh_backward_workspace_bytes(E, D);
    FGNN_REQUIRE(workspace && workspace_bytes >= need, FGNN_ERR_WORKSPACE, "fgnn_edge_linear_tanh_backward: workspace %zu < %zu bytes", workspace_bytes, need);
    const int nblk = elt_blocks(E);
    float *part = (float *)workspace;
    switch (D) {
    case 1: hipLaunchKernelGGL(edge_linear_tanh_bwd_kernel<1>, dim3(nblk), dim3(256), 0, st, E, (const float2 *)x, y, grad_y, part); break;
    case 2: hipLaunchKernelGGL(edge_linear_tanh_bwd_kernel<2>, dim3(nblk), dim3(256), 0, st, E, (const float2 *)x, y, grad_y, part); break;
    case 3: hipLaunchKernelGGL(edge_linear_tanh_bwd_kernel<3>, dim3(nblk), dim3(256), 0, st, E, (const float2 *)x, y, grad_y, part); break;
    default: hipLaunchKernelGGL(edge_linear_tanh_bwd_kernel<4>, dim3(nblk), dim3(256), 0, st, E, (const float2 *)x, y, grad_y, part); break;
    }
    int rc = fgnn_launch_status("edge_linear_tanh_bwd_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(edge_linear_tanh_finish_kernel, dim3(1), dim3(64), 0, st, nblk, D, part, grad_W, grad_b);
    return fgnn_launch_status("edge_linear_tanh_finish_kernel");
}
