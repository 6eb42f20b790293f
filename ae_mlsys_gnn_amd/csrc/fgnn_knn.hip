// Brute-force k-nearest-neighbour graph builder for batched point clouds (the graph the fused
// EdgeConv consumes).  The reference builds it with DGL's KNNGraph on every layer of its DGCNN
// loop (script/train/train_edgeconv_our.py:51-55): per cloud, for every point the k nearest points
// of the same cloud, the point itself included, grouped by destination.
//
//
// A wave owns KNN_QW query points at a time and all 64 lanes share them: lane l holds the running
// squared distances from each of the queries to 4*RG candidate points in registers (candidates
// 4l..4l+3 of every 256-point group of the tile).  The candidate coordinates of a tile stream
// through LDS in slices of KNN_DC dimensions, transposed ([dimension][point]) so that a lane
// fetches its 4 candidates with one 128-bit LDS read and uses them for all KNN_QW queries; the
// query coordinates are wave-uniform and come through scalar registers.  Distances accumulate
// dimension by dimension in ascending order with one subtract and one fma each, so a point is at
// distance exactly 0 from itself.
//
// Selection (k <= 64): the k-th smallest of the 64 lane minima is a threshold that at least k
// candidates pass; the candidates under it (usually k to 2k of the 1024) are compacted into LDS with
// ballots and ordered by one bitonic sort over the wave.  When more than 64 pass (many equal distances)
// and for 64 < k <= 128 the selection runs k extraction rounds instead: wave-wide minimum (DPP
// butterfly), holder with the smallest node id by ballots, retire it.  Either way the order is total
// (smaller distance first, smaller node id on equal distance), so the result is deterministic.  Clouds
// with more points than one tile keep the best k of the tiles seen so far in registers and run them
// through the next tile's selection, where they win ties because their ids are smaller.
#include "fgnn_common.h"
#include <float.h>

#define KNN_QW 4         // queries a wave processes together
#define KNN_WAVES 4      // waves per workgroup
#define KNN_DC 8         // dimensions per LDS slice
#define KNN_MAX_K 128    // KR = 2 result registers per lane

// Takes the k best of {prior list (pd, pi), the tile's distances} in order; the new list replaces
// the prior one.  List position p lives in lane p % 64 of register p / 64.
template <int NR, int KR>
__device__ __forceinline__ void knn_select_rounds(float (&dist)[NR], int tile0, float (&pd)[KR], int (&pi)[KR], int k, int lane, int fallback_id)
{
    float nd[KR];
    int ni[KR];
#pragma unroll
    for (int t = 0; t < KR; ++t) { nd[t] = INFINITY; ni[t] = fallback_id; }
    for (int j = 0; j < k; ++j) {
        float lm = dist[0];
#pragma unroll
        for (int r = 1; r < NR; ++r) lm = fminf(lm, dist[r]);
#pragma unroll
        for (int t = 0; t < KR; ++t) lm = fminf(lm, pd[t]);
        const float m = -fg_wave_max(-lm);
        int id = fallback_id;
        bool found = false;
#pragma unroll
        for (int t = 0; t < KR; ++t) {
            if (!found) {
                unsigned long long b = __ballot(pd[t] == m);
                if (b) {
                    int L = __builtin_ctzll(b);
                    id = __builtin_amdgcn_readlane(pi[t], L);
                    if (lane == L) pd[t] = INFINITY;
                    found = true;
                }
            }
        }
#pragma unroll
        for (int g = 0; g < NR / 4; ++g) {
            if (!found) {
                unsigned long long b0 = __ballot(dist[4 * g] == m), b1 = __ballot(dist[4 * g + 1] == m);
                unsigned long long b2 = __ballot(dist[4 * g + 2] == m), b3 = __ballot(dist[4 * g + 3] == m);
                unsigned long long any = b0 | b1 | b2 | b3;
                if (any) {
                    int L = __builtin_ctzll(any);
                    int i = ((b0 >> L) & 1) ? 0 : ((b1 >> L) & 1) ? 1 : ((b2 >> L) & 1) ? 2 : 3;
                    id = tile0 + g * 256 + L * 4 + i;
                    if (lane == L) {
#pragma unroll
                        for (int u = 0; u < 4; ++u) if (i == u) dist[4 * g + u] = INFINITY;
                    }
                    found = true;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < KR; ++t)
            if ((j >> 6) == t && lane == (j & 63)) { nd[t] = m; ni[t] = id; }
    }
#pragma unroll
    for (int t = 0; t < KR; ++t) { pd[t] = nd[t]; pi[t] = ni[t]; }
}

// Bitonic sort of one value per lane over the wave, ascending by (d, i).
__device__ __forceinline__ void knn_sort_wave(float &d, int &i, int lane)
{
#pragma unroll
    for (int size = 2; size <= 64; size <<= 1) {
#pragma unroll
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const float od = fg_bperm(d, lane ^ stride);
            const int oi = __builtin_amdgcn_ds_bpermute((lane ^ stride) << 2, i);
            const bool keep_small = (((lane & size) == 0) || size == 64) == ((lane & stride) == 0);
            const bool other_smaller = od < d || (od == d && oi < i);
            if (keep_small == other_smaller) { d = od; i = oi; }
        }
    }
}

// The k best of {prior list, tile} for k <= 64: (1) a threshold that at least k candidates pass, the
// k-th smallest of the 64 lane minima; (2) the candidates under it (usually k to 2k) are compacted
// into wave-private LDS with ballots; (3) one bitonic sort over the wave orders them.  More than 64
// candidates under the threshold (many equal distances, or fewer than k lanes with a candidate) fall
// back to the extraction rounds.  sd/si: 64 floats / ints of LDS owned by this wave.
template <int NR>
__device__ __forceinline__ void knn_select(float (&dist)[NR], int tile0, float (&pd)[1], int (&pi)[1], int k, int lane, int fallback_id,
                                           float *sd, int *si)
{
    float lm = pd[0];
#pragma unroll
    for (int r = 0; r < NR; ++r) lm = fminf(lm, dist[r]);
    int dummy = lane;
    knn_sort_wave(lm, dummy, lane);
    const float tau = fg_readlane(lm, k - 1);
    int cnt = __popcll(__ballot(pd[0] <= tau));
#pragma unroll
    for (int r = 0; r < NR; ++r) cnt += __popcll(__ballot(dist[r] <= tau));
    if (cnt > 64 || !(tau < INFINITY)) {
        knn_select_rounds<NR, 1>(dist, tile0, pd, pi, k, lane, fallback_id);
        return;
    }
    const unsigned long long lt = (1ull << lane) - 1ull;
    int base = 0;
    {
        const bool in = pd[0] <= tau;
        const unsigned long long m = __ballot(in);
        if (in) { int pos = base + __popcll(m & lt); sd[pos] = pd[0]; si[pos] = pi[0]; }
        base += __popcll(m);
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const bool in = dist[r] <= tau;
        const unsigned long long m = __ballot(in);
        if (in) { int pos = base + __popcll(m & lt); sd[pos] = dist[r]; si[pos] = tile0 + (r / 4) * 256 + lane * 4 + (r % 4); }
        base += __popcll(m);
    }
    fg_wave_lds_sync();
    float cd = lane < cnt ? sd[lane] : INFINITY;
    int ci = lane < cnt ? si[lane] : 0x7fffffff;
    fg_wave_lds_sync();
    knn_sort_wave(cd, ci, lane);
    pd[0] = lane < k ? cd : INFINITY;
    pi[0] = lane < k ? ci : fallback_id;
}
template <int NR>
__device__ __forceinline__ void knn_select(float (&dist)[NR], int tile0, float (&pd)[2], int (&pi)[2], int k, int lane, int fallback_id,
                                           float *, int *)
{
    knn_select_rounds<NR, 2>(dist, tile0, pd, pi, k, lane, fallback_id);       // 64 < k <= 128
}

template <int RG, int KR>
__global__ __launch_bounds__(KNN_WAVES * 64) void knn_kernel(int P, int D, int k, int rows_aligned, const float *__restrict__ pts, int *__restrict__ out)
{
    constexpr int NR = 4 * RG;                  // distances per lane and query
    constexpr int TILE = 256 * RG;              // candidate points per tile
    __shared__ __attribute__((aligned(16))) float cs[KNN_DC * TILE];        // [dimension of the slice][point of the tile]
    __shared__ float sel_d[KNN_WAVES * 64];                                 // selection scratch, 64 entries per wave
    __shared__ int sel_i[KNN_WAVES * 64];
    const int tid = (int)threadIdx.x;
    const int lane = fg_lane();
    const int cloud = (int)blockIdx.y;
    const float *cp = pts + (size_t)cloud * P * D;
    const int qbase = fg_uni(((int)blockIdx.x * KNN_WAVES + fg_wave()) * KNN_QW);
    int qrow[KNN_QW];                           // clamped query rows (wave-uniform)
#pragma unroll
    for (int a = 0; a < KNN_QW; ++a) qrow[a] = min(qbase + a, P - 1);
    float pd[KNN_QW][KR];
    int pi[KNN_QW][KR];
#pragma unroll
    for (int a = 0; a < KNN_QW; ++a)
#pragma unroll
        for (int t = 0; t < KR; ++t) { pd[a][t] = INFINITY; pi[a][t] = qrow[a]; }

    for (int tile0 = 0; tile0 < P; tile0 += TILE) {
        float acc[KNN_QW][NR];
#pragma unroll
        for (int a = 0; a < KNN_QW; ++a)
#pragma unroll
            for (int r = 0; r < NR; ++r) acc[a][r] = 0.f;
        for (int d0 = 0; d0 < D; d0 += KNN_DC) {
            const int dn = min(KNN_DC, D - d0);
            __syncthreads();                    // the previous slice has been consumed
#pragma unroll
            for (int i = 0; i < RG; ++i) {
                const int c = tid + 256 * i;
                const bool ok = tile0 + c < P;
                const float *src = cp + (size_t)(ok ? tile0 + c : 0) * D + d0;
                if (dn == KNN_DC && rows_aligned) {              // every row starts on 16 bytes: two 128-bit loads
                    const float4 lo = *reinterpret_cast<const float4 *>(src), hi = *reinterpret_cast<const float4 *>(src + 4);
                    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                    for (int dd = 0; dd < KNN_DC; ++dd) cs[dd * TILE + c] = ok ? v[dd] : 0.f;
                } else {
                    for (int dd = 0; dd < dn; ++dd) cs[dd * TILE + c] = ok ? src[dd] : 0.f;
                }
            }
            __syncthreads();
            auto step = [&](int dd) {
                float qv[KNN_QW];
#pragma unroll
                for (int a = 0; a < KNN_QW; ++a) qv[a] = cp[(size_t)qrow[a] * D + d0 + dd];
#pragma unroll
                for (int g = 0; g < RG; ++g) {
                    const float4 c4 = *reinterpret_cast<const float4 *>(&cs[dd * TILE + g * 256 + lane * 4]);
                    const float cv[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
                    for (int a = 0; a < KNN_QW; ++a)
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            float df = qv[a] - cv[u];
                            acc[a][4 * g + u] = fmaf(df, df, acc[a][4 * g + u]);
                        }
                }
            };
            if (dn == KNN_DC) {
#pragma unroll
                for (int dd = 0; dd < KNN_DC; ++dd) step(dd);
            } else {
                for (int dd = 0; dd < dn; ++dd) step(dd);
            }
        }
        // points past the end of the cloud never win; NaN distances sort last among the real ones
#pragma unroll
        for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const bool ok = tile0 + g * 256 + lane * 4 + u < P;
#pragma unroll
                for (int a = 0; a < KNN_QW; ++a) acc[a][4 * g + u] = ok ? fminf(acc[a][4 * g + u], FLT_MAX) : INFINITY;
            }
#pragma unroll
        for (int a = 0; a < KNN_QW; ++a) knn_select<NR>(acc[a], tile0, pd[a], pi[a], k, lane, qrow[a], sel_d + fg_wave() * 64, sel_i + fg_wave() * 64);
    }
#pragma unroll
    for (int a = 0; a < KNN_QW; ++a) {
        const int q = qbase + a;
        if (q < P) {
            int *o = out + ((size_t)cloud * P + q) * k;
#pragma unroll
            for (int t = 0; t < KR; ++t) {
                const int j = t * 64 + lane;
                if (j < k) o[j] = cloud * P + pi[a][t];
            }
        }
    }
}

template <int RG, int KR>
static void knn_launch(int n_clouds, int P, int D, int k, const float *points, int32_t *src_ind, hipStream_t st)
{
    const int qwg = KNN_WAVES * KNN_QW;
    dim3 grid((unsigned)((P + qwg - 1) / qwg), (unsigned)n_clouds);
    hipLaunchKernelGGL((knn_kernel<RG, KR>), grid, dim3(KNN_WAVES * 64), 0, st, P, D, k,
                       (D % 4 == 0 && fgnn_aligned16(points)) ? 1 : 0, points, src_ind);
}

extern "C" int fgnn_knn_graph(int n_clouds, int P, int D, int k, const float *points, int32_t *src_ind, void *stream)
{
    FGNN_REQUIRE(n_clouds >= 0 && P >= 1 && D >= 1 && k >= 1, FGNN_ERR_SHAPE, "fgnn_knn_graph: bad sizes clouds=%d P=%d D=%d k=%d", n_clouds, P, D, k);
    FGNN_REQUIRE(k <= P, FGNN_ERR_SHAPE, "fgnn_knn_graph: k=%d exceeds the %d points of a cloud", k, P);
    FGNN_REQUIRE(k <= KNN_MAX_K, FGNN_ERR_LIMIT, "fgnn_knn_graph: k=%d exceeds the limit of %d neighbours", k, KNN_MAX_K);
    FGNN_REQUIRE((int64_t)n_clouds * P * k <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_knn_graph: more than 2^31 edges");
    FGNN_REQUIRE(points && src_ind, FGNN_ERR_NULL, "fgnn_knn_graph: NULL argument");
    FGNN_REQUIRE(n_clouds <= 65535, FGNN_ERR_LIMIT, "fgnn_knn_graph: more than 65535 clouds");
    if (n_clouds == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    const int rg = P <= 256 ? 1 : P <= 512 ? 2 : 4;     // tile = 256 * rg candidate points
    if (k <= 64) {
        if (rg == 1) knn_launch<1, 1>(n_clouds, P, D, k, points, src_ind, st);
        else if (rg == 2) knn_launch<2, 1>(n_clouds, P, D, k, points, src_ind, st);
        else knn_launch<4, 1>(n_clouds, P, D, k, points, src_ind, st);
    } else {
        if (rg == 1) knn_launch<1, 2>(n_clouds, P, D, k, points, src_ind, st);
        else if (rg == 2) knn_launch<2, 2>(n_clouds, P, D, k, points, src_ind, st);
        else knn_launch<4, 2>(n_clouds, P, D, k, points, src_ind, st);
    }
    return fgnn_launch_status("knn_kernel");
}
