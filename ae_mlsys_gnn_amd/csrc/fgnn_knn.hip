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
// Selection: k rounds per query; a round takes the wave-wide minimum (DPP butterfly), finds the
// holder with the smallest node id by ballots, records it in lane (round % 64) of the result
// registers and retires it.  The order is total (smaller distance first, smaller node id on equal
// distance), so the result is deterministic.  Clouds with more points than one tile keep the best
// k of the tiles seen so far in registers and run them through the next tile's selection, where
// they win ties because their ids are smaller.
#include "fgnn_common.h"
#include <float.h>

#define KNN_QW 4         // queries a wave processes together
#define KNN_WAVES 4      // waves per workgroup
#define KNN_DC 8         // dimensions per LDS slice
#define KNN_MAX_K 128    // KR = 2 result registers per lane

// Takes the k best of {prior list (pd, pi), the tile's distances} in order; the new list replaces
// the prior one.  List position p lives in lane p % 64 of register p / 64.
template <int NR, int KR>
__device__ __forceinline__ void knn_select(float (&dist)[NR], int tile0, float (&pd)[KR], int (&pi)[KR], int k, int lane, int fallback_id)
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

template <int RG, int KR>
__global__ __launch_bounds__(KNN_WAVES * 64) void knn_kernel(int P, int D, int k, int rows_aligned, const float *__restrict__ pts, int *__restrict__ out)
{
    constexpr int NR = 4 * RG;                  // distances per lane and query
    constexpr int TILE = 256 * RG;              // candidate points per tile
    __shared__ __attribute__((aligned(16))) float cs[KNN_DC * TILE];        // [dimension of the slice][point of the tile]
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
        for (int a = 0; a < KNN_QW; ++a) knn_select<NR, KR>(acc[a], tile0, pd[a], pi[a], k, lane, qrow[a]);
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
