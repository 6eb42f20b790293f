// Brute-force k-nearest-neighbour graph builder for batched point clouds (the graph the fused
// EdgeConv consumes).  The reference builds it with DGL's KNNGraph on every layer of its DGCNN
// loop (script/train/train_edgeconv_our.py:51-55): per cloud, for every point the k nearest points
// of the same cloud, the point itself included, grouped by destination.
//
// One thread per query point, 64 queries per workgroup.  Candidates of the cloud stream through LDS
// in tiles of 64 points; squared distances are accumulated dimension by dimension in a fixed order;
// every thread keeps its current best k as a sorted list in LDS (insertion on improvement).  The
// order is total: smaller distance first, smaller node id on equal distance, so the result is
// deterministic.
#include "fgnn_common.h"

#define KNN_Q 64        // queries per workgroup
#define KNN_T 64        // candidates per LDS tile

__global__ __launch_bounds__(KNN_Q) void knn_kernel(int P, int D, int k, const float *__restrict__ pts, int *__restrict__ out)
{
    extern __shared__ float lds[];
    const int DP = D + 1;                               // padded row: conflict-free per-thread query reads
    float *qs = lds;                                    // [KNN_Q][DP]
    float *cs = qs + KNN_Q * DP;                        // [KNN_T][D]
    float *bd = cs + KNN_T * D;                         // [k][KNN_Q] best distances, ascending in k
    int *bi = (int *)(bd + (size_t)k * KNN_Q);          // [k][KNN_Q] their node ids (local to the cloud)
    const int tid = (int)threadIdx.x;
    const int cloud = (int)blockIdx.y;
    const int q0 = (int)blockIdx.x * KNN_Q;
    const float *cp = pts + (size_t)cloud * P * D;
    const int q = q0 + tid;
    const bool live = q < P;
    for (int i = tid; i < KNN_Q * D; i += KNN_Q) {
        int r = i / D, d = i - r * D;
        qs[r * DP + d] = (q0 + r < P) ? cp[(size_t)(q0 + r) * D + d] : 0.f;
    }
    for (int j = 0; j < k; ++j) { bd[j * KNN_Q + tid] = INFINITY; bi[j * KNN_Q + tid] = 0x7fffffff; }
    __syncthreads();
    for (int c0 = 0; c0 < P; c0 += KNN_T) {
        const int nc = min(KNN_T, P - c0);
        for (int i = tid; i < nc * D; i += KNN_Q) cs[i] = cp[(size_t)c0 * D + i];
        __syncthreads();
        if (live) {
            for (int c = 0; c < nc; ++c) {
                float dist = 0.f;
                for (int d = 0; d < D; ++d) {
                    float df = qs[tid * DP + d] - cs[c * D + d];
                    dist = fmaf(df, df, dist);
                }
                const int id = c0 + c;
                float wd = bd[(k - 1) * KNN_Q + tid];
                int wi = bi[(k - 1) * KNN_Q + tid];
                if (dist < wd || (dist == wd && id < wi)) {
                    int j = k - 1;
                    while (j > 0) {
                        float pd = bd[(j - 1) * KNN_Q + tid];
                        int pi = bi[(j - 1) * KNN_Q + tid];
                        if (pd < dist || (pd == dist && pi < id)) break;
                        bd[j * KNN_Q + tid] = pd;
                        bi[j * KNN_Q + tid] = pi;
                        --j;
                    }
                    bd[j * KNN_Q + tid] = dist;
                    bi[j * KNN_Q + tid] = id;
                }
            }
        }
        __syncthreads();
    }
    if (live) {
        int *o = out + ((size_t)cloud * P + q) * k;
        for (int j = 0; j < k; ++j) o[j] = cloud * P + bi[j * KNN_Q + tid];
    }
}

extern "C" int fgnn_knn_graph(int n_clouds, int P, int D, int k, const float *points, int32_t *src_ind, void *stream)
{
    FGNN_REQUIRE(n_clouds >= 0 && P >= 1 && D >= 1 && k >= 1, FGNN_ERR_SHAPE, "fgnn_knn_graph: bad sizes clouds=%d P=%d D=%d k=%d", n_clouds, P, D, k);
    FGNN_REQUIRE(k <= P, FGNN_ERR_SHAPE, "fgnn_knn_graph: k=%d exceeds the %d points of a cloud", k, P);
    FGNN_REQUIRE((int64_t)n_clouds * P * k <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_knn_graph: more than 2^31 edges");
    FGNN_REQUIRE(points && src_ind, FGNN_ERR_NULL, "fgnn_knn_graph: NULL argument");
    size_t shm = ((size_t)KNN_Q * (D + 1) + (size_t)KNN_T * D + 2 * (size_t)k * KNN_Q) * sizeof(float);
    FGNN_REQUIRE(shm <= 64 * 1024, FGNN_ERR_LIMIT, "fgnn_knn_graph: D=%d, k=%d need %zu bytes of LDS (limit 64 KiB)", D, k, shm);
    FGNN_REQUIRE(n_clouds <= 65535, FGNN_ERR_LIMIT, "fgnn_knn_graph: more than 65535 clouds");
    if (n_clouds == 0) return 0;
    dim3 grid((unsigned)((P + KNN_Q - 1) / KNN_Q), (unsigned)n_clouds);
    hipLaunchKernelGGL(knn_kernel, grid, dim3(KNN_Q), shm, (hipStream_t)stream, P, D, k, points, src_ind);
    return fgnn_launch_status("knn_kernel");
}
