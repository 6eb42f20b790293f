// Fused EdgeConv forward / backward for gfx950.
//
// Contract (operators/fused_edgeconv.py:18-29 of the reference; tie rule of the DGL max
// reducer that layers/edgeconv_layer.py:102-109 uses):
//   out[i,f]    = max_p (h_dst[i,f] + h_src[src_ind[p],f]),  p in [i*k, (i+1)*k)
//   argmax[i,f] = src_ind[p*] for the FIRST maximal p (strict > update), stored as int32.
// One fp32 add per candidate, so the maximum is bit-identical to the composed form.
//
// Mapping: a thread owns VEC consecutive features of one node and walks the k neighbours in
// position order with 4 row loads in flight; the F/VEC threads of a node read one contiguous
// feature row per neighbour.  The problem is tiny (hundreds of MB), so there is no LDS staging.
#include "fgnn_common.h"

template <int VEC>
__global__ __launch_bounds__(256) void edgeconv_fwd_kernel(int N, int F, int k, const int *__restrict__ src_ind,
                                                           const float *__restrict__ h_src, const float *__restrict__ h_dst,
                                                           float *__restrict__ out, int *__restrict__ argmax)
{
    const int per = F / VEC;
    const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= (long long)N * per) return;
    const int node = (int)(tid / per);
    const int fo = (int)(tid - (long long)node * per) * VEC;
    fg_vec<VEC> d;
    d.load(h_dst + (size_t)node * F + fo);
    const int *nb = src_ind + (size_t)node * k;
    float best[VEC];
    int arg[VEC];
    auto consider = [&](int j, const fg_vec<VEC> &s, bool first) {
        const float *sv = reinterpret_cast<const float *>(&s);
        const float *dv = reinterpret_cast<const float *>(&d);
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            float v = dv[c] + sv[c];
            if (first || v > best[c]) { best[c] = v; arg[c] = j; }
        }
    };
    int t = 0;
    for (; t + 4 <= k; t += 4) {
        int j0 = nb[t], j1 = nb[t + 1], j2 = nb[t + 2], j3 = nb[t + 3];
        fg_vec<VEC> s0, s1, s2, s3;
        s0.load(h_src + (size_t)j0 * F + fo);
        s1.load(h_src + (size_t)j1 * F + fo);
        s2.load(h_src + (size_t)j2 * F + fo);
        s3.load(h_src + (size_t)j3 * F + fo);
        consider(j0, s0, t == 0);
        consider(j1, s1, false);
        consider(j2, s2, false);
        consider(j3, s3, false);
    }
    for (; t < k; ++t) {
        int j = nb[t];
        fg_vec<VEC> s;
        s.load(h_src + (size_t)j * F + fo);
        consider(j, s, t == 0);
    }
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
        out[(size_t)node * F + fo + c] = best[c];
        argmax[(size_t)node * F + fo + c] = arg[c];
    }
}

__global__ __launch_bounds__(256) void fgnn_fill_f32_kernel(float *p, size_t n, float v)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// grad_src[argmax[i,f], f] += grad_out[i,f].  grad_src is cleared by a fill kernel on the same
// stream first (the reference clears inside the scattering kernel and races,
// src/fused_edgeconv/fused_edgeconv.cu:184-185).
__global__ __launch_bounds__(256) void edgeconv_bwd_kernel(long long total, int F, const int *__restrict__ argmax,
                                                           const float *__restrict__ grad_out, float *__restrict__ grad_src)
{
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int f = (int)(i % F);
    unsafeAtomicAdd(grad_src + (size_t)argmax[i] * F + f, grad_out[i]);     // hardware float add (device memory), no CAS loop
}

int fgnn_fill_f32(float *p, size_t n, float v, hipStream_t st)
{
    if (n == 0) return 0;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fgnn_fill_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p, n, v);
    return fgnn_launch_status("fill");
}

extern "C" int fgnn_edgeconv_forward(int N, int n_src, int F, int k, const int32_t *src_ind, const float *h_src,
                                     const float *h_dst, float *out, int32_t *argmax, void *stream)
{
    FGNN_REQUIRE(N >= 0 && n_src >= 0 && F >= 1 && k >= 1, FGNN_ERR_SHAPE, "fgnn_edgeconv_forward: bad sizes N=%d n_src=%d F=%d k=%d", N, n_src, F, k);
    FGNN_REQUIRE(src_ind && h_src && h_dst && out && argmax, FGNN_ERR_NULL, "fgnn_edgeconv_forward: NULL argument");
    FGNN_REQUIRE((int64_t)N * k <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_edgeconv_forward: N*k exceeds int32");
    if (N == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    bool v4 = (F % 4 == 0) && fgnn_aligned16(h_src) && fgnn_aligned16(h_dst);
    long long threads = (long long)N * (v4 ? F / 4 : F);
    unsigned grid = (unsigned)((threads + 255) / 256);
    if (v4) hipLaunchKernelGGL(edgeconv_fwd_kernel<4>, dim3(grid), dim3(256), 0, st, N, F, k, src_ind, h_src, h_dst, out, argmax);
    else hipLaunchKernelGGL(edgeconv_fwd_kernel<1>, dim3(grid), dim3(256), 0, st, N, F, k, src_ind, h_src, h_dst, out, argmax);
    return fgnn_launch_status("edgeconv_fwd_kernel");
}

extern "C" int fgnn_edgeconv_backward(int N, int n_src, int F, const int32_t *argmax, const float *grad_out,
                                      float *grad_src, void *stream)
{
    FGNN_REQUIRE(N >= 0 && n_src >= 0 && F >= 1, FGNN_ERR_SHAPE, "fgnn_edgeconv_backward: bad sizes");
    FGNN_REQUIRE(argmax && grad_out && grad_src, FGNN_ERR_NULL, "fgnn_edgeconv_backward: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    int rc = fgnn_fill_f32(grad_src, (size_t)n_src * F, 0.f, st);
    if (rc) return rc;
    long long total = (long long)N * F;
    if (total == 0) return 0;
    unsigned grid = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(edgeconv_bwd_kernel, dim3(grid), dim3(256), 0, st, total, F, argmax, grad_out, grad_src);
    return fgnn_launch_status("edgeconv_bwd_kernel");
}
