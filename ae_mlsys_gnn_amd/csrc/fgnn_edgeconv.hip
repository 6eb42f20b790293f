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
#include <mutex>
#include "fgnn_common.h"

// per_xcd > 0: the workgroups of one XCD (blockIdx.x % FGNN_NUM_XCD) take one contiguous eighth of the nodes.  The neighbours of
// a node of a batched kNN graph lie in its own cloud; with the workgroups dealt round-robin every XCD gathered from every
// cloud and the feature matrix crossed the fabric eight times (106 MB fetched for 32 clouds of 1024 points x 64 floats).
template <int VEC>
__global__ __launch_bounds__(256) void edgeconv_fwd_kernel(int N, int F, int k, unsigned per_xcd, const int *__restrict__ src_ind,
                                                           const float *__restrict__ h_src, const float *__restrict__ h_dst,
                                                           float out_slope, float *__restrict__ out, int *__restrict__ argmax)
{
    const int per = F / VEC;
    const unsigned chunk = per_xcd ? (blockIdx.x % FGNN_NUM_XCD) * per_xcd + blockIdx.x / FGNN_NUM_XCD : blockIdx.x;
    const long long tid = (long long)chunk * blockDim.x + threadIdx.x;
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
        // optional LeakyReLU on the way out (out_slope == 1: the identity, bit for bit)
        out[(size_t)node * F + fo + c] = best[c] > 0.f ? best[c] : best[c] * out_slope;
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
// act_out != NULL: the forward ended in LeakyReLU(act_slope) and act_out is its output; the gradient of the
// pre-activation, grad_out * (act_out > 0 ? 1 : act_slope), is what gets scattered, and it is written to grad_dst
// (the gradient of h_dst) on the way.
__device__ __forceinline__ float ec_masked(float g, const float *act_out, float act_slope, long long i)
{
    return act_out ? (act_out[i] > 0.f ? g : g * act_slope) : g;
}
__global__ __launch_bounds__(256) void edgeconv_bwd_kernel(long long total, int F, const int *__restrict__ argmax,
                                                           const float *__restrict__ grad_out, const float *__restrict__ act_out, float act_slope,
                                                           float *__restrict__ grad_src, float *__restrict__ grad_dst)
{
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int f = (int)(i % F);
    const float g = ec_masked(grad_out[i], act_out, act_slope, i);
    if (grad_dst) grad_dst[i] = g;
    unsafeAtomicAdd(grad_src + (size_t)argmax[i] * F + f, g);     // hardware float add (device memory), no CAS loop
}

int fgnn_fill_f32(float *p, size_t n, float v, hipStream_t st)
{
    if (n == 0) return 0;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fgnn_fill_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p, n, v);
    return fgnn_launch_status("fill");
}

static int edgeconv_forward_run(const char *fn, int N, int n_src, int F, int k, const int32_t *src_ind, const float *h_src,
                                const float *h_dst, float out_slope, float *out, int32_t *argmax, void *stream)
{
    FGNN_REQUIRE(N >= 0 && n_src >= 0 && F >= 1 && k >= 1, FGNN_ERR_SHAPE, "%s: bad sizes N=%d n_src=%d F=%d k=%d", fn, N, n_src, F, k);
    FGNN_REQUIRE(src_ind && h_src && h_dst && out && argmax, FGNN_ERR_NULL, "%s: NULL argument", fn);
    FGNN_REQUIRE((int64_t)N * k <= 2147483647LL, FGNN_ERR_LIMIT, "%s: N*k exceeds int32", fn);
    if (N == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    bool v4 = (F % 4 == 0) && fgnn_aligned16(h_src) && fgnn_aligned16(h_dst);
    long long threads = (long long)N * (v4 ? F / 4 : F);
    unsigned grid = (unsigned)((threads + 255) / 256);
    unsigned per_xcd = 0;
    if (grid >= 8 * FGNN_NUM_XCD && fgnn_current_device_has_xcd_mapping()) {
        per_xcd = (grid + FGNN_NUM_XCD - 1) / FGNN_NUM_XCD;
        grid = per_xcd * FGNN_NUM_XCD;
    }
    if (v4) hipLaunchKernelGGL(edgeconv_fwd_kernel<4>, dim3(grid), dim3(256), 0, st, N, F, k, per_xcd, src_ind, h_src, h_dst, out_slope, out, argmax);
    else hipLaunchKernelGGL(edgeconv_fwd_kernel<1>, dim3(grid), dim3(256), 0, st, N, F, k, per_xcd, src_ind, h_src, h_dst, out_slope, out, argmax);
    return fgnn_launch_status("edgeconv_fwd_kernel");
}

extern "C" int fgnn_edgeconv_forward(int N, int n_src, int F, int k, const int32_t *src_ind, const float *h_src,
                                     const float *h_dst, float *out, int32_t *argmax, void *stream)
{
    return edgeconv_forward_run("fgnn_edgeconv_forward", N, n_src, F, k, src_ind, h_src, h_dst, 1.f, out, argmax, stream);
}

extern "C" int fgnn_edgeconv_forward_lrelu(int N, int n_src, int F, int k, const int32_t *src_ind, const float *h_src,
                                           const float *h_dst, float out_slope, float *out, int32_t *argmax, void *stream)
{
    FGNN_REQUIRE(out_slope > 0.f, FGNN_ERR_LIMIT, "fgnn_edgeconv_forward_lrelu: out_slope=%g; the backward reads the sign of the pre-activation "
                 "off the output, which needs a positive slope", (double)out_slope);
    return edgeconv_forward_run("fgnn_edgeconv_forward_lrelu", N, n_src, F, k, src_ind, h_src, h_dst, out_slope, out, argmax, stream);
}

// fn: the entry point the caller used, for the error messages
static int edgeconv_backward_run(const char *fn, int N, int n_src, int F, const int32_t *argmax, const float *grad_out, const float *act_out,
                                 float act_slope, float *grad_src, float *grad_dst, void *stream)
{
    FGNN_REQUIRE(N >= 0 && n_src >= 0 && F >= 1, FGNN_ERR_SHAPE, "%s: bad sizes", fn);
    FGNN_REQUIRE(argmax && grad_out && grad_src, FGNN_ERR_NULL, "%s: NULL argument", fn);
    hipStream_t st = (hipStream_t)stream;
    int rc = fgnn_fill_f32(grad_src, (size_t)n_src * F, 0.f, st);
    if (rc) return rc;
    long long total = (long long)N * F;
    if (total == 0) return 0;
    unsigned grid = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(edgeconv_bwd_kernel, dim3(grid), dim3(256), 0, st, total, F, argmax, grad_out, act_out, act_slope, grad_src, grad_dst);
    return fgnn_launch_status("edgeconv_bwd_kernel");
}

extern "C" int fgnn_edgeconv_backward(int N, int n_src, int F, const int32_t *argmax, const float *grad_out,
                                      float *grad_src, void *stream)
{
    return edgeconv_backward_run("fgnn_edgeconv_backward", N, n_src, F, argmax, grad_out, nullptr, 1.f, grad_src, nullptr, stream);
}

// ---------------------------------------------------------------------------------------------------
// Backward for batched point clouds.  `block` is a hint: the neighbours of destination rows
// [b*block, (b+1)*block) mostly lie in source rows of the same range (a kNN graph of clouds of `block`
// points each has them all there).  A workgroup owns block b and FS feature columns, accumulates its
// contributions in an LDS tile with LDS float atomics and writes the tile out with plain stores: no
// clearing pass, no global atomics.  A contribution whose source lies outside the block is appended to
// an overflow list and applied by a second, normally empty, kernel with global atomics, so a wrong
// hint costs time, never correctness.
#define EC_OVF_HEADER 64        // ints in front of the overflow list (counter + padding)

#define EC_BT 1024      // threads per workgroup of the blocked backward
// n_tiles > 0: a one-dimensional grid in which the n_tiles column tiles of a block all run on one XCD (workgroup w runs on XCD
// w % FGNN_NUM_XCD): a tile row is FS * 4 = 32 bytes of a 128-byte line of grad_out and argmax, and with the tiles of a block
// spread over the XCDs every line crossed the fabric once per XCD that held one of its four tiles (67 MB fetched for 16.8 MB).
template <int FS>
__global__ __launch_bounds__(EC_BT) void edgeconv_bwd_blocked_kernel(int N, int F, int block, int n_tiles, const int *__restrict__ argmax,
                                                                     const float *__restrict__ grad_out, const float *__restrict__ act_out,
                                                                     float act_slope, float *__restrict__ grad_src, float *__restrict__ grad_dst,
                                                                     int *__restrict__ ovf)
{
    extern __shared__ float tile[];                 // [rows of the block][FS]
    int b = (int)blockIdx.y, tx = (int)blockIdx.x;
    if (n_tiles > 0) {
        const unsigned j = blockIdx.x / FGNN_NUM_XCD;
        b = (int)((j / (unsigned)n_tiles) * FGNN_NUM_XCD + blockIdx.x % FGNN_NUM_XCD);
        tx = (int)(j % (unsigned)n_tiles);
        if ((long long)b * block >= N) return;          // the last round of blocks may be incomplete (uniform over the workgroup)
    }
    const int f0 = tx * FS;
    const int r0 = b * block, rows = min(block, N - r0), fs = min(FS, F - f0);
    const int total = rows * FS;
    for (int i = (int)threadIdx.x; i < total; i += EC_BT) tile[i] = 0.f;
    __syncthreads();
    constexpr int U = 4;                            // elements in flight per thread
    for (int i0 = (int)threadIdx.x; i0 < total; i0 += EC_BT * U) {
        int g[U], a[U];
        float v[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * EC_BT;
            const int r = i / FS, ff = i - r * FS;
            ok[u] = i < total && ff < fs;
            g[u] = (r0 + r) * F + f0 + ff;           // N*F < 2^31 is checked on the host
            a[u] = ok[u] ? argmax[g[u]] : 0;
            v[u] = ok[u] ? ec_masked(grad_out[g[u]], act_out, act_slope, g[u]) : 0.f;
            if (ok[u] && grad_dst) grad_dst[g[u]] = v[u];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!ok[u]) continue;
            const int i = i0 + u * EC_BT;
            const int ff = i % FS;
            const int local = a[u] - r0;
            if ((unsigned)local < (unsigned)rows) {
                __hip_atomic_fetch_add(&tile[local * FS + ff], v[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            } else {
                int slot = atomicAdd(ovf, 1);
                ovf[EC_OVF_HEADER + slot] = g[u];
            }
        }
    }
    __syncthreads();
    for (int i = (int)threadIdx.x; i < total; i += EC_BT) {
        const int r = i / FS, ff = i - r * FS;
        if (ff < fs) grad_src[(size_t)(r0 + r) * F + f0 + ff] = tile[i];
    }
}

__global__ __launch_bounds__(256) void edgeconv_bwd_overflow_kernel(int F, const int *__restrict__ argmax, const float *__restrict__ grad_out,
                                                                    const float *__restrict__ act_out, float act_slope,
                                                                    float *__restrict__ grad_src, const int *__restrict__ ovf)
{
    const int count = ovf[0];
    for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < count; i += (int)(gridDim.x * 256)) {
        const int g = ovf[EC_OVF_HEADER + i];
        unsafeAtomicAdd(grad_src + (size_t)argmax[g] * F + (g % F), ec_masked(grad_out[g], act_out, act_slope, g));
    }
}

extern "C" size_t fgnn_edgeconv_backward_blocked_workspace_bytes(int N, int F)
{
    return ((size_t)N * F + EC_OVF_HEADER) * sizeof(int32_t);
}

// Tile width of the blocked kernel for a block size (0: no usable LDS tile)
static inline int ec_blocked_fs(int block) { return block <= 2048 ? 8 : block <= 4096 ? 4 : 0; }

// The two launches of the blocked backward; ovf: (N*F + EC_OVF_HEADER) ints of device scratch.
static int edgeconv_backward_blocked_run(int N, int F, int block, int fs, const int32_t *argmax, const float *grad_out, float *grad_src,
                                         int *ovf, hipStream_t st, const float *act_out = nullptr, float act_slope = 1.f, float *grad_dst = nullptr)
{
    int rc = fgnn_fill_f32((float *)ovf, 1, 0.f, st);        // the counter (bit pattern of 0.0f is integer 0); a kernel, so capturable
    if (rc) return rc;
    const long long n_tiles = (F + fs - 1) / fs, n_blocks = ((long long)N + block - 1) / block;
    dim3 grid((unsigned)n_tiles, (unsigned)n_blocks);
    FGNN_REQUIRE(n_blocks <= 65535, FGNN_ERR_LIMIT, "fgnn_edgeconv_backward_blocked: more than 65535 blocks");
    int tiles_arg = 0;
    if (n_tiles > 1 && fgnn_current_device_has_xcd_mapping()) {          // all column tiles of a block on one XCD
        grid = dim3((unsigned)(((n_blocks + FGNN_NUM_XCD - 1) / FGNN_NUM_XCD) * FGNN_NUM_XCD * n_tiles));
        tiles_arg = (int)n_tiles;
    }
    const size_t shm = (size_t)block * fs * sizeof(float);
    if (fs == 8) hipLaunchKernelGGL(edgeconv_bwd_blocked_kernel<8>, grid, dim3(EC_BT), shm, st, N, F, block, tiles_arg, argmax, grad_out, act_out, act_slope, grad_src, grad_dst, ovf);
    else hipLaunchKernelGGL(edgeconv_bwd_blocked_kernel<4>, grid, dim3(EC_BT), shm, st, N, F, block, tiles_arg, argmax, grad_out, act_out, act_slope, grad_src, grad_dst, ovf);
    rc = fgnn_launch_status("edgeconv_bwd_blocked_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(edgeconv_bwd_overflow_kernel, dim3(64), dim3(256), 0, st, F, argmax, grad_out, act_out, act_slope, grad_src, ovf);
    return fgnn_launch_status("edgeconv_bwd_overflow_kernel");
}

extern "C" int fgnn_edgeconv_backward_blocked(int N, int n_src, int F, int block, const int32_t *argmax, const float *grad_out,
                                              float *grad_src, void *workspace, size_t workspace_bytes, void *stream)
{
    FGNN_REQUIRE(N >= 0 && n_src >= 0 && F >= 1 && block >= 1, FGNN_ERR_SHAPE, "fgnn_edgeconv_backward_blocked: bad sizes");
    FGNN_REQUIRE(argmax && grad_out && grad_src, FGNN_ERR_NULL, "fgnn_edgeconv_backward_blocked: NULL argument");
    FGNN_REQUIRE((int64_t)N * F <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_edgeconv_backward_blocked: N*F exceeds int32");
    // tile of the largest FS that fits 64 KiB of LDS; without a usable tile, or with source rows that no
    // destination block covers, the plain scatter does the job
    const int fs = ec_blocked_fs(block);
    if (fs == 0 || n_src != N || (size_t)block * fs * sizeof(float) > 64 * 1024)
        return edgeconv_backward_run("fgnn_edgeconv_backward_blocked", N, n_src, F, argmax, grad_out, nullptr, 1.f, grad_src, nullptr, stream);
    size_t need = fgnn_edgeconv_backward_blocked_workspace_bytes(N, F);
    FGNN_REQUIRE(N == 0 || (workspace && workspace_bytes >= need), FGNN_ERR_WORKSPACE, "fgnn_edgeconv_backward_blocked: workspace %zu < %zu bytes",
                 workspace_bytes, need);
    if (N == 0) return 0;
    return edgeconv_backward_blocked_run(N, F, block, fs, argmax, grad_out, grad_src, (int *)workspace, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------------
// The blocked backward for callers that cannot allocate.  Its overflow list lives in a file-scope device
// array of a fixed size: every GPU the library runs on holds one copy (at its own address) until the
// process ends.  The array's name is only a host-side handle; the device address is looked up once per
// device with hipGetSymbolAddress and that pointer is what the kernels get.
#define EC_STATIC_MAX_ELEMS (4 * 1024 * 1024)         // largest N*F the static scratch serves (16 MiB + header)
#define EC_STATIC_MAX_DEVICES 64
static __device__ __align__(256) int32_t ec_static_scratch[EC_STATIC_MAX_ELEMS + EC_OVF_HEADER];
static std::mutex ec_static_mutex;
static int32_t *ec_static_ptr[EC_STATIC_MAX_DEVICES];   // per device: address of that device's copy (NULL until looked up)

static int ec_static_scratch_for_current_device(int32_t **out)
{
    int dev = -1;
    FGNN_HIP(hipGetDevice(&dev));
    FGNN_REQUIRE(dev >= 0 && dev < EC_STATIC_MAX_DEVICES, FGNN_ERR_LIMIT, "fgnn_edgeconv_backward_blocked_static: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(ec_static_mutex);
    if (!ec_static_ptr[dev]) {
        void *p = nullptr;
        FGNN_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(ec_static_scratch)));
        FGNN_REQUIRE(p != nullptr, FGNN_ERR_NULL, "fgnn_edgeconv_backward_blocked_static: no device address for the scratch array");
        ec_static_ptr[dev] = (int32_t *)p;
    }
    *out = ec_static_ptr[dev];
    return 0;
}

extern "C" size_t fgnn_edgeconv_backward_blocked_static_max_elems(void) { return (size_t)EC_STATIC_MAX_ELEMS; }

extern "C" int fgnn_edgeconv_backward_blocked_static(int N, int n_src, int F, int block, const int32_t *argmax, const float *grad_out,
                                                     float *grad_src, void *stream)
{
    FGNN_REQUIRE(N >= 0 && n_src >= 0 && F >= 1 && block >= 1, FGNN_ERR_SHAPE, "fgnn_edgeconv_backward_blocked_static: bad sizes");
    FGNN_REQUIRE(argmax && grad_out && grad_src, FGNN_ERR_NULL, "fgnn_edgeconv_backward_blocked_static: NULL argument");
    FGNN_REQUIRE((int64_t)N * F <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_edgeconv_backward_blocked_static: N*F exceeds int32");
    const int fs = ec_blocked_fs(block);
    if (fs == 0 || n_src != N || (size_t)block * fs * sizeof(float) > 64 * 1024)      // fill + scatter: no scratch, no allocation, any size
        return edgeconv_backward_run("fgnn_edgeconv_backward_blocked_static", N, n_src, F, argmax, grad_out, nullptr, 1.f, grad_src, nullptr, stream);
    // only the blocked form uses the static array, so only it is bound by its size
    FGNN_REQUIRE((int64_t)N * F <= (int64_t)EC_STATIC_MAX_ELEMS, FGNN_ERR_LIMIT,
                 "fgnn_edgeconv_backward_blocked_static: N*F = %lld exceeds the static scratch of %d elements; use fgnn_edgeconv_backward_blocked with a workspace",
                 (long long)N * F, EC_STATIC_MAX_ELEMS);
    if (N == 0) return 0;
    int32_t *ovf = nullptr;
    int rc = ec_static_scratch_for_current_device(&ovf);
    if (rc) return rc;
    // the list is rebuilt from its counter (cleared first) on every call: nothing of an earlier call is read
    return edgeconv_backward_blocked_run(N, F, block, fs, argmax, grad_out, grad_src, ovf, (hipStream_t)stream);
}

// The backward of fgnn_edgeconv_forward_lrelu: the LeakyReLU mask is replayed from the forward's output while the
// gradient is scattered, and the masked gradient (the gradient of h_dst) is written on the way: no separate
// elementwise pass in either direction.  block <= 0: plain scatter; block > 0: the blocked form (workspace as for
// fgnn_edgeconv_backward_blocked).
extern "C" int fgnn_edgeconv_backward_lrelu(int N, int n_src, int F, int block, const int32_t *argmax, const float *out, float out_slope,
                                            const float *grad_out, float *grad_src, float *grad_dst, void *workspace, size_t workspace_bytes,
                                            void *stream)
{
    FGNN_REQUIRE(N >= 0 && n_src >= 0 && F >= 1, FGNN_ERR_SHAPE, "fgnn_edgeconv_backward_lrelu: bad sizes");
    FGNN_REQUIRE(argmax && out && grad_out && grad_src && grad_dst, FGNN_ERR_NULL, "fgnn_edgeconv_backward_lrelu: NULL argument");
    FGNN_REQUIRE(out_slope > 0.f, FGNN_ERR_LIMIT, "fgnn_edgeconv_backward_lrelu: out_slope=%g must be positive", (double)out_slope);
    FGNN_REQUIRE((int64_t)N * F <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_edgeconv_backward_lrelu: N*F exceeds int32");
    const int fs = block > 0 ? ec_blocked_fs(block) : 0;
    if (fs == 0 || n_src != N || (size_t)block * fs * sizeof(float) > 64 * 1024)
        return edgeconv_backward_run("fgnn_edgeconv_backward_lrelu", N, n_src, F, argmax, grad_out, out, out_slope, grad_src, grad_dst, stream);
    size_t need = fgnn_edgeconv_backward_blocked_workspace_bytes(N, F);
    FGNN_REQUIRE(N == 0 || (workspace && workspace_bytes >= need), FGNN_ERR_WORKSPACE, "fgnn_edgeconv_backward_lrelu: workspace %zu < %zu bytes",
                 workspace_bytes, need);
    if (N == 0) return 0;
    return edgeconv_backward_blocked_run(N, F, block, fs, argmax, grad_out, grad_src, (int *)workspace, (hipStream_t)stream, out, out_slope, grad_dst);
}
