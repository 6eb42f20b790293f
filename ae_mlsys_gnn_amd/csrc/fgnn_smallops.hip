// The small per-edge operators of the reference's operators/ package: multi-head SDDMM,
// permuted row gather (mhtranspose), edge softmax and u_add_v, each with its backward.
// One wave per CSR row, lanes over (edge, head) or (edge, column) pairs.
#include "fgnn_common.h"

// out[p,h] = <a[row,h,:], b[col_ind[p],h,:]> (src/sddmm/mhsddmm.cu:5-81 of the reference, which
// finds the row of each edge by binary search; here the row is the work item).
template <int VEC, int R, bool FULL, int LPH>
__global__ __launch_bounds__(FGNN_TPB) void mhsddmm_kernel(int N, int H, int F, int HF, int lphp, const int *ptr, const int *idx,
                                                           const float *a, const float *b, float *out)
{
    extern __shared__ float lds[];
    int row = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (row >= N) return;
    const int lane = fg_lane();
    float *scr = lds + fg_wave() * (64 * R);
    const int pb = fg_uni(ptr[row]), pe = fg_uni(ptr[row + 1]);
    fg_lanemap<VEC, R> lm;
    if (lphp) lm.init_padded(lane, H, F, lphp); else lm.init(lane, HF, F);      // lphp: head-aligned lanes for DPP sums
    fg_vec<VEC> ar[R];
#pragma unroll
    for (int r = 0; r < R; ++r) { if (FULL || lm.ok[r]) ar[r].load(a + (size_t)row * HF + lm.eoff[r]); else ar[r].zero(); }
    for (int c = pb; c < pe; c += 64) {
        int q = c + lane;
        int cnt = min(64, pe - c);
        int id = idx[q < pe ? q : c];
        for (int t = 0; t < cnt; t += 4) {
            fg_vec<VEC> ld[4][R];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int j = __builtin_amdgcn_readlane(id, t + u);
#pragma unroll
                for (int r = 0; r < R; ++r) { if (FULL || lm.ok[r]) ld[u][r].load(b + (size_t)j * HF + lm.eoff[r]); else ld[u][r].zero(); }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (t + u >= cnt) break;
                float d[R];
#pragma unroll
                for (int r = 0; r < R; ++r) d[r] = ld[u][r].dot(ar[r]);
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
}

extern "C" int fgnn_mhsddmm(int N, int64_t E, int H, int F, const int32_t *row_ptr, const int32_t *col_ind, const float *a,
                            const float *b, float *out, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1 && F >= 1, FGNN_ERR_SHAPE, "fgnn_mhsddmm: bad sizes");
    FGNN_REQUIRE(H <= 64 && (int64_t)H * F <= 1024, FGNN_ERR_LIMIT, "fgnn_mhsddmm: H=%d H*F=%lld unsupported", H, (long long)H * F);
    FGNN_REQUIRE(row_ptr && (col_ind || E == 0) && a && b && (out || E == 0), FGNN_ERR_NULL, "fgnn_mhsddmm: NULL argument");
    if (N == 0 || E == 0) return 0;
    const int HF = H * F;
    fgnn_rowcfg cfg;
    FGNN_REQUIRE(fgnn_pick_rowcfg(HF, F, fgnn_aligned16(a) && fgnn_aligned16(b), &cfg), FGNN_ERR_LIMIT, "fgnn_mhsddmm: unsupported row width %d", HF);
    const int lphp = fgnn_pad_lph(cfg.vec, H, F);
    if (lphp) { int w = H * lphp * 4; cfg.r = w <= 256 ? 1 : w <= 512 ? 2 : 4; cfg.full = false; }
    const int lph = lphp ? lphp : fgnn_pick_lph(cfg.vec, F);
    const unsigned grid = (unsigned)((N + FGNN_WPB - 1) / FGNN_WPB);
    hipStream_t st = (hipStream_t)stream;
    return fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
        return fgnn_dispatch_lph(VEC == 4 ? lph : 0, [&]<int LPH>() -> int {
            hipLaunchKernelGGL((mhsddmm_kernel<VEC, R, FULL, (VEC == 4 ? LPH : 0)>), dim3(grid), dim3(FGNN_TPB),
                               (size_t)FGNN_WPB * 64 * R * sizeof(float), st, N, H, F, HF, lphp, row_ptr, col_ind, a, b, out);
            return fgnn_launch_status("mhsddmm_kernel");
        });
    });
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

// out[q,:] = in[permute[q],:]  (src/csr2csc/mhtranspose.cu:6-26)
__global__ __launch_bounds__(256) void gather_rows_kernel(int64_t total, int W, const int *permute, const float *in, float *out)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int64_t q = i / W;
    int w = (int)(i - q * W);
    out[i] = in[(size_t)permute[q] * W + w];
}

extern "C" int fgnn_gather_rows(int64_t E, int W, const int32_t *permute, const float *in, float *out, void *stream)
{
    FGNN_REQUIRE(E >= 0 && W >= 1, FGNN_ERR_SHAPE, "fgnn_gather_rows: bad sizes");
    FGNN_REQUIRE(E == 0 || (permute && in && out), FGNN_ERR_NULL, "fgnn_gather_rows: NULL argument");
    if (E == 0) return 0;
    int64_t total = E * W;
    FGNN_REQUIRE((total + 255) / 256 <= 2147483647LL, FGNN_ERR_LIMIT, "fgnn_gather_rows: too many elements");
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, total, W, permute, in, out);
    return fgnn_launch_status("gather_rows_kernel");
}

// Per-row, per-head softmax over [E,H] (src/edge_softmax/edge_softmax.cu:7-61) and its backward
// s*(g - sum_row s*g) (:63-98).  Lanes stride over the row's edges, one head at a time.
__global__ __launch_bounds__(FGNN_TPB) void edge_softmax_kernel(int N, int H, const int *ptr, const float *in, float *out)
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

__global__ __launch_bounds__(FGNN_TPB) void edge_softmax_bwd_kernel(int N, int H, const int *ptr, const float *sm, const float *g, float *gin)
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
    hipLaunchKernelGGL(edge_softmax_kernel, dim3((unsigned)((N + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, (hipStream_t)stream, N, H, row_ptr, in, out);
    return fgnn_launch_status("edge_softmax_kernel");
}

extern "C" int fgnn_edge_softmax_backward(int N, int64_t E, int H, const int32_t *row_ptr, const float *sm, const float *grad_out,
                                          float *grad_in, void *stream)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1, FGNN_ERR_SHAPE, "fgnn_edge_softmax_backward: bad sizes");
    FGNN_REQUIRE(row_ptr && (E == 0 || (sm && grad_out && grad_in)), FGNN_ERR_NULL, "fgnn_edge_softmax_backward: NULL argument");
    if (N == 0 || E == 0) return 0;
    hipLaunchKernelGGL(edge_softmax_bwd_kernel, dim3((unsigned)((N + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, (hipStream_t)stream, N, H, row_ptr, sm,
                       grad_out, grad_in);
    return fgnn_launch_status("edge_softmax_bwd_kernel");
}

// out[p,w] = row_val[row(p),w] + col_val[col_ind[p],w]  (src/u_add_v/u_add_v.cu:4-26)
__global__ __launch_bounds__(FGNN_TPB) void u_add_v_kernel(int N, int W, const int *ptr, const int *idx, const float *rv, const float *cv, float *out)
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

// grad_row[i,w] = sum over the row's edges; grad_col[j,w] += g[p,w] with float atomics into a
// zero-filled buffer (the reference adds into uninitialised memory, src/u_add_v/u_add_v.cu:67,87).
__global__ __launch_bounds__(FGNN_TPB) void u_add_v_bwd_kernel(int N, int W, const int *ptr, const int *idx, const float *g, float *grow, float *gcol)
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
    hipLaunchKernelGGL(u_add_v_kernel, dim3((unsigned)((N + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, (hipStream_t)stream, N, W, row_ptr, col_ind,
                       row_val, col_val, out);
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
    hipLaunchKernelGGL(u_add_v_bwd_kernel, dim3((unsigned)((N + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, st, N, W, row_ptr, col_ind, grad_out,
                       grad_row, grad_col);
    return fgnn_launch_status("u_add_v_bwd_kernel");
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
