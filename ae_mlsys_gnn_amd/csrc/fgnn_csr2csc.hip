// GPU CSR -> CSC transpose (stable), replacing the reference's cuSPARSE call
// (src/csr2csc/csr2csc.cu:10-23).
//
// The transpose is a stable sort of the CSR positions by column: an LSD radix sort with 8-bit
// digits over key = col_ind[p], payload = p.  Each pass is histogram -> scan -> stable scatter:
// a workgroup owns a contiguous tile, each of its 4 waves a contiguous quarter of it, and a wave
// walks its quarter 64 elements at a time, ranking equal digits inside the wave with ballots, so
// equal keys keep their order (the order of CSR positions).  After the last pass the payload IS
// `permute`; col_ptr is read off the boundaries of the sorted keys and row_ind by a binary search
// of each position in row_ptr.  Integer work only, bit-exact and deterministic.
#include "fgnn_common.h"

#define RS_TPB 256
#define RS_ITEMS 16                    // elements per thread
#define RS_TILE (RS_TPB * RS_ITEMS)    // 4096 elements per workgroup
#define RS_SUB (64 * RS_ITEMS)         // 1024 per wave

__device__ __forceinline__ int rs_index(int block, int wave, int it, int lane) { return block * RS_TILE + wave * RS_SUB + it * 64 + lane; }

__global__ __launch_bounds__(RS_TPB) void rs_hist_kernel(const int *__restrict__ keys, int64_t n, int shift, int nblocks, int *__restrict__ hist)
{
    __shared__ int cnt[256];
    cnt[threadIdx.x] = 0;
    __syncthreads();
    const int wave = fg_wave(), lane = fg_lane();
#pragma unroll 4
    for (int it = 0; it < RS_ITEMS; ++it) {
        int64_t i = (int64_t)blockIdx.x * RS_TILE + wave * RS_SUB + it * 64 + lane;
        if (i < n) atomicAdd(&cnt[(keys[i] >> shift) & 255], 1);
    }
    __syncthreads();
    hist[(size_t)threadIdx.x * nblocks + blockIdx.x] = cnt[threadIdx.x];
}

// One workgroup per digit: exclusive scan of that digit's per-block counts in place.
__global__ __launch_bounds__(RS_TPB) void rs_scan_kernel(int *__restrict__ hist, int nblocks, int *__restrict__ digit_total)
{
    __shared__ int sh[RS_TPB];
    __shared__ int carry;
    int *row = hist + (size_t)blockIdx.x * nblocks;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    for (int base = 0; base < nblocks; base += RS_TPB) {
        int i = base + (int)threadIdx.x;
        int v = i < nblocks ? row[i] : 0;
        sh[threadIdx.x] = v;
        __syncthreads();
        for (int off = 1; off < RS_TPB; off <<= 1) {
            int t = (int)threadIdx.x >= off ? sh[threadIdx.x - off] : 0;
            __syncthreads();
            sh[threadIdx.x] += t;
            __syncthreads();
        }
        int incl = sh[threadIdx.x];
        int c = carry;
        if (i < nblocks) row[i] = c + incl - v;
        __syncthreads();
        if (threadIdx.x == RS_TPB - 1) carry = c + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) digit_total[blockIdx.x] = carry;
}

__global__ __launch_bounds__(256) void rs_digit_base_kernel(const int *__restrict__ digit_total, int *__restrict__ digit_base)
{
    __shared__ int sh[256];
    int v = digit_total[threadIdx.x];
    sh[threadIdx.x] = v;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
        int t = (int)threadIdx.x >= off ? sh[threadIdx.x - off] : 0;
        __syncthreads();
        sh[threadIdx.x] += t;
        __syncthreads();
    }
    digit_base[threadIdx.x] = sh[threadIdx.x] - v;
}

// Stable scatter of one pass.  pay_in == NULL: the payload is the element's own index (first pass).
__global__ __launch_bounds__(RS_TPB) void rs_scatter_kernel(const int *__restrict__ keys_in, const int *__restrict__ pay_in, int64_t n, int shift,
                                                            int nblocks, const int *__restrict__ hist, const int *__restrict__ digit_base,
                                                            int *__restrict__ keys_out, int *__restrict__ pay_out)
{
    __shared__ int wcnt[4][256];
    const int wave = fg_wave(), lane = fg_lane();
    for (int i = (int)threadIdx.x; i < 4 * 256; i += RS_TPB) (&wcnt[0][0])[i] = 0;
    __syncthreads();
    int key[RS_ITEMS];
#pragma unroll
    for (int it = 0; it < RS_ITEMS; ++it) {
        int64_t i = (int64_t)blockIdx.x * RS_TILE + wave * RS_SUB + it * 64 + lane;
        key[it] = i < n ? keys_in[i] : 0;
        if (i < n) atomicAdd(&wcnt[wave][(key[it] >> shift) & 255], 1);
    }
    __syncthreads();
    {
        int d = (int)threadIdx.x;
        int base = digit_base[d] + hist[(size_t)d * nblocks + blockIdx.x];
#pragma unroll
        for (int w = 0; w < 4; ++w) { int t = wcnt[w][d]; wcnt[w][d] = base; base += t; }
    }
    __syncthreads();
    const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
    for (int it = 0; it < RS_ITEMS; ++it) {
        int64_t i = (int64_t)blockIdx.x * RS_TILE + wave * RS_SUB + it * 64 + lane;
        bool ok = i < n;
        int d = (key[it] >> shift) & 255;
        unsigned long long peers = __builtin_amdgcn_ballot_w64(ok);
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
            unsigned long long bal = __builtin_amdgcn_ballot_w64(((d >> bit) & 1) != 0);
            peers &= ((d >> bit) & 1) ? bal : ~bal;
        }
        int rank = __popcll(peers & lt);
        int base = wcnt[wave][d];
        if (ok) {
            int dst = base + rank;
            keys_out[dst] = key[it];
            pay_out[dst] = pay_in ? pay_in[i] : (int)i;
        }
        fg_wave_lds_sync();
        // the highest lane of every peer group advances the wave's counter of that digit
        if (ok && (peers >> lane) == 1ull) wcnt[wave][d] = base + __popcll(peers);
        fg_wave_lds_sync();
    }
}

__global__ __launch_bounds__(256) void csc_finalize_kernel(int64_t n, int n_rows, int n_cols, const int *__restrict__ sorted_keys,
                                                           const int *__restrict__ permute, const int *__restrict__ row_ptr,
                                                           int *__restrict__ col_ptr, int *__restrict__ row_ind)
{
    int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= n) return;
    int key = sorted_keys[q];
    int prev = q > 0 ? sorted_keys[q - 1] : -1;
    for (int c = prev + 1; c <= key; ++c) col_ptr[c] = (int)q;
    if (q == n - 1)
        for (int c = key + 1; c <= n_cols; ++c) col_ptr[c] = (int)n;
    // row of CSR position p: the last r with row_ptr[r] <= p
    int p = permute[q];
    int lo = 0, hi = n_rows;            // invariant: row_ptr[lo] <= p < row_ptr[hi]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (row_ptr[mid] <= p) lo = mid; else hi = mid;
    }
    row_ind[q] = lo;
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int *p, size_t n, int v)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

static int rs_num_passes(int n_cols)
{
    int bits = 1;
    while (bits < 31 && (1LL << bits) < (long long)n_cols) ++bits;
    return (bits + 7) / 8;
}

extern "C" size_t fgnn_csr2csc_workspace_bytes(int n_rows, int n_cols, int64_t E)
{
    (void)n_rows; (void)n_cols;
    size_t nblocks = (size_t)((E + RS_TILE - 1) / RS_TILE);
    return 3 * fgnn_align256((size_t)E * sizeof(int)) + fgnn_align256(256 * nblocks * sizeof(int)) + 2 * fgnn_align256(256 * sizeof(int));
}

extern "C" int fgnn_csr2csc(int n_rows, int n_cols, int64_t E, const int32_t *row_ptr, const int32_t *col_ind, int32_t *col_ptr,
                            int32_t *row_ind, int32_t *permute, void *workspace, size_t workspace_bytes, void *stream)
{
    FGNN_REQUIRE(n_rows >= 0 && n_cols >= 0 && E >= 0, FGNN_ERR_SHAPE, "fgnn_csr2csc: bad sizes");
    FGNN_REQUIRE(E <= 2147483647LL - RS_TILE, FGNN_ERR_LIMIT, "fgnn_csr2csc: E=%lld exceeds int32 positions", (long long)E);
    FGNN_REQUIRE(row_ptr && col_ptr && (E == 0 || (col_ind && row_ind && permute)), FGNN_ERR_NULL, "fgnn_csr2csc: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    if (E == 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)((n_cols + 1 + 255) / 256)), dim3(256), 0, st, col_ptr, (size_t)n_cols + 1, 0);
        return fgnn_launch_status("fill_i32_kernel");
    }
    FGNN_REQUIRE(n_cols >= 1 && n_rows >= 1, FGNN_ERR_SHAPE, "fgnn_csr2csc: edges without rows or columns");
    size_t need = fgnn_csr2csc_workspace_bytes(n_rows, n_cols, E);
    FGNN_REQUIRE(workspace && workspace_bytes >= need, FGNN_ERR_WORKSPACE, "fgnn_csr2csc: workspace %zu < %zu bytes", workspace_bytes, need);
    const int nblocks = (int)((E + RS_TILE - 1) / RS_TILE);
    char *w = (char *)workspace;
    int *keys[2];
    keys[0] = (int *)w; w += fgnn_align256((size_t)E * sizeof(int));
    keys[1] = (int *)w; w += fgnn_align256((size_t)E * sizeof(int));
    int *pay[2];
    pay[0] = permute;
    pay[1] = (int *)w; w += fgnn_align256((size_t)E * sizeof(int));
    int *hist = (int *)w; w += fgnn_align256(256 * (size_t)nblocks * sizeof(int));
    int *digit_total = (int *)w; w += fgnn_align256(256 * sizeof(int));
    int *digit_base = (int *)w;

    const int passes = rs_num_passes(n_cols);
    const int *kin = col_ind;
    const int *pin = nullptr;
    for (int i = 0; i < passes; ++i) {
        int shift = 8 * i;
        int *kout = keys[i & 1];
        int *pout = pay[(passes - 1 - i) & 1];      // the last pass lands in `permute`
        hipLaunchKernelGGL(rs_hist_kernel, dim3(nblocks), dim3(RS_TPB), 0, st, kin, E, shift, nblocks, hist);
        int rc = fgnn_launch_status("rs_hist_kernel");
        if (rc) return rc;
        hipLaunchKernelGGL(rs_scan_kernel, dim3(256), dim3(RS_TPB), 0, st, hist, nblocks, digit_total);
        rc = fgnn_launch_status("rs_scan_kernel");
        if (rc) return rc;
        hipLaunchKernelGGL(rs_digit_base_kernel, dim3(1), dim3(256), 0, st, digit_total, digit_base);
        rc = fgnn_launch_status("rs_digit_base_kernel");
        if (rc) return rc;
        hipLaunchKernelGGL(rs_scatter_kernel, dim3(nblocks), dim3(RS_TPB), 0, st, kin, pin, E, shift, nblocks, hist, digit_base, kout, pout);
        rc = fgnn_launch_status("rs_scatter_kernel");
        if (rc) return rc;
        kin = kout;
        pin = pout;
    }
    hipLaunchKernelGGL(csc_finalize_kernel, dim3((unsigned)((E + 255) / 256)), dim3(256), 0, st, E, n_rows, n_cols, kin, permute, row_ptr, col_ptr, row_ind);
    return fgnn_launch_status("csc_finalize_kernel");
}
